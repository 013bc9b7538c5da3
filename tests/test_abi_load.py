"""CPU-side checks of the boundary: the C-ABI library loads, exports every symbol the
header declares, and refuses to run without a GPU instead of falling back."""
import ctypes
import os
import re
import pytest
import zerocool_amd as z

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "zc_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(zc_hip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = z.load_library()
    names = declared_symbols()
    assert len(names) >= 30
    for name in names:
        assert hasattr(lib, name), name


def test_structs_match_header_sizes():
    assert ctypes.sizeof(z.Linear) == 3 * 8 + 6 * 4
    assert ctypes.sizeof(z.Config) == 9 * 4
    assert ctypes.sizeof(z.Layer) == 6 * 8
    assert ctypes.sizeof(z.Trace) == 6 * 8


def test_record_layout_sizes():  # storage.hpp:32 (2,764,800 B) and the benchmark shapes
    lib = z.load_library()
    from zerocool_amd import workload
    ref = workload.config("ref")
    assert lib.zc_hip_projection_bytes(2560, 640, 64, 4) == 921600
    assert lib.zc_hip_record_bytes(ctypes.byref(ref), 0) == 2764800
    assert lib.zc_hip_record_bytes(ctypes.byref(workload.config("S")), 0) == 1769472
    assert lib.zc_hip_record_bytes(ctypes.byref(workload.config("F")), 0) == 5308416
    assert lib.zc_hip_record_bytes(ctypes.byref(workload.config("S-mixed")), 0) == 2 * 589824 + 1114112
    assert lib.zc_hip_record_bytes(ctypes.byref(workload.config("S-mixed")), 1) == 3 * 1114112
    l = z.Linear()
    assert lib.zc_hip_expert_linear(ctypes.byref(ref), 0, ctypes.c_void_p(4096), 2, ctypes.byref(l)) == 0
    assert (l.weight, l.scales, l.biases) == (4096 + 2 * 921600, 4096 + 2 * 921600 + 819200, 4096 + 2 * 921600 + 870400)
    assert (l.input, l.output, l.group, l.bits, l.quantized) == (640, 2560, 64, 4, 1)   # metal.mm:1124-1129


def test_no_gpu_means_loud_failure_not_fallback():
    import subprocess, sys
    probe = subprocess.run([sys.executable, "-c", "import zerocool_amd as z\ntry:\n z.Context()\n print('created')\nexcept z.ZcError as e:\n print('refused', e.status)"],
                           capture_output=True, text=True, cwd=ROOT)
    assert probe.stdout.strip() in ("created", "refused 2"), probe.stdout + probe.stderr


def test_host_generator_is_counter_based():
    from zerocool_amd import synth
    a = synth.words(64, 7); b = synth.words(32, 7)
    assert (a[:32] == b).all() and len(set(a.tolist())) > 60
    n = synth.normal(20000, 3)
    assert abs(float(n.mean())) < 0.03 and abs(float(n.std()) - 1) < 0.03
    assert ((n.view("uint32") & 0xffff) == 0).all()
    sc, bi = synth.scales(1000, 5, 0.002, 0.018, -8.0)
    s = (sc.astype("uint32") << 16).view("float32"); b_ = (bi.astype("uint32") << 16).view("float32")
    assert s.min() >= 0.00199 and s.max() <= 0.0201 and (b_ == -8 * s).all()
    off = synth.zipf_offsets(512, 11)
    assert abs(float(off.mean())) < 1e-5 and off.max() > 3
