/*
 * C ABI of the MI355X (gfx950) implementation of ZeroCool's mixture-of-experts
 * layer path.  Plain pointers and sizes only; every data pointer is a DEVICE
 * pointer unless the parameter name says host.  Each entry point replaces one
 * piece of the reference's operator layer (include/engine/metal.hpp,
 * src/engine/metal.mm), cited beside it.
 *
 * Execution model (metal.hpp:45-47): calls only ENQUEUE work on the context's
 * stream; results are defined after zc_hip_finish() or after zc_hip_wait() on a
 * ticket taken later.  Errors: every call returns a zc_status; the text is in
 * zc_hip_last_error() (thread local).  The C++ shim turns the status back into
 * the reference's exception classes.
 */
#ifndef ZC_HIP_H
#define ZC_HIP_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    ZC_OK = 0,
    ZC_INVALID_ARGUMENT = 1, /* std::invalid_argument in the reference */
    ZC_RUNTIME_ERROR = 2,    /* std::runtime_error ("HIP execution: …", "invalid router output") */
    ZC_LOGIC_ERROR = 3,      /* std::logic_error (protocol misuse) */
    ZC_OUT_OF_RANGE = 4,     /* std::out_of_range */
    ZC_BUDGET_EXCEEDED = 5   /* "engine memory budget exceeded", metal.mm:395 */
} zc_status;

typedef struct zc_hip_ctx zc_hip_ctx;

/* metal.hpp:8-13 (Linear) with bindings resolved to device addresses.
 * quantized: affine Q4/Q8 (qwen.metal:46-62, 112-125); otherwise a plain matrix of
 * dtype 0 = BF16, 1 = F32 (qwen.metal:23-27). */
typedef struct {
    const void* weight;
    const void* scales;
    const void* biases;
    uint32_t input, output, group, dtype;
    uint32_t quantized, bits;
} zc_linear;

/* Shapes the reference hard-codes (storage.hpp:26-27) become parameters. */
typedef struct {
    uint32_t hidden, experts, topk, inter, group;
    uint32_t bits_gate_up, bits_down;               /* routed experts */
    uint32_t shared_bits_gate_up, shared_bits_down; /* shared expert */
} zc_moe_config;

/* One layer's weights: what Model::moe reads through Resident and the expert
 * store (model.cpp:433-434, 483-485, 508-513).  A record is
 * [gate W,S,B | up W,S,B | down W,S,B] (metal.mm:1124-1129). */
typedef struct {
    const void* router;          /* [E][H] BF16 */
    const float* router_offsets; /* [E] fp32 added to the logits, or NULL (benchmark load skew) */
    const void* shared_gate;     /* [1][H] BF16, shared_expert_gate */
    const void* shared_record;   /* shared expert record */
    const void* expert_records;  /* E records, record_stride bytes apart */
    uint64_t record_stride;
} zc_moe_layer;

const char* zc_hip_last_error(void);
const char* zc_hip_version(void);

/* Metal::Metal / ~Metal (metal.mm:291-355), Metal::budget (metal.hpp:70). budget 0 = unlimited. */
zc_status zc_hip_create(int device, uint64_t budget_bytes, zc_hip_ctx** out);
zc_status zc_hip_destroy(zc_hip_ctx* ctx);
/* Metal::allocate / zeros / upload (metal.hpp:61-65); download stands in for reading Buffer::data. */
zc_status zc_hip_alloc(zc_hip_ctx* ctx, uint64_t bytes, void** out);
zc_status zc_hip_free(zc_hip_ctx* ctx, void* ptr);
/* Host-visible allocation (pinned, mapped into the device's address space, coherent): the
 * stand-in for the reference's unified-memory Buffer::data (storage.hpp:54-63).  The same
 * pointer is valid on the host and in kernels; meant for activations and small tensors. */
zc_status zc_hip_alloc_host(zc_hip_ctx* ctx, uint64_t bytes, void** out);
zc_status zc_hip_memset(zc_hip_ctx* ctx, void* dst, int byte, uint64_t bytes);
zc_status zc_hip_upload(zc_hip_ctx* ctx, void* dst, const void* host_src, uint64_t bytes);
zc_status zc_hip_download(zc_hip_ctx* ctx, void* host_dst, const void* src, uint64_t bytes);
/* Metal::copy (metal.hpp:66-68) */
zc_status zc_hip_copy(zc_hip_ctx* ctx, void* dst, const void* src, uint64_t bytes);
/* Metal::allocated / peak (metal.hpp:127-128) */
uint64_t zc_hip_allocated(const zc_hip_ctx* ctx);
uint64_t zc_hip_peak(const zc_hip_ctx* ctx);
/* Metal::submit / wait / finish (metal.hpp:105-108): a ticket is done when all work
 * enqueued before it has run. */
zc_status zc_hip_submit(zc_hip_ctx* ctx, uint64_t* ticket);
zc_status zc_hip_wait(zc_hip_ctx* ctx, uint64_t ticket);
zc_status zc_hip_finish(zc_hip_ctx* ctx);
/* Metal::configure (metal.hpp:87; KernelConfig::policy, metal.hpp:17-26): which kernels
 * serve the affine products.  0 = the literal lane kernels for every shape (the
 * reference's "reference" policy); 1 = the exact-integer matrix-core kernels wherever
 * the shape allows (wide Q4, group 64), literal otherwise.  Default 1.  Both policies
 * produce identical bytes; only speed differs. */
zc_status zc_hip_configure(zc_hip_ctx* ctx, uint32_t affine_policy);
/* HIP-event stopwatch on the context's stream: start enqueues an event, stop enqueues a
 * second one, waits for it and returns the milliseconds between them. */
zc_status zc_hip_timer_start(zc_hip_ctx* ctx);
zc_status zc_hip_timer_stop(zc_hip_ctx* ctx, float* milliseconds);
/* The raw hipStream_t the context enqueues on (for event timing by the caller). */
void* zc_hip_stream(zc_hip_ctx* ctx);

/* Metal::linear_into (metal.mm:775-827): quantized -> q4_mm/q8_mm arithmetic;
 * plain -> plain_mm (qwen.metal:499-506). out[tokens][output]. */
zc_status zc_hip_linear_into(zc_hip_ctx* ctx, const zc_linear* layer, const float* x,
                             uint32_t tokens, float* out, int float_output);
/* The router branch of linear_into (metal.mm:818-822; qwen.metal:512-534). */
zc_status zc_hip_router_logits(zc_hip_ctx* ctx, const void* w_bf16, const float* x, uint32_t tokens,
                               uint32_t hidden, uint32_t experts, const float* offsets, float* logits);
/* Metal::gated_linear (metal.mm:845-880; qwen.metal:71-81, 134-144). rows may be NULL.
 * x_rows is the number of rows x holds (bounds for the gather). */
zc_status zc_hip_gated_linear(zc_hip_ctx* ctx, const zc_linear* gate, const zc_linear* up,
                              const float* x, uint32_t x_rows, uint32_t tokens,
                              const int32_t* rows, float* out);
/* Metal::route (metal.mm:261-266; qwen.metal:742-795) */
zc_status zc_hip_route(zc_hip_ctx* ctx, const float* logits, uint32_t tokens, uint32_t experts,
                       uint32_t topk, int32_t* ids, float* weights);
/* The positions/selected lists Model::moe builds on the CPU (model.cpp:449-479), built on
 * the device: offsets[E+1], slots[tokens*topk] (flat p = t*topk+k, ascending inside each
 * expert), selected[E] (ascending ids of non-empty experts), count[1], status[1]
 * (non-zero: an id outside [0,E) -> "invalid router output"). */
zc_status zc_hip_build_dispatch(zc_hip_ctx* ctx, const int32_t* ids, uint32_t tokens, uint32_t topk,
                                uint32_t experts, int32_t* offsets, int32_t* slots,
                                int32_t* selected, int32_t* count, int32_t* status);
/* dispatch("scatter_experts") (pipeline.cpp:28; qwen.metal:800-803) */
zc_status zc_hip_scatter_experts(zc_hip_ctx* ctx, const float* x, const int32_t* positions,
                                 uint32_t n, uint32_t hidden, float* out);
/* dispatch("moe_sum") (model.cpp:555; qwen.metal:804-816) */
zc_status zc_hip_moe_sum(zc_hip_ctx* ctx, const float* experts, const float* weights,
                         const float* shared, const float* gate, uint32_t tokens,
                         uint32_t hidden, uint32_t topk, float* out);
/* The callers' glue either side of Model::moe: Model::unary / Model::binary (model.cpp:328-336 ->
 * dispatch("unary"), dispatch("binary"); qwen.metal:567-581).  op: 0 SiLU, 1 sigmoid, 2 SiLU(x/4),
 * 3 2*sigmoid(x/4), 4 softplus; binary op 0 adds, any other multiplies.  Results are BF16-valued fp32. */
zc_status zc_hip_unary(zc_hip_ctx* ctx, const float* x, uint64_t n, uint32_t op, float* y);
zc_status zc_hip_binary(zc_hip_ctx* ctx, const float* x, const float* y, uint64_t n, uint32_t op, float* out);
/* dispatch("hc_mix") in Model::hyper (model.cpp:343; qwen.metal:582-588): x, w [tokens][4][hidden] ->
 * out [tokens][hidden]. */
zc_status zc_hip_hc_mix(zc_hip_ctx* ctx, const float* x, const float* w, uint32_t tokens, uint32_t hidden, float* out);
/* dispatch("hc_add") after attention and after the MoE layer (model.cpp:651, 662; qwen.metal:589-595):
 * hyper [tokens][4][hidden], x [tokens][hidden], inject [tokens][4] -> out [tokens][4][hidden]. */
zc_status zc_hip_hc_add(zc_hip_ctx* ctx, const float* hyper, const float* x, const float* inject,
                        uint32_t tokens, uint32_t hidden, float* out);
/* Model::norm -> dispatch("norm") / dispatch("norm_wide") (model.cpp:312-326; qwen.metal:545-566, 403-426):
 * RMS norm over groups of `group` elements (<= 4096) of rows of `width`; w: `width` weights, dtype 0 BF16, 1 fp32. */
zc_status zc_hip_norm(zc_hip_ctx* ctx, const float* x, const void* w, uint32_t dtype, uint32_t group,
                      uint32_t width, uint32_t tokens, float* out);
/* Metal::grouped_experts (metal.mm:881-912): n<=8 records (host array of device
 * pointers), distinct positions < topk (host array); scratch holds n*inter floats. */
zc_status zc_hip_grouped_experts(zc_hip_ctx* ctx, const zc_moe_config* cfg,
                                 const void* const* host_records, const uint32_t* host_positions,
                                 uint32_t n, const float* x, float* out, float* scratch);

/* Model::moe (model.cpp:431-557) as one enqueue with routing and dispatch kept on the
 * device (no CPU readback).  workspace: zc_hip_moe_workspace_bytes() bytes.
 * trace (optional, host struct of device pointers, any NULL): copies of the
 * intermediates the reference dumps with --trace-dir (model.cpp:447-448, 549-552). */
typedef struct {
    float* logits;     /* [T][E]      router_<layer>  */
    int32_t* ids;      /* [T][topk]   route_<layer>   */
    float* weights;    /* [T][topk]   .mlp.weights    */
    float* expert_out; /* [T][topk][H] .mlp.expert_out */
    float* shared;     /* [T][H]      .mlp.shared     */
    float* gate;       /* [T]         .mlp.gate       */
} zc_moe_trace;
uint64_t zc_hip_moe_workspace_bytes(const zc_moe_config* cfg, uint32_t tokens);
zc_status zc_hip_moe_forward(zc_hip_ctx* ctx, const zc_moe_config* cfg, const zc_moe_layer* layer,
                             const float* x, uint32_t tokens, float* out, void* workspace,
                             const zc_moe_trace* trace);
/* zc_hip_moe_forward without a workspace argument and without any allocation.  It has no counterpart in the reference
 * (whose scratch arenas come from Metal::allocate, metal.mm:386-433); it is for callers that cannot allocate: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The workspace lives in a static device array
 * of zc_hip_moe_static_scratch_bytes() bytes (4 MiB) that every GPU the library runs on holds until the process ends;
 * its address is looked up once per device in zc_hip_create.  A call whose workspace
 * (zc_hip_moe_workspace_bytes(cfg, tokens)) does not fit is refused with ZC_INVALID_ARGUMENT and a message that names
 * both sizes.  The call itself performs no hipMalloc / hipFree and creates no stream or event, also while a recording
 * is on (zc_hip_profile: this entry point records no row); inputs, outputs and the optional trace buffers are the caller's.  All calls on one GPU share the one array, whatever context they come
 * through: calls that can overlap on that GPU (two contexts, two threads) race; calls on one context's stream are
 * ordered and safe.  Nothing in the array has to start at zero (every word a kernel reads has been written by an earlier
 * kernel of the same call), so a call leaves the previous call's contents in place without reading them. */
uint64_t zc_hip_moe_static_scratch_bytes(void);
zc_status zc_hip_moe_forward_static(zc_hip_ctx* ctx, const zc_moe_config* cfg, const zc_moe_layer* layer,
                                    const float* x, uint32_t tokens, float* out, const zc_moe_trace* trace);
/* Prefill (many tokens): the same layer with the expert products as a sorted-token grouped GEMM on the bf16 matrix
 * cores with fp32 accumulation -- what encode_expert_rows batches per expert in the reference (pipeline.cpp:7-31 over
 * q4_mm / q4_gate_up, qwen.metal:289-376; affine Q8 projections the same way over q8_mm / q8_gate_up, qwen.metal:126-144,
 * 192-196, so the mixed 4/8-bit artifact has a prefill path too).  Router ids, softmax weights and the dispatch are the exact kernels (bit-equal
 * to zc_hip_moe_forward); expert outputs agree with zc_hip_moe_forward to a few fp32 ulps before their BF16 rounding, so
 * the layer output is checked against a tolerance (max relative error 2e-3), not bit for bit.  Every projection affine
 * Q4 or affine Q8, group 64; hidden and intermediate sizes multiples of 128 up to 4096; x must be BF16-valued (else status bit 4 at zc_hip_moe_check).
 * From 128 tokens on the router logits are formed exactly only for the experts that can reach the top k (a matrix-core
 * product with a rigorous bound decides which; ids and weights are unchanged); a trace that asks for the logits gets
 * all of them from the exact kernel.
 * The workspace is larger than zc_hip_moe_forward's: zc_hip_moe_prefill_workspace_bytes (0: shape not supported). */
uint64_t zc_hip_moe_prefill_workspace_bytes(const zc_moe_config* cfg, uint32_t tokens);
zc_status zc_hip_moe_prefill(zc_hip_ctx* ctx, const zc_moe_config* cfg, const zc_moe_layer* layer,
                             const float* x, uint32_t tokens, float* out, void* workspace,
                             const zc_moe_trace* trace);
/* Drains the stream, then reports ZC_RUNTIME_ERROR "invalid router output" if any
 * zc_hip_moe_forward since the last check saw an id outside [0,E) (model.cpp:459).
 * Clears the flag. */
zc_status zc_hip_moe_check(zc_hip_ctx* ctx);

/* Stacked decode: n_layers MoE layers (Model::moe, model.cpp:431-557, called once per
 * layer by Model::forward_impl, model.cpp:637-672) chained for a few tokens.  The trunk
 * between the reference's MoE layers (attention / GDN / hyper-connections) is outside
 * this path; the stack stands in for it with a glue that keeps activations bounded and
 * BF16-valued: x_next = bf(y * (1 / max|y|)) per token (zc_hip_stack_glue).
 * Up to 64 tokens run as ONE persistent kernel launch for the whole stack (routing,
 * dispatch and combine stay on the device, no host synchronisation between layers; one
 * kernel each for one token, two to eight, and nine to sixty-four), larger batches as
 * one such launch per 64 tokens; shapes those kernels do not take run layer by layer
 * through zc_hip_moe_forward.  All give identical bytes.
 * out: [tokens][hidden], the last layer's output.  flags bit 0: force the layer-by-layer path. */
typedef struct zc_hip_stack zc_hip_stack;
typedef struct {       /* optional device buffers, any may be NULL */
    int32_t* ids;      /* [n_layers][tokens][topk] */
    float* weights;    /* [n_layers][tokens][topk] */
    float* outputs;    /* [n_layers][tokens][hidden] layer outputs before the glue */
    uint64_t* clocks;  /* [n_layers * 24][workgroups] timestamps (100 MHz) of the persistent kernels, 24 slots
                          per layer: the one-token kernel fills 0..14 from every workgroup's first thread at its
                          phase boundaries and 15..21 from the first lane of its fifth wave inside the gate/up
                          and down phases; the kernels for more tokens write their own, smaller number of stamps per
                          layer back to back (tuning aid; persistent path only; workgroups = compute units) */
} zc_stack_trace;
zc_status zc_hip_stack_create(zc_hip_ctx* ctx, const zc_moe_config* cfg, const zc_moe_layer* host_layers,
                              uint32_t n_layers, uint32_t max_tokens, zc_hip_stack** out);
zc_status zc_hip_stack_destroy(zc_hip_ctx* ctx, zc_hip_stack* stack);
zc_status zc_hip_stack_decode(zc_hip_ctx* ctx, zc_hip_stack* stack, const float* x, uint32_t tokens,
                              float* out, const zc_stack_trace* trace, uint32_t flags);
/* 1 if zc_hip_stack_decode would take the persistent single-launch path for `tokens`. */
int zc_hip_stack_is_persistent(zc_hip_ctx* ctx, zc_hip_stack* stack, uint32_t tokens);
/* Bound of every wait of the persistent kernel on another workgroup, in polls (0 restores the default, about four
 * seconds' worth).  A wait that runs out makes the launch give up everywhere and zc_hip_moe_check report it; the stack
 * stays usable.  No counterpart in the reference (its command buffers cannot wait on each other); tests use a bound of
 * one poll to exercise the give-up path without a lost workgroup. */
zc_status zc_hip_stack_set_wait_limit(zc_hip_ctx* ctx, zc_hip_stack* stack, uint32_t polls);
/* One-token launches of the persistent kernel start every layer's gate/up tiles on the experts that layer picked at the
 * previous one-token step, before this step's ids are known, and redo only the slots that were guessed wrong (the
 * reference predicts a layer's experts to prefetch their records, model.cpp:438-445, 489-500; here the guess hides the
 * router, the logits exchange and the selection).  Outputs are the same bytes with or without it.  on = 0 switches the
 * guessing off (every slot is then computed after the selection); default on. */
zc_status zc_hip_stack_set_speculation(zc_hip_ctx* ctx, zc_hip_stack* stack, int on);
zc_status zc_hip_stack_glue(zc_hip_ctx* ctx, const float* y, uint32_t tokens, uint32_t hidden, float* x_next);

/* ---- Expert store: ExpertStore + ExpertCache (include/engine/storage.hpp:168-269; src/engine/storage.cpp:493-725)
 * with the SSD replaced by pinned host memory and the slots living in HBM.  Every record has a home in pinned host
 * memory (zc_hip_store_backing: write the record there before its first use); `slots` HBM slots cache the records in
 * use and are filled by hipMemcpyAsync on the store's own side stream.  The rules are the reference's: a lease pins
 * its slot until it is released (release it only after the GPU work that reads the slot has finished, e.g. after
 * zc_hip_wait on a later ticket); victims are chosen by CLOCK second chance and are never pinned or still loading;
 * prefetch() fills speculatively without a lease and never evicts a pinned or loading slot; counters as
 * CacheStats (storage.hpp:183-192).  With slots >= layers * experts the store is HBM-resident after the first touch.
 * A NULL context gives a store with host-memory slots whose fills can be held back (zc_hip_store_hold): the
 * policy, loading joins included, can then be tested without a GPU.  One coordinator thread owns a store. */
typedef struct zc_hip_store zc_hip_store;
typedef struct { uint64_t hits, misses, evictions, bytes, ready_hits, loading_joins, prefetches, prefetch_claims, prefetch_unclaimed; } zc_store_stats;
typedef struct {
    uint64_t lease;      /* pass to wait / release */
    void* record;        /* the slot: device address of the record (valid for GPU work enqueued after zc_hip_store_wait) */
    int32_t acquisition; /* 0 new miss, 1 ready hit, 2 loading join (Lease::acquisition, storage.cpp:600-602) */
} zc_store_lease;
zc_status zc_hip_store_create(zc_hip_ctx* ctx, uint32_t layers, uint32_t experts, uint64_t record_bytes, uint64_t slots, zc_hip_store** out);
/* The same with the replacement policy by name (parse_cache_policy, storage.cpp:536-540): "clock" (second chance, the
 * default) or "slru" (segmented LRU, storage.cpp:547-573: probation and protected queues, protected at most three quarters
 * of the slots; takes no prefetches).  Any other name: ZC_INVALID_ARGUMENT "cache policy must be clock or slru". */
zc_status zc_hip_store_create_with_policy(zc_hip_ctx* ctx, uint32_t layers, uint32_t experts, uint64_t record_bytes, uint64_t slots,
                                          const char* policy, zc_hip_store** out);
/* The same with fewer homes than layers: layer l's records live in home (l mod home_layers), i.e. layers l and l + home_layers
 * hold the same bytes, while the slot cache still keys every (layer, expert) separately.  For measuring the capped-HBM run
 * of a model whose records exceed what the host can pin (no counterpart in the reference, which reads from SSD). */
zc_status zc_hip_store_create_shared_homes(zc_hip_ctx* ctx, uint32_t layers, uint32_t experts, uint64_t record_bytes, uint64_t slots,
                                           const char* policy, uint32_t home_layers, zc_hip_store** out);
const char* zc_hip_store_policy(const zc_hip_store* store);                 /* "clock" or "slru" (ExpertCache::json "policy") */
uint64_t zc_hip_store_protected_entries(const zc_hip_store* store);         /* ExpertCache::json "protected_entries" */
zc_status zc_hip_store_destroy(zc_hip_store* store);
void* zc_hip_store_backing(zc_hip_store* store, uint32_t layer, uint32_t expert);   /* HOST pointer: the record's home */
uint64_t zc_hip_store_stride(const zc_hip_store* store);
uint64_t zc_hip_store_capacity(const zc_hip_store* store);
uint64_t zc_hip_store_occupancy(const zc_hip_store* store);
/* ExpertCache::acquire (storage.cpp:628-676).  ZC_RUNTIME_ERROR "expert cache exhausted by outstanding leases; ..." when
 * every slot is pinned or loading. */
zc_status zc_hip_store_acquire(zc_hip_store* store, uint32_t layer, uint32_t expert, zc_store_lease* out);
/* Lease::wait (storage.cpp:588-591) without blocking the host: the context's stream waits for the slot's fill. */
zc_status zc_hip_store_wait(zc_hip_store* store, uint64_t lease);
zc_status zc_hip_store_release(zc_hip_store* store, uint64_t lease);   /* Lease::~Lease */
/* ExpertCache::prefetch (storage.cpp:677-692): *issued = 0 when the record is present or no slot is free to take. */
zc_status zc_hip_store_prefetch(zc_hip_store* store, uint32_t layer, uint32_t expert, int* issued);
int zc_hip_store_ready(zc_hip_store* store, uint32_t layer, uint32_t expert);   /* ExpertCache::ready */
zc_status zc_hip_store_clear(zc_hip_store* store);                    /* ZC_LOGIC_ERROR while a lease is out */
zc_status zc_hip_store_resize(zc_hip_store* store, uint64_t slots);   /* survivors keep their bytes; ZC_LOGIC_ERROR while a lease is out */
zc_status zc_hip_store_stats(const zc_hip_store* store, zc_store_stats* out);
zc_status zc_hip_store_layer_stats(const zc_hip_store* store, uint32_t layer, uint64_t* hits, uint64_t* misses);
/* The store as a kernel sees it: a table of layers * experts record addresses, entry [layer * experts + expert].  An entry
 * points at the record's HBM slot while that slot holds the finished record and at the record's home otherwise (pinned
 * host memory, which the GPU reads over the host link), so a kernel that takes its records from the table always finds
 * the right bytes and never waits for the host: the reference's acquire -> wait -> encode -> release around every expert
 * (pipeline.cpp:158-214, storage.cpp:628-676) becomes one table lookup on the device and the two host calls below around
 * a whole launch.  Create the table while the store is empty.
 *   zc_hip_store_table_refresh  before a launch: entries of fills that have finished switch to their slots; the changed
 *                               table is copied to the device on the context's stream.
 *   zc_hip_store_table_observe  after the launch has FINISHED (the host has synchronised): the expert ids one layer chose.
 *                               First the records read from a slot are touched (ExpertCache::acquire's hit), then the records
 *                               read from home are admitted (its miss: a victim by the store's policy that this call did not
 *                               touch, the fill starts on the side stream and serves later launches); no lease stays out.  A fill never starts while a launch that may read
 *                               its slot is in flight, because fills start here only.
 * Leases and the table may not be mixed on one store while launches are in flight. */
typedef struct {
    uint64_t reads;            /* distinct (layer, expert) records that observed launches read */
    uint64_t slot_reads;       /* ... from an HBM slot */
    uint64_t home_reads;       /* ... from the record's home over the host link */
    uint64_t home_read_bytes;
    uint64_t switched;         /* fills whose table entry moved to the slot (finished, or joined) */
    uint64_t joined;           /* ... of which the next launch was made to wait for the fill (zc_hip_store_table_refresh_joining) */
    uint64_t not_admitted;     /* misses that found every slot still loading */
} zc_store_table_stats;
zc_status zc_hip_store_table(zc_hip_store* store, const void* const** table);
zc_status zc_hip_store_table_refresh(zc_hip_store* store);
/* The same, and the entries of fills still in flight switch to their slots too: whatever the context's stream runs next
 * waits for those fills on the device (ExpertCache::acquire's "loading join", storage.cpp:636-641, for a whole launch), so a
 * record that an earlier launch read over the host link is not read over it a second time.  zc_hip_stack_decode uses this. */
zc_status zc_hip_store_table_refresh_joining(zc_hip_store* store);
zc_status zc_hip_store_table_observe(zc_hip_store* store, uint32_t layer, const int32_t* ids, uint32_t count);
/* The same for a launch that ran every layer: ids [layers][per_layer].  All records that the launch read from slots are touched
 * before any record read from home is admitted, whatever their layers, so a miss never takes the slot of a record the same
 * launch used. */
zc_status zc_hip_store_table_observe_layers(zc_hip_store* store, const int32_t* ids, uint32_t per_layer);
zc_status zc_hip_store_table_stats(const zc_hip_store* store, zc_store_table_stats* out);
zc_status zc_hip_store_geometry(const zc_hip_store* store, uint32_t* layers, uint32_t* experts, uint64_t* record_bytes);
/* A decode stack whose routed records live in an expert store (the capped-HBM run: model.cpp:431-557 with the cache of
 * storage.cpp:525-725 in the loop).  host_layers[l].expert_records is ignored; the store must have n_layers layers of
 * cfg's records, and max_tokens <= 64.  zc_hip_stack_decode on such a stack is ONE launch that reads every record
 * through the store's table (zc_hip_store_table).  Before the launch the fills that earlier launches caused switch to
 * their slots, and the launch waits for the unfinished ones on the device (zc_hip_store_table_refresh_joining); after it
 * the routes are copied back and handed to zc_hip_store_table_observe_layers, so that the records this step read from
 * their homes are in HBM slots for the steps to come (the previous step's experts, which the next step is most likely to
 * pick again -- the reference's prefetch on predicted experts, model.cpp:438-445, 489-500 -- are therefore in their slots
 * before the launch that needs them).  While launches read nothing from a home, the host looks at a launch's routes only
 * after the next launch has been enqueued and never waits for the GPU; a launch that read from a home is observed at once
 * until that stops.  zc_hip_stack_settle observes a launch that is still waiting to be looked at (before reading the
 * store's statistics, say).  Output bytes are those of a stack with all records resident.  flags bit 0 (layer by layer)
 * is refused with ZC_INVALID_ARGUMENT. */
zc_status zc_hip_stack_create_with_store(zc_hip_ctx* ctx, const zc_moe_config* cfg, const zc_moe_layer* host_layers,
                                         uint32_t n_layers, uint32_t max_tokens, zc_hip_store* store, zc_hip_stack** out);
zc_status zc_hip_stack_settle(zc_hip_ctx* ctx, zc_hip_stack* stack);
/* ---- Statistics and stage labels (Metal::label, metal.mm:267-270; KernelConfig::profile; Model::stats, model.cpp:706-732)
 * zc_hip_profile(on != 0) starts a recording: from then on every operator call through the context adds one row -- the
 * label current at the call, the operator's name, and the GPU time between two events placed around its launches (an
 * operator that calls other operators counts once).  At most 16384 rows are kept; further calls are counted as dropped.
 * zc_hip_label names the stage, layer, token count and token offset of the calls that follow; like the reference's it
 * does nothing unless a recording is on.  zc_hip_stats waits for the context's stream and writes one JSON object:
 * "memory", "profile" (per (stage, operator) call counts and GPU microseconds, then the rows) and, with a store,
 * "expert_cache" (the counters of zc_hip_store_stats and zc_hip_store_table_stats, capacity, occupancy).  *needed receives
 * the text's length including the terminator; ZC_OUT_OF_RANGE with a truncated text if capacity is smaller. */
zc_status zc_hip_label(zc_hip_ctx* ctx, const char* stage, int32_t layer, uint32_t tokens, uint32_t offset);
zc_status zc_hip_profile(zc_hip_ctx* ctx, int on);
zc_status zc_hip_stats(zc_hip_ctx* ctx, const zc_hip_store* store, char* json, uint64_t capacity, uint64_t* needed);
/* Stores without a context only: fills of this record stay "loading" while held (what a slow read is to the reference's tests). */
zc_status zc_hip_store_hold(zc_hip_store* store, uint32_t layer, uint32_t expert, int hold);

/* Counter-based synthetic tensors: element i depends only on (seed, i).
 * kind 0: uint32 words of uniform bits (Q4/Q8 codes), count = words
 * kind 1: BF16 scale in [lo, lo+span) and BF16 bias = scale*factor, interleaved
 *         as two arrays scales[count], biases[count]
 * kind 2: BF16-valued N(0,1)*sigma stored as fp32, count = floats
 * kind 3: the same stored as BF16 (uint16), count = elements */
zc_status zc_hip_synth_words(zc_hip_ctx* ctx, uint32_t* dst, uint64_t count, uint64_t seed);
zc_status zc_hip_synth_scales(zc_hip_ctx* ctx, uint16_t* scales, uint16_t* biases, uint64_t count,
                              uint64_t seed, float lo, float span, float factor);
zc_status zc_hip_synth_normal_f32(zc_hip_ctx* ctx, float* dst, uint64_t count, uint64_t seed, float sigma);
zc_status zc_hip_synth_normal_bf16(zc_hip_ctx* ctx, uint16_t* dst, uint64_t count, uint64_t seed, float sigma);
/* A whole expert record (or E of them, stride apart) in one launch:
 * projection p of record r uses seed + r*3 + p. */
zc_status zc_hip_synth_records(zc_hip_ctx* ctx, const zc_moe_config* cfg, int shared, void* records,
                               uint64_t stride, uint32_t count, uint64_t seed);

uint64_t zc_hip_projection_bytes(uint32_t input, uint32_t output, uint32_t group, uint32_t bits);
uint64_t zc_hip_record_bytes(const zc_moe_config* cfg, int shared);
/* expert_linear (metal.mm:1124-1129) for parameterised shapes. */
zc_status zc_hip_expert_linear(const zc_moe_config* cfg, int shared, const void* record,
                               int projection, zc_linear* out);
#ifdef __cplusplus
}
#endif
#endif
