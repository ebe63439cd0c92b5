// Host-side internals of libllama2j_hip.so shared by its translation units: the context, its options, error plumbing.
//   l2j_context.hip   contexts, options, the load path (uploads, on-device quantization, finalize), taps
//   l2j_forward.hip   launch shapes, hipGraph capture, forward passes, the decode loops, kernel timing
//   l2j_sampler.hip   the device sampler's host side, running sums
//   l2j_batch.hip     several sequences at once
#pragma once

#include "kernels.hpp"
#include "phase_kernels.hpp"
#include "sampler_state.hpp"

#include <hip/hip_ext.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/llama2j_hip.h"
#include "host_internal.h"

namespace l2j {

inline thread_local std::string g_err;

inline int fail(int code, const std::string &msg)
{
    g_err = msg;
    return code;
}

#define HIPCHK(expr)                                                                              \
    do {                                                                                          \
        hipError_t e_ = (expr);                                                                   \
        if (e_ != hipSuccess)                                                                     \
            return fail(e_ == hipErrorOutOfMemory ? L2J_E_OOM : L2J_E_HIP,                        \
                        std::string(#expr) + ": " + hipGetErrorString(e_));                      \
    } while (0)

struct QTensor {
    uint8_t *codes = nullptr;  // one byte per weight, flat, padded to whole groups
    float2 *gs = nullptr;      // ((max-min)/255, min) per group
    float2 *mm = nullptr;      // (min, max) per group
    uint64_t nfloats = 0, ngroups = 0;
    uint64_t groups_loaded = 0;
    std::mutex mu;             // uploads of this tensor take turns (those of different tensors copy side by side)
};

// Launch-shape and algorithm switches of a context.  kAuto = the library picks (by shape, at l2j_finalize).  A context
// starts from the process defaults (environment variable L2J_<NAME IN CAPITALS>, read once by l2j_create) and
// l2j_set_option overrides them per context; nothing reads the environment afterwards.
enum {
    OPT_THREADS = 0, OPT_GRID, OPT_ATTN_THREADS, OPT_ATTN_ROWS, OPT_ATTN_NSPLIT, OPT_FUSED_ATTN_ROWS, OPT_FUSED_ATTN_SPLITS,
    OPT_BARRIER_SPINS, OPT_FUSE, OPT_LAYERS_PER_LAUNCH, OPT_BY_VALUE, OPT_TOKEN_SPECIAL, OPT_SAMPLER_SCAN, OPT_SAMPLER_EXP_WGS,
    OPT_GRAPH, OPT_SELF_CONTAINED, OPT_GRAPH_TOKENS, OPT_FAST_STEPS, OPT_FALLBACK, OPT_BATCH_FUSE, OPT_SAMPLER_WIDE, OPT_PREFILL_FLASH, OPT_PREFILL, OPT_PREFILL_SPLIT, OPT_COUNT
};
constexpr int kAuto = -1;
struct OptionDef {
    const char *name;
    int dflt;
    bool after_finalize;  // may still be changed once the launch shapes are fixed
};
inline const OptionDef kOptions[OPT_COUNT] = {
    {"threads", kAuto, false},         // workgroup size of the weight-streaming kernels (auto: 1024; 512 / 640 for rows of at most 4096 / 1024 weights, measured)
    {"grid", kAuto, false},            // their workgroups (auto: one per compute unit)
    {"attn_threads", 256, false},      // k_attention as a kernel of its own
    {"attn_rows", 32, false},
    {"attn_nsplit", 32, false},
    {"fused_attn_rows", 64, false},    // cache rows per attention split inside k_token
    {"fused_attn_splits", kAuto, false},
    {"barrier_spins", 20000, false},    // polls of a bounded wait inside k_token before it gives up
    {"fuse", kAuto, false},            // 1: whole-token kernel, 0: one launch per phase (auto: by layer size)
    {"layers_per_launch", kAuto, false},
    {"by_value", 1, false},            // k_token hands vectors over by value (0: grid barriers)
    {"token_special", 1, false},       // use the k_token instances specialised for the published shapes
    {"sampler_scan", 1, true},         // running sums by the parallel scan (0: one lane, element after element)
    {"sampler_exp_wgs", 32, true},     // workgroups of k_sample_exp (0: the exponentials in k_sample_probs)
    {"graph", 1, false},               // 1: replay a captured hipGraph per token, 0: launch the kernels one by one
    {"self_contained", 3, false},      // k_token (by value): bit 0 alternates two sets of vectors (no k_fill_unset), bit 1 steps the token loop itself (no k_finish)
    {"graph_tokens", 32, false},       // tokens per replay of the decode loops' graph (1: only the one-token graph)
    {"fast_steps", 1, false},          // k_token folds rows of dim codes without clamping when they are exactly one step
    {"fallback", 1, true},             // a whole-token kernel whose bounded wait ran out: switch to one launch per phase and repeat
    {"batch_fuse", 0, true},           // batched decode: 1: the layers of a step in one launch with grid barriers (slower, measured); 0: eight launches per layer
    {"sampler_wide", 1, true},         // sampling step: 1: one launch over many workgroups (vocabularies that fit in LDS), 0: one launch per stage
    {"prefill_flash", 1, true},        // l2j_prefill's attention: 1: 16 positions at a time on the fp32 matrix cores from position 64 on, every position for itself before; 2: always; 0: never
    {"prefill", 0, true},              // decode loops: 1: the prompt positions 32 at a time through the batched products (l2j_prefill), 0: one by one as the reference
    {"prefill_split", 0, true},        // workgroups that share the keys of one head and 16 positions in that attention: 1..4, 0: one below position 192, then as many as the GPU has compute units for
};

inline int option_from_env(int i)
{
    char var[64] = "L2J_";
    size_t k = 4;
    for (const char *p = kOptions[i].name; *p && k + 1 < sizeof(var); p++) var[k++] = (char)toupper((unsigned char)*p);
    var[k] = 0;
    const char *v = getenv(var);
    return v && *v ? atoi(v) : kOptions[i].dflt;
}

struct BatchBufs;   // l2j_batch.hip

}  // namespace l2j

using namespace l2j;

struct l2j_ctx {
    l2j_config cfg{};
    std::mutex err_mu;
    std::string last_err;  // text of the last failed call on this context, whatever thread made it
    int opt[OPT_COUNT];
    int head_size = 0, kv_dim = 0, kv_mul = 0;
    int n_cu = 256;
    hipStream_t stream = nullptr;
    std::mutex upload_mu;
    bool finalized = false;

    QTensor qt[L2J_TENSOR_COUNT];
    uint8_t *bt_codes[L2J_TENSOR_COUNT] = {};   // the batched path's copy of the matrices in tile order (k_btile), made by its first call
    float2 *bt_gs[L2J_TENSOR_COUNT] = {};
    bool bt_done[L2J_TENSOR_COUNT] = {};        // the copy of this tensor has been launched
    bool bt_ready = false;
    BatchBufs *batch = nullptr;                 // buffers and captured step of l2j_decode_greedy_batch, made by its first call
    float *emb = nullptr, *wcls = nullptr;
    bool emb_loaded = false, wcls_loaded = false;

    // Activations.  Every vector of a token has an address of its own (stride = length rounded up to 256
    // bytes): x holds the 2L+1 versions of the residual stream (version 2l+1 after the attention residual of
    // layer l, 2l+2 after its FFN residual), xb, hb and q one vector per layer.
    // They live in one allocation, twice: a whole-token kernel that hands over by value alternates between the two sets.
    float *acts = nullptr;
    uint64_t set_floats = 0;  // floats of one set: x | xb | q | hb | knew | vnew
    float *x = nullptr, *xb = nullptr, *hb = nullptr, *q = nullptr, *logits = nullptr;  // set 0
    uint64_t sd = 0, sh = 0;  // strides of dim-long and hidden_dim-long vectors, in floats
    float *kcache = nullptr, *vcache = nullptr;
    float2 *rope = nullptr;
    float *silu = nullptr;
    unsigned *counters = nullptr;  // n_heads attention counters + 1 classifier counter
    DevState *st = nullptr;
    int *prompt = nullptr, *out_tokens = nullptr;
    DevState *h_st = nullptr;  // pinned
    int *h_tokens = nullptr;   // pinned, seq_len

    // per-layer taps (allocated on first l2j_forward_taps)
    float *taps[L2J_B_COUNT] = {};


    // launch shape of the phase kernels and their scratch
    int pk_grid = 0, pk_threads = 1024, attn_threads = 256, attn_grid = 0, attn_nsplit = 1, attn_rows = 32;
    unsigned long long *cls_part = nullptr;  // per workgroup: (index, value) of the first maximum of its classifier rows
    unsigned long long *tstamp = nullptr;    // per position: the device's wall clock at the end of that token
    unsigned long long *h_tstamp = nullptr;  // pinned
    double wall_clock_hz = 0.0;              // rate of the device's wall clock (hipDeviceAttributeWallClockRate); 0: unknown
    float *attn_part = nullptr;
    float *rmsw = nullptr;  // dequantized rmsnorm weights: att (L*dim), ffn (L*dim), final (dim)

    // k_token: a range of layers (by default the whole token) per launch, grid barriers between the phases
    bool fused = false;
    int layers_per_launch = 0;
    unsigned *bar_ctr = nullptr;  // kBarStride words per barrier instance, 5 instances per layer
    int nbar = 0;
    int *fault = nullptr;         // set by a kernel whose barrier wait ran out
    int *h_fault = nullptr;       // pinned
    int fused_attn_rows = 64;
    bool by_value = false;        // k_token hands activations over by value (no grid barriers)
    int self_contained = 0;       // ... bit 0: and needs no k_fill_unset before it, bit 1: no k_finish after it
    bool acts_dirty = false;      // kernels other than a self-contained k_token wrote activation vectors (of set 0) last
    float *knew = nullptr, *vnew = nullptr;  // this token's k and v rows per layer
    uint64_t skv = 0;
    TokenGeom geom{};             // set by l2j_finalize

    hipGraph_t graph = nullptr;
    hipGraphExec_t graph_exec = nullptr;
    hipGraph_t graph_n = nullptr;           // graph_tokens tokens in one graph (the decode loops replay it)
    hipGraphExec_t graph_n_exec = nullptr;
    int graph_tokens = 1;
    std::vector<hipEvent_t> events;

    // device sampler (allocated by its first use): the reference's Sampler object
    SamplerState *ss = nullptr;
    SamplerState *h_ss = nullptr;               // pinned
    float *pi_prob[2] = {nullptr, nullptr};     // the ProbIndex array, before and after the sort of a call
    int *pi_idx[2] = {nullptr, nullptr};
    int pi_cur = 0;                             // which of the two holds the array between calls
    float *sort_k[2] = {nullptr, nullptr};   // intermediate runs of the sort (padded to whole runs of 4096)
    int *sort_v[2] = {nullptr, nullptr};
    float *sample_exp = nullptr;   // exp(logit / temperature - max) of one sampling step (k_sample_exp)
    bool pflash_ready = false;           // k_pflash's LDS attributes are set
    unsigned char *wide_mem = nullptr;   // what the workgroups of the one-launch sampling step hand each other (k_sample_wide)
};

namespace l2j {

// Every entry point that takes a context passes its return code through here: the text of a failure is kept in the
// context as well as in the calling thread, so that a caller whose threads migrate between calls (Java virtual threads)
// can fetch it with l2j_ctx_last_error.
inline int ctx_rc(l2j_ctx *c, int rc)
{
    if (rc < 0 && c) {
        std::lock_guard<std::mutex> lock(c->err_mu);
        c->last_err = g_err;
    }
    return rc;
}

inline uint64_t tensor_floats(const l2j_config &c, int t)
{
    const uint64_t L = c.n_layers, dim = c.dim, hid = c.hidden_dim, hs = c.dim / c.n_heads;
    const uint64_t kvd = (uint64_t)c.n_kv_heads * hs;
    switch (t) {
    case L2J_TOK_EMB: case L2J_WCLS: return (uint64_t)c.vocab_size * dim;
    case L2J_RMS_ATT: case L2J_RMS_FFN: return L * dim;
    case L2J_WQ: case L2J_WO: return L * dim * dim;
    case L2J_WK: case L2J_WV: return L * dim * kvd;
    case L2J_W1: case L2J_W2: case L2J_W3: return L * dim * hid;
    case L2J_RMS_FINAL: return dim;
    default: return 0;
    }
}

inline bool is_quant(int t) { return t >= L2J_RMS_ATT && t <= L2J_RMS_FINAL; }
inline bool per_layer(int t) { return t >= L2J_RMS_ATT && t <= L2J_W3; }

template <typename T>
int dev_alloc(T **p, uint64_t count)
{
    HIPCHK(hipMalloc(reinterpret_cast<void **>(p), std::max<uint64_t>(count, 1) * sizeof(T)));
    return L2J_OK;
}

inline uint64_t quant_bytes_of(uint64_t weights) { return (weights / kGroup) * kGroupBytes + (weights % kGroup ? kGroupBytes : 0); }

// ---- l2j_forward.hip
extern std::mutex g_forward_mu;   // the whole-token kernel needs every compute unit: forwards of all contexts take turns
constexpr int kRepeatToken = 1;   // check_barrier_error: the context now launches phase by phase; run the token(s) again
int setup_forward(l2j_ctx *c);    // launch shapes, kernel attributes, scratch of the phases, graph capture (end of l2j_finalize)
void release_forward(l2j_ctx *c); // what setup_forward allocated
hipError_t launch_one_token(l2j_ctx *c);
int check_barrier_error(l2j_ctx *c);
int set_state(l2j_ctx *c, int token, int pos, int n_prompt);

// ---- l2j_sampler.hip
int resolve_scratch(int device);
void free_sampler(l2j_ctx *c);
int seed_sampler(l2j_ctx *c, int64_t rng_seed);
hipError_t launch_sampler(l2j_ctx *c, float temperature, float topp, float coin, bool in_loop);
// The samplers of the sequences of the batched decode (each the reference's Sampler object: generator, flags, its ProbIndex
// array twice) and what their steps work in; device memory, (sequence, stride) each.
struct BatchSamplers {
    int nseq = 0;
    SamplerState *ss = nullptr;
    float *pi_prob[2] = {nullptr, nullptr};
    int *pi_idx[2] = {nullptr, nullptr};
    size_t pi_stride = 0;
    float *sort_k[2] = {nullptr, nullptr};   // the sort's tiles and runs
    int *sort_v[2] = {nullptr, nullptr};
    size_t sort_stride = 0;
};
int alloc_batch_samplers(l2j_ctx *c, int nseq, BatchSamplers *bs);
void free_batch_samplers(BatchSamplers *bs);
// One sampling step for the sequences whose bit is set in `active` (cur: bit s = the copy of its array that sequence s's last
// top-p step left), on the rows of logits; the tokens go to token[s] and out[s * out_stride].
hipError_t launch_samplers(l2j_ctx *c, const BatchSamplers &bs, unsigned active, unsigned cur, float *logits, float temperature,
                           float topp, int *token, int *out, long out_stride);
// l2j_batch.hip: l2j_prefill without the lock (the decode loops call it holding it)
int prefill_positions(l2j_ctx *c, const int32_t *tokens, int32_t n, int32_t pos0, float *logits, double *seconds);
int check_sampler_status(l2j_ctx *c);
int check_sampler_args(float temperature, float topp);

// ---- l2j_batch.hip
void free_batch(l2j_ctx *c);                      // buffers, graph and tile-ordered copies of the batched path
void invalidate_batch_tiles(l2j_ctx *c, int tensor);   // the tensor's codes changed: its tile-ordered copy is stale

}  // namespace l2j
