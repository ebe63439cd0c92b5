// libllama2j_hip.so: device side of the C ABI declared in include/llama2j_hip.h.
// Owns device memory, converts the reference's weight formats to the streaming layout, captures
// the per-token launch sequence as a hipGraph and replays it.
#include "kernels.hpp"
#include "phase_kernels.hpp"
#include "sampler_kernels.hpp"
#include "batch_kernels.hpp"

#include <hip/hip_ext.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/llama2j_hip.h"
#include "host_internal.h"

using namespace l2j;

// Device memory of l2j_running_sums_noalloc: the terms and their sums of one call.  Every GPU the library runs on holds
// its own copy of the array until the process ends; in host code the name is only a handle for hipGetSymbolAddress.
static __device__ __align__(256) float scratch[kSampleMaxVocab];

namespace {

thread_local std::string g_err;

int fail(int code, const std::string &msg)
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
};

// The address of `scratch` on each device, looked up by the first l2j_create on that device (with the device current).
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
float *g_scratch_ptr[kMaxDevices] = {};

int resolve_scratch(int device)
{
    if (device < 0 || device >= kMaxDevices) return fail(L2J_E_ARG, "device ordinal above 63");
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (g_scratch_ptr[device]) return L2J_OK;
    float *p = nullptr;
    HIPCHK(hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(scratch)));
    if (!p) return fail(L2J_E_HIP, "hipGetSymbolAddress(scratch) returned a null address");
    // (the largest input needs more than the default 64 KB of dynamic LDS)
    const int lds = (((kSampleMaxVocab + kChainStep - 1) & ~(kChainStep - 1)) + kChainStep) * (int)sizeof(float);
    HIPCHK(hipFuncSetAttribute((const void *)k_running_sums<true>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    g_scratch_ptr[device] = p;
    return L2J_OK;
}

// Launch-shape and algorithm switches of a context.  kAuto = the library picks (by shape, at l2j_finalize).  A context
// starts from the process defaults (environment variable L2J_<NAME IN CAPITALS>, read once by l2j_create) and
// l2j_set_option overrides them per context; nothing reads the environment afterwards.
enum {
    OPT_THREADS = 0, OPT_GRID, OPT_ATTN_THREADS, OPT_ATTN_ROWS, OPT_ATTN_NSPLIT, OPT_FUSED_ATTN_ROWS, OPT_FUSED_ATTN_SPLITS,
    OPT_BARRIER_SPINS, OPT_FUSE, OPT_LAYERS_PER_LAUNCH, OPT_BY_VALUE, OPT_TOKEN_SPECIAL, OPT_SAMPLER_SCAN, OPT_SAMPLER_EXP_WGS,
    OPT_GRAPH, OPT_SELF_CONTAINED, OPT_GRAPH_TOKENS, OPT_FAST_STEPS, OPT_FALLBACK, OPT_COUNT
};
constexpr int kAuto = -1;
struct OptionDef {
    const char *name;
    int dflt;
    bool after_finalize;  // may still be changed once the launch shapes are fixed
};
const OptionDef kOptions[OPT_COUNT] = {
    {"threads", 1024, false},          // workgroup size of the weight-streaming kernels
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
};

int option_from_env(int i)
{
    char var[64] = "L2J_";
    size_t k = 4;
    for (const char *p = kOptions[i].name; *p && k + 1 < sizeof(var); p++) var[k++] = (char)toupper((unsigned char)*p);
    var[k] = 0;
    const char *v = getenv(var);
    return v && *v ? atoi(v) : kOptions[i].dflt;
}

}  // namespace

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
    double wall_clock_hz = 1e8;
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
};

namespace {

// Every entry point that takes a context passes its return code through here: the text of a failure is kept in the
// context as well as in the calling thread, so that a caller whose threads migrate between calls (Java virtual threads)
// can fetch it with l2j_ctx_last_error.
int ctx_rc(l2j_ctx *c, int rc)
{
    if (rc < 0 && c) {
        std::lock_guard<std::mutex> lock(c->err_mu);
        c->last_err = g_err;
    }
    return rc;
}

uint64_t tensor_floats(const l2j_config &c, int t)
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

bool is_quant(int t) { return t >= L2J_RMS_ATT && t <= L2J_RMS_FINAL; }
bool per_layer(int t) { return t >= L2J_RMS_ATT && t <= L2J_W3; }

int validate_config(const l2j_config &c)
{
    if (c.dim <= 0 || c.hidden_dim <= 0 || c.n_layers <= 0 || c.n_heads <= 0 || c.n_kv_heads <= 0 || c.vocab_size <= 0 ||
        c.seq_len <= 0)
        return fail(L2J_E_ARG, "config: every dimension must be positive");
    if (c.group_size != 256 || c.bits != 8) return fail(L2J_E_ARG, "config: only group_size 256 / 8 bits (J/Run.java:27-28)");
    if (c.dim % c.n_heads || c.n_heads % c.n_kv_heads) return fail(L2J_E_ARG, "config: dim %% n_heads or n_heads %% n_kv_heads != 0");
    const int hs = c.dim / c.n_heads;
    if (hs % 4 || hs > 256) return fail(L2J_E_ARG, "config: head_size must be a multiple of 4, at most 256");
    if (c.dim % 16 || c.hidden_dim % 16 || (c.n_kv_heads * hs) % 16)
        return fail(L2J_E_ARG, "config: dim, hidden_dim and kv_dim must be multiples of 16 (16-byte weight loads)");
    if ((uint64_t)c.hidden_dim * 4 + c.hidden_dim / 4 + 256 > 160 * 1024)
        return fail(L2J_E_ARG, "config: hidden_dim does not fit the 160 KB LDS");
    return L2J_OK;
}

template <typename T>
int dev_alloc(T **p, uint64_t count)
{
    HIPCHK(hipMalloc(reinterpret_cast<void **>(p), std::max<uint64_t>(count, 1) * sizeof(T)));
    return L2J_OK;
}

QMat qmat(const l2j_ctx *c, int t, uint64_t off)
{
    QMat m;
    m.codes = c->qt[t].codes;
    m.gs = c->qt[t].gs;
    m.off = (long)off;
    return m;
}

size_t mv_smem(int n) { return (size_t)n * 4 + (size_t)(n / 16) * 4 + 64 * sizeof(float); }

int attn_lpr(const l2j_ctx *c) { return c->head_size <= 64 ? 16 : c->head_size <= 128 ? 32 : 64; }

size_t attn_smem_for(const l2j_ctx *c, int threads)
{
    const int nent = (threads / 64) * (64 / attn_lpr(c));
    return (size_t)(3 * nent + 4 + nent * c->head_size + 1) * sizeof(float);
}

size_t attn_smem(const l2j_ctx *c) { return attn_smem_for(c, c->attn_threads); }

// k_token: the largest LDS need of its phases (rounded to 16 bytes), then its arrival counters
size_t phase_smem(const l2j_ctx *c)
{
    return (std::max(mv_smem(std::max(c->cfg.dim, c->cfg.hidden_dim)), attn_smem_for(c, c->pk_threads)) + 15) / 16 * 16;
}
size_t layer_smem(const l2j_ctx *c) { return phase_smem(c) + kTokenLdsExtra; }

static_assert(K_QKV == L2J_K_QKV && K_ATT == L2J_K_ATTENTION && K_WO == L2J_K_WO && K_W13 == L2J_K_W13 && K_W2 == L2J_K_W2 &&
              K_CLS == L2J_K_CLASSIFIER, "kernel classes of the C ABI and of the device code must agree");

MatvecPhase matvec_phase(const l2j_ctx *c, int kclass, int l) { return matvec_phase_of(c->geom, kclass, l); }
AttnPhase attn_phase(const l2j_ctx *c, int l) { return attn_phase_of(c->geom, l, c->attn_rows, c->attn_threads, c->attn_nsplit); }
ClsPhase cls_phase(const l2j_ctx *c) { return cls_phase_of(c->geom, c->pk_grid); }

void build_geom(l2j_ctx *c)
{
    const l2j_config &g = c->cfg;
    TokenGeom &t = c->geom;
    t.dim = g.dim; t.hidden = g.hidden_dim; t.n_layers = g.n_layers; t.n_heads = g.n_heads; t.kv_mul = c->kv_mul;
    t.head_size = c->head_size; t.kv_dim = c->kv_dim; t.seq_len = g.seq_len; t.vocab = g.vocab_size;
    t.exact_silu = (g.flags & L2J_F_EXACT_SILU) ? 1 : 0;
    t.threads = c->pk_threads;
    t.sd = (long)c->sd; t.sh = (long)c->sh;
    t.emb = c->emb; t.rmsw = c->rmsw; t.silu = c->silu; t.wcls = c->wcls; t.rope = c->rope;
    t.set_stride = (long)c->set_floats;
    t.x = c->x; t.xb = c->xb; t.hb = c->hb; t.q = c->q; t.kcache = c->kcache; t.vcache = c->vcache; t.logits = c->logits;
    t.wq = qmat(c, L2J_WQ, 0); t.wk = qmat(c, L2J_WK, 0); t.wv = qmat(c, L2J_WV, 0); t.wo = qmat(c, L2J_WO, 0);
    t.w1 = qmat(c, L2J_W1, 0); t.w2 = qmat(c, L2J_W2, 0); t.w3 = qmat(c, L2J_W3, 0);
    t.knew = c->knew; t.vnew = c->vnew; t.skv = (long)c->skv;
    t.attn_part = c->attn_part; t.attn_counters = c->counters; t.attn_nsplit = c->attn_nsplit;
    t.sqrt_hs = sqrtf((float)c->head_size);
    t.st = c->st; t.cls_part = c->cls_part; t.tstamp = c->tstamp; t.prompt = c->prompt; t.out_tokens = c->out_tokens;
    t.bar_ctr = c->bar_ctr; t.nbar = c->nbar; t.fault = c->fault;
}

// Every buffer a kernel may touch exists (checked on the host before anything is launched).
bool geom_complete(const TokenGeom &t)
{
    const void *ptrs[] = {t.emb, t.rmsw, t.silu, t.wcls, t.rope, t.x, t.xb, t.hb, t.q, t.kcache, t.vcache, t.logits,
                          t.wq.codes, t.wq.gs, t.wk.codes, t.wk.gs, t.wv.codes, t.wv.gs, t.wo.codes, t.wo.gs,
                          t.w1.codes, t.w1.gs, t.w2.codes, t.w2.gs, t.w3.codes, t.w3.gs,
                          t.knew, t.vnew, t.attn_part, t.attn_counters, t.st, t.cls_part, t.tstamp, t.prompt, t.out_tokens, t.bar_ctr, t.fault};
    for (const void *p : ptrs)
        if (!p) return false;
    return true;
}

// Splits per attention head inside k_token: one (head, split) item per workgroup at most.
int fused_splits(const l2j_ctx *c)
{
    const int o = c->opt[OPT_FUSED_ATTN_SPLITS];
    return std::max(1, o != kAuto ? o : c->pk_grid / c->cfg.n_heads);
}

// Marks the activation vectors unwritten: set 0 before a k_token that hands over by value, both sets (and the
// per-workgroup classifier results) before a self-contained one whose vectors others have written.
hipError_t launch_fill_unset(const l2j_ctx *c, hipStream_t s)
{
    FillArgs f{};
    f.p = c->acts;
    f.n = (long)((c->self_contained & 1) ? 2 * c->set_floats : c->set_floats);
    f.part = c->cls_part;
    f.nparts = (c->self_contained & 2) ? c->pk_grid : 0;
    hipLaunchKernelGGL(k_fill_unset, dim3(c->n_cu), dim3(1024), 0, s, f);
    return hipGetLastError();
}

// The instantiation of k_token for this context: by lanes per cache row, and, for the shapes of the published models,
// by the chunks per lane that make a row of dim / hidden codes one step (tu_for); the general instantiation runs any shape.
template <typename F>
auto with_token_kernel(const l2j_ctx *c, F f)
{
    const int lpr = attn_lpr(c);
    const int tud = tu_for(c->cfg.dim), tuh = tu_for(c->cfg.hidden_dim);
    const bool special = c->opt[OPT_TOKEN_SPECIAL] != 0;
    if (special && c->opt[OPT_FAST_STEPS] != 0 && lpr == 32 && c->cfg.dim == 1024 * tud && c->cfg.dim % 256 == 0) {
        // (its Wo phase stages one 16-byte word per thread and folds one item per wave: run_by_quarters)
        if (tud == kTU && c->pk_threads == 1024 && 16 * c->pk_grid >= c->cfg.dim / 2) return f(k_token<32, kTU, kTU, true>);
        if (tud == 5) return f(k_token<32, 5, kTU, true>);
    }
    if (special && lpr == 16 && tud == 1 && tuh == 1) return f(k_token<16, 1, 1>);
    if (special && lpr == 16 && tud == 1 && tuh == 2) return f(k_token<16, 1, 2>);
    if (special && lpr == 32 && tud == 5) return f(k_token<32, 5, kTU>);
    if (lpr == 16) return f(k_token<16>);
    if (lpr == 32) return f(k_token<32>);
    return f(k_token<64>);
}


// Layers [l0, l1) (and the classifier after the last layer) in one launch of k_token.
hipError_t launch_layers(const l2j_ctx *c, int l0, int l1, hipStream_t s, hipEvent_t e0 = nullptr, hipEvent_t e1 = nullptr)
{
    TokenArgs a{};
    a.g = c->geom;
    a.l0 = l0; a.l1 = l1; a.with_cls = l1 == c->cfg.n_layers;
    a.attn_rows = c->fused_attn_rows;
    a.attn_splits = fused_splits(c);
    a.maxspin = std::max(0, c->opt[OPT_BARRIER_SPINS]);  // each poll is a memory round trip, >= 1 us
    a.ctr_off = (int)(phase_smem(c) / sizeof(float));
    a.by_value = c->by_value ? 1 : 0;
    a.self_contained = l0 == 0 && l1 == c->cfg.n_layers ? c->self_contained : 0;
    const dim3 grid(c->pk_grid), block(c->pk_threads);
    const size_t smem = layer_smem(c);
    with_token_kernel(c, [&](auto kernel) {
        if (e0) hipExtLaunchKernelGGL(kernel, grid, block, (unsigned)smem, s, e0, e1, 0, a);
        else hipLaunchKernelGGL(kernel, grid, block, smem, s, a);
        return 0;
    });
    return hipGetLastError();
}

template <typename K, typename A>
hipError_t launch1(K kernel, dim3 grid, dim3 block, size_t smem, hipStream_t s, const A &args, hipEvent_t e0, hipEvent_t e1)
{
    if (e0) {
        hipExtLaunchKernelGGL(kernel, grid, block, (unsigned)smem, s, e0, e1, 0, args);
    } else {
        hipLaunchKernelGGL(kernel, grid, block, smem, s, args);
    }
    return hipGetLastError();
}

// k_matvec<MODE, TU> for rows of n codes streamed as row pairs (QKV, W13, and Wo / W2 with rows of up to 320 chunks).
template <int MODE, typename A>
hipError_t launch_pairs(int n, dim3 grid, dim3 block, size_t smem, hipStream_t s, const A &args, hipEvent_t e0, hipEvent_t e1)
{
    switch (tu_for(n)) {
    case 1: return launch1(k_matvec<MODE, 1>, grid, block, smem, s, args, e0, e1);
    case 2: return launch1(k_matvec<MODE, 2>, grid, block, smem, s, args, e0, e1);
    case 5: return launch1(k_matvec<MODE, 5>, grid, block, smem, s, args, e0, e1);
    default: return launch1(k_matvec<MODE, kTU>, grid, block, smem, s, args, e0, e1);
    }
}

// One kernel class of layer l.  Optional start/stop events bracket the kernel itself.
hipError_t launch_class(const l2j_ctx *c, int kclass, int l, hipStream_t s, hipEvent_t e0 = nullptr, hipEvent_t e1 = nullptr)
{
    const dim3 grid(c->pk_grid), block(c->pk_threads);
    switch (kclass) {
    case L2J_K_QKV: return launch_pairs<PH_QKV>(c->cfg.dim, grid, block, mv_smem(c->cfg.dim), s, matvec_phase(c, kclass, l), e0, e1);
    case L2J_K_W13: return launch_pairs<PH_W13>(c->cfg.dim, grid, block, mv_smem(c->cfg.dim), s, matvec_phase(c, kclass, l), e0, e1);
    case L2J_K_WO:
    case L2J_K_W2: {
        const int n = kclass == L2J_K_WO ? c->cfg.dim : c->cfg.hidden_dim;
        if (n / 16 <= 320) return launch_pairs<PH_RES>(n, grid, block, mv_smem(n), s, matvec_phase(c, kclass, l), e0, e1);
        const int mode = row_mode(n);  // long rows: one row per wave keeps every wave busy
        if (mode == PH_ROW6) return launch1(k_matvec<PH_ROW6>, grid, block, mv_smem(n), s, matvec_phase(c, kclass, l), e0, e1);
        return launch1(k_matvec<PH_ROW>, grid, block, mv_smem(n), s, matvec_phase(c, kclass, l), e0, e1);
    }
    case L2J_K_ATTENTION: {
        const dim3 ag(c->attn_grid), ab(c->attn_threads);
        const int lpr = attn_lpr(c);
        if (lpr == 16) return launch1(k_attention<16>, ag, ab, attn_smem(c), s, attn_phase(c, l), e0, e1);
        if (lpr == 32) return launch1(k_attention<32>, ag, ab, attn_smem(c), s, attn_phase(c, l), e0, e1);
        return launch1(k_attention<64>, ag, ab, attn_smem(c), s, attn_phase(c, l), e0, e1);
    }
    case L2J_K_CLASSIFIER:
        return launch1(k_classifier, grid, block, mv_smem(c->cfg.dim), s, cls_phase(c), e0, e1);
    }
    return hipErrorInvalidValue;
}

hipError_t tap_copy(l2j_ctx *c, int which, int l, const float *src, uint64_t n, hipStream_t s)
{
    return hipMemcpyAsync(c->taps[which] + (uint64_t)l * n, src, n * sizeof(float), hipMemcpyDeviceToDevice, s);
}

// The launch sequence of one token (J/Run.java:62-169).  With taps, per-layer copies follow each
// kernel (the pattern of Mode.TEST).
hipError_t launch_token(l2j_ctx *c, hipStream_t s, bool taps, hipEvent_t e0 = nullptr, hipEvent_t e1 = nullptr)
{
    const l2j_config &g = c->cfg;
    hipError_t e;
    if (c->fused && !taps) {
        // (a kernel that alternates its sets of vectors marks them itself; whoever launches it marks both first when others wrote them)
        if (c->by_value && !(c->self_contained & 1) && (e = launch_fill_unset(c, s)) != hipSuccess) return e;
        for (int l = 0; l < g.n_layers; l += c->layers_per_launch)
            if ((e = launch_layers(c, l, std::min(g.n_layers, l + c->layers_per_launch), s, e0, e1)) != hipSuccess) return e;
        if (c->self_contained & 2) return hipSuccess;
        hipLaunchKernelGGL(k_finish, dim3(1), dim3(256), 0, s, cls_phase(c));
        return hipGetLastError();
    }
    for (int l = 0; l < g.n_layers; l++) {
        const uint64_t kvoff = (uint64_t)l * g.seq_len * c->kv_dim;
        if ((e = launch_class(c, L2J_K_QKV, l, s)) != hipSuccess) return e;
        if (taps) {  // rows of the caches at the current position; pos is known on the host in this mode
            const uint64_t row = (uint64_t)c->h_st->pos * c->kv_dim;
            if ((e = tap_copy(c, L2J_B_Q, l, c->q + l * c->sd, g.dim, s)) != hipSuccess) return e;
            if ((e = tap_copy(c, L2J_B_K, l, c->kcache + kvoff + row, c->kv_dim, s)) != hipSuccess) return e;
            if ((e = tap_copy(c, L2J_B_V, l, c->vcache + kvoff + row, c->kv_dim, s)) != hipSuccess) return e;
        }
        if ((e = launch_class(c, L2J_K_ATTENTION, l, s)) != hipSuccess) return e;
        if (taps && (e = tap_copy(c, L2J_B_XB, l, c->xb + l * c->sd, g.dim, s)) != hipSuccess) return e;
        if ((e = launch_class(c, L2J_K_WO, l, s)) != hipSuccess) return e;
        if (taps && (e = tap_copy(c, L2J_B_XB2, l, c->x + (2 * l + 1) * c->sd, g.dim, s)) != hipSuccess) return e;
        if ((e = launch_class(c, L2J_K_W13, l, s)) != hipSuccess) return e;
        if (taps && (e = tap_copy(c, L2J_B_HB, l, c->hb + l * c->sh, g.hidden_dim, s)) != hipSuccess) return e;
        if ((e = launch_class(c, L2J_K_W2, l, s)) != hipSuccess) return e;
        if (taps && (e = tap_copy(c, L2J_B_X, l, c->x + (2 * l + 2) * c->sd, g.dim, s)) != hipSuccess) return e;
    }
    if ((e = launch_class(c, L2J_K_CLASSIFIER, 0, s)) != hipSuccess) return e;
    hipLaunchKernelGGL(k_finish, dim3(1), dim3(256), 0, s, cls_phase(c));
    return hipGetLastError();
}

// With option "graph" = 0 the kernels are launched one by one instead of replaying the graph (for tools that do
// not follow graph launches).
hipError_t clean_activations(l2j_ctx *c)
{
    if (!(c->self_contained & 1) || !c->acts_dirty) return hipSuccess;
    c->acts_dirty = false;
    return launch_fill_unset(c, c->stream);
}

hipError_t launch_one_token(l2j_ctx *c)
{
    hipError_t e = clean_activations(c);
    if (e != hipSuccess) return e;
    return c->graph_exec ? hipGraphLaunch(c->graph_exec, c->stream) : launch_token(c, c->stream, false);
}

// The whole-token kernel needs every compute unit of the device for itself, so forwards of different contexts
// of this process take turns (each entry point synchronizes before it returns).
std::mutex g_forward_mu;

void destroy_graph(l2j_ctx *c)
{
    if (c->graph_exec) (void)hipGraphExecDestroy(c->graph_exec);
    if (c->graph) (void)hipGraphDestroy(c->graph);
    if (c->graph_n_exec) (void)hipGraphExecDestroy(c->graph_n_exec);
    if (c->graph_n) (void)hipGraphDestroy(c->graph_n);
    c->graph_exec = c->graph_n_exec = nullptr;
    c->graph = c->graph_n = nullptr;
}

// One token per replay, and graph_tokens tokens per replay for the decode loops: the kernels read the token, the
// position and the prompt from device memory, so the same nodes serve every position.
int capture_graphs(l2j_ctx *c)
{
    destroy_graph(c);
    if (c->opt[OPT_GRAPH] == 0) return L2J_OK;
    c->graph_tokens = std::max(1, std::min(c->opt[OPT_GRAPH_TOKENS], c->cfg.seq_len));
    for (int which = 0; which < (c->graph_tokens > 1 ? 2 : 1); which++) {
        hipGraph_t *gr = which ? &c->graph_n : &c->graph;
        hipGraphExec_t *ex = which ? &c->graph_n_exec : &c->graph_exec;
        HIPCHK(hipStreamBeginCapture(c->stream, hipStreamCaptureModeThreadLocal));
        hipError_t le = hipSuccess;
        for (int i = 0; i < (which ? c->graph_tokens : 1) && le == hipSuccess; i++) le = launch_token(c, c->stream, false);
        hipError_t ce = hipStreamEndCapture(c->stream, gr);
        if (le != hipSuccess) return fail(L2J_E_HIP, std::string("capture launch: ") + hipGetErrorString(le));
        HIPCHK(ce);
        HIPCHK(hipGraphInstantiate(ex, *gr, nullptr, nullptr, 0));
    }
    return L2J_OK;
}

constexpr int kRepeatToken = 1;  // check_barrier_error: the context now launches phase by phase; run the token(s) again

// After a synchronize: a workgroup whose bounded wait ran out has set the flag.  The whole-token kernel needs all its
// workgroups resident at once; when something else holds compute units (another process on the GPU) its waits run
// out.  With the "fallback" option the context then gives the whole-token kernel up for good: one launch per phase
// needs no residency, and the caller repeats what failed (kRepeatToken).
int check_barrier_error(l2j_ctx *c)
{
    if (!c->fused) return L2J_OK;
    HIPCHK(hipMemcpy(c->h_fault, c->fault, sizeof(int), hipMemcpyDeviceToHost));
    if (*c->h_fault == 0) return L2J_OK;
    HIPCHK(hipStreamSynchronize(c->stream));  // (tokens enqueued ahead fall through their waits as well)
    *c->h_fault = 0;
    HIPCHK(hipMemcpy(c->fault, c->h_fault, sizeof(int), hipMemcpyHostToDevice));
    HIPCHK(hipMemset(c->bar_ctr, 0, (size_t)c->nbar * kBarStride * sizeof(unsigned)));  // leave the context usable
    HIPCHK(hipMemset(c->counters, 0, ((size_t)c->cfg.n_layers * c->cfg.n_heads + 1) * sizeof(unsigned)));
    c->acts_dirty = true;
    if (c->opt[OPT_FALLBACK] != 0) {
        c->fused = false;
        c->by_value = false;
        c->self_contained = 0;
        c->opt[OPT_FUSE] = 0;
        int rc = capture_graphs(c);
        if (rc) return rc;
        return kRepeatToken;
    }
    return fail(L2J_E_HIP, "a bounded wait of the whole-token kernel ran out (barrier or input vector; its workgroups were not all resident)");
}

int set_state(l2j_ctx *c, int token, int pos, int n_prompt)
{
    c->h_st->token = token;
    c->h_st->pos = pos;
    c->h_st->n_prompt = n_prompt;
    // (the device owns DevState::epoch: every token adds one, and a self-contained k_token picks its set of vectors by it)
    HIPCHK(hipMemcpyAsync(c->st, c->h_st, offsetof(DevState, epoch), hipMemcpyHostToDevice, c->stream));
    return L2J_OK;
}

int check_forward_args(l2j_ctx *c, int32_t token, int32_t pos)
{
    if (!c) return fail(L2J_E_ARG, "null context");
    if (!c->finalized) return fail(L2J_E_STATE, "forward before l2j_finalize");
    if (token < 0 || token >= c->cfg.vocab_size) return fail(L2J_E_ARG, "token out of range");
    if (pos < 0 || pos >= c->cfg.seq_len) return fail(L2J_E_ARG, "pos out of range");
    HIPCHK(hipSetDevice(c->cfg.device));
    return L2J_OK;
}

int unpack_into(l2j_ctx *c, QTensor &t, uint64_t group0, const uint8_t *ref_bytes, uint64_t ngroups)
{
    // staged through a device buffer in slices of at most 64 MiB
    const uint64_t slice_groups = (64ull << 20) / kGroupBytes;
    uint8_t *stage = nullptr;
    HIPCHK(hipMalloc(reinterpret_cast<void **>(&stage), std::min(ngroups, slice_groups) * kGroupBytes));
    int rc = L2J_OK;
    for (uint64_t g = 0; g < ngroups && rc == L2J_OK; g += slice_groups) {
        const uint64_t ng = std::min(slice_groups, ngroups - g);
        hipError_t e = hipMemcpy(stage, ref_bytes + g * kGroupBytes, ng * kGroupBytes, hipMemcpyHostToDevice);
        if (e == hipSuccess) {
            const int grid = (int)std::min<uint64_t>(ng, 1u << 20);
            hipLaunchKernelGGL(k_unpack_groups, dim3(grid), dim3(64), 0, c->stream, stage, (long)ng, t.codes + (group0 + g) * kGroup,
                               t.gs + group0 + g, t.mm + group0 + g);
            e = hipGetLastError();
            if (e == hipSuccess) e = hipStreamSynchronize(c->stream);
        }
        if (e != hipSuccess) rc = fail(L2J_E_HIP, std::string("upload: ") + hipGetErrorString(e));
    }
    (void)hipFree(stage);
    return rc;
}


uint64_t quant_bytes_of(uint64_t weights) { return (weights / kGroup) * kGroupBytes + (weights % kGroup ? kGroupBytes : 0); }

// ---- device sampler ------------------------------------------------------------------------------------

void free_sampler(l2j_ctx *c)
{
    (void)hipFree(c->ss);
    c->ss = nullptr;
    for (int i = 0; i < 2; i++) {
        (void)hipFree(c->pi_prob[i]);
        (void)hipFree(c->pi_idx[i]);
        c->pi_prob[i] = nullptr;
        c->pi_idx[i] = nullptr;
    }
    for (int i = 0; i < 2; i++) {
        (void)hipFree(c->sort_k[i]); (void)hipFree(c->sort_v[i]);
        c->sort_k[i] = nullptr; c->sort_v[i] = nullptr;
    }
    (void)hipFree(c->sample_exp);
    c->sample_exp = nullptr;
    if (c->h_ss) (void)hipHostFree(c->h_ss);
    c->h_ss = nullptr;
}

// dynamic LDS of the sampler's one-workgroup kernels: the terms, padded to whole steps of the single-lane sum plus one
size_t sampler_lds_bytes(int n)
{
    return n <= kSampleMaxVocab ? (size_t)(((n + kChainStep - 1) & ~(kChainStep - 1)) + kChainStep) * sizeof(float) : 0;
}

int alloc_sampler(l2j_ctx *c)
{
    const int n = c->cfg.vocab_size;
    int rc;
    for (int i = 0; i < 2; i++) {
        if ((rc = dev_alloc(&c->pi_prob[i], (uint64_t)n + 4))) return rc;   // (read in 16-byte words: stage_terms)
        if ((rc = dev_alloc(&c->pi_idx[i], (uint64_t)n))) return rc;
    }
    if ((rc = dev_alloc(&c->sample_exp, (uint64_t)n + 4))) return rc;
    HIPCHK(hipHostMalloc((void **)&c->h_ss, sizeof(SamplerState), hipHostMallocDefault));
    const int npad = (n + kSortRun - 1) / kSortRun * kSortRun;
    for (int i = 0; i < 2; i++) {
        if ((rc = dev_alloc(&c->sort_k[i], (uint64_t)npad))) return rc;
        if ((rc = dev_alloc(&c->sort_v[i], (uint64_t)npad))) return rc;
    }
    if (n <= kSampleMaxVocab) {
        HIPCHK(hipFuncSetAttribute((const void *)k_merge_runs, hipFuncAttributeMaxDynamicSharedMemorySize, npad * (int)sizeof(float)));
        const int lds = (int)sampler_lds_bytes(n);
        HIPCHK(hipFuncSetAttribute((const void *)k_sample_probs<true>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        HIPCHK(hipFuncSetAttribute((const void *)k_topp_pick<true>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    }
    return dev_alloc(&c->ss, 1);   // last: its presence says that the sampler is complete
}

int ensure_sampler(l2j_ctx *c)
{
    if (c->ss) return L2J_OK;
    const int n = c->cfg.vocab_size;
    if (n < 2) return fail(L2J_E_SIZE, "device sampler: vocab_size below 2");
    const int rc = alloc_sampler(c);
    if (rc) free_sampler(c);
    return rc;
}

// new Sampler(rngSeed, vocab_size) (J/Sampler.java:24-31): Random(seed) scrambles its seed, every ProbIndex is (0, 0)
int seed_sampler(l2j_ctx *c, int64_t rng_seed)
{
    int rc = ensure_sampler(c);
    if (rc) return rc;
    memset(c->h_ss, 0, sizeof(SamplerState));
    c->h_ss->rng = ((unsigned long long)rng_seed ^ kJavaRandMult) & kJavaRandMask;
    HIPCHK(hipMemcpyAsync(c->ss, c->h_ss, sizeof(SamplerState), hipMemcpyHostToDevice, c->stream));
    const size_t n = (size_t)c->cfg.vocab_size;
    for (int i = 0; i < 2; i++) {
        HIPCHK(hipMemsetAsync(c->pi_prob[i], 0, n * sizeof(float), c->stream));
        HIPCHK(hipMemsetAsync(c->pi_idx[i], 0, n * sizeof(int), c->stream));
    }
    HIPCHK(hipStreamSynchronize(c->stream));
    c->pi_cur = 0;
    return L2J_OK;
}

// The sampling step of J/Run.java:643-665 on c->logits; in_loop: the token replaces what k_finish stored.
hipError_t launch_sampler(l2j_ctx *c, float temperature, float topp, float coin, bool in_loop)
{
    const int n = c->cfg.vocab_size;
    const int cur = c->pi_cur, other = cur ^ 1;
    SampleArgs a{};
    a.logits = c->logits; a.n = n;
    a.temperature = temperature; a.topp = topp; a.coin = coin;
    a.plain = (double)topp > 0.999;
    a.ss = c->ss;
    a.cand_prob = c->pi_prob[cur]; a.cand_idx = c->pi_idx[cur];
    a.sorted_prob = c->pi_prob[other]; a.sorted_idx = c->pi_idx[other];
    a.st = in_loop ? c->st : nullptr;
    a.out_tokens = c->out_tokens;
    a.scan = c->opt[OPT_SAMPLER_SCAN] != 0 ? 1 : 0;
    const bool in_lds = n <= kSampleMaxVocab;   // else the kernels work in device memory, where k_sample_exp leaves the exponentials
    const int exp_wgs = std::min(1024, std::max(in_lds ? 0 : 1, c->opt[OPT_SAMPLER_EXP_WGS]));   // 0: the exponentials in k_sample_probs' one workgroup
    a.expbuf = exp_wgs > 0 ? c->sample_exp : nullptr;
    if (a.expbuf) {
        hipLaunchKernelGGL(k_sample_exp, dim3(exp_wgs), dim3(1024), 0, c->stream, a);
        hipError_t ee = hipGetLastError();
        if (ee != hipSuccess) return ee;
    }
    const size_t lds = sampler_lds_bytes(n);
    if (in_lds) hipLaunchKernelGGL(k_sample_probs<true>, dim3(1), dim3(1024), lds, c->stream, a);
    else hipLaunchKernelGGL(k_sample_probs<false>, dim3(1), dim3(1024), 0, c->stream, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || a.plain) return e;
    // J/Sampler.java:97 by counting kernels: tiles, runs of tiles, then all runs at once (in LDS) or sixteen at a time
    const int npad = (n + kSortRun - 1) / kSortRun * kSortRun;
    hipLaunchKernelGGL(k_sort_tiles, dim3(npad / kSortTile), dim3(kSortTile), 0, c->stream, c->pi_prob[cur], c->pi_idx[cur], n,
                       c->sort_k[0], c->sort_v[0]);
    hipLaunchKernelGGL(k_merge_tiles, dim3(npad / kSortRun, 16), dim3(256), 0, c->stream, c->sort_k[0], c->sort_v[0], c->sort_k[1], c->sort_v[1]);
    if (in_lds) {
        hipLaunchKernelGGL(k_merge_runs, dim3(npad / 256), dim3(256), (size_t)npad * sizeof(float), c->stream, c->sort_k[1], c->sort_v[1], n,
                           npad, c->pi_prob[other], c->pi_idx[other]);
    } else {
        int from = 1;
        for (long run_len = kSortRun; run_len < npad; run_len *= kSortFanIn, from ^= 1) {
            const long group_len = run_len * kSortFanIn;
            const bool last = group_len >= npad;
            hipLaunchKernelGGL(k_merge_far, dim3(npad / 256), dim3(256), 0, c->stream, c->sort_k[from], c->sort_v[from], npad,
                               last ? n : npad, (int)run_len, (int)group_len, last ? c->pi_prob[other] : c->sort_k[from ^ 1],
                               last ? c->pi_idx[other] : c->sort_v[from ^ 1]);
        }
    }
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    a.sorted_prob = c->pi_prob[other]; a.sorted_idx = c->pi_idx[other];   // the array stays there until the next call
    c->pi_cur = other;
    if (in_lds) hipLaunchKernelGGL(k_topp_pick<true>, dim3(1), dim3(1024), lds, c->stream, a);
    else hipLaunchKernelGGL(k_topp_pick<false>, dim3(1), dim3(1024), 0, c->stream, a);
    return hipGetLastError();
}

// After a synchronize with h_ss read back: the reference's exceptions as an error return; the flag is cleared.
int check_sampler_status(l2j_ctx *c)
{
    const int st = c->h_ss->nan;
    if (!st) return L2J_OK;
    c->h_ss->nan = 0;
    HIPCHK(hipMemcpy(&c->ss->nan, &c->h_ss->nan, sizeof(int), hipMemcpyHostToDevice));
    if (st & 1) return fail(L2J_E_ARG, "sampler: NaN among the logits (J/Sampler.java:88-90)");
    return fail(L2J_E_ARG, "sampler: no probability reaches the top-p cutoff (ArrayIndexOutOfBoundsException at J/Sampler.java:119)");
}

int check_sampler_args(float temperature, float topp)
{
    if (!(temperature >= 0.0f) || !(topp >= 0.0f && topp <= 1.0f)) return fail(L2J_E_ARG, "temperature must be >= 0 and topp in [0, 1]");
    return L2J_OK;
}

// J/Run.java:611-685; temperature 0 is the greedy loop, else every unforced token is sampled on the device.
int decode_loop(l2j_ctx *c, const int32_t *prompt, int32_t n_prompt, int32_t steps, bool sampled, float temperature, float topp,
                int64_t rng_seed, int32_t *out_tokens, int32_t *n_out, double *seconds)
{
    if (!c || !out_tokens || !n_out || (n_prompt > 0 && !prompt) || n_prompt < 0) return fail(L2J_E_ARG, "bad argument");
    if (!c->finalized) return fail(L2J_E_STATE, "decode before l2j_finalize");
    HIPCHK(hipSetDevice(c->cfg.device));
    const int S = c->cfg.seq_len;
    if (steps <= 0 || steps > S) steps = S;  // J/Run.java:599-603
    const int np = std::min(n_prompt, S);
    for (int i = 0; i < np; i++)
        if (prompt[i] < 0 || prompt[i] >= c->cfg.vocab_size) return fail(L2J_E_ARG, "prompt id out of range");
    int rc;
    if (sampled && (rc = seed_sampler(c, rng_seed))) return rc;  // J/Run.java:620
    if (np > 0) {
        memcpy(c->h_tokens, prompt, (size_t)np * sizeof(int));
        HIPCHK(hipMemcpyAsync(c->prompt, c->h_tokens, (size_t)np * sizeof(int), hipMemcpyHostToDevice, c->stream));
        HIPCHK(hipStreamSynchronize(c->stream));
    }
    if ((rc = set_state(c, 1, 0, np))) return rc;  // token 1 = BOS at pos 0 (J/Run.java:614)

    // The stop rule (next == 1) is checked per batch of tokens, and the clock runs from the end of the first token to
    // the end of the token that ended the loop.
    float total_ms = 0.f;
    int pos = 0;
    bool stopped = false;
    if (!sampled) {
        // Greedy: the last kernel of every token stores the device's wall clock for its position; a full batch is one
        // replay of the multi-token graph; and the next batch is enqueued before the host waits for the results of
        // this one, so the GPU does not idle while the host looks for the stop token (a loop that stops has then
        // run up to one batch too many, whose outputs are dropped).
        const int batch = std::max(32, c->graph_tokens);
        while ((int)c->events.size() < 2) {
            hipEvent_t ev;
            HIPCHK(hipEventCreate(&ev));
            c->events.push_back(ev);
        }
        unsigned long long t_first = 0, t_last = 0;
        int enq = 0, nbatch = 0, done_batches = 0;  // positions enqueued; batches enqueued and processed
        auto enqueue = [&]() -> int {
            const int nb = std::min(batch, steps - enq);
            if (c->graph_n_exec && nb == c->graph_tokens) {
                HIPCHK(clean_activations(c));
                HIPCHK(hipGraphLaunch(c->graph_n_exec, c->stream));
            } else {
                for (int i = 0; i < nb; i++) HIPCHK(launch_one_token(c));
            }
            HIPCHK(hipMemcpyAsync(c->h_tokens + enq, c->out_tokens + enq, (size_t)nb * sizeof(int), hipMemcpyDeviceToHost, c->stream));
            HIPCHK(hipMemcpyAsync(c->h_tstamp + enq, c->tstamp + enq, (size_t)nb * sizeof(unsigned long long), hipMemcpyDeviceToHost, c->stream));
            HIPCHK(hipEventRecord(c->events[nbatch & 1], c->stream));
            enq += nb;
            nbatch++;
            return L2J_OK;
        };
        while (pos < steps && !stopped) {
            if (enq == pos && (rc = enqueue())) return rc;
            const int nb = std::min(batch, steps - pos);  // the batch that starts at pos
            if (enq < steps && nbatch == done_batches + 1 && (rc = enqueue())) return rc;
            HIPCHK(hipEventSynchronize(c->events[done_batches & 1]));
            done_batches++;
            if ((rc = check_barrier_error(c))) return rc;
            int used = nb;
            for (int i = 0; i < nb; i++) {
                out_tokens[pos + i] = c->h_tokens[pos + i];
                if (c->h_tokens[pos + i] == 1) {  // J/Run.java:670-672
                    used = i + 1;
                    stopped = true;
                    break;
                }
            }
            if (pos == 0) t_first = c->h_tstamp[0];
            t_last = c->h_tstamp[pos + used - 1];
            pos += used;
        }
        HIPCHK(hipStreamSynchronize(c->stream));  // a batch enqueued ahead of a stop
        if ((rc = check_barrier_error(c))) return rc;
        total_ms = (float)((double)(t_last - t_first) / c->wall_clock_hz * 1e3);
    } else {
        // Sampled: the sampler's kernels follow each token's graph, and an event after every token marks its end.
        const int batch = 32;
        while ((int)c->events.size() < batch + 1) {
            hipEvent_t ev;
            HIPCHK(hipEventCreate(&ev));
            c->events.push_back(ev);
        }
        hipEvent_t ev_first = c->events[batch];
        while (pos < steps && !stopped) {
            const int nb = std::min(batch, steps - pos);
            for (int i = 0; i < nb; i++) {
                HIPCHK(launch_one_token(c));
                if (pos + i >= np) HIPCHK(launch_sampler(c, temperature, topp, -1.0f, true));  // J/Run.java:635-665
                if (pos + i == 0) HIPCHK(hipEventRecord(ev_first, c->stream));
                HIPCHK(hipEventRecord(c->events[i], c->stream));
            }
            HIPCHK(hipMemcpyAsync(c->h_tokens, c->out_tokens + pos, (size_t)nb * sizeof(int), hipMemcpyDeviceToHost, c->stream));
            HIPCHK(hipMemcpyAsync(c->h_ss, c->ss, sizeof(SamplerState), hipMemcpyDeviceToHost, c->stream));
            HIPCHK(hipStreamSynchronize(c->stream));
            if ((rc = check_barrier_error(c))) return rc;
            if ((rc = check_sampler_status(c))) return rc;
            int used = nb;
            for (int i = 0; i < nb; i++) {
                out_tokens[pos + i] = c->h_tokens[i];
                if (c->h_tokens[i] == 1) {  // J/Run.java:670-672
                    used = i + 1;
                    stopped = true;
                    break;
                }
            }
            if (pos + used - 1 > 0) HIPCHK(hipEventElapsedTime(&total_ms, ev_first, c->events[used - 1]));
            pos += used;
        }
    }
    *n_out = pos;
    if (seconds) *seconds = (double)total_ms * 1e-3;
    return L2J_OK;
}

}  // namespace

// ------------------------------------------------------------------------------------------
// C ABI
// ------------------------------------------------------------------------------------------

extern "C" {

const char *l2j_last_error(void) { return g_err.c_str(); }

void l2j_set_error_(const char *msg) { g_err = msg ? msg : ""; }

int l2j_ctx_last_error(l2j_ctx *c, char *buf, int32_t cap)
{
    if (!c || !buf || cap <= 0) return fail(L2J_E_ARG, "null argument");
    std::lock_guard<std::mutex> lock(c->err_mu);
    const size_t n = std::min(c->last_err.size(), (size_t)cap - 1);
    memcpy(buf, c->last_err.data(), n);
    buf[n] = 0;
    return (int)n;
}

int l2j_device_count(void)
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

int l2j_create(const l2j_config *cfg, l2j_ctx **out)
{
    if (!cfg || !out) return fail(L2J_E_ARG, "l2j_create: null argument");
    *out = nullptr;
    int rc = validate_config(*cfg);
    if (rc) return rc;
    int ndev = 0;
    hipError_t e = hipGetDeviceCount(&ndev);
    if (e != hipSuccess || ndev == 0)
        return fail(L2J_E_HIP, "l2j_create: no HIP device (this library has no CPU fallback)");
    if (cfg->device < 0 || cfg->device >= ndev) return fail(L2J_E_ARG, "l2j_create: device ordinal out of range");
    HIPCHK(hipSetDevice(cfg->device));
    if ((rc = resolve_scratch(cfg->device))) return rc;
    l2j_ctx *c = new (std::nothrow) l2j_ctx();
    if (!c) return fail(L2J_E_OOM, "l2j_create: host allocation failed");
    c->cfg = *cfg;
    for (int i = 0; i < OPT_COUNT; i++) c->opt[i] = option_from_env(i);
    c->head_size = cfg->dim / cfg->n_heads;
    c->kv_dim = cfg->n_kv_heads * c->head_size;
    c->kv_mul = cfg->n_heads / cfg->n_kv_heads;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, cfg->device) == hipSuccess && prop.multiProcessorCount > 0) c->n_cu = prop.multiProcessorCount;

#define TRY(expr)                \
    do {                         \
        rc = (expr);             \
        if (rc) {                \
            l2j_destroy(c);      \
            return rc;           \
        }                        \
    } while (0)
#define TRYHIP(expr)                                                                               \
    do {                                                                                           \
        hipError_t e2_ = (expr);                                                                   \
        if (e2_ != hipSuccess) {                                                                   \
            l2j_destroy(c);                                                                        \
            return fail(e2_ == hipErrorOutOfMemory ? L2J_E_OOM : L2J_E_HIP, std::string(#expr) + ": " + hipGetErrorString(e2_)); \
        }                                                                                          \
    } while (0)

    TRYHIP(hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking));
    for (int t = 0; t < L2J_TENSOR_COUNT; t++) {
        if (!is_quant(t)) continue;
        QTensor &q = c->qt[t];
        q.nfloats = tensor_floats(*cfg, t);
        q.ngroups = (q.nfloats + kGroup - 1) / kGroup;
        TRY(dev_alloc(&q.codes, q.ngroups * kGroup + 64));
        TRY(dev_alloc(&q.gs, q.ngroups));
        TRY(dev_alloc(&q.mm, q.ngroups));
    }
    const uint64_t vd = (uint64_t)cfg->vocab_size * cfg->dim;
    TRY(dev_alloc(&c->emb, vd));
    if (cfg->shared_weights) c->wcls = c->emb;
    else TRY(dev_alloc(&c->wcls, vd));
    const uint64_t kvn = (uint64_t)cfg->n_layers * cfg->seq_len * c->kv_dim;
    const uint64_t NL = cfg->n_layers;
    c->sd = ((uint64_t)cfg->dim + 63) / 64 * 64;
    c->sh = ((uint64_t)cfg->hidden_dim + 63) / 64 * 64;
    c->skv = ((uint64_t)c->kv_dim + 63) / 64 * 64;
    c->set_floats = (2 * NL + 1) * c->sd + 2 * NL * c->sd + NL * c->sh + 2 * NL * c->skv;
    TRY(dev_alloc(&c->acts, 2 * c->set_floats));
    c->x = c->acts;
    c->xb = c->x + (2 * NL + 1) * c->sd;
    c->q = c->xb + NL * c->sd;
    c->hb = c->q + NL * c->sd;
    c->knew = c->hb + NL * c->sh;
    c->vnew = c->knew + NL * c->skv;
    TRY(dev_alloc(&c->logits, cfg->vocab_size));
    TRY(dev_alloc(&c->kcache, kvn));
    TRY(dev_alloc(&c->vcache, kvn));
    TRY(dev_alloc(&c->rope, (uint64_t)cfg->seq_len * (c->head_size / 2)));
    TRY(dev_alloc(&c->silu, kSiluTable));
    TRY(dev_alloc(&c->counters, NL * cfg->n_heads + 1));
    TRY(dev_alloc(&c->tstamp, cfg->seq_len));
    TRYHIP(hipHostMalloc(reinterpret_cast<void **>(&c->h_tstamp), (size_t)cfg->seq_len * sizeof(unsigned long long), hipHostMallocDefault));
    {
        int khz = 0;
        if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, cfg->device) == hipSuccess && khz > 0) c->wall_clock_hz = 1e3 * khz;
    }
    TRY(dev_alloc(&c->st, 1));
    TRY(dev_alloc(&c->prompt, cfg->seq_len));
    TRY(dev_alloc(&c->out_tokens, cfg->seq_len));
    TRYHIP(hipHostMalloc(reinterpret_cast<void **>(&c->h_st), sizeof(DevState), hipHostMallocDefault));
    TRYHIP(hipHostMalloc(reinterpret_cast<void **>(&c->h_tokens), (size_t)cfg->seq_len * sizeof(int), hipHostMallocDefault));
    TRYHIP(hipMemset(c->counters, 0, (NL * cfg->n_heads + 1) * sizeof(unsigned)));
    TRYHIP(hipMemset(c->prompt, 0, (size_t)cfg->seq_len * sizeof(int)));
    TRYHIP(hipMemset(c->out_tokens, 0, (size_t)cfg->seq_len * sizeof(int)));
    TRYHIP(hipMemset(c->st, 0, sizeof(DevState)));
    TRYHIP(hipMemset(c->kcache, 0, kvn * sizeof(float)));
    TRYHIP(hipMemset(c->vcache, 0, kvn * sizeof(float)));
#undef TRY
#undef TRYHIP
    *out = c;
    return L2J_OK;
}

// What l2j_finalize allocates (also after a finalize that failed part-way, so that it can be called again).
static void release_finalize(l2j_ctx *c)
{
    destroy_graph(c);
    (void)hipFree(c->cls_part);
    (void)hipFree(c->attn_part);
    (void)hipFree(c->rmsw);
    (void)hipFree(c->bar_ctr);
    (void)hipFree(c->fault);
    if (c->h_fault) (void)hipHostFree(c->h_fault);
    c->cls_part = nullptr; c->attn_part = nullptr; c->rmsw = nullptr; c->bar_ctr = nullptr;
    c->fault = nullptr; c->h_fault = nullptr;
}

void l2j_destroy(l2j_ctx *c)
{
    if (!c) return;
    // Order: nothing of the context may still run, then the graph (its nodes name kernels and buffers of the
    // context), the events, the buffers, and the stream last.
    std::lock_guard<std::mutex> forward_lock(g_forward_mu);
    (void)hipSetDevice(c->cfg.device);
    if (c->stream) (void)hipStreamSynchronize(c->stream);
    release_finalize(c);
    for (hipEvent_t ev : c->events) (void)hipEventDestroy(ev);
    for (int t = 0; t < L2J_TENSOR_COUNT; t++) {
        (void)hipFree(c->qt[t].codes);
        (void)hipFree(c->qt[t].gs);
        (void)hipFree(c->qt[t].mm);
        (void)hipFree(c->bt_codes[t]);
        (void)hipFree(c->bt_gs[t]);
    }
    if (c->wcls != c->emb) (void)hipFree(c->wcls);
    (void)hipFree(c->emb);
    float *bufs[] = {c->acts, c->logits, c->kcache, c->vcache, c->silu};
    for (float *b : bufs) (void)hipFree(b);
    (void)hipFree(c->rope);
    (void)hipFree(c->counters);
    (void)hipFree(c->tstamp);
    if (c->h_tstamp) (void)hipHostFree(c->h_tstamp);
    (void)hipFree(c->st);
    (void)hipFree(c->prompt);
    (void)hipFree(c->out_tokens);
    free_sampler(c);
    for (float *t : c->taps) (void)hipFree(t);
    if (c->h_st) (void)hipHostFree(c->h_st);
    if (c->h_tokens) (void)hipHostFree(c->h_tokens);
    if (c->stream) (void)hipStreamDestroy(c->stream);
    delete c;
}

int l2j_set_option(l2j_ctx *c, const char *name, int32_t value)
{
    return ctx_rc(c, [&]() -> int {
        if (!c || !name) return fail(L2J_E_ARG, "null argument");
        for (int i = 0; i < OPT_COUNT; i++) {
            if (strcmp(name, kOptions[i].name) != 0) continue;
            std::lock_guard<std::mutex> lock(c->upload_mu);
            if (c->finalized && !kOptions[i].after_finalize)
                return fail(L2J_E_STATE, std::string("option '") + name + "' fixes a launch shape: set it before l2j_finalize");
            c->opt[i] = value;
            return L2J_OK;
        }
        return fail(L2J_E_ARG, std::string("unknown option '") + name + "'");
    }());
}

int l2j_get_option(l2j_ctx *c, const char *name, int32_t *value)
{
    return ctx_rc(c, [&]() -> int {
        if (!c || !name || !value) return fail(L2J_E_ARG, "null argument");
        for (int i = 0; i < OPT_COUNT; i++) {
            if (strcmp(name, kOptions[i].name) != 0) continue;
            std::lock_guard<std::mutex> lock(c->upload_mu);
            *value = c->opt[i];
            return L2J_OK;
        }
        return fail(L2J_E_ARG, std::string("unknown option '") + name + "'");
    }());
}

int l2j_get_config(l2j_ctx *c, l2j_config *cfg)
{
    return ctx_rc(c, [&]() -> int {
        if (!c || !cfg) return fail(L2J_E_ARG, "null argument");
        *cfg = c->cfg;
        return L2J_OK;
    }());
}

// whole: the call replaces the tensor (its count of loaded groups starts again)
static int upload_quant_range(l2j_ctx *c, int tensor, uint64_t group0, uint64_t ngroups, const uint8_t *bytes, uint64_t nbytes, bool whole)
{
    if (nbytes != ngroups * kGroupBytes)
        return fail(L2J_E_SIZE, "totalByteSize != quant.numberOfBytesByFloatSize(floatSize)");
    std::lock_guard<std::mutex> lock(c->upload_mu);
    if (c->finalized) return fail(L2J_E_STATE, "upload after l2j_finalize");
    HIPCHK(hipSetDevice(c->cfg.device));
    QTensor &t = c->qt[tensor];
    if (whole) t.groups_loaded = 0;
    int rc = unpack_into(c, t, group0, bytes, ngroups);
    if (rc == L2J_OK) t.groups_loaded += ngroups;
    return rc;
}

int l2j_upload_quant(l2j_ctx *c, int tensor, const uint8_t *ref_bytes, uint64_t nbytes)
{
    return ctx_rc(c, [&]() -> int {
        if (!c || !ref_bytes) return fail(L2J_E_ARG, "null argument");
        if (!is_quant(tensor)) return fail(L2J_E_ARG, "not a quantized tensor");
        return upload_quant_range(c, tensor, 0, c->qt[tensor].ngroups, ref_bytes, nbytes, true);
    }());
}

int l2j_upload_quant_layer(l2j_ctx *c, int tensor, int layer, const uint8_t *ref_bytes, uint64_t nbytes)
{
    return ctx_rc(c, [&]() -> int {
        if (!c || !ref_bytes) return fail(L2J_E_ARG, "null argument");
        if (!is_quant(tensor) || !per_layer(tensor)) return fail(L2J_E_ARG, "not a per-layer quantized tensor");
        if (layer < 0 || layer >= c->cfg.n_layers) return fail(L2J_E_ARG, "layer out of range");
        const uint64_t per = c->qt[tensor].nfloats / c->cfg.n_layers;
        if (per % kGroup) return fail(L2J_E_ARG, "layer size is not a multiple of the group size; upload the whole tensor");
        return upload_quant_range(c, tensor, (uint64_t)layer * (per / kGroup), per / kGroup, ref_bytes, nbytes, false);
    }());
}

int l2j_upload_f32(l2j_ctx *c, int tensor, const float *data, uint64_t nfloats)
{
    return ctx_rc(c, [&]() -> int {
        if (!c || !data) return fail(L2J_E_ARG, "null argument");
        if (tensor != L2J_TOK_EMB && tensor != L2J_WCLS) return fail(L2J_E_ARG, "only the embedding and the classifier are fp32");
        if (nfloats != (uint64_t)c->cfg.vocab_size * c->cfg.dim) return fail(L2J_E_SIZE, "float count != vocab_size * dim");
        std::lock_guard<std::mutex> lock(c->upload_mu);
        if (c->finalized) return fail(L2J_E_STATE, "upload after l2j_finalize");
        HIPCHK(hipSetDevice(c->cfg.device));
        if (tensor == L2J_WCLS && c->cfg.shared_weights) return L2J_OK;  // J/TransformerWeights.java:122
        HIPCHK(hipMemcpy(tensor == L2J_TOK_EMB ? c->emb : c->wcls, data, nfloats * sizeof(float), hipMemcpyHostToDevice));
        (tensor == L2J_TOK_EMB ? c->emb_loaded : c->wcls_loaded) = true;
        return L2J_OK;
    }());
}

int l2j_upload_f32_quantize(l2j_ctx *c, int tensor, uint64_t first, const float *data, uint64_t nfloats)
{
    return ctx_rc(c, [&]() -> int {
        if (!c || !data) return fail(L2J_E_ARG, "null argument");
        if (!is_quant(tensor)) return fail(L2J_E_ARG, "not a quantized tensor");
        QTensor &t = c->qt[tensor];
        if (first % kGroup) return fail(L2J_E_ARG, "first must be a multiple of the group size");
        if (first + nfloats > t.nfloats) return fail(L2J_E_SIZE, "range exceeds the tensor");
        if (nfloats % kGroup && first + nfloats != t.nfloats) return fail(L2J_E_ARG, "only the tensor's tail may be a partial group");
        std::lock_guard<std::mutex> lock(c->upload_mu);
        if (c->finalized) return fail(L2J_E_STATE, "upload after l2j_finalize");
        HIPCHK(hipSetDevice(c->cfg.device));
        const uint64_t slice = 16ull << 20;  // floats per staging slice (64 MiB)
        float *stage = nullptr;
        HIPCHK(hipMalloc(reinterpret_cast<void **>(&stage), std::min(slice, std::max<uint64_t>(nfloats, 1)) * sizeof(float)));
        int rc = L2J_OK;
        for (uint64_t o = 0; o < nfloats && rc == L2J_OK; o += slice) {
            const uint64_t nf = std::min(slice, nfloats - o);
            const uint64_t ng = (nf + kGroup - 1) / kGroup;
            hipError_t e = hipMemcpy(stage, data + o, nf * sizeof(float), hipMemcpyHostToDevice);
            if (e == hipSuccess) {
                hipLaunchKernelGGL(k_encode_groups, dim3((unsigned)std::min<uint64_t>(ng, 1u << 20)), dim3(256), 0, c->stream, stage, (long)nf,
                                   (long)((first + o) / kGroup), (long)ng, (long)t.nfloats, 0ull, 0.0f, t.codes, t.gs, t.mm);
                e = hipGetLastError();
                if (e == hipSuccess) e = hipStreamSynchronize(c->stream);
            }
            if (e != hipSuccess) rc = fail(L2J_E_HIP, std::string("quantize: ") + hipGetErrorString(e));
            else t.groups_loaded += ng;
        }
        (void)hipFree(stage);
        return rc;
    }());
}

int l2j_read_quant(l2j_ctx *c, int tensor, uint64_t group0, uint64_t ngroups, uint8_t *out)
{
    return ctx_rc(c, [&]() -> int {
        if (!c || !out) return fail(L2J_E_ARG, "null argument");
        if (!is_quant(tensor)) return fail(L2J_E_ARG, "not a quantized tensor");
        QTensor &t = c->qt[tensor];
        if (group0 + ngroups > t.ngroups) return fail(L2J_E_SIZE, "group range exceeds the tensor");
        if (ngroups == 0) return L2J_OK;
        std::lock_guard<std::mutex> lock(c->upload_mu);
        HIPCHK(hipSetDevice(c->cfg.device));
        const uint64_t slice_groups = (64ull << 20) / kGroupBytes;
        uint8_t *stage = nullptr;
        HIPCHK(hipMalloc(reinterpret_cast<void **>(&stage), std::min(ngroups, slice_groups) * kGroupBytes));
        int rc = L2J_OK;
        for (uint64_t g = 0; g < ngroups && rc == L2J_OK; g += slice_groups) {
            const uint64_t ng = std::min(slice_groups, ngroups - g);
            hipLaunchKernelGGL(k_pack_groups, dim3((unsigned)std::min<uint64_t>(ng, 1u << 20)), dim3(64), 0, c->stream, stage, (long)ng,
                               t.codes + (group0 + g) * kGroup, t.mm + group0 + g);
            hipError_t e = hipGetLastError();
            if (e == hipSuccess) e = hipStreamSynchronize(c->stream);
            if (e == hipSuccess) e = hipMemcpy(out + g * kGroupBytes, stage, ng * kGroupBytes, hipMemcpyDeviceToHost);
            if (e != hipSuccess) rc = fail(L2J_E_HIP, std::string("read_quant: ") + hipGetErrorString(e));
        }
        (void)hipFree(stage);
        return rc;
    }());
}

int l2j_fill_synthetic(l2j_ctx *c, uint64_t seed, float sigma)
{
    return ctx_rc(c, [&]() -> int {
        if (!c) return fail(L2J_E_ARG, "null context");
        std::lock_guard<std::mutex> lock(c->upload_mu);
        if (c->finalized) return fail(L2J_E_STATE, "upload after l2j_finalize");
        HIPCHK(hipSetDevice(c->cfg.device));
        const float scale = sigma / 37837.2265625f;
        auto base_of = [&](uint32_t stream) { return seed * 0x9E3779B97F4A7C15ULL + (uint64_t)stream * 0xD1B54A32D192ED03ULL; };
        const uint64_t vd = (uint64_t)c->cfg.vocab_size * c->cfg.dim;
        hipLaunchKernelGGL(k_synth_f32, dim3(4096), dim3(256), 0, c->stream, c->emb, (long)vd, base_of(0), scale);
        HIPCHK(hipGetLastError());
        if (c->wcls != c->emb) {
            hipLaunchKernelGGL(k_synth_f32, dim3(4096), dim3(256), 0, c->stream, c->wcls, (long)vd, base_of(11), scale);
            HIPCHK(hipGetLastError());
        }
        for (int t = L2J_RMS_ATT; t <= L2J_RMS_FINAL; t++) {
            QTensor &q = c->qt[t];
            hipLaunchKernelGGL(k_encode_groups, dim3((unsigned)std::min<uint64_t>(q.ngroups, 1u << 20)), dim3(256), 0, c->stream,
                               (const float *)nullptr, 0L, 0L, (long)q.ngroups, (long)q.nfloats, base_of((uint32_t)t), scale, q.codes, q.gs,
                               q.mm);
            HIPCHK(hipGetLastError());
            q.groups_loaded = q.ngroups;
        }
        HIPCHK(hipStreamSynchronize(c->stream));
        c->emb_loaded = c->wcls_loaded = true;
        return L2J_OK;
    }());
}

int l2j_finalize(l2j_ctx *c)
{
    const int rc = ctx_rc(c, [&]() -> int {
        if (!c) return fail(L2J_E_ARG, "null context");
        std::lock_guard<std::mutex> lock(c->upload_mu);
        if (c->finalized) return fail(L2J_E_STATE, "already finalized");
        HIPCHK(hipSetDevice(c->cfg.device));
        if (!c->emb_loaded) return fail(L2J_E_STATE, "token_embedding_table was not uploaded");
        if (!c->cfg.shared_weights && !c->wcls_loaded) return fail(L2J_E_STATE, "wcls was not uploaded");
        for (int t = L2J_RMS_ATT; t <= L2J_RMS_FINAL; t++)
            if (c->qt[t].groups_loaded < c->qt[t].ngroups)
                return fail(L2J_E_STATE, std::string("tensor not fully uploaded: ") + l2j_host::tensor_stem(t));

        // RoPE table (K/ApplyRope.java:34-59): freq = (float)(1.0 / pow(10000.0f, (i % hs) / (float) hs)),
        // val = pos * freq in fp32, cos/sin in double then narrowed.  Only i % head_size matters.
        const int hs = c->head_size, half = hs / 2, S = c->cfg.seq_len;
        std::vector<float2> rope((size_t)S * half);
        for (int k = 0; k < half; k++) {
            const float ex = (float)(2 * k) / (float)hs;
            const float freq = (float)(1.0 / std::pow((double)10000.0f, (double)ex));
            for (int pos = 0; pos < S; pos++) {
                const float val = (float)pos * freq;
                rope[(size_t)pos * half + k] = make_float2((float)std::cos((double)val), (float)std::sin((double)val));
            }
        }
        HIPCHK(hipMemcpy(c->rope, rope.data(), rope.size() * sizeof(float2), hipMemcpyHostToDevice));
        // sigmoid table (K/Silu.java:47-57)
        std::vector<float> tab(kSiluTable);
        for (int i = 0; i < kSiluTable; i++) {
            const double v = ((double)i / (double)kSiluTable) * 10.0 - 5.0;
            tab[i] = (float)(1.0 / (1.0 + std::exp(-v)));
        }
        HIPCHK(hipMemcpy(c->silu, tab.data(), tab.size() * sizeof(float), hipMemcpyHostToDevice));

        // rmsnorm weights dequantized once with the reference's expression
        {
            const uint64_t dim = c->cfg.dim, L = c->cfg.n_layers;
            int rc2;
            if ((rc2 = dev_alloc(&c->rmsw, (2 * L + 1) * dim))) return rc2;
            const int src[3] = {L2J_RMS_ATT, L2J_RMS_FFN, L2J_RMS_FINAL};
            float *dst[3] = {c->rmsw, c->rmsw + L * dim, c->rmsw + 2 * L * dim};
            for (int i = 0; i < 3; i++) {
                const long n = (long)c->qt[src[i]].nfloats;
                hipLaunchKernelGGL(k_dequant_rms, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, c->stream, c->qt[src[i]].codes,
                                   c->qt[src[i]].mm, n, dst[i]);
                HIPCHK(hipGetLastError());
            }
        }
        // launch shapes: one 1024-thread workgroup per compute unit for the weight-streaming kernels
        {
            const int nmax = std::max(c->cfg.dim, c->cfg.hidden_dim);
            const int *o = c->opt;
            c->pk_threads = std::min(1024, std::max(64, o[OPT_THREADS] / 64 * 64));
            c->pk_grid = std::max(1, o[OPT_GRID] != kAuto ? o[OPT_GRID] : c->n_cu);  // one workgroup per compute unit
            c->attn_threads = std::min(1024, std::max(64, o[OPT_ATTN_THREADS] / 64 * 64));
            c->attn_rows = std::max(1, o[OPT_ATTN_ROWS]);
            c->attn_nsplit = std::max(1, o[OPT_ATTN_NSPLIT]);
            c->attn_grid = c->cfg.n_heads * c->attn_nsplit;
            c->fused_attn_rows = std::max(1, o[OPT_FUSED_ATTN_ROWS]);
            if (std::max(mv_smem(nmax), attn_smem(c)) > 160 * 1024) return fail(L2J_E_ARG, "hidden_dim does not fit the 160 KB LDS");
            // (a whole-token kernel whose LDS would exceed the compute unit's is not used, see below)
            const size_t need = std::min<size_t>(160 * 1024, std::max(std::max(mv_smem(nmax), attn_smem(c)), layer_smem(c)));
            if (need > 64 * 1024) {
                const void *ks[] = {reinterpret_cast<const void *>(k_matvec<PH_QKV>), reinterpret_cast<const void *>(k_matvec<PH_W13>),
                                    reinterpret_cast<const void *>(k_matvec<PH_RES>), reinterpret_cast<const void *>(k_matvec<PH_ROW>),
                                    reinterpret_cast<const void *>(k_matvec<PH_ROW6>),
                                    reinterpret_cast<const void *>(k_matvec<PH_QKV, 5>), reinterpret_cast<const void *>(k_matvec<PH_W13, 5>),
                                    reinterpret_cast<const void *>(k_matvec<PH_RES, 5>),
                                    reinterpret_cast<const void *>(k_classifier), reinterpret_cast<const void *>(k_token<16>),
                                    reinterpret_cast<const void *>(k_token<32>), reinterpret_cast<const void *>(k_token<64>),
                                    reinterpret_cast<const void *>(k_token<16, 1, 1>), reinterpret_cast<const void *>(k_token<16, 1, 2>),
                                    reinterpret_cast<const void *>(k_token<32, 5, kTU>),
                                    reinterpret_cast<const void *>(k_token<32, kTU, kTU, true>), reinterpret_cast<const void *>(k_token<32, 5, kTU, true>)};
                for (const void *k : ks) HIPCHK(hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)need));
            }
            int rc2;
            if ((rc2 = dev_alloc(&c->cls_part, c->pk_grid))) return rc2;
            if ((rc2 = dev_alloc(&c->attn_part, (uint64_t)c->cfg.n_layers * c->cfg.n_heads * c->attn_nsplit * (c->head_size + 2)))) return rc2;
            c->nbar = 5 * c->cfg.n_layers;
            if ((rc2 = dev_alloc(&c->bar_ctr, (uint64_t)c->nbar * kBarStride))) return rc2;
            if ((rc2 = dev_alloc(&c->fault, 1))) return rc2;
            HIPCHK(hipMemset(c->bar_ctr, 0, (size_t)c->nbar * kBarStride * sizeof(unsigned)));
            HIPCHK(hipMemset(c->fault, 0, sizeof(int)));
            HIPCHK(hipHostMalloc(reinterpret_cast<void **>(&c->h_fault), sizeof(int), hipHostMallocDefault));
            *c->h_fault = 0;
            // k_token needs its whole grid resident at once (grid barriers): at most what the occupancy allows.
            // One launch per token pays off when a layer streams enough to hide its five hand-overs (7B shape, 208 MB a
            // layer: 645 vs 511 tok/s; 110M shape, 7 MB: 3240 vs 3080); the smallest models run faster as one launch per
            // phase (15M shape, 1 MB a layer: 6300 vs 5400 tok/s).
            const uint64_t layer_floats = 2ull * c->cfg.dim * c->cfg.dim + 2ull * c->cfg.dim * c->kv_dim + 3ull * c->cfg.dim * c->cfg.hidden_dim;
            c->fused = (c->opt[OPT_FUSE] != kAuto ? c->opt[OPT_FUSE] : layer_floats >= (4ull << 20) ? 1 : 0) != 0;
            c->layers_per_launch = std::max(1, std::min(c->cfg.n_layers, c->opt[OPT_LAYERS_PER_LAUNCH] != kAuto ? c->opt[OPT_LAYERS_PER_LAUNCH] : c->cfg.n_layers));
            if (c->fused && layer_smem(c) > 160 * 1024) c->fused = false;
            if (c->fused) {
                const void *kl = with_token_kernel(c, [](auto kernel) { return reinterpret_cast<const void *>(kernel); });
                int per_cu = 0;
                HIPCHK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kl, c->pk_threads, layer_smem(c)));
                if (per_cu < 1 || c->pk_grid > per_cu * c->n_cu) c->fused = false;
            }
            c->by_value = c->fused && c->layers_per_launch == c->cfg.n_layers && c->opt[OPT_BY_VALUE] != 0 &&
                          std::max(c->cfg.dim, c->cfg.hidden_dim) <= 4 * kPollWords * c->pk_threads;
            c->self_contained = c->by_value ? c->opt[OPT_SELF_CONTAINED] & 3 : 0;
            c->acts_dirty = true;  // marked unwritten ahead of the first token
            build_geom(c);
            if (!geom_complete(c->geom)) return fail(L2J_E_STATE, "internal: a device buffer of the forward pass was not allocated");
        }

        HIPCHK(hipStreamSynchronize(c->stream));
        const int rcg = capture_graphs(c);
        if (rcg) return rcg;
        c->finalized = true;
        return L2J_OK;
    }());
    if (rc && c) {  // a finalize that failed part-way leaves nothing behind: it may be called again
        std::lock_guard<std::mutex> lock(c->upload_mu);
        if (!c->finalized) {
            (void)hipSetDevice(c->cfg.device);
            release_finalize(c);
        }
    }
    return rc;
}

int l2j_reset(l2j_ctx *c)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        if (!c) return fail(L2J_E_ARG, "null context");
        HIPCHK(hipSetDevice(c->cfg.device));
        const uint64_t kvn = (uint64_t)c->cfg.n_layers * c->cfg.seq_len * c->kv_dim;
        HIPCHK(hipMemsetAsync(c->kcache, 0, kvn * sizeof(float), c->stream));
        HIPCHK(hipMemsetAsync(c->vcache, 0, kvn * sizeof(float), c->stream));
        HIPCHK(hipStreamSynchronize(c->stream));
        return L2J_OK;
    }());
}

int l2j_sync(l2j_ctx *c)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        if (!c) return fail(L2J_E_ARG, "null context");
        HIPCHK(hipSetDevice(c->cfg.device));
        HIPCHK(hipStreamSynchronize(c->stream));
        return L2J_OK;
    }());
}

int l2j_forward(l2j_ctx *c, int32_t token, int32_t pos, float *logits)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        int rc = check_forward_args(c, token, pos);
        if (rc) return rc;
        do {  // (a second time, phase by phase, when the whole-token kernel's waits ran out)
            if ((rc = set_state(c, token, pos, 0))) return rc;
            HIPCHK(launch_one_token(c));
            if (logits) HIPCHK(hipMemcpyAsync(logits, c->logits, (size_t)c->cfg.vocab_size * sizeof(float), hipMemcpyDeviceToHost, c->stream));
            HIPCHK(hipStreamSynchronize(c->stream));
        } while ((rc = check_barrier_error(c)) == kRepeatToken);
        return rc;
    }());
}

int l2j_forward_argmax(l2j_ctx *c, int32_t token, int32_t pos, int32_t *next)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        if (!next) return fail(L2J_E_ARG, "null argument");
        int rc = check_forward_args(c, token, pos);
        if (rc) return rc;
        do {
            if ((rc = set_state(c, token, pos, 0))) return rc;
            HIPCHK(launch_one_token(c));
            HIPCHK(hipMemcpyAsync(c->h_tokens, &c->st->token, sizeof(int), hipMemcpyDeviceToHost, c->stream));
            HIPCHK(hipStreamSynchronize(c->stream));
            *next = c->h_tokens[0];
        } while ((rc = check_barrier_error(c)) == kRepeatToken);
        return rc;
    }());
}

int l2j_forward_taps(l2j_ctx *c, int32_t token, int32_t pos, float *logits)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        int rc = check_forward_args(c, token, pos);
        if (rc) return rc;
        const uint64_t L = c->cfg.n_layers;
        const int which[] = {L2J_B_X, L2J_B_XB, L2J_B_XB2, L2J_B_HB, L2J_B_Q, L2J_B_K, L2J_B_V};
        for (int w : which) {
            if (c->taps[w]) continue;
            const uint64_t n = w == L2J_B_HB ? c->cfg.hidden_dim : (w == L2J_B_K || w == L2J_B_V) ? c->kv_dim : c->cfg.dim;
            if ((rc = dev_alloc(&c->taps[w], L * n))) return rc;
        }
        if ((rc = set_state(c, token, pos, 0))) return rc;
        c->acts_dirty = true;  // the phases launched one by one leave values in the vectors of set 0
        hipError_t e = launch_token(c, c->stream, true);
        if (e != hipSuccess) return fail(L2J_E_HIP, std::string("launch: ") + hipGetErrorString(e));
        if (logits) HIPCHK(hipMemcpyAsync(logits, c->logits, (size_t)c->cfg.vocab_size * sizeof(float), hipMemcpyDeviceToHost, c->stream));
        HIPCHK(hipStreamSynchronize(c->stream));
        return L2J_OK;
    }());
}

int l2j_decode_greedy(l2j_ctx *c, const int32_t *prompt, int32_t n_prompt, int32_t steps, int32_t *out_tokens, int32_t *n_out,
                      double *seconds)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        int rc;  // (the whole loop once more, phase by phase, when the whole-token kernel's waits ran out)
        while ((rc = decode_loop(c, prompt, n_prompt, steps, false, 0.0f, 0.0f, 0, out_tokens, n_out, seconds)) == kRepeatToken) {}
        return rc;
    }());
}

int l2j_decode_sample(l2j_ctx *c, const int32_t *prompt, int32_t n_prompt, int32_t steps, float temperature, float topp,
                      int64_t rng_seed, int32_t *out_tokens, int32_t *n_out, double *seconds)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        int rc = check_sampler_args(temperature, topp);
        if (rc) return rc;
        while ((rc = decode_loop(c, prompt, n_prompt, steps, temperature != 0.0f, temperature, topp, rng_seed, out_tokens, n_out, seconds)) ==
               kRepeatToken) {}
        return rc;
    }());
}

int l2j_sampler_seed(l2j_ctx *c, int64_t rng_seed)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        if (!c) return fail(L2J_E_ARG, "null context");
        HIPCHK(hipSetDevice(c->cfg.device));
        return seed_sampler(c, rng_seed);
    }());
}

int l2j_sample(l2j_ctx *c, const float *logits, float temperature, float topp, float coin, int32_t *next)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        if (!c || !next) return fail(L2J_E_ARG, "null argument");
        int rc = check_sampler_args(temperature, topp);
        if (rc) return rc;
        if (coin >= 1.0f) return fail(L2J_E_ARG, "coin must be below 1 (negative: the context's generator draws)");
        HIPCHK(hipSetDevice(c->cfg.device));
        if (!c->ss && (rc = seed_sampler(c, 0))) return rc;
        const int n = c->cfg.vocab_size;
        if (logits) HIPCHK(hipMemcpyAsync(c->logits, logits, (size_t)n * sizeof(float), hipMemcpyHostToDevice, c->stream));
        if (temperature == 0.0f) {
            hipLaunchKernelGGL(k_argmax_logits, dim3(1), dim3(1024), 0, c->stream, c->logits, n, c->ss);  // J/Run.java:644-646
            HIPCHK(hipGetLastError());
        } else {
            HIPCHK(launch_sampler(c, temperature, topp, coin, false));
        }
        HIPCHK(hipMemcpyAsync(c->h_ss, c->ss, sizeof(SamplerState), hipMemcpyDeviceToHost, c->stream));
        HIPCHK(hipStreamSynchronize(c->stream));
        if ((rc = check_sampler_status(c))) return rc;
        *next = c->h_ss->result;
        return L2J_OK;
    }());
}

int l2j_running_sums(l2j_ctx *c, const float *terms, int32_t n, float *sums)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        if (!c || !terms || !sums) return fail(L2J_E_ARG, "null argument");
        if (n <= 0 || n > (1 << 24)) return fail(L2J_E_SIZE, "1 to 16777216 terms");
        HIPCHK(hipSetDevice(c->cfg.device));
        float *d = nullptr;
        HIPCHK(hipMalloc(reinterpret_cast<void **>(&d), (size_t)n * sizeof(float)));
        const size_t lds = sampler_lds_bytes(n);
        hipError_t e = hipMemcpyAsync(d, terms, (size_t)n * sizeof(float), hipMemcpyHostToDevice, c->stream);
        if (e == hipSuccess) {
            const int scan_on = c->opt[OPT_SAMPLER_SCAN] != 0 ? 1 : 0;
            if (n <= kSampleMaxVocab) hipLaunchKernelGGL(k_running_sums<true>, dim3(1), dim3(1024), lds, c->stream, d, n, scan_on);
            else hipLaunchKernelGGL(k_running_sums<false>, dim3(1), dim3(1024), 0, c->stream, d, n, 1);
            e = hipGetLastError();
        }
        if (e == hipSuccess) e = hipMemcpyAsync(sums, d, (size_t)n * sizeof(float), hipMemcpyDeviceToHost, c->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(c->stream);
        (void)hipFree(d);
        if (e != hipSuccess) return fail(L2J_E_HIP, std::string("running sums: ") + hipGetErrorString(e));
        return L2J_OK;
    }());
}

int l2j_running_sums_noalloc(l2j_ctx *c, const float *terms, int32_t n, float *sums)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        if (!c || !terms || !sums) return fail(L2J_E_ARG, "null argument");
        if (n <= 0 || n > kSampleMaxVocab) return fail(L2J_E_SIZE, "l2j_running_sums_noalloc: 1 to 36864 terms (the size of the library's static device buffer)");
        HIPCHK(hipSetDevice(c->cfg.device));
        float *d = nullptr;
        {
            std::lock_guard<std::mutex> lock(g_scratch_mu);
            d = g_scratch_ptr[c->cfg.device];
        }
        if (!d) return fail(L2J_E_STATE, "l2j_running_sums_noalloc: the static device buffer was not resolved on this device");
        // The buffer keeps the last call's contents; the kernel reads only the n terms copied in here, so nothing needs clearing.
        const size_t lds = sampler_lds_bytes(n);
        HIPCHK(hipMemcpyAsync(d, terms, (size_t)n * sizeof(float), hipMemcpyHostToDevice, c->stream));
        hipLaunchKernelGGL(k_running_sums<true>, dim3(1), dim3(1024), lds, c->stream, d, n, c->opt[OPT_SAMPLER_SCAN] != 0 ? 1 : 0);
        HIPCHK(hipGetLastError());
        HIPCHK(hipMemcpyAsync(sums, d, (size_t)n * sizeof(float), hipMemcpyDeviceToHost, c->stream));
        HIPCHK(hipStreamSynchronize(c->stream));
        return L2J_OK;
    }());
}

// rows and row length of one layer's matrix of a quantized matrix tensor (false: not one)
static bool matrix_shape(const l2j_config &cf, int tensor, int *rows, int *K)
{
    const int kvd = cf.dim / cf.n_heads * cf.n_kv_heads;
    switch (tensor) {
    case L2J_WQ: case L2J_WO: *rows = cf.dim; *K = cf.dim; return true;
    case L2J_WK: case L2J_WV: *rows = kvd; *K = cf.dim; return true;
    case L2J_W1: case L2J_W3: *rows = cf.hidden_dim; *K = cf.dim; return true;
    case L2J_W2: *rows = cf.dim; *K = cf.hidden_dim; return true;
    default: return false;
    }
}

// The tile-ordered copy of `tensor` for the batched path (rows % 16 == 0 and K % 256 == 0 checked by the caller).
static int ensure_batch_tiles(l2j_ctx *c, int tensor)
{
    if (c->bt_done[tensor]) return L2J_OK;
    int rows = 0, K = 0;
    if (!matrix_shape(c->cfg, tensor, &rows, &K)) return fail(L2J_E_ARG, "not a matrix tensor");
    const QTensor &t = c->qt[tensor];
    if (t.groups_loaded != t.ngroups) return fail(L2J_E_STATE, "tensor not uploaded");
    const uint64_t n = (uint64_t)c->cfg.n_layers * rows * K;
    int rc;
    if (!c->bt_codes[tensor] && (rc = dev_alloc(&c->bt_codes[tensor], n))) return rc;
    if (!c->bt_gs[tensor] && (rc = dev_alloc(&c->bt_gs[tensor], n / 256))) return rc;
    const long n16 = (long)(n / 16);
    hipLaunchKernelGGL(k_btile, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, c->stream, t.codes, t.gs, n16, rows, K, c->bt_codes[tensor],
                       c->bt_gs[tensor]);
    HIPCHK(hipGetLastError());
    c->bt_done[tensor] = true;
    return L2J_OK;
}

static QMat bqmat(const l2j_ctx *c, int t, uint64_t off)
{
    QMat m;
    m.codes = c->bt_codes[t];
    m.gs = c->bt_gs[t];
    m.off = (long)off;
    return m;
}

int l2j_batch_matmul(l2j_ctx *c, int tensor, int layer, const float *x, float *y, int32_t groups_per_slice, int32_t rounds,
                     double *mean_us)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        if (!c || !x || !y) return fail(L2J_E_ARG, "null argument");
        int rows = 0, K = 0;
        if (!matrix_shape(c->cfg, tensor, &rows, &K)) return fail(L2J_E_ARG, "not a matrix tensor");
        if (layer < 0 || layer >= c->cfg.n_layers) return fail(L2J_E_ARG, "layer out of range");
        if (K % 256 || rows % 16) return fail(L2J_E_SIZE, "the batched matrix product needs rows of whole groups (K % 256 == 0) and rows % 16 == 0");
        const QTensor &t = c->qt[tensor];
        if (t.groups_loaded != t.ngroups) return fail(L2J_E_STATE, "tensor not uploaded");
        const int ngroups = K / 256, gps = std::max(1, std::min(std::min(ngroups, kBgMaxGps), (int)groups_per_slice));
        const int slices = (ngroups + gps - 1) / gps;
        const size_t lds = bg_lds_bytes(gps, kBatch);
        if (lds + sizeof(float) * kBatch * kBgMaxGps > 160 * 1024) return fail(L2J_E_SIZE, "groups_per_slice: the slice of the activations does not fit the LDS");
        HIPCHK(hipSetDevice(c->cfg.device));
        int trc = ensure_batch_tiles(c, tensor);
        if (trc) return trc;
        float *dx = nullptr, *dpart = nullptr, *dy = nullptr;
        hipEvent_t e0 = nullptr, e1 = nullptr;
        auto release = [&]() {
            (void)hipFree(dx); (void)hipFree(dpart); (void)hipFree(dy);
            if (e0) (void)hipEventDestroy(e0);
            if (e1) (void)hipEventDestroy(e1);
        };
        hipError_t e = hipMalloc(reinterpret_cast<void **>(&dx), (size_t)kBatch * K * sizeof(float));
        if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&dpart), (size_t)slices * kBatch * rows * sizeof(float));
        if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&dy), (size_t)kBatch * rows * sizeof(float));
        if (e == hipSuccess) e = hipEventCreate(&e0);
        if (e == hipSuccess) e = hipEventCreate(&e1);
        if (e == hipSuccess) e = hipFuncSetAttribute((const void *)k_bgemm<2, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e == hipSuccess) e = hipMemcpyAsync(dx, x, (size_t)kBatch * K * sizeof(float), hipMemcpyHostToDevice, c->stream);
        if (e == hipSuccess) {
            BGemm a{};
            a.m[0] = bqmat(c, tensor, (uint64_t)layer * rows * K);
            a.rows[0] = rows; a.part[0] = dpart; a.nmat = 1; a.K = K; a.x = dx; a.gps = gps;
            const dim3 grid((bg_units(rows, 2) + 3) / 4, slices);
            const int n = std::max(1, (int)rounds);
            hipLaunchKernelGGL((k_bgemm<2, 1>), grid, dim3(kBgThreads), lds, c->stream, a);   // warm
            (void)hipEventRecord(e0, c->stream);
            for (int i = 0; i < n; i++) hipLaunchKernelGGL((k_bgemm<2, 1>), grid, dim3(kBgThreads), lds, c->stream, a);
            (void)hipEventRecord(e1, c->stream);
            hipLaunchKernelGGL(k_breduce, dim3(256), dim3(256), 0, c->stream, dpart, dy, rows, slices);
            e = hipGetLastError();
            if (e == hipSuccess) e = hipMemcpyAsync(y, dy, (size_t)kBatch * rows * sizeof(float), hipMemcpyDeviceToHost, c->stream);
            if (e == hipSuccess) e = hipStreamSynchronize(c->stream);
            float ms = 0.0f;
            if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
            if (mean_us) *mean_us = (double)ms * 1e3 / n;
        }
        release();
        if (e != hipSuccess) return fail(L2J_E_HIP, std::string("batch matmul: ") + hipGetErrorString(e));
        return L2J_OK;
    }());
}

// ---- several sequences at once ----------------------------------------------------------------------------------

namespace {

struct BatchBufs {   // device memory of one l2j_decode_greedy_batch call
    float *x = nullptr, *xn = nullptr, *xb = nullptr, *hb = nullptr, *logits = nullptr;
    float *part[3] = {nullptr, nullptr, nullptr};
    float *kc = nullptr, *vc = nullptr;
    BatchState *st = nullptr;
    int *prompts = nullptr, *out = nullptr;
    unsigned *done = nullptr;
    int *h_pin = nullptr;   // pinned: every transfer of the call goes through it, as in the single-sequence loops
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    void release()
    {
        if (exec) (void)hipGraphExecDestroy(exec);
        if (graph) (void)hipGraphDestroy(graph);
        if (e0) (void)hipEventDestroy(e0);
        if (e1) (void)hipEventDestroy(e1);
        void *ps[] = {x, xn, xb, hb, logits, part[0], part[1], part[2], kc, vc, st, prompts, out, done};
        for (void *p : ps) (void)hipFree(p);
        if (h_pin) (void)hipHostFree(h_pin);
    }
};

#ifdef L2J_BATCH_TIMES
struct BtRec { std::string name; hipEvent_t e0, e1; };
static std::vector<BtRec> g_bt;
static bool g_bt_on = false;
struct BtScope {
    hipStream_t s; bool on; BtRec r;
    BtScope(const char *n, hipStream_t st) : s(st), on(g_bt_on) { if (on) { r.name = n; (void)hipEventCreate(&r.e0); (void)hipEventCreate(&r.e1); (void)hipEventRecord(r.e0, s); } }
    ~BtScope() { if (on) { (void)hipEventRecord(r.e1, s); g_bt.push_back(r); } }
};
#define BT(name) BtScope bt_scope_(name, c->stream)
#else
#define BT(name)
#endif

constexpr int kBatchGps = 2;   // groups of 256 codes per slice of K (measured: 1, 2, 4 -> 26, 24, 30 us for W1 of the 7B shape)

int batch_slices(int K) { return (K / 256 + kBatchGps - 1) / kBatchGps; }
size_t batch_lds(int nseq) { return bg_lds_bytes(kBatchGps, nseq); }   // k_bgemm: bf16 planes
size_t batch_lds_f32(int nseq) { return (size_t)nseq * (kBatchGps * 256 + kXPad) * sizeof(float); }   // k_bgemm_f32: floats
// workgroups of k_bgemm a compute unit holds at once: its 160 KB of LDS, and at most three by their registers
int batch_resident(int nseq) { return std::max(1, std::min(3, (int)((160 * 1024) / (batch_lds(nseq) + sizeof(float) * nseq * kBgMaxGps)))); }

// The products of one layer's matrices `tensors` (the same input, the same row length) in one launch.
void launch_bgemm(l2j_ctx *c, std::initializer_list<int> tensors, int layer, const float *x, float *const *part, int nseq)
{
    BGemm a{};
    int K = 0;
    for (int tensor : tensors) {
        int rows = 0;
        matrix_shape(c->cfg, tensor, &rows, &K);
        a.m[a.nmat] = bqmat(c, tensor, (uint64_t)layer * rows * K);
        a.rows[a.nmat] = rows; a.part[a.nmat] = part[a.nmat];
        a.nmat++;
    }
    a.K = K; a.x = x; a.gps = kBatchGps;
    // All workgroups of the launch are resident at once (batch_resident() per compute unit); a wave takes one unit of 16 or 32 rows
    // after the other.  Whichever unit size gives a wave fewer rows in all is taken (32 on a tie: two tiles share the
    // activations they fetch from LDS).
    const int nb = nseq / kBatch, waves = 4 * nb;
    const int S = batch_slices(K), gmax = std::max(1, batch_resident(nseq) * c->n_cu / S);
    int tiles = 2, gx = 1, best = 1 << 30;
    for (int t = 2; t >= 1; t--) {
        int units = 0;
        for (int i = 0; i < a.nmat; i++) units += bg_units(a.rows[i], t);
        const int g = std::min(gmax, (units + waves - 1) / waves), iters = (units + waves * g - 1) / (waves * g);
        if (iters * t < best) {
            best = iters * t; tiles = t;
            gx = (units + waves * iters - 1) / (waves * iters);   // no more workgroups than that many rounds need
        }
    }
    BT(*tensors.begin() == L2J_WQ ? "gemm qkv" : *tensors.begin() == L2J_WO ? "gemm wo" : *tensors.begin() == L2J_W2 ? "gemm w2" : "gemm w1,w3");
    const dim3 grid(gx, S), block(kBgThreads * nb);
    const size_t lds = batch_lds(nseq);
    if (nb == 1) {
        if (tiles == 1) hipLaunchKernelGGL((k_bgemm<1, 1>), grid, block, lds, c->stream, a);
        else hipLaunchKernelGGL((k_bgemm<2, 1>), grid, block, lds, c->stream, a);
    } else {
        if (tiles == 1) hipLaunchKernelGGL((k_bgemm<1, 2>), grid, block, lds, c->stream, a);
        else hipLaunchKernelGGL((k_bgemm<2, 2>), grid, block, lds, c->stream, a);
    }
}

// One position of all sequences: embedding, the layers, the classifier, the next tokens.
void launch_batch_step(l2j_ctx *c, BatchBufs &b, int max_pos, int prompt_stride, int nseq)
{
    const l2j_config &cf = c->cfg;
    const int dim = cf.dim, hidden = cf.hidden_dim, L = cf.n_layers, hs = c->head_size, kvd = c->kv_dim;
    const int sd = batch_slices(dim), sh = batch_slices(hidden);
    hipStream_t s = c->stream;
    { BT("embed"); hipLaunchKernelGGL(k_bembed, dim3(nseq), dim3(256), 0, s, c->emb, b.st, b.x, dim); }
    { BT("rms"); hipLaunchKernelGGL(k_brms, dim3(nseq), dim3(1024), 0, s, b.x, c->rmsw, b.xn, dim); }
    for (int l = 0; l < L; l++) {
        launch_bgemm(c, {L2J_WQ, L2J_WK, L2J_WV}, l, b.xn, b.part, nseq);
        BAttn t{};
        t.pq = b.part[0]; t.pk = b.part[1]; t.pv = b.part[2]; t.slices = sd; t.rope = c->rope;
        t.kc = b.kc + (size_t)l * max_pos * kvd; t.vc = b.vc + (size_t)l * max_pos * kvd;
        t.seq_stride = (long)L * max_pos; t.out = b.xb; t.st = b.st;
        t.n_heads = cf.n_heads; t.kv_mul = cf.n_heads / cf.n_kv_heads; t.head_size = hs; t.kv_dim = kvd; t.dim = dim;
        t.sqrt_hs = sqrtf((float)hs);
        const dim3 ag(cf.n_heads, nseq);
        {
            BT("attention");
            if (hs == 64) hipLaunchKernelGGL(k_battn<16>, ag, dim3(256), 0, s, t);
            else if (hs == 128) hipLaunchKernelGGL(k_battn<32>, ag, dim3(256), 0, s, t);
            else hipLaunchKernelGGL(k_battn<64>, ag, dim3(256), 0, s, t);
        }
        launch_bgemm(c, {L2J_WO}, l, b.xb, b.part, nseq);
        { BT("res + rms"); hipLaunchKernelGGL(k_bres_rms, dim3(nseq), dim3(1024), 0, s, b.part[0], sd, b.x, c->rmsw + (size_t)(L + l) * dim, b.xn, dim); }
        launch_bgemm(c, {L2J_W1, L2J_W3}, l, b.xn, b.part, nseq);
        { BT("epi swiglu"); hipLaunchKernelGGL(k_bepi_swiglu, dim3(hidden / 256, nseq), dim3(256), 0, s, b.part[0], b.part[1], sd, hidden, c->silu,
                           (cf.flags & L2J_F_EXACT_SILU) ? 1 : 0, b.hb); }
        launch_bgemm(c, {L2J_W2}, l, b.hb, b.part, nseq);
        // the residual, then the norm of what follows: the next layer's attention norm, or the final one (rmsw: att, ffn, final)
        const float *wn = c->rmsw + (l + 1 < L ? (size_t)(l + 1) * dim : (size_t)2 * L * dim);
        { BT("res + rms"); hipLaunchKernelGGL(k_bres_rms, dim3(nseq), dim3(1024), 0, s, b.part[0], sh, b.x, wn, b.xn, dim); }
    }
    {
        BGemmF32 g{};
        g.w = c->wcls; g.rows = cf.vocab_size; g.K = dim; g.x = b.xn; g.part = b.part[0]; g.gps = kBatchGps;
        BT("classifier");
        const dim3 cg((cf.vocab_size + kBgRowsPerWG - 1) / kBgRowsPerWG, sd);
        if (nseq == kBatch) hipLaunchKernelGGL(k_bgemm_f32<1>, cg, dim3(kBgThreads), batch_lds_f32(nseq), s, g);
        else hipLaunchKernelGGL(k_bgemm_f32<2>, cg, dim3(kBgThreads), batch_lds_f32(nseq), s, g);
    }
    BNext n{};
    n.part = b.part[0]; n.slices = sd; n.vocab = cf.vocab_size; n.logits = b.logits; n.st = b.st; n.prompts = b.prompts;
    n.prompt_stride = prompt_stride; n.out_tokens = b.out; n.out_stride = max_pos;
    { BT("next"); hipLaunchKernelGGL(k_bnext, dim3(nseq), dim3(1024), 0, s, n, b.done); }
}

}  // namespace

int l2j_decode_greedy_batch(l2j_ctx *c, const int32_t *prompts, const int32_t *n_prompt, int32_t n_seq, int32_t prompt_stride,
                            int32_t steps, int32_t *out_tokens, double *seconds)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        if (!c || !n_prompt || !out_tokens || (prompt_stride > 0 && !prompts) || prompt_stride < 0) return fail(L2J_E_ARG, "bad argument");
        if (!c->finalized) return fail(L2J_E_STATE, "decode before l2j_finalize");
        if (n_seq != kBatch && n_seq != kMaxBatch) return fail(L2J_E_ARG, "n_seq must be 16 or 32");
        const int nseq = n_seq;
        const l2j_config &cf = c->cfg;
        const int hs = c->head_size;
        if (cf.dim % 256 || cf.hidden_dim % 256 || c->kv_dim % 16 || cf.vocab_size % 16 || (hs != 64 && hs != 128 && hs != 256))
            return fail(L2J_E_SIZE, "batched decode needs dim and hidden_dim in whole groups of 256, kv_dim and vocab_size multiples of 16, "
                                    "head_size 64, 128 or 256");
        if (steps <= 0 || steps > cf.seq_len) return fail(L2J_E_ARG, "steps must be 1..seq_len");
        for (int b = 0; b < nseq; b++) {
            if (n_prompt[b] < 0 || n_prompt[b] > prompt_stride) return fail(L2J_E_ARG, "n_prompt out of range");
            for (int i = 0; i < n_prompt[b]; i++)
                if (prompts[(size_t)b * prompt_stride + i] < 0 || prompts[(size_t)b * prompt_stride + i] >= cf.vocab_size)
                    return fail(L2J_E_ARG, "prompt id out of range");
        }
        HIPCHK(hipSetDevice(cf.device));
        if (!c->bt_ready) {   // the matrices once more, in the order the batched products read them
            for (int t : {L2J_WQ, L2J_WK, L2J_WV, L2J_WO, L2J_W1, L2J_W2, L2J_W3}) {
                const int trc = ensure_batch_tiles(c, t);
                if (trc) return trc;
            }
            c->bt_ready = true;
        }
        const int dim = cf.dim, hidden = cf.hidden_dim, L = cf.n_layers, kvd = c->kv_dim, vocab = cf.vocab_size;
        const int sd = batch_slices(dim), sh = batch_slices(hidden);
        const size_t part_floats = (size_t)nseq * std::max({(size_t)sd * std::max(hidden, vocab), (size_t)sh * dim});
        const size_t cache_floats = (size_t)nseq * L * steps * kvd;
        const int pstride = std::max(1, (int)prompt_stride);
        BatchBufs b;
        auto done = [&](int rc) { b.release(); return rc; };
        hipError_t e = hipSuccess;
        auto alloc = [&](auto **p, size_t n) {
            if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(p), n * sizeof(**p));
        };
        alloc(&b.x, (size_t)nseq * dim); alloc(&b.xn, (size_t)nseq * std::max(dim, hidden));
        alloc(&b.xb, (size_t)nseq * dim); alloc(&b.hb, (size_t)nseq * hidden); alloc(&b.logits, (size_t)nseq * vocab);
        for (int i = 0; i < 3; i++) alloc(&b.part[i], part_floats);
        alloc(&b.kc, cache_floats); alloc(&b.vc, cache_floats);
        alloc(&b.st, 1); alloc(&b.prompts, (size_t)nseq * pstride); alloc(&b.out, (size_t)nseq * steps); alloc(&b.done, 1);
        if (e == hipSuccess) e = hipEventCreate(&b.e0);
        if (e == hipSuccess) e = hipEventCreate(&b.e1);
        const size_t state_ints = sizeof(BatchState) / sizeof(int), prompt_ints = (size_t)nseq * pstride, out_ints = (size_t)nseq * steps;
        if (e == hipSuccess) e = hipHostMalloc(reinterpret_cast<void **>(&b.h_pin), std::max(state_ints + prompt_ints, out_ints) * sizeof(int), hipHostMallocDefault);
        if (e != hipSuccess) return done(fail(L2J_E_HIP, std::string("batched decode: ") + hipGetErrorString(e)));
        BatchState h{};
        h.pos = 0;
        for (int i = 0; i < nseq; i++) { h.token[i] = 1; h.n_prompt[i] = n_prompt[i]; }   // BOS first (J/Run.java:612)
        memcpy(b.h_pin, &h, sizeof(h));
        if (prompt_stride > 0) memcpy(b.h_pin + state_ints, prompts, prompt_ints * sizeof(int));
        if (hipMemcpyAsync(b.st, b.h_pin, sizeof(h), hipMemcpyHostToDevice, c->stream) != hipSuccess ||
            (prompt_stride > 0 && hipMemcpyAsync(b.prompts, b.h_pin + state_ints, prompt_ints * sizeof(int), hipMemcpyHostToDevice, c->stream) != hipSuccess) ||
            hipMemsetAsync(b.done, 0, sizeof(unsigned), c->stream) != hipSuccess ||
            hipFuncSetAttribute((const void *)k_bgemm<1, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)batch_lds(kBatch)) != hipSuccess ||
            hipFuncSetAttribute((const void *)k_bgemm<2, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)batch_lds(kBatch)) != hipSuccess ||
            hipFuncSetAttribute((const void *)k_bgemm<1, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)batch_lds(kMaxBatch)) != hipSuccess ||
            hipFuncSetAttribute((const void *)k_bgemm<2, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)batch_lds(kMaxBatch)) != hipSuccess ||
            hipFuncSetAttribute((const void *)k_bgemm_f32<1>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)batch_lds_f32(kBatch)) != hipSuccess ||
            hipFuncSetAttribute((const void *)k_bgemm_f32<2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)batch_lds_f32(kMaxBatch)) != hipSuccess ||
            hipStreamSynchronize(c->stream) != hipSuccess)
            return done(fail(L2J_E_HIP, "batched decode: set-up failed"));
        // one position as a graph: every kernel reads the position and the tokens from device memory ("graph" = 0: the
        // kernels are launched one by one, for profilers)
        const bool use_graph = c->opt[OPT_GRAPH] != 0;
        if (use_graph) {
            e = hipStreamBeginCapture(c->stream, hipStreamCaptureModeThreadLocal);
            if (e == hipSuccess) {
                launch_batch_step(c, b, steps, pstride, nseq);
                const hipError_t le = hipGetLastError();
                e = hipStreamEndCapture(c->stream, &b.graph);
                if (e == hipSuccess) e = le;
            }
            if (e == hipSuccess) e = hipGraphInstantiate(&b.exec, b.graph, nullptr, nullptr, 0);
            if (e != hipSuccess) return done(fail(L2J_E_HIP, std::string("batched decode: graph capture: ") + hipGetErrorString(e)));
        }
        for (int pos = 0; pos < steps && e == hipSuccess; pos++) {
            if (use_graph) {
                e = hipGraphLaunch(b.exec, c->stream);
            } else {
                launch_batch_step(c, b, steps, pstride, nseq);
                e = hipGetLastError();
            }
            if (pos == 0 && e == hipSuccess) e = hipEventRecord(b.e0, c->stream);   // the clock starts after the first step (J/Run.java:682-684)
        }
        if (e == hipSuccess) e = hipEventRecord(b.e1, c->stream);
#ifdef L2J_BATCH_TIMES
        if (e == hipSuccess && steps > 8) {   // one more step, kernel by kernel, each between two events (position steps - 1 again)
            (void)hipStreamSynchronize(c->stream);
            BatchState h2{};
            (void)hipMemcpy(&h2, b.st, sizeof(h2), hipMemcpyDeviceToHost);
            h2.pos = steps - 1;
            (void)hipMemcpy(b.st, &h2, sizeof(h2), hipMemcpyHostToDevice);
            g_bt_on = true; g_bt.clear();
            launch_batch_step(c, b, steps, pstride, nseq);
            g_bt_on = false;
            (void)hipStreamSynchronize(c->stream);
            std::map<std::string, std::pair<double, int>> acc;
            for (auto &t : g_bt) { float ms = 0; (void)hipEventElapsedTime(&ms, t.e0, t.e1); acc[t.name].first += ms * 1e3; acc[t.name].second++; (void)hipEventDestroy(t.e0); (void)hipEventDestroy(t.e1); }
            double tot = 0; for (auto &kv : acc) tot += kv.second.first;
            for (auto &kv : acc) fprintf(stderr, "[batch step] %-14s %4d launches %9.1f us total %7.2f us each\n", kv.first.c_str(), kv.second.second, kv.second.first, kv.second.first / kv.second.second);
            fprintf(stderr, "[batch step] sum %.1f us\n", tot);
        }
#endif
        if (e == hipSuccess) e = hipMemcpyAsync(b.h_pin, b.out, out_ints * sizeof(int), hipMemcpyDeviceToHost, c->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(c->stream);
        if (e == hipSuccess) memcpy(out_tokens, b.h_pin, out_ints * sizeof(int));
        float ms = 0.0f;
        if (e == hipSuccess && steps > 1) e = hipEventElapsedTime(&ms, b.e0, b.e1);
        if (seconds) *seconds = (double)ms * 1e-3;
        if (e != hipSuccess) return done(fail(L2J_E_HIP, std::string("batched decode: ") + hipGetErrorString(e)));
        return done(L2J_OK);
    }());
}

int l2j_read(l2j_ctx *c, int which, int layer, uint64_t off, float *dst, uint64_t n)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        if (!c || !dst) return fail(L2J_E_ARG, "null argument");
        if (which < 0 || which >= L2J_B_COUNT) return fail(L2J_E_ARG, "unknown buffer");
        HIPCHK(hipSetDevice(c->cfg.device));
        const l2j_config &g = c->cfg;
        const float *src = nullptr;
        uint64_t len = 0;
        if (which == L2J_B_KCACHE || which == L2J_B_VCACHE) {
            if (layer < 0 || layer >= g.n_layers) return fail(L2J_E_ARG, "layer out of range");
            len = (uint64_t)g.seq_len * c->kv_dim;
            src = (which == L2J_B_KCACHE ? c->kcache : c->vcache) + (uint64_t)layer * len;
        } else if (which == L2J_B_LOGITS) {
            src = c->logits; len = g.vocab_size;
        } else if (layer < 0) {
            // the vectors of the last token: set 0, or with a self-contained token kernel the set it picked by the epoch
            uint64_t so = 0;
            if ((c->self_contained & 1) && !c->acts_dirty) {
                int epoch = 0;
                HIPCHK(hipStreamSynchronize(c->stream));
                HIPCHK(hipMemcpy(&epoch, &c->st->epoch, sizeof(int), hipMemcpyDeviceToHost));
                so = ((epoch - 1) & 1) ? c->set_floats : 0;
            }
            switch (which) {
            case L2J_B_X: src = c->x + so + 2ull * g.n_layers * c->sd; len = g.dim; break;  // the last layer's vectors
            case L2J_B_XB: src = c->xb + so + (uint64_t)(g.n_layers - 1) * c->sd; len = g.dim; break;
            case L2J_B_HB: src = c->hb + so + (uint64_t)(g.n_layers - 1) * c->sh; len = g.hidden_dim; break;
            case L2J_B_Q: src = c->q + so + (uint64_t)(g.n_layers - 1) * c->sd; len = g.dim; break;
            default: return fail(L2J_E_ARG, "this buffer only exists as a per-layer tap");
            }
        } else {
            if (layer >= g.n_layers) return fail(L2J_E_ARG, "layer out of range");
            if (!c->taps[which]) return fail(L2J_E_STATE, "no taps recorded: call l2j_forward_taps first");
            len = which == L2J_B_HB ? g.hidden_dim : (which == L2J_B_K || which == L2J_B_V) ? c->kv_dim : g.dim;
            src = c->taps[which] + (uint64_t)layer * len;
        }
        if (off + n > len) return fail(L2J_E_SIZE, "read past the end of the buffer");
        HIPCHK(hipStreamSynchronize(c->stream));
        HIPCHK(hipMemcpy(dst, src + off, n * sizeof(float), hipMemcpyDeviceToHost));
        return L2J_OK;
    }());
}

int l2j_write_kv(l2j_ctx *c, int layer, int32_t pos0, int32_t npos, const float *k, const float *v)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        if (!c || !k || !v) return fail(L2J_E_ARG, "null argument");
        if (layer < 0 || layer >= c->cfg.n_layers) return fail(L2J_E_ARG, "layer out of range");
        if (pos0 < 0 || npos < 0 || (int64_t)pos0 + npos > c->cfg.seq_len) return fail(L2J_E_ARG, "positions out of range");
        HIPCHK(hipSetDevice(c->cfg.device));
        const uint64_t o = ((uint64_t)layer * c->cfg.seq_len + pos0) * c->kv_dim, n = (uint64_t)npos * c->kv_dim;
        HIPCHK(hipStreamSynchronize(c->stream));
        HIPCHK(hipMemcpy(c->kcache + o, k, n * sizeof(float), hipMemcpyHostToDevice));
        HIPCHK(hipMemcpy(c->vcache + o, v, n * sizeof(float), hipMemcpyHostToDevice));
        return L2J_OK;
    }());
}

int l2j_calibration_copy(l2j_ctx *c, uint64_t nbytes, int32_t rounds)
{
    return ctx_rc(c, [&]() -> int {
        if (!c || nbytes < 16 || rounds <= 0) return fail(L2J_E_ARG, "bad argument");
        HIPCHK(hipSetDevice(c->cfg.device));
        uint4 *a = nullptr, *b = nullptr;
        const long n = (long)(nbytes / 16);
        HIPCHK(hipMalloc(reinterpret_cast<void **>(&a), (size_t)n * 16));
        hipError_t e = hipMalloc(reinterpret_cast<void **>(&b), (size_t)n * 16);
        if (e == hipSuccess) e = hipMemsetAsync(a, 1, (size_t)n * 16, c->stream);
        for (int r = 0; r < rounds && e == hipSuccess; r++) {
            hipLaunchKernelGGL(k_copy16, dim3(c->n_cu * 8), dim3(256), 0, c->stream, a, b, n);
            e = hipGetLastError();
        }
        if (e == hipSuccess) e = hipStreamSynchronize(c->stream);
        (void)hipFree(a);
        (void)hipFree(b);
        if (e != hipSuccess) return fail(L2J_E_HIP, std::string("calibration copy: ") + hipGetErrorString(e));
        return L2J_OK;
    }());
}

uint64_t l2j_bytes_per_token(const l2j_config *g, int32_t pos)
{
    if (!g) return 0;
    const uint64_t L = g->n_layers, dim = g->dim, hid = g->hidden_dim;
    const uint64_t kvd = (uint64_t)g->n_kv_heads * (g->dim / g->n_heads);
    const uint64_t mat = L * (2 * dim * dim + 2 * dim * kvd + 3 * dim * hid);
    return quant_bytes_of(mat) + 2 * quant_bytes_of(L * dim) + quant_bytes_of(dim) + (uint64_t)g->vocab_size * dim * 4 + dim * 4 +
           2 * L * (uint64_t)(pos + 1) * kvd * 4 + 2 * L * kvd * 4;
}

int l2j_time_kernel(l2j_ctx *c, int kclass, int32_t pos, int32_t rounds, double *mean_us, uint64_t *bytes)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        if (!c || !mean_us) return fail(L2J_E_ARG, "null argument");
        if (kclass < 0 || kclass >= L2J_K_COUNT || rounds <= 0) return fail(L2J_E_ARG, "bad kernel class or rounds");
        int rc = check_forward_args(c, 1, pos);
        if (rc) return rc;
        const l2j_config &g = c->cfg;
        const uint64_t dim = g.dim, hid = g.hidden_dim, kvd = c->kv_dim;
        uint64_t b = 0;
        switch (kclass) {
        case L2J_K_QKV: b = quant_bytes_of(dim * dim + 2 * dim * kvd) + quant_bytes_of(dim); break;
        case L2J_K_ATTENTION: b = 2ull * (pos + 1) * kvd * 4; break;
        case L2J_K_WO: b = quant_bytes_of(dim * dim); break;
        case L2J_K_W13: b = quant_bytes_of(2 * dim * hid) + quant_bytes_of(dim); break;
        case L2J_K_W2: b = quant_bytes_of(dim * hid); break;
        case L2J_K_CLASSIFIER: b = (uint64_t)g.vocab_size * dim * 4 + quant_bytes_of(dim); break;
        case L2J_K_TOKEN: b = l2j_bytes_per_token(&g, pos); break;
        }
        if (bytes) *bytes = b;
        if (kclass == L2J_K_TOKEN) {  // the whole-token kernel (and, unless it is self-contained, k_finish after it, untimed)
            if (!c->fused) return fail(L2J_E_STATE, "the whole-token kernel is switched off or does not fit this shape");
            if (rounds > 256) return fail(L2J_E_ARG, "at most 256 rounds of the whole-token kernel");
            while ((int)c->events.size() < 33 + 2 * rounds) {
                hipEvent_t ev;
                HIPCHK(hipEventCreate(&ev));
                c->events.push_back(ev);
            }
            // the rounds follow each other on the stream without a host round trip in between, as the tokens of a decode do
            for (int r = 0; r < rounds; r++) {
                if ((rc = set_state(c, 1, pos, 0))) return rc;
                HIPCHK(clean_activations(c));
                if (c->layers_per_launch != g.n_layers) return fail(L2J_E_STATE, "the token is split over several launches");
                hipError_t e = launch_token(c, c->stream, false, c->events[33 + 2 * r], c->events[34 + 2 * r]);
                if (e != hipSuccess) return fail(L2J_E_HIP, std::string("launch: ") + hipGetErrorString(e));
            }
            HIPCHK(hipStreamSynchronize(c->stream));
            if ((rc = check_barrier_error(c)))
                return rc == kRepeatToken ? fail(L2J_E_HIP, "a bounded wait of the whole-token kernel ran out; the context now launches phase by phase") : rc;
            double total = 0.0;
            for (int r = 0; r < rounds; r++) {
                float ms = 0.f;
                HIPCHK(hipEventElapsedTime(&ms, c->events[33 + 2 * r], c->events[34 + 2 * r]));
                total += ms;
            }
            *mean_us = total * 1e3 / rounds;
            return L2J_OK;
        }
        c->acts_dirty = true;  // a phase launched on its own leaves values in its output vector
        const int per_round = kclass == L2J_K_CLASSIFIER ? 1 : g.n_layers;
        while ((int)c->events.size() < 2 * per_round + 33) {
            hipEvent_t ev;
            HIPCHK(hipEventCreate(&ev));
            c->events.push_back(ev);
        }
        // The activations hold whatever the last forward left; timing does not depend on their values.
        double total_ms = 0.0;
        long count = 0;
        for (int r = 0; r < rounds; r++) {
            if ((rc = set_state(c, 1, pos, 0))) return rc;
            for (int l = 0; l < per_round; l++) {
                hipError_t e = launch_class(c, kclass, l, c->stream, c->events[33 + 2 * l], c->events[34 + 2 * l]);
                if (e != hipSuccess) return fail(L2J_E_HIP, std::string("launch: ") + hipGetErrorString(e));
            }
            HIPCHK(hipStreamSynchronize(c->stream));
            for (int l = 0; l < per_round; l++) {
                float ms = 0.f;
                HIPCHK(hipEventElapsedTime(&ms, c->events[33 + 2 * l], c->events[34 + 2 * l]));
                total_ms += ms;
                count++;
            }
        }
        *mean_us = total_ms * 1e3 / (double)count;
        return L2J_OK;
    }());
}

}  // extern "C"
