// libllama2j_hip.so: launch shapes, hipGraph capture, the forward passes, the decode loops and kernel timing.
#include "l2j_internal.hpp"

using namespace l2j;

namespace l2j {
std::mutex g_forward_mu;
}

namespace {

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

// k_token: the largest LDS need of its phases
size_t layer_smem(const l2j_ctx *c)
{
    return std::max(mv_smem(std::max(c->cfg.dim, c->cfg.hidden_dim)), attn_smem_for(c, c->pk_threads));
}

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
        if (tud == kTU) return f(k_token<32, kTU, kTU, true>);
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

}  // namespace

hipError_t l2j::launch_one_token(l2j_ctx *c)
{
    hipError_t e = clean_activations(c);
    if (e != hipSuccess) return e;
    return c->graph_exec ? hipGraphLaunch(c->graph_exec, c->stream) : launch_token(c, c->stream, false);
}

namespace {


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

}  // namespace

// After a synchronize: a workgroup whose bounded wait ran out has set the flag.  The whole-token kernel needs all its
// workgroups resident at once; when something else holds compute units (another process on the GPU) its waits run
// out.  With the "fallback" option the context then gives the whole-token kernel up for good: one launch per phase
// needs no residency, and the caller repeats what failed (kRepeatToken).
int l2j::check_barrier_error(l2j_ctx *c)
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

namespace {

}  // namespace

int l2j::set_state(l2j_ctx *c, int token, int pos, int n_prompt)
{
    c->h_st->token = token;
    c->h_st->pos = pos;
    c->h_st->n_prompt = n_prompt;
    // (the device owns DevState::epoch: every token adds one, and a self-contained k_token picks its set of vectors by it)
    HIPCHK(hipMemcpyAsync(c->st, c->h_st, offsetof(DevState, epoch), hipMemcpyHostToDevice, c->stream));
    return L2J_OK;
}

namespace {

int check_forward_args(l2j_ctx *c, int32_t token, int32_t pos)
{
    if (!c) return fail(L2J_E_ARG, "null context");
    if (!c->finalized) return fail(L2J_E_STATE, "forward before l2j_finalize");
    if (token < 0 || token >= c->cfg.vocab_size) return fail(L2J_E_ARG, "token out of range");
    if (pos < 0 || pos >= c->cfg.seq_len) return fail(L2J_E_ARG, "pos out of range");
    HIPCHK(hipSetDevice(c->cfg.device));
    return L2J_OK;
}

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

    // Option prefill: the first P prompt positions (whole steps of 32; their outputs are the prompt's own ids, J/Run.java:635-637)
    // through the batched products, the loop then goes on at position P.  Not when one of those ids is 1 (the loop would
    // have stopped there, J/Run.java:670-672), nor for shapes the batched products do not take.
    int P = 0;
    double prefill_s = 0.0;
    if (c->opt[OPT_PREFILL] != 0 && np >= 32 && steps > 32) {
        P = std::min(np, steps - 1) / 32 * 32;
        for (int i = 0; i < P; i++)
            if (prompt[i] == 1) P = 0;
        if (P > 0) {
            std::vector<int32_t> in((size_t)P);
            in[0] = 1;
            for (int i = 1; i < P; i++) in[i] = prompt[i - 1];
            rc = prefill_positions(c, in.data(), P, 0, nullptr, &prefill_s);
            if (rc == L2J_E_SIZE) {
                P = 0;   // (a shape for l2j_forward only)
            } else if (rc) {
                return rc;
            } else {
                for (int i = 0; i < P; i++) out_tokens[i] = prompt[i];
                if ((rc = set_state(c, prompt[P - 1], P, np))) return rc;
            }
        }
    }

    // The stop rule (next == 1) is checked per batch of tokens, and the clock runs from the end of the first token to
    // the end of the token that ended the loop (plus, with option prefill, the device time of its steps).
    float total_ms = 0.f;
    int pos = P;
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
        int enq = P, nbatch = 0, done_batches = 0;  // positions enqueued; batches enqueued and processed
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
            if (pos == P) t_first = c->h_tstamp[P];
            t_last = c->h_tstamp[pos + used - 1];
            pos += used;
        }
        HIPCHK(hipStreamSynchronize(c->stream));  // a batch enqueued ahead of a stop
        if ((rc = check_barrier_error(c))) return rc;
        // (a device that does not tell its wall-clock rate: the loop is not timed, *seconds = 0)
        total_ms = c->wall_clock_hz > 0.0 ? (float)((double)(t_last - t_first) / c->wall_clock_hz * 1e3) : 0.0f;
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
                if (pos + i == P) HIPCHK(hipEventRecord(ev_first, c->stream));
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
            if (pos + used - 1 > P) HIPCHK(hipEventElapsedTime(&total_ms, ev_first, c->events[used - 1]));
            pos += used;
        }
    }
    *n_out = pos;
    if (seconds) *seconds = (double)total_ms * 1e-3 + prefill_s;
    return L2J_OK;
}


}  // namespace

// The end of l2j_finalize: launch shapes (one 1024-thread workgroup per compute unit for the weight-streaming kernels),
// kernel attributes, the scratch of the phases, then the graphs.
int l2j::setup_forward(l2j_ctx *c)
{
    {
        const int nmax = std::max(c->cfg.dim, c->cfg.hidden_dim);
        const int *o = c->opt;
        // Short rows leave most of 1024 threads without a chunk while every workgroup barrier and hand-over still waits for
        // all sixteen waves: 110M shape 239 / 228 / 222 / 227 us per token with 1024 / 768 / 512 / 384 threads, 15M shape
        // 123 / 118 / 121 / 125 with 1024 / 640 / 512 / 384.
        const int auto_threads = nmax <= 1024 ? 640 : nmax <= 4096 ? 512 : 1024;
        c->pk_threads = std::min(1024, std::max(64, (o[OPT_THREADS] != kAuto ? o[OPT_THREADS] : auto_threads) / 64 * 64));
        c->pk_grid = std::max(1, o[OPT_GRID] != kAuto ? o[OPT_GRID] : c->n_cu);  // one workgroup per compute unit
        c->attn_threads = std::min(1024, std::max(64, o[OPT_ATTN_THREADS] / 64 * 64));
        c->attn_rows = std::max(1, o[OPT_ATTN_ROWS]);
        c->attn_nsplit = std::max(1, o[OPT_ATTN_NSPLIT]);
        c->attn_grid = c->cfg.n_heads * c->attn_nsplit;
        c->fused_attn_rows = std::max(1, o[OPT_FUSED_ATTN_ROWS]);
        const size_t need = std::max(std::max(mv_smem(nmax), attn_smem(c)), layer_smem(c));
        if (need > 160 * 1024) return fail(L2J_E_ARG, "hidden_dim does not fit the 160 KB LDS");
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
        // One launch per token pays off when a hand-over inside the kernel costs less than a kernel boundary of the
        // replayed graph: measured whole-token / one launch per phase, 7B shape (208 MB a layer) 1.44 / 1.96 ms per token,
        // 110M shape (7 MB) 0.241 / 0.278 ms, 15M shape (1 MB) 0.123 / 0.134 ms.  Below half a million weights a layer
        // (test models) the phases stay separate launches.
        const uint64_t layer_floats = 2ull * c->cfg.dim * c->cfg.dim + 2ull * c->cfg.dim * c->kv_dim + 3ull * c->cfg.dim * c->cfg.hidden_dim;
        c->fused = (c->opt[OPT_FUSE] != kAuto ? c->opt[OPT_FUSE] : layer_floats >= (1ull << 19) ? 1 : 0) != 0;
        c->layers_per_launch = std::max(1, std::min(c->cfg.n_layers, c->opt[OPT_LAYERS_PER_LAUNCH] != kAuto ? c->opt[OPT_LAYERS_PER_LAUNCH] : c->cfg.n_layers));
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
    return capture_graphs(c);
}

// What setup_forward allocates (also after a finalize that failed part-way, so that it can be called again).
void l2j::release_forward(l2j_ctx *c)
{
    destroy_graph(c);
    (void)hipFree(c->cls_part);
    (void)hipFree(c->attn_part);
    (void)hipFree(c->bar_ctr);
    (void)hipFree(c->fault);
    if (c->h_fault) (void)hipHostFree(c->h_fault);
    c->cls_part = nullptr; c->attn_part = nullptr; c->bar_ctr = nullptr;
    c->fault = nullptr; c->h_fault = nullptr;
}

extern "C" {

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
