// libllama2j_hip.so: several sequences at once (l2j_decode_greedy_batch, l2j_batch_matmul).
#include "l2j_internal.hpp"
#include "batch_kernels.hpp"
#include "batch_step.hpp"

using namespace l2j;

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

// The tile-ordered copy of `tensor` for the batched path (rows % 16 == 0 and K % 256 == 0 checked by the caller; the
// caller holds the context's upload lock: an upload of the tensor marks the copy stale, invalidate_batch_tiles).
static int ensure_batch_tiles(l2j_ctx *c, int tensor)
{
    if (c->bt_done[tensor]) return L2J_OK;
    int rows = 0, K = 0;
    if (!matrix_shape(c->cfg, tensor, &rows, &K)) return fail(L2J_E_ARG, "not a matrix tensor");
    const QTensor &t = c->qt[tensor];
    if (t.groups_loaded < t.ngroups) return fail(L2J_E_STATE, "tensor not uploaded");
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

extern "C" {

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
        (void)groups_per_slice;   // (a slice of K is four groups since the activations stay in the waves' registers)
        const int slices = bg_slices(K);
        const size_t lds = bg_lds_bytes(kBatch, 2);
        HIPCHK(hipSetDevice(c->cfg.device));
        {
            std::lock_guard<std::mutex> lock(c->upload_mu);
            const int trc = ensure_batch_tiles(c, tensor);
            if (trc) return trc;
        }
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
        if (e == hipSuccess) e = hipFuncSetAttribute((const void *)k_bgemm<1, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e == hipSuccess) e = hipMemcpyAsync(dx, x, (size_t)kBatch * K * sizeof(float), hipMemcpyHostToDevice, c->stream);
        if (e == hipSuccess) {
            BGemm a{};
            a.m[0] = bqmat(c, tensor, (uint64_t)layer * rows * K);
            a.rows[0] = rows; a.part[0] = dpart; a.nmat = 1; a.K = K; a.x = dx;
            const dim3 grid(std::min(rows / 16, std::max(1, c->n_cu / slices)), slices);
            const int n = std::max(1, (int)rounds);
            hipLaunchKernelGGL((k_bgemm<1, 2>), grid, dim3(2 * kBgThreads), lds, c->stream, a);   // warm
            (void)hipEventRecord(e0, c->stream);
            for (int i = 0; i < n; i++) hipLaunchKernelGGL((k_bgemm<1, 2>), grid, dim3(2 * kBgThreads), lds, c->stream, a);
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
        if (e != hipSuccess) return fail(e == hipErrorOutOfMemory ? L2J_E_OOM : L2J_E_HIP, std::string("batch matmul: ") + hipGetErrorString(e));
        return L2J_OK;
    }());
}

}  // extern "C"

// ---- several sequences at once ----------------------------------------------------------------------------------

// Device memory, pinned staging and the captured step of the batched decode.  The context owns one set, made by the first
// l2j_decode_greedy_batch and kept until l2j_destroy; a call that needs more (other sequence count, more steps, longer
// prompts) replaces it.  No call allocates or captures anything once the set fits.
struct l2j::BatchBufs {
    int nseq = 0, cap_steps = 0, cap_pstride = 0;   // what the buffers and the graph's kernel arguments are made for
    float *x = nullptr, *xn = nullptr, *xb = nullptr, *hb = nullptr, *logits = nullptr;
    float *part[3] = {nullptr, nullptr, nullptr};
    float *kc = nullptr, *vc = nullptr;             // (sequence, layer, kv head, cap_steps, head_size)
    BatchState *st = nullptr;
    int *prompts = nullptr, *out = nullptr;         // (sequence, cap_pstride), (sequence, cap_steps)
    unsigned *done = nullptr;
    unsigned *bar_ctr = nullptr;   // k_bstep: the counters of its grid barrier,
    int *fault = nullptr;          // the flag a bounded wait sets when it runs out,
    float *ssq = nullptr;          // the sums of squares behind the two norms of a layer,
    BStep *step_args = nullptr;    // its argument (fixed for the life of the buffers)
    int step_grid = 0;             // workgroups of k_bstep (0: the layers run as eight launches each)
    int fuse_opt = 0;              // option batch_fuse when the step was planned
    int h_fault = 0;
    int *h_pin = nullptr;   // pinned: every transfer of a call goes through it, as in the single-sequence loops
    BatchSamplers samplers;   // l2j_decode_sample_batch: a sampler per sequence (made by its first call)
    float *pf_part = nullptr;      // l2j_prefill: what the workgroups that share a head's keys leave for the one that merges,
    unsigned *pf_cnt = nullptr;    // and how many have (zero between launches)
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    void release()
    {
        if (exec) (void)hipGraphExecDestroy(exec);
        if (graph) (void)hipGraphDestroy(graph);
        if (e0) (void)hipEventDestroy(e0);
        if (e1) (void)hipEventDestroy(e1);
        void *ps[] = {x, xn, xb, hb, logits, part[0], part[1], part[2], kc, vc, st, prompts, out, done, bar_ctr, fault, ssq, step_args,
                      pf_part, pf_cnt};
        for (void *p : ps) (void)hipFree(p);
        free_batch_samplers(&samplers);
        if (h_pin) (void)hipHostFree(h_pin);
    }
};

void l2j::free_batch(l2j_ctx *c)
{
    if (c->batch) {
        c->batch->release();
        delete c->batch;
        c->batch = nullptr;
    }
    for (int t = 0; t < L2J_TENSOR_COUNT; t++) {
        (void)hipFree(c->bt_codes[t]);
        (void)hipFree(c->bt_gs[t]);
        c->bt_codes[t] = nullptr; c->bt_gs[t] = nullptr; c->bt_done[t] = false;
    }
    c->bt_ready = false;
}

void l2j::invalidate_batch_tiles(l2j_ctx *c, int tensor)
{
    c->bt_done[tensor] = false;
    c->bt_ready = false;
}

namespace {

constexpr int kClsGps = 2;   // k_bgemm_f32: groups of 256 floats per slice of K

int batch_slices(int K) { return bg_slices(K); }
int cls_slices(int K) { return (K / 256 + kClsGps - 1) / kClsGps; }
size_t batch_lds(int nseq) { return bg_lds_bytes(nseq, 2); }                 // k_bgemm: two waves per group for 16 and for 32 sequences
size_t step_lds(int nseq) { return bg_lds_bytes(nseq, nseq / kBatch); }       // k_bstep: 256 threads per 16 sequences
size_t batch_lds_f32(int nseq) { return (size_t)nseq * (kClsGps * 256 + kXPad) * sizeof(float); }   // k_bgemm_f32: floats
// workgroups of k_bgemm a compute unit holds at once (eight waves each: two per SIMD by their registers)
int batch_resident(int) { return 1; }

// The product of one layer's matrices `tensors` (the same input, the same row length) as one k_bgemm argument.
BGemm bgemm_args(l2j_ctx *c, std::initializer_list<int> tensors, int layer, const float *x, float *const *part)
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
    a.K = K; a.x = x;
    return a;
}

// The workgroups per slice of K: at most gmax (all of a launch resident at once); every workgroup takes every gx-th tile of
// 16 rows, in batches of as many tiles as it has waves, so no more workgroups than the number of rounds needs.
int bgemm_shape(const BGemm &a, int gmax)
{
    int tiles = 0;
    for (int i = 0; i < a.nmat; i++) tiles += a.rows[i] / 16;
    const int g = std::max(1, std::min(gmax, tiles)), iters = (tiles + g - 1) / g;
    return (tiles + iters - 1) / iters;
}

// The products of one layer's matrices in one launch.
void launch_bgemm(l2j_ctx *c, std::initializer_list<int> tensors, int layer, const float *x, float *const *part, int nseq)
{
    const BGemm a = bgemm_args(c, tensors, layer, x, part);
    const int nb = nseq / kBatch;
    const int S = batch_slices(a.K), gmax = std::max(1, batch_resident(nseq) * c->n_cu / S);
    const dim3 grid(bgemm_shape(a, gmax), S), block(kBgThreads * 2);
    if (nb == 1) hipLaunchKernelGGL((k_bgemm<1, 2>), grid, block, batch_lds(nseq), c->stream, a);
    else hipLaunchKernelGGL((k_bgemm<2, 2>), grid, block, batch_lds(nseq), c->stream, a);
}

// The grid of k_bstep: one workgroup per compute unit, all resident (by the runtime's count for the kernel and its LDS);
// 0 when the shape does not fit (a product with more slices of K than workgroups) or the option is off.
hipError_t plan_bstep(l2j_ctx *c, BatchBufs &b, int nseq)
{
    b.step_grid = 0;
    if (!c->opt[OPT_BATCH_FUSE]) return hipSuccess;
    const void *kernel = nseq == kBatch ? (const void *)k_bstep<1> : (const void *)k_bstep<2>;
    hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)step_lds(nseq));
    if (e != hipSuccess) return e;
    int per_cu = 0;
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, kBgThreads * (nseq / kBatch), step_lds(nseq));
    if (e != hipSuccess) return e;
    if (per_cu < 1 || c->n_cu < batch_slices(c->cfg.hidden_dim) || c->n_cu < batch_slices(c->cfg.dim)) return hipSuccess;
    b.step_grid = c->n_cu;
    return hipSuccess;
}

// The argument of k_bstep for these buffers.
BStep bstep_args(l2j_ctx *c, BatchBufs &b, int max_pos, int nseq)
{
    const l2j_config &cf = c->cfg;
    BStep a{};
    a.g[BS_QKV] = bgemm_args(c, {L2J_WQ, L2J_WK, L2J_WV}, 0, b.xn, b.part);
    a.g[BS_WO] = bgemm_args(c, {L2J_WO}, 0, b.xb, b.part);
    a.g[BS_W13] = bgemm_args(c, {L2J_W1, L2J_W3}, 0, b.xn, b.part);
    a.g[BS_W2] = bgemm_args(c, {L2J_W2}, 0, b.hb, b.part);
    for (int k = 0; k < 4; k++) a.gx[k] = bgemm_shape(a.g[k], std::max(1, b.step_grid / batch_slices(a.g[k].K)));
    a.n_layers = cf.n_layers; a.nseq = nseq; a.dim = cf.dim; a.hidden = cf.hidden_dim; a.n_heads = cf.n_heads;
    a.kv_mul = cf.n_heads / cf.n_kv_heads; a.head_size = c->head_size; a.kv_dim = c->kv_dim;
    a.sqrt_hs = sqrtf((float)c->head_size);
    a.rope = c->rope; a.kc = b.kc; a.vc = b.vc; a.seq_stride = (long)cf.n_layers * max_pos * c->kv_dim; a.layer_stride = (long)max_pos * c->kv_dim; a.cap = max_pos; a.st = b.st;
    a.x = b.x; a.xn = b.xn; a.xb = b.xb; a.hb = b.hb; a.rmsw = c->rmsw; a.ssq = b.ssq;
    a.silu = c->silu; a.exact = (cf.flags & L2J_F_EXACT_SILU) ? 1 : 0;
    a.bar.ctr = b.bar_ctr; a.bar.fault = b.fault; a.bar.ngroups = kBarGroups; a.bar.maxspin = c->opt[OPT_BARRIER_SPINS];
    return a;
}

// All layers of a step in one launch.
void launch_bstep(l2j_ctx *c, BatchBufs &b, int nseq)
{
    const dim3 grid(b.step_grid), block(kBgThreads * (nseq / kBatch));
    const BStep *args = b.step_args;
    if (nseq == kBatch) hipLaunchKernelGGL(k_bstep<1>, grid, block, step_lds(nseq), c->stream, args);
    else hipLaunchKernelGGL(k_bstep<2>, grid, block, step_lds(nseq), c->stream, args);
}

// One position of all sequences: embedding, the layers, the classifier, the next tokens.
void launch_batch_step(l2j_ctx *c, BatchBufs &b, int max_pos, int prompt_stride, int nseq)
{
    const l2j_config &cf = c->cfg;
    const int dim = cf.dim, hidden = cf.hidden_dim, L = cf.n_layers, hs = c->head_size, kvd = c->kv_dim;
    const int sd = batch_slices(dim), sh = batch_slices(hidden);
    hipStream_t s = c->stream;
    { hipLaunchKernelGGL(k_bembed, dim3(nseq), dim3(256), 0, s, c->emb, b.st, b.x, dim, b.step_grid > 0 ? b.bar_ctr : nullptr); }
    { hipLaunchKernelGGL(k_brms, dim3(nseq), dim3(1024), 0, s, b.x, c->rmsw, b.xn, dim); }
    if (b.step_grid > 0) {
        launch_bstep(c, b, nseq);
        { hipLaunchKernelGGL(k_brms, dim3(nseq), dim3(1024), 0, s, b.x, c->rmsw + (size_t)2 * L * dim, b.xn, dim); }   // the final norm
    }
    for (int l = 0; l < L && b.step_grid == 0; l++) {
        launch_bgemm(c, {L2J_WQ, L2J_WK, L2J_WV}, l, b.xn, b.part, nseq);
        BAttn t{};
        t.pq = b.part[0]; t.pk = b.part[1]; t.pv = b.part[2]; t.slices = sd; t.rope = c->rope;
        t.kc = b.kc + (size_t)l * max_pos * kvd; t.vc = b.vc + (size_t)l * max_pos * kvd;
        t.seq_stride = (long)L * max_pos * kvd; t.cap = max_pos; t.out = b.xb; t.st = b.st;
        t.n_heads = cf.n_heads; t.kv_mul = cf.n_heads / cf.n_kv_heads; t.head_size = hs; t.kv_dim = kvd; t.dim = dim;
        t.sqrt_hs = sqrtf((float)hs);
        const dim3 ag(cf.n_heads, nseq);
        {
            if (hs == 64) hipLaunchKernelGGL(k_battn<16>, ag, dim3(256), 0, s, t);
            else if (hs == 128) hipLaunchKernelGGL(k_battn<32>, ag, dim3(256), 0, s, t);
            else hipLaunchKernelGGL(k_battn<64>, ag, dim3(256), 0, s, t);
        }
        launch_bgemm(c, {L2J_WO}, l, b.xb, b.part, nseq);
        { hipLaunchKernelGGL(k_bres_rms, dim3(nseq), dim3(1024), 0, s, b.part[0], sd, b.x, c->rmsw + (size_t)(L + l) * dim, b.xn, dim); }
        launch_bgemm(c, {L2J_W1, L2J_W3}, l, b.xn, b.part, nseq);
        { hipLaunchKernelGGL(k_bepi_swiglu, dim3(hidden / 256, nseq), dim3(256), 0, s, b.part[0], b.part[1], sd, hidden, c->silu,
                           (cf.flags & L2J_F_EXACT_SILU) ? 1 : 0, b.hb); }
        launch_bgemm(c, {L2J_W2}, l, b.hb, b.part, nseq);
        // the residual, then the norm of what follows: the next layer's attention norm, or the final one (rmsw: att, ffn, final)
        const float *wn = c->rmsw + (l + 1 < L ? (size_t)(l + 1) * dim : (size_t)2 * L * dim);
        { hipLaunchKernelGGL(k_bres_rms, dim3(nseq), dim3(1024), 0, s, b.part[0], sh, b.x, wn, b.xn, dim); }
    }
    {
        BGemmF32 g{};
        g.w = c->wcls; g.rows = cf.vocab_size; g.K = dim; g.x = b.xn; g.part = b.part[0]; g.gps = kClsGps;
        const dim3 cg((cf.vocab_size + kBgRowsPerWG - 1) / kBgRowsPerWG, cls_slices(dim));
        if (nseq == kBatch) hipLaunchKernelGGL(k_bgemm_f32<1>, cg, dim3(kBgThreads), batch_lds_f32(nseq), s, g);
        else hipLaunchKernelGGL(k_bgemm_f32<2>, cg, dim3(kBgThreads), batch_lds_f32(nseq), s, g);
    }
    BNext n{};
    n.part = b.part[0]; n.slices = cls_slices(dim); n.vocab = cf.vocab_size; n.logits = b.logits; n.st = b.st; n.prompts = b.prompts;
    n.prompt_stride = prompt_stride; n.out_tokens = b.out; n.out_stride = max_pos;
    { hipLaunchKernelGGL(k_bnext, dim3(nseq), dim3(1024), 0, s, n, b.done); }
}


// Measured at the 7B shape (kernel trace, per launch, a step's first position p): every row for itself (k_battn<LPR, 2>) 6.1 us at
// p = 0, 8.8 at 32, 11.0 at 64 and 2.1 more per 32 positions; k_pflash in one workgroup per head and half 8.1, 9.7, 11.2 and
// then 0.6-1 more per 32 positions; with the keys split over four workgroups 12.4 at p = 0, 14.4 at 160, 14.6 at 192, 18.0 at 608.
constexpr int kPflashFrom = 64;         // k_pflash from this position on
constexpr int kPflashSplitFrom = 192;   // and the keys of a head split over several workgroups from this one on

constexpr int kPflashMaxSplit = 4;
// Workgroups per (head, 16 positions): the keys split so that the launch has a workgroup for every compute unit.
int pflash_split(l2j_ctx *c, int first_pos)
{
    const int opt = c->opt[OPT_PREFILL_SPLIT];
    if (opt <= 0 && first_pos < kPflashSplitFrom) return 1;
    const int fit = opt > 0 ? opt : c->n_cu / (2 * c->cfg.n_heads);
    return std::min(kPflashMaxSplit, std::max(1, fit));
}

size_t pflash_lds(int hs, int waves) { return (size_t)(16 * (hs + 4) + 32 * waves + 16 * waves * hs) * sizeof(float); }

// The forward passes of `rows` consecutive positions of one sequence (st: their tokens and the first position) as one batched
// step into the context's own KV cache: launch_batch_step's kernels, the attention as two launches (every position stores
// its k and v, then every position attends over the rows up to its own), and the classifier only when `last_logits`.
void launch_prefill_block(l2j_ctx *c, BatchBufs &b, const BatchState *st, int first_pos, int rows, bool last_logits)
{
    const l2j_config &cf = c->cfg;
    const int dim = cf.dim, hidden = cf.hidden_dim, L = cf.n_layers, hs = c->head_size, kvd = c->kv_dim, nseq = kMaxBatch;
    const int sd = batch_slices(dim), sh = batch_slices(hidden);
    hipStream_t s = c->stream;
    hipLaunchKernelGGL(k_bembed, dim3(nseq), dim3(256), 0, s, c->emb, st, b.x, dim, (unsigned *)nullptr);
    hipLaunchKernelGGL(k_brms, dim3(nseq), dim3(1024), 0, s, b.x, c->rmsw, b.xn, dim);
    for (int l = 0; l < L; l++) {
        launch_bgemm(c, {L2J_WQ, L2J_WK, L2J_WV}, l, b.xn, b.part, nseq);
        BAttn t{};
        t.pq = b.part[0]; t.pk = b.part[1]; t.pv = b.part[2]; t.slices = sd; t.rope = c->rope;
        t.kc = c->kcache + (size_t)l * cf.seq_len * kvd; t.vc = c->vcache + (size_t)l * cf.seq_len * kvd;   // (position, kv_dim) per layer
        t.seq_stride = 0; t.cap = cf.seq_len; t.out = b.xb; t.st = st;
        t.n_heads = cf.n_heads; t.kv_mul = cf.n_heads / cf.n_kv_heads; t.head_size = hs; t.kv_dim = kvd; t.dim = dim;
        t.sqrt_hs = sqrtf((float)hs);
        t.head_stride = hs; t.row_stride = kvd; t.nrows = rows; t.nseq = nseq;
        t.pf_part = b.pf_part; t.pf_cnt = b.pf_cnt;
        const dim3 ag(cf.n_heads, nseq), fg(cf.n_heads, 2, pflash_split(c, first_pos));
        // 16 positions at a time on the fp32 matrix cores from where that is the faster way: every cache row fetched once per 16
        // queries instead of once per query
        const bool flash = c->opt[OPT_PREFILL_FLASH] == 2 || (c->opt[OPT_PREFILL_FLASH] == 1 && first_pos >= kPflashFrom);
        if (hs == 64) {
            hipLaunchKernelGGL((k_battn<16, 1>), ag, dim3(256), 0, s, t);
            if (flash) hipLaunchKernelGGL((k_pflash<64, 16>), fg, dim3(1024), pflash_lds(64, 16), s, t);
            else hipLaunchKernelGGL((k_battn<16, 2>), ag, dim3(256), 0, s, t);
        } else if (hs == 128) {
            hipLaunchKernelGGL((k_battn<32, 1>), ag, dim3(256), 0, s, t);
            if (flash) hipLaunchKernelGGL((k_pflash<128, 16>), fg, dim3(1024), pflash_lds(128, 16), s, t);
            else hipLaunchKernelGGL((k_battn<32, 2>), ag, dim3(256), 0, s, t);
        } else {
            hipLaunchKernelGGL((k_battn<64, 1>), ag, dim3(256), 0, s, t);
            if (flash) hipLaunchKernelGGL((k_pflash<256, 8>), fg, dim3(512), pflash_lds(256, 8), s, t);
            else hipLaunchKernelGGL((k_battn<64, 2>), ag, dim3(256), 0, s, t);
        }
        launch_bgemm(c, {L2J_WO}, l, b.xb, b.part, nseq);
        hipLaunchKernelGGL(k_bres_rms, dim3(nseq), dim3(1024), 0, s, b.part[0], sd, b.x, c->rmsw + (size_t)(L + l) * dim, b.xn, dim);
        launch_bgemm(c, {L2J_W1, L2J_W3}, l, b.xn, b.part, nseq);
        hipLaunchKernelGGL(k_bepi_swiglu, dim3(hidden / 256, nseq), dim3(256), 0, s, b.part[0], b.part[1], sd, hidden, c->silu,
                           (cf.flags & L2J_F_EXACT_SILU) ? 1 : 0, b.hb);
        launch_bgemm(c, {L2J_W2}, l, b.hb, b.part, nseq);
        const float *wn = c->rmsw + (l + 1 < L ? (size_t)(l + 1) * dim : (size_t)2 * L * dim);
        hipLaunchKernelGGL(k_bres_rms, dim3(nseq), dim3(1024), 0, s, b.part[0], sh, b.x, wn, b.xn, dim);
    }
    if (last_logits) {
        BGemmF32 g{};
        g.w = c->wcls; g.rows = cf.vocab_size; g.K = dim; g.x = b.xn; g.part = b.part[0]; g.gps = kClsGps;
        const dim3 cg((cf.vocab_size + kBgRowsPerWG - 1) / kBgRowsPerWG, cls_slices(dim));
        hipLaunchKernelGGL(k_bgemm_f32<2>, cg, dim3(kBgThreads), batch_lds_f32(nseq), s, g);
        hipLaunchKernelGGL(k_brow, dim3(64), dim3(256), 0, s, b.part[0], c->logits, cf.vocab_size, cls_slices(dim), nseq, rows - 1);
    }
}

int hip_rc(hipError_t e, const char *what)
{
    return fail(e == hipErrorOutOfMemory ? L2J_E_OOM : L2J_E_HIP, std::string("batched decode: ") + what + ": " + hipGetErrorString(e));
}

// The context's buffers for n_seq sequences over `steps` positions with prompts of up to `pstride` ids: kept when they fit.
int ensure_batch(l2j_ctx *c, int nseq, int steps, int pstride)
{
    BatchBufs *old = c->batch;
    if (old && old->nseq == nseq && old->cap_steps >= steps && old->cap_pstride >= pstride && old->fuse_opt == c->opt[OPT_BATCH_FUSE]) return L2J_OK;
    if (old) {
        hipError_t se = hipStreamSynchronize(c->stream);
        if (se != hipSuccess) return hip_rc(se, "synchronize");
        old->release();
        delete old;
        c->batch = nullptr;
    }
    const l2j_config &cf = c->cfg;
    const int dim = cf.dim, hidden = cf.hidden_dim, L = cf.n_layers, kvd = c->kv_dim, vocab = cf.vocab_size;
    const int sd = batch_slices(dim), sh = batch_slices(hidden);
    const size_t part_floats = (size_t)nseq * std::max({(size_t)sd * hidden, (size_t)cls_slices(dim) * vocab, (size_t)sh * dim, (size_t)sd * dim});
    const size_t cache_floats = (size_t)nseq * L * steps * kvd;
    BatchBufs *b = new (std::nothrow) BatchBufs();
    if (!b) return fail(L2J_E_OOM, "batched decode: host allocation failed");
    b->nseq = nseq; b->cap_steps = steps; b->cap_pstride = pstride; b->fuse_opt = c->opt[OPT_BATCH_FUSE];
    hipError_t e = hipSuccess;
    auto alloc = [&](auto **p, size_t n) {
        if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(p), n * sizeof(**p));
    };
    alloc(&b->x, (size_t)nseq * dim); alloc(&b->xn, (size_t)nseq * std::max(dim, hidden));
    alloc(&b->xb, (size_t)nseq * dim); alloc(&b->hb, (size_t)nseq * hidden); alloc(&b->logits, (size_t)nseq * vocab);
    for (int i = 0; i < 3; i++) alloc(&b->part[i], part_floats);
    alloc(&b->kc, cache_floats); alloc(&b->vc, cache_floats);
    alloc(&b->st, 1); alloc(&b->prompts, (size_t)nseq * pstride); alloc(&b->out, (size_t)nseq * steps); alloc(&b->done, 1);
    alloc(&b->bar_ctr, (size_t)kBarStride); alloc(&b->fault, 1); alloc(&b->ssq, (size_t)2 * nseq * (dim / 256));
    if (e == hipSuccess) e = hipMemsetAsync(b->bar_ctr, 0, kBarStride * sizeof(unsigned), c->stream);
    if (e == hipSuccess) e = hipMemsetAsync(b->fault, 0, sizeof(int), c->stream);
    alloc(&b->step_args, 1);
    if (e == hipSuccess) e = plan_bstep(c, *b, nseq);
    if (e == hipSuccess && b->step_grid > 0) {
        const BStep a = bstep_args(c, *b, steps, nseq);
        e = hipMemcpy(b->step_args, &a, sizeof(a), hipMemcpyHostToDevice);
    }
    if (e == hipSuccess) e = hipEventCreate(&b->e0);
    if (e == hipSuccess) e = hipEventCreate(&b->e1);
    const size_t state_ints = sizeof(BatchState) / sizeof(int), prompt_ints = (size_t)nseq * pstride, out_ints = (size_t)nseq * steps;
    if (e == hipSuccess) e = hipHostMalloc(reinterpret_cast<void **>(&b->h_pin), std::max(state_ints + prompt_ints, out_ints) * sizeof(int), hipHostMallocDefault);
    if (e == hipSuccess) e = hipFuncSetAttribute((const void *)k_bgemm<1, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)batch_lds(kBatch));
    if (e == hipSuccess) e = hipFuncSetAttribute((const void *)k_bgemm<2, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)batch_lds(kMaxBatch));
    if (e == hipSuccess) e = hipFuncSetAttribute((const void *)k_bgemm_f32<1>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)batch_lds_f32(kBatch));
    if (e == hipSuccess) e = hipFuncSetAttribute((const void *)k_bgemm_f32<2>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)batch_lds_f32(kMaxBatch));
    // one position as a graph: every kernel reads the position and the tokens from device memory, so the same nodes serve
    // every step of every call ("graph" = 0: the kernels are launched one by one, for tools that do not follow graph launches)
    if (e == hipSuccess && c->opt[OPT_GRAPH] != 0) {
        e = hipStreamBeginCapture(c->stream, hipStreamCaptureModeThreadLocal);
        if (e == hipSuccess) {
            launch_batch_step(c, *b, steps, pstride, nseq);
            const hipError_t le = hipGetLastError();
            e = hipStreamEndCapture(c->stream, &b->graph);
            if (e == hipSuccess) e = le;
        }
        if (e == hipSuccess) e = hipGraphInstantiate(&b->exec, b->graph, nullptr, nullptr, 0);
    }
    if (e != hipSuccess) {
        b->release();
        delete b;
        return hip_rc(e, "set-up");
    }
    c->batch = b;
    return L2J_OK;
}

// The samplers of the sequences, as new Sampler(seeds[s], vocab_size) (J/Sampler.java:24-31) leaves them.
int seed_batch_samplers(l2j_ctx *c, BatchBufs &b, const int64_t *seeds)
{
    BatchSamplers &bs = b.samplers;
    if (!bs.ss) {
        const int rc = alloc_batch_samplers(c, b.nseq, &bs);
        if (rc) return rc;
    }
    SamplerState h[kMaxBatch] = {};
    for (int s = 0; s < b.nseq; s++) h[s].rng = ((unsigned long long)seeds[s] ^ kJavaRandMult) & kJavaRandMask;
    HIPCHK(hipMemcpyAsync(bs.ss, h, (size_t)b.nseq * sizeof(SamplerState), hipMemcpyHostToDevice, c->stream));
    for (int i = 0; i < 2; i++) {
        HIPCHK(hipMemsetAsync(bs.pi_prob[i], 0, (size_t)b.nseq * bs.pi_stride * sizeof(float), c->stream));
        HIPCHK(hipMemsetAsync(bs.pi_idx[i], 0, (size_t)b.nseq * bs.pi_stride * sizeof(int), c->stream));
    }
    HIPCHK(hipStreamSynchronize(c->stream));   // (h is pageable host memory)
    return L2J_OK;
}

// logits_log: null, or steps x n_seq x vocab_size floats of the caller that receive the logits of every step.
// seeds: null (every unforced token is the argmax), or the seed of every sequence's sampler: unforced tokens are sampled as
// l2j_sample does at this temperature (not 0) and topp.
int decode_batch(l2j_ctx *c, const int32_t *prompts, const int32_t *n_prompt, int32_t n_seq, int32_t prompt_stride, int32_t steps,
                 int32_t *out_tokens, double *seconds, float *logits_log, float temperature = 0.0f, float topp = 0.0f,
                 const int64_t *seeds = nullptr)
{
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
        std::lock_guard<std::mutex> lock(c->upload_mu);
        for (int t : {L2J_WQ, L2J_WK, L2J_WV, L2J_WO, L2J_W1, L2J_W2, L2J_W3}) {
            const int trc = ensure_batch_tiles(c, t);
            if (trc) return trc;
        }
        c->bt_ready = true;
    }
    int rc = ensure_batch(c, nseq, steps, std::max(1, (int)prompt_stride));
    if (rc) return rc;
    BatchBufs &b = *c->batch;
    const int vocab = cf.vocab_size, cap = b.cap_steps, pcap = b.cap_pstride;
    const size_t state_ints = sizeof(BatchState) / sizeof(int);
    unsigned cur = 0;   // bit s: the copy of its ProbIndex array that sequence s's last top-p step left
    if (seeds && (rc = seed_batch_samplers(c, b, seeds))) return rc;
    float *dlog = nullptr;
    if (logits_log) {
        hipError_t me = hipMalloc(reinterpret_cast<void **>(&dlog), (size_t)steps * nseq * vocab * sizeof(float));
        if (me != hipSuccess) return hip_rc(me, "logits of every step");
    }
    auto fail_hip = [&](hipError_t e, const char *what) {
        (void)hipStreamSynchronize(c->stream);
        (void)hipFree(dlog);
        return hip_rc(e, what);
    };
    BatchState h{};
    h.pos = 0;
    for (int i = 0; i < nseq; i++) { h.token[i] = 1; h.n_prompt[i] = n_prompt[i]; }   // BOS first (J/Run.java:612)
    memcpy(b.h_pin, &h, sizeof(h));
    memset(b.h_pin + state_ints, 0, (size_t)nseq * pcap * sizeof(int));
    for (int s = 0; s < nseq && prompt_stride > 0; s++)
        memcpy(b.h_pin + state_ints + (size_t)s * pcap, prompts + (size_t)s * prompt_stride, (size_t)n_prompt[s] * sizeof(int));
    hipError_t e = hipMemcpyAsync(b.st, b.h_pin, sizeof(h), hipMemcpyHostToDevice, c->stream);
    if (e == hipSuccess) e = hipMemcpyAsync(b.prompts, b.h_pin + state_ints, (size_t)nseq * pcap * sizeof(int), hipMemcpyHostToDevice, c->stream);
    if (e == hipSuccess) e = hipMemsetAsync(b.done, 0, sizeof(unsigned), c->stream);
    if (e != hipSuccess) return fail_hip(e, "state upload");
    for (int pos = 0; pos < steps && e == hipSuccess; pos++) {
        if (b.exec) {
            e = hipGraphLaunch(b.exec, c->stream);
        } else {
            launch_batch_step(c, b, cap, pcap, nseq);
            e = hipGetLastError();
        }
        if (dlog && e == hipSuccess)
            e = hipMemcpyAsync(dlog + (size_t)pos * nseq * vocab, b.logits, (size_t)nseq * vocab * sizeof(float), hipMemcpyDeviceToDevice, c->stream);
        // J/Run.java:643-665 for the sequences whose prompt is used up: the sampled token replaces the argmax k_bnext stored
        if (seeds && e == hipSuccess) {
            unsigned active = 0;
            for (int s = 0; s < nseq; s++) active |= pos >= n_prompt[s] ? 1u << s : 0u;
            if (active) {
                e = launch_samplers(c, b.samplers, active, cur, b.logits, temperature, topp, b.st->token, b.out + pos, cap);
                if ((double)topp <= 0.999) cur ^= active;   // (a top-p step leaves the array in its other copy)
            }
        }
        if (pos == 0 && e == hipSuccess) e = hipEventRecord(b.e0, c->stream);   // the clock starts after the first step (J/Run.java:682-684)
    }
    if (e == hipSuccess) e = hipEventRecord(b.e1, c->stream);
    if (e == hipSuccess) e = hipMemcpyAsync(b.h_pin, b.out, (size_t)nseq * cap * sizeof(int), hipMemcpyDeviceToHost, c->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(c->stream);
    if (e != hipSuccess) return fail_hip(e, "step");
    for (int s = 0; s < nseq; s++) memcpy(out_tokens + (size_t)s * steps, b.h_pin + (size_t)s * cap, (size_t)steps * sizeof(int));
    if (dlog) {
        e = hipMemcpy(logits_log, dlog, (size_t)steps * nseq * vocab * sizeof(float), hipMemcpyDeviceToHost);
        (void)hipFree(dlog);
        dlog = nullptr;
        if (e != hipSuccess) return hip_rc(e, "logits read-back");
    }
    if (seeds) {   // the reference's exceptions, as in l2j_sample
        SamplerState h[kMaxBatch] = {};
        if ((e = hipMemcpy(h, b.samplers.ss, (size_t)nseq * sizeof(SamplerState), hipMemcpyDeviceToHost)) != hipSuccess) return hip_rc(e, "sampler flags");
        int st = 0;
        for (int s = 0; s < nseq; s++) st |= h[s].nan;
        if (st & 1) return fail(L2J_E_ARG, "sampler: NaN among the logits (J/Sampler.java:88-90)");
        if (st & 2) return fail(L2J_E_ARG, "sampler: no probability reaches the top-p cutoff (ArrayIndexOutOfBoundsException at J/Sampler.java:119)");
    }
    if (b.step_grid > 0) {
        int fault = 0;
        if ((e = hipMemcpy(&fault, b.fault, sizeof(int), hipMemcpyDeviceToHost)) != hipSuccess) return hip_rc(e, "fault flag");
        if (fault) {
            (void)hipMemset(b.fault, 0, sizeof(int));
            return fail(L2J_E_HIP, "batched decode: a bounded wait at a grid barrier ran out (is another process using the GPU?); "
                                   "option batch_fuse = 0 runs the same step without grid barriers");
        }
    }
    float ms = 0.0f;
    if (steps > 1 && (e = hipEventElapsedTime(&ms, b.e0, b.e1)) != hipSuccess) return hip_rc(e, "timing");
    if (seconds) *seconds = (double)ms * 1e-3;
    return L2J_OK;
}

}  // namespace

int l2j::prefill_positions(l2j_ctx *c, const int32_t *tokens, int32_t n, int32_t pos0, float *logits, double *seconds)
{
    if (!c || !tokens) return fail(L2J_E_ARG, "null argument");
    if (!c->finalized) return fail(L2J_E_STATE, "prefill before l2j_finalize");
    const l2j_config &cf = c->cfg;
    const int hs = c->head_size;
    if (cf.dim % 256 || cf.hidden_dim % 256 || c->kv_dim % 16 || cf.vocab_size % 16 || (hs != 64 && hs != 128 && hs != 256))
        return fail(L2J_E_SIZE, "prefill needs dim and hidden_dim in whole groups of 256, kv_dim and vocab_size multiples of 16, "
                                "head_size 64, 128 or 256 (as the batched decode); take l2j_forward position by position");
    if (n <= 0 || pos0 < 0 || (long)pos0 + n > cf.seq_len) return fail(L2J_E_ARG, "positions pos0 .. pos0 + n - 1 must lie in 0 .. seq_len - 1");
    for (int i = 0; i < n; i++)
        if (tokens[i] < 0 || tokens[i] >= cf.vocab_size) return fail(L2J_E_ARG, "token id out of range");
    HIPCHK(hipSetDevice(cf.device));
    if (!c->bt_ready) {   // the matrices once more, in the order the batched products read them
        std::lock_guard<std::mutex> lock(c->upload_mu);
        for (int t : {L2J_WQ, L2J_WK, L2J_WV, L2J_WO, L2J_W1, L2J_W2, L2J_W3}) {
            const int trc = ensure_batch_tiles(c, t);
            if (trc) return trc;
        }
        c->bt_ready = true;
    }
    int rc = c->batch && c->batch->nseq == kMaxBatch ? L2J_OK : ensure_batch(c, kMaxBatch, 1, 1);
    if (rc) return rc;
    BatchBufs &b = *c->batch;
    if (!c->pflash_ready) {   // (more than the default 64 KB of dynamic LDS)
        HIPCHK(hipFuncSetAttribute(reinterpret_cast<const void *>(k_pflash<64, 16>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)pflash_lds(64, 16)));
        HIPCHK(hipFuncSetAttribute(reinterpret_cast<const void *>(k_pflash<128, 16>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)pflash_lds(128, 16)));
        HIPCHK(hipFuncSetAttribute(reinterpret_cast<const void *>(k_pflash<256, 8>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)pflash_lds(256, 8)));
        c->pflash_ready = true;
    }
    if (!b.pf_cnt) {   // (the counters last: their presence says that both are there and cleared)
        if (!b.pf_part && (rc = dev_alloc(&b.pf_part, (uint64_t)cf.n_heads * 2 * kPflashMaxSplit * (32 + 16 * hs)))) return rc;
        unsigned *cnt = nullptr;
        if ((rc = dev_alloc(&cnt, (uint64_t)cf.n_heads * 2))) return rc;
        if (hipMemset(cnt, 0, (size_t)cf.n_heads * 2 * sizeof(unsigned)) != hipSuccess) {
            (void)hipFree(cnt);
            return fail(L2J_E_HIP, "prefill: clearing the counters of the attention's workgroups");
        }
        b.pf_cnt = cnt;
    }
    const int nblocks = (n + kMaxBatch - 1) / kMaxBatch;
    std::vector<BatchState> hst((size_t)nblocks);
    for (int k = 0; k < nblocks; k++) {
        hst[k] = BatchState{};
        hst[k].pos = pos0 + k * kMaxBatch;
        for (int r = 0; r < kMaxBatch; r++) hst[k].token[r] = tokens[std::min(k * kMaxBatch + r, n - 1)];   // (rows past the end: not stored, not read)
    }
    BatchState *dst = nullptr;
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&dst), (size_t)nblocks * sizeof(BatchState));
    if (e != hipSuccess) return hip_rc(e, "prefill: positions");
    e = hipMemcpyAsync(dst, hst.data(), (size_t)nblocks * sizeof(BatchState), hipMemcpyHostToDevice, c->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(c->stream);   // (hst is pageable host memory)
    if (e == hipSuccess) e = hipEventRecord(b.e0, c->stream);
    for (int k = 0; k < nblocks && e == hipSuccess; k++) {
        launch_prefill_block(c, b, dst + k, pos0 + k * kMaxBatch, std::min(kMaxBatch, n - k * kMaxBatch), k + 1 == nblocks);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipEventRecord(b.e1, c->stream);
    if (e == hipSuccess && logits) e = hipMemcpyAsync(logits, c->logits, (size_t)cf.vocab_size * sizeof(float), hipMemcpyDeviceToHost, c->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(c->stream);
    (void)hipFree(dst);
    if (e != hipSuccess) return hip_rc(e, "prefill");
    float ms = 0.0f;
    if ((e = hipEventElapsedTime(&ms, b.e0, b.e1)) != hipSuccess) return hip_rc(e, "prefill: timing");
    if (seconds) *seconds = (double)ms * 1e-3;
    return L2J_OK;
}

extern "C" {

int l2j_prefill(l2j_ctx *c, const int32_t *tokens, int32_t n, int32_t pos0, float *logits, double *seconds)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        return prefill_positions(c, tokens, n, pos0, logits, seconds);
    }());
}

int l2j_release_batch(l2j_ctx *c)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        if (!c) return fail(L2J_E_ARG, "null context");
        HIPCHK(hipSetDevice(c->cfg.device));
        HIPCHK(hipStreamSynchronize(c->stream));
        std::lock_guard<std::mutex> lock(c->upload_mu);
        free_batch(c);
        return L2J_OK;
    }());
}

int l2j_decode_greedy_batch(l2j_ctx *c, const int32_t *prompts, const int32_t *n_prompt, int32_t n_seq, int32_t prompt_stride,
                            int32_t steps, int32_t *out_tokens, double *seconds)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        return decode_batch(c, prompts, n_prompt, n_seq, prompt_stride, steps, out_tokens, seconds, nullptr);
    }());
}

int l2j_decode_sample_batch(l2j_ctx *c, const int32_t *prompts, const int32_t *n_prompt, int32_t n_seq, int32_t prompt_stride,
                            int32_t steps, float temperature, float topp, const int64_t *rng_seeds, int32_t *out_tokens, double *seconds,
                            float *logits)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        const int rc = check_sampler_args(temperature, topp);
        if (rc) return rc;
        if (temperature != 0.0f && !rng_seeds) return fail(L2J_E_ARG, "null argument");
        return decode_batch(c, prompts, n_prompt, n_seq, prompt_stride, steps, out_tokens, seconds, logits, temperature, topp,
                            temperature != 0.0f ? rng_seeds : nullptr);   // (temperature 0: Sampler.argmax, J/Run.java:644-646)
    }());
}

int l2j_decode_greedy_batch_logits(l2j_ctx *c, const int32_t *prompts, const int32_t *n_prompt, int32_t n_seq, int32_t prompt_stride,
                                   int32_t steps, int32_t *out_tokens, float *logits)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        if (!logits) return fail(L2J_E_ARG, "null argument");
        return decode_batch(c, prompts, n_prompt, n_seq, prompt_stride, steps, out_tokens, nullptr, logits);
    }());
}

}  // extern "C"
