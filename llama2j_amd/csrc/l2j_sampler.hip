// libllama2j_hip.so: host side of the device sampler (J/Sampler.java, J/Run.java:643-665) and the running sums.
#include "l2j_internal.hpp"
#include "sampler_kernels.hpp"
#include "sampler_wide.hpp"

using namespace l2j;

// Device memory of l2j_running_sums_noalloc: the terms and their sums of one call.  Every GPU the library runs on holds
// its own copy of the array until the process ends; in host code the name is only a handle for hipGetSymbolAddress.
static __device__ __align__(256) float scratch[kSampleMaxVocab];

namespace {

// The address of `scratch` on each device, looked up by the first l2j_create on that device (with the device current).
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
float *g_scratch_ptr[kMaxDevices] = {};

}  // namespace

int l2j::resolve_scratch(int device)
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

namespace {

// ---- device sampler ------------------------------------------------------------------------------------

}  // namespace

void l2j::free_sampler(l2j_ctx *c)
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
    (void)hipFree(c->wide_mem);
    c->wide_mem = nullptr;
    if (c->h_ss) (void)hipHostFree(c->h_ss);
    c->h_ss = nullptr;
}

namespace {

// dynamic LDS of the sampler's one-workgroup kernels: the terms, padded to whole steps of the single-lane sum plus one
size_t sampler_lds_bytes(int n)
{
    return n <= kSampleMaxVocab ? (size_t)(((n + kChainStep - 1) & ~(kChainStep - 1)) + kChainStep) * sizeof(float) : 0;
}

// k_sample_wide's device memory, carved out of one allocation (WideWs says what is what)
constexpr size_t kWideSync = 0, kWideSsum = (sizeof(WideSync) + 63) / 64 * 64, kWideSeg = kWideSsum + 8 * kWideMaxSlices,
                 kWideCmask = kWideSeg + 16 * kWideMaxSlices, kWideT = kWideCmask + 32 * kWideMaxSlices, kWideD = kWideT + 3 * 8 * kWideMaxSlices, kWideBytes = kWideD + 3 * 8 * 64 * kWideMaxSlices;

WideWs wide_ws(l2j_ctx *c)
{
    unsigned char *m = c->wide_mem;
    WideWs w{};
    w.sync = reinterpret_cast<WideSync *>(m + kWideSync);
    w.ssum = reinterpret_cast<double *>(m + kWideSsum);
    w.seg = reinterpret_cast<unsigned long long *>(m + kWideSeg);
    w.cmask = reinterpret_cast<unsigned long long *>(m + kWideCmask);
    int *t = reinterpret_cast<int *>(m + kWideT);
    w.t_x0 = t; w.t_x1 = t + 2 * kWideMaxSlices; w.t_m = t + 4 * kWideMaxSlices;
    int *d = reinterpret_cast<int *>(m + kWideD);
    w.d_x0 = d; w.d_x1 = d + 2 * 64 * kWideMaxSlices; w.d_m = d + 4 * 64 * kWideMaxSlices;
    w.maxspin = std::max(0, c->opt[OPT_BARRIER_SPINS]);
    return w;
}

size_t wide_lds_bytes(int n)
{
    const size_t keys = (size_t)((n + kSortRun - 1) / kSortRun * kSortRun) * sizeof(float);
    return std::max(keys, sizeof(WideWalk));
}

int alloc_sampler(l2j_ctx *c)
{
    const int n = c->cfg.vocab_size;
    const int npad = (n + kSortRun - 1) / kSortRun * kSortRun;
    int rc;
    for (int i = 0; i < 2; i++) {
        if ((rc = dev_alloc(&c->pi_prob[i], (uint64_t)n + 4))) return rc;   // (read in 16-byte words: stage_terms)
        if ((rc = dev_alloc(&c->pi_idx[i], (uint64_t)n))) return rc;
    }
    if ((rc = dev_alloc(&c->sample_exp, (uint64_t)npad + 4))) return rc;   // (k_sample_wide stores whole slices of 256)
    HIPCHK(hipHostMalloc((void **)&c->h_ss, sizeof(SamplerState), hipHostMallocDefault));
    if (n <= kSampleMaxVocab) {
        if ((rc = dev_alloc(&c->wide_mem, kWideBytes))) return rc;
        HIPCHK(hipMemset(c->wide_mem, 0, kWideBytes));
        HIPCHK(hipFuncSetAttribute((const void *)k_sample_wide, hipFuncAttributeMaxDynamicSharedMemorySize, (int)wide_lds_bytes(n)));
        HIPCHK(hipFuncSetAttribute((const void *)k_sum_probe, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(WideWalk)));
    }
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

}  // namespace

// new Sampler(rngSeed, vocab_size) (J/Sampler.java:24-31): Random(seed) scrambles its seed, every ProbIndex is (0, 0)
int l2j::seed_sampler(l2j_ctx *c, int64_t rng_seed)
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

namespace {

}  // namespace

// ---- a sampler per sequence of the batched decode: the launch-per-stage step with the sequence as grid z ----

void l2j::free_batch_samplers(BatchSamplers *bs)
{
    void *ps[] = {bs->ss, bs->pi_prob[0], bs->pi_prob[1], bs->pi_idx[0], bs->pi_idx[1], bs->sort_k[0], bs->sort_k[1], bs->sort_v[0],
                  bs->sort_v[1]};
    for (void *p : ps) (void)hipFree(p);
    *bs = BatchSamplers{};
}

int l2j::alloc_batch_samplers(l2j_ctx *c, int nseq, BatchSamplers *bs)
{
    const size_t n = (size_t)c->cfg.vocab_size;
    if (n > (size_t)kSampleMaxVocab || c->opt[OPT_SAMPLER_SCAN] == 0)
        return fail(L2J_E_STATE, "sampling for several sequences keeps a step's probabilities in LDS: vocab_size up to 36864 and the "
                                 "option sampler_scan left on");
    const size_t npad = (n + kSortRun - 1) / kSortRun * kSortRun;
    bs->nseq = nseq;
    bs->pi_stride = (n + 4 + 3) / 4 * 4;   // (rows 16-byte aligned, read in 16-byte words)
    bs->sort_stride = npad;
    int rc = dev_alloc(&bs->ss, (uint64_t)nseq);
    for (int i = 0; i < 2 && !rc; i++) {
        if (!rc) rc = dev_alloc(&bs->pi_prob[i], (uint64_t)nseq * bs->pi_stride);
        if (!rc) rc = dev_alloc(&bs->pi_idx[i], (uint64_t)nseq * bs->pi_stride);
        if (!rc) rc = dev_alloc(&bs->sort_k[i], (uint64_t)nseq * bs->sort_stride);
        if (!rc) rc = dev_alloc(&bs->sort_v[i], (uint64_t)nseq * bs->sort_stride);
    }
    if (!rc) {   // (more than the default 64 KB of dynamic LDS)
        const int lds = (int)sampler_lds_bytes((int)n);
        if (hipFuncSetAttribute((const void *)k_sample_probs<true>, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess ||
            hipFuncSetAttribute((const void *)k_topp_pick<true>, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
            rc = fail(L2J_E_HIP, "sampler: dynamic LDS of a step");
    }
    if (rc) free_batch_samplers(bs);
    return rc;
}

hipError_t l2j::launch_samplers(l2j_ctx *c, const BatchSamplers &bs, unsigned active, unsigned cur, float *logits, float temperature,
                                float topp, int *token, int *out, long out_stride)
{
    const int n = c->cfg.vocab_size, nseq = bs.nseq;
    const int npad = (n + kSortRun - 1) / kSortRun * kSortRun;
    SampleArgs a{};
    a.logits = logits; a.n = n;
    a.temperature = temperature; a.topp = topp; a.coin = -1.0f;
    a.plain = (double)topp > 0.999;
    a.ss = bs.ss;
    a.scan = 1;
    a.nseq = nseq; a.active = active; a.cur = cur;
    a.pi_prob0 = bs.pi_prob[0]; a.pi_prob1 = bs.pi_prob[1]; a.pi_idx0 = bs.pi_idx[0]; a.pi_idx1 = bs.pi_idx[1];
    a.logits_stride = n; a.pi_stride = (long)bs.pi_stride;
    a.btoken = token; a.bout = out; a.bout_stride = out_stride;
    // (no k_sample_exp: with the sequences' workgroups side by side the exponentials cost less inside k_sample_probs than
    // a launch of their own, in which every workgroup reads all of its sequence's logits for the maximum: 81 us measured)
    const size_t lds = sampler_lds_bytes(n);
    hipLaunchKernelGGL(k_sample_probs<true>, dim3(1, 1, nseq), dim3(1024), lds, c->stream, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || a.plain) return e;
    SortBatch sb{};
    sb.active = active; sb.cur = cur;
    sb.pi_prob0 = bs.pi_prob[0]; sb.pi_prob1 = bs.pi_prob[1]; sb.pi_idx0 = bs.pi_idx[0]; sb.pi_idx1 = bs.pi_idx[1];
    sb.tiles_k = bs.sort_k[0]; sb.tiles_v = bs.sort_v[0]; sb.runs_k = bs.sort_k[1]; sb.runs_v = bs.sort_v[1];
    sb.pi_stride = (long)bs.pi_stride; sb.sort_stride = (long)bs.sort_stride;
    hipLaunchKernelGGL(k_sort_tiles_b, dim3(npad / kSortTile, 1, nseq), dim3(kSortTile), 0, c->stream, sb, n);
    hipLaunchKernelGGL(k_merge_tiles_b, dim3(npad / kSortRun, 16, nseq), dim3(256), 0, c->stream, sb);
    hipLaunchKernelGGL(k_merge_far_b, dim3(npad / 256, 1, nseq), dim3(256), 0, c->stream, sb, npad, n);
    hipLaunchKernelGGL(k_topp_pick<true>, dim3(1, 1, nseq), dim3(1024), lds, c->stream, a);
    return hipGetLastError();
}

// The sampling step of J/Run.java:643-665 on c->logits; in_loop: the token replaces what k_finish stored.
hipError_t l2j::launch_sampler(l2j_ctx *c, float temperature, float topp, float coin, bool in_loop)
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
    if (in_lds && c->opt[OPT_SAMPLER_WIDE] != 0 && a.scan) {
        WideArgs wa{};
        wa.logits = c->logits; wa.n = n;
        wa.temperature = temperature; wa.topp = topp; wa.coin = coin;
        wa.plain = a.plain;
        wa.ss = c->ss;
        wa.old_prob = c->pi_prob[cur]; wa.old_idx = c->pi_idx[cur];
        wa.new_prob = c->pi_prob[other]; wa.new_idx = c->pi_idx[other];
        wa.k0 = c->sort_k[0]; wa.v0 = c->sort_v[0]; wa.k1 = c->sort_k[1]; wa.v1 = c->sort_v[1];
        wa.expbuf = c->sample_exp;
        wa.st = a.st; wa.out_tokens = a.out_tokens;
        wa.w = wide_ws(c);
        hipLaunchKernelGGL(k_sample_wide, dim3((n + kWideSlice - 1) / kWideSlice), dim3(kWideSlice), wide_lds_bytes(n), c->stream, wa);
        if (!a.plain) c->pi_cur = other;   // the array stays there until the next call
        return hipGetLastError();
    }
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

namespace {

}  // namespace

// After a synchronize with h_ss read back: the reference's exceptions as an error return; the flag is cleared.
int l2j::check_sampler_status(l2j_ctx *c)
{
    const int st = c->h_ss->nan;
    if (!st) return L2J_OK;
    c->h_ss->nan = 0;
    HIPCHK(hipMemcpy(&c->ss->nan, &c->h_ss->nan, sizeof(int), hipMemcpyHostToDevice));
    if (st & 4) {   // (the counters of the launch are not where the next one expects them)
        if (c->wide_mem) HIPCHK(hipMemset(c->wide_mem, 0, sizeof(WideSync)));
        c->opt[OPT_SAMPLER_WIDE] = 0;   // (something else holds compute units: from here on one launch per stage, which waits for nobody)
        return fail(L2J_E_HIP, "sampler: a workgroup waited too long for the others (k_sample_wide needs a compute unit per 256 "
                               "probabilities); the step was not completed, the context takes one launch per stage from now on: "
                               "seed the sampler again (l2j_sampler_seed, or a new l2j_decode_sample)");
    }
    if (st & 1) return fail(L2J_E_ARG, "sampler: NaN among the logits (J/Sampler.java:88-90)");
    return fail(L2J_E_ARG, "sampler: no probability reaches the top-p cutoff (ArrayIndexOutOfBoundsException at J/Sampler.java:119)");
}

namespace {

}  // namespace

int l2j::check_sampler_args(float temperature, float topp)
{
    if (!(temperature >= 0.0f) || !(topp >= 0.0f && topp <= 1.0f)) return fail(L2J_E_ARG, "temperature must be >= 0 and topp in [0, 1]");
    return L2J_OK;
}

namespace {


}  // namespace

extern "C" {

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

int l2j_sum_probe(l2j_ctx *c, const float *terms, int32_t n, const float *limits, int32_t n_limits, int32_t *index_out, float *sum_out,
                  float *total_out)
{
    return ctx_rc(c, [&]() -> int {
        std::lock_guard<std::mutex> forward_lock(g_forward_mu);
        if (!c || !terms || !total_out || (n_limits > 0 && (!limits || !index_out || !sum_out))) return fail(L2J_E_ARG, "null argument");
        if (n <= 0 || n > kSampleMaxVocab) return fail(L2J_E_SIZE, "l2j_sum_probe: 1 to 36864 terms");
        if (n_limits < 0 || n_limits > 4096) return fail(L2J_E_SIZE, "l2j_sum_probe: 0 to 4096 limits");
        HIPCHK(hipSetDevice(c->cfg.device));
        int rc;
        if (!c->ss && (rc = seed_sampler(c, 0))) return rc;
        if (!c->wide_mem) return fail(L2J_E_STATE, "l2j_sum_probe: the context's vocabulary does not fit the one-launch sampler");
        const int slices = (n + kWideSlice - 1) / kWideSlice;
        // terms padded to whole slices | limits | sums at the hits | the total | the hits
        const size_t nt = (size_t)slices * kWideSlice, nl = (size_t)std::max(n_limits, 1);
        float *d = nullptr;
        HIPCHK(hipMalloc(reinterpret_cast<void **>(&d), (nt + 2 * nl + 1) * sizeof(float) + nl * sizeof(int)));
        float *d_lim = d + nt, *d_sum = d_lim + nl, *d_total = d_sum + nl;
        int *d_idx = reinterpret_cast<int *>(d_total + 1);
        hipError_t e = hipMemsetAsync(d, 0, nt * sizeof(float), c->stream);
        if (e == hipSuccess) e = hipMemcpyAsync(d, terms, (size_t)n * sizeof(float), hipMemcpyHostToDevice, c->stream);
        if (e == hipSuccess && n_limits > 0) e = hipMemcpyAsync(d_lim, limits, (size_t)n_limits * sizeof(float), hipMemcpyHostToDevice, c->stream);
        if (e == hipSuccess) {
            hipLaunchKernelGGL(k_sum_probe, dim3(slices), dim3(kWideSlice), sizeof(WideWalk), c->stream, d, n, d_lim, n_limits, d_idx, d_sum,
                               d_total, c->ss, wide_ws(c));
            e = hipGetLastError();
        }
        if (e == hipSuccess && n_limits > 0) e = hipMemcpyAsync(index_out, d_idx, (size_t)n_limits * sizeof(int), hipMemcpyDeviceToHost, c->stream);
        if (e == hipSuccess && n_limits > 0) e = hipMemcpyAsync(sum_out, d_sum, (size_t)n_limits * sizeof(float), hipMemcpyDeviceToHost, c->stream);
        if (e == hipSuccess) e = hipMemcpyAsync(total_out, d_total, sizeof(float), hipMemcpyDeviceToHost, c->stream);
        if (e == hipSuccess) e = hipMemcpyAsync(c->h_ss, c->ss, sizeof(SamplerState), hipMemcpyDeviceToHost, c->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(c->stream);
        (void)hipFree(d);
        if (e != hipSuccess) return fail(L2J_E_HIP, std::string("sum probe: ") + hipGetErrorString(e));
        return check_sampler_status(c);
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


}  // extern "C"
