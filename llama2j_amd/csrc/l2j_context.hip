// libllama2j_hip.so: contexts, options and the load path of the C ABI declared in include/llama2j_hip.h.
// Owns device memory and converts the reference's weight formats to the streaming layout.
#include "l2j_internal.hpp"

using namespace l2j;

namespace {

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

// A slice of the caller's host memory in a device buffer of the call's own, copied on a stream of the call's own and
// without the context's lock: the copies of calls on different threads (the loader's, or a JVM's ten virtual threads)
// run side by side, and only the kernel that takes the slice apart runs under the lock.
struct Staged {
    void *dev = nullptr;
    size_t cap = 0;
    hipStream_t s = nullptr;
    ~Staged()
    {
        if (dev) (void)hipFree(dev);
        if (s) (void)hipStreamDestroy(s);
    }
    int in(const void *host, size_t bytes, size_t cap_bytes)
    {
        if (!s) HIPCHK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
        if (!dev) {
            HIPCHK(hipMalloc(&dev, std::max<size_t>(cap_bytes, 1)));
            cap = cap_bytes;
        }
        HIPCHK(hipMemcpyAsync(dev, host, bytes, hipMemcpyHostToDevice, s));
        HIPCHK(hipStreamSynchronize(s));
        return L2J_OK;
    }
};

constexpr uint64_t kStageBytes = 1ull << 30;   // at most this much of a tensor at a time

// `ngroups` groups of reference bytes, already in device memory, into the tensor's arrays from group0 on (under the lock)
int unpack_staged(l2j_ctx *c, QTensor &t, uint64_t group0, const uint8_t *stage, uint64_t ngroups)
{
    const int grid = (int)std::min<uint64_t>(ngroups, 1u << 20);
    hipLaunchKernelGGL(k_unpack_groups, dim3(grid), dim3(64), 0, c->stream, stage, (long)ngroups, t.codes + group0 * kGroup, t.gs + group0,
                       t.mm + group0);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) e = hipStreamSynchronize(c->stream);
    if (e != hipSuccess) return fail(L2J_E_HIP, std::string("upload: ") + hipGetErrorString(e));
    return L2J_OK;
}

}  // namespace

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
    release_forward(c);
    (void)hipFree(c->rmsw);
    c->rmsw = nullptr;
}

void l2j_destroy(l2j_ctx *c)
{
    if (!c) return;
    // Order: nothing of the context may still run, then the graph (its nodes name kernels and buffers of the
    // context), the events, the buffers, and the stream last.
    std::lock_guard<std::mutex> forward_lock(g_forward_mu);
    (void)hipSetDevice(c->cfg.device);
    if (c->stream) (void)hipStreamSynchronize(c->stream);
    free_batch(c);
    release_finalize(c);
    for (hipEvent_t ev : c->events) (void)hipEventDestroy(ev);
    for (int t = 0; t < L2J_TENSOR_COUNT; t++) {
        (void)hipFree(c->qt[t].codes);
        (void)hipFree(c->qt[t].gs);
        (void)hipFree(c->qt[t].mm);
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
        if (strcmp(name, "wall_clock_khz") == 0) {  // read-only: the clock l2j_decode_greedy times itself with (0: unknown)
            *value = (int32_t)(c->wall_clock_hz / 1e3);
            return L2J_OK;
        }
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
    QTensor &t = c->qt[tensor];
    std::lock_guard<std::mutex> tensor_lock(t.mu);
    HIPCHK(hipSetDevice(c->cfg.device));
    const uint64_t slice_groups = kStageBytes / kGroupBytes;
    Staged st;
    bool first = true;
    for (uint64_t g = 0; g < ngroups || first; g += slice_groups) {
        const uint64_t ng = std::min(slice_groups, ngroups - g);
        if (ng) {
            const int rc = st.in(bytes + g * kGroupBytes, ng * kGroupBytes, std::min(ngroups, slice_groups) * kGroupBytes);
            if (rc) return rc;
        }
        std::lock_guard<std::mutex> lock(c->upload_mu);
        if (c->finalized) return fail(L2J_E_STATE, "upload after l2j_finalize");
        if (first) {
            if (whole) t.groups_loaded = 0;
            invalidate_batch_tiles(c, tensor);
            first = false;
        }
        if (ng) {
            const int rc = unpack_staged(c, t, group0 + g, static_cast<const uint8_t *>(st.dev), ng);
            if (rc) return rc;
            t.groups_loaded += ng;
        }
    }
    return L2J_OK;
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
        std::lock_guard<std::mutex> tensor_lock(t.mu);
        HIPCHK(hipSetDevice(c->cfg.device));
        const uint64_t slice = kStageBytes / sizeof(float);   // floats per staging slice
        Staged st;
        bool first_slice = true;
        for (uint64_t o = 0; o < nfloats || first_slice; o += slice) {
            const uint64_t nf = std::min(slice, nfloats - o);
            const uint64_t ng = (nf + kGroup - 1) / kGroup;
            if (nf) {   // (the copy: without the context's lock)
                const int rc = st.in(data + o, nf * sizeof(float), std::min(slice, nfloats) * sizeof(float));
                if (rc) return rc;
            }
            std::lock_guard<std::mutex> lock(c->upload_mu);
            if (c->finalized) return fail(L2J_E_STATE, "upload after l2j_finalize");
            if (first_slice) {
                invalidate_batch_tiles(c, tensor);
                first_slice = false;
            }
            if (nf) {
                hipLaunchKernelGGL(k_encode_groups, dim3((unsigned)std::min<uint64_t>(ng, 1u << 20)), dim3(256), 0, c->stream,
                                   static_cast<const float *>(st.dev), (long)nf, (long)((first + o) / kGroup), (long)ng, (long)t.nfloats, 0ull,
                                   0.0f, t.codes, t.gs, t.mm);
                hipError_t e = hipGetLastError();
                if (e == hipSuccess) e = hipStreamSynchronize(c->stream);
                if (e != hipSuccess) return fail(L2J_E_HIP, std::string("quantize: ") + hipGetErrorString(e));
                t.groups_loaded += ng;
            }
        }
        return L2J_OK;
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
            invalidate_batch_tiles(c, t);
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
        // launch shapes, scratch of the phases, graphs (l2j_forward.hip)
        const int rcf = setup_forward(c);
        if (rcf) return rcf;
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

}  // extern "C"
