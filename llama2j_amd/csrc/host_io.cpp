// Host side of the load path: the group-int8 codec, the .quant cache files and the llama2.c v0
// checkpoint reader that feeds the device uploads.  No GPU code here.
//
// Reference: J/Quant.java (codec), J/BinFileReader.java + J/BinFileWriter.java (files),
// J/TransformerWeights.java:43-144,191-356 (load order, cache naming, size check),
// J/Run.java:561-573 (header).  J/ = src/main/java/com/lastbot/llama2j/.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "../../include/llama2j_hip.h"
#include "host_internal.h"

namespace {

constexpr uint64_t kGroup = 256, kGroupBytes = 264;

int fail(int code, const std::string &msg)
{
    l2j_set_error_(msg.c_str());
    return code;
}

inline void store_be(uint8_t *dst, float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    u = __builtin_bswap32(u);
    memcpy(dst, &u, 4);
}

inline float load_be(const uint8_t *src)
{
    uint32_t u;
    memcpy(&u, src, 4);
    u = __builtin_bswap32(u);
    float f;
    memcpy(&f, &u, 4);
    return f;
}

// One group: min/max scan from element 0, header, then round-half-up codes.
void encode_group(const float *in, uint64_t count, uint8_t *out)
{
    float lo = in[0], hi = in[0];
    for (uint64_t j = 1; j < count; j++) {
        const float v = in[j];
        if (v < lo) lo = v;
        if (v > hi) hi = v;
    }
    const float range = hi - lo;
    store_be(out, lo);
    store_be(out + 4, hi);
    uint8_t *codes = out + 8;
    for (uint64_t j = 0; j < count; j++) {
        const float s = (in[j] - lo) / range * 255.0f;
        int code = 0;
        if (s == s) {  // NaN (constant group) encodes as 0, like Math.round
            const float fl = std::floor(s);
            code = (int)fl + ((s - fl) >= 0.5f ? 1 : 0);  // floor(s + 1/2) without rounding the sum
        }
        codes[j] = (uint8_t)code;
    }
    for (uint64_t j = count; j < kGroup; j++) codes[j] = 0;  // filler
}

template <typename F>
void parallel_groups(uint64_t ngroups, F &&body)
{
    unsigned nt = std::max(1u, std::min(std::thread::hardware_concurrency(), 16u));
    if (ngroups < 4096) nt = 1;
    if (nt == 1) {
        body(0, ngroups);
        return;
    }
    std::vector<std::thread> th;
    const uint64_t per = (ngroups + nt - 1) / nt;
    for (unsigned t = 0; t < nt; t++) {
        const uint64_t a = t * per, b = std::min(ngroups, a + per);
        if (a < b) th.emplace_back([=, &body] { body(a, b); });
    }
    for (auto &x : th) x.join();
}

struct Mapped {
    const uint8_t *p = nullptr;
    size_t len = 0;
    int fd = -1;
    ~Mapped()
    {
        if (p) munmap(const_cast<uint8_t *>(p), len);
        if (fd >= 0) close(fd);
    }
};

int map_file(const char *path, Mapped &m)
{
    m.fd = open(path, O_RDONLY);
    if (m.fd < 0) return fail(L2J_E_IO, std::string("cannot open ") + path);
    struct stat st;
    if (fstat(m.fd, &st) != 0) return fail(L2J_E_IO, std::string("cannot stat ") + path);
    m.len = (size_t)st.st_size;
    void *p = mmap(nullptr, m.len, PROT_READ, MAP_PRIVATE, m.fd, 0);
    if (p == MAP_FAILED) return fail(L2J_E_IO, std::string("cannot map ") + path);
    m.p = static_cast<const uint8_t *>(p);
    return L2J_OK;
}

const char *const kStems[L2J_TENSOR_COUNT] = {"", "l_rms_att_weight", "l_wq", "l_wk", "l_wv", "l_wo", "l_rms_ffn_weight",
                                              "l_w1", "l_w2", "l_w3", "rms_final_weight", ""};

uint64_t quant_floats(const l2j_config &c, int t)
{
    const uint64_t L = c.n_layers, dim = c.dim, hid = c.hidden_dim, hs = c.dim / c.n_heads;
    switch (t) {
    case L2J_RMS_ATT: case L2J_RMS_FFN: return L * dim;
    case L2J_WQ: return L * dim * (c.n_heads * hs);
    case L2J_WK: case L2J_WV: return L * dim * (c.n_kv_heads * hs);
    case L2J_WO: return L * (c.n_heads * hs) * dim;
    case L2J_W1: case L2J_W2: case L2J_W3: return L * dim * hid;
    case L2J_RMS_FINAL: return dim;
    default: return 0;
    }
}

}  // namespace

namespace l2j_host {
const char *tensor_stem(int tensor) { return tensor >= 0 && tensor < L2J_TENSOR_COUNT ? kStems[tensor] : ""; }
}  // namespace l2j_host

extern "C" {

uint64_t l2j_quant_nbytes(uint64_t nfloats) { return (nfloats + kGroup - 1) / kGroup * kGroupBytes; }

int l2j_quant_encode(const float *in, uint64_t nfloats, uint8_t *out)
{
    if (!in || !out) return fail(L2J_E_ARG, "null argument");
    const uint64_t ngroups = (nfloats + kGroup - 1) / kGroup;
    parallel_groups(ngroups, [&](uint64_t a, uint64_t b) {
        for (uint64_t g = a; g < b; g++)
            encode_group(in + g * kGroup, std::min(kGroup, nfloats - g * kGroup), out + g * kGroupBytes);
    });
    return L2J_OK;
}

int l2j_quant_decode(const uint8_t *enc, uint64_t float_index, uint64_t size, float *out)
{
    if (!enc || !out) return fail(L2J_E_ARG, "null argument");
    uint64_t done = 0;
    while (done < size) {
        const uint64_t f = float_index + done, g = f / kGroup, j0 = f % kGroup;
        const uint8_t *base = enc + g * kGroupBytes;
        const float lo = load_be(base), range = load_be(base + 4) - lo;
        const uint64_t cnt = std::min(kGroup - j0, size - done);
        for (uint64_t j = 0; j < cnt; j++) out[done + j] = (float)base[8 + j0 + j] / 255.0f * range + lo;
        done += cnt;
    }
    return L2J_OK;
}

int l2j_write_quant_file(const char *path, const uint8_t *bytes, uint64_t nbytes)
{
    if (!path || !bytes) return fail(L2J_E_ARG, "null argument");
    if (nbytes > 0x7fffffffull) return fail(L2J_E_SIZE, "a .quant file holds at most 2^31-1 bytes (int32 length prefix)");
    FILE *f = fopen(path, "wb");
    if (!f) return fail(L2J_E_IO, std::string("cannot create ") + path);
    const uint32_t n = (uint32_t)nbytes;  // little-endian host
    const bool ok = fwrite(&n, 4, 1, f) == 1 && fwrite(bytes, 1, nbytes, f) == nbytes;
    fclose(f);
    return ok ? L2J_OK : fail(L2J_E_IO, std::string("short write to ") + path);
}

int64_t l2j_read_quant_file(const char *path, uint8_t *dst, uint64_t cap)
{
    if (!path || !dst) return fail(L2J_E_ARG, "null argument");
    FILE *f = fopen(path, "rb");
    if (!f) return fail(L2J_E_IO, std::string("cannot open ") + path);
    int32_t n = 0;
    if (fread(&n, 4, 1, f) != 1 || n < 0) {
        fclose(f);
        return fail(L2J_E_IO, std::string("bad length prefix in ") + path);
    }
    if ((uint64_t)n > cap) {
        fclose(f);
        return fail(L2J_E_SIZE, "totalByteSize != quant.numberOfBytesByFloatSize(floatSize)");
    }
    const size_t got = fread(dst, 1, (size_t)n, f);
    fclose(f);
    if (got != (size_t)n) return fail(L2J_E_IO, std::string("short read from ") + path);
    return n;
}

int l2j_quant_cache_path(const char *bin_path, int tensor, char *out, int cap)
{
    if (!bin_path || !out || cap <= 0) return fail(L2J_E_ARG, "null argument");
    const char *stem = l2j_host::tensor_stem(tensor);
    if (!*stem) return fail(L2J_E_ARG, "not a quantized tensor");
    std::string p(bin_path), dir = ".", base = p;
    const size_t slash = p.rfind('/');
    if (slash != std::string::npos) {
        dir = p.substr(0, slash);
        base = p.substr(slash + 1);
    }
    const size_t dot = base.rfind('.');
    if (dot != std::string::npos && dot > 0) base = base.substr(0, dot);  // J/BinFileReader.java:41-49
    const std::string r = dir + "/" + base + "_" + stem + "_256_8.quant";
    if ((int)r.size() + 1 > cap) return fail(L2J_E_SIZE, "path buffer too small");
    memcpy(out, r.c_str(), r.size() + 1);
    return (int)r.size();
}

int l2j_read_checkpoint_header(const char *bin_path, l2j_config *cfg)
{
    if (!bin_path || !cfg) return fail(L2J_E_ARG, "null argument");
    FILE *f = fopen(bin_path, "rb");
    if (!f) return fail(L2J_E_IO, std::string("cannot open ") + bin_path);
    int32_t h[7];
    const bool ok = fread(h, 4, 7, f) == 7;
    fclose(f);
    if (!ok) return fail(L2J_E_IO, "short header");
    memset(cfg, 0, sizeof *cfg);
    cfg->dim = h[0]; cfg->hidden_dim = h[1]; cfg->n_layers = h[2]; cfg->n_heads = h[3]; cfg->n_kv_heads = h[4];
    cfg->shared_weights = h[5] > 0;            // J/Run.java:572
    cfg->vocab_size = h[5] < 0 ? -h[5] : h[5]; // J/Run.java:573
    cfg->seq_len = h[6];
    cfg->group_size = 256;
    cfg->bits = 8;
    return L2J_OK;
}

int l2j_load_checkpoint(const char *bin_path, int device, uint32_t flags, int write_caches, l2j_ctx **out)
{
    if (!bin_path || !out) return fail(L2J_E_ARG, "null argument");
    *out = nullptr;
    l2j_config cfg;
    int rc = l2j_read_checkpoint_header(bin_path, &cfg);
    if (rc) return rc;
    if (cfg.dim <= 0 || cfg.n_heads <= 0 || cfg.dim % cfg.n_heads) return fail(L2J_E_IO, "implausible header");
    cfg.device = device;
    cfg.flags = flags;
    Mapped m;
    if ((rc = map_file(bin_path, m))) return rc;
    l2j_ctx *ctx = nullptr;
    if ((rc = l2j_create(&cfg, &ctx))) return rc;

    const uint64_t vd = (uint64_t)cfg.vocab_size * cfg.dim;
    uint64_t off = 28;  // bytes consumed
    auto need = [&](uint64_t nfloats) { return off + nfloats * 4 <= m.len; };
#define BAIL(code, msg)            \
    do {                           \
        l2j_destroy(ctx);          \
        return fail((code), (msg)); \
    } while (0)
#define TRY(expr)             \
    do {                      \
        rc = (expr);          \
        if (rc) {             \
            l2j_destroy(ctx); \
            return rc;        \
        }                     \
    } while (0)

    if (!need(vd)) BAIL(L2J_E_IO, "checkpoint too short: token_embedding_table");
    const uint64_t emb_off = off;
    off += vd * 4;

    // The tensors by a few threads, as the reference's readAsQuant takes them (ten virtual threads,
    // J/TransformerWeights.java:52,204): the uploads themselves take turns inside the library, but reading a cache file (or
    // writing one) goes on beside them.  A thread's error text is its own: the first failure's is handed to the caller's.
    struct Job { int tensor; uint64_t off, nf, nb; };   // (the two fp32 tensors too: nb = 0)
    std::vector<Job> jobs;
    jobs.push_back({L2J_TOK_EMB, emb_off, vd, 0});
    for (int t = L2J_RMS_ATT; t <= L2J_RMS_FINAL; t++) {
        const uint64_t nf = quant_floats(cfg, t), nb = l2j_quant_nbytes(nf);
        if (!need(nf)) BAIL(L2J_E_IO, std::string("checkpoint too short: ") + kStems[t]);
        jobs.push_back({t, off, nf, nb});
        off += nf * 4;
    }
    off += 2ull * ((uint64_t)cfg.seq_len * (cfg.dim / cfg.n_heads) / 2) * 4;  // freq_cis_real, freq_cis_imag: skipped
    if (!cfg.shared_weights) {
        if (!need(vd)) BAIL(L2J_E_IO, "checkpoint too short: wcls");
        jobs.push_back({L2J_WCLS, off, vd, 0});
    }
    std::sort(jobs.begin(), jobs.end(), [](const Job &a, const Job &b) { return a.nf > b.nf; });   // (the long ones first)
    std::atomic<size_t> next{0};
    std::mutex err_mu;
    int first_rc = L2J_OK;
    std::string first_msg;
    auto work = [&]() {
        std::vector<uint8_t> bytes;
        for (size_t k = next.fetch_add(1); k < jobs.size(); k = next.fetch_add(1)) {
            const Job &j = jobs[k];
            int r = L2J_OK;
            char qpath[4096];
            struct stat st;
            if (j.nb == 0) {
                r = l2j_upload_f32(ctx, j.tensor, reinterpret_cast<const float *>(m.p + j.off), j.nf);
            } else if (l2j_quant_cache_path(bin_path, j.tensor, qpath, sizeof qpath) < 0) {
                r = fail(L2J_E_ARG, "cache file name too long");
            } else if (stat(qpath, &st) == 0) {
                // cache branch: the floats are skipped (J/TransformerWeights.java:198-203,219-232).  The file is uploaded out of
                // a mapping of it (as l2j_read_quant_file checks it: the length prefix, then that many bytes).
                Mapped q;
                r = map_file(qpath, q);
                if (r == L2J_OK) {
                    int32_t n = -1;
                    if (q.len >= 4) memcpy(&n, q.p, 4);
                    if (n < 0) r = fail(L2J_E_IO, std::string("bad length prefix in ") + qpath);
                    else if ((uint64_t)n > q.len - 4) r = fail(L2J_E_IO, std::string("short read from ") + qpath);
                    else r = l2j_upload_quant(ctx, j.tensor, q.p + 4, (uint64_t)n);   // (a size other than the tensor's: L2J_E_SIZE)
                }
            } else {
                r = l2j_upload_f32_quantize(ctx, j.tensor, 0, reinterpret_cast<const float *>(m.p + j.off), j.nf);
                if (r == L2J_OK && write_caches && j.nb <= 0x7fffffffull) {
                    bytes.resize(j.nb);
                    r = l2j_read_quant(ctx, j.tensor, 0, j.nb / kGroupBytes, bytes.data());
                    if (r == L2J_OK) r = l2j_write_quant_file(qpath, bytes.data(), j.nb);
                }
            }
            if (r != L2J_OK) {
                std::lock_guard<std::mutex> lock(err_mu);
                if (first_rc == L2J_OK) { first_rc = r; first_msg = l2j_last_error(); }
                next.store(jobs.size());   // (the others stop after the tensor they are at)
                return;
            }
        }
    };
    {
        const unsigned hw = std::thread::hardware_concurrency();
        const size_t nthreads = std::min<size_t>(jobs.size(), std::max(1u, std::min(6u, hw ? hw : 1u)));
        std::vector<std::thread> pool;
        for (size_t i = 1; i < nthreads; i++) pool.emplace_back(work);
        work();
        for (std::thread &th : pool) th.join();
    }
    if (first_rc != L2J_OK) BAIL(first_rc, first_msg);
    TRY(l2j_finalize(ctx));
#undef TRY
#undef BAIL
    *out = ctx;
    return L2J_OK;
}

}  // extern "C"
