// All layers of a batched step in one launch (option batch_fuse; slower than the eight launches per layer it replaces,
// measured, and off by default): the four products of a layer (k_bgemm's waves) and what lies between them (attention,
// residual + rmsnorm, SwiGLU) as eight phases with a grid barrier after each, all workgroups resident.  The first codes
// of a product are requested before the barrier that precedes it, and the phases between the products spread over all
// workgroups: the rmsnorm scalar is deferred (sum_k w_k (g_k ss x_k) = ss sum_k w_k g_k x_k), so a norm is no pass of one
// workgroup over a vector but a sum of squares per 256 floats, written beside g x, and a multiplication by ss where the
// product's partial sums are added up.  What one phase hands to the next goes through write-through stores and
// device-coherent 16-byte loads: the L2 caches of the XCDs are not coherent with each other inside a launch.
#pragma once

#include "batch_kernels.hpp"

namespace l2j {

enum { BS_QKV = 0, BS_WO = 1, BS_W13 = 2, BS_W2 = 3 };

struct BStep {
    BGemm g[4];               // the four products of layer 0 (m.off = 0): a layer further, rows * K codes further
    int gx[4];                // workgroups per slice of K
    int n_layers, nseq, dim, hidden, n_heads, kv_mul, head_size, kv_dim;
    float sqrt_hs;
    const float2 *rope;       // (seq_len, head_size / 2) cos, sin
    float *kc, *vc;           // the batch cache, head-major: b * seq_stride + l * layer_stride + (kv head * cap + pos) * head_size
    long seq_stride, layer_stride;   // floats
    int cap;
    const BatchState *st;
    float *x;                 // residual stream (nseq, dim): always read and written by the same wave
    float *xn, *xb, *hb;      // inputs of the products: g * x (nseq, dim), attention output (nseq, dim), SwiGLU output (nseq, hidden)
    const float *rmsw;        // rmsnorm weights: attention norm of layer l at l * dim, feed-forward norm at (n_layers + l) * dim
    float *ssq;               // [2][nseq][dim / 256] sums of squares of x: after Wo (read by the SwiGLU phase), after W2 (by the next attention)
    const float *silu;
    int exact;
    GridBar bar;              // one set of counters, zero at launch (the launch before clears them)
};

// Eight 16-byte device-coherent loads in flight, one wait.  (Loads and wait are one statement: the compiler must not
// touch the destination registers in between.)
__device__ __forceinline__ void ld_coh16_8(const float *const (&p)[8], float4 (&v)[8])
{
    asm volatile("global_load_dwordx4 %0, %8, off sc1\n\tglobal_load_dwordx4 %1, %9, off sc1\n\t"
                 "global_load_dwordx4 %2, %10, off sc1\n\tglobal_load_dwordx4 %3, %11, off sc1\n\t"
                 "global_load_dwordx4 %4, %12, off sc1\n\tglobal_load_dwordx4 %5, %13, off sc1\n\t"
                 "global_load_dwordx4 %6, %14, off sc1\n\tglobal_load_dwordx4 %7, %15, off sc1\n\t"
                 "s_waitcnt vmcnt(0)"
                 : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]), "=&v"(v[7])
                 : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]), "v"(p[7])
                 : "memory");
}

// The 16 bytes at p summed over n slices (stride floats apart) in slice order, from partial sums other workgroups of
// this launch wrote.
__device__ __forceinline__ float4 sum_slices_coh(const float *p, long stride, int n)
{
    float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int s0 = 0; s0 < n; s0 += 8) {
        const float *q[8];
        float4 v[8];
#pragma unroll
        for (int i = 0; i < 8; i++) q[i] = p + (long)min(s0 + i, n - 1) * stride;
        ld_coh16_8(q, v);
#pragma unroll
        for (int i = 0; i < 8; i++)
            if (s0 + i < n) { t.x += v[i].x; t.y += v[i].y; t.z += v[i].z; t.w += v[i].w; }
    }
    return t;
}

// The k-th grid barrier of a launch (k = 0, 1, ..) on one set of counters that are zero when the launch starts and only
// grow: the last workgroup of a group to arrive bumps the top counter, everybody waits until the top counter has reached
// (k + 1) times the number of groups.  Before it a wave has waited for its own write-through stores (s_waitcnt
// vmcnt(0)); the wait is bounded like k_token's.
__device__ __forceinline__ void step_barrier(const GridBar &b, unsigned k)
{
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned ng = min((unsigned)b.ngroups, gridDim.x);
        const unsigned g = blockIdx.x % ng;
        const unsigned gsize = (gridDim.x - g + ng - 1) / ng;
        const unsigned old = __hip_atomic_fetch_add(b.ctr + 64 * (1 + g), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (old + 1u == gsize * (k + 1u)) __hip_atomic_fetch_add(b.ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned want = ng * (k + 1u);
        int spins = 0;
        while (__hip_atomic_load(b.ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < want) {
            __builtin_amdgcn_s_sleep(1);
            if (++spins > b.maxspin || ((spins & 255) == 0 && ld_coh(b.fault) != 0)) {
                st_coh(b.fault, 1);
                break;
            }
        }
    }
    __syncthreads();
}

__device__ __forceinline__ void wait_own_stores() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// ss of every sequence from the sums of squares per 256 floats: 16 threads per sequence (the workgroup has 16 per sequence).
__device__ __forceinline__ void bstep_scalars(const float *ssq, int nch, int dim, float *ss_lds)
{
    const int b = threadIdx.x >> 4, c = threadIdx.x & 15;
    float v = 0.0f;
    for (int i = c; i < nch; i += 16) v += ld_coh(ssq + b * nch + i);
    v = row16_sum(v);
    if (c == 0) ss_lds[b] = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(__fdiv_rn(v, (float)dim), 1e-5f)));
    __syncthreads();
}

__device__ __forceinline__ void rope_pair(float &v0, float &v1, float c, float s)   // K/ApplyRope.java:74-90
{
    const float r0 = __fsub_rn(__fmul_rn(v0, c), __fmul_rn(v1, s));
    const float r1 = __fadd_rn(__fmul_rn(v0, s), __fmul_rn(v1, c));
    v0 = r0; v1 = r1;
}

// (m, l, acc) of two sets of cache rows into one (online softmax; an empty set has m = -3e38, l = 0)
__device__ __forceinline__ void fold_sets(float &m, float &l, float4 &acc, float mo, float lo, const float4 &ao)
{
    const float M = fmaxf(m, mo), w = expf(m - M), wo = expf(mo - M);
    l = l * w + lo * wo;
    acc.x = acc.x * w + ao.x * wo; acc.y = acc.y * w + ao.y * wo; acc.z = acc.z * w + ao.z * wo; acc.w = acc.w * w + ao.w * wo;
    m = M;
}

// Attention of every head of every sequence over positions 0..pos as k_battn computes it, two waves per (sequence, head):
// q, k, v of the head from the partial sums of Wq, Wk, Wv (times ss when the norm before them deferred it), RoPE, the
// cache row of this position stored by the first head of the kv group, then the rows of the cache dealt to the 2 * 64 / LPR
// row slots of the two waves, U rows in flight per slot, with an online softmax; the slots are folded inside each wave by
// lane exchanges and between the two waves through LDS.  Items (sequence-major) go to the workgroups in rounds of 2 NB each.
template <int LPR, int NB>
__device__ __forceinline__ void bstep_attention(const BStep &a, int l, float *lds, const float *ss_lds)
{
    constexpr int RPL = 64 / LPR, NW = 4 * NB, IPW = NW / 2, U = 4, NSL = 2 * RPL;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, sub = wave & 1, it = wave >> 1;
    const int j = lane % LPR, rsub = lane / LPR, slot = sub * RPL + rsub;
    const int hs = a.head_size, half = hs >> 1;
    const int pos = a.st->pos;
    const int items = a.n_heads * a.nseq, G = gridDim.x;
    const int rounds = (items + G * IPW - 1) / (G * IPW);
    const int S = bg_slices(a.g[BS_QKV].K);
    float *kc = a.kc + l * a.layer_stride, *vc = a.vc + l * a.layer_stride;
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    float *mine = lds + it * (hs + 4);   // of this pair of waves: m, l, then the head's accumulators
    for (int rd = 0; rd < rounds; rd++) {
        const int item = (rd * G + (int)blockIdx.x) * IPW + it;
        const bool live = item < items;
        float m = -3.0e38f, lsum = 0.0f;
        float4 acc = zero;
        int b = 0, h = 0;
        if (live) {
            b = item / a.n_heads; h = item - b * a.n_heads;
            const int kvh = h / a.kv_mul;
            const long strq = (long)a.nseq * a.dim, strk = (long)a.nseq * a.kv_dim;
            float4 q4 = sum_slices_coh(a.g[BS_QKV].part[0] + (long)b * a.dim + h * hs + 4 * j, strq, S);
            float4 k4 = sum_slices_coh(a.g[BS_QKV].part[1] + (long)b * a.kv_dim + kvh * hs + 4 * j, strk, S);
            float4 v4 = sum_slices_coh(a.g[BS_QKV].part[2] + (long)b * a.kv_dim + kvh * hs + 4 * j, strk, S);
            if (ss_lds) {
                const float ss = ss_lds[b];
                q4.x = __fmul_rn(ss, q4.x); q4.y = __fmul_rn(ss, q4.y); q4.z = __fmul_rn(ss, q4.z); q4.w = __fmul_rn(ss, q4.w);
                k4.x = __fmul_rn(ss, k4.x); k4.y = __fmul_rn(ss, k4.y); k4.z = __fmul_rn(ss, k4.z); k4.w = __fmul_rn(ss, k4.w);
                v4.x = __fmul_rn(ss, v4.x); v4.y = __fmul_rn(ss, v4.y); v4.z = __fmul_rn(ss, v4.z); v4.w = __fmul_rn(ss, v4.w);
            }
            const float4 cs = *reinterpret_cast<const float4 *>(a.rope + (long)pos * half + 2 * j);   // (cos, sin) of pairs 2 j and 2 j + 1
            rope_pair(q4.x, q4.y, cs.x, cs.y); rope_pair(q4.z, q4.w, cs.z, cs.w);
            rope_pair(k4.x, k4.y, cs.x, cs.y); rope_pair(k4.z, k4.w, cs.z, cs.w);
            const long base = (long)b * a.seq_stride + (long)kvh * a.cap * hs + 4 * j;
            if (slot == 0 && h % a.kv_mul == 0) {   // J/Run.java:95-99
                *reinterpret_cast<float4 *>(kc + base + (long)pos * hs) = k4;
                *reinterpret_cast<float4 *>(vc + base + (long)pos * hs) = v4;
            }
            for (int t0 = 0; t0 < pos; t0 += NSL * U) {
                float4 kk[U], vv[U];
                bool ok[U];
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const int t = t0 + u * NSL + slot;
                    ok[u] = t < pos;
                    kk[u] = ok[u] ? *reinterpret_cast<const float4 *>(kc + base + (long)t * hs) : zero;
                    vv[u] = ok[u] ? *reinterpret_cast<const float4 *>(vc + base + (long)t * hs) : zero;
                }
                float s[U];
#pragma unroll
                for (int u = 0; u < U; u++)
                    s[u] = group_sum<LPR>((q4.x * kk[u].x + q4.y * kk[u].y) + (q4.z * kk[u].z + q4.w * kk[u].w));
                float mb = m;
#pragma unroll
                for (int u = 0; u < U; u++) {
                    s[u] = ok[u] ? __fdiv_rn(s[u], a.sqrt_hs) : -3.0e38f;
                    mb = fmaxf(mb, s[u]);
                }
                const float sc = expf(m - mb);
                lsum *= sc; acc.x *= sc; acc.y *= sc; acc.z *= sc; acc.w *= sc;
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const float p = ok[u] ? expf(s[u] - mb) : 0.0f;
                    lsum += p;
                    acc.x += p * vv[u].x; acc.y += p * vv[u].y; acc.z += p * vv[u].z; acc.w += p * vv[u].w;
                }
                m = mb;
            }
            {   // the row of this position, from the registers: slot 0
                float s = group_sum<LPR>((q4.x * k4.x + q4.y * k4.y) + (q4.z * k4.z + q4.w * k4.w));
                s = __fdiv_rn(s, a.sqrt_hs);
                if (slot == 0) {
                    const float mb = fmaxf(m, s), sc = expf(m - mb), p = expf(s - mb);
                    lsum = lsum * sc + p;
                    acc.x = acc.x * sc + p * v4.x; acc.y = acc.y * sc + p * v4.y; acc.z = acc.z * sc + p * v4.z; acc.w = acc.w * sc + p * v4.w;
                    m = mb;
                }
            }
#pragma unroll
            for (int off = LPR; off < 64; off <<= 1) {   // the slots of this wave (both partners compute the same)
                const float mo = __shfl_xor(m, off), lo = __shfl_xor(lsum, off);
                const float4 ao = make_float4(__shfl_xor(acc.x, off), __shfl_xor(acc.y, off), __shfl_xor(acc.z, off), __shfl_xor(acc.w, off));
                fold_sets(m, lsum, acc, mo, lo, ao);
            }
            if (sub == 1 && rsub == 0) {
                if (j == 0) { mine[0] = m; mine[1] = lsum; }
                *reinterpret_cast<float4 *>(mine + 4 + 4 * j) = acc;
            }
        }
        __syncthreads();
        if (live && sub == 0 && rsub == 0) {
            const float4 ao = *reinterpret_cast<const float4 *>(mine + 4 + 4 * j);
            fold_sets(m, lsum, acc, mine[0], mine[1], ao);
            const v4f32 o = {__fdiv_rn(acc.x, lsum), __fdiv_rn(acc.y, lsum), __fdiv_rn(acc.z, lsum), __fdiv_rn(acc.w, lsum)};
            st_coh16(a.xb + (long)b * a.dim + h * hs + 4 * j, o);
        }
        if (rd + 1 < rounds) __syncthreads();   // (the next round writes the same LDS)
    }
}

// x[b] += the slices of a product summed in order (K/Accum.java:26-30), one wave per 256 floats (always the same wave for
// the same floats, so x needs no coherent access); then, unless nothing follows (`last`), the sum of squares of those 256
// floats and g * x as the next product's input: the consumer of that product's sums multiplies them by
// ss = 1 / sqrt(sum(x^2) / n + 1e-5) (K/RootMeanSquare.java:25-35, K/WeightNormalizeAndScale.java:73).
template <int NB>
__device__ __forceinline__ void bstep_residual(const BStep &a, const float *part, int slices, const float *g, float *ssq_out, bool last)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nch = a.dim >> 8, total = a.nseq * nch, GW = gridDim.x * 4 * NB;
    for (int wc = wave * (int)gridDim.x + (int)blockIdx.x; wc < total; wc += GW) {   // (spread over the compute units first)
        const int b = wc / nch, ch = wc - b * nch, i = (ch << 8) + 4 * lane;
        const float4 t = sum_slices_coh(part + (long)b * a.dim + i, (long)a.nseq * a.dim, slices);
        float4 *xp = reinterpret_cast<float4 *>(a.x + (long)b * a.dim + i);
        float4 v = *xp;
        v.x = __fadd_rn(v.x, t.x); v.y = __fadd_rn(v.y, t.y); v.z = __fadd_rn(v.z, t.z); v.w = __fadd_rn(v.w, t.w);
        *xp = v;
        if (!last) {
            const float q = wave_sum((v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w));
            if (lane == 0) st_coh(ssq_out + wc, q);
            const float4 gv = *reinterpret_cast<const float4 *>(g + i);
            const v4f32 o = {__fmul_rn(gv.x, v.x), __fmul_rn(gv.y, v.y), __fmul_rn(gv.z, v.z), __fmul_rn(gv.w, v.w)};
            st_coh16(a.xn + (long)b * a.dim + i, o);
        }
    }
}

// hb = silu(h1) * h3 with the reference's sigmoid table (K/Silu.java:72-74), h1 and h3 = ss * the slices of W1's and W3's
// products summed in order; four floats per thread.
__device__ __forceinline__ void bstep_swiglu(const BStep &a, const float *ss_lds)
{
    const long n = (long)a.nseq * a.hidden, n4 = n >> 2;
    const int S = bg_slices(a.g[BS_W13].K);
    const float *p1 = a.g[BS_W13].part[0], *p3 = a.g[BS_W13].part[1];
    for (long f = (long)blockIdx.x * blockDim.x + threadIdx.x; f < n4; f += (long)gridDim.x * blockDim.x) {
        const long i = 4 * f;
        const float ss = ss_lds[(int)(i / a.hidden)];
        const float4 s1 = sum_slices_coh(p1 + i, n, S), s3 = sum_slices_coh(p3 + i, n, S);
        const float h1[4] = {__fmul_rn(ss, s1.x), __fmul_rn(ss, s1.y), __fmul_rn(ss, s1.z), __fmul_rn(ss, s1.w)};
        const float h3[4] = {__fmul_rn(ss, s3.x), __fmul_rn(ss, s3.y), __fmul_rn(ss, s3.z), __fmul_rn(ss, s3.w)};
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = __fmul_rn(h1[e], __fmul_rn(silu_sigma(a.silu, h1[e], a.exact), h3[e]));
        st_coh16(a.hb + i, v4f32{o[0], o[1], o[2], o[3]});
    }
}

// grid: as many workgroups of 256 NB threads as are resident at once (one per compute unit); dynamic LDS as k_bgemm.
// Before: x = the embeddings, xn = their rmsnorm (normalized: the first attention multiplies by no ss), the barrier
// counters zero.  After: x = the residual stream after the last layer (the final norm is the caller's).
template <int NB>
__global__ void __launch_bounds__(kBgThreads * NB) k_bstep(const BStep *__restrict__ args)
{
    const BStep &a = *args;   // (in device memory: the kernel aims pointers at its parts, which an argument passed by value would be copied to scratch memory for)
    constexpr int NSEQ = kBatch * NB;
    extern __shared__ __align__(16) float lds[];   // the products' (bg_lds_bytes); the attention's hand-over between two waves
    __shared__ float ss_lds[NSEQ];
    const int wg = blockIdx.x, nch = a.dim >> 8;
    unsigned nbar = 0;
    BgWave<NB, NB> w(a.g[BS_QKV]);   // aimed at the four products of the argument in turn (the argument is never copied)
    int S = bg_slices(a.g[BS_QKV].K);
    bool in = wg < a.gx[BS_QKV] * S;
    if (in) w.begin(wg / S, wg % S, a.gx[BS_QKV], true);
    for (int l = 0; l < a.n_layers; l++) {
#pragma unroll 1
        for (int k = 0; k < 4; k++) {
            if (in) w.template run<true>(lds, true);
            wait_own_stores();
            step_barrier(a.bar, nbar++);
            const bool last = l + 1 == a.n_layers;
            switch (k) {
            case BS_QKV:
                if (l > 0) bstep_scalars(a.ssq + a.nseq * nch, nch, a.dim, ss_lds);
                if (a.head_size == 64) bstep_attention<16, NB>(a, l, lds, l > 0 ? ss_lds : nullptr);
                else if (a.head_size == 128) bstep_attention<32, NB>(a, l, lds, l > 0 ? ss_lds : nullptr);
                else bstep_attention<64, NB>(a, l, lds, l > 0 ? ss_lds : nullptr);
                break;
            case BS_WO:
                bstep_residual<NB>(a, a.g[BS_WO].part[0], S, a.rmsw + (long)(a.n_layers + l) * a.dim, a.ssq, false);
                break;
            case BS_W13:
                bstep_scalars(a.ssq, nch, a.dim, ss_lds);
                bstep_swiglu(a, ss_lds);
                break;
            default:
                bstep_residual<NB>(a, a.g[BS_W2].part[0], S, a.rmsw + (long)(l + 1) * a.dim, a.ssq + a.nseq * nch, last);
                break;
            }
            if (last && k == BS_W2) break;
            const int nk = (k + 1) & 3;
            wait_own_stores();
            w.ap = &a.g[nk];
            w.layer = l + (k == BS_W2 ? 1 : 0);
            S = bg_slices(a.g[nk].K);
            in = wg < a.gx[nk] * S;
            if (in) w.begin(wg / S, wg % S, a.gx[nk], true);   // the first codes travel while the others arrive
            step_barrier(a.bar, nbar++);
        }
    }
}

}  // namespace l2j
