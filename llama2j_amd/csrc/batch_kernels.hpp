// Several sequences per pass over the weights ("parallel processing of multiple queries", the reference's README
// wish-list): with sixteen activation vectors per weight matrix the multiply-adds are a 16-wide GEMM and run on the
// matrix cores.  v_mfma_f32_16x16x4_f32 multiplies and accumulates in fp32, so the arithmetic of the single-sequence
// path is kept (byte code -> float, fp32 activations, fp32 sums, rm * sum(code * x) + min * sum(x) per group of 256;
// K/MatMul.java:117-151 is the loop it restates); the vector units only convert the codes.
#pragma once

#include "kernels.hpp"

namespace l2j {

constexpr int kBatch = 16;          // sequences per step: the 16 columns of one MFMA
constexpr int kBgThreads = 256;     // four waves share the staged activations (measured at the 7B shape, ms per step: 64: 7.2, 128: 6.0, 256: 4.8, 512: 5.3, 1024: 6.0)
constexpr int kBgRowsPerWave = 32;  // two 16-row tiles share the activations fetched from LDS
constexpr int kBgRowsPerWG = kBgRowsPerWave * (kBgThreads / 64);
constexpr int kXPad = 4;            // floats between the slices of two sequences in LDS: a quarter wave's 16-byte reads then cover every bank once

typedef float v4f32 __attribute__((ext_vector_type(4)));

// y[b][r] = sum_k dequant(W[r][k]) * x[b][k], split over slices of K: part[slice][b][r].  Up to three matrices that
// share the input (Wq, Wk, Wv; W1, W3) go into one launch: their row blocks follow each other in grid.x.
constexpr int kBgMaxMat = 3;
constexpr int kBgMaxGps = 16;       // most groups per slice
struct BGemm {
    QMat m[kBgMaxMat];        // m.off: the layer's matrix (a multiple of 256), rows of K codes
    int rows[kBgMaxMat];      // rows % 16 == 0
    float *part[kBgMaxMat];   // (slices, kBatch, rows)
    int nmat;
    int K;                    // K % 256 == 0
    const float *x;           // (kBatch, K)
    int gps;                  // groups of 256 codes per slice
};


__device__ __forceinline__ float code_f(const uint4 &w, int j)
{
    const uint32_t d = (j >> 2) == 0 ? w.x : (j >> 2) == 1 ? w.y : (j >> 2) == 2 ? w.z : w.w;
    return ubyte_f(d, j & 3);
}

__host__ __device__ inline int bg_units(int rows, int tiles) { return (rows + 16 * tiles - 1) / (16 * tiles); }

// Workgroup (y: one slice of K; x: a share of the rows): the slice of the sixteen activation vectors is staged in LDS once,
// then every wave takes units of 16 * TILES rows (of all the launch's matrices, in order) in turn: unit
// blockIdx.x * 4 + wave, then every gridDim.x * 4-th.  A lane (r = lane % 16, s = lane / 16) holds the codes of row r at
// k = 64 T + 16 s + j (T < 4, j < 16: four 16-byte loads per group and tile); step (T, j) of the MFMA multiplies the 16
// rows by the 16 sequences over the four k of the four s.  After the 64 steps of a group the 16 x 16 sums get the
// group's scale and offset.  TILES = 2: two tiles share the activations fetched from LDS.
template <int TILES>
__global__ void __launch_bounds__(kBgThreads) k_bgemm(const BGemm a)
{
    extern __shared__ float xs[];
    __shared__ float sxs[kBatch][kBgMaxGps];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ngroups = a.K >> 8;
    const int g0 = blockIdx.y * a.gps, g1 = min(ngroups, g0 + a.gps), nk = (g1 - g0) << 8;
    const int r = lane & 15, s = lane >> 4;
    int total = 0;
    for (int i = 0; i < a.nmat; i++) total += bg_units(a.rows[i], TILES);
    const int stride = gridDim.x * (kBgThreads / 64);
    int u = blockIdx.x * (kBgThreads / 64) + wave;

    QMat mat;
    int rows = 0, row0 = 0;
    float *part = nullptr;
    bool two = false;
    const uint4 *c0 = nullptr, *c1 = nullptr;
    const float2 *gs0 = nullptr, *gs1 = nullptr;
    uint4 w0[4], w1[4];
    auto begin_unit = [&](int unit) {   // where the unit's rows are, and its first group of codes requested
        int mi = 0;
        while (mi + 1 < a.nmat && unit >= bg_units(a.rows[mi], TILES)) { unit -= bg_units(a.rows[mi], TILES); mi++; }
        mat = a.m[mi]; rows = a.rows[mi]; part = a.part[mi];
        row0 = unit * 16 * TILES;
        two = TILES == 2 && row0 + 16 < rows;
        c0 = reinterpret_cast<const uint4 *>(mat.codes + mat.off + (long)(row0 + r) * a.K + (g0 << 8) + 16 * s);
        c1 = reinterpret_cast<const uint4 *>(reinterpret_cast<const uint8_t *>(c0) + (two ? 16L * a.K : 0L));
        gs0 = mat.gs + ((mat.off + (long)(row0 + 4 * s) * a.K) >> 8) + g0;
        gs1 = gs0 + (two ? 16L * ngroups : 0L);
#pragma unroll
        for (int T = 0; T < 4; T++) { w0[T] = load_stream(c0 + 4 * T); if (TILES == 2) w1[T] = load_stream(c1 + 4 * T); }
    };
    if (u < total) begin_unit(u);   // the first codes are requested before the activations are staged

    const int pitch = nk + kXPad;   // LDS: sequence-major, xs[b * pitch + k]
    {
        const int nk4 = nk >> 2;   // 16-byte words per sequence in the slice
#pragma unroll 8
        for (int f = tid; f < kBatch * nk4; f += kBgThreads) {
            const int b = f / nk4, k4 = f - b * nk4;
            *reinterpret_cast<float4 *>(xs + b * pitch + 4 * k4) = *reinterpret_cast<const float4 *>(a.x + (long)b * a.K + (g0 << 8) + 4 * k4);
        }
    }
    __syncthreads();
    // sum of every sequence's activations over each group of the slice (for the groups' offsets): 16 threads per sequence,
    // while the first codes are on their way
    {
        const int b = tid >> 4, pt = tid & 15;
        for (int gi = 0; gi < g1 - g0; gi++) {
            const float4 *xp = reinterpret_cast<const float4 *>(xs + b * pitch + (gi << 8) + 16 * pt);
            const float4 v0 = xp[0], v1 = xp[1], v2 = xp[2], v3 = xp[3];
            float t = ((v0.x + v0.y) + (v0.z + v0.w)) + ((v1.x + v1.y) + (v1.z + v1.w)) + ((v2.x + v2.y) + (v2.z + v2.w)) +
                      ((v3.x + v3.y) + (v3.z + v3.w));
#pragma unroll
            for (int off = 8; off > 0; off >>= 1) t += __shfl_xor(t, off);
            if (pt == 0) sxs[b][gi] = t;
        }
    }
    __syncthreads();
    bool first = true;
    for (; u < total; u += stride) {
        if (!first) begin_unit(u);
        first = false;
        v4f32 y0 = {0.f, 0.f, 0.f, 0.f}, y1 = {0.f, 0.f, 0.f, 0.f};
        for (int g = g0; g < g1; g++) {
            uint4 u0[4], u1[4];
#pragma unroll
            for (int T = 0; T < 4; T++) { u0[T] = w0[T]; u1[T] = w1[T]; }
            if (g + 1 < g1) {   // the next group's codes are requested before this one is multiplied
                c0 += 16; c1 += 16;
#pragma unroll
                for (int T = 0; T < 4; T++) { w0[T] = load_stream(c0 + 4 * T); if (TILES == 2) w1[T] = load_stream(c1 + 4 * T); }
            }
            float2 sc0[4], sc1[4];
#pragma unroll
            for (int i = 0; i < 4; i++) { sc0[i] = gs0[(long)i * ngroups]; if (TILES == 2) sc1[i] = gs1[(long)i * ngroups]; }
            const float sxv = sxs[r][g - g0];   // this lane's column is sequence r
            v4f32 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f}, acc3 = {0.f, 0.f, 0.f, 0.f};
            const float4 *xk = reinterpret_cast<const float4 *>(xs + r * pitch + ((g - g0) << 8) + 16 * s);   // sequence r, k = 64 T + 16 s + j
            float4 xn[4];
#pragma unroll
            for (int q = 0; q < 4; q++) xn[q] = xk[q];
#pragma unroll
            for (int T = 0; T < 4; T++) {
                float4 xc[4];
#pragma unroll
                for (int q = 0; q < 4; q++) xc[q] = xn[q];
                if (T < 3) {   // the activations of the next 16 steps are fetched while these are multiplied
#pragma unroll
                    for (int q = 0; q < 4; q++) xn[q] = xk[16 * (T + 1) + q];
                }
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const float bx[4] = {xc[q].x, xc[q].y, xc[q].z, xc[q].w};
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int j = 4 * q + e;
                        if (e & 1) {   // two sums per tile: independent chains of MFMAs
                            acc2 = __builtin_amdgcn_mfma_f32_16x16x4f32(code_f(u0[T], j), bx[e], acc2, 0, 0, 0);
                            if (TILES == 2) acc3 = __builtin_amdgcn_mfma_f32_16x16x4f32(code_f(u1[T], j), bx[e], acc3, 0, 0, 0);
                        } else {
                            acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(code_f(u0[T], j), bx[e], acc0, 0, 0, 0);
                            if (TILES == 2) acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(code_f(u1[T], j), bx[e], acc1, 0, 0, 0);
                        }
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < 4; i++) {
                y0[i] += fmaf(sc0[i].x, acc0[i] + acc2[i], sc0[i].y * sxv);
                if (TILES == 2) y1[i] += fmaf(sc1[i].x, acc1[i] + acc3[i], sc1[i].y * sxv);
            }
            gs0++; gs1++;
        }
        // lane holds rows row0 + 4 s + (0..3) of sequence r
        float *p = part + ((long)blockIdx.y * kBatch + r) * rows + row0 + 4 * s;
        *reinterpret_cast<v4f32 *>(p) = y0;
        if (two) *reinterpret_cast<v4f32 *>(p + 16) = y1;
    }
}

// ---- the classifier: fp32 weights (K/MatMul.java:37-60), the same tiling -------------------------------------------

struct BGemmF32 {
    const float *w;    // (rows, K) fp32
    int rows, K;       // rows % 16 == 0, K % 256 == 0
    const float *x;    // (kBatch, K)
    float *part;       // (slices, kBatch, rows)
    int gps;
};

// As k_bgemm with float weights: a lane (r, s) holds row r at k = 64 T + 16 s + j as four 16-byte loads per block of 64 k.
__global__ void __launch_bounds__(kBgThreads) k_bgemm_f32(const BGemmF32 a)
{
    extern __shared__ float xs[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ngroups = a.K >> 8;
    const int g0 = blockIdx.y * a.gps, g1 = min(ngroups, g0 + a.gps), nk = (g1 - g0) << 8;
    const int row0 = min(blockIdx.x * kBgRowsPerWG + wave * kBgRowsPerWave, a.rows - 16);
    const bool live = blockIdx.x * kBgRowsPerWG + wave * kBgRowsPerWave < a.rows;
    const int r = lane & 15, s = lane >> 4;
    const bool two = row0 + 16 < a.rows;
    const float4 *c0 = reinterpret_cast<const float4 *>(a.w + (long)(row0 + r) * a.K + (g0 << 8) + 16 * s);
    const float4 *c1 = c0 + (two ? 4L * a.K : 0L);   // 16 rows on, in 16-byte words
    float4 w0[4], w1[4];
#pragma unroll
    for (int q = 0; q < 4; q++) { w0[q] = load_stream(c0 + q); w1[q] = load_stream(c1 + q); }
    const int pitch = nk + kXPad;
    {
        const int nk4 = nk >> 2;
#pragma unroll 8
        for (int f = tid; f < kBatch * nk4; f += kBgThreads) {
            const int b = f / nk4, k4 = f - b * nk4;
            *reinterpret_cast<float4 *>(xs + b * pitch + 4 * k4) = *reinterpret_cast<const float4 *>(a.x + (long)b * a.K + (g0 << 8) + 4 * k4);
        }
    }
    __syncthreads();
    if (!live) return;
    v4f32 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f}, acc3 = {0.f, 0.f, 0.f, 0.f};
    const float4 *xk = reinterpret_cast<const float4 *>(xs + r * pitch + 16 * s);
    const int nblocks = nk >> 6;   // blocks of 64 k
    for (int T = 0; T < nblocks; T++) {
        float4 u0[4], u1[4], xc[4];
#pragma unroll
        for (int q = 0; q < 4; q++) { u0[q] = w0[q]; u1[q] = w1[q]; xc[q] = xk[16 * T + q]; }
        if (T + 1 < nblocks) {
            c0 += 16; c1 += 16;   // 64 floats on
#pragma unroll
            for (int q = 0; q < 4; q++) { w0[q] = load_stream(c0 + q); w1[q] = load_stream(c1 + q); }
        }
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const float bx[4] = {xc[q].x, xc[q].y, xc[q].z, xc[q].w};
            const float a0[4] = {u0[q].x, u0[q].y, u0[q].z, u0[q].w}, a1[4] = {u1[q].x, u1[q].y, u1[q].z, u1[q].w};
#pragma unroll
            for (int e = 0; e < 4; e++) {
                if (e & 1) {
                    acc2 = __builtin_amdgcn_mfma_f32_16x16x4f32(a0[e], bx[e], acc2, 0, 0, 0);
                    acc3 = __builtin_amdgcn_mfma_f32_16x16x4f32(a1[e], bx[e], acc3, 0, 0, 0);
                } else {
                    acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a0[e], bx[e], acc0, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a1[e], bx[e], acc1, 0, 0, 0);
                }
            }
        }
    }
    float *p = a.part + ((long)blockIdx.y * kBatch + r) * a.rows + row0 + 4 * s;
    *reinterpret_cast<v4f32 *>(p) = acc0 + acc2;
    if (two) *reinterpret_cast<v4f32 *>(p + 16) = acc1 + acc3;
}

// ---- the element-wise kernels between the products --------------------------------------------------------------

// Loop state of a batched decode, on the device.
struct BatchState {
    int pos;              // position of the step being computed
    int token[kBatch];    // input token of every sequence at this position
    int n_prompt[kBatch];
};

// x[b] = row token[b] of the embedding table (J/Run.java:72)
__global__ void __launch_bounds__(256) k_bembed(const float *__restrict__ emb, const BatchState *st, float *__restrict__ x, int dim)
{
    const int b = blockIdx.x;
    const float4 *src = reinterpret_cast<const float4 *>(emb + (long)st->token[b] * dim);
    float4 *dst = reinterpret_cast<float4 *>(x + (long)b * dim);
    for (int i = threadIdx.x; i < (dim >> 2); i += blockDim.x) dst[i] = src[i];
}

// xn[b] = w * (ss * x[b]), ss = 1 / sqrt(sum(x^2) / n + 1e-5) (K/RootMeanSquare.java:25-35, K/WeightNormalizeAndScale.java:73).
// One workgroup of 1024 threads per sequence.
__global__ void __launch_bounds__(1024) k_brms(const float *__restrict__ x, const float *__restrict__ w, float *__restrict__ xn, int n)
{
    __shared__ float red[16];
    const int b = blockIdx.x, tid = threadIdx.x, n4 = n >> 2;
    const float4 *xp = reinterpret_cast<const float4 *>(x + (long)b * n);
    float ssq = 0.0f;
    for (int i = tid; i < n4; i += 1024) {
        const float4 v = xp[i];
        ssq += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
    }
    ssq = block_sum(ssq, red, 16);
    const float ss = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(__fdiv_rn(ssq, (float)n), 1e-5f)));
    const float4 *wp = reinterpret_cast<const float4 *>(w);
    float4 *op = reinterpret_cast<float4 *>(xn + (long)b * n);
    for (int i = tid; i < n4; i += 1024) {
        float4 v = xp[i];
        const float4 wv = wp[i];
        v.x = __fmul_rn(wv.x, __fmul_rn(ss, v.x));
        v.y = __fmul_rn(wv.y, __fmul_rn(ss, v.y));
        v.z = __fmul_rn(wv.z, __fmul_rn(ss, v.z));
        v.w = __fmul_rn(wv.w, __fmul_rn(ss, v.w));
        op[i] = v;
    }
}

// x[b] += the slices of a product summed in order (K/Accum.java:26-30), then xn[b] as k_brms does: the
// hand-over from Wo to W1/W3 and from W2 to the next layer's Wq/Wk/Wv (or to the classifier) in one kernel.
__global__ void __launch_bounds__(1024) k_bres_rms(const float *__restrict__ part, int slices, float *__restrict__ x, const float *__restrict__ w,
                                                   float *__restrict__ xn, int n)
{
    __shared__ float red[16];
    const int b = blockIdx.x, tid = threadIdx.x, n4 = n >> 2;
    const long stride4 = (long)kBatch * n4;   // 16-byte words between two slices
    const float4 *pp = reinterpret_cast<const float4 *>(part) + (long)b * n4;
    float4 *xp = reinterpret_cast<float4 *>(x + (long)b * n);
    float ssq = 0.0f;
    for (int i = tid; i < n4; i += 1024) {
        float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll 8
        for (int s = 0; s < slices; s++) {   // (independent loads, added in slice order)
            const float4 v = pp[(long)s * stride4 + i];
            t.x += v.x; t.y += v.y; t.z += v.z; t.w += v.w;
        }
        float4 v = xp[i];
        v.x = __fadd_rn(v.x, t.x); v.y = __fadd_rn(v.y, t.y); v.z = __fadd_rn(v.z, t.z); v.w = __fadd_rn(v.w, t.w);
        xp[i] = v;
        ssq += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
    }
    ssq = block_sum(ssq, red, 16);   // (its barriers also order the stores above before the loads below)
    const float ss = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(__fdiv_rn(ssq, (float)n), 1e-5f)));
    const float4 *wp = reinterpret_cast<const float4 *>(w);
    float4 *op = reinterpret_cast<float4 *>(xn + (long)b * n);
    for (int i = tid; i < n4; i += 1024) {
        float4 v = xp[i];   // (written by this same thread)
        const float4 wv = wp[i];
        v.x = __fmul_rn(wv.x, __fmul_rn(ss, v.x));
        v.y = __fmul_rn(wv.y, __fmul_rn(ss, v.y));
        v.z = __fmul_rn(wv.z, __fmul_rn(ss, v.z));
        v.w = __fmul_rn(wv.w, __fmul_rn(ss, v.w));
        op[i] = v;
    }
}

// hb[b][r] = silu(h1) * h3 with the reference's sigmoid table (K/Silu.java:72-74), h1 and h3 the slices summed in order.
// grid (hidden / 256, kBatch), 256 threads.
__global__ void __launch_bounds__(256) k_bepi_swiglu(const float *__restrict__ p1, const float *__restrict__ p3, int slices, int hidden,
                                                     const float *__restrict__ silu, int exact, float *__restrict__ hb)
{
    const int b = blockIdx.y, rix = blockIdx.x * 256 + threadIdx.x;
    const long n = (long)kBatch * hidden, i = (long)b * hidden + rix;
    float h1 = 0.0f, h3 = 0.0f;
#pragma unroll 8
    for (int s = 0; s < slices; s++) { h1 += p1[(long)s * n + i]; h3 += p3[(long)s * n + i]; }
    const float sg = silu_sigma(silu, h1, exact);
    hb[i] = __fmul_rn(h1, __fmul_rn(sg, h3));
}

struct BAttn {
    const float *pq, *pk, *pv;   // partial products of Wq, Wk, Wv: (slices, kBatch, dim | kv_dim)
    int slices;
    const float2 *rope;          // (seq_len, head_size / 2) cos, sin
    float *kc, *vc;              // this layer's rows of the batch cache: + (b * seq_stride + pos) * kv_dim
    long seq_stride;             // cache rows between two sequences
    float *out;                  // (kBatch, dim)
    const BatchState *st;
    int n_heads, kv_mul, head_size, kv_dim, dim;
    float sqrt_hs;
};

// Attention of one head of one sequence over positions 0..pos (K/AttentionLoop.java:29-54, K/ExpSumNormalize.java:25-38,
// K/AccumWeightedValue.java).  First q of the head and k, v of its kv head at this position: the slices of the products
// summed in order, RoPE on the pairs of q and k (K/ApplyRope.java:74-90), k and v into the cache row (J/Run.java:95-99; by
// the first head of the kv group).  Then LPR lanes per cache row (four floats of the head each): the row slots of the
// workgroup take the positions in turn with an online softmax, and the slots are folded at the end.  grid (n_heads, kBatch).
template <int LPR>
__global__ void __launch_bounds__(256) k_battn(const BAttn a)
{
    constexpr int RPW = 64 / LPR, NSLOT = 4 * RPW;
    __shared__ float sm_m[NSLOT], sm_l[NSLOT];
    __shared__ float4 sm_acc[NSLOT * LPR];
    __shared__ __align__(16) float sm_qkv[3][4 * LPR];
    const int h = blockIdx.x, b = blockIdx.y, tid = threadIdx.x, lane = tid & 63;
    const int j = lane % LPR, slot = (tid >> 6) * RPW + lane / LPR;
    const int pos = a.st->pos, len = pos + 1, hs = a.head_size, kvh = h / a.kv_mul;
    const int half = hs >> 1;
    for (int p = tid; p < 3 * half; p += 256) {   // one thread per pair of q, k, v
        const int which = p / half, idx = p - which * half;
        {
            const int rows = which == 0 ? a.dim : a.kv_dim, row = (which == 0 ? h : kvh) * hs + 2 * idx;
            const float *part = which == 0 ? a.pq : which == 1 ? a.pk : a.pv;
            float v0 = 0.0f, v1 = 0.0f;
            for (int s = 0; s < a.slices; s++) {
                const float2 t = *reinterpret_cast<const float2 *>(part + ((long)s * kBatch + b) * rows + row);
                v0 += t.x; v1 += t.y;
            }
            if (which < 2) {
                const float2 cs = a.rope[(long)pos * half + idx];
                const float r0 = __fsub_rn(__fmul_rn(v0, cs.x), __fmul_rn(v1, cs.y));
                const float r1 = __fadd_rn(__fmul_rn(v0, cs.y), __fmul_rn(v1, cs.x));
                v0 = r0; v1 = r1;
            }
            sm_qkv[which][2 * idx] = v0;
            sm_qkv[which][2 * idx + 1] = v1;
            if (which > 0 && h % a.kv_mul == 0)
                *reinterpret_cast<float2 *>((which == 1 ? a.kc : a.vc) + ((long)b * a.seq_stride + pos) * a.kv_dim + kvh * hs + 2 * idx) =
                    make_float2(v0, v1);
        }
    }
    __syncthreads();
    const bool on = 4 * j < hs;
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    const float4 q4 = on ? *reinterpret_cast<const float4 *>(&sm_qkv[0][4 * j]) : zero;
    const float4 kp = on ? *reinterpret_cast<const float4 *>(&sm_qkv[1][4 * j]) : zero;   // the row of this position
    const float4 vp = on ? *reinterpret_cast<const float4 *>(&sm_qkv[2][4 * j]) : zero;
    const long base = (long)b * a.seq_stride * a.kv_dim + kvh * hs + 4 * j;
    float m = -3.0e38f, l = 0.0f;
    float4 acc = zero;
    for (int t0 = slot; t0 < len; t0 += 2 * NSLOT) {   // two rows in flight per slot
        const int t1 = t0 + NSLOT;
        const bool ok1 = t1 < len;
        const bool c0 = on && t0 < pos, c1 = on && t1 < pos;   // rows of earlier positions come from the cache
        float4 k0 = c0 ? *reinterpret_cast<const float4 *>(a.kc + base + (long)t0 * a.kv_dim) : zero;
        float4 v0 = c0 ? *reinterpret_cast<const float4 *>(a.vc + base + (long)t0 * a.kv_dim) : zero;
        float4 k1 = c1 ? *reinterpret_cast<const float4 *>(a.kc + base + (long)t1 * a.kv_dim) : zero;
        float4 v1 = c1 ? *reinterpret_cast<const float4 *>(a.vc + base + (long)t1 * a.kv_dim) : zero;
        if (t0 == pos) { k0 = kp; v0 = vp; }
        if (t1 == pos) { k1 = kp; v1 = vp; }
        float s0 = (q4.x * k0.x + q4.y * k0.y) + (q4.z * k0.z + q4.w * k0.w);
        float s1 = (q4.x * k1.x + q4.y * k1.y) + (q4.z * k1.z + q4.w * k1.w);
#pragma unroll
        for (int off = LPR / 2; off > 0; off >>= 1) { s0 += __shfl_xor(s0, off); s1 += __shfl_xor(s1, off); }
        s0 = __fdiv_rn(s0, a.sqrt_hs);
        s1 = ok1 ? __fdiv_rn(s1, a.sqrt_hs) : -3.0e38f;
        const float mb = fmaxf(m, fmaxf(s0, s1));
        const float sc = expf(m - mb), p0 = expf(s0 - mb), p1 = ok1 ? expf(s1 - mb) : 0.0f;
        l = l * sc + p0 + p1;
        acc.x = acc.x * sc + p0 * v0.x + p1 * v1.x;
        acc.y = acc.y * sc + p0 * v0.y + p1 * v1.y;
        acc.z = acc.z * sc + p0 * v0.z + p1 * v1.z;
        acc.w = acc.w * sc + p0 * v0.w + p1 * v1.w;
        m = mb;
    }
    if (j == 0) { sm_m[slot] = m; sm_l[slot] = l; }
    sm_acc[slot * LPR + j] = acc;
    __syncthreads();
    if (tid < LPR && 4 * tid < hs) {
        float M = sm_m[0];
#pragma unroll
        for (int e = 1; e < NSLOT; e++) M = fmaxf(M, sm_m[e]);
        float L = 0.0f;
        float4 o = zero;
#pragma unroll
        for (int e = 0; e < NSLOT; e++) {
            const float w = expf(sm_m[e] - M);   // an empty slot has m = -3e38: weight 0
            const float4 v = sm_acc[e * LPR + tid];
            L += w * sm_l[e];
            o.x += w * v.x; o.y += w * v.y; o.z += w * v.z; o.w += w * v.w;
        }
        o.x = __fdiv_rn(o.x, L); o.y = __fdiv_rn(o.y, L); o.z = __fdiv_rn(o.z, L); o.w = __fdiv_rn(o.w, L);
        *reinterpret_cast<float4 *>(a.out + (long)b * a.dim + h * hs + 4 * tid) = o;
    }
}

struct BNext {
    const float *part;    // (slices, kBatch, vocab) partial logits
    int slices, vocab;
    float *logits;        // (kBatch, vocab)
    BatchState *st;
    const int *prompts;   // (kBatch, prompt_stride)
    int prompt_stride;
    int *out_tokens;      // (kBatch, out_stride): `next` of every step
    int out_stride;
};

// Logits of every sequence (the slices summed in order), first index of the maximum (J/Sampler.java:46-57) and the step of
// the token loop (J/Run.java:635-642, 668, 680): forced prompt id or argmax.  One workgroup per sequence; the last
// workgroup to finish advances the position.
__global__ void __launch_bounds__(1024) k_bnext(const BNext a, unsigned *done)
{
    __shared__ float bval[16];
    __shared__ int bidx[16];
    const int b = blockIdx.x, tid = threadIdx.x;
    const long n = (long)kBatch * a.vocab;
    float bv = -__builtin_inff();
    int bi = 0x7fffffff;
    for (int i = tid; i < a.vocab; i += 1024) {
        float t = 0.0f;
#pragma unroll 8
        for (int s = 0; s < a.slices; s++) t += a.part[(long)s * n + (long)b * a.vocab + i];
        a.logits[(long)b * a.vocab + i] = t;
        if (better(t, i, bv, bi)) { bv = t; bi = i; }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off);
        const int oi = __shfl_xor(bi, off);
        if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
    }
    if ((tid & 63) == 0) { bval[tid >> 6] = bv; bidx[tid >> 6] = bi; }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < 16; w++)
            if (better(bval[w], bidx[w], bv, bi)) { bv = bval[w]; bi = bidx[w]; }
        if (bi == 0x7fffffff) bi = 0;
        const int pos = a.st->pos;
        const int next = pos < a.st->n_prompt[b] ? a.prompts[(long)b * a.prompt_stride + pos] : bi;
        a.out_tokens[(long)b * a.out_stride + pos] = next;
        a.st->token[b] = next;
        __threadfence();
        if (atomicAdd(done, 1u) == kBatch - 1) {   // every sequence has its token: the step is over
            *done = 0u;
            a.st->pos = pos + 1;
        }
    }
}

// y[b][r] = sum over the slices, in slice order
__global__ void __launch_bounds__(256) k_breduce(const float *__restrict__ part, float *__restrict__ y, int rows, int slices)
{
    const long n = (long)kBatch * rows;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        float t = 0.0f;
        for (int sl = 0; sl < slices; sl++) t += part[(long)sl * n + i];
        y[i] = t;
    }
}

}  // namespace l2j
