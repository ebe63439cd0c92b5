// gfx950 kernels of the per-token forward pass (W8A32, batch 1).
//
// Every kernel is HBM-bandwidth bound: int8 codes are streamed with 16-byte loads, one wavefront
// per pair of output rows, the activation vector sits in LDS, accumulation is fp32, and the
// 64-lane reduction uses DPP.  MFMA is deliberately unused (a GEMV has no reuse to feed it).
//
// Reference semantics (paths relative to the reference root, J/ = src/main/java/com/lastbot/llama2j/,
// K/ = J/kernel/):
//   rmsnorm            K/RootMeanSquare.java:25-35 + K/WeightNormalizeAndScale.java:32-77
//   int8 matvec        K/MatMul.java:97-212        (dequant (code*((max-min)/255) + min))
//   RoPE               K/ApplyRope.java:34-92
//   attention          K/AttentionLoop.java:29-54, K/ExpSumNormalize.java:25-38, K/AccumWeightedValue.java:31-88
//   SwiGLU (LUT)       K/Silu.java:41-78
//   residual           K/Accum.java:26-30
//   classifier/argmax  K/MatMul.java:29-60, J/Sampler.java:46-57
//   encoder            J/Quant.java:156-193
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace l2j {

constexpr int kGroup = 256;       // weights per quantization group (J/Run.java:27)
constexpr int kGroupBytes = 264;  // reference bytes per group (J/Quant.java:35-37)
constexpr int kSiluTable = 8192;  // K/Silu.java:41

struct DevState {
    int token;     // token fed to the next forward
    int pos;       // its position
    int n_prompt;  // positions below this take prompt[pos] as output instead of the argmax
    int pad;
};

// ------------------------------------------------------------------------------------------
// wavefront helpers (64 lanes)
// ------------------------------------------------------------------------------------------

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

__device__ __forceinline__ float readlane_f(float v, int lane)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// Sum over each aligned group of 16 lanes (a DPP row); every lane of the row gets the sum.
__device__ __forceinline__ float row16_sum(float v)
{
    v += dpp_f<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_f<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_f<0x124>(v);  // row_ror:4
    v += dpp_f<0x128>(v);  // row_ror:8
    return v;
}

__device__ __forceinline__ float row16_max(float v)
{
    v = fmaxf(v, dpp_f<0xB1>(v));
    v = fmaxf(v, dpp_f<0x4E>(v));
    v = fmaxf(v, dpp_f<0x124>(v));
    v = fmaxf(v, dpp_f<0x128>(v));
    return v;
}

// Sum over all 64 lanes, result uniform.
__device__ __forceinline__ float wave_sum(float v)
{
    v = row16_sum(v);
    return (readlane_f(v, 0) + readlane_f(v, 16)) + (readlane_f(v, 32) + readlane_f(v, 48));
}

__device__ __forceinline__ float wave_max(float v)
{
    v = row16_max(v);
    return fmaxf(fmaxf(readlane_f(v, 0), readlane_f(v, 16)), fmaxf(readlane_f(v, 32), readlane_f(v, 48)));
}

// Sum over aligned groups of LPR lanes (16, 32 or 64); every lane of the group gets the sum.
template <int LPR>
__device__ __forceinline__ float group_sum(float v)
{
    v = row16_sum(v);
    if (LPR == 32) {
        v += __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));  // lane ^ 16
    } else if (LPR == 64) {
        v = (readlane_f(v, 0) + readlane_f(v, 16)) + (readlane_f(v, 32) + readlane_f(v, 48));
    }
    return v;
}

// Block-wide sum / max through LDS; `red` holds one float per wave.  All threads get the result.
__device__ __forceinline__ float block_sum(float v, float *red)
{
    const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float t = 0.0f;
    for (int w = 0; w < nw; w++) t += red[w];
    return t;
}

__device__ __forceinline__ float block_max(float v, float *red)
{
    const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    v = wave_max(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float t = red[0];
    for (int w = 1; w < nw; w++) t = fmaxf(t, red[w]);
    return t;
}

typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));

// streaming (read-once) 16-byte loads
__device__ __forceinline__ float4 load_stream(const float4 *p)
{
    const v4f v = __builtin_nontemporal_load(reinterpret_cast<const v4f *>(p));
    return make_float4(v.x, v.y, v.z, v.w);
}

__device__ __forceinline__ uint4 load_stream(const uint4 *p)
{
    const v4u v = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}

__device__ __forceinline__ float ubyte_f(uint32_t w, int b) { return (float)((w >> (8 * b)) & 0xffu); }

// sum_j code_j * x_j over 16 codes (one 16-byte load) against 16 activations
__device__ __forceinline__ float dot16(const uint4 w, const float4 x0, const float4 x1, const float4 x2, const float4 x3)
{
    float a = ubyte_f(w.x, 0) * x0.x;
    float b = ubyte_f(w.z, 0) * x2.x;
    a = fmaf(ubyte_f(w.x, 1), x0.y, a);
    b = fmaf(ubyte_f(w.z, 1), x2.y, b);
    a = fmaf(ubyte_f(w.x, 2), x0.z, a);
    b = fmaf(ubyte_f(w.z, 2), x2.z, b);
    a = fmaf(ubyte_f(w.x, 3), x0.w, a);
    b = fmaf(ubyte_f(w.z, 3), x2.w, b);
    a = fmaf(ubyte_f(w.y, 0), x1.x, a);
    b = fmaf(ubyte_f(w.w, 0), x3.x, b);
    a = fmaf(ubyte_f(w.y, 1), x1.y, a);
    b = fmaf(ubyte_f(w.w, 1), x3.y, b);
    a = fmaf(ubyte_f(w.y, 2), x1.z, a);
    b = fmaf(ubyte_f(w.w, 2), x3.z, b);
    a = fmaf(ubyte_f(w.y, 3), x1.w, a);
    b = fmaf(ubyte_f(w.w, 3), x3.w, b);
    return a + b;
}

__device__ __forceinline__ float dot4(const float4 a, const float4 b)
{
    return fmaf(a.w, b.w, fmaf(a.z, b.z, fmaf(a.y, b.y, a.x * b.x)));
}

// The reference's sigmoid: 8192-entry table on [-5,5) with linear interpolation and the integer
// index multiplier 819 (K/Silu.java:41-70); exact outside the table.
__device__ __forceinline__ float silu_sigma(const float *__restrict__ table, float val, int exact)
{
    const float position = __fmul_rn(__fadd_rn(val, 5.0f), 819.0f);
    if (!exact && position > 0.0f && position < 8191.0f) {
        const int idx = (int)position;
        const float lo = table[idx];
        return __fadd_rn(lo, __fmul_rn(__fsub_rn(position, (float)idx), __fsub_rn(table[idx + 1], lo)));
    }
    return (float)(1.0 / (1.0 + exp(-(double)val)));
}

// ------------------------------------------------------------------------------------------
// activation vector -> LDS
//
// LDS layout for an n-float vector (n % 16 == 0, nch = n/16 chunks): float4 xs[q*nch + c] holds
// x[16c+4q .. 16c+4q+3], so that lane c of a wave reads consecutive 16-byte words for a fixed q
// (bank-conflict free); sumx[c] = sum of the 16 activations of chunk c (for the group-min term).
// ------------------------------------------------------------------------------------------

struct RmsW {
    const uint8_t *codes;  // flat codes of the rms tensor
    const float2 *mm;      // (min, max) per group
    long off;              // float offset of this layer's weights inside the tensor (multiple of 16)
};

template <bool RMS>
__device__ __forceinline__ void stage_vector(const float *__restrict__ xin, int n, const RmsW rw, float4 *xs,
                                             float *sumx, float *red)
{
    const int nch = n >> 4;
    const int tid = threadIdx.x, T = blockDim.x;
    if (RMS) {
        float ssq = 0.0f;
        for (int c = tid; c < nch; c += T) {
            const float4 *xp = reinterpret_cast<const float4 *>(xin + 16 * c);
            const float4 a = xp[0], b = xp[1], cc = xp[2], d = xp[3];
            xs[c] = a;
            xs[nch + c] = b;
            xs[2 * nch + c] = cc;
            xs[3 * nch + c] = d;
            ssq += (a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w) + (b.x * b.x + b.y * b.y + b.z * b.z + b.w * b.w) +
                   (cc.x * cc.x + cc.y * cc.y + cc.z * cc.z + cc.w * cc.w) + (d.x * d.x + d.y * d.y + d.z * d.z + d.w * d.w);
        }
        ssq = block_sum(ssq, red);
        // ss /= size; ss += 1e-5f; ss = 1.0f / sqrt(ss)   (K/RootMeanSquare.java:31-33)
        const float ss = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(__fdiv_rn(ssq, (float)n), 1e-5f)));
        for (int c = tid; c < nch; c += T) {
            const long f = rw.off + 16L * c;
            const float2 mm = rw.mm[f >> 8];
            const float mn = mm.x, range = __fsub_rn(mm.y, mm.x);
            const uint4 codes = *reinterpret_cast<const uint4 *>(rw.codes + f);
            const uint32_t cw[4] = {codes.x, codes.y, codes.z, codes.w};
            float s = 0.0f;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                float4 xv = xs[q * nch + c];
                float *xe = reinterpret_cast<float *>(&xv);
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    // value = byte / 255f * range + min ; out = value * (ss * x)   (K/WeightNormalizeAndScale.java:71-73)
                    const float wv = __fadd_rn(__fmul_rn(__fdiv_rn(ubyte_f(cw[q], b), 255.0f), range), mn);
                    xe[b] = __fmul_rn(wv, __fmul_rn(ss, xe[b]));
                    s += xe[b];
                }
                xs[q * nch + c] = xv;
            }
            sumx[c] = s;
        }
    } else {
        for (int c = tid; c < nch; c += T) {
            const float4 *xp = reinterpret_cast<const float4 *>(xin + 16 * c);
            const float4 a = xp[0], b = xp[1], cc = xp[2], d = xp[3];
            xs[c] = a;
            xs[nch + c] = b;
            xs[2 * nch + c] = cc;
            xs[3 * nch + c] = d;
            sumx[c] = ((a.x + a.y) + (a.z + a.w)) + ((b.x + b.y) + (b.z + b.w)) + ((cc.x + cc.y) + (cc.z + cc.w)) +
                      ((d.x + d.y) + (d.z + d.w));
        }
    }
    __syncthreads();
}

// ------------------------------------------------------------------------------------------
// W8A32 matvec: one wavefront per pair of output rows
// ------------------------------------------------------------------------------------------

struct QMat {
    const uint8_t *codes;  // flat codes of the whole tensor, index = float index in the tensor
    const float2 *gs;      // per group: ((max-min)/255, min)
    long off;              // float offset of this layer's matrix inside the tensor
};

enum { MV_QKV = 0, MV_W13 = 1, MV_RES = 2 };

struct MatvecArgs {
    const float *xin;  // input vector (n floats)
    int n;
    RmsW rms;  // rmsnorm weights (QKV, W13)
    QMat m0, m1, m2;
    int d0, d1, d2;  // rows: QKV (dim, kv_dim, kv_dim); W13 (hidden, hidden, 0); RES (d, 0, 0)
    float *out0;     // QKV: q        W13: hb      RES: x (accumulated in place)
    float *out1;     // QKV: key cache of this layer (seq_len, kv_dim)
    float *out2;     // QKV: value cache of this layer
    const float2 *rope;  // (cos, sin) at [pos * head_size/2 + (i % head_size)/2]
    int head_size, kv_dim;
    const float *silu_table;
    int exact_silu;
    const DevState *st;
};

constexpr int kMvUnroll = 4;

template <int MODE>
__global__ void __launch_bounds__(1024) k_matvec(const MatvecArgs a)
{
    extern __shared__ float4 smem4[];
    const int n = a.n, nch = n >> 4;
    float4 *xs = smem4;
    float *sumx = reinterpret_cast<float *>(smem4 + 4 * nch);
    float *red = sumx + nch;

    stage_vector<MODE != MV_RES>(a.xin, n, a.rms, xs, sumx, red);

    const int lane = threadIdx.x & 63;
    const int wpb = blockDim.x >> 6;
    const int gw = blockIdx.x * wpb + (threadIdx.x >> 6);
    const int total_w = gridDim.x * wpb;
    const int npairs = MODE == MV_QKV ? (a.d0 + a.d1 + a.d2) >> 1 : MODE == MV_W13 ? a.d0 : (a.d0 + 1) >> 1;

    for (int p = gw; p < npairs; p += total_w) {
        const uint8_t *ca, *cb;
        const float2 *ga, *gb;
        long fa, fb;
        int which = 0, r = 0;
        bool has_b = true;
        if (MODE == MV_QKV) {
            r = 2 * p;
            QMat m = a.m0;
            if (r >= a.d0 + a.d1) { which = 2; r -= a.d0 + a.d1; m = a.m2; }
            else if (r >= a.d0) { which = 1; r -= a.d0; m = a.m1; }
            ca = cb = m.codes; ga = gb = m.gs;
            fa = m.off + (long)r * n; fb = fa + n;
        } else if (MODE == MV_W13) {
            r = p;
            ca = a.m0.codes; ga = a.m0.gs; fa = a.m0.off + (long)r * n;
            cb = a.m1.codes; gb = a.m1.gs; fb = a.m1.off + (long)r * n;
        } else {
            r = 2 * p;
            has_b = r + 1 < a.d0;
            ca = cb = a.m0.codes; ga = gb = a.m0.gs;
            fa = a.m0.off + (long)r * n; fb = has_b ? fa + n : fa;
        }

        float accA = 0.0f, accB = 0.0f;
        for (int c0 = lane; c0 < nch; c0 += 64 * kMvUnroll) {
            uint4 wa[kMvUnroll], wb[kMvUnroll];
            float2 sa[kMvUnroll], sb[kMvUnroll];
            int cc[kMvUnroll];
            bool ok[kMvUnroll];
#pragma unroll
            for (int u = 0; u < kMvUnroll; u++) {
                const int c = c0 + 64 * u;
                ok[u] = c < nch;
                cc[u] = ok[u] ? c : c0;
                const long ia = fa + 16L * cc[u], ib = fb + 16L * cc[u];
                wa[u] = *reinterpret_cast<const uint4 *>(ca + ia);
                wb[u] = *reinterpret_cast<const uint4 *>(cb + ib);
                sa[u] = ga[ia >> 8];
                sb[u] = gb[ib >> 8];
            }
#pragma unroll
            for (int u = 0; u < kMvUnroll; u++) {
                const float4 x0 = xs[cc[u]], x1 = xs[nch + cc[u]], x2 = xs[2 * nch + cc[u]], x3 = xs[3 * nch + cc[u]];
                const float sx = sumx[cc[u]];
                const float da = dot16(wa[u], x0, x1, x2, x3);
                const float db = dot16(wb[u], x0, x1, x2, x3);
                // sum (c*rm + min)*x = rm * sum c*x + min * sum x over the chunk
                const float ta = fmaf(sa[u].x, da, sa[u].y * sx);
                const float tb = fmaf(sb[u].x, db, sb[u].y * sx);
                accA += ok[u] ? ta : 0.0f;
                accB += ok[u] ? tb : 0.0f;
            }
        }
        accA = wave_sum(accA);
        accB = wave_sum(accB);

        if (lane == 0) {
            if (MODE == MV_QKV) {
                const int pos = a.st->pos;
                float v0 = accA, v1 = accB;
                if (which < 2) {
                    // RoPE on the interleaved pair (r, r+1)  (K/ApplyRope.java:74-90)
                    const float2 cs = a.rope[(long)pos * (a.head_size >> 1) + ((r % a.head_size) >> 1)];
                    v0 = __fsub_rn(__fmul_rn(accA, cs.x), __fmul_rn(accB, cs.y));
                    v1 = __fadd_rn(__fmul_rn(accA, cs.y), __fmul_rn(accB, cs.x));
                }
                float *dst = which == 0 ? a.out0 + r : (which == 1 ? a.out1 : a.out2) + (long)pos * a.kv_dim + r;
                dst[0] = v0;
                dst[1] = v1;
            } else if (MODE == MV_W13) {
                // hb[i] = hb[i] * (sigma(hb[i]) * hb2[i])   (K/Silu.java:72-74)
                const float s = silu_sigma(a.silu_table, accA, a.exact_silu);
                a.out0[r] = __fmul_rn(accA, __fmul_rn(s, accB));
            } else {
                a.out0[r] = __fadd_rn(a.out0[r], accA);  // residual (K/Accum.java:26-30)
                if (has_b) a.out0[r + 1] = __fadd_rn(a.out0[r + 1], accB);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// decode attention: split over the sequence, last split to finish combines
// ------------------------------------------------------------------------------------------

struct AttnArgs {
    const float *q;        // (n_heads * head_size) after RoPE
    const float *kc;       // this layer's key cache (seq_len, kv_dim)
    const float *vc;       // this layer's value cache
    float *out;            // xb (dim)
    float *part;           // (n_heads, nsplit, head_size + 2) partial (max, sum, acc)
    unsigned *counters;    // (n_heads) arrival counters, zero between launches
    const DevState *st;
    int n_heads, kv_mul, head_size, kv_dim, nsplit, chunk_max;
    float sqrt_hs;
};

constexpr int kAttnThreads = 256;
constexpr int kAttnUnroll = 4;
constexpr int kAttnMinChunk = 8;

// LPR = lanes per cache row: each lane owns 4 consecutive floats of the head (head_size <= 4*LPR).
template <int LPR>
__global__ void __launch_bounds__(kAttnThreads) k_attention(const AttnArgs a)
{
    extern __shared__ float smem[];
    constexpr int RPW = 64 / LPR;                   // rows per wave per load
    constexpr int NW = kAttnThreads / 64;
    constexpr int RPI = RPW * NW;                   // rows per block per load
    float *sc = smem;                               // chunk_max scores / probabilities
    float *red = sc + a.chunk_max;                  // NW
    float *accs = red + NW;                         // NW * head_size
    __shared__ int s_last;

    const int hs = a.head_size;
    const int h = blockIdx.x / a.nsplit, s = blockIdx.x % a.nsplit;
    const int len = a.st->pos + 1;
    int chunk = (len + a.nsplit - 1) / a.nsplit;
    if (chunk < kAttnMinChunk) chunk = kAttnMinChunk;
    const int nact = (len + chunk - 1) / chunk;
    if (s >= nact) return;
    const int t0 = s * chunk;
    const int cnt = min(chunk, len - t0);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int j = lane % LPR;           // which 4 floats of the head
    const int rs = wave * RPW + lane / LPR;  // row slot inside one block-wide load
    const bool active = 4 * j < hs;
    const long col = (long)(h / a.kv_mul) * hs + 4 * j;

    float4 q4 = make_float4(0.f, 0.f, 0.f, 0.f);
    if (active) q4 = *reinterpret_cast<const float4 *>(a.q + h * hs + 4 * j);

    // ---- scores: att[t] = (q . k_t) / sqrt(head_size)     (K/AttentionLoop.java:36-48)
    for (int tb = 0; tb < cnt; tb += RPI * kAttnUnroll) {
        float4 k4[kAttnUnroll];
        bool ok[kAttnUnroll];
#pragma unroll
        for (int u = 0; u < kAttnUnroll; u++) {
            const int tl = tb + u * RPI + rs;
            ok[u] = tl < cnt;
            k4[u] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (ok[u] && active) k4[u] = *reinterpret_cast<const float4 *>(a.kc + (long)(t0 + tl) * a.kv_dim + col);
        }
#pragma unroll
        for (int u = 0; u < kAttnUnroll; u++) {
            const float d = group_sum<LPR>(dot4(q4, k4[u]));
            if (ok[u] && j == 0) sc[tb + u * RPI + rs] = __fdiv_rn(d, a.sqrt_hs);
        }
    }
    __syncthreads();

    // ---- softmax numerators over this split, shifted by the split's true maximum
    // (the reference shifts by a running maximum of element products, K/AttentionLoop.java:44-51;
    //  softmax is shift invariant, so only rounding differs)
    float m = -3.402823466e+38f;
    for (int t = tid; t < cnt; t += kAttnThreads) m = fmaxf(m, sc[t]);
    m = block_max(m, red);
    float l = 0.0f;
    for (int t = tid; t < cnt; t += kAttnThreads) {
        const float e = expf(sc[t] - m);
        sc[t] = e;
        l += e;
    }
    l = block_sum(l, red);  // barriers inside make sc visible

    // ---- weighted values                                   (K/AccumWeightedValue.java:48-62)
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int tb = 0; tb < cnt; tb += RPI * kAttnUnroll) {
        float4 v4[kAttnUnroll];
        float pw[kAttnUnroll];
#pragma unroll
        for (int u = 0; u < kAttnUnroll; u++) {
            const int tl = tb + u * RPI + rs;
            const bool ok = tl < cnt;
            v4[u] = make_float4(0.f, 0.f, 0.f, 0.f);
            pw[u] = ok ? sc[tl] : 0.0f;
            if (ok && active) v4[u] = *reinterpret_cast<const float4 *>(a.vc + (long)(t0 + tl) * a.kv_dim + col);
        }
#pragma unroll
        for (int u = 0; u < kAttnUnroll; u++) {
            acc.x = fmaf(pw[u], v4[u].x, acc.x);
            acc.y = fmaf(pw[u], v4[u].y, acc.y);
            acc.z = fmaf(pw[u], v4[u].z, acc.z);
            acc.w = fmaf(pw[u], v4[u].w, acc.w);
        }
    }
    // fold the row slots of a wave (lanes with equal j), then the waves
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1) {
        acc.x += __shfl_xor(acc.x, off);
        acc.y += __shfl_xor(acc.y, off);
        acc.z += __shfl_xor(acc.z, off);
        acc.w += __shfl_xor(acc.w, off);
    }
    if (lane < LPR && active) *reinterpret_cast<float4 *>(accs + wave * hs + 4 * j) = acc;
    __syncthreads();

    float total = 0.0f;
    if (tid < hs) {
        for (int w = 0; w < NW; w++) total += accs[w * hs + tid];
    }
    if (nact == 1) {
        if (tid < hs) a.out[h * hs + tid] = __fdiv_rn(total, l);
        return;
    }

    float *mypart = a.part + ((long)h * a.nsplit + s) * (hs + 2);
    if (tid < hs) mypart[2 + tid] = total;
    if (tid == 0) { mypart[0] = m; mypart[1] = l; }
    __threadfence();
    __syncthreads();
    if (tid == 0) s_last = (atomicAdd(a.counters + h, 1u) == (unsigned)(nact - 1));
    __syncthreads();
    if (!s_last) return;
    __threadfence();
    // fixed combine order (split 0, 1, ...) whichever block arrives last: deterministic
    const float *hp = a.part + (long)h * a.nsplit * (hs + 2);
    float M = -3.402823466e+38f;
    for (int i = 0; i < nact; i++) M = fmaxf(M, hp[(long)i * (hs + 2)]);
    if (tid < hs) {
        float L = 0.0f, o = 0.0f;
        for (int i = 0; i < nact; i++) {
            const float *pp = hp + (long)i * (hs + 2);
            const float w = expf(pp[0] - M);
            L = fmaf(pp[1], w, L);
            o = fmaf(pp[2 + tid], w, o);
        }
        a.out[h * hs + tid] = __fdiv_rn(o, L);
    }
    if (tid == 0) a.counters[h] = 0u;
}

// ------------------------------------------------------------------------------------------
// final rmsnorm + fp32 classifier + first-max argmax + token-loop state update
// ------------------------------------------------------------------------------------------

struct ClsArgs {
    const float *xin;  // residual stream
    int n;             // dim
    RmsW rms;          // rms_final_weight
    const float *w;    // (vocab, dim) fp32
    int vocab;
    float *logits;
    float *part_val;   // gridDim.x
    int *part_idx;     // gridDim.x
    unsigned *counter; // 1, zero between launches
    DevState *st;
    const int *prompt; // seq_len
    int *out_tokens;   // seq_len
};

constexpr int kClsUnroll = 8;

__device__ __forceinline__ bool better(float v, int i, float bv, int bi) { return v > bv || (v == bv && i < bi); }

__global__ void __launch_bounds__(1024) k_classifier(const ClsArgs a)
{
    extern __shared__ float4 smem4[];
    const int n = a.n, nch = n >> 4, n4 = n >> 2;
    float4 *xs = smem4;
    float *sumx = reinterpret_cast<float *>(smem4 + 4 * nch);
    float *red = sumx + nch;            // 16 floats used by the staging reduction
    float *bval = red + 16;             // per wave best value
    int *bidx = reinterpret_cast<int *>(bval + 16);
    __shared__ int s_last;

    stage_vector<true>(a.xin, n, a.rms, xs, sumx, red);

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wpb = blockDim.x >> 6;
    const int gw = blockIdx.x * wpb + wave;
    const int total_w = gridDim.x * wpb;
    const int npairs = (a.vocab + 1) >> 1;

    float best_v = -__builtin_inff();
    int best_i = 0x7fffffff;
    for (int p = gw; p < npairs; p += total_w) {
        const int r = 2 * p;
        const bool has_b = r + 1 < a.vocab;
        const float4 *wa = reinterpret_cast<const float4 *>(a.w + (long)r * n);
        const float4 *wb = has_b ? wa + n4 : wa;
        float accA = 0.0f, accB = 0.0f;
        for (int c0 = lane; c0 < n4; c0 += 64 * kClsUnroll) {
            float4 ra[kClsUnroll], rb[kClsUnroll];
            int cc[kClsUnroll];
            bool ok[kClsUnroll];
#pragma unroll
            for (int u = 0; u < kClsUnroll; u++) {
                const int c = c0 + 64 * u;
                ok[u] = c < n4;
                cc[u] = ok[u] ? c : c0;
                ra[u] = load_stream(wa + cc[u]);
                rb[u] = load_stream(wb + cc[u]);
            }
#pragma unroll
            for (int u = 0; u < kClsUnroll; u++) {
                const float4 xv = xs[(cc[u] & 3) * nch + (cc[u] >> 2)];
                const float ta = dot4(ra[u], xv), tb = dot4(rb[u], xv);
                accA += ok[u] ? ta : 0.0f;
                accB += ok[u] ? tb : 0.0f;
            }
        }
        accA = wave_sum(accA);
        accB = wave_sum(accB);
        if (lane == 0) {
            a.logits[r] = accA;
            if (better(accA, r, best_v, best_i)) { best_v = accA; best_i = r; }
            if (has_b) {
                a.logits[r + 1] = accB;
                if (better(accB, r + 1, best_v, best_i)) { best_v = accB; best_i = r + 1; }
            }
        }
    }
    if (lane == 0) { bval[wave] = best_v; bidx[wave] = best_i; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < wpb; w++)
            if (better(bval[w], bidx[w], best_v, best_i)) { best_v = bval[w]; best_i = bidx[w]; }
        a.part_val[blockIdx.x] = best_v;
        a.part_idx[blockIdx.x] = best_i;
        __threadfence();
        s_last = (atomicAdd(a.counter, 1u) == gridDim.x - 1);
    }
    __syncthreads();
    if (!s_last || threadIdx.x != 0) return;
    __threadfence();
    // first index of the strict maximum (J/Sampler.java:46-57): ties resolve to the lower index
    best_v = -__builtin_inff();
    best_i = 0x7fffffff;
    for (unsigned b = 0; b < gridDim.x; b++) {
        const float v = a.part_val[b];
        const int i = a.part_idx[b];
        if (better(v, i, best_v, best_i)) { best_v = v; best_i = i; }
    }
    if (best_i == 0x7fffffff) best_i = 0;  // all NaN: the reference's scan never leaves index 0
    // token loop step (J/Run.java:635-642, 668, 680): forced prompt id or argmax, then advance
    const int pos = a.st->pos;
    const int next = pos < a.st->n_prompt ? a.prompt[pos] : best_i;
    a.out_tokens[pos] = next;
    a.st->token = next;
    a.st->pos = pos + 1;
    *a.counter = 0u;
}

// x = token_embedding_table[token]   (J/Run.java:72)
__global__ void k_embed(const float *__restrict__ emb, const DevState *st, float *__restrict__ x, int dim)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < (dim >> 2))
        reinterpret_cast<float4 *>(x)[i] = reinterpret_cast<const float4 *>(emb + (long)st->token * dim)[i];
}

// ------------------------------------------------------------------------------------------
// load path: reference bytes <-> device layout, encoder, seeded tensors
// ------------------------------------------------------------------------------------------

__device__ __forceinline__ float be_bits_to_float(uint32_t le_loaded) { return __builtin_bit_cast(float, __builtin_bswap32(le_loaded)); }

// One 64-thread block per group: 264 reference bytes -> 256 codes + (rm, min) + (min, max).
__global__ void __launch_bounds__(64) k_unpack_groups(const uint8_t *__restrict__ ref, long ngroups, uint8_t *__restrict__ codes,
                                                      float2 *__restrict__ gs, float2 *__restrict__ mm)
{
    for (long g = blockIdx.x; g < ngroups; g += gridDim.x) {
        const uint32_t *src = reinterpret_cast<const uint32_t *>(ref + g * kGroupBytes);
        reinterpret_cast<uint32_t *>(codes + g * kGroup)[threadIdx.x] = src[2 + threadIdx.x];
        if (threadIdx.x == 0) {
            const float mn = be_bits_to_float(src[0]), mx = be_bits_to_float(src[1]);
            gs[g] = make_float2(__fdiv_rn(__fsub_rn(mx, mn), 255.0f), mn);  // K/MatMul.java:137-139
            mm[g] = make_float2(mn, mx);
        }
    }
}

__global__ void __launch_bounds__(64) k_pack_groups(uint8_t *__restrict__ ref, long ngroups, const uint8_t *__restrict__ codes,
                                                    const float2 *__restrict__ mm)
{
    for (long g = blockIdx.x; g < ngroups; g += gridDim.x) {
        uint32_t *dst = reinterpret_cast<uint32_t *>(ref + g * kGroupBytes);
        dst[2 + threadIdx.x] = reinterpret_cast<const uint32_t *>(codes + g * kGroup)[threadIdx.x];
        if (threadIdx.x == 0) {
            const float2 v = mm[g];
            dst[0] = __builtin_bswap32(__builtin_bit_cast(uint32_t, v.x));
            dst[1] = __builtin_bswap32(__builtin_bit_cast(uint32_t, v.y));
        }
    }
}

__device__ __forceinline__ uint64_t splitmix64(uint64_t z)
{
    z += 0x9E3779B97F4A7C15ULL;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

__device__ __forceinline__ float synth_value(uint64_t base, long i, float scale)
{
    const uint64_t r = splitmix64(base + (uint64_t)i);
    const int s = (int)(r & 0xFFFF) + (int)((r >> 16) & 0xFFFF) + (int)((r >> 32) & 0xFFFF) + (int)(r >> 48) - 131070;
    return __fmul_rn((float)s, scale);
}

__global__ void k_synth_f32(float *__restrict__ out, long n, uint64_t base, float scale)
{
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        out[i] = synth_value(base, i, scale);
}

// Quant.encode (J/Quant.java:156-193), one 256-thread block per group.  Source is either fp32
// data (src != null, float index 0 = first float of group `g0`) or the seeded generator.
__global__ void __launch_bounds__(256) k_encode_groups(const float *__restrict__ src, long n_src, long g0, long ngroups,
                                                       long tensor_floats, uint64_t synth_base, float synth_scale,
                                                       uint8_t *__restrict__ codes, float2 *__restrict__ gs, float2 *__restrict__ mm)
{
    __shared__ float red[8];
    const int t = threadIdx.x;
    for (long gi = blockIdx.x; gi < ngroups; gi += gridDim.x) {
        const long g = g0 + gi;
        const long fi = g * kGroup + t;          // float index in the tensor
        const bool valid = fi < tensor_floats && (src == nullptr || gi * kGroup + t < n_src);
        float v = 0.0f;
        if (valid) v = src ? src[gi * kGroup + t] : synth_value(synth_base, fi, synth_scale);
        // min / max over the valid elements (the reference's scan, J/Quant.java:166-177; NaN weights
        // and the sign of a zero extremum are not distinguished here)
        float lo = valid ? v : __builtin_inff();
        float hi = valid ? v : -__builtin_inff();
        lo = -block_max(-lo, red);
        hi = block_max(hi, red);
        const float range = __fsub_rn(hi, lo);
        int code = 0;
        if (valid) {
            const float s = __fmul_rn(__fdiv_rn(__fsub_rn(v, lo), range), 255.0f);
            if (s == s) {  // NaN (range 0) -> 0, as Math.round
                const float fl = floorf(s);
                code = (int)fl + ((s - fl) >= 0.5f ? 1 : 0);  // floor(s + 1/2) without the rounding of the add
            }
        }
        codes[g * kGroup + t] = (uint8_t)code;
        if (t == 0) {
            gs[g] = make_float2(__fdiv_rn(range, 255.0f), lo);
            mm[g] = make_float2(lo, hi);
        }
        __syncthreads();
    }
}

}  // namespace l2j
