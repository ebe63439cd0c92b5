// gfx950 kernels of the per-token forward pass (W8A32, batch 1).
//
// Shared device helpers (wavefront reductions, streaming loads, the code/activation dot product,
// the reference's sigmoid table) and the kernels of the load path (format conversion, the group-int8
// encoder, seeded tensors).  The forward pass itself is in phase_kernels.hpp.
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
    int epoch;     // tokens since the host last set the state: a whole-token kernel that hands its vectors over by value
                   // alternates between two sets of activation vectors by its parity
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

// Block-wide sum / max through LDS; `red` holds one float per wave (nw waves).  All threads get the result.
__device__ __forceinline__ float block_sum(float v, float *red, int nw)
{
    const int wave = threadIdx.x >> 6;
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

// Two consecutive floats of a read-only table at a wave-uniform address, through the scalar data path: a scalar load
// does not queue behind the wave's outstanding vector loads (weights requested ahead), which return in order.
__device__ __forceinline__ float2 uniform_pair(const float *p)
{
    const unsigned long long a = (unsigned long long)p;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)a), hi = __builtin_amdgcn_readfirstlane((unsigned)(a >> 32));
    const unsigned long long ua = ((unsigned long long)hi << 32) | lo;
    unsigned long long v;
    asm volatile("s_load_dwordx2 %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(ua) : "memory");
    return make_float2(__uint_as_float((unsigned)v), __uint_as_float((unsigned)(v >> 32)));
}

// The reference's sigmoid: 8192-entry table on [-5,5) with linear interpolation and the integer
// index multiplier 819 (K/Silu.java:41-70); exact outside the table.
// UNIFORM: val is the same in every lane (a wave's row sum): the two table entries come through the scalar data path.
template <bool UNIFORM = false>
__device__ __forceinline__ float silu_sigma(const float *__restrict__ table, float val, int exact)
{
    const float position = __fmul_rn(__fadd_rn(val, 5.0f), 819.0f);
    if (!exact && position > 0.0f && position < 8191.0f) {
        const int idx = (int)position;
        float lo, hi;
        if (UNIFORM) {
            const float2 t = uniform_pair(table + idx);
            lo = t.x; hi = t.y;
        } else {
            lo = table[idx]; hi = table[idx + 1];
        }
        return __fadd_rn(lo, __fmul_rn(__fsub_rn(position, (float)idx), __fsub_rn(hi, lo)));
    }
    // outside the table (|val| >= 5, saturated): the reference evaluates this in double and narrows;
    // fp32 differs by at most a couple of ulp
    return __fdiv_rn(1.0f, 1.0f + expf(-val));
}

// ------------------------------------------------------------------------------------------
// shared small types
// ------------------------------------------------------------------------------------------

// One quantized matrix inside its tensor.
struct QMat {
    const uint8_t *codes;  // flat codes of the whole tensor, index = float index in the tensor
    const float2 *gs;      // per group: ((max-min)/255, min)
    long off;              // float offset of this layer's matrix inside the tensor
};

// first-max order: larger value wins, equal values resolve to the lower index (J/Sampler.java:46-57)
__device__ __forceinline__ bool better(float v, int i, float bv, int bi) { return v > bv || (v == bv && i < bi); }

// ------------------------------------------------------------------------------------------
// load path: reference bytes <-> device layout, encoder, seeded tensors
// ------------------------------------------------------------------------------------------

__device__ __forceinline__ float be_bits_to_float(uint32_t le_loaded) { return __builtin_bit_cast(float, __builtin_bswap32(le_loaded)); }

// One 64-thread block per group: 264 reference bytes -> 256 codes + (rm, min) + (min, max).
static __global__ void __launch_bounds__(64) k_unpack_groups(const uint8_t *__restrict__ ref, long ngroups, uint8_t *__restrict__ codes,
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

static __global__ void __launch_bounds__(64) k_pack_groups(uint8_t *__restrict__ ref, long ngroups, const uint8_t *__restrict__ codes,
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

static __global__ void k_synth_f32(float *__restrict__ out, long n, uint64_t base, float scale)
{
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        out[i] = synth_value(base, i, scale);
}

// Quant.encode (J/Quant.java:156-193), one 256-thread block per group.  Source is either fp32
// data (src != null, float index 0 = first float of group `g0`) or the seeded generator.
static __global__ void __launch_bounds__(256) k_encode_groups(const float *__restrict__ src, long n_src, long g0, long ngroups,
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

// Plain copy of n 16-byte words: the known-size kernel against which hardware byte counters are scaled.
static __global__ void __launch_bounds__(256) k_copy16(const uint4 *__restrict__ src, uint4 *__restrict__ dst, long n)
{
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) dst[i] = src[i];
}

}  // namespace l2j
