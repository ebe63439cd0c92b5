// The per-token forward pass (J/Run.java:62-169) on gfx950.  Per layer there are five phases:
//   PH_QKV      rmsnorm + Wq,Wk,Wv matvec + RoPE + KV-cache store
//   attention   decode attention, split over the sequence, online softmax
//   PH_RES/ROW  Wo matvec + residual (row pairs, or one row per wave when rows are long: PH_ROW, PH_ROW6)
//   PH_W13      rmsnorm + W1,W3 matvec + SwiGLU (the reference's sigmoid table)
//   PH_RES/ROW  W2 matvec + residual
// and once per token k_classifier (final rmsnorm + fp32 classifier + per-workgroup first-max) and k_finish
// (fold the maxima, step the token loop state).  k_token runs all phases of a range of layers (by default
// the whole token, classifier included) in one launch, one 1024-thread workgroup per compute unit; each phase
// also exists as a kernel of its own (k_matvec<MODE>, k_attention, k_classifier) for per-layer taps, per-phase
// timing and small models.  The launches of a token are captured once in a hipGraph and replayed.
//
// Every phase is HBM-bandwidth bound (batch-1 GEMV: no reuse, so no MFMA): int8 codes are streamed
// with 16-byte nontemporal loads, one wavefront per pair of sub-rows, the activation vector is staged
// in LDS once per workgroup, accumulation is fp32 and the 64-lane reduction uses DPP.  All arguments are
// passed by value so that every pointer is a kernel argument (global address space, scalar base + 32-bit
// lane offset addressing).
//
// Inside k_token a vector passes from one phase to the next without cache maintenance: producers store it
// with device-scope relaxed atomics (write-through) and every activation vector of a token has a
// cache-line-aligned address of its own that nothing reads before its producer has finished.  Consumers
// either wait for the data itself (the vectors are pre-filled with a NaN pattern and re-read with
// device-coherent loads until it is gone) or, after a grid barrier of relaxed counters, use plain loads.
// In both cases the first weights of the next phase are requested before the wait, so HBM stays busy while
// the slowest workgroups finish the phase.
//
// The weight registers of the waves are the only buffer between the phases, so when and by whom they are filled
// decides how busy the memory system stays: a wave requests the first step of its next phase as soon as its own
// items are done (before the workgroup's barrier); while it folds a step it requests the next one chunk by chunk
// (two vector instructions per weight are a fifth of a layer's time and would otherwise leave gaps); waves without
// a Wo item lend their registers to their first W13 item during the attention and Wo phases; W2's long rows are
// held whole (PH_ROW6), two thirds requested ahead of the hand-over.
//
// A wave holds TU 16-byte chunks per lane and sub-row (64 * TU chunks = one step).  Four fit the 7B shape (rows of
// 256 chunks); the kernels are also instantiated with one, two and five chunks for the rows of the small models
// (18..128 chunks) and of the 13B shape (320 chunks), so that a row is one full step there too (tu_for).
#pragma once

#include "kernels.hpp"

namespace l2j {

__device__ __forceinline__ float ld_coh(const float *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_coh(float *p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ int ld_coh(const int *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_coh(int *p, int v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_coh(unsigned *p, unsigned v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

__device__ __forceinline__ unsigned long long ld_coh(const unsigned long long *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_coh(unsigned long long *p, unsigned long long v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// ---- hand-over by value ---------------------------------------------------------------------------------
// Instead of a barrier, a consumer can wait for the data itself: before a token every activation vector is
// filled with kUnset (a NaN bit pattern no computation produces), producers overwrite it with write-through
// stores, and consumers re-read their part of the vector with device-coherent 16-byte loads until no kUnset
// word is left.  The wait is bounded like the barrier's.
constexpr unsigned kUnset = 0x7FC0DEADu;
constexpr unsigned long long kUnset64 = 0x7FC0DEAD7FC0DEADull;

// A workgroup's classifier result, (index, value) in one 64-bit word so that it is stored and read whole.
__device__ __forceinline__ unsigned long long pack_max(float v, int i) { return ((unsigned long long)(unsigned)i << 32) | __float_as_uint(v); }
__device__ __forceinline__ float max_val(unsigned long long w) { return __uint_as_float((unsigned)w); }
__device__ __forceinline__ int max_idx(unsigned long long w) { return (int)(unsigned)(w >> 32); }

__device__ __forceinline__ float4 ld_coh16(const float *p)
{
    float4 v;
    // (the wait is part of the statement: the compiler does not count this load)
    asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    return v;
}

__device__ __forceinline__ bool all_set(const float4 &v)
{
    return __float_as_uint(v.x) != kUnset && __float_as_uint(v.y) != kUnset && __float_as_uint(v.z) != kUnset &&
           __float_as_uint(v.w) != kUnset;
}

struct Poll {
    int on;       // 1: wait for the data itself (k_token without barriers); 0: plain loads
    int maxspin;
    int *fault;
};

// The 16-byte word at p once its producers have written all of it.
__device__ __forceinline__ float4 wait_word(const float *p, const Poll &pl)
{
    float4 v = ld_coh16(p);
    int spins = 0;
    while (!all_set(v)) {
        if (++spins > pl.maxspin || ((spins & 63) == 0 && ld_coh(pl.fault) != 0)) { st_coh(pl.fault, 1); break; }
        __builtin_amdgcn_s_sleep(4);
        v = ld_coh16(p);
    }
    return v;
}

__device__ __forceinline__ float wait_float(const float *p, const Poll &pl)
{
    float v = ld_coh(p);
    int spins = 0;
    while (__float_as_uint(v) == kUnset) {
        if (++spins > pl.maxspin || ((spins & 63) == 0 && ld_coh(pl.fault) != 0)) { st_coh(pl.fault, 1); break; }
        __builtin_amdgcn_s_sleep(4);
        v = ld_coh(p);
    }
    return v;
}

// Several 16-byte words at once: all are requested before the one wait, so the words cost one trip to memory
// together instead of one each.  (Loads and wait are one asm statement: the compiler must not touch the
// destination registers in between.)  Words that are still unset are requested again, with the others: a few
// redundant loads are cheaper than divergent bookkeeping.
__device__ __forceinline__ void load_words(const float *const (&p)[3], float4 (&v)[3])
{
    asm volatile("global_load_dwordx4 %0, %3, off sc1\n\tglobal_load_dwordx4 %1, %4, off sc1\n\t"
                 "global_load_dwordx4 %2, %5, off sc1\n\ts_waitcnt vmcnt(0)"
                 : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]) : "v"(p[0]), "v"(p[1]), "v"(p[2]) : "memory");
}

// Four 8-byte and four 4-byte device-coherent loads at byte offsets from one uniform base, one wait.
__device__ __forceinline__ void load4x2_coh(const float *base, const unsigned (&off2)[4], float2 (&v2)[4], const unsigned (&off1)[4],
                                            float (&v1)[4])
{
    asm volatile("global_load_dwordx2 %0, %8, %16 sc1\n\tglobal_load_dwordx2 %1, %9, %16 sc1\n\t"
                 "global_load_dwordx2 %2, %10, %16 sc1\n\tglobal_load_dwordx2 %3, %11, %16 sc1\n\t"
                 "global_load_dword %4, %12, %16 sc1\n\tglobal_load_dword %5, %13, %16 sc1\n\t"
                 "global_load_dword %6, %14, %16 sc1\n\tglobal_load_dword %7, %15, %16 sc1\n\ts_waitcnt vmcnt(0)"
                 : "=&v"(v2[0]), "=&v"(v2[1]), "=&v"(v2[2]), "=&v"(v2[3]), "=&v"(v1[0]), "=&v"(v1[1]), "=&v"(v1[2]), "=&v"(v1[3])
                 : "v"(off2[0]), "v"(off2[1]), "v"(off2[2]), "v"(off2[3]), "v"(off1[0]), "v"(off1[1]), "v"(off1[2]), "v"(off1[3]), "s"(base)
                 : "memory");
}

template <int N>
__device__ __forceinline__ void wait_words(const float *const (&p)[N], float4 (&v)[N], const Poll &pl)
{
    int spins = 0;
    while (true) {
        load_words(p, v);
        bool ok = true;
#pragma unroll
        for (int i = 0; i < N; i++) ok = ok && all_set(v[i]);
        if (ok) break;
        if (++spins > pl.maxspin || ((spins & 63) == 0 && ld_coh(pl.fault) != 0)) { st_coh(pl.fault, 1); break; }
        __builtin_amdgcn_s_sleep(4);
    }
}

// ---- grid barrier ------------------------------------------------------------------------------------
// Two levels of relaxed device-scope counters: a workgroup bumps the counter of its group (blockIdx % ngroups),
// the last of a group bumps the top counter, everybody polls the top counter.  Every barrier instance of a
// token has counters of its own (zeroed by k_finish), each on its own 256-byte line.  All workgroups of the
// grid must be resident (one per compute unit).  The wait is bounded: when it runs out *fault is set, the
// remaining barriers fall through and the host reports the token as failed.
struct GridBar {
    unsigned *ctr;   // instance i: top counter at ctr[i * kBarStride], group g at ctr[i * kBarStride + 64 * (1 + g)]
    int *fault;
    int ngroups, maxspin;
};
constexpr int kBarGroups = 4;   // measured: 4 groups of 64 beat 8 of 32 and 2 of 128 at 256 workgroups
constexpr int kBarStride = 64 * (1 + kBarGroups);  // unsigned words per barrier instance

// Called when every store of the workgroup that the other workgroups will read has been acknowledged
// (s_waitcnt vmcnt(0) in the storing waves, then a workgroup barrier if thread 0 is not the only one).
__device__ __forceinline__ void bar_arrive(const GridBar &b, int inst)
{
    if (threadIdx.x == 0) {
        unsigned *base = b.ctr + (long)inst * kBarStride;
        const unsigned g = blockIdx.x % (unsigned)b.ngroups;
        const unsigned gsize = (gridDim.x - g + b.ngroups - 1) / b.ngroups;
        const unsigned old = __hip_atomic_fetch_add(base + 64 * (1 + g), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (old + 1u == gsize) __hip_atomic_fetch_add(base, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

__device__ __forceinline__ void bar_wait(const GridBar &b, int inst)
{
    if (threadIdx.x == 0) {
        const unsigned *top = b.ctr + (long)inst * kBarStride;
        const unsigned want = min((unsigned)b.ngroups, gridDim.x);
        int spins = 0;
        while (__hip_atomic_load(top, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < want) {
            __builtin_amdgcn_s_sleep(1);
            if (++spins > b.maxspin || ((spins & 255) == 0 && ld_coh(b.fault) != 0)) {
                st_coh(b.fault, 1);
                break;
            }
        }
    }
    __syncthreads();
}

// The thread index as the phases see it.  It goes through an empty asm so that, inside k_token's layer loop,
// the compiler cannot hoist every phase's lane-dependent addresses and predicates out of the loop and keep
// them all live in vector registers (which spills).
__device__ __forceinline__ int phase_tid()
{
    int t = threadIdx.x;
    asm volatile("" : "+v"(t));
    return t;
}

enum { PH_QKV = 0, PH_W13 = 1, PH_RES = 2, PH_ROW = 3, PH_ROW6 = 4 };  // PH_RES: row pairs + residual; PH_ROW, PH_ROW6: one row per wave + residual

// One matvec phase.  Passed by value.
struct MatvecPhase {
    int n;          // input vector length (multiple of 16)
    int from_emb;   // the input vector is the embedding row of the current token (QKV of layer 0)
    int res_emb;    // PH_RES / PH_ROW: the residual input is the embedding row of the current token (Wo of layer 0)
    int d0, d1, d2; // rows: QKV (dim, kv_dim, kv_dim); W13 (hidden); RES (dim)
    const float *xin;   // input vector (ignored when from_emb)
    const float *rmsw;  // dequantized rmsnorm weights (fp32) or null: input = rmsw[e] * (ss * x[e])
    QMat m0, m1, m2;
    float *out0, *out1, *out2;  // QKV: q, key cache of the layer, value cache of the layer; W13: hb; RES: x
    const float *res_src;       // PH_RES: residual input (ignored when res_emb)
    const float *emb;           // token embedding table
    const float2 *rope;         // (cos, sin) at [pos * head_size/2 + (i % head_size)/2]
    const float *silu;          // sigmoid table
    const DevState *st;
    int head_size, kv_dim, exact_silu;
    int threads;    // workgroup size (a kernel argument: reading it from the dispatch costs a vector load per phase)
    Poll poll;      // how the input vector and the residual are read
    float *knew, *vnew;  // QKV with poll.on: this token's k and v rows once more, where attention waits for them
};

// ---- activation vector -> LDS ------------------------------------------------------------------
// LDS layout for an n-float vector (nch = n/16 chunks): float4 xs[q*nch + c] holds x[16c+4q .. 16c+4q+3],
// so that lane c of a wave reads consecutive 16-byte words for a fixed q (bank-conflict free);
// sumx[c] = sum of the 16 activations of chunk c (for the group-minimum term of the dequantization).

// The rmsnorm scalar is not applied to the staged vector: sum_e w_e * (g_e * (ss * x_e)) = ss * sum_e w_e * (g_e * x_e), so
// the vector is staged as g_e * x_e as its words arrive, the waves leave their sums of squares in `red`, and the one
// workgroup barrier that publishes the vector publishes them too; the caller multiplies its row sums by the returned
// ss = 1 / sqrt(sum x^2 / n + 1e-5) (K/RootMeanSquare.java:31-33).  The block-wide reduction and its two barriers are
// thereby off the path between the arrival of the input and the first multiply-add (only rounding differs from
// K/WeightNormalizeAndScale.java:73, by a few 1e-7 of a result).  Returns 1 without rmsnorm weights.
__device__ __forceinline__ float rms_scalar(const float *red, int nw, int n)
{
    // the waves' sums, one per lane of a row of sixteen, added across the row (at most 16 waves)
    const int w = phase_tid() & 15;
    const float ssq = row16_sum(w < nw ? red[w] : 0.0f);
    // ss /= size; ss += 1e-5f; ss = 1.0f / sqrt(ss)   (K/RootMeanSquare.java:31-33)
    const float ss = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(__fdiv_rn(ssq, (float)n), 1e-5f)));
    return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, ss)));  // uniform: a scalar register
}

__device__ __forceinline__ float stage_vector(const float *__restrict__ xin, int n, const float *__restrict__ rmsw, float4 *xs,
                                              float *sumx, float *red, int T)
{
    const int nch = n >> 4, tid = phase_tid();
    float ssq = 0.0f;
    for (int c = tid; c < nch; c += T) {
        const float4 *xp = reinterpret_cast<const float4 *>(xin + 16 * c);
        float4 v[4] = {xp[0], xp[1], xp[2], xp[3]};
        float s = 0.0f;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            ssq += (v[q].x * v[q].x + v[q].y * v[q].y) + (v[q].z * v[q].z + v[q].w * v[q].w);
            if (rmsw) {
                const float4 wv = reinterpret_cast<const float4 *>(rmsw + 16 * c)[q];
                v[q].x = __fmul_rn(wv.x, v[q].x);
                v[q].y = __fmul_rn(wv.y, v[q].y);
                v[q].z = __fmul_rn(wv.z, v[q].z);
                v[q].w = __fmul_rn(wv.w, v[q].w);
            }
            s += (v[q].x + v[q].y) + (v[q].z + v[q].w);
            xs[q * nch + c] = v[q];
        }
        sumx[c] = s;
    }
    if (rmsw) {
        ssq = wave_sum(ssq);
        if ((tid & 63) == 0) red[tid >> 6] = ssq;
    }
    __syncthreads();
    return rmsw ? rms_scalar(red, T >> 6, n) : 1.0f;
}

// The same with the vector read word by word as soon as its producers have written it (hand-over by value).
// Thread t takes the 16-byte words t, t+T, ...; the four lanes of a quad hold the four words of a chunk.
// (Letting a few waves stage the vector and request their weights afterwards, so that the vector is not queued
// behind them, was slower: 1.96 against 1.76 ms per 7B token.)
// WORDS = 16-byte words per thread: n <= 4 * WORDS * T (8 words spill registers in k_token)
constexpr int kPollWords = 4;

template <int WORDS>
__device__ __forceinline__ float stage_vector_poll(const float *__restrict__ xin, int n, const float *__restrict__ rmsw, float4 *xs,
                                                   float *sumx, float *red, int T, const Poll &pl)
{
    const int nch = n >> 4, nq = n >> 2, tid = phase_tid();
    const int S = T;  // n <= 4 * WORDS * T is checked on the host
    float ssq = 0.0f;
#pragma unroll
    for (int k = 0; k < WORDS; k++) {
        const int i = tid + k * S;
        float4 xv = make_float4(0.f, 0.f, 0.f, 0.f);
        if (i < nq) {
            float4 wv = make_float4(1.f, 1.f, 1.f, 1.f);
            if (rmsw) wv = reinterpret_cast<const float4 *>(rmsw)[i];
            xv = wait_word(xin + 4 * i, pl);
            ssq += (xv.x * xv.x + xv.y * xv.y) + (xv.z * xv.z + xv.w * xv.w);
            if (rmsw) {
                xv.x = __fmul_rn(wv.x, xv.x);
                xv.y = __fmul_rn(wv.y, xv.y);
                xv.z = __fmul_rn(wv.z, xv.z);
                xv.w = __fmul_rn(wv.w, xv.w);
            }
        }
        const float s0 = (xv.x + xv.y) + (xv.z + xv.w);
        const float s1 = dpp_f<0x55>(s0), s2 = dpp_f<0xAA>(s0), s3 = dpp_f<0xFF>(s0);  // quad lanes 1, 2, 3
        if (i < nq) {
            xs[(i & 3) * nch + (i >> 2)] = xv;
            if ((i & 3) == 0) sumx[i >> 2] = ((s0 + s1) + s2) + s3;
        }
    }
    if (rmsw) {
        ssq = wave_sum(ssq);
        if ((tid & 63) == 0) red[tid >> 6] = ssq;
    }
    __syncthreads();
    return rmsw ? rms_scalar(red, T >> 6, n) : 1.0f;
}

// The number of splits per head the attention phase uses at a position, and the rows of each.
__device__ __forceinline__ int attn_splits_at(int len, int rows_per_split, int max_splits, int &chunk)
{
    int nsplit = (len + rows_per_split - 1) / rows_per_split;  // short contexts: fewer, fuller splits
    if (nsplit > max_splits) nsplit = max_splits;
    chunk = (len + nsplit - 1) / nsplit;
    return (len + chunk - 1) / chunk;
}

// ---- W8A32 matvec: an item is a pair of rows, one wavefront per item ---------------------------------

constexpr int kTU = 4;  // 16-byte chunks in flight per lane per sub-row

// One matvec phase of one workgroup: preload() requests the first weights (they do not depend on the input
// vector), run() stages the vector and streams the items.  (Two items in flight per wave with 512-thread
// workgroups, so that a wave may use 256 registers, was measured: 1.82 against 1.78 ms per 7B token.)
// TU_ = 16-byte chunks per lane and sub-row that a wave holds at a time (64 * TU_ chunks are one step of a sub-row):
// rows of up to 64 * TU_ chunks are one step, and a phase whose rows are shorter than its step folds empty chunks.
// FAST (row pairs whose rows are exactly one step: n == 16 * 64 * TU codes): no lane ever falls outside a row, so fold()
// neither clamps nor masks and reads the staged vector at constant distances from one per-lane address: 20 vector
// instructions fewer per step of 380 (7B shape: 13 us per token).  The requests keep their general form: with the scale
// loads issued from a scalar base at constant offsets the token took 35 us longer, without the clamps 2 us longer.
template <int MODE, int TU_ = (MODE == PH_ROW6 ? 6 : kTU), bool FAST = false>
struct MatvecRun {
    static_assert(!FAST || (MODE != PH_ROW && MODE != PH_ROW6), "whole-step streaming is for row pairs");
    // PH_ROW streams one row with 2*kTU chunks in flight: "sub-row 1" is the same row kTU*64 chunks further on.
    // PH_ROW6 holds six chunks per lane and sub-row instead of four: a row of 513..768 chunks (11008 codes are 688) is
    // then one step, requested whole ahead of the hand-over, where PH_ROW would request its tail only after the first
    // step (1.72 -> 1.70 ms per 7B token; for shorter or longer rows the extra registers and masked loads cost more
    // than they gain: 3.24 -> 3.60 ms per 13B token).
    static constexpr bool kRow = MODE == PH_ROW || MODE == PH_ROW6;
    static constexpr int TU = TU_;
    static constexpr int kStep = kRow ? 2 * 64 * TU : 64 * TU;
    static constexpr int kOff1 = kRow ? 64 * TU : 0;
    // Runners with more than kTU chunks request only kAhead of them ahead of the hand-over and the others once the input
    // vector is staged: the wait for the vector ends when the wave's own requests have arrived, and with the whole row
    // requested ahead all the multiply-adds of the phase would follow after the last arrival instead of overlapping it.
    // Measured per 7B token for W2's six chunks: all ahead 1.573 ms, four 1.551, three 1.568, two 1.556; per 13B token
    // for the five chunks of QKV and W13: all ahead 3.14 ms, four 2.92, three 2.74, two 2.79 (four for QKV and three for W13
    // 2.89, three and two 2.73, two and three 2.73 against 2.70); three of QKV's or W13's four
    // at the 7B shape: no change.  Wo's row pairs are always requested whole: that phase only waits for its input.
    static constexpr int kAhead = TU == 6 ? kTU : TU == 5 && MODE != PH_RES ? 3 : TU;
    static constexpr bool kSplitAhead = kAhead < TU;

    const MatvecPhase d;
    int n, nch, lane, W, G, nitems, item;
    // The codes of an item: two sub-rows, each a scalar base pointer + the lane's 16-byte chunk index.
    const uint8_t *cb0 = nullptr, *cb1 = nullptr;  // first code of each sub-row (uniform)
    const float2 *gb0 = nullptr, *gb1 = nullptr;   // scale entry of the group holding that code
    unsigned r0 = 0, r1 = 0;                       // position of that code inside its group
    int which = 0, r = 0;
    bool has1 = true, first = false;
    int wave = 0;
    uint4 w0[TU], w1[TU];
    float2 s0[TU], s1[TU];

    __device__ __forceinline__ MatvecRun(const MatvecPhase &d_) : d(d_)
    {
        const int tid = phase_tid();
        n = d.n;
        nch = n >> 4;
        lane = tid & 63;
        W = d.threads >> 6;
        G = gridDim.x;
        nitems = MODE == PH_QKV ? (d.d0 + d.d1 + d.d2) >> 1 : MODE == PH_RES ? (d.d0 + 1) >> 1 : d.d0;
        // Items are dealt block-minor (item -> workgroup item % G), so every compute unit gets the same
        // number of rows even when the rows do not fill all waves.
        wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        item = wave * G + blockIdx.x;
    }

    __device__ __forceinline__ void resolve(int it)
    {
        long f0, f1;
        QMat m = d.m0, mb = d.m0;
        which = 0;
        has1 = true;
        if (MODE == PH_QKV) {  // rows (2p, 2p+1) of q, k or v: RoPE rotates the pair
            r = 2 * it;
            if (r >= d.d0 + d.d1) { which = 2; r -= d.d0 + d.d1; m = d.m2; }
            else if (r >= d.d0) { which = 1; r -= d.d0; m = d.m1; }
            mb = m;
            f0 = m.off + (long)r * n;
            f1 = f0 + n;
        } else if (MODE == PH_W13) {  // row p of w1 and row p of w3: SwiGLU needs both
            r = it;
            mb = d.m1;
            f0 = m.off + (long)r * n;
            f1 = mb.off + (long)r * n;
        } else if (MODE == PH_RES) {  // rows (2p, 2p+1)
            r = 2 * it;
            has1 = r + 1 < d.d0;
            f0 = m.off + (long)r * n;
            f1 = has1 ? f0 + n : f0;
        } else {  // PH_ROW, long rows: one row per wave so every wave has work
            r = it;
            f0 = m.off + (long)r * n;
            f1 = f0;
        }
        cb0 = m.codes + f0; gb0 = m.gs + (f0 >> 8); r0 = (unsigned)(f0 & 255);
        cb1 = mb.codes + f1; gb1 = mb.gs + (f1 >> 8); r1 = (unsigned)(f1 & 255);
    }

    // Requests chunk u (of TU per lane and sub-row) of step `base` of the resolved item.
    // (Members are used by name in every helper: a reference to a member keeps the whole object in memory.)
    __device__ __forceinline__ void issue_chunk(int base, int u)
    {
        const int c = base + 64 * u + lane, c1 = c + kOff1;
        const unsigned cc = c < nch ? c : nch - 1;  // out-of-range lanes repeat the last chunk (weight 0 in fold)
        const unsigned cc1 = c1 < nch ? c1 : nch - 1;
        const uint4 a0 = load_stream(reinterpret_cast<const uint4 *>(cb0) + cc);
        const uint4 a1 = load_stream(reinterpret_cast<const uint4 *>(cb1) + cc1);
        const float2 g0 = gb0[(r0 + 16u * cc) >> 8];
        const float2 g1 = gb1[(r1 + 16u * cc1) >> 8];
        w0[u] = a0; w1[u] = a1; s0[u] = g0; s1[u] = g1;
    }

    // Requests one step of the resolved item.
    __device__ __forceinline__ void issue(int base)
    {
#pragma unroll
        for (int u = 0; u < TU; u++) issue_chunk(base, u);
    }

    // Defined on every path: otherwise the registers stay reserved for the whole layer loop of k_token.
    __device__ __forceinline__ void zero()
    {
#pragma unroll
        for (int u = 0; u < TU; u++) {
            w0[u] = w1[u] = make_uint4(0u, 0u, 0u, 0u);
            s0[u] = s1[u] = make_float2(0.f, 0.f);
        }
    }

    __device__ __forceinline__ void preload()
    {
        first = item < nitems;
        if (first) {
            resolve(item);
            if (kSplitAhead) {
                zero();
#pragma unroll
                for (int u = 0; u < kAhead; u++) issue_chunk(0, u);
            } else {
                issue(0);
            }
        } else {
            zero();
        }
    }

    __device__ __forceinline__ bool has_item() const { return item < nitems; }

    // A wave without an item of this phase lends its registers: the first item of a later phase `o` (rows of the
    // same length, the same sub-row layout) is requested into them now, while the memory system has little to
    // do, and `o` takes it over with adopt() when its turn comes.
    template <class Other>
    __device__ __forceinline__ void preload_for(Other &o)
    {
        static_assert(TU == Other::TU && kOff1 == Other::kOff1, "the two phases must hold an item the same way");
        first = false;
        o.resolve(o.item);
        cb0 = o.cb0; cb1 = o.cb1; gb0 = o.gb0; gb1 = o.gb1; r0 = o.r0; r1 = o.r1;
        issue(0);
    }

    template <class Other>
    __device__ __forceinline__ void adopt(const Other &o)
    {
#pragma unroll
        for (int u = 0; u < TU; u++) {
            w0[u] = o.w0[u]; w1[u] = o.w1[u];
            s0[u] = o.s0[u]; s1[u] = o.s1[u];
        }
        first = true;
    }

    // Destination of the results of an item (second pointer null when the item has one result).
    __device__ __forceinline__ void dst_of(int it, int pos, float *&p0, float *&p1) const
    {
        if (MODE == PH_QKV) {
            int rr = 2 * it;
            float *base = d.out0;
            if (rr >= d.d0 + d.d1) { rr -= d.d0 + d.d1; base = d.out2 + (long)pos * d.kv_dim; }
            else if (rr >= d.d0) { rr -= d.d0; base = d.out1 + (long)pos * d.kv_dim; }
            p0 = base + rr;
            p1 = p0 + 1;
        } else if (MODE == PH_RES) {
            p0 = d.out0 + 2 * it;
            p1 = 2 * it + 1 < d.d0 ? p0 + 1 : nullptr;
        } else {
            p0 = d.out0 + it;
            p1 = nullptr;
        }
    }

    // The residual inputs of the resolved item (lane 0; in flight while the rows stream).
    __device__ __forceinline__ void residual(const float *res, float &resv0, float &resv1)
    {
        resv0 = resv1 = 0.0f;
        if ((MODE == PH_RES || kRow) && lane == 0) {
            if (d.poll.on && !d.res_emb) {  // a line of the vector may have been cached while it was half written
                resv0 = wait_float(res + r, d.poll);
                if (MODE == PH_RES && has1) resv1 = wait_float(res + r + 1, d.poll);
            } else {
                resv0 = res[r];
                if (MODE == PH_RES && has1) resv1 = res[r + 1];
            }
        }
    }

    // One step of weights against the staged vector: sum (code*rm + min)*x = rm * sum code*x + min * sum x per chunk.
    // With REFILL, the registers of a chunk are requested anew (step `nbase` of the item resolved last) as soon as the
    // chunk is folded: the requests of the next step go out between the multiply-adds of this one instead of after them,
    // so the memory system is not left idle while all the waves of a workgroup work off a step at the same time (at the
    // start of a phase in particular, when every wave holds a step that was requested ahead).
    template <bool REFILL>
    __device__ __forceinline__ void fold(int base, const float4 *xs, const float *sumx, float &acc0, float &acc1, int nbase)
    {
        if constexpr (FAST) {
            const float4 *xp = xs + lane;
            const float *sp = sumx + lane;
#pragma unroll
            for (int u = 0; u < TU; u++) {
                const uint4 a0 = w0[u], a1 = w1[u];
                const float2 g0 = s0[u], g1 = s1[u];
                const float4 x0 = xp[64 * u], x1 = xp[nch + 64 * u], x2 = xp[2 * nch + 64 * u], x3 = xp[3 * nch + 64 * u];
                const float sx = sp[64 * u];
                acc0 += fmaf(g0.x, dot16(a0, x0, x1, x2, x3), g0.y * sx);
                acc1 += fmaf(g1.x, dot16(a1, x0, x1, x2, x3), g1.y * sx);
                if (REFILL) {
                    __builtin_amdgcn_sched_barrier(0);
                    issue_chunk(nbase, u);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            return;
        }
#pragma unroll
        for (int u = 0; u < TU; u++) {
            const uint4 a0 = w0[u], a1 = w1[u];
            const float2 g0 = s0[u], g1 = s1[u];
            const int c = base + 64 * u + lane;
            const bool ok = c < nch;
            const int cc = ok ? c : nch - 1;
            const float4 x0 = xs[cc], x1 = xs[nch + cc], x2 = xs[2 * nch + cc], x3 = xs[3 * nch + cc];
            const float sx = sumx[cc];
            const float t0 = fmaf(g0.x, dot16(a0, x0, x1, x2, x3), g0.y * sx);
            acc0 += ok ? t0 : 0.0f;
            if (kRow) {
                const int c1 = c + kOff1;
                const bool ok1 = c1 < nch;
                const int cc1 = ok1 ? c1 : nch - 1;
                const float4 y0 = xs[cc1], y1 = xs[nch + cc1], y2 = xs[2 * nch + cc1], y3 = xs[3 * nch + cc1];
                const float t1 = fmaf(g1.x, dot16(a1, y0, y1, y2, y3), g1.y * sumx[cc1]);
                acc1 += ok1 ? t1 : 0.0f;
            } else {
                const float t1 = fmaf(g1.x, dot16(a1, x0, x1, x2, x3), g1.y * sx);
                acc1 += ok ? t1 : 0.0f;
            }
            if (REFILL) {  // fenced: left alone, the scheduler moves all the requests to the top, into registers of their own
                __builtin_amdgcn_sched_barrier(0);
                issue_chunk(nbase, u);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }

    // Reduces the sums of the resolved item over the wave, applies the phase's epilogue and stores the results.
    // ss: the rmsnorm scalar of the input vector, which was staged without it (stage_vector); 1 for phases without a norm.
    template <bool COH>
    __device__ __forceinline__ void finish(int it, int wh, int rr, float acc0, float acc1, float resv0, float resv1, int pos, float ss)
    {
        acc0 = wave_sum(acc0);
        acc1 = wave_sum(acc1);
        if (MODE == PH_QKV || MODE == PH_W13) {
            acc0 = __fmul_rn(ss, acc0);
            acc1 = __fmul_rn(ss, acc1);
        }
        if (lane == 0) {
            float v0, v1 = 0.0f;
            if (MODE == PH_QKV) {
                v0 = acc0;
                v1 = acc1;
                if (wh < 2) {  // RoPE on the interleaved pair (r, r+1)  (K/ApplyRope.java:74-90)
                    // (the row index is the same in every lane: through the scalar data path, see uniform_pair)
                    const float2 cs = uniform_pair(reinterpret_cast<const float *>(d.rope + ((long)pos * (d.head_size >> 1) + ((rr % d.head_size) >> 1))));
                    v0 = __fsub_rn(__fmul_rn(acc0, cs.x), __fmul_rn(acc1, cs.y));
                    v1 = __fadd_rn(__fmul_rn(acc0, cs.y), __fmul_rn(acc1, cs.x));
                }
            } else if (MODE == PH_W13) {
                const float s = silu_sigma<true>(d.silu, acc0, d.exact_silu);  // K/Silu.java:72-74
                v0 = __fmul_rn(acc0, __fmul_rn(s, acc1));
            } else if (MODE == PH_RES) {
                v0 = __fadd_rn(resv0, acc0);  // K/Accum.java:26-30
                v1 = __fadd_rn(resv1, acc1);
            } else {
                v0 = __fadd_rn(resv0, acc0 + acc1);
            }
            float *p0, *p1;
            dst_of(it, pos, p0, p1);
            if (COH) {
                st_coh(p0, v0);
                if (p1) st_coh(p1, v1);
                if (MODE == PH_QKV && d.knew && wh > 0) {  // where attention waits for this token's rows
                    float *p = (wh == 1 ? d.knew : d.vnew) + rr;
                    st_coh(p, v0);
                    st_coh(p + 1, v1);
                }
            } else {
                *p0 = v0;
                if (p1) *p1 = v1;
            }
        }
    }

    // smem: 4*nch float4 (vector), nch floats (chunk sums), 16 floats (reduction).
    // COH: results are written through to memory for consumers in the same launch (k_token); a kernel of its
    // own leaves them to the end-of-kernel write-back.
    template <bool COH>
    __device__ __forceinline__ void run(float4 *smem4, int token, int pos)
    {
        float4 *xs = smem4;
        float *sumx = reinterpret_cast<float *>(smem4 + 4 * nch);
        float *red = sumx + nch;
        const float *emb_row = d.emb + (long)token * n;  // J/Run.java:72 (only used when n == dim)
        const float *res = d.res_emb ? emb_row : d.res_src;
        float ss;
        if (d.poll.on && !d.from_emb) {
            ss = stage_vector_poll<kPollWords>(d.xin, n, d.rmsw, xs, sumx, red, d.threads, d.poll);
        } else {
            ss = stage_vector(d.from_emb ? emb_row : d.xin, n, d.rmsw, xs, sumx, red, d.threads);
        }

        if (item >= nitems) return;
        if (!first) {
            resolve(item);
            issue(0);
        } else if (kSplitAhead) {
#pragma unroll
            for (int u = kAhead; u < TU; u++) issue_chunk(0, u);
        }
        first = false;
        // The steps of this wave's items in order; while a step is folded, the step after it is requested.
        int cur = item, cur_which = which, cur_r = r, base = 0;
        float resv0, resv1, acc0 = 0.0f, acc1 = 0.0f;
        residual(res, resv0, resv1);
        // Everything requested so far has arrived before the loop is entered (the first step is needed at once anyway).
        // With requests pending from the several paths that lead here, the compiler's wait insertion loses their order
        // inside the loop and waits for all of them (vmcnt(0)) at the top of every step instead of chunk by chunk.
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        while (true) {
            int nbase = base + kStep, nitem = cur;
            const bool last_step = nbase >= nch;
            if (last_step) {
                nbase = 0;
                nitem = cur + W * G;
            }
            if (nitem >= nitems) break;  // the step in the registers is the wave's last one
            float nres0 = 0.0f, nres1 = 0.0f;
            if (last_step) {  // (the residual of the next item is fetched ahead of its weights: its wait is in order)
                resolve(nitem);
                residual(res, nres0, nres1);
            }
            fold<true>(base, xs, sumx, acc0, acc1, nbase);
            if (last_step) {
                finish<COH>(cur, cur_which, cur_r, acc0, acc1, resv0, resv1, pos, ss);
                cur = nitem; cur_which = which; cur_r = r;
                resv0 = nres0; resv1 = nres1;
                acc0 = acc1 = 0.0f;
            }
            base = nbase;
        }
        fold<false>(base, xs, sumx, acc0, acc1, 0);
        finish<COH>(cur, cur_which, cur_r, acc0, acc1, resv0, resv1, pos, ss);
        item = nitems;
    }
};

template <int MODE, int TU = (MODE == PH_ROW6 ? 6 : kTU)>
__global__ void __launch_bounds__(1024) k_matvec(const MatvecPhase d)
{
    extern __shared__ float4 smem4[];
    MatvecRun<MODE, TU> run(d);
    // The weights do not depend on the input vector: the first loads go out before it is staged, so
    // HBM latency overlaps the rmsnorm prologue.
    run.preload();
    run.template run<false>(smem4, d.st->token, d.st->pos);
}

// ---- decode attention: workgroup = (head, split); waves share the split's rows; online softmax ----

struct AttnPhase {
    const float *q;        // (n_heads * head_size) after RoPE
    const float *kc;       // this layer's key cache (seq_len, kv_dim)
    const float *vc;       // this layer's value cache
    float *out;            // xb (dim)
    float *part;           // (n_heads, nsplit, head_size + 2) partial (max, sum, acc)
    unsigned *counters;    // (n_heads) arrival counters, zero between launches
    const DevState *st;
    int n_heads, kv_mul, head_size, kv_dim, nsplit, rows_per_split;
    float sqrt_hs;
    int threads;           // workgroup size
    int max_splits;        // at most this many splits per head (<= nsplit, the stride of `part`)
    Poll poll;             // how q and this token's k, v rows are read
    const float *knew, *vnew;  // with poll.on: this token's k and v rows (kv_dim each)
};

constexpr int kAU = 2;  // cache rows in flight per lane group (K and V each)

// LPR = lanes per cache row: each lane owns 4 consecutive floats of the head (head_size <= 4*LPR).
// prefetch() requests the first cache rows of the workgroup's first item; rows of earlier positions do not
// depend on this token, so in k_layer it runs before the wait for the phase that writes q and the row of
// this position (that row is fetched in run()).
template <int LPR>
struct AttnRun {
    static constexpr int RPW = 64 / LPR;
    const AttnPhase a;
    int hs, W, tid, lane, nent, len, chunk, nact, j, slot, nitems;
    bool active, early = false;
    float4 k4[kAU], v4[kAU];

    __device__ __forceinline__ AttnRun(const AttnPhase &a_, int pos) : a(a_)
    {
        hs = a.head_size;
        W = a.threads >> 6;
        tid = phase_tid();
        lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        nent = W * RPW;
        len = pos + 1;
        nact = attn_splits_at(len, a.rows_per_split, a.max_splits, chunk);
        j = lane % LPR;
        slot = wave * RPW + lane / LPR;
        active = 4 * j < hs;
        nitems = a.n_heads * nact;
    }

    // rows tb + u*nent (u < kAU) below t1; `part` 0: all of them, 1: only positions before this token's, 2: only this token's
    __device__ __forceinline__ void fetch(int h, int tb, int t1, int part)
    {
        const long col = (long)(h / a.kv_mul) * hs + 4 * j;
#pragma unroll
        for (int u = 0; u < kAU; u++) {
            const int t = tb + u * nent;
            const bool want = part == 0 || (part == 1 ? t < len - 1 : t == len - 1);
            if (t < t1 && active && want) {
                if (a.poll.on && t == len - 1) {  // written in this launch: wait for it where its producer parks it
                    k4[u] = wait_word(a.knew + col, a.poll);
                    v4[u] = wait_word(a.vnew + col, a.poll);
                } else {
                    k4[u] = load_stream(reinterpret_cast<const float4 *>(a.kc + (long)t * a.kv_dim + col));
                    v4[u] = load_stream(reinterpret_cast<const float4 *>(a.vc + (long)t * a.kv_dim + col));
                }
            }
        }
    }

    __device__ __forceinline__ void clear()
    {
#pragma unroll
        for (int u = 0; u < kAU; u++) k4[u] = v4[u] = make_float4(0.f, 0.f, 0.f, 0.f);
    }

    __device__ __forceinline__ int store_waves() const { return (hs + 63) >> 6; }  // waves that store the output
    __device__ __forceinline__ void preload() { prefetch(); }

    __device__ __forceinline__ void prefetch()
    {
        clear();
        early = true;
        if ((int)blockIdx.x < nitems) {
            const int s = blockIdx.x / a.n_heads, t0 = s * chunk;
            fetch(blockIdx.x % a.n_heads, t0 + slot, min(len, t0 + chunk), 1);
        }
    }

    // smem: 3*nent + 4 floats (max, sum, weights), nent*hs floats (acc), 1 int.  COH as for the matvec phases (the partials of
    // a split always travel write-through: other workgroups of the same launch read them).
    template <bool COH>
    __device__ __forceinline__ void run(float *smem)
    {
        float *sm_m = smem;           // nent
        float *sm_l = sm_m + nent;    // nent
        float *sm_w = sm_l + nent;    // nent + 4 (unused: the fold keeps the weights in registers)
        float *sm_acc = sm_w + nent + 4;  // nent * hs
        int &s_last = *reinterpret_cast<int *>(sm_acc + nent * hs);

        for (int it = blockIdx.x; it < nitems; it += gridDim.x) {
            const int h = it % a.n_heads, s = it / a.n_heads;
            const int t0 = s * chunk, t1 = min(len, t0 + chunk);
            float4 q4 = make_float4(0.f, 0.f, 0.f, 0.f);
            bool kv_done = false;  // this token's k and v row arrived together with q
            if (active && a.poll.on) {
                // with preloaded cache rows only this position's row is missing: if it is one of this lane group's
                // rows, wait for q, k and v in one trip to memory instead of three
                int ucur = -1;
                if (early && it == (int)blockIdx.x) {
#pragma unroll
                    for (int u = 0; u < kAU; u++)
                        if (t0 + slot + u * nent == len - 1) ucur = u;
                }
                if (ucur >= 0) {
                    const long col = (long)(h / a.kv_mul) * hs + 4 * j;
                    const float *pp[3] = {a.q + h * hs + 4 * j, a.knew + col, a.vnew + col};
                    float4 vv[3];
                    wait_words(pp, vv, a.poll);
                    q4 = vv[0];
#pragma unroll
                    for (int u = 0; u < kAU; u++)
                        if (u == ucur) { k4[u] = vv[1]; v4[u] = vv[2]; }
                    kv_done = true;
                } else {
                    q4 = wait_word(a.q + h * hs + 4 * j, a.poll);
                }
            } else if (active) {
                q4 = *reinterpret_cast<const float4 *>(a.q + h * hs + 4 * j);
            }
            float m = -3.402823466e+38f, l = 0.0f;
            float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
            for (int tb = t0 + slot; tb < t1; tb += nent * kAU) {
                bool ok[kAU];
#pragma unroll
                for (int u = 0; u < kAU; u++) ok[u] = tb + u * nent < t1;
                if (early && it == (int)blockIdx.x && tb == t0 + slot) {
                    if (!kv_done) fetch(h, tb, t1, 2);  // only the row of this position is still missing
                } else {
                    clear();
                    fetch(h, tb, t1, 0);
                }
                float sc[kAU], mb = m;
#pragma unroll
                for (int u = 0; u < kAU; u++) {
                    // att[t] = (q . k_t) / sqrt(head_size)   (K/AttentionLoop.java:36-48)
                    sc[u] = __fdiv_rn(group_sum<LPR>(dot4(q4, k4[u])), a.sqrt_hs);
                    if (ok[u]) mb = fmaxf(mb, sc[u]);
                }
                // Online softmax, shifted by the running maximum of the scores.  The reference shifts by a
                // running maximum of element products (K/AttentionLoop.java:44-51); softmax is shift
                // invariant, so only rounding differs.
                const float scale = expf(m - mb);  // 0 on the first batch (m = -FLT_MAX)
                l *= scale;
                acc.x *= scale; acc.y *= scale; acc.z *= scale; acc.w *= scale;
#pragma unroll
                for (int u = 0; u < kAU; u++) {
                    const float p = ok[u] ? expf(sc[u] - mb) : 0.0f;
                    l += p;
                    acc.x = fmaf(p, v4[u].x, acc.x);  // K/AccumWeightedValue.java:48-62
                    acc.y = fmaf(p, v4[u].y, acc.y);
                    acc.z = fmaf(p, v4[u].z, acc.z);
                    acc.w = fmaf(p, v4[u].w, acc.w);
                }
                m = mb;
            }
            if (it != (int)blockIdx.x) __syncthreads();  // LDS reuse across items (the first finds it free)
            if (j == 0) { sm_m[slot] = m; sm_l[slot] = l; }
            if (active) *reinterpret_cast<float4 *>(sm_acc + slot * hs + 4 * j) = acc;
            __syncthreads();
            // Fold the row slots (at most 64) in a fixed order, so the result does not depend on timing.  Each of the waves
            // that hold the head's elements does the whole fold for itself, without another workgroup barrier: lane e
            // takes slot e's maximum and sum and computes its weight exp(m_e - M), the weighted sums are added across the
            // wave, and every thread folds its element over the slots with the weights read lane by lane.
            float M = 0.0f, L = 0.0f, o = 0.0f;
            if (tid < 64 * store_waves()) {
                const float me = lane < nent ? sm_m[lane] : -3.402823466e+38f;
                const float le = lane < nent ? sm_l[lane] : 0.0f;
                M = wave_max(me);
                const float w = expf(me - M);  // empty slots: exp(-huge) = 0
                L = wave_sum(le * w);
                const float *ap = sm_acc + min(tid, hs - 1);
                int e = 0;
                for (; e + 4 <= nent; e += 4) {  // four slots per step: their LDS reads are issued together
                    const float a0 = ap[(e + 0) * hs], a1 = ap[(e + 1) * hs], a2 = ap[(e + 2) * hs], a3 = ap[(e + 3) * hs];
                    o = fmaf(a0, readlane_f(w, e), o);
                    o = fmaf(a1, readlane_f(w, e + 1), o);
                    o = fmaf(a2, readlane_f(w, e + 2), o);
                    o = fmaf(a3, readlane_f(w, e + 3), o);
                }
                for (; e < nent; e++) o = fmaf(ap[e * hs], readlane_f(w, e), o);
            }
            if (nact == 1) {
                if (tid < hs) {
                    if (COH) st_coh(a.out + h * hs + tid, __fdiv_rn(o, L));
                    else a.out[h * hs + tid] = __fdiv_rn(o, L);
                }
                continue;
            }
            // Several splits: partials travel through memory with device-scope relaxed atomics (write-through
            // stores, cache-bypassing loads), which is far cheaper here than a fence that writes back and
            // invalidates the L2 of every XCD.  The split that arrives last folds them in split order.
            float *mypart = a.part + ((long)h * a.nsplit + s) * (hs + 2);
            if (tid < hs) st_coh(mypart + 2 + tid, o);
            if (tid == 0) { st_coh(mypart, M); st_coh(mypart + 1, L); }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's partial stores have been acknowledged
            __syncthreads();
            if (tid == 0) s_last = (__hip_atomic_fetch_add(a.counters + h, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (unsigned)(nact - 1));
            __syncthreads();
            if (!s_last) continue;
            const float *hp = a.part + (long)h * a.nsplit * (hs + 2);
            if (tid < hs) {
                float MM = -3.402823466e+38f, LL = 0.0f, oo = 0.0f;
                for (int i0 = 0; i0 < nact; i0 += 4) {
                    // the (maximum, sum) pairs and this thread's element of four partials: one trip to memory
                    float pm[4], pl[4], po[4];
                    float2 ml[4];
                    unsigned off2[4], off1[4];
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        off2[i] = (unsigned)(min(i0 + i, nact - 1) * (hs + 2)) * 4u;
                        off1[i] = off2[i] + (unsigned)(2 + tid) * 4u;
                    }
                    load4x2_coh(hp, off2, ml, off1, po);
                    float mb = MM;
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        pm[i] = ml[i].x;
                        pl[i] = ml[i].y;
                        if (i0 + i < nact) mb = fmaxf(mb, pm[i]);
                    }
                    const float scale = expf(MM - mb);
                    LL *= scale;
                    oo *= scale;
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        if (i0 + i < nact) {
                            const float w = expf(pm[i] - mb);
                            LL = fmaf(pl[i], w, LL);
                            oo = fmaf(po[i], w, oo);
                        }
                    }
                    MM = mb;
                }
                if (COH) st_coh(a.out + h * hs + tid, __fdiv_rn(oo, LL));
                else a.out[h * hs + tid] = __fdiv_rn(oo, LL);
            }
            if (tid == 0) st_coh(a.counters + h, 0u);
        }
    }
};

template <int LPR>
__global__ void __launch_bounds__(1024) k_attention(const AttnPhase a)
{
    extern __shared__ float smem[];
    AttnRun<LPR> run(a, a.st->pos);
    run.clear();
    run.template run<false>(smem);
}

// ---- final rmsnorm + fp32 classifier + per-workgroup first-max -----------------------------------

struct ClsPhase {
    const float *xin;    // residual stream
    const float *rmsw;   // dequantized rms_final_weight
    const float *w;      // (vocab, dim) fp32
    int n, vocab;
    float *logits;
    unsigned long long *part;  // one (index, value) per workgroup: the first maximum of its rows
    int nparts;
    DevState *st;
    const int *prompt;   // seq_len
    int *out_tokens;     // seq_len
    unsigned *bar_ctr;   // grid barrier counters of the token, zeroed for the next one
    int nbar;
    int threads;         // workgroup size of the classifier
    Poll poll;           // how the input vector is read
    unsigned long long *tstamp;  // seq_len: the device's wall clock at the end of the token of each position
    float4 *unset_p;     // self-contained k_token: vectors to mark unwritten for the next token (nothing touches them
    long unset_n4;       // during this launch), unset_n4 16-byte words; 0: none
};

constexpr int kCU = 8;

struct ClsRun {
    const ClsPhase a;
    int n, nch, n4, lane, wave, W, G, row;
    bool first = false;
    float4 pre[kCU];

    __device__ __forceinline__ ClsRun(const ClsPhase &a_) : a(a_)
    {
        n = a.n;
        nch = n >> 4;
        n4 = n >> 2;
        const int tid = phase_tid();
        lane = tid & 63;
        wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        W = a.threads >> 6;
        G = gridDim.x;
        row = wave * G + blockIdx.x;
    }

    __device__ __forceinline__ void issue(int r, int base)
    {
        const float4 *wr = reinterpret_cast<const float4 *>(a.w + (long)r * n);
#pragma unroll
        for (int u = 0; u < kCU; u++) {
            const int c = base + 64 * u + lane;
            pre[u] = load_stream(wr + (c < n4 ? c : n4 - 1));
        }
    }

    __device__ __forceinline__ void preload()
    {
        first = row < a.vocab;
        if (first) {
            issue(row, 0);
        } else {
#pragma unroll
            for (int u = 0; u < kCU; u++) pre[u] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }

    // This thread's share of the vectors to mark unwritten.  The stores are written through to memory: left dirty in the
    // caches, 4.6 MB of marks (7B shape) made the write-back at the end of the launch 13 us longer.
    __device__ __forceinline__ void mark_unset()
    {
        const float u = __uint_as_float(kUnset);
        v4f uv;
        uv.x = uv.y = uv.z = uv.w = u;
        const long step = (long)G * a.threads;
        for (long i = (long)blockIdx.x * a.threads + 64 * wave + lane; i < a.unset_n4; i += step)
            asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 2" ::"v"(a.unset_p + i), "v"(uv) : "memory");   // (wait states: a 16-byte store reads its data registers after it has issued)
    }

    // smem: as for a matvec phase, then 16 floats and 16 ints for the per-wave maxima
    __device__ __forceinline__ void run(float4 *smem4)
    {
        float4 *xs = smem4;
        float *sumx = reinterpret_cast<float *>(smem4 + 4 * nch);
        float *red = sumx + nch;
        float *bval = red + 16;
        int *bidx = reinterpret_cast<int *>(red + 32);
        float ss;
        if (a.poll.on) {
            ss = stage_vector_poll<kPollWords>(a.xin, n, a.rmsw, xs, sumx, red, a.threads, a.poll);
        } else {
            ss = stage_vector(a.xin, n, a.rmsw, xs, sumx, red, a.threads);
        }

        float best_v = -__builtin_inff();
        int best_i = 0x7fffffff;
        bool marked = a.unset_n4 == 0;
        for (; row < a.vocab; row += W * G) {
            float acc = 0.0f;
            for (int base = 0; base < n4; base += 64 * kCU) {
                if (!(first && base == 0)) issue(row, base);
#pragma unroll
                for (int u = 0; u < kCU; u++) {
                    const int c = base + 64 * u + lane;
                    const bool ok = c < n4;
                    const int cc = ok ? c : n4 - 1;
                    const float t = dot4(pre[u], xs[(cc & 3) * nch + (cc >> 2)]);
                    acc += ok ? t : 0.0f;
                }
            }
            first = false;
            acc = __fmul_rn(ss, wave_sum(acc));
            if (lane == 0) {
                a.logits[row] = acc;
                if (better(acc, row, best_v, best_i)) { best_v = acc; best_i = row; }
            }
            if (!marked) {  // between two rows, where the stores hide among the row loads
                marked = true;
                mark_unset();
            }
        }
        if (!marked) mark_unset();
        if (lane == 0) { bval[wave] = best_v; bidx[wave] = best_i; }
        __syncthreads();
        if (threadIdx.x == 0) {
            for (int w = 1; w < W; w++)
                if (better(bval[w], bidx[w], best_v, best_i)) { best_v = bval[w]; best_i = bidx[w]; }
            st_coh(a.part + blockIdx.x, pack_max(best_v, best_i));  // written through: workgroup 0 may wait for it in this launch
        }
    }
};

static __global__ void __launch_bounds__(1024) k_classifier(const ClsPhase a)
{
    extern __shared__ float4 smem4[];
    ClsRun run(a);
    run.preload();
    run.run(smem4);
}

// ---- layers [l0, l1) and optionally the classifier in one launch ------------------------------------
// Grid: one workgroup per compute unit, all resident.  Barrier instance 5*l + k follows phase k of layer l.

enum { K_QKV = 0, K_ATT = 1, K_WO = 2, K_W13 = 3, K_W2 = 4, K_CLS = 5 };

// Everything the phases of a token are built from.  The phase arguments of layer l are derived from it on
// the host (one launch per phase) and on the device (k_token) by the same functions.
struct TokenGeom {
    int dim, hidden, n_layers, n_heads, kv_mul, head_size, kv_dim, seq_len, vocab, exact_silu;
    int threads;  // workgroup size of the matvec phases, the classifier and k_token
    long sd, sh;  // strides of dim-long and hidden-long activation vectors, in floats
    const float *emb, *rmsw, *silu, *wcls;
    const float2 *rope;
    float *x, *xb, *hb, *q, *kcache, *vcache, *logits;  // x, xb, hb, q, knew, vnew: set 0 of two, `set_stride` floats apart
    long set_stride;
    QMat wq, wk, wv, wo, w1, w2, w3;  // off = 0: layer 0
    float *knew, *vnew;  // this token's k and v rows per layer (stride skv), for the hand-over by value
    long skv;
    float *attn_part;    // per layer: (n_heads, attn_nsplit, head_size + 2)
    unsigned *attn_counters;  // per layer: n_heads
    int attn_nsplit;
    float sqrt_hs;
    DevState *st;
    unsigned long long *cls_part;
    unsigned long long *tstamp;
    const int *prompt;
    int *out_tokens;
    unsigned *bar_ctr;
    int nbar;
    int *fault;
};

// The builders below are templates on the geometry's type so that the device can read it straight from the
// kernel-argument segment (constant address space, scalar loads) instead of from a copy in registers.
template <class M>
__host__ __device__ inline QMat at_layer(const M &m, long floats_per_layer, int l)
{
    QMat r;
    r.codes = m.codes;
    r.gs = m.gs;
    r.off = m.off + floats_per_layer * l;
    return r;
}

// Arguments of the phases of layer l (J/Run.java:76-159).
// `set`: which of the two sets of activation vectors (always 0 outside a whole-token kernel that alternates them).
template <class G>
__host__ __device__ inline MatvecPhase matvec_phase_of(const G &g, int kclass, int l, int set = 0)
{
    const long dim = g.dim, hid = g.hidden, kvd = g.kv_dim;
    const long kvoff = (long)l * g.seq_len * kvd;
    const long so = set * g.set_stride;
    float *const x = g.x + so, *const xb = g.xb + so, *const hb = g.hb + so, *const q = g.q + so;
    MatvecPhase d{};
    d.emb = g.emb; d.rope = g.rope; d.silu = g.silu; d.st = g.st;
    d.head_size = g.head_size; d.kv_dim = g.kv_dim; d.exact_silu = g.exact_silu; d.threads = g.threads;
    switch (kclass) {
    case K_QKV:
        d.n = g.dim; d.from_emb = l == 0; d.xin = x + 2 * l * g.sd; d.rmsw = g.rmsw + l * dim;
        d.d0 = g.dim; d.d1 = d.d2 = g.kv_dim;
        d.m0 = at_layer(g.wq, dim * dim, l); d.m1 = at_layer(g.wk, dim * kvd, l); d.m2 = at_layer(g.wv, dim * kvd, l);
        d.out0 = q + l * g.sd; d.out1 = g.kcache + kvoff; d.out2 = g.vcache + kvoff;
        break;
    case K_WO:
        d.n = g.dim; d.xin = xb + l * g.sd; d.d0 = g.dim; d.m0 = at_layer(g.wo, dim * dim, l);
        d.out0 = x + (2 * l + 1) * g.sd; d.res_src = x + 2 * l * g.sd; d.res_emb = l == 0;
        break;
    case K_W13:
        d.n = g.dim; d.xin = x + (2 * l + 1) * g.sd; d.rmsw = g.rmsw + (g.n_layers + l) * dim; d.d0 = g.hidden;
        d.m0 = at_layer(g.w1, dim * hid, l); d.m1 = at_layer(g.w3, dim * hid, l); d.out0 = hb + l * g.sh;
        break;
    default:  // K_W2
        d.n = g.hidden; d.xin = hb + l * g.sh; d.d0 = g.dim; d.m0 = at_layer(g.w2, dim * hid, l);
        d.out0 = x + (2 * l + 2) * g.sd; d.res_src = x + (2 * l + 1) * g.sd;
        break;
    }
    return d;
}

template <class G>
__host__ __device__ inline AttnPhase attn_phase_of(const G &g, int l, int rows_per_split, int threads, int max_splits, int set = 0)
{
    const long kvoff = (long)l * g.seq_len * g.kv_dim;
    const long so = set * g.set_stride;
    AttnPhase t{};
    t.q = g.q + so + l * g.sd; t.kc = g.kcache + kvoff; t.vc = g.vcache + kvoff; t.out = g.xb + so + l * g.sd;
    t.part = g.attn_part + (long)l * g.n_heads * g.attn_nsplit * (g.head_size + 2); t.counters = g.attn_counters + l * g.n_heads; t.st = g.st;
    t.n_heads = g.n_heads; t.kv_mul = g.kv_mul; t.head_size = g.head_size; t.kv_dim = g.kv_dim;
    t.nsplit = g.attn_nsplit; t.rows_per_split = rows_per_split; t.threads = threads;
    t.max_splits = max_splits < g.attn_nsplit ? max_splits : g.attn_nsplit;
    t.sqrt_hs = g.sqrt_hs;  // (float) Math.sqrt(head_size), K/AttentionLoop.java:48
    return t;
}

template <class G>
__host__ __device__ inline ClsPhase cls_phase_of(const G &g, int nparts, int set = 0)
{
    ClsPhase a{};
    a.xin = g.x + set * g.set_stride + 2L * g.n_layers * g.sd; a.rmsw = g.rmsw + 2L * g.n_layers * g.dim; a.w = g.wcls;
    a.n = g.dim; a.vocab = g.vocab; a.logits = g.logits; a.part = g.cls_part; a.nparts = nparts;
    a.st = g.st; a.prompt = g.prompt; a.out_tokens = g.out_tokens; a.bar_ctr = g.bar_ctr; a.nbar = g.nbar; a.threads = g.threads;
    a.tstamp = g.tstamp;
    return a;
}

// Long rows are streamed one row per wave (PH_ROW) so every wave has work; shorter ones as row pairs (PH_RES).
// The mode of a matvec + residual phase for rows of n codes: pairs of rows while a row fits one step of a sub-row.
__host__ __device__ inline int row_mode(int n)
{
    const int nch = n / 16;
    return nch <= 64 * kTU ? PH_RES : nch > 2 * 64 * kTU && nch <= 2 * 64 * 6 ? PH_ROW6 : PH_ROW;
}

// Chunks per lane and sub-row for rows of n codes streamed as row pairs in one step each: the smallest of 1, 2, 4, 5
// that holds a row (short rows would otherwise fold three empty chunks out of four; rows of 257..320 chunks, the 13B
// shape's, would take a second step for a quarter of a step's worth).  kTU for everything longer.
__host__ __device__ inline int tu_for(int n)
{
    const int nch = n / 16;
    return nch <= 64 ? 1 : nch <= 128 ? 2 : nch <= 256 ? 4 : nch <= 320 ? 5 : kTU;
}

struct TokenArgs {
    TokenGeom g;
    int l0, l1, with_cls;   // layers [l0, l1), then the classifier when with_cls
    int attn_rows;          // cache rows per attention split in this kernel (more when the splits run out)
    int attn_splits;        // at most this many splits per head: one (head, split) item per workgroup
    int maxspin;
    int by_value;           // 1: consumers wait for the data itself (activations pre-filled with kUnset); 0: grid barriers
    int self_contained;     // (with by_value, the whole token in this launch) bit 0: the kernel alternates between two sets of
                            // activation vectors and marks the other one unwritten for the next token (no k_fill_unset
                            // before it); bit 1: it does the token-loop step itself (no k_finish after it)
};

// Before a token whose phases hand over by value: the activation vectors it will write (n floats at p, a multiple of
// 4) and, for a self-contained token, the per-workgroup classifier results (nparts words) are marked unwritten.
struct FillArgs {
    float *p;
    long n;
    unsigned long long *part;
    int nparts;
};

static __global__ void k_fill_unset(const FillArgs a)
{
    const float u = __uint_as_float(kUnset);
    const float4 u4 = make_float4(u, u, u, u);
    float4 *p = reinterpret_cast<float4 *>(a.p);
    const long nq = a.n >> 2;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < nq; i += (long)gridDim.x * blockDim.x) p[i] = u4;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < a.nparts; i += gridDim.x * blockDim.x) a.part[i] = kUnset64;
}

// Between two phases: every wave waits for its own stores to be acknowledged, the workgroup arrives at the
// barrier, requests the first weights of the next phase, and only then waits for the other workgroups.
template <class Next>
__device__ __forceinline__ void handoff(const GridBar &b, int inst, Next &nx)
{
    if (b.ngroups == 0) {  // hand-over by value: the next phase waits for its input itself
        nx.preload();      // per wave, as soon as its own items are done: it fills the tail of the phase
        __syncthreads();   // every wave is done with the LDS of the phase that ends here
        return;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    bar_arrive(b, inst);
    nx.preload();
    bar_wait(b, inst);
}

// The kernel arguments, re-read from the kernel-argument segment by every phase: the pointer goes through an
// empty asm so the compiler cannot keep all ~100 argument words live in scalar registers across the layer
// loop (which spills), and each phase loads just the words it uses.
typedef const __attribute__((address_space(4))) TokenArgs *TokenArgsPtr;
__device__ __forceinline__ TokenArgsPtr token_args()
{
    TokenArgsPtr p = (TokenArgsPtr)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(p));
    return p;
}

__device__ __forceinline__ Poll token_poll()
{
    Poll p;
    p.on = token_args()->by_value;
    p.maxspin = token_args()->maxspin;
    p.fault = token_args()->g.fault;
    return p;
}

// A matvec phase of k_token: the arguments of layer l plus how its input arrives.
__device__ __forceinline__ MatvecPhase token_phase(int kclass, int l, int set)
{
    MatvecPhase d = matvec_phase_of(token_args()->g, kclass, l, set);
    d.poll = token_poll();
    if (d.poll.on && kclass == K_QKV) {
        d.knew = token_args()->g.knew + set * token_args()->g.set_stride + l * token_args()->g.skv;
        d.vnew = token_args()->g.vnew + set * token_args()->g.set_stride + l * token_args()->g.skv;
    }
    return d;
}

template <int W2_MODE, int TU = (W2_MODE == PH_ROW6 ? 6 : kTU)>
__device__ __forceinline__ void token_w2(const GridBar &b, int l, int set, float4 *smem4, int token, int pos)
{
    MatvecRun<W2_MODE, TU> w2(token_phase(K_W2, l, set));
    handoff(b, 5 * l + 3, w2);
    w2.template run<true>(smem4, token, pos);
}

// What handoff() calls on the phase that follows: either the runner's own preload() or one of these.
template <class A, class B>
struct LendRegisters {   // a's registers take b's first item when this wave has no item of a
    A &a;
    B &b;
    bool lend;
    __device__ __forceinline__ void preload()
    {
        if (lend) a.preload_for(b);
        else a.preload();
    }
};

template <class A, class B>
struct TakeRegisters {   // a takes over what LendRegisters requested into b's registers
    A &a;
    B &b;
    bool lend;
    __device__ __forceinline__ void preload()
    {
        if (lend) a.adopt(b);
        else a.preload();
    }
};

// Wo + residual, then rmsnorm + W1,W3 + SwiGLU.  With Wo in row pairs only half the waves of the 7B shape have a Wo item;
// the others request their first W13 item already when the Wo phase begins (the attention and Wo phases leave the
// memory system two thirds idle), so that only half of W13's first items remain to be requested at its hand-over.
template <int WO_MODE, int TUD = kTU, bool LEND = true, bool FAST = false>
__device__ __forceinline__ void token_wo_w13(const GridBar &b, int l, int set, float4 *smem4, int token, int pos)
{
    typedef MatvecRun<WO_MODE, (WO_MODE == PH_RES ? TUD : WO_MODE == PH_ROW6 ? 6 : kTU), FAST && WO_MODE == PH_RES> WoRun;
    typedef MatvecRun<PH_W13, TUD, FAST> W13Run;
    WoRun wo(token_phase(K_WO, l, set));
    W13Run w13(token_phase(K_W13, l, set));
    bool lend = false;
    if constexpr (WO_MODE == PH_RES && LEND) {
        // only in workgroups that had no attention item: the others come late, and their wait for the attention
        // output would queue behind the extra loads
        int chunk;
        const int busy = token_args()->g.n_heads * attn_splits_at(pos + 1, token_args()->attn_rows, token_args()->attn_splits, chunk);
        lend = !wo.has_item() && w13.has_item() && wo.n == w13.n && (int)blockIdx.x >= busy;
    }
    if constexpr (WO_MODE == PH_RES && LEND) {
        LendRegisters<WoRun, W13Run> first{wo, w13, lend};
        handoff(b, 5 * l + 1, first);
    } else {
        handoff(b, 5 * l + 1, wo);
    }
    wo.template run<true>(smem4, token, pos);
    if constexpr (WO_MODE == PH_RES && LEND) {
        TakeRegisters<W13Run, WoRun> second{w13, wo, lend};
        handoff(b, 5 * l + 2, second);
    } else {
        handoff(b, 5 * l + 2, w13);
    }
    w13.template run<true>(smem4, token, pos);
}

// The end of a self-contained token, in workgroup 0 once its own rows are done: it waits for the maximum of every
// workgroup by value (the words were marked unwritten before the launch; bounded like the other waits), folds them
// (first index of the strict maximum, J/Sampler.java:46-57), steps the token loop (J/Run.java:635-642, 668, 680)
// as k_finish does, and marks the words unwritten again.
__device__ __forceinline__ void token_finish(const ClsPhase &a, float4 *smem4)
{
    float *bval = reinterpret_cast<float *>(smem4);
    int *bidx = reinterpret_cast<int *>(smem4) + 16;
    __syncthreads();  // the classifier is done with its LDS
    float bv = -__builtin_inff();
    int bi = 0x7fffffff;
    for (int b = threadIdx.x; b < a.nparts; b += blockDim.x) {
        unsigned long long w = ld_coh(a.part + b);
        int spins = 0;
        while (w == kUnset64) {
            if (++spins > a.poll.maxspin || ((spins & 63) == 0 && ld_coh(a.poll.fault) != 0)) { st_coh(a.poll.fault, 1); break; }
            __builtin_amdgcn_s_sleep(4);
            w = ld_coh(a.part + b);
        }
        if (better(max_val(w), max_idx(w), bv, bi)) { bv = max_val(w); bi = max_idx(w); }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off);
        const int oi = __shfl_xor(bi, off);
        if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
    }
    if ((threadIdx.x & 63) == 0) { bval[threadIdx.x >> 6] = bv; bidx[threadIdx.x >> 6] = bi; }
    __syncthreads();  // every word has been read
    for (int b = threadIdx.x; b < a.nparts; b += blockDim.x) a.part[b] = kUnset64;
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x >> 6); w++)
            if (better(bval[w], bidx[w], bv, bi)) { bv = bval[w]; bi = bidx[w]; }
        if (bi == 0x7fffffff) bi = 0;  // all NaN: the reference's scan never leaves index 0
        const int pos = a.st->pos;
        const int next = pos < a.st->n_prompt ? a.prompt[pos] : bi;
        a.out_tokens[pos] = next;
        a.tstamp[pos] = wall_clock64();
        a.st->token = next;
        a.st->pos = pos + 1;
        a.st->epoch = a.st->epoch + 1;
    }
}

// TUD, TUH: chunks per lane and sub-row for the phases whose rows are dim and hidden codes long (tu_for); kTU is
// the general case, in which the Wo and W2 phases pick their mode by the row length (row_mode).
// FASTD: a row of dim codes is exactly one step of TUD chunks per lane (dim == 1024 * TUD, checked on the host): the
// phases whose rows are dim long (QKV, Wo, W1/W3) fold it without clamping (MatvecRun).
template <int LPR, int TUD = kTU, int TUH = kTU, bool FASTD = false>
__global__ void __launch_bounds__(1024) k_token(const TokenArgs)
{
    extern __shared__ float4 smem4[];
    TokenArgsPtr t = token_args();
    const int token = t->g.st->token, pos = t->g.st->pos;
    const int set = (t->self_contained & 1) ? t->g.st->epoch & 1 : 0;  // the other set is marked unwritten for the next token
    const int l0 = t->l0, l1 = t->l1;
    const int wo_mode = row_mode(t->g.dim), w2_mode = row_mode(t->g.hidden);
    GridBar b;
    b.ctr = t->g.bar_ctr; b.fault = t->g.fault; b.ngroups = t->by_value ? 0 : kBarGroups; b.maxspin = t->maxspin;
    for (int l = l0; l < l1; l++) {
        {
            MatvecRun<PH_QKV, TUD, FASTD> qkv(token_phase(K_QKV, l, set));
            if (l == l0) qkv.preload();             // launch order guarantees the input
            else handoff(b, 5 * (l - 1) + 4, qkv);  // after W2 of the previous layer
            qkv.template run<true>(smem4, token, pos);
        }
        {
            AttnPhase ap = attn_phase_of(token_args()->g, l, token_args()->attn_rows, token_args()->g.threads, token_args()->attn_splits, set);
            ap.poll = token_poll();
            ap.knew = token_args()->g.knew + set * token_args()->g.set_stride + l * token_args()->g.skv;
            ap.vnew = token_args()->g.vnew + set * token_args()->g.set_stride + l * token_args()->g.skv;
            AttnRun<LPR> att(ap, pos);
            handoff(b, 5 * l, att);
            att.template run<true>(reinterpret_cast<float *>(smem4));
        }
        if constexpr (FASTD) {  // (lending as below: only with four chunks per lane)
            token_wo_w13<PH_RES, TUD, TUD == kTU, true>(b, l, set, smem4, token, pos);
        } else if constexpr (TUD < kTU) {  // the host picked TUD so that a row of dim codes is one step
            token_wo_w13<PH_RES, TUD>(b, l, set, smem4, token, pos);
        } else if constexpr (TUD > kTU) {  // without lending (measured at the 13B shape: 2.77 with, 2.74 ms without)
            token_wo_w13<PH_RES, TUD, false>(b, l, set, smem4, token, pos);
        } else {
            if (wo_mode == PH_ROW6) token_wo_w13<PH_ROW6>(b, l, set, smem4, token, pos);
            else if (wo_mode == PH_ROW) token_wo_w13<PH_ROW>(b, l, set, smem4, token, pos);
            else token_wo_w13<PH_RES>(b, l, set, smem4, token, pos);
        }
        if constexpr (TUH != kTU) {  // likewise for a row of hidden codes
            token_w2<PH_RES, TUH>(b, l, set, smem4, token, pos);
        } else {
            if (w2_mode == PH_ROW6) token_w2<PH_ROW6>(b, l, set, smem4, token, pos);
            else if (w2_mode == PH_ROW) token_w2<PH_ROW>(b, l, set, smem4, token, pos);
            else token_w2<PH_RES>(b, l, set, smem4, token, pos);
        }
    }
    if (token_args()->with_cls) {
        ClsPhase cp = cls_phase_of(token_args()->g, gridDim.x, set);
        cp.poll = token_poll();
        if (token_args()->self_contained & 1) {  // the other set, for the token after this one
            cp.unset_p = reinterpret_cast<float4 *>(token_args()->g.x + (1 - set) * token_args()->g.set_stride);
            cp.unset_n4 = token_args()->g.set_stride >> 2;
        }
        ClsRun cls(cp);
        handoff(b, 5 * (l1 - 1) + 4, cls);
        cls.run(smem4);
        if ((token_args()->self_contained & 2) && blockIdx.x == 0) token_finish(cp, smem4);
    }
}

// First index of the strict maximum (J/Sampler.java:46-57), then the token-loop step
// (J/Run.java:635-642, 668, 680): forced prompt id or argmax, then advance.  One workgroup.
static __global__ void __launch_bounds__(1024) k_finish(const ClsPhase a)
{
    __shared__ float bval[16];
    __shared__ int bidx[16];
    float bv = -__builtin_inff();
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < a.nbar * (1 + kBarGroups); i += blockDim.x)
        st_coh(a.bar_ctr + (long)(i / (1 + kBarGroups)) * kBarStride + 64 * (i % (1 + kBarGroups)), 0u);
    for (int b = threadIdx.x; b < a.nparts; b += blockDim.x) {
        const unsigned long long w = a.part[b];
        if (better(max_val(w), max_idx(w), bv, bi)) { bv = max_val(w); bi = max_idx(w); }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off);
        const int oi = __shfl_xor(bi, off);
        if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
    }
    if ((threadIdx.x & 63) == 0) { bval[threadIdx.x >> 6] = bv; bidx[threadIdx.x >> 6] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x >> 6); w++)
            if (better(bval[w], bidx[w], bv, bi)) { bv = bval[w]; bi = bidx[w]; }
        if (bi == 0x7fffffff) bi = 0;  // all NaN: the reference's scan never leaves index 0
        const int pos = a.st->pos;
        const int next = pos < a.st->n_prompt ? a.prompt[pos] : bi;
        a.out_tokens[pos] = next;
        a.tstamp[pos] = wall_clock64();
        a.st->token = next;
        a.st->pos = pos + 1;
        a.st->epoch = a.st->epoch + 1;
    }
}

// rmsnorm weights dequantized once (K/WeightNormalizeAndScale.java:71-72): value = byte / 255f * range + min
static __global__ void k_dequant_rms(const uint8_t *__restrict__ codes, const float2 *__restrict__ mm, long n, float *__restrict__ out)
{
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const float2 v = mm[i >> 8];
        out[i] = __fadd_rn(__fmul_rn(__fdiv_rn((float)codes[i], 255.0f), __fsub_rn(v.y, v.x)), v.x);
    }
}

}  // namespace l2j
