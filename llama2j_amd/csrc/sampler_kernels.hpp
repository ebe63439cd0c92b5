// Sampling of the next token on the device: the temperature / softmax step of J/Run.java:643-665 and
// J/Sampler.java's sample and sample_topp, with the same float32 operations in the same order, so that
// the logits never travel to the host.
//
// The reference adds the probabilities one by one into a float (the softmax denominator, the CDF of
// sample, the cumulative probability of sample_topp); float addition is not associative, so those sums
// run here as one dependent chain in a single lane (about 2.5 ns per element) and everything else
// (divide, max, exp, normalize, candidate filter, the search in the running sums) is spread over the
// workgroup.  The probabilities live in LDS; the chain overwrites them with its running sums, stops
// at the end of the 64-element chunk in which the sum passes the draw / topp, and the first
// element past it is then found in parallel.
//
// sample_topp sorts its whole ProbIndex array, not just the candidates of the call: entries of earlier calls
// stay behind them and take part (J/Sampler.java:92-97).  The array therefore lives in device memory between
// calls (SampleArgs::cand_*, sorted_*) and is sorted whole, by a stable descending radix sort on the host side.
#pragma once

#include "kernels.hpp"

namespace l2j {

constexpr int kSampleMaxVocab = 36864;  // the probabilities of one call in LDS: 144 KB
constexpr unsigned long long kJavaRandMult = 0x5DEECE66DULL, kJavaRandMask = (1ULL << 48) - 1;

struct SamplerState {        // the reference's Sampler object, device resident
    unsigned long long rng;  // java.util.Random's 48-bit state
    int n0;                  // candidates of the current sample_topp call
    int nan;                 // a NaN among the probabilities (J/Sampler.java:88-90 throws)
    int result;              // the token of the last call
    int pad;
};

struct SampleArgs {
    float *logits;           // in: logits; out: the probabilities, as the reference leaves them (J/Run.java:647-659)
    int n;
    float temperature, topp;
    float coin;              // >= 0: the caller's Random.nextFloat(); < 0: the context's java.util.Random draws
    int plain;               // topp > 0.999 (J/Run.java:661): sample, else sample_topp
    SamplerState *ss;
    float *cand_prob;        // ProbIndex array as it enters the sort: this call's candidates, then what was there
    int *cand_idx;
    const float *sorted_prob;  // ProbIndex array after the sort
    const int *sorted_idx;
    DevState *st;            // token loop (null outside it): the sampled token replaces the argmax
    int *out_tokens;         //   that k_finish stored for position st->pos - 1
};

// java.util.Random.nextFloat(): next(24) / (float)(1 << 24)
__device__ __forceinline__ float java_next_float(unsigned long long *rng)
{
    const unsigned long long s = (*rng * kJavaRandMult + 0xBULL) & kJavaRandMask;
    *rng = s;
    return __fdiv_rn((float)(int)(s >> 24), 16777216.0f);
}

// Running sums of p[0..n) in element order, in place, by the calling thread alone.  Stops after the
// 64-element chunk at whose end the sum satisfies `STOP_ABOVE ? sum > limit : limit < sum`
// (both are monotone: the terms are not negative).  Returns the number of elements summed; *total = the
// last running sum.  p is 16-byte aligned and padded to a multiple of 8 with zeros.
template <bool WRITE>
__device__ __forceinline__ int chain_sums(float *p, int n, float limit, bool stop_above, bool bounded, float *total)
{
    float acc = 0.0f;
    int i = 0;
    const int n8 = (n + 7) & ~7;
    while (i < n8) {
        const int end = min(n8, i + 64);
#pragma unroll 2
        for (; i < end; i += 8) {
            float4 a = *(const float4 *)(p + i), b = *(const float4 *)(p + i + 4);
            a.x = __fadd_rn(acc, a.x);
            a.y = __fadd_rn(a.x, a.y);
            a.z = __fadd_rn(a.y, a.z);
            a.w = __fadd_rn(a.z, a.w);
            b.x = __fadd_rn(a.w, b.x);
            b.y = __fadd_rn(b.x, b.y);
            b.z = __fadd_rn(b.y, b.z);
            b.w = __fadd_rn(b.z, b.w);
            acc = b.w;
            if (WRITE) {
                *(float4 *)(p + i) = a;
                *(float4 *)(p + i + 4) = b;
            }
        }
        if (bounded && (stop_above ? acc > limit : limit < acc)) break;
    }
    *total = acc;
    return min(i, n);
}

// First index in [0, m) whose running sum s satisfies (above ? s > limit : limit < s), or m if none.
// All threads call; `slot` is an LDS word.
__device__ __forceinline__ int first_past(const float *sums, int m, float limit, bool above, int *slot)
{
    if (threadIdx.x == 0) *slot = m;
    __syncthreads();
    int best = m;
    for (int i = threadIdx.x; i < m; i += blockDim.x) {
        const float s = sums[i];
        if (above ? s > limit : limit < s) { best = i; break; }   // a thread's indices ascend
    }
    if (best < m) atomicMin(slot, best);
    __syncthreads();
    const int r = *slot;
    __syncthreads();
    return r;
}

// J/Run.java:645-659 (divide by the temperature, FindMax, ExpSumNormalize), then either J/Sampler.java:33-44
// (plain) or the candidate filter of J/Sampler.java:85-96.  One workgroup; dynamic LDS: (n rounded up to 8) floats.
__global__ void __launch_bounds__(1024) k_sample_probs(const SampleArgs a)
{
    extern __shared__ __align__(16) float sp[];
    __shared__ float red[16];
    __shared__ int cnt[1024];
    __shared__ float s_sum, s_coin;
    __shared__ int s_slot, s_m;
    const int tid = threadIdx.x, n = a.n, nt = blockDim.x;
    const int n8 = (n + 7) & ~7;

    // logits[q] /= temperature; max
    float mx = -__builtin_inff();
    int bad = 0;
    for (int i = tid; i < n8; i += nt) {
        float v = 0.0f;
        if (i < n) {
            v = __fdiv_rn(a.logits[i], a.temperature);
            bad |= v != v;
            mx = fmaxf(mx, v);
        }
        sp[i] = v;
    }
    mx = block_max(mx, red);
    // x = (float) Math.exp(x - max)
    for (int i = tid; i < n; i += nt) sp[i] = (float)exp((double)__fsub_rn(sp[i], mx));
    __syncthreads();
    // sum += x, in element order
    if (tid == 0) {
        float t;
        chain_sums<false>(sp, n, 0.0f, false, false, &t);
        s_sum = t;
    }
    __syncthreads();
    const float sum = s_sum;
    // if (sum != 0) x /= sum; the probabilities replace the logits
    for (int i = tid; i < n; i += nt) {
        float v = sp[i];
        if (sum != 0.0f) v = __fdiv_rn(v, sum);
        bad |= v != v;
        sp[i] = v;
        a.logits[i] = v;
    }
    if (bad) a.ss->nan = 1;
    __syncthreads();

    if (a.plain) {
        // J/Sampler.java:33-44: the first i with r < cdf(i), else n - 1
        if (tid == 0) {
            float r = a.coin;
            if (r < 0.0f) r = java_next_float(&a.ss->rng);
            s_coin = r;
            float t;
            s_m = chain_sums<true>(sp, n, r, false, true, &t);
        }
        __syncthreads();
        const int m = s_m;
        int pick = first_past(sp, m, s_coin, false, &s_slot);
        if (pick >= m) pick = n - 1;
        if (tid == 0) {
            a.ss->result = pick;
            if (a.st) {
                a.out_tokens[a.st->pos - 1] = pick;
                a.st->token = pick;
            }
        }
        return;
    }

    // J/Sampler.java:85-96: candidates in index order into the front of the ProbIndex array
    const float cutoff = __fdiv_rn(__fsub_rn(1.0f, a.topp), (float)(n - 1));
    const int per = (n + nt - 1) / nt, lo = min(n, tid * per), hi = min(n, lo + per);
    int c = 0;
    for (int i = lo; i < hi; i++) c += sp[i] >= cutoff;
    cnt[tid] = c;
    __syncthreads();
    for (int off = 1; off < nt; off <<= 1) {   // inclusive scan of the per-thread counts
        const int v = tid >= off ? cnt[tid - off] : 0;
        __syncthreads();
        cnt[tid] += v;
        __syncthreads();
    }
    int at = cnt[tid] - c;
    for (int i = lo; i < hi; i++) {
        const float v = sp[i];
        if (v >= cutoff) {
            a.cand_prob[at] = v;
            a.cand_idx[at] = i;
            at++;
        }
    }
    if (tid == nt - 1) a.ss->n0 = cnt[tid];
}

// J/Sampler.java:99-119 on the sorted ProbIndex array.  One workgroup; dynamic LDS: (n0 rounded up to 8) floats,
// n0 <= n.
__global__ void __launch_bounds__(1024) k_topp_pick(const SampleArgs a)
{
    extern __shared__ __align__(16) float sp[];
    __shared__ float s_cum, s_r;
    __shared__ int s_slot, s_m;
    const int tid = threadIdx.x, nt = blockDim.x;
    const int n0 = a.ss->n0;
    if (n0 <= 0) {   // only with NaN probabilities; the host reports the call as failed
        if (tid == 0) a.ss->result = 0;
        return;
    }
    const int n8 = (n0 + 7) & ~7;
    for (int i = tid; i < n8; i += nt) sp[i] = i < n0 ? a.sorted_prob[i] : 0.0f;
    __syncthreads();
    // cumulative_prob += prob until it exceeds topp
    if (tid == 0) {
        float t;
        s_m = chain_sums<true>(sp, n0, a.topp, true, true, &t);
        s_cum = t;
    }
    __syncthreads();
    const int m = s_m;
    int last = first_past(sp, m, a.topp, true, &s_slot);
    if (last >= m) last = n0 - 1;   // never exceeded: all candidates, cumulative_prob = their sum
    if (tid == 0) {
        const float cum = last < m ? sp[last] : s_cum;
        float coin = a.coin;
        if (coin < 0.0f) coin = java_next_float(&a.ss->rng);
        s_r = __fmul_rn(coin, cum);
    }
    __syncthreads();
    // the first i <= last_idx with r < cdf(i), else last_idx
    int pick = first_past(sp, last + 1, s_r, false, &s_slot);
    if (pick > last) pick = last;
    if (tid == 0) {
        const int token = a.sorted_idx[pick];
        a.ss->result = token;
        if (a.st) {
            a.out_tokens[a.st->pos - 1] = token;
            a.st->token = token;
        }
    }
}

// J/Sampler.java:46-57 on an array given by the caller: first index of the strict maximum.  One workgroup.
__global__ void __launch_bounds__(1024) k_argmax_logits(const float *__restrict__ x, int n, SamplerState *ss)
{
    __shared__ float bval[16];
    __shared__ int bidx[16];
    float bv = -__builtin_inff();
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const float v = x[i];
        if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off);
        const int oi = __shfl_xor(bi, off);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if ((threadIdx.x & 63) == 0) { bval[threadIdx.x >> 6] = bv; bidx[threadIdx.x >> 6] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x >> 6); w++)
            if (bval[w] > bv || (bval[w] == bv && bidx[w] < bi)) { bv = bval[w]; bi = bidx[w]; }
        ss->result = bi == 0x7fffffff ? 0 : bi;
    }
}

}  // namespace l2j
