// Sampling of the next token on the device: the temperature / softmax step of J/Run.java:643-665 and
// J/Sampler.java's sample and sample_topp, with the same float32 operations in the same order, so that
// the logits never travel to the host.
//
// The reference adds the probabilities one by one into a float (the softmax denominator, the CDF of
// sample, the cumulative probability of sample_topp); float addition is not associative, so those sums
// run here as one dependent chain in a single lane (3.4 ns per element: the eight-cycle latency of a
// dependent v_add_f32, measured; 0.11 ms for 32000 probabilities) and everything else
// (divide, max, exp, normalize, candidate filter, the search in the running sums) is spread over the
// workgroup.  The probabilities live in LDS; the chain keeps its running sum after every 32 elements, stops
// at the end of the step in which the sum passes the draw / topp, and the first element past it is
// then found from those step sums.
//
// sample_topp sorts its whole ProbIndex array, not just the candidates of the call: entries of earlier calls
// stay behind them and take part (J/Sampler.java:92-97).  The array therefore lives in device memory between
// calls (SampleArgs::cand_*, sorted_*) and is sorted whole by rocPRIM's stable descending sort of (key, value) pairs,
// which the host launches between the two kernels below.
#pragma once

#include "kernels.hpp"

namespace l2j {

constexpr int kSampleMaxVocab = 36864;  // the probabilities of one call in LDS: 144 KB
constexpr unsigned long long kJavaRandMult = 0x5DEECE66DULL, kJavaRandMask = (1ULL << 48) - 1;

struct SamplerState {        // the reference's Sampler object, device resident
    unsigned long long rng;  // java.util.Random's 48-bit state
    int n0;                  // candidates of the current sample_topp call
    int nan;                 // bit 0: a NaN among the probabilities (J/Sampler.java:88-90 throws); bit 1: no top-p candidate
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

// Sum of p[0..n) in element order by the calling thread alone; ends[k] (if not null) receives the running sum
// after step k of 32 elements.  With `bounded` it stops after the step at whose end the sum satisfies
// `stop_above ? sum > limit : limit < sum` (monotone: the terms are not negative).  Returns the number of steps
// done; *total = the last running sum.  p is 16-byte aligned, padded to a multiple of 32 with zeros and followed by
// one more step of readable padding.  The next
// 32 elements are fetched from LDS while the current ones are added, and nothing but the additions and one
// store per step is issued in between: a lone wavefront issues an instruction every four cycles or so, so
// every instruction beside the dependent additions lengthens the chain.
constexpr int kChainStep = 32;
constexpr int kChainMaxSteps = kSampleMaxVocab / kChainStep;

struct ChainRegs {
    float4 v[kChainStep / 4];
};

__device__ __forceinline__ void chain_load(ChainRegs &r, const float *p)
{
#pragma unroll
    for (int u = 0; u < kChainStep / 4; u++) r.v[u] = *(const float4 *)(p + 4 * u);
}

__device__ __forceinline__ float chain_step(const ChainRegs &r, float acc)
{
#pragma unroll
    for (int u = 0; u < kChainStep / 4; u++) {
        acc = __fadd_rn(acc, r.v[u].x);
        acc = __fadd_rn(acc, r.v[u].y);
        acc = __fadd_rn(acc, r.v[u].z);
        acc = __fadd_rn(acc, r.v[u].w);
    }
    return acc;
}

template <bool ENDS>
__device__ __forceinline__ int chain_sums(const float *p, int n, float *ends, float limit, bool stop_above, bool bounded, float *total)
{
    const int steps = (n + kChainStep - 1) / kChainStep;
    ChainRegs ra, rb;
    float acc = 0.0f;
    int k = 0;
    chain_load(ra, p);
    while (k < steps) {
        // The loads are unconditional (hence the step of padding) and fenced: behind a branch the compiler would
        // wait for them before it uses the older ones, and left alone it moves them down next to their use.
        chain_load(rb, p + (k + 1) * kChainStep);
        __builtin_amdgcn_sched_barrier(0);
        acc = chain_step(ra, acc);
        if (ENDS) ends[k] = acc;
        k++;
        if (k >= steps || (bounded && (stop_above ? acc > limit : limit < acc))) break;
        chain_load(ra, p + (k + 1) * kChainStep);
        __builtin_amdgcn_sched_barrier(0);
        acc = chain_step(rb, acc);
        if (ENDS) ends[k] = acc;
        k++;
        if (bounded && (stop_above ? acc > limit : limit < acc)) break;
    }
    *total = acc;
    return k;
}

// The first element i < m (m within the `steps` steps summed) whose running sum s satisfies
// (above ? s > limit : limit < s), found from the step-end sums: all threads look for the first step whose end
// passes, thread 0 then walks that step.  Returns the index (m if none); *sum_at = its running sum.  All threads
// call; slot and fslot are LDS words.
__device__ __forceinline__ int first_past(const float *p, const float *ends, int steps, int m, float limit, bool above, int *slot,
                                          float *fslot, float *sum_at)
{
    if (threadIdx.x == 0) *slot = steps;
    __syncthreads();
    for (int k = threadIdx.x; k < steps; k += blockDim.x) {
        const float s = ends[k];
        if (above ? s > limit : limit < s) {   // a thread's indices ascend
            atomicMin(slot, k);
            break;
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const int k = *slot;
        int found = m;
        float acc = 0.0f;
        if (k < steps) {
            acc = k > 0 ? ends[k - 1] : 0.0f;
            for (int i = k * kChainStep; i < min(m, (k + 1) * kChainStep); i++) {
                acc = __fadd_rn(acc, p[i]);
                if (above ? acc > limit : limit < acc) { found = i; break; }
            }
        }
        *slot = found;
        *fslot = acc;
    }
    __syncthreads();
    const int r = *slot;
    *sum_at = *fslot;
    __syncthreads();
    return r;
}

// J/Run.java:645-659 (divide by the temperature, FindMax, ExpSumNormalize), then either J/Sampler.java:33-44
// (plain) or the candidate filter of J/Sampler.java:85-96.  One workgroup; dynamic LDS: (n rounded up to 32) + 32 floats.
__global__ void __launch_bounds__(1024) k_sample_probs(const SampleArgs a)
{
    extern __shared__ __align__(16) float sp[];
    __shared__ float ends[kChainMaxSteps];
    __shared__ float red[16];
    __shared__ int cnt[1024];
    __shared__ float s_sum, s_coin, s_f;
    __shared__ int s_slot, s_m;
    const int tid = threadIdx.x, n = a.n, nt = blockDim.x;
    const int np = (n + kChainStep - 1) & ~(kChainStep - 1);

    // logits[q] /= temperature; max
    float mx = -__builtin_inff();
    int bad = 0;
    for (int i = tid; i < np; i += nt) {
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
        chain_sums<false>(sp, n, nullptr, 0.0f, false, false, &t);
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
    if (bad) atomicOr(&a.ss->nan, 1);
    __syncthreads();

    if (a.plain) {
        // J/Sampler.java:33-44: the first i with r < cdf(i), else n - 1
        if (tid == 0) {
            float r = a.coin;
            if (r < 0.0f) r = java_next_float(&a.ss->rng);
            s_coin = r;
            float t;
            s_m = chain_sums<true>(sp, n, ends, r, false, true, &t);
        }
        __syncthreads();
        float at;
        int pick = first_past(sp, ends, s_m, n, s_coin, false, &s_slot, &s_f, &at);
        if (pick >= n) pick = n - 1;
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

// J/Sampler.java:99-119 on the sorted ProbIndex array.  One workgroup; dynamic LDS: (n rounded up to 32) + 32 floats,
// n0 <= n.
__global__ void __launch_bounds__(1024) k_topp_pick(const SampleArgs a)
{
    extern __shared__ __align__(16) float sp[];
    __shared__ float ends[kChainMaxSteps];
    __shared__ float s_cum, s_r, s_f;
    __shared__ int s_slot, s_m;
    const int tid = threadIdx.x, nt = blockDim.x;
    const int n0 = a.ss->n0;
    if (n0 <= 0) {   // no probability reaches the cutoff (NaNs, or topp near 0 on a flat distribution): the reference
        if (tid == 0) {   // indexes probIndex[-1] and throws; the host reports the call as failed
            a.ss->result = 0;
            a.ss->nan |= 2;
        }
        return;
    }
    const int np = (n0 + kChainStep - 1) & ~(kChainStep - 1);
    for (int i = tid; i < np; i += nt) sp[i] = i < n0 ? a.sorted_prob[i] : 0.0f;
    __syncthreads();
    // cumulative_prob += prob until it exceeds topp
    if (tid == 0) {
        float t;
        s_m = chain_sums<true>(sp, n0, ends, a.topp, true, true, &t);
        s_cum = t;
    }
    __syncthreads();
    const int steps = s_m;
    float cum;
    int last = first_past(sp, ends, steps, n0, a.topp, true, &s_slot, &s_f, &cum);
    if (last >= n0) {   // never exceeded: all candidates, cumulative_prob = their sum
        last = n0 - 1;
        cum = s_cum;
    }
    if (tid == 0) {
        float coin = a.coin;
        if (coin < 0.0f) coin = java_next_float(&a.ss->rng);
        s_r = __fmul_rn(coin, cum);
    }
    __syncthreads();
    // the first i <= last_idx with r < cdf(i), else last_idx
    float at;
    int pick = first_past(sp, ends, min(steps, last / kChainStep + 1), last + 1, s_r, false, &s_slot, &s_f, &at);
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
