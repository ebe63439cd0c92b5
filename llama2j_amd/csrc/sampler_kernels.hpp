// Sampling of the next token on the device: the temperature / softmax step of J/Run.java:643-665 and
// J/Sampler.java's sample and sample_topp, with the same float32 operations in the same order, so that
// the logits never travel to the host.
//
// The reference adds the probabilities one by one into a float (the softmax denominator, the CDF of
// sample, the cumulative probability of sample_topp); float addition is not associative, so the order
// matters.  As one dependent chain in a single lane such a sum costs 3.4 ns per element (the eight-cycle
// latency of a dependent v_add_f32, measured; 0.11 ms for 32000 probabilities): chain_sums, kept for the head
// of every sum and as a switch (SampleArgs::scan = 0).  By default the sums are formed by chain_scan, which
// reproduces the sequential sums bit for bit from integer prefix sums inside each binade of the running sum
// (about 0.045 ms for 32000 probabilities).  Everything else (divide, max, exp, normalize, candidate filter,
// the search in the running sums) is spread over the workgroup.  The probabilities live in LDS.
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
    int scan;                // 1: the running sums by windows of equal exponent (chain_scan), 0: one lane adds them all
    float *expbuf;           // not null: k_sample_exp has left exp(x / temperature - max) here (n floats)
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

// ---- the same running sums, most of them in parallel -----------------------------------------------------
// While the running sum s of non-negative terms stays in one binade [2^E, 2^(E+1)) every addition rounds to a multiple
// of u = 2^(E-23): s = S * u with an integer S < 2^24, and s + e rounds to (S + a) * u or (S + a + 1) * u, where
// a = floor(e / u), by the fraction e / u - a alone (below, above or equal to 1/2; a tie goes to the even sum, so it
// depends on the parity of S + a).  Inside a binade the sequential float sum is therefore an integer prefix sum whose
// steps depend on nothing but the parity of what came before, which composes: a run of terms maps an incoming parity to
// an increment, (inc0, inc1), and two runs combine as (x0 + y[x0 & 1], x1 + y[(1 + x1) & 1]).  The workgroup scans a tile
// of terms that way, finds the first term whose sum reaches 2^24 * u (it leaves the binade), adds that one term with a real
// float addition and starts over behind it in the new binade.  The results are the reference's sums bit for bit.  A sum
// grows through a binade per doubling, so after a short head that one lane adds (where the sum doubles every few terms)
// a few rounds per tile remain; an input that leaves binades faster than that falls back to the single lane.
constexpr int kScanHead = 1024;      // terms added by one lane before the scan starts
constexpr int kScanPer = 9;          // terms per thread and round; odd: the lanes of a wave then read different LDS banks
                                     // (measured per sampled 7B token: 7: 1.729, 8: 1.740, 9: 1.730, 13: 1.741 ms)
constexpr int kScanMaxRounds = 48;
constexpr int kScanBig = 1 << 25;    // an increment that leaves any binade; sums saturate here

struct ScanShared {
    float sum;
    int i0, cross, send, rounds;
    int w0[16], w1[16];
};

__device__ __forceinline__ int sat_add(int a, int b) { return min(a + b, kScanBig); }

// increments of the integer sum for a term e in the binade E, for an even / odd sum before it
__device__ __forceinline__ void scan_quant(float e, int E, int &inc0, int &inc1)
{
    const unsigned b = __float_as_uint(e), ef = (b >> 23) & 0xffu, m = b & 0x7fffffu;
    if (ef == 0xffu) { inc0 = inc1 = kScanBig; return; }
    const int Ee = ef ? (int)ef - 127 : -126;
    const unsigned M = ef ? (m | 0x800000u) : m;
    const int d = E - Ee;
    if (M == 0u || d >= 25) { inc0 = inc1 = 0; return; }
    if (d < 0) { inc0 = inc1 = kScanBig; return; }
    if (d == 0) { inc0 = inc1 = (int)M; return; }
    const unsigned a = M >> d, rem = M & ((1u << d) - 1u), half = 1u << (d - 1);
    if (rem < half) { inc0 = inc1 = (int)a; }
    else if (rem > half) { inc0 = inc1 = (int)a + 1; }
    else { inc0 = (int)(a + (a & 1u)); inc1 = (int)(a + ((a + 1u) & 1u)); }
}

// S * 2^(E-23) for S < 2^24 (S >= 2^23 unless E = -126)
__device__ __forceinline__ float scan_value(int S, int E)
{
    return __uint_as_float(S >= (1 << 23) ? (((unsigned)(E + 127) << 23) | ((unsigned)S & 0x7fffffu)) : (unsigned)S);
}

// Running sums of p[0..n) in element order (all threads of a 1024-thread workgroup call; p in LDS).  With STORE every
// p[i] is replaced by the sum up to and including it.  Returns the total.
template <bool STORE>
__device__ __forceinline__ float chain_scan(float *p, int n, ScanShared &sh, float *ends)
{
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int h = min(n, kScanHead);
    if (tid == 0) {   // the head: one lane, with the sum after every 32 terms kept
        float acc;
        chain_sums<true>(p, h, ends, 0.0f, false, false, &acc);
        sh.sum = acc; sh.i0 = h; sh.cross = 0x7fffffff; sh.send = 0; sh.rounds = 0;
    }
    if (STORE) {      // the sums inside each step of 32, one thread per step, from the step's exact starting sum
        __syncthreads();
        if (tid * kChainStep < h) {
            float acc = tid ? ends[tid - 1] : 0.0f;
            for (int i = tid * kChainStep; i < min(h, (tid + 1) * kChainStep); i++) {
                acc = __fadd_rn(acc, p[i]);
                p[i] = acc;
            }
        }
    }
    while (true) {
        __syncthreads();
        const int i0 = sh.i0, rounds = sh.rounds;
        const float s = sh.sum;
        if (i0 >= n) break;
        const unsigned sb = __float_as_uint(s), sef = (sb >> 23) & 0xffu;
        if (rounds >= kScanMaxRounds || s == 0.0f || sef == 0xffu) {  // the single lane takes the rest
            __syncthreads();
            if (tid == 0) {
                float acc = s;
                for (int i = i0; i < n; i++) {
                    acc = __fadd_rn(acc, p[i]);
                    if (STORE) p[i] = acc;
                }
                sh.sum = acc; sh.i0 = n;
            }
            continue;
        }
        const int E = sef ? (int)sef - 127 : -126;
        const int S0 = (int)(sef ? ((sb & 0x7fffffu) | 0x800000u) : (sb & 0x7fffffu));
        const int tile_end = min(n, i0 + 1024 * kScanPer), base = i0 + tid * kScanPer;
        int inc0[kScanPer], inc1[kScanPer], t0 = 0, t1 = 0;
#pragma unroll
        for (int k = 0; k < kScanPer; k++) {
            inc0[k] = inc1[k] = 0;
            if (base + k < tile_end) scan_quant(p[base + k], E, inc0[k], inc1[k]);
            t0 = sat_add(t0, (t0 & 1) ? inc1[k] : inc0[k]);
            t1 = sat_add(t1, ((1 + t1) & 1) ? inc1[k] : inc0[k]);
        }
        // inclusive scan of the compositions over the wave, then over the waves
        int x0 = t0, x1 = t1;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int l0 = __shfl_up(x0, off), l1 = __shfl_up(x1, off);
            if (lane >= off) {
                const int n0 = sat_add(l0, (l0 & 1) ? x1 : x0), n1 = sat_add(l1, ((1 + l1) & 1) ? x1 : x0);
                x0 = n0; x1 = n1;
            }
        }
        if (lane == 63) { sh.w0[wave] = x0; sh.w1[wave] = x1; }
        int e0 = __shfl_up(x0, 1), e1 = __shfl_up(x1, 1);   // exclusive within the wave
        if (lane == 0) { e0 = 0; e1 = 0; }
        __syncthreads();
        int q0 = 0, q1 = 0;   // everything before this wave
        for (int w = 0; w < wave; w++) {
            const int y0 = sh.w0[w], y1 = sh.w1[w];
            const int n0 = sat_add(q0, (q0 & 1) ? y1 : y0), n1 = sat_add(q1, ((1 + q1) & 1) ? y1 : y0);
            q0 = n0; q1 = n1;
        }
        const int pre = (S0 & 1) ? q1 : q0;                       // increment up to this wave for the actual parity
        const int Sw = sat_add(S0, pre);
        int S = sat_add(Sw, (Sw & 1) ? e1 : e0);                   // the sum before this thread's terms
        int my_cross = 0x7fffffff, my_pre = 0;
#pragma unroll
        for (int k = 0; k < kScanPer; k++) {
            if (base + k < tile_end && S < (1 << 24)) {
                const int Sn = sat_add(S, (S & 1) ? inc1[k] : inc0[k]);
                if (Sn >= (1 << 24)) {
                    my_cross = base + k; my_pre = S;
                } else {
                    if (STORE) p[base + k] = scan_value(Sn, E);
                    if (base + k == tile_end - 1) sh.send = Sn;
                }
                S = Sn;
            }
        }
        if (my_cross != 0x7fffffff) atomicMin(&sh.cross, my_cross);
        __syncthreads();
        const int cross = sh.cross;
        __syncthreads();
        if (cross != 0x7fffffff) {
            if (my_cross == cross) {   // the term that leaves the binade: a real addition, then on from the term behind it
                const float v = __fadd_rn(scan_value(my_pre, E), p[cross]);
                if (STORE) p[cross] = v;
                sh.sum = v; sh.i0 = cross + 1; sh.cross = 0x7fffffff; sh.rounds = rounds + 1;
            }
        } else if (tid == 0) {
            sh.sum = scan_value(sh.send, E); sh.i0 = tile_end; sh.rounds = rounds + 1;
        }
    }
    __syncthreads();
    return sh.sum;
}

// The first i < m with (above ? p[i] > limit : limit < p[i]) in a non-decreasing p (m if none).  All threads call.
__device__ __forceinline__ int first_over(const float *p, int m, float limit, bool above, int *slot)
{
    if (threadIdx.x == 0) *slot = m;
    __syncthreads();
    const int per = ((m + blockDim.x - 1) / blockDim.x) | 1, lo = min(m, (int)threadIdx.x * per), hi = min(m, lo + per);
    for (int i = lo; i < hi; i++) {
        const float s = p[i];
        if (above ? s > limit : limit < s) { atomicMin(slot, i); break; }
    }
    __syncthreads();
    const int r = *slot;
    __syncthreads();
    return r;
}

// The element-wise front of the step spread over many workgroups (the double-precision exponential of 32000 logits
// takes 0.04 ms on one compute unit): every workgroup divides all the logits by the temperature and takes the maximum
// (the same value everywhere: a maximum does not depend on the order), then exponentiates its own slice into expbuf.
__global__ void __launch_bounds__(1024) k_sample_exp(const SampleArgs a)
{
    __shared__ float red[16];
    const int tid = threadIdx.x, n = a.n, nt = blockDim.x;
    float mx = -__builtin_inff();
    int bad = 0;
    for (int i = tid; i < n; i += nt) {
        const float v = __fdiv_rn(a.logits[i], a.temperature);
        bad |= v != v;
        mx = fmaxf(mx, v);
    }
    mx = block_max(mx, red);
    const int per = (n + gridDim.x - 1) / gridDim.x, lo = blockIdx.x * per, hi = min(n, lo + per);
    for (int i = lo + tid; i < hi; i += nt)
        a.expbuf[i] = (float)exp((double)__fsub_rn(__fdiv_rn(a.logits[i], a.temperature), mx));
    if (bad && blockIdx.x == 0) atomicOr(&a.ss->nan, 1);
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
    __shared__ ScanShared scan;
    const int tid = threadIdx.x, n = a.n, nt = blockDim.x;
    const int np = (n + kChainStep - 1) & ~(kChainStep - 1);

    int bad = 0;
    if (a.expbuf) {
        for (int i = tid; i < np; i += nt) sp[i] = i < n ? a.expbuf[i] : 0.0f;
    } else {
        // logits[q] /= temperature; max
        float mx = -__builtin_inff();
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
    }
    __syncthreads();
    // sum += x, in element order
    if (a.scan) {
        const float t = chain_scan<false>(sp, n, scan, ends);
        if (tid == 0) s_sum = t;
    } else if (tid == 0) {
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
            if (!a.scan) {
                float t;
                s_m = chain_sums<true>(sp, n, ends, r, false, true, &t);
            }
        }
        __syncthreads();
        int pick;
        if (a.scan) {
            chain_scan<true>(sp, n, scan, ends);   // the probabilities are in a.logits by now: sp becomes the cdf
            pick = first_over(sp, n, s_coin, false, &s_slot);
        } else {
            float at;
            pick = first_past(sp, ends, s_m, n, s_coin, false, &s_slot, &s_f, &at);
        }
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
    // (an odd number of elements per thread: the lanes of a wave then read different LDS banks)
    const int per = ((n + nt - 1) / nt) | 1, lo = min(n, tid * per), hi = min(n, lo + per);
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
    __shared__ ScanShared scan;
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
    if (a.scan) {
        // sp becomes the running sums; cumulative_prob is the first of them above topp (else the last), and the cdf of
        // the pick below runs over the same terms from zero again: the same sums
        chain_scan<true>(sp, n0, scan, ends);
        int last = first_over(sp, n0, a.topp, true, &s_slot);
        if (last >= n0) last = n0 - 1;
        if (tid == 0) {
            float coin = a.coin;
            if (coin < 0.0f) coin = java_next_float(&a.ss->rng);
            s_r = __fmul_rn(coin, sp[last]);
        }
        __syncthreads();
        int pick = first_over(sp, last + 1, s_r, false, &s_slot);
        if (pick > last) pick = last;
        if (tid == 0) {
            const int token = a.sorted_idx[pick];
            a.ss->result = token;
            if (a.st) {
                a.out_tokens[a.st->pos - 1] = token;
                a.st->token = token;
            }
        }
        return;
    }
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

// The running sums of x[0..n) by the sampler's routine (scan: chain_scan, else one lane).  One workgroup; dynamic LDS as above.
__global__ void __launch_bounds__(1024) k_running_sums(float *x, int n, int scan_on)
{
    extern __shared__ __align__(16) float sp[];
    __shared__ float ends[kChainMaxSteps];
    __shared__ ScanShared scan;
    const int np = ((n + kChainStep - 1) & ~(kChainStep - 1)) + kChainStep;
    for (int i = threadIdx.x; i < np; i += blockDim.x) sp[i] = i < n ? x[i] : 0.0f;
    __syncthreads();
    if (scan_on) {
        chain_scan<true>(sp, n, scan, ends);
    } else if (threadIdx.x == 0) {
        float acc = 0.0f;
        for (int i = 0; i < n; i++) {
            acc = __fadd_rn(acc, sp[i]);
            sp[i] = acc;
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += blockDim.x) x[i] = sp[i];
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
