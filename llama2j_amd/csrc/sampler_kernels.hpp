// Sampling of the next token on the device: the temperature / softmax step of J/Run.java:643-665 and
// J/Sampler.java's sample and sample_topp, with the same float32 operations in the same order, so that
// the logits never travel to the host.
//
// The reference adds the probabilities one by one into a float (the softmax denominator, the CDF of
// sample, the cumulative probability of sample_topp); float addition is not associative, so the order
// matters.  As one dependent chain in a single lane such a sum costs 3.4 ns per element (the eight-cycle
// latency of a dependent v_add_f32, measured; 0.11 ms for 32000 probabilities): chain_sums, kept as a switch
// (SampleArgs::scan = 0).  By default the sums are formed by spec_sums, which reproduces the sequential sums bit
// for bit from integer prefix sums inside each binade of the running sum.  Everything else (divide, max, exp,
// normalize, candidate filter, the search in the running sums) is spread over the workgroup.  Up to kSampleMaxVocab
// probabilities live in LDS; larger vocabularies are worked on where they are, in device memory.
//
// sample_topp sorts its whole ProbIndex array, not just the candidates of the call: entries of earlier calls
// stay behind them and take part (J/Sampler.java:92-97).  The array therefore lives in device memory between
// calls (SampleArgs::cand_*, sorted_*) and is sorted whole between the two kernels below: by k_sort_tiles, k_merge_tiles
// and k_merge_runs when it fits in LDS, else by k_sort_tiles, k_merge_tiles and as many levels of k_merge_far as it takes.
#pragma once

#include "kernels.hpp"
#include "sampler_state.hpp"

namespace l2j {

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
    int scan;                // 1: the running sums by spec_sums, 0: one lane adds them all (vocabularies that fit in LDS only)
    float *expbuf;           // not null: k_sample_exp has left exp(x / temperature - max) here (n floats)
    int *tok0, *tok1;        // null, or two more places that receive the token
    // Several samplers in one launch (the sequences of the batched decode; nseq 0: one): grid z = sequence.  The fields above
    // are those of sequence 0 (cand_*, sorted_* unused; expbuf null: k_sample_probs forms the exponentials itself, the
    // sequences' workgroups side by side); the arrays of the others follow at these strides.
    int nseq;
    unsigned active;         // bit s: sequence s samples in this step (the others' workgroups leave at once)
    unsigned cur;            // bit s: the copy of its ProbIndex array that sequence s's last top-p step left
    float *pi_prob0, *pi_prob1;   // the two copies, (sequence, pi_stride); named one by one: a member array indexed by a
    int *pi_idx0, *pi_idx1;       // variable would move the whole argument to scratch memory
    long logits_stride, pi_stride;
    int *btoken;             // (sequence): the token goes here (the sequence's next input)
    int *bout;               // and to bout[s * bout_stride]
    long bout_stride;
};

// The arguments of this workgroup's sequence; false: it does not sample in this step.
__device__ __forceinline__ bool sample_seq(SampleArgs &a)
{
    if (a.nseq == 0) return true;
    const int s = blockIdx.z;
    if (!((a.active >> s) & 1u)) return false;
    const bool cur = (a.cur >> s) & 1u;
    a.logits += s * a.logits_stride;
    a.ss += s;
    a.cand_prob = (cur ? a.pi_prob1 : a.pi_prob0) + s * a.pi_stride;
    a.cand_idx = (cur ? a.pi_idx1 : a.pi_idx0) + s * a.pi_stride;
    a.sorted_prob = (cur ? a.pi_prob0 : a.pi_prob1) + s * a.pi_stride;
    a.sorted_idx = (cur ? a.pi_idx0 : a.pi_idx1) + s * a.pi_stride;
    a.tok0 = a.btoken + s;
    a.tok1 = a.bout + s * a.bout_stride;
    return true;
}

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
// an increment, (inc0, inc1), and two runs combine as (x0 + y[x0 & 1], x1 + y[(1 + x1) & 1]).
//
// Which binade the sum is in when it reaches a term is not known in advance, but it can be guessed well: every thread
// takes a contiguous run of terms, a double-precision prefix sum over the threads (any order: it is only a guess) gives
// the sum at both ends of the run, and when both ends lie in one binade the thread reduces its run to (inc0, inc1) for
// that binade ("clean"); else ("dirty": a binade boundary inside the run, zero, denormal, infinite or NaN sums) it
// reduces nothing.  Each wave combines the pairs of its clean threads between one dirty thread and the next (a
// segmented scan).  Then one wave walks the sequence with the real float sum F in hand: a stretch of clean threads whose
// guessed binade is the binade of F, and whose increment keeps F inside it, advances F by integer arithmetic, exactly as
// the additions would have; anything else (a dirty thread, a wrong guess) is added term by term.  A guess is never
// trusted: it only decides how fast F moves.  Sums of 32000 probabilities have about a dozen dirty threads (one per
// doubling of the sum), so the walk has some forty steps; in the worst case (every thread dirty) it is the sequential
// sum.  The results are the reference's sums bit for bit.
constexpr int kSpecThreads = 1024;
constexpr int kSpecBig = 1 << 25;        // an increment that leaves any binade; sums saturate here
constexpr int kSpecIdentity = 254;       // binade code of a stretch of zeros (or of no terms): leaves any sum as it is
constexpr int kSpecNoStop = 1 << 30;

struct SpecShared {
    int x0[kSpecThreads], x1[kSpecThreads];   // per thread: increments of its stretch up to and including it (even / odd sum before)
    float fst[kSpecThreads];                  // the sum before a thread's terms, where the walk has stored it
    unsigned char mm[kSpecThreads];           // binade code of that stretch: 1..253 exponent field, 254 zeros, 0 unusable
    unsigned char took[kSpecThreads];         // at the first thread of a stretch: the walk advanced over it by integers
    double wsum[16];
    unsigned dirty_lo[16], dirty_hi[16];      // per wave: its dirty threads
    float total;                              // the sum of all terms (when the walk did not stop early)
    int t_stop;                               // last thread whose starting sum is known (kSpecNoStop: all)
};

struct SpecThread {
    int lo, hi;      // this thread's terms
    float start;     // the running sum before them
    bool valid;
};

__device__ __forceinline__ int sat_add(int a, int b) { return min(a + b, kSpecBig); }

// F advanced by the increments (c0, c1) guessed for the binade with exponent field m; false when the guess does not
// hold (F is in another binade, or leaves this one on the way): F is then unchanged.
__device__ __forceinline__ bool spec_apply(float &F, int c0, int c1, int m)
{
    const unsigned b = __float_as_uint(F);
    if ((int)(b >> 23) != m) return false;
    const int S = (int)((b & 0x7fffffu) | 0x800000u);
    const int Sn = S + ((S & 1) ? c1 : c0);
    if (Sn >= (1 << 24)) return false;
    F = __uint_as_float(((unsigned)m << 23) | ((unsigned)Sn & 0x7fffffu));
    return true;
}

__device__ __forceinline__ int spec_merge(int a, int b)   // binade code of two stretches in a row
{
    return a == kSpecIdentity ? b : (b == kSpecIdentity || a == b) ? a : 0;
}

__device__ __forceinline__ float spec_uniform(float F)
{
    return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(F)));
}

// F + p[lo] + ... + p[hi - 1], one after the other (every lane of the wave the same)
__device__ __forceinline__ float spec_add_terms(float F, const float *p, int lo, int hi)
{
#pragma unroll 8
    for (int i = lo; i < hi; i++) F = __fadd_rn(F, p[i]);
    return spec_uniform(F);
}

// Starting sums of every thread's terms of p[0..n), in element order (all threads of a 1024-thread workgroup call).
// With `bounded` the walk stops behind the first stretch or thread at whose end the sum exceeds `limit`; later threads
// come back invalid.  sh.total = the whole sum when it did not stop.
__device__ __forceinline__ SpecThread spec_sums(const float *p, int n, SpecShared &sh, float limit, bool bounded)
{
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int T = ((n + kSpecThreads - 1) / kSpecThreads) | 1;   // odd: the lanes of a wave read different LDS banks
    SpecThread me;
    me.lo = min(n, tid * T);
    me.hi = min(n, me.lo + T);
    // the guess: double-precision sums at both ends of the thread's terms
    double loc = 0.0;
#pragma unroll 4
    for (int i = me.lo; i < me.hi; i++) loc += (double)p[i];
    double inc = loc;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const double l = __shfl_up(inc, off);
        if (lane >= off) inc += l;
    }
    if (lane == 63) sh.wsum[wave] = inc;
    __syncthreads();
    double before = 0.0;
    for (int w = 0; w < wave; w++) before += sh.wsum[w];
    const double p_end = before + inc, p_start = p_end - loc;
    const unsigned bs = __float_as_uint((float)p_start) >> 23, be = __float_as_uint((float)p_end) >> 23;
    int m = 0, x0 = 0, x1 = 0;
    if (me.lo >= me.hi || loc == 0.0) {
        m = kSpecIdentity;
    } else if (p_start > 0.0 && bs == be && bs >= 1u && bs <= 253u) {
        m = (int)bs;
        const int shift = 23 - ((int)bs - 127);
#pragma unroll 4
        for (int i = me.lo; i < me.hi; i++) {
            // e / u (NaN becomes the large increment too); off a tie the increment is the nearest integer, whatever the parity
            const float t = fminf(ldexpf(p[i], shift), 33554432.0f);
            const float fl = floorf(t);
            int i0 = (int)rintf(t), i1 = i0;
            if (t - fl == 0.5f) {
                const int a = (int)fl;
                i0 = a + (a & 1);
                i1 = a + (~a & 1);
            }
            x0 = sat_add(x0, (x0 & 1) ? i1 : i0);
            x1 = sat_add(x1, ((1 + x1) & 1) ? i1 : i0);
        }
    }
    // inclusive scan over the wave, started anew behind every dirty thread
    const unsigned long long dirty = __ballot(m == 0);
    int brk = (lane == 0 || ((dirty >> (lane - 1)) & 1ull) || m == 0) ? 1 : 0;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int l0 = __shfl_up(x0, off), l1 = __shfl_up(x1, off), lmb = __shfl_up(m * 2 + brk, off);
        if (lane >= off && !brk) {
            const int n0 = sat_add(l0, (l0 & 1) ? x1 : x0), n1 = sat_add(l1, ((1 + l1) & 1) ? x1 : x0);
            x0 = n0; x1 = n1;
            m = spec_merge(lmb >> 1, m);
            brk = lmb & 1;
        }
    }
    sh.x0[tid] = x0;
    sh.x1[tid] = x1;
    sh.mm[tid] = (unsigned char)m;
    if (lane == 0) {
        sh.dirty_lo[wave] = (unsigned)dirty;
        sh.dirty_hi[wave] = (unsigned)(dirty >> 32);
    }
    if (tid == 0) sh.t_stop = kSpecNoStop;
    __syncthreads();
    // the walk
    if (wave == 0) {
        float F = 0.0f;
        bool stopped = false;
        for (int w = 0; w < kSpecThreads / 64 && !stopped; w++) {
            unsigned long long mask = ((unsigned long long)sh.dirty_hi[w] << 32) | sh.dirty_lo[w];
            const int wx0 = sh.x0[w * 64 + lane], wx1 = sh.x1[w * 64 + lane], wmm = sh.mm[w * 64 + lane];
            int first = 0;   // first thread of the stretch at hand
            while (true) {
                const int d = mask ? __ffsll((long long)mask) - 1 : 64;   // the dirty thread behind it
                if (d > first) {
                    const int t0 = w * 64 + first, t1 = w * 64 + d - 1;
                    const int sm = __builtin_amdgcn_readlane(wmm, d - 1);
                    const float before = F;
                    bool took = sm == kSpecIdentity;
                    if (!took && sm != 0)
                        took = spec_apply(F, __builtin_amdgcn_readlane(wx0, d - 1), __builtin_amdgcn_readlane(wx1, d - 1), sm);
                    sh.fst[t0] = before;   // (every lane the same value)
                    sh.took[t0] = took ? 1 : 0;
                    if (!took) {   // thread by thread, term by term
                        for (int t = t0; t <= t1; t++) {
                            sh.fst[t] = F;
                            F = spec_add_terms(F, p, min(n, t * T), min(n, t * T + T));
                        }
                    }
                    if (bounded && F > limit) {
                        sh.t_stop = t1;
                        stopped = true;
                        break;
                    }
                }
                if (d == 64) break;
                const int t = w * 64 + d;
                sh.fst[t] = F;
                F = spec_add_terms(F, p, min(n, t * T), min(n, t * T + T));
                if (bounded && F > limit) {
                    sh.t_stop = t;
                    stopped = true;
                    break;
                }
                first = d + 1;
                mask &= mask - 1ull;
            }
        }
        sh.total = F;
    }
    __syncthreads();
    me.valid = tid <= sh.t_stop;
    me.start = 0.0f;
    // a thread of a stretch that was taken whole: the sum before the stretch, advanced by the threads before it
    const int e0 = __shfl_up(x0, 1), e1 = __shfl_up(x1, 1), em = __shfl_up(m, 1);
    if (me.valid) {
        const unsigned long long below = dirty & ((1ull << lane) - 1ull);
        const int first = below ? 64 - __clzll((long long)below) : 0;
        const int t0 = wave * 64 + first;
        if (((dirty >> lane) & 1ull) || !sh.took[t0]) {
            me.start = sh.fst[tid];
        } else {
            float F = sh.fst[t0];
            if (lane > first && em != kSpecIdentity) spec_apply(F, e0, e1, em);
            me.start = F;
        }
    }
    return me;
}

// The first i < m whose running sum exceeds `limit` (m if none), *sum_at = that running sum.  All threads call; the
// runs up to that element must be valid.  slot and fslot are LDS words.
__device__ __forceinline__ int spec_first_over(const float *p, const SpecThread &me, int m, float limit, int *slot, float *fslot,
                                               float *sum_at)
{
    if (threadIdx.x == 0) { *slot = m; *fslot = 0.0f; }
    __syncthreads();
    int found = m;
    float at = 0.0f;
    if (me.valid) {
        float acc = me.start;
        const int hi = min(me.hi, m);
#pragma unroll 4
        for (int i = me.lo; i < hi; i++) {   // (no early exit: the loads of an unrolled loop can then go out together)
            acc = __fadd_rn(acc, p[i]);
            if (found == m && acc > limit) { found = i; at = acc; }
        }
        if (found < m) atomicMin(slot, found);
    }
    __syncthreads();
    const int r = *slot;
    if (found < m && found == r) *fslot = at;
    __syncthreads();
    *sum_at = *fslot;
    __syncthreads();
    return r;
}

// The element-wise front of the step spread over many workgroups (the double-precision exponential of 32000 logits
// takes 0.04 ms on one compute unit): every workgroup divides all the logits by the temperature and takes the maximum
// (the same value everywhere: a maximum does not depend on the order), then exponentiates its own slice into expbuf.
static __global__ void __launch_bounds__(1024) k_sample_exp(const SampleArgs a)
{
    __shared__ float red[16];
    const int tid = threadIdx.x, n = a.n, nt = blockDim.x;
    float mx = -__builtin_inff();
    int bad = 0;
    const int n4 = n & ~3;   // (16-byte loads, several in flight: the loop is bound by their latency)
#pragma unroll 4
    for (int i = 4 * tid; i < n4; i += 4 * nt) {
        const float4 x = *reinterpret_cast<const float4 *>(a.logits + i);
        const float v0 = __fdiv_rn(x.x, a.temperature), v1 = __fdiv_rn(x.y, a.temperature);
        const float v2 = __fdiv_rn(x.z, a.temperature), v3 = __fdiv_rn(x.w, a.temperature);
        bad |= (v0 != v0) | (v1 != v1) | (v2 != v2) | (v3 != v3);
        mx = fmaxf(fmaxf(fmaxf(mx, v0), fmaxf(v1, v2)), v3);
    }
    for (int i = n4 + tid; i < n; i += nt) {
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

// dst[0..np) in LDS = src[0..n) followed by zeros; src is 16-byte aligned and readable up to n rounded up to 4, np a
// multiple of 4.  All threads call.
__device__ __forceinline__ void stage_terms(float *dst, const float *src, int n, int np)
{
#pragma unroll 4
    for (int i = 4 * threadIdx.x; i < np; i += 4 * blockDim.x) {
        float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (i < n) v = *reinterpret_cast<const float4 *>(src + i);
        if (i + 1 >= n) v.y = 0.0f;
        if (i + 2 >= n) v.z = 0.0f;
        if (i + 3 >= n) v.w = 0.0f;
        *reinterpret_cast<float4 *>(dst + i) = v;
    }
}

// What the sampler's one-workgroup kernels keep in LDS besides the probabilities; the members are used one after the other.
union SamplerShared {
    SpecShared spec;
    float ends[kChainMaxSteps];
    int cnt[16];
};

// J/Run.java:645-659 (divide by the temperature, FindMax, ExpSumNormalize), then either J/Sampler.java:33-44
// (plain) or the candidate filter of J/Sampler.java:85-96.  One workgroup.  IN_LDS: the probabilities live in LDS
// (dynamic LDS: (n rounded up to 32) + 32 floats, n <= kSampleMaxVocab); else in a.expbuf, where k_sample_exp has
// left the exponentials (any n).
template <bool IN_LDS>
__global__ void __launch_bounds__(1024) k_sample_probs(const SampleArgs a0)
{
    SampleArgs a = a0;
    if (!sample_seq(a)) return;
    extern __shared__ __align__(16) float lds_sp[];
    __shared__ SamplerShared u;
    __shared__ float red[16];
    __shared__ float s_sum, s_coin, s_f;
    __shared__ int s_slot, s_m;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n = a.n, nt = blockDim.x;
    float *sp;
    if constexpr (IN_LDS) sp = lds_sp; else sp = a.expbuf;

    int bad = 0;
    if constexpr (IN_LDS) {
        const int np = (n + kChainStep - 1) & ~(kChainStep - 1);
        if (a.expbuf) {
            stage_terms(sp, a.expbuf, n, np);
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
    }
    // sum += x, in element order
    const bool scan = !IN_LDS || a.scan;
    if (scan) {
        spec_sums(sp, n, u.spec, 0.0f, false);
        if (tid == 0) s_sum = u.spec.total;
    } else if (tid == 0) {
        float t;
        chain_sums<false>(sp, n, nullptr, 0.0f, false, false, &t);
        s_sum = t;
    }
    __syncthreads();
    const float sum = s_sum;
    // if (sum != 0) x /= sum; the probabilities replace the logits
#pragma unroll 4
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
            if (!scan) {
                float t;
                s_m = chain_sums<true>(sp, n, u.ends, r, false, true, &t);
            }
        }
        __syncthreads();
        int pick;
        float at;
        if (scan) {
            const SpecThread me = spec_sums(sp, n, u.spec, s_coin, true);
            pick = spec_first_over(sp, me, n, s_coin, &s_slot, &s_f, &at);
        } else {
            pick = first_past(sp, u.ends, s_m, n, s_coin, false, &s_slot, &s_f, &at);
        }
        if (pick >= n) pick = n - 1;
        if (tid == 0) {
            a.ss->result = pick;
            if (a.tok0) *a.tok0 = pick;
            if (a.tok1) *a.tok1 = pick;
            if (a.st) {
                a.out_tokens[a.st->pos - 1] = pick;
                a.st->token = pick;
            }
        }
        return;
    }

    // J/Sampler.java:85-96: candidates in index order into the front of the ProbIndex array
    const float cutoff = __fdiv_rn(__fsub_rn(1.0f, a.topp), (float)(n - 1));
    // every wave takes a contiguous part of the indices and goes through it 64 at a time, so that the candidates of a
    // step go out to consecutive addresses
    const int per_wave = (((n + nt - 1) / nt) * 64 + 63) & ~63, w_lo = min(n, wave * per_wave), w_hi = min(n, w_lo + per_wave);
    int c = 0;
#pragma unroll 4
    for (int i = w_lo + lane; i < w_hi; i += 64) c += sp[i] >= cutoff;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off);
    if (lane == 0) u.cnt[wave] = c;
    __syncthreads();
    int at = 0, total = 0;
    for (int w = 0; w < nt / 64; w++) {
        const int cw = u.cnt[w];
        if (w < wave) at += cw;
        total += cw;
    }
    if (tid == 0) a.ss->n0 = total;
    for (int i0 = w_lo; i0 < w_hi; i0 += 64) {
        const int i = i0 + lane;
        const float v = i < w_hi ? sp[i] : 0.0f;
        const bool is = i < w_hi && v >= cutoff;
        const unsigned long long m = __ballot(is);
        if (is) {
            const int r = at + __popcll(m & ((1ull << lane) - 1ull));
            a.cand_prob[r] = v;
            a.cand_idx[r] = i;
        }
        at += __popcll(m);
    }
}

// J/Sampler.java:99-119 on the sorted ProbIndex array.  One workgroup.  IN_LDS: the candidates are copied to LDS first
// (dynamic LDS as above, n0 <= n <= kSampleMaxVocab); else they are read where they are.
template <bool IN_LDS>
__global__ void __launch_bounds__(1024) k_topp_pick(const SampleArgs a0)
{
    SampleArgs a = a0;
    if (!sample_seq(a)) return;
    extern __shared__ __align__(16) float lds_sp[];
    __shared__ SamplerShared u;
    __shared__ float s_cum, s_r, s_f;
    __shared__ int s_slot, s_m;
    const int tid = threadIdx.x;
    const int n0 = a.ss->n0;
    if (n0 <= 0) {   // no probability reaches the cutoff (NaNs, or topp near 0 on a flat distribution): the reference
        if (tid == 0) {   // indexes probIndex[-1] and throws; the host reports the call as failed
            a.ss->result = 0;
            a.ss->nan |= 2;
        }
        return;
    }
    const float *sp;
    if constexpr (IN_LDS) {
        const int np = (n0 + kChainStep - 1) & ~(kChainStep - 1);
        stage_terms(lds_sp, a.sorted_prob, n0, np);
        __syncthreads();
        sp = lds_sp;
    } else {
        sp = a.sorted_prob;
    }
    if (!IN_LDS || a.scan) {
        // cumulative_prob is the first running sum above topp (else the last), and the cdf of the pick below runs over
        // the same terms from zero again: the same sums
        const SpecThread me = spec_sums(sp, n0, u.spec, a.topp, true);
        float cum;
        int last = spec_first_over(sp, me, n0, a.topp, &s_slot, &s_f, &cum);
        if (last >= n0) {   // never exceeded: all candidates, cumulative_prob = their sum
            last = n0 - 1;
            cum = u.spec.total;
        }
        if (tid == 0) {
            float coin = a.coin;
            if (coin < 0.0f) coin = java_next_float(&a.ss->rng);
            s_r = __fmul_rn(coin, cum);
        }
        __syncthreads();
        float at;
        int pick = spec_first_over(sp, me, last + 1, s_r, &s_slot, &s_f, &at);
        if (pick > last) pick = last;
        if (tid == 0) {
            const int token = a.sorted_idx[pick];
            a.ss->result = token;
            if (a.tok0) *a.tok0 = token;
            if (a.tok1) *a.tok1 = token;
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
        s_m = chain_sums<true>(sp, n0, u.ends, a.topp, true, true, &t);
        s_cum = t;
    }
    __syncthreads();
    const int steps = s_m;
    float cum;
    int last = first_past(sp, u.ends, steps, n0, a.topp, true, &s_slot, &s_f, &cum);
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
    int pick = first_past(sp, u.ends, min(steps, last / kChainStep + 1), last + 1, s_r, false, &s_slot, &s_f, &at);
    if (pick > last) pick = last;
    if (tid == 0) {
        const int token = a.sorted_idx[pick];
        a.ss->result = token;
        if (a.tok0) *a.tok0 = token;
        if (a.tok1) *a.tok1 = token;
        if (a.st) {
            a.out_tokens[a.st->pos - 1] = token;
            a.st->token = token;
        }
    }
}

// The running sums of x[0..n) by the sampler's routine (scan_on: spec_sums, else one lane).  One workgroup.  IN_LDS: the
// terms are staged in LDS (dynamic LDS as above, n <= kSampleMaxVocab); else they are read where they are (any n).
template <bool IN_LDS>
__global__ void __launch_bounds__(1024) k_running_sums(float *x, int n, int scan_on)
{
    extern __shared__ __align__(16) float lds_sp[];
    __shared__ SamplerShared u;
    const float *sp = x;
    if constexpr (IN_LDS) {
        const int np = ((n + kChainStep - 1) & ~(kChainStep - 1)) + kChainStep;
        for (int i = threadIdx.x; i < np; i += blockDim.x) lds_sp[i] = i < n ? x[i] : 0.0f;
        __syncthreads();
        sp = lds_sp;
    }
    if (!IN_LDS || scan_on) {
        const SpecThread me = spec_sums(sp, n, u.spec, 0.0f, false);
        float acc = me.start;
        for (int i = me.lo; i < me.hi; i++) {
            acc = __fadd_rn(acc, sp[i]);
            x[i] = acc;
        }
    } else if (threadIdx.x == 0) {
        float acc = 0.0f;
        for (int i = 0; i < n; i++) {
            acc = __fadd_rn(acc, sp[i]);
            x[i] = acc;
        }
    }
}

// ---- Arrays.sort(probIndex) (J/Sampler.java:97): stable, by descending probability -------------------------------------
// Three launches, each of which places every pair at its final position within a larger sorted run by counting:
// the rank of a pair is the number of pairs that come before it, i.e. those with a greater probability plus those with
// an equal one that stood earlier (compareTo, J/Sampler.java:64-73, only says greater / less / equal; the sort is stable).
//   k_sort_tiles:   tiles of 256 pairs, every pair compared with the 255 others of its tile;
//   k_merge_tiles:  runs of 16 sorted tiles (4096 pairs): the rank inside the run = the rank inside the tile + what a
//                   binary search counts in each of the 15 other tiles (>= for tiles that stood earlier, > for later ones);
//   k_merge_runs:   the same over the (at most nine) runs, every workgroup holding all keys in LDS;
//   k_merge_far:    larger arrays: sixteen runs at a time become one, level by level, the keys read from device memory.
// Pairs past n (the array is padded to whole runs) carry the key -1 and sort behind everything.
constexpr int kSortTile = 256, kSortRun = 4096, kSortTilesPerRun = kSortRun / kSortTile;

// o >= k is o > the float just below k: a search that counts ">= k" in stretches that stood earlier and "> k" in later
// ones then makes one comparison per probe, against sort_below(k) or k (two comparisons and a choice between their
// results kept the compiler from issuing the probes of a step together).
__device__ __forceinline__ float sort_below(float k)
{
    return __uint_as_float(k > 0.0f ? __float_as_uint(k) - 1u : k == 0.0f ? 0x80000001u : __float_as_uint(k) + 1u);
}

// grid: padded n / 256 workgroups of 256 threads
__device__ __forceinline__ void sort_tiles_of(const float *__restrict__ kin, const int *__restrict__ vin, int n,
                                              float *__restrict__ kout, int *__restrict__ vout)
{
    // a pair stands before another when its probability is greater, or equal and its position lower: one unsigned
    // comparison of (probability bits, 255 - position); the bits of a non-negative float ascend with it, the padding's -1
    // counts as 0 (it stands behind every position of the array anyway)
    __shared__ __align__(16) unsigned long long keys[kSortTile];
    const int tid = threadIdx.x, i = blockIdx.x * kSortTile + tid;
    const float k = i < n ? kin[i] : -1.0f;
    const int v = i < n ? vin[i] : 0;
    const unsigned long long mine = ((unsigned long long)(k < 0.0f ? 0u : __float_as_uint(k)) << 32) | (unsigned)(kSortTile - 1 - tid);
    keys[tid] = mine;
    __syncthreads();
    int rank = 0;
#pragma unroll 16
    for (int j2 = 0; j2 < kSortTile / 2; j2++) {
        const ulonglong2 o = *reinterpret_cast<const ulonglong2 *>(&keys[2 * j2]);
        rank += (o.x > mine) + (o.y > mine);
    }
    kout[blockIdx.x * kSortTile + rank] = k;
    vout[blockIdx.x * kSortTile + rank] = v;
}

// grid: (padded n / 4096, 16) workgroups of 256 threads: a workgroup holds the keys of its run in LDS and places a
// sixteenth of them, one per thread.  The fifteen binary searches of a pair advance together, step by step (their LDS reads are
// independent: one after the other they cost fifteen times the latency).
static __global__ void __launch_bounds__(kSortTile) k_sort_tiles(const float *__restrict__ kin, const int *__restrict__ vin, int n,
                                                          float *__restrict__ kout, int *__restrict__ vout)
{
    sort_tiles_of(kin, vin, n, kout, vout);
}

// The sort for several samplers in one launch (grid z = sequence; SampleArgs says which take part and where their arrays
// lie): a sequence's ProbIndex array goes from the copy its last step left through its own runs into the other copy.
struct SortBatch {
    unsigned active, cur;
    float *pi_prob0, *pi_prob1;   // the two copies of the ProbIndex arrays, (sequence, pi_stride)
    int *pi_idx0, *pi_idx1;
    long pi_stride;
    float *tiles_k, *runs_k;      // (sequence, sort_stride): the sorted tiles, then the sorted runs
    int *tiles_v, *runs_v;
    long sort_stride;
};

static __global__ void __launch_bounds__(kSortTile) k_sort_tiles_b(const SortBatch b, int n)
{
    const int s = blockIdx.z;
    const bool cur = (b.cur >> s) & 1u;
    if (!((b.active >> s) & 1u)) return;
    sort_tiles_of((cur ? b.pi_prob1 : b.pi_prob0) + s * b.pi_stride, (cur ? b.pi_idx1 : b.pi_idx0) + s * b.pi_stride, n,
                  b.tiles_k + s * b.sort_stride, b.tiles_v + s * b.sort_stride);
}

__device__ __forceinline__ void merge_tiles_of(const float *__restrict__ kin, const int *__restrict__ vin, float *__restrict__ kout,
                                               int *__restrict__ vout)
{
    __shared__ __align__(16) float keys[kSortRun];
    const int tid = threadIdx.x, base = blockIdx.x * kSortRun;
#pragma unroll
    for (int q = 0; q < 4; q++)
        *reinterpret_cast<float4 *>(&keys[4 * (tid + 256 * q)]) = *reinterpret_cast<const float4 *>(kin + base + 4 * (tid + 256 * q));
    __syncthreads();
    const int i = blockIdx.y * 256 + tid;
    const float k = keys[i];
    const int v = vin[base + i];
    const int ti = i / kSortTile;
    const float kb = sort_below(k);
    int pos[kSortTilesPerRun];
#pragma unroll
    for (int tj = 0; tj < kSortTilesPerRun; tj++) pos[tj] = 0;
#pragma unroll
    for (int st = kSortTile / 2; st > 0; st >>= 1) {
#pragma unroll
        for (int tj = 0; tj < kSortTilesPerRun; tj++) {
            const float o = keys[tj * kSortTile + pos[tj] + st - 1];
            pos[tj] += o > (tj < ti ? kb : k) ? st : 0;   // tiles that stood earlier win ties
        }
    }
    int rank = i - ti * kSortTile;
#pragma unroll
    for (int tj = 0; tj < kSortTilesPerRun; tj++) {
        const float o = keys[tj * kSortTile + pos[tj]];
        const int cnt = pos[tj] + (o > (tj < ti ? kb : k) ? 1 : 0);
        rank += tj == ti ? 0 : cnt;
    }
    kout[base + rank] = k;
    vout[base + rank] = v;
}

static __global__ void __launch_bounds__(256) k_merge_tiles(const float *__restrict__ kin, const int *__restrict__ vin, float *__restrict__ kout,
                                                     int *__restrict__ vout)
{
    merge_tiles_of(kin, vin, kout, vout);
}

static __global__ void __launch_bounds__(256) k_merge_tiles_b(const SortBatch b)
{
    const int s = blockIdx.z;
    if (!((b.active >> s) & 1u)) return;
    merge_tiles_of(b.tiles_k + s * b.sort_stride, b.tiles_v + s * b.sort_stride, b.runs_k + s * b.sort_stride,
                   b.runs_v + s * b.sort_stride);
}

constexpr int kSortMaxRuns = (kSampleMaxVocab + kSortRun - 1) / kSortRun;

// grid: padded n / 256 workgroups of 256 threads; dynamic LDS: padded n floats.  Only the first n pairs are written.
static __global__ void __launch_bounds__(256) k_merge_runs(const float *__restrict__ kin, const int *__restrict__ vin, int n, int npad,
                                                     float *__restrict__ kout, int *__restrict__ vout)
{
    extern __shared__ __align__(16) float keys[];
    const int tid = threadIdx.x;
#pragma unroll 8
    for (int i = 4 * tid; i < npad; i += 1024) *reinterpret_cast<float4 *>(keys + i) = *reinterpret_cast<const float4 *>(kin + i);
    __syncthreads();
    const int i = blockIdx.x * 256 + tid;
    const float k = keys[i];
    const int v = vin[i];
    const int ri = i / kSortRun, nruns = npad / kSortRun;
    const float kb = sort_below(k);
    int pos[kSortMaxRuns];
#pragma unroll
    for (int rj = 0; rj < kSortMaxRuns; rj++) pos[rj] = 0;
#pragma unroll
    for (int st = kSortRun / 2; st > 0; st >>= 1) {
#pragma unroll
        for (int rj = 0; rj < kSortMaxRuns; rj++) {
            if (rj < nruns) {
                const float o = keys[rj * kSortRun + pos[rj] + st - 1];
                pos[rj] += o > (rj < ri ? kb : k) ? st : 0;
            }
        }
    }
    int rank = i - ri * kSortRun;
#pragma unroll
    for (int rj = 0; rj < kSortMaxRuns; rj++) {
        if (rj < nruns && rj != ri) {
            const float o = keys[rj * kSortRun + pos[rj]];
            rank += pos[rj] + (o > (rj < ri ? kb : k) ? 1 : 0);
        }
    }
    if (rank < n) {
        kout[rank] = k;
        vout[rank] = v;
    }
}

// The same step for arrays that do not fit in LDS: the keys stay in device memory (the caches hold them).  The array
// consists of sorted runs of run_len pairs; a launch merges every group of group_len / run_len neighbouring runs (at
// most kSortFanIn) into one run of group_len pairs.  The last run of the array may be shorter.  Pairs whose rank is nout
// or more are dropped (the padding, at the last level).  The sixteen searches of a pair advance together.
// grid: padded n / 256 workgroups of 256 threads; run_len and group_len are powers of two, npad a multiple of 256.
constexpr int kSortFanIn = 16;

template <int FANIN = kSortFanIn>
__device__ __forceinline__ void merge_far_of(const float *__restrict__ kin, const int *__restrict__ vin, int npad, int nout,
                                             int run_len, int group_len, float *__restrict__ kout, int *__restrict__ vout)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    const float k = kin[i];
    const int v = vin[i];
    const int g0 = i & ~(group_len - 1);
    const int off = i - g0, ri = off / run_len;
    const int gend = min(npad, g0 + group_len);
    int rank = g0 + off - ri * run_len;
    int pos[FANIN], len[FANIN];
#pragma unroll
    for (int u = 0; u < FANIN; u++) {
        len[u] = max(0, min(run_len, gend - g0 - u * run_len));   // 0: no such run in this group
        pos[u] = 0;
    }
    const float *run = kin + g0;
    const float kb = sort_below(k);
    for (int st = run_len >> 1; st > 0; st >>= 1) {
#pragma unroll
        for (int u = 0; u < FANIN; u++) {
            const int at = pos[u] + st - 1;
            const float o = run[min(u * run_len + at, gend - g0 - 1)];
            pos[u] += (at < len[u] && o > (u < ri ? kb : k)) ? st : 0;   // runs that stood earlier win ties
        }
    }
#pragma unroll
    for (int u = 0; u < FANIN; u++) {
        const float o = run[min(u * run_len + pos[u], gend - g0 - 1)];
        const int cnt = pos[u] + ((pos[u] < len[u] && o > (u < ri ? kb : k)) ? 1 : 0);
        rank += u != ri ? cnt : 0;
    }
    if (rank < nout) {
        kout[rank] = k;
        vout[rank] = v;
    }
}

static __global__ void __launch_bounds__(256) k_merge_far(const float *__restrict__ kin, const int *__restrict__ vin, int npad, int nout,
                                                    int run_len, int group_len, float *__restrict__ kout, int *__restrict__ vout)
{
    merge_far_of(kin, vin, npad, nout, run_len, group_len, kout, vout);
}

// The last merge of k_sort_tiles_b's sort (at most kSortFanIn runs of kSortRun pairs: padded n up to 65536): the runs of a
// sequence into the other copy of its ProbIndex array, the keys read where they lie (32 sequences' keys fit the caches;
// holding a sequence's keys in LDS as k_merge_runs does would leave one workgroup per compute unit).
static __global__ void __launch_bounds__(256) k_merge_far_b(const SortBatch b, int npad, int nout)
{
    const int s = blockIdx.z;
    const bool cur = (b.cur >> s) & 1u;
    if (!((b.active >> s) & 1u)) return;
    const float *kin = b.runs_k + s * b.sort_stride;
    const int *vin = b.runs_v + s * b.sort_stride;
    float *kout = (cur ? b.pi_prob0 : b.pi_prob1) + s * b.pi_stride;
    int *vout = (cur ? b.pi_idx0 : b.pi_idx1) + s * b.pi_stride;
    if (npad <= 8 * kSortRun) merge_far_of<8>(kin, vin, npad, nout, kSortRun, kSortRun * kSortFanIn, kout, vout);   // (eight searches per pair)
    else merge_far_of<kSortFanIn>(kin, vin, npad, nout, kSortRun, kSortRun * kSortFanIn, kout, vout);
}

// J/Sampler.java:46-57 on an array given by the caller: first index of the strict maximum.  One workgroup.
static __global__ void __launch_bounds__(1024) k_argmax_logits(const float *__restrict__ x, int n, SamplerState *ss)
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
