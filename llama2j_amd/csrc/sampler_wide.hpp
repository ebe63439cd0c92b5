// The sampling step of J/Run.java:643-665 and J/Sampler.java:33-44, 76-120 as ONE launch spread over many workgroups
// (vocabularies that fit in LDS; sampler_kernels.hpp has the launch-per-stage form, which larger ones take).
//
// A workgroup of 256 threads owns a slice of 256 consecutive terms; the stages are separated by grid barriers (a counter
// that only grows during the launch; the last workgroup to leave clears it).  What one stage hands to the next is stored
// write-through and read with device-coherent loads.
//
//   A  max, exp((double)(x / t - max)) of the slice, and the slice reduced for the sequential float sum (below; the guess
//      it needs, the sum of what stands before the slice, from fast exponentials of the logits the maximum was taken of)
//   C  every workgroup walks the slices (the same walk everywhere: nobody waits for a result), divides its slice by
//      the sum, writes the probabilities over the logits and flags its top-p candidates (J/Sampler.java:85-96)
//   D  the ProbIndex array of this call (candidates in index order, then what the last call left, which is sorted)
//      taken tile by tile and every tile of 256 sorted by counting
//   E  runs of 16 tiles merged by counting (binary searches in LDS), F all runs merged: Arrays.sort, stable, descending
//   G  the sorted candidates reduced like A's slices; then workgroup 0 walks them until the sum exceeds topp, draws
//      (java.util.Random), and walks again until the sum exceeds r (J/Sampler.java:99-119)
// sample (topp > 0.999) is A, C, a reduction of the probabilities and one walk until the sum exceeds the draw.
//
// The sequential float sums.  spec_sums (sampler_kernels.hpp) explains the arithmetic: inside a binade of the running
// sum a run of terms is a pair of integer increments (for an even / odd sum before it), pairs compose, and the binade a
// run will meet is guessed from double-precision sums; a guess is never trusted, the walk checks it against the real sum
// and adds term by term where it does not hold.  Here the runs have two levels.  Level 0: a lane holds four terms, a
// wave the 64 lanes of a slice; neighbouring lanes with the same guessed binade form a segment, and a segmented scan
// leaves in every lane the pair of its segment up to and including it.  Level 1: a slice whose 64 lanes are one segment
// is a single pair ("uniform"); the walker scans those the same way, 64 slices per lane-parallel step.  A walk is then
// a few dozen steps: per binade of the sum one stretch of uniform slices taken by integer arithmetic and one mixed slice
// entered lane segment by lane segment.  The steps are first written down as a list (wide_plan, lane-parallel) and then
// taken from registers one after the other (wide_run: a lone wave needs 0.1 us for a step whatever it does, so nothing but
// the steps themselves is left in that loop).  Where the sum first exceeds a limit is found by the walk that takes no list
// (wide_walk), started again at the slice the step belongs to: the stretch that crosses, then (every lane advancing the
// stretch's start by the pair before it) the slice, the lane, the term.
//
// What the stages cost on an MI355X (vocabulary 32000, flat distribution, in-kernel time stamps): a grid barrier of 125
// workgroups 2.5-3 us (arrivals counted per group of sixteen at the time; one counter took 3.5-6 us, an atomic on one address every ~30 ns), a
// dependent device-coherent load 1-2.5 us, A 4.3, B 1.6, staging + plan 7.7, the walk 6.8, D 4.8, E 3.2, F 7.0 (4.7 of it
// the 128 KB of keys every workgroup fetches), G 3.2, the two walks of the pick 8.5 + 3.8: 77 us, against 105 us for the
// six launches of the launch-per-stage form as it was, 88 us now that its sort probes the same way as E and F here.
#pragma once

#include "phase_kernels.hpp"
#include "sampler_kernels.hpp"

namespace l2j {

constexpr int kWideSlice = 256;                                // terms of a slice = threads of a workgroup
constexpr int kWideMaxSlices = kSampleMaxVocab / kWideSlice;   // 144
constexpr int kWideSlots = 16;                                 // mixed slices staged in LDS ahead of a walk
constexpr int kWideItems = 192;                                // steps of a planned walk

constexpr int kWideGroups = 4;   // arrivals are counted per group of workgroups first: a counter takes one atomic every ~30 ns
                                 // (per sampled token: 2, 3, 4 groups the same, 8 +1.3 us, 16 +5 us, one counter +12 us)
struct WideSync {
    unsigned ctr;    // groups that have arrived at the barriers of the launch in flight
    unsigned pad0[15];
    unsigned done;   // workgroups that have left their last barrier
    unsigned pad1[15];
    int fault;       // a bounded wait ran out
    int pad2[15];
    struct { unsigned n; unsigned pad[15]; } group[kWideGroups];   // arrivals per group (workgroup g: group g % kWideGroups)
};

// Device memory of a launch besides the arrays of SampleArgs.  The reductions exist twice: a workgroup may write its
// second one while others still walk the first.
struct WideWs {
    double *ssum;               // [slices] double-precision sum of a slice's terms (k_sum_probe)
    int *t_x0, *t_x1, *t_m;     // [2][slices] a slice as one pair; t_m 0: not uniform
    unsigned long long *seg;    // [2][slices] lanes that start a segment
    int *d_x0, *d_x1, *d_m;     // [2][slices * 64] per lane: the pair of its segment up to and including it, its binade code
    unsigned long long *cmask;  // [slices * 4] which terms of a slice are top-p candidates
    WideSync *sync;
    int maxspin;
};

struct WideArgs {
    float *logits;              // in: logits; out: probabilities
    int n;
    float temperature, topp, coin;
    int plain;
    SamplerState *ss;
    const float *old_prob;      // the ProbIndex array as the last call left it
    const int *old_idx;
    float *new_prob;            // and as this call leaves it
    int *new_idx;
    float *k0, *k1;             // the sort's tiles and runs
    int *v0, *v1;
    float *expbuf;              // slices * 256 floats
    DevState *st;
    int *out_tokens;
    WideWs w;
};

// Before: every thread's stores for the other workgroups are issued.  k counts the barriers of the launch from 0.
__device__ __forceinline__ void wide_barrier(const WideWs &w, unsigned k)
{
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned ng = min((unsigned)kWideGroups, gridDim.x), grp = blockIdx.x % ng;
        const unsigned gsize = (gridDim.x - grp + ng - 1) / ng;
        const unsigned old = __hip_atomic_fetch_add(&w.sync->group[grp].n, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (old + 1u == gsize * (k + 1u)) __hip_atomic_fetch_add(&w.sync->ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned want = (k + 1u) * ng;
        int spins = 0;
        while (__hip_atomic_load(&w.sync->ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < want) {
            __builtin_amdgcn_s_sleep(1);
            if (++spins > w.maxspin || ((spins & 255) == 0 && ld_coh(&w.sync->fault) != 0)) {
                st_coh(&w.sync->fault, 1);
                break;
            }
        }
    }
    __syncthreads();
}

// The last workgroup to get here (all have then left every barrier) clears the counters for the next launch.
__device__ __forceinline__ void wide_leave(const WideWs &w, SamplerState *ss)
{
    if (threadIdx.x == 0) {
        if (ld_coh(&w.sync->fault) != 0) atomicOr(&ss->nan, 4);
        const unsigned old = __hip_atomic_fetch_add(&w.sync->done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (old + 1u == gridDim.x) {
            __hip_atomic_store(&w.sync->ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&w.sync->done, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            for (int q = 0; q < kWideGroups; q++) __hip_atomic_store(&w.sync->group[q].n, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// Terms idx .. idx + 3 of p[0..count) (zeros past the end), device-coherent; p is 16-byte aligned, idx a multiple of 4.
__device__ __forceinline__ float4 wide_terms(const float *p, int idx, int count)
{
    if (idx + 3 < count) return ld_coh16(p + idx);
    float4 t = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (idx < count) t.x = ld_coh(p + idx);
    if (idx + 1 < count) t.y = ld_coh(p + idx + 1);
    if (idx + 2 < count) t.z = ld_coh(p + idx + 2);
    return t;
}

// One more term e of a run whose sum stays in the binade with 2^shift units per 1.0: the increments of the run for an
// even (x0) and an odd (x1) sum before it.
__device__ __forceinline__ void wide_term(int &x0, int &x1, float e, int shift)
{
    // e / u (NaN becomes the large increment too); off a tie the increment is the nearest integer, whatever the parity
    const float t = fminf(ldexpf(e, shift), 33554432.0f);
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

// Lanes 0 .. count - 1 of the wave hold a run each: its pair (x0, x1) and binade code m (0: unusable, kSpecIdentity:
// nothing but zeros).  Neighbours with the same usable code form a segment; on return every lane holds the pair of its
// segment up to and including itself.  Returns the lanes that start a segment.
__device__ __forceinline__ unsigned long long wide_segscan(int &x0, int &x1, int m, int count)
{
    const int lane = threadIdx.x & 63;
    const int pm = __shfl_up(m, 1);
    int brk = (lane == 0 || lane >= count || m == 0 || pm == 0 || m != pm) ? 1 : 0;
    unsigned long long segs = __ballot(brk);
    if (count < 64) segs &= (1ull << count) - 1ull;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int l0 = __shfl_up(x0, off), l1 = __shfl_up(x1, off), lb = __shfl_up(brk, off);
        if (lane >= off && !brk) {
            const int n0 = sat_add(l0, (l0 & 1) ? x1 : x0), n1 = sat_add(l1, ((1 + l1) & 1) ? x1 : x0);
            x0 = n0;
            x1 = n1;
            brk = lb;
        }
    }
    return segs;
}

// Level 0 of slice g by one wave: lane l holds the terms 4 l .. 4 l + 3 of the slice, base = the (double-precision,
// approximate) sum of everything before the slice.  Leaves the lanes' scanned pairs and the slice's own pair in set `set`.
__device__ __forceinline__ void wide_reduce(const WideWs &w, int set, int g, float4 t, double base, double mark = -1.0)
{
    const int lane = threadIdx.x & 63;
    const double loc = (double)t.x + (double)t.y + (double)t.z + (double)t.w;
    double inc = loc;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const double l = __shfl_up(inc, off);
        if (lane >= off) inc += l;
    }
    const double p_end = base + inc, p_start = p_end - loc;
    const unsigned bs = __float_as_uint((float)p_start) >> 23, be = __float_as_uint((float)p_end) >> 23;
    int m = 0, x0 = 0, x1 = 0;
    if (loc == 0.0) {
        m = kSpecIdentity;
    } else if (p_start > 0.0 && bs == be && bs >= 1u && bs <= 253u) {
        m = (int)bs;
        const int shift = 23 - ((int)bs - 127);
        wide_term(x0, x1, t.x, shift);
        wide_term(x0, x1, t.y, shift);
        wide_term(x0, x1, t.z, shift);
        wide_term(x0, x1, t.w, shift);
    }
    const unsigned long long segs = wide_segscan(x0, x1, m, 64);
    const long at = ((long)set * kWideMaxSlices + g) * 64 + lane;
    st_coh(w.d_x0 + at, x0);
    st_coh(w.d_x1 + at, x1);
    st_coh(w.d_m + at, m);
    if (lane == 63) {
        const int s = set * kWideMaxSlices + g;
        st_coh(w.t_x0 + s, x0);
        st_coh(w.t_x1 + s, x1);
        // (a slice near which the sum is expected to pass `mark` is handed over as not uniform: the walker stages those
        // in LDS, and the walk that looks for the crossing inside it finds its lanes there instead of in memory)
        const bool near = mark >= 0.0 && base <= mark * 1.002 && p_end >= mark * 0.998;
        st_coh(w.t_m + s, (segs == 1ull && !near) ? m : 0);
        st_coh(w.seg + s, segs);
    }
}

// What a walking workgroup keeps in LDS: every slice's pair, and the lanes and terms of the first kWideSlots slices
// that are not uniform (the walk enters those; fetching them from memory one after the other would cost a round trip each).
struct WideWalk {
    int t_x0[kWideMaxSlices], t_x1[kWideMaxSlices], t_m[kWideMaxSlices];
    int slot_s[kWideSlots];
    int s_x0[kWideSlots][64], s_x1[kWideSlots][64], s_m[kWideSlots][64];
    float4 s_t[kWideSlots][64];
    unsigned long long s_seg[kWideSlots];
    unsigned char slot_of[kWideMaxSlices];
    int nslots;
    // the plan: the walk's steps one after the other, see wide_plan
    int it_m[kWideItems], it_a[kWideItems], it_b[kWideItems], it_c[kWideItems], it_d[kWideItems], it_at[kWideItems];
    float it_fb[kWideItems];   // the sum before a step, as the last planned walk found it
    int nrun;      // steps of the plan before which the last planned walk has left its sum in it_fb
    int nitems;    // -1: no plan (too many steps, or a slice that is not uniform is not staged)
    float total;   // a walk's results: the sum where it ended,
    int hit;       //   the first term whose running sum exceeded the limit (-1: none),
    float at;      //   and that sum
};

// All threads: set `set` of the first nsl slices of terms[0..count) into L.
__device__ __forceinline__ void wide_stage(const WideWs &w, int set, WideWalk &L, int nsl, const float *terms, int count)
{
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nw = blockDim.x >> 6;
    const int sb = set * kWideMaxSlices;
    if (tid < nsl) {
        L.t_x0[tid] = ld_coh(w.t_x0 + sb + tid);
        L.t_x1[tid] = ld_coh(w.t_x1 + sb + tid);
        L.t_m[tid] = ld_coh(w.t_m + sb + tid);
    }
    __syncthreads();
    if (wave == 0) {
        int base = 0;
        for (int c = 0; c * 64 < nsl; c++) {
            const int s = c * 64 + lane;
            const bool mixed = s < nsl && L.t_m[s] == 0;
            const unsigned long long b = __ballot(mixed);
            const int slot = base + __popcll(b & ((1ull << lane) - 1ull));
            if (s < nsl) L.slot_of[s] = (unsigned char)((mixed && slot < kWideSlots) ? slot : 255);
            if (mixed && slot < kWideSlots) L.slot_s[slot] = s;
            base += __popcll(b);
        }
        if (lane == 0) L.nslots = min(base, kWideSlots);
    }
    __syncthreads();
    for (int k = wave; k < L.nslots; k += nw) {
        const int s = L.slot_s[k];
        const long at = ((long)sb + s) * 64 + lane;
        L.s_x0[k][lane] = ld_coh(w.d_x0 + at);
        L.s_x1[k][lane] = ld_coh(w.d_x1 + at);
        L.s_m[k][lane] = ld_coh(w.d_m + at);
        L.s_t[k][lane] = wide_terms(terms, s * kWideSlice + 4 * lane, count);
        if (lane == 0) L.s_seg[k] = ld_coh(w.seg + sb + s);
    }
    __syncthreads();
}

__device__ __forceinline__ int wide_rl(int v, int lane) { return __builtin_amdgcn_readlane(v, lane); }
__device__ __forceinline__ float wide_rl(float v, int lane) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane)); }

// One level of a walk (one wave, every lane the same F).  Lanes 0 .. count - 1 hold the members: m their binade code,
// (sx0, sx1) the scanned pair, (ox0, ox1) the member's own (OWN; else a member of a segment that cannot be taken whole
// goes straight to leaf).  leaf(j, F) advances F over member j piece by piece and returns true when the sum exceeded the
// limit inside it (it records where).  Returns true when the limit was exceeded.
template <bool OWN, class Leaf>
__device__ __forceinline__ bool wide_level(float &F, int count, int ox0, int ox1, int sx0, int sx1, int m, unsigned long long segs,
                                           float limit, bool bounded, Leaf &&leaf)
{
    const int lane = threadIdx.x & 63;
    while (segs) {
        const int first = __ffsll((long long)segs) - 1;
        segs &= segs - 1ull;
        const int last = (segs ? __ffsll((long long)segs) - 1 : count) - 1;
        const int sm = wide_rl(m, last);
        const float before = F;
        bool took = sm == kSpecIdentity;
        if (!took && sm != 0) took = spec_apply(F, wide_rl(sx0, last), wide_rl(sx1, last), sm);
        F = spec_uniform(F);
        if (took) {
            if (bounded && F > limit) {
                // the sum after every member of the segment (the whole stayed in the binade, so every part does)
                float fe = before;
                const bool in = lane >= first && lane <= last;
                if (in) spec_apply(fe, sx0, sx1, sm);
                const unsigned long long over = __ballot(in && fe > limit);
                const int j = over ? __ffsll((long long)over) - 1 : last;
                F = j > first ? wide_rl(fe, j - 1) : before;
                for (int jj = j; jj <= last; jj++)
                    if (leaf(jj, F)) return true;
            }
            continue;
        }
        for (int j = first; j <= last; j++) {
            bool t2 = false;
            const float b2 = F;
            if (OWN && sm != 0 && first != last) {
                t2 = spec_apply(F, wide_rl(ox0, j), wide_rl(ox1, j), sm);
                F = spec_uniform(F);
            }
            if (t2) {
                if (bounded && F > limit) {
                    F = b2;
                    if (leaf(j, F)) return true;
                }
            } else if (leaf(j, F)) {
                return true;
            }
        }
    }
    return false;
}

// One wave walks the first nsl slices of terms[0..count) (staged in L from set `set`), from slice s_from (the first of a
// segment) with the sum F before it; with `bounded` until the running sum exceeds `limit`.  Results in L.total, L.hit, L.at.
__device__ __forceinline__ void wide_walk(const WideWs &w, int set, WideWalk &L, int nsl, const float *terms, int count, float limit,
                                          bool bounded, int s_from = 0, float F = 0.0f)
{
    const int lane = threadIdx.x & 63;
    float at = 0.0f;
    int hit = -1;
    bool done = false;
    for (int c = s_from / 64; c * 64 < nsl && !done; c++) {
        const int cn = min(64, nsl - 64 * c);
        int ox0 = 0, ox1 = 0, m = 0;
        if (lane < cn) {
            ox0 = L.t_x0[c * 64 + lane];
            ox1 = L.t_x1[c * 64 + lane];
            m = L.t_m[c * 64 + lane];
        }
        int sx0 = ox0, sx1 = ox1;
        unsigned long long segs = wide_segscan(sx0, sx1, m, cn);
        if (c == s_from / 64) segs &= ~0ull << (s_from & 63);   // (s_from starts a segment)
        auto enter = [&](int j, float &Fs) -> bool {   // slice c * 64 + j, lane segment by lane segment
            const int s = c * 64 + j;
            const int slot = L.slot_of[s];
            int dx0, dx1, dm;
            float4 t;
            unsigned long long sg;
            if (slot != 255) {
                dx0 = L.s_x0[slot][lane];
                dx1 = L.s_x1[slot][lane];
                dm = L.s_m[slot][lane];
                t = L.s_t[slot][lane];
                sg = L.s_seg[slot];
            } else {
                const long a = ((long)set * kWideMaxSlices + s) * 64 + lane;
                dx0 = ld_coh(w.d_x0 + a);
                dx1 = ld_coh(w.d_x1 + a);
                dm = ld_coh(w.d_m + a);
                t = wide_terms(terms, s * kWideSlice + 4 * lane, count);
                sg = ld_coh(w.seg + set * kWideMaxSlices + s);
            }
            auto add4 = [&](int jj, float &Ft) -> bool {   // the four terms of lane jj, one after the other
                const float e[4] = {wide_rl(t.x, jj), wide_rl(t.y, jj), wide_rl(t.z, jj), wide_rl(t.w, jj)};
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    Ft = __fadd_rn(Ft, e[q]);
                    if (bounded && Ft > limit) {
                        hit = s * kWideSlice + 4 * jj + q;
                        at = Ft;
                        return true;
                    }
                }
                return false;
            };
            return wide_level<false>(Fs, 64, 0, 0, dx0, dx1, dm, sg, limit, bounded, add4);
        };
        done = wide_level<true>(F, cn, ox0, ox1, sx0, sx1, m, segs, limit, bounded, enter);
    }
    if (lane == 0) {
        L.total = F;
        L.hit = hit;
        L.at = at;
    }
}

// The walk as a list of steps (one wave, after wide_stage; a workgroup barrier before the list is used: other lanes read it): per segment of uniform slices its pair, per slice that is
// not uniform its lane segments' pairs and the four terms of every lane that has none.  it_m: the binade code (0: four
// terms in it_a .. it_d); it_at: the slice at which a walk that has to look inside the step starts again, and in the
// upper half the step with which that slice begins.
__device__ __forceinline__ void wide_plan(WideWalk &L, int nsl)
{
    const int lane = threadIdx.x & 63;
    int base = 0;
    bool ok = true;
    for (int c = 0; c * 64 < nsl; c++) {
        const int cn = min(64, nsl - 64 * c), s = c * 64 + lane;
        int x0 = 0, x1 = 0, m = 0, slot = 255;
        if (lane < cn) {
            x0 = L.t_x0[s];
            x1 = L.t_x1[s];
            m = L.t_m[s];
            slot = L.slot_of[s];
        }
        const unsigned long long segs = wide_segscan(x0, x1, m, cn);
        const bool in = lane < cn, mixed = in && m == 0;
        if (__ballot(mixed && slot == 255)) ok = false;
        const bool end = in && (lane + 1 == cn || ((segs >> (lane + 1)) & 1ull));
        const unsigned long long sg = (mixed && slot != 255) ? L.s_seg[slot] : 0ull;
        const int cnt = mixed ? __popcll(sg) : (end ? 1 : 0);
        int inc = cnt;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int l = __shfl_up(inc, off);
            if (lane >= off) inc += l;
        }
        const int at = base + inc - cnt;   // this slice's first step
        const int total = wide_rl(inc, 63);
        if (base + total > kWideItems) ok = false;
        if (ok) {
            if (in && !mixed && end) {
                const unsigned long long below = segs & ((2ull << lane) - 1ull);
                const int first = 63 - __clzll((long long)below);
                L.it_m[at] = m;
                L.it_a[at] = x0;
                L.it_b[at] = x1;
                L.it_at[at] = (c * 64 + first) | (at << 16);
            }
            unsigned long long mx = __ballot(mixed);
            while (mx) {   // the lanes of a slice that is not uniform, one slice after the other
                const int j = __ffsll((long long)mx) - 1;
                mx &= mx - 1ull;
                const int k = wide_rl(slot, j), ib = wide_rl(at, j);
                const unsigned long long sj = L.s_seg[k];
                if (lane == 63 || ((sj >> (lane + 1)) & 1ull)) {
                    const int idx = ib + __popcll(sj & ((2ull << lane) - 1ull)) - 1;
                    const int dm = L.s_m[k][lane];
                    L.it_m[idx] = dm;
                    if (dm == 0) {
                        const float4 t = L.s_t[k][lane];
                        L.it_a[idx] = __float_as_int(t.x);
                        L.it_b[idx] = __float_as_int(t.y);
                        L.it_c[idx] = __float_as_int(t.z);
                        L.it_d[idx] = __float_as_int(t.w);
                    } else {
                        L.it_a[idx] = L.s_x0[k][lane];
                        L.it_b[idx] = L.s_x1[k][lane];
                    }
                    L.it_at[idx] = (c * 64 + j) | (ib << 16);
                }
            }
        }
        base += total;
    }
    if (lane == 0) {
        L.nitems = ok ? base : -1;
        L.nrun = 0;
    }
}

// wide_walk from zero along the plan; a step that does not hold, or inside which the sum exceeds the limit, hands over
// to wide_walk at the slice it belongs to.
__device__ __forceinline__ void wide_run(const WideWs &w, int set, WideWalk &L, int nsl, const float *terms, int count, float limit,
                                         bool bounded, bool again = false)
{
    const int lane = threadIdx.x & 63;
    const int ni = L.nitems;
    if (ni < 0) {
        wide_walk(w, set, L, nsl, terms, count, limit, bounded);
        return;
    }
    // `again`: the walk before this one went along the same plan and got at least as far as this one will (its limit
    // was not lower): it starts at the last step before which that walk's sum did not exceed the limit
    int k_start = 0;
    if (again && bounded) {
        int le = 0;
        for (int k = lane; k < L.nrun; k += 64) le += L.it_fb[k] <= limit;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) le += __shfl_xor(le, off);
        k_start = max(le - 1, 0);
    }
    float F = k_start > 0 ? L.it_fb[k_start] : 0.0f;
    const int kb = k_start & ~63;
    for (int k0 = kb; k0 < ni; k0 += 64) {
        int im = 0, ia = 0, ib = 0, ic = 0, id = 0;
        if (k0 + lane < ni) {
            im = L.it_m[k0 + lane];
            ia = L.it_a[k0 + lane];
            ib = L.it_b[k0 + lane];
            ic = L.it_c[k0 + lane];
            id = L.it_d[k0 + lane];
        }
        const int kn = min(64, ni - k0);
        for (int l = k0 == kb ? k_start - kb : 0; l < kn; l++) {
            const int m = wide_rl(im, l), a = wide_rl(ia, l), b = wide_rl(ib, l);
            L.it_fb[k0 + l] = F;   // (every lane: each reads back what it wrote itself)
            bool held = true;
            if (m == 0) {
                F = __fadd_rn(__fadd_rn(__fadd_rn(__fadd_rn(F, __int_as_float(a)), __int_as_float(b)), __int_as_float(wide_rl(ic, l))),
                              __int_as_float(wide_rl(id, l)));
            } else if (m != kSpecIdentity) {
                held = spec_apply(F, a, b, m);
            }
            F = spec_uniform(F);
            if (!held || (bounded && F > limit)) {
                // again from the slice the step belongs to, with the sum before that slice's first step
                const int ref = L.it_at[k0 + l];
                const float f0 = L.it_fb[ref >> 16];
                L.nrun = k0 + l + 1;
                wide_walk(w, set, L, nsl, terms, count, limit, bounded, ref & 0xffff, spec_uniform(f0));
                return;
            }
        }
    }
    L.nrun = ni;
    if (lane == 0) {
        L.total = F;
        L.hit = -1;
        L.at = 0.0f;
    }
}

__device__ __forceinline__ double wide_wave_sum(double v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

// The k-th (from 0) set bit of the 256-bit mask m[0..3] (k below the number of set bits).
__device__ __forceinline__ int wide_kth_bit(const unsigned long long *m, int k)
{
    int word = 0;
#pragma unroll
    for (int q = 0; q < 3; q++) {
        const int c = __popcll(m[q]);
        if (word == q && k >= c) {
            k -= c;
            word = q + 1;
        }
    }
    unsigned long long v = word == 0 ? m[0] : word == 1 ? m[1] : word == 2 ? m[2] : m[3];
    int pos = 0;
#pragma unroll
    for (int width = 32; width > 0; width >>= 1) {
        const int c = __popcll(v & ((1ull << width) - 1ull));
        if (k >= c) {
            k -= c;
            v >>= width;
            pos += width;
        }
    }
    return word * 64 + pos;
}

// keys[0..len) (LDS) = src[0..len), device-coherent, where the position is below `written`; -1 beyond (positions nobody
// stored: they sort behind everything).  len a multiple of 4096, written a multiple of 256; all threads of the workgroup.
// (8-byte relaxed loads: the compiler keeps a batch of them in flight, which it cannot with an asm statement's.)
template <int BATCH>
__device__ __forceinline__ void wide_load_keys(float *keys, const float *src, int len, int written)
{
    constexpr unsigned long long none = 0xBF800000BF800000ull;   // (-1, -1)
    const unsigned long long *s2 = reinterpret_cast<const unsigned long long *>(src);
    unsigned long long *k2 = reinterpret_cast<unsigned long long *>(keys);
    const int len2 = len / 2, w2 = written / 2;
    for (int q0 = 0; q0 < len2; q0 += BATCH * kWideSlice) {   // BATCH loads per thread in flight (past the end: the last pair again)
        unsigned long long v[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; u++) {
            const int q = q0 + u * kWideSlice + threadIdx.x;
            v[u] = ld_coh(s2 + min(q, w2 - 1));
        }
#pragma unroll
        for (int u = 0; u < BATCH; u++) {
            const int q = q0 + u * kWideSlice + threadIdx.x;
            if (q < len2) k2[q] = q < w2 ? v[u] : none;
        }
    }
}

// grid: ceil(n / 256) workgroups of 256 threads, all resident at once (n <= kSampleMaxVocab: at most 144); dynamic LDS:
// max(sizeof(WideWalk), 4 bytes per key of the array padded to whole runs of 4096).
static __global__ void __launch_bounds__(kWideSlice) k_sample_wide(const WideArgs a)
{
    extern __shared__ __align__(16) unsigned char wide_lds[];
    __shared__ __align__(16) float es[kWideSlice];
    __shared__ int cp[kWideMaxSlices + 1];
    __shared__ unsigned long long cmw[4 * kWideMaxSlices];
    __shared__ float red[4];
    __shared__ double dred[4];
    __shared__ int s_cnt[4];
    __shared__ float s_r;
    WideWalk &L = *reinterpret_cast<WideWalk *>(wide_lds);
    float *keys = reinterpret_cast<float *>(wide_lds);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = blockIdx.x, G = gridDim.x, n = a.n;
    const int i = g * kWideSlice + tid;
    unsigned bar = 0;

    // ---- A: x / t, max (FindMax: the rounded quotient of the largest logit is the largest rounded quotient), exp, and B:
    // the slice reduced for the sum of the exponentials.  B's guess, the sum of what stands before the slice, needs no
    // other workgroup: every thread has loaded its share of all logits for the maximum, and the fast exponential will do.
    float mxl = -__builtin_inff();
    const int n4 = n & ~3;
    double before = 0.0;   // (the sum before this slice, approximately)
    {   // (every load in flight at once, past the end the last one again: the loop is bound by their latency)
        constexpr int kMax4 = kSampleMaxVocab / (4 * kWideSlice);
        float4 x[kMax4];
#pragma unroll
        for (int u = 0; u < kMax4; u++) x[u] = *reinterpret_cast<const float4 *>(a.logits + max(min(4 * (tid + u * kWideSlice), n4 - 4), 0));
        if (n4 > 0) {
#pragma unroll
            for (int u = 0; u < kMax4; u++) mxl = fmaxf(fmaxf(fmaxf(mxl, x[u].x), fmaxf(x[u].y, x[u].z)), x[u].w);
        }
        for (int q = n4 + tid; q < n; q += kWideSlice) mxl = fmaxf(mxl, a.logits[q]);
        mxl = block_max(mxl, red);
        const float it = 1.0f / a.temperature;
        float part = 0.0f;
#pragma unroll
        for (int u = 0; u < kMax4; u++)   // (whole float4s: a slice starts at a multiple of 256, below n rounded down to 4)
            if (4 * (tid + u * kWideSlice) < g * kWideSlice)
                part += __expf((x[u].x - mxl) * it) + __expf((x[u].y - mxl) * it) + __expf((x[u].z - mxl) * it) + __expf((x[u].w - mxl) * it);
        const double ds = wide_wave_sum((double)part);
        if (lane == 0) dred[wave] = ds;
    }
    const float mx = __fdiv_rn(mxl, a.temperature);
    int bad = 0;
    float e = 0.0f;
    if (i < n) {
        const float v = __fdiv_rn(a.logits[i], a.temperature);
        bad |= v != v;
        e = (float)exp((double)__fsub_rn(v, mx));
    }
    st_coh(a.expbuf + i, e);
    es[tid] = e;
    __syncthreads();
    before = dred[0] + dred[1] + dred[2] + dred[3];
    if (wave == 0) wide_reduce(a.w, 0, g, *reinterpret_cast<const float4 *>(es + 4 * lane), before);
    wide_barrier(a.w, bar++);

    // ---- C: sum += x in element order (ExpSumNormalize), x /= sum, the probabilities replace the logits
    wide_stage(a.w, 0, L, G, a.expbuf, G * kWideSlice);
    if (wave == 0) wide_walk(a.w, 0, L, G, a.expbuf, G * kWideSlice, 0.0f, false);   // (once: writing the list of steps first does not pay)
    __syncthreads();
    const float sum = L.total;
    float p = e;
    if (sum != 0.0f) p = __fdiv_rn(e, sum);
    if (i < n) {
        bad |= p != p;
        st_coh(a.logits + i, p);
    }
    if (bad) atomicOr(&a.ss->nan, 1);

    if (a.plain) {
        // J/Sampler.java:33-44: the first i with r < cdf(i), else n - 1
        __syncthreads();   // (every wave has read L.total)
        es[tid] = i < n ? p : 0.0f;
        __syncthreads();
        if (wave == 0) wide_reduce(a.w, 1, g, *reinterpret_cast<const float4 *>(es + 4 * lane), sum != 0.0f ? before / (double)sum : before);
        wide_barrier(a.w, bar++);
        if (g == 0) {
            wide_stage(a.w, 1, L, G, a.logits, n);
            if (wave == 0) wide_plan(L, G);
            __syncthreads();
            if (tid == 0) {
                float r = a.coin;
                if (r < 0.0f) r = java_next_float(&a.ss->rng);
                s_r = r;
            }
            __syncthreads();
            if (wave == 0) wide_run(a.w, 1, L, G, a.logits, n, s_r, true);
            __syncthreads();
            if (tid == 0) {
                int pick = L.hit;
                if (pick < 0 || pick >= n) pick = n - 1;
                a.ss->result = pick;
                if (a.st) {
                    a.out_tokens[a.st->pos - 1] = pick;
                    a.st->token = pick;
                }
            }
        }
        wide_leave(a.w, a.ss);
        return;
    }

    // J/Sampler.java:85-96: which terms are candidates
    const float cutoff = __fdiv_rn(__fsub_rn(1.0f, a.topp), (float)(n - 1));
    {
        const unsigned long long cm = __ballot(i < n && p >= cutoff);
        if (lane == 0) st_coh(a.w.cmask + g * 4 + wave, cm);
    }
    wide_barrier(a.w, bar++);

    // ---- D: the ProbIndex array of this call, tile by tile, every tile sorted
    {
        // which terms of every slice are candidates (one round trip), and from that how many stand before a slice
        unsigned long long mw[3];
#pragma unroll
        for (int u = 0; u < 3; u++) mw[u] = ld_coh(a.w.cmask + min(tid + u * kWideSlice, 4 * G - 1));   // (4 G <= 576 < 768)
#pragma unroll
        for (int u = 0; u < 3; u++)
            if (tid + u * kWideSlice < 4 * G) cmw[tid + u * kWideSlice] = mw[u];
        __syncthreads();
        int c = tid < G ? __popcll(cmw[4 * tid]) + __popcll(cmw[4 * tid + 1]) + __popcll(cmw[4 * tid + 2]) + __popcll(cmw[4 * tid + 3]) : 0;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int l = __shfl_up(c, off);
            if (lane >= off) c += l;
        }
        if (lane == 63) s_cnt[wave] = c;
        __syncthreads();
        for (int w2 = 0; w2 < wave; w2++) c += s_cnt[w2];
        if (tid < G) cp[tid + 1] = c;
        if (tid == 0) cp[0] = 0;
        __syncthreads();
    }
    const int n0 = min(cp[G], n);   // (more only after a barrier that gave up: what follows stays inside the arrays)
    if (g == 0 && tid == 0) a.ss->n0 = n0;
    if (n0 <= 0) {   // no probability reaches the cutoff (NaNs, or topp near 0 on a flat distribution): the reference
        if (g == 0 && tid == 0) {   // indexes probIndex[-1] and throws; the host reports the call as failed
            a.ss->result = 0;
            atomicOr(&a.ss->nan, 2);
        }
        wide_leave(a.w, a.ss);
        return;
    }
    {
        float key = -1.0f;
        int val = 0;
        if (i < n0) {
            int h = 0;   // the slice of candidate i: the last h with cp[h] <= i
            for (int st = 128; st > 0; st >>= 1)
                if (h + st < G && cp[h + st] <= i) h += st;
            const unsigned long long cm[4] = {cmw[4 * h], cmw[4 * h + 1], cmw[4 * h + 2], cmw[4 * h + 3]};
            val = min(h * kWideSlice + wide_kth_bit(cm, i - cp[h]), n - 1);
            key = ld_coh(a.logits + val);
        } else if (i < n) {
            key = a.old_prob[i];
            val = a.old_idx[i];
        }
        int rank = tid;   // (what the last call left is sorted)
        if (g * kWideSlice < n0) {
            // a pair stands before another when its probability is greater, or equal and its position lower: one unsigned
            // comparison of (probability bits, 255 - position); the bits of a non-negative float ascend with it, the
            // padding's -1 counts as 0 (it stands behind every position of the array anyway)
            unsigned long long *k64 = reinterpret_cast<unsigned long long *>(wide_lds);
            const unsigned long long mine = ((unsigned long long)(key < 0.0f ? 0u : __float_as_uint(key)) << 32) | (unsigned)(kWideSlice - 1 - tid);
            k64[tid] = mine;
            __syncthreads();
            rank = 0;
#pragma unroll 16
            for (int j2 = 0; j2 < kWideSlice / 2; j2++) {
                const ulonglong2 o = *reinterpret_cast<const ulonglong2 *>(&k64[2 * j2]);
                rank += (o.x > mine) + (o.y > mine);
            }
        }
        st_coh(a.k0 + g * kWideSlice + rank, key);
        st_coh(a.v0 + g * kWideSlice + rank, val);
    }
    wide_barrier(a.w, bar++);

    // ---- E: runs of 16 tiles
    const int written = G * kWideSlice;
    {
        const int base = (g / kSortTilesPerRun) * kSortRun, ti = g % kSortTilesPerRun, ii = ti * kWideSlice + tid;
        int rank = ii;
        float k;
        const int v = ld_coh(a.v0 + base + ii);
        if (base >= n0) {
            k = ld_coh(a.k0 + base + ii);
        } else {
            wide_load_keys<kSortRun / 2 / kWideSlice>(keys, a.k0 + base, kSortRun, written - base);
            __syncthreads();
            k = keys[ii];
            const float kb = sort_below(k);
            int pos[kSortTilesPerRun];
#pragma unroll
            for (int tj = 0; tj < kSortTilesPerRun; tj++) pos[tj] = 0;
#pragma unroll
            for (int st = kSortTile / 2; st > 0; st >>= 1) {
                float o[kSortTilesPerRun];
#pragma unroll
                for (int tj = 0; tj < kSortTilesPerRun; tj++) o[tj] = keys[tj * kSortTile + pos[tj] + st - 1];
                __builtin_amdgcn_sched_barrier(0);   // (all reads of a step in flight before the first is used)
#pragma unroll
                for (int tj = 0; tj < kSortTilesPerRun; tj++) pos[tj] += o[tj] > (tj < ti ? kb : k) ? st : 0;   // tiles that stood earlier win ties
            }
            rank = tid;
#pragma unroll
            for (int tj = 0; tj < kSortTilesPerRun; tj++) {
                const float o = keys[tj * kSortTile + pos[tj]];
                const int cnt = pos[tj] + (o > (tj < ti ? kb : k) ? 1 : 0);
                rank += tj == ti ? 0 : cnt;
            }
        }
        st_coh(a.k1 + base + rank, k);
        st_coh(a.v1 + base + rank, v);
    }
    wide_barrier(a.w, bar++);

    // ---- F: all runs; the sorted array, and the sums of its candidates per 256 for the guess of G
    {
        const int npad = (n + kSortRun - 1) / kSortRun * kSortRun, nruns = npad / kSortRun;
        const int v = ld_coh(a.v1 + i);
        wide_load_keys<kSampleMaxVocab / 2 / kWideSlice>(keys, a.k1, npad, written);
        __syncthreads();
        const float k = keys[i];
        const int ri = i / kSortRun;
        const float kb = sort_below(k);
        int pos[kSortMaxRuns];   // (the searches advance together: their LDS reads are independent)
#pragma unroll
        for (int rj = 0; rj < kSortMaxRuns; rj++) pos[rj] = 0;
#pragma unroll
        for (int st = kSortRun / 2; st > 0; st >>= 1) {
            float o[kSortMaxRuns];
#pragma unroll
            for (int rj = 0; rj < kSortMaxRuns; rj++) o[rj] = keys[min(rj, nruns - 1) * kSortRun + pos[rj] + st - 1];
            __builtin_amdgcn_sched_barrier(0);   // (all reads of a step in flight before the first is used)
#pragma unroll
            for (int rj = 0; rj < kSortMaxRuns; rj++) pos[rj] += o[rj] > (rj < ri ? kb : k) ? st : 0;   // runs that stood earlier win ties
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
            st_coh(a.new_prob + rank, k);
            st_coh(a.new_idx + rank, v);
        }
    }
    wide_barrier(a.w, bar++);

    // ---- G: the sorted candidates reduced
    const int gsl = (n0 + kWideSlice - 1) / kWideSlice;
    if (g < gsl) {   // (the guess: what stands before the slice, added in double precision, any order)
        double b2 = 0.0;
        const unsigned long long *s2 = reinterpret_cast<const unsigned long long *>(a.new_prob);
        for (int q0 = 0; q0 < g * (kWideSlice / 2); q0 += 16 * kWideSlice) {
            unsigned long long v[16];
#pragma unroll
            for (int u = 0; u < 16; u++) v[u] = ld_coh(s2 + min(q0 + u * kWideSlice + tid, g * (kWideSlice / 2) - 1));
#pragma unroll
            for (int u = 0; u < 16; u++)
                if (q0 + u * kWideSlice + tid < g * (kWideSlice / 2))
                    b2 += (double)__uint_as_float((unsigned)v[u]) + (double)__uint_as_float((unsigned)(v[u] >> 32));
        }
        b2 = wide_wave_sum(b2);
        if (lane == 0) dred[wave] = b2;
        __syncthreads();
        if (wave == 0) wide_reduce(a.w, 1, g, wide_terms(a.new_prob, g * kWideSlice + 4 * lane, n0), dred[0] + dred[1] + dred[2] + dred[3], (double)a.topp);
    }
    wide_barrier(a.w, bar++);

    // J/Sampler.java:99-119 on the sorted array: cumulative_prob is the first running sum above topp (else the last),
    // r = coin * cumulative_prob, the pick the first index whose running sum (from zero again: the same sums) exceeds r
    if (g == 0) {
        wide_stage(a.w, 1, L, gsl, a.new_prob, n0);
        if (wave == 0) wide_plan(L, gsl);
        __syncthreads();
        if (wave == 0) wide_run(a.w, 1, L, gsl, a.new_prob, n0, a.topp, true);
        __syncthreads();
        int last = L.hit;
        float cum = L.at;
        if (last < 0) {   // never exceeded: all candidates, cumulative_prob = their sum
            last = n0 - 1;
            cum = L.total;
        }
        if (tid == 0) {
            float coin = a.coin;
            if (coin < 0.0f) coin = java_next_float(&a.ss->rng);
            s_r = __fmul_rn(coin, cum);
        }
        __syncthreads();
        if (wave == 0) wide_run(a.w, 1, L, gsl, a.new_prob, n0, s_r, true, true);   // (r is below cumulative_prob)
        __syncthreads();
        if (tid == 0) {
            int pick = L.hit;
            if (pick < 0 || pick > last) pick = last;
            const int token = ld_coh(a.new_idx + min(pick, n - 1));
            a.ss->result = token;
            if (a.st) {
                a.out_tokens[a.st->pos - 1] = token;
                a.st->token = token;
            }
        }
    }
    wide_leave(a.w, a.ss);
}

// The walk by itself, for tests: terms[0..n) (non-negative; readable up to whole slices, zeros beyond n) summed in
// order; for every limit the first index whose running sum exceeds it (-1: none) and that sum; the sum of all terms.
// grid: ceil(n / 256) workgroups of 256 threads, all resident; dynamic LDS: sizeof(WideWalk).
static __global__ void __launch_bounds__(kWideSlice) k_sum_probe(const float *terms, int n, const float *limits, int nl, int *out_idx,
                                                                 float *out_sum, float *out_total, SamplerState *ss, const WideWs w)
{
    extern __shared__ __align__(16) unsigned char wide_lds[];
    __shared__ double dred[4];
    WideWalk &L = *reinterpret_cast<WideWalk *>(wide_lds);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = blockIdx.x, G = gridDim.x;
    const float4 t = wide_terms(terms, g * kWideSlice + 4 * lane, n);   // (wave 0's are the slice's)
    {
        const int i = g * kWideSlice + tid;
        const double ds = wide_wave_sum(i < n ? (double)terms[i] : 0.0);
        if (lane == 0) dred[wave] = ds;
        __syncthreads();
        if (tid == 0) __hip_atomic_store(w.ssum + g, dred[0] + dred[1] + dred[2] + dred[3], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    wide_barrier(w, 0);
    if (wave == 0) {
        double before = 0.0;
        for (int h = lane; h < g; h += 64) before += __hip_atomic_load(w.ssum + h, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        wide_reduce(w, 0, g, t, wide_wave_sum(before));
    }
    wide_barrier(w, 1);
    if (g == 0) {
        wide_stage(w, 0, L, G, terms, n);
        if (wave == 0) wide_plan(L, G);
        __syncthreads();
        for (int q = 0; q <= nl; q++) {
            if (wave == 0) wide_run(w, 0, L, G, terms, n, q < nl ? limits[q] : 0.0f, q < nl);
            __syncthreads();
            if (tid == 0) {
                if (q < nl) {
                    out_idx[q] = L.hit;
                    out_sum[q] = L.at;
                } else {
                    *out_total = L.total;
                }
            }
            __syncthreads();
        }
    }
    wide_leave(w, ss);
}

}  // namespace l2j
