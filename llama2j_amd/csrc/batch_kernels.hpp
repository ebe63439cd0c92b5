// Several sequences per pass over the weights ("parallel processing of multiple queries", the reference's README
// wish-list): with sixteen activation vectors per weight matrix the multiply-adds are a 16-wide GEMM and run on the
// matrix cores.  The arithmetic of the single-sequence path is kept (byte code -> float, fp32 activations, fp32 sums,
// rm * sum(code * x) + min * sum(x) per group of 256; K/MatMul.java:117-151 is the loop it restates) although the
// products run on the bf16 cores, sixteen times as fast as the fp32 ones: a code (0..255) is a bf16 exactly, and an
// fp32 activation is the sum of three bf16 (its 24 significant bits cut into 8 + 8 + 8), so code * x is the sum of
// three products that v_mfma_f32_16x16x32_bf16 forms exactly and accumulates in fp32.  The vector units only convert
// the codes.  The fp32 classifier keeps the fp32 cores (v_mfma_f32_16x16x4_f32).
#pragma once

#include "kernels.hpp"
#include "phase_kernels.hpp"   // grid barrier, device-coherent loads and stores

namespace l2j {

constexpr int kBatch = 16;          // sequences per column block: the 16 columns of one MFMA
constexpr int kMaxBatch = 32;       // sequences per step: one or two column blocks
constexpr int kBgThreads = 256;     // threads per column block: four waves per 16 sequences share the staged activations
constexpr int kBgRowsPerWave = 32;  // k_bgemm_f32: two 16-row tiles share the activations fetched from LDS
constexpr int kBgRowsPerWG = kBgRowsPerWave * (kBgThreads / 64);
constexpr int kXPad = 4;            // floats between the slices of two sequences in LDS: a quarter wave's 16-byte reads then cover every bank once

typedef float v4f32 __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf16 __attribute__((ext_vector_type(8)));

// Device-coherent 16-byte accesses for what the workgroups of one launch hand to each other (a load per float would
// fetch the same lines once per float: such loads do not stay in the L2).  Loads and their wait are one statement: the
// compiler must not touch the destination registers in between.
__device__ __forceinline__ void ld_coh64x2(const float *p0, const float *p1, float (&v0)[16], float (&v1)[16])   // 64 bytes at p0, 64 bytes at p1
{
    float4 v[8];
    asm volatile("global_load_dwordx4 %0, %8, off sc1\n\tglobal_load_dwordx4 %1, %8, off offset:16 sc1\n\t"
                 "global_load_dwordx4 %2, %8, off offset:32 sc1\n\tglobal_load_dwordx4 %3, %8, off offset:48 sc1\n\t"
                 "global_load_dwordx4 %4, %9, off sc1\n\tglobal_load_dwordx4 %5, %9, off offset:16 sc1\n\t"
                 "global_load_dwordx4 %6, %9, off offset:32 sc1\n\tglobal_load_dwordx4 %7, %9, off offset:48 sc1\n\t"
                 "s_waitcnt vmcnt(0)"
                 : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]), "=&v"(v[7])
                 : "v"(p0), "v"(p1)
                 : "memory");
#pragma unroll
    for (int q = 0; q < 4; q++) {
        v0[4 * q] = v[q].x; v0[4 * q + 1] = v[q].y; v0[4 * q + 2] = v[q].z; v0[4 * q + 3] = v[q].w;
        v1[4 * q] = v[4 + q].x; v1[4 * q + 1] = v[4 + q].y; v1[4 * q + 2] = v[4 + q].z; v1[4 * q + 3] = v[4 + q].w;
    }
}

// write-through; acknowledged by the next s_waitcnt vmcnt(0).  (The wait states are part of the statement: a store of more
// than 8 bytes reads its data registers after it has issued, and the compiler, which does not look inside the statement,
// would let the next instruction overwrite them.)
__device__ __forceinline__ void st_coh16(float *p, v4f32 v)
{
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 2" : : "v"(p), "v"(v) : "memory");
}

// y[b][r] = sum_k dequant(W[r][k]) * x[b][k], split over slices of K: part[slice][b][r].  Up to three matrices that
// share the input (Wq, Wk, Wv; W1, W3) go into one launch: their row blocks follow each other in grid.x.
constexpr int kBgMaxMat = 3;
constexpr int kBgGroups = 4;        // groups of 256 codes per slice of K: one per wave (16 sequences) or per pair of waves (32)
constexpr int kBgDepth = 2;         // tiles whose codes a wave has in flight (divides the number of waves: a tile's register set is known at
                                    // compile time).  Measured, 32 / 16 sequences: 1: 3.95 / 3.05 ms per step, 2: 3.84 / 2.97, 4: 3.85 / 3.07
struct BGemm {
    QMat m[kBgMaxMat];        // the tensor's copy in tile order (k_btile), m.off: the layer's matrix (a multiple of 4096)
    int rows[kBgMaxMat];      // rows % 16 == 0
    float *part[kBgMaxMat];   // (slices, nseq, rows)
    int nmat;
    int K;                    // K % 256 == 0
    const float *x;           // (nseq, K)
};

__host__ __device__ inline int bg_slices(int K) { return ((K >> 8) + kBgGroups - 1) / kBgGroups; }

// The batched path keeps its own copy of the quantized matrices, in the order its waves read them: the 16 rows x 256
// codes of a (tile of 16 rows, group) block are 4 KB in a row, [T][lane][16 codes] with lane = r + 16 s holding row r of
// the tile at k = 64 T + 16 s + j, so that each of a wave's four load instructions per block reads 1 KB in one piece
// (row by row a wave's instruction touches 16 rows, 64 bytes each: a third slower, measured); the blocks of a tile
// follow each other group by group, then come those of the next tile.  The scales likewise: 16 (rm, min) per block.
// One thread per 16 codes of the whole tensor (layers x rows x K); rows % 16 == 0, K % 256 == 0.
static __global__ void __launch_bounds__(256) k_btile(const uint8_t *__restrict__ codes, const float2 *__restrict__ gs, long n16, int rows, int K,
                                               uint8_t *__restrict__ tcodes, float2 *__restrict__ tgs)
{
    const long o = (long)blockIdx.x * 256 + threadIdx.x;   // index of the 16 codes in the tiled copy
    if (o >= n16) return;
    const int ngroups = K >> 8;
    const long per = (long)rows * K >> 4, layer = o / per;
    const long w = o - layer * per;                         // within the layer's matrix
    const int block = (int)(w >> 8), in = (int)(w & 255), T = in >> 6, lane = in & 63, r = lane & 15, sq = lane >> 4;
    const int tile = block / ngroups, g = block - tile * ngroups;
    const long src = layer * (long)rows * K + (long)(16 * tile + r) * K + (g << 8) + 64 * T + 16 * sq;
    reinterpret_cast<uint4 *>(tcodes)[o] = *reinterpret_cast<const uint4 *>(codes + src);
    if (in < 16)   // the block's 16 scales: rows 16 tile + in
        tgs[(layer * (long)rows * K >> 8) + (long)block * 16 + in] = gs[((layer * (long)rows * K + (long)(16 * tile + in) * K) >> 8) + g];
}

// LDS of k_bgemm: the sums of a batch of tiles (as many tiles as the workgroup has waves; per tile, wave and column block
// 64 lanes x 16 bytes), then every wave's sums of its activations per sequence
__host__ __device__ inline size_t bg_lds_bytes(int nseq, int hv)
{
    const size_t nb = nseq / kBatch, waves = 4 * hv;
    return waves * waves * nb * 1024 + waves * nseq * sizeof(float);
}

// eight codes (two words of a row) as eight bf16: the upper halves of the codes' floats, two to a register
__device__ __forceinline__ v8bf16 codes_bf16(uint32_t d0, uint32_t d1)
{
    uint4 o;
    o.x = __builtin_amdgcn_perm(__float_as_uint(ubyte_f(d0, 1)), __float_as_uint(ubyte_f(d0, 0)), 0x07060302u);
    o.y = __builtin_amdgcn_perm(__float_as_uint(ubyte_f(d0, 3)), __float_as_uint(ubyte_f(d0, 2)), 0x07060302u);
    o.z = __builtin_amdgcn_perm(__float_as_uint(ubyte_f(d1, 1)), __float_as_uint(ubyte_f(d1, 0)), 0x07060302u);
    o.w = __builtin_amdgcn_perm(__float_as_uint(ubyte_f(d1, 3)), __float_as_uint(ubyte_f(d1, 2)), 0x07060302u);
    return __builtin_bit_cast(v8bf16, o);
}

// x = h[0] + h[1] + h[2] exactly, each the upper half of a float (a bf16): 8 of x's 24 significant bits at a time
__device__ __forceinline__ void split_bf16(float x, uint32_t h[3])
{
    const uint32_t b0 = __float_as_uint(x) & 0xffff0000u;
    const float r1 = x - __uint_as_float(b0);
    const uint32_t b1 = __float_as_uint(r1) & 0xffff0000u;
    const float r2 = r1 - __uint_as_float(b1);
    h[0] = b0 >> 16; h[1] = b1 >> 16; h[2] = __float_as_uint(r2) >> 16;
}

// Workgroup (by: one slice of K, four groups of 256; bx of gx: a share of the 16-row tiles of the launch's matrices, in
// order: tile bx, then every gx-th).  The ACTIVATIONS stay in registers and the codes stream past them: a wave owns one
// group of the slice (with 32 sequences, NB = 2: half a group; two waves per group) and holds, for every one of its 64-k
// blocks, the three bf16 planes of its 16 NB sequences as MFMA operands (96 registers); all waves of the workgroup take
// the same tiles, each the part of the tile's codes that belongs to its k (4 KB, or 2 KB: [T][lane][16 codes] in tile
// order, lane (r = lane % 16, s = lane / 16) holding row r at k = 64 T + 16 s + j; one MFMA multiplies the 16 rows by 16
// sequences over the eight k (j < 8, or j >= 8) of each of the four s, once per plane and column block), kBgDepth
// tiles' codes in flight.  The waves' 16 x 16 sums of a tile meet in LDS: after every batch of as many tiles as the
// workgroup has waves, wave w adds up tile w of the batch: per group the halves, times the group's scale, plus its
// offset times the sum of the activations, group after group (K/MatMul.java:137-147), and writes the slice's partial
// sums.  (A first version staged the activations in LDS as bf16 planes and every wave fetched them from there for every
// tile: 12 bytes of LDS reads per byte of codes, two thirds of the time of a group, measured with time stamps in the
// kernel; here LDS carries 2 bytes per byte of codes.)
// The work of one wave, in two steps so that a kernel with several phases can request the first codes of a product
// before the phase (and the grid barrier) that produces its activations: begin(), then run().
template <int NB, int HV>   // HV: waves per group (1: a wave takes the group's 256 k, 2: 128 k)
struct BgWave {
    static constexpr int NSEQ = kBatch * NB, WAVES = 4 * HV, TB = 4 / HV;   // TB: blocks of 64 k per wave
    struct Mat {
        const uint8_t *codes;
        const float2 *gs;
        float *part;
        int rows, tiles;
    };
    struct Tile {   // a 16-row tile of one of the matrices
        const uint8_t *codes;   // its first block (group 0)
        const float2 *gs;
        float *out;             // row0 of sequence 0 of this slice
        int rows;
    };
    const BGemm *ap;   // (a pointer, so that a kernel with several products can aim one BgWave at each in turn)
    long layer;        // the matrices of this layer: layer * rows * K codes behind m.off
    Mat m0, m1, m2;    // (named, not an array: indexed by a variable the wave's whole state would move to scratch memory)
    int nmat, ntiles, by, lane, c, s, wave, gq, h, ngroups, g0, ng, first, gx, cnt;
    bool active;       // this wave's group exists (the last slice of K may have fewer than four)
    uint4 cw[kBgDepth][TB];

    __device__ __forceinline__ BgWave(const BGemm &a_) : ap(&a_), layer(0) {}

    __device__ __forceinline__ Tile locate(int tile) const
    {
        Mat m = m0;
        if (nmat > 1 && tile >= m0.tiles) {
            tile -= m0.tiles;
            m = m1;
            if (nmat > 2 && tile >= m1.tiles) { tile -= m1.tiles; m = m2; }
        }
        Tile t;
        t.rows = m.rows;
        const long block = (long)tile * ngroups;
        t.codes = m.codes + (block << 12);
        t.gs = m.gs + (block << 4);
        t.out = m.part + (long)by * NSEQ * m.rows + 16 * tile;
        return t;
    }

    // The codes of this wave's k of the i-th tile of the workgroup into register set `slot`.  Unconditionally (past the
    // workgroup's last tile: that tile again; a wave without a group: the slice's last group): after a load that may or
    // may not have been issued the compiler can only wait for all loads, and the sets in flight would be waited for too.
    __device__ __forceinline__ void request(int slot, int i)
    {
        const Tile t = locate(max(min(first + min(i, cnt - 1) * gx, ntiles - 1), 0));
        const uint4 *p = reinterpret_cast<const uint4 *>(t.codes + ((long)(g0 + min(gq, ng - 1)) << 12)) + (h * TB) * 64 + lane;
#pragma unroll
        for (int T = 0; T < TB; T++) cw[slot][T] = load_stream(p + 64 * T);
    }

    // This wave's share of workgroup (bx, by) of a gx-wide grid; first = false: the first codes are not requested yet
    // (run() does it once the activations are requested: a wave's loads return in order, and behind the codes the
    // activations would arrive with them).
    __device__ __forceinline__ void begin(int bx, int by_, int gx_, bool first_codes)
    {
        const BGemm &a = *ap;
        const int tid = threadIdx.x;
        by = by_;
        lane = tid & 63; wave = tid >> 6;
        c = lane & 15; s = lane >> 4;
        gq = wave / HV; h = wave % HV;
        ngroups = a.K >> 8;
        g0 = by * kBgGroups; ng = min(kBgGroups, ngroups - g0);
        active = gq < ng;
        nmat = a.nmat;
        auto matrix = [&](int i) {
            Mat m{};
            if (i < a.nmat) {
                const long off = a.m[i].off + layer * a.rows[i] * a.K;
                m.codes = a.m[i].codes + off;
                m.gs = a.m[i].gs + (off >> 8);
                m.part = a.part[i];
                m.rows = a.rows[i];
                m.tiles = a.rows[i] >> 4;
            }
            return m;
        };
        m0 = matrix(0); m1 = matrix(1); m2 = matrix(2);
        ntiles = m0.tiles + m1.tiles + m2.tiles;
        first = bx; gx = gx_;
        cnt = bx < ntiles ? (ntiles - bx + gx - 1) / gx : 0;
        if (first_codes) {
#pragma unroll
            for (int d = 0; d < kBgDepth; d++) request(d, d);
        }
    }

    // requested = begin(.., true) was called.  COH: the activations were written by other workgroups of this launch and
    // the partial sums are read by other workgroups of it (device-coherent loads, write-through stores).
    // lds: bg_lds_bytes(NSEQ, HV) bytes, free when the workgroup's waves get here.
    template <bool COH>
    __device__ __forceinline__ void run(float *lds, bool requested)
    {
        const BGemm &a = *ap;
        v4f32 *raw = reinterpret_cast<v4f32 *>(lds);                      // [tile of the batch][wave][column block][lane]
        float *sxw = lds + (size_t)WAVES * WAVES * NB * 256;              // [wave][sequence]
        // This wave's activations: sequence c (+ 16 per column block) at k = 64 T + 16 s + j of its blocks T, as the
        // three bf16 planes, eight k (j < 8, j >= 8) to an MFMA operand; and their sum per sequence.
        v8bf16 bx[NB][TB][2][3];
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            const float *xsrc = a.x + (long)(16 * nb + c) * a.K + ((long)(g0 + (active ? gq : 0)) << 8) + h * (64 * TB) + 16 * s;
            float t = 0.0f;
#pragma unroll
            for (int T2 = 0; T2 < TB; T2 += 2) {
                float v[2][16];
                if (COH) {
                    ld_coh64x2(xsrc + 64 * T2, xsrc + 64 * (T2 + 1), v[0], v[1]);
                } else {
#pragma unroll
                    for (int e = 0; e < 2; e++)
#pragma unroll
                        for (int q = 0; q < 4; q++) {
                            const float4 f = reinterpret_cast<const float4 *>(xsrc + 64 * (T2 + e))[q];
                            v[e][4 * q] = f.x; v[e][4 * q + 1] = f.y; v[e][4 * q + 2] = f.z; v[e][4 * q + 3] = f.w;
                        }
                }
#pragma unroll
                for (int e = 0; e < 2; e++) {
                    const float (&w)[16] = v[e];
                    t += ((w[0] + w[1]) + (w[2] + w[3])) + ((w[4] + w[5]) + (w[6] + w[7])) + ((w[8] + w[9]) + (w[10] + w[11])) +
                         ((w[12] + w[13]) + (w[14] + w[15]));
#pragma unroll
                    for (int hf = 0; hf < 2; hf++) {
                        uint32_t pk[3][4];
#pragma unroll
                        for (int q = 0; q < 4; q++) {
                            uint32_t lo[3], hi[3];
                            split_bf16(w[8 * hf + 2 * q], lo);
                            split_bf16(w[8 * hf + 2 * q + 1], hi);
#pragma unroll
                            for (int pl = 0; pl < 3; pl++) pk[pl][q] = lo[pl] | (hi[pl] << 16);
                        }
#pragma unroll
                        for (int pl = 0; pl < 3; pl++)
                            bx[nb][T2 + e][hf][pl] = __builtin_bit_cast(v8bf16, make_uint4(pk[pl][0], pk[pl][1], pk[pl][2], pk[pl][3]));
                    }
                }
            }
            t += __shfl_xor(t, 16);
            t += __shfl_xor(t, 32);
            if (s == 0) sxw[wave * NSEQ + 16 * nb + c] = active ? t : 0.0f;
        }
        if (!requested) {
#pragma unroll
            for (int d = 0; d < kBgDepth; d++) request(d, d);
        }
        __syncthreads();
        for (int i0 = 0; i0 < cnt; i0 += WAVES) {
            const int nbatch = min(WAVES, cnt - i0);
            // the scales of the tile this wave will add up, requested ahead of the batch's codes
            float4 sc[kBgGroups][2];
            const Tile mine = locate(max(min(first + min(i0 + wave, cnt - 1) * gx, ntiles - 1), 0));   // (unconditionally, as the codes)
#pragma unroll
            for (int q = 0; q < kBgGroups; q++) {
                const float4 *gp = reinterpret_cast<const float4 *>(mine.gs + ((g0 + min(q, ng - 1)) << 4) + 4 * s);   // (rm, min) of rows 4 s + (0..3)
                sc[q][0] = gp[0]; sc[q][1] = gp[1];
            }
#pragma unroll
            for (int ii = 0; ii < WAVES; ii++) {
                // (the register set of a tile is fixed: moving sets along as in a queue would wait for the loads in flight)
                uint4 (&cu)[TB] = cw[ii % kBgDepth];
                v8bf16 a0[TB], a1[TB];
#pragma unroll
                for (int T = 0; T < TB; T++) { a0[T] = codes_bf16(cu[T].x, cu[T].y); a1[T] = codes_bf16(cu[T].z, cu[T].w); }
                request(ii % kBgDepth, i0 + ii + kBgDepth);   // the set is free: the tile kBgDepth further on
                if (active && ii < nbatch) {
                    // two sums per column block: independent chains of MFMAs (one chain: 9 % slower, measured); each chain's
                    // first MFMA takes a zero as the sum it adds to
                    v4f32 acc0[NB], acc1[NB];
#pragma unroll
                    for (int T = 0; T < TB; T++) {
#pragma unroll
                        for (int nb = 0; nb < NB; nb++) {
                            const v4f32 zero = {0.f, 0.f, 0.f, 0.f};
                            acc0[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0[T], bx[nb][T][0][2], T == 0 ? zero : acc0[nb], 0, 0, 0);   // the small parts first
                            acc1[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1[T], bx[nb][T][1][2], T == 0 ? zero : acc1[nb], 0, 0, 0);
#pragma unroll
                            for (int pl = 1; pl >= 0; pl--) {
                                acc0[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0[T], bx[nb][T][0][pl], acc0[nb], 0, 0, 0);
                                acc1[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1[T], bx[nb][T][1][pl], acc1[nb], 0, 0, 0);
                            }
                        }
                    }
#pragma unroll
                    for (int nb = 0; nb < NB; nb++) raw[((ii * WAVES + wave) * NB + nb) * 64 + lane] = acc0[nb] + acc1[nb];
                }
            }
            __syncthreads();
            if (wave < nbatch) {   // this lane: rows 4 s + (0..3) of sequence c (+ 16 per column block) of tile `wave` of the batch
#pragma unroll
                for (int nb = 0; nb < NB; nb++) {
                    v4f32 y = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int q = 0; q < kBgGroups; q++) {
                        if (q < ng) {
                            v4f32 t = raw[((wave * WAVES + q * HV) * NB + nb) * 64 + lane];
                            float sx = sxw[(q * HV) * NSEQ + 16 * nb + c];
                            if (HV == 2) {
                                t += raw[((wave * WAVES + q * HV + 1) * NB + nb) * 64 + lane];
                                sx += sxw[(q * HV + 1) * NSEQ + 16 * nb + c];
                            }
                            y[0] += fmaf(sc[q][0].x, t[0], sc[q][0].y * sx);
                            y[1] += fmaf(sc[q][0].z, t[1], sc[q][0].w * sx);
                            y[2] += fmaf(sc[q][1].x, t[2], sc[q][1].y * sx);
                            y[3] += fmaf(sc[q][1].z, t[3], sc[q][1].w * sx);
                        }
                    }
                    float *o = mine.out + (long)(16 * nb + c) * mine.rows + 4 * s;
                    if (COH) st_coh16(o, y);
                    else *reinterpret_cast<v4f32 *>(o) = y;
                }
            }
            __syncthreads();   // (the next batch writes the same LDS)
        }
    }
};

// grid (workgroups per slice, slices of K), 256 HV threads; dynamic LDS: bg_lds_bytes(16 NB, HV)
template <int NB, int HV>
__global__ void __launch_bounds__(kBgThreads * HV) k_bgemm(const BGemm a)
{
    extern __shared__ __align__(16) float bg_lds[];
    BgWave<NB, HV> w(a);
    w.begin(blockIdx.x, blockIdx.y, gridDim.x, false);
    w.template run<false>(bg_lds, false);
}

// ---- the classifier: fp32 weights (K/MatMul.java:37-60), the same tiling -------------------------------------------

struct BGemmF32 {
    const float *w;    // (rows, K) fp32
    int rows, K;       // rows % 16 == 0, K % 256 == 0
    const float *x;    // (nseq, K)
    float *part;       // (slices, nseq, rows)
    int gps;
};

// As k_bgemm with float weights on the fp32 matrix cores (v_mfma_f32_16x16x4_f32), rows as they lie in memory: a lane
// (r, s) holds row r at k = 64 T + 16 q + 4 s + e as four 16-byte loads (q) per block of 64 k, so that the four lanes of a
// row read 64 bytes in one piece per load; step (q, e) multiplies the 16 rows by 16 sequences over the four k of the four s.
// NB = 2: two column blocks of 16 sequences share the weights.  256 threads, 32 rows per wave.
template <int NB>
__global__ void __launch_bounds__(kBgThreads) k_bgemm_f32(const BGemmF32 a)
{
    constexpr int NSEQ = kBatch * NB;
    extern __shared__ float xs[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ngroups = a.K >> 8;
    const int g0 = blockIdx.y * a.gps, g1 = min(ngroups, g0 + a.gps), nk = (g1 - g0) << 8;
    const int row0 = min(blockIdx.x * kBgRowsPerWG + wave * kBgRowsPerWave, a.rows - 16);
    const bool live = blockIdx.x * kBgRowsPerWG + wave * kBgRowsPerWave < a.rows;
    const int r = lane & 15, s = lane >> 4;
    const bool two = row0 + 16 < a.rows;
    const float4 *c0 = reinterpret_cast<const float4 *>(a.w + (long)(row0 + r) * a.K + (g0 << 8) + 4 * s);
    const float4 *c1 = c0 + (two ? 4L * a.K : 0L);   // 16 rows on, in 16-byte words
    float4 w0[4], w1[4];
#pragma unroll
    for (int q = 0; q < 4; q++) { w0[q] = load_stream(c0 + 4 * q); w1[q] = load_stream(c1 + 4 * q); }
    const int pitch = nk + kXPad;
    {
        const int nk4 = nk >> 2;
#pragma unroll 8
        for (int f = tid; f < NSEQ * nk4; f += kBgThreads) {
            const int b = f / nk4, k4 = f - b * nk4;
            *reinterpret_cast<float4 *>(xs + b * pitch + 4 * k4) = *reinterpret_cast<const float4 *>(a.x + (long)b * a.K + (g0 << 8) + 4 * k4);
        }
    }
    __syncthreads();
    if (!live) return;
    v4f32 acc0[NB], acc1[NB], acc2[NB], acc3[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) acc0[nb] = acc1[nb] = acc2[nb] = acc3[nb] = v4f32{0.f, 0.f, 0.f, 0.f};
    const float4 *xk = reinterpret_cast<const float4 *>(xs + r * pitch + 4 * s);
    const int nblocks = nk >> 6;   // blocks of 64 k
    for (int T = 0; T < nblocks; T++) {
        float4 u0[4], u1[4];
#pragma unroll
        for (int q = 0; q < 4; q++) { u0[q] = w0[q]; u1[q] = w1[q]; }
        if (T + 1 < nblocks) {
            c0 += 16; c1 += 16;   // 64 floats on
#pragma unroll
            for (int q = 0; q < 4; q++) { w0[q] = load_stream(c0 + 4 * q); w1[q] = load_stream(c1 + 4 * q); }
        }
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            float4 xc[4];
#pragma unroll
            for (int q = 0; q < 4; q++) xc[q] = xk[nb * 4 * pitch + 16 * T + 4 * q];   // (16 sequences on: 16 pitch floats)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float bx[4] = {xc[q].x, xc[q].y, xc[q].z, xc[q].w};
                const float a0[4] = {u0[q].x, u0[q].y, u0[q].z, u0[q].w}, a1[4] = {u1[q].x, u1[q].y, u1[q].z, u1[q].w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    if (e & 1) {
                        acc2[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0[e], bx[e], acc2[nb], 0, 0, 0);
                        acc3[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1[e], bx[e], acc3[nb], 0, 0, 0);
                    } else {
                        acc0[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0[e], bx[e], acc0[nb], 0, 0, 0);
                        acc1[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1[e], bx[e], acc1[nb], 0, 0, 0);
                    }
                }
            }
        }
    }
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        float *p = a.part + ((long)blockIdx.y * NSEQ + 16 * nb + r) * a.rows + row0 + 4 * s;
        *reinterpret_cast<v4f32 *>(p) = acc0[nb] + acc2[nb];
        if (two) *reinterpret_cast<v4f32 *>(p + 16) = acc1[nb] + acc3[nb];
    }
}

// ---- the element-wise kernels between the products --------------------------------------------------------------

// Loop state of a batched decode, on the device.
struct BatchState {
    int pos;              // position of the step being computed
    int token[kMaxBatch];    // input token of every sequence at this position
    int n_prompt[kMaxBatch];
};

// x[b] = row token[b] of the embedding table (J/Run.java:72).  As the first kernel of a step it also clears the
// counters of the grid barrier of k_bstep (bar_ctr: null without that kernel).
static __global__ void __launch_bounds__(256) k_bembed(const float *__restrict__ emb, const BatchState *st, float *__restrict__ x, int dim,
                                                unsigned *bar_ctr)
{
    const int b = blockIdx.x;
    if (bar_ctr && b == 0 && threadIdx.x < 1 + kBarGroups) bar_ctr[64 * threadIdx.x] = 0u;
    const float4 *src = reinterpret_cast<const float4 *>(emb + (long)st->token[b] * dim);
    float4 *dst = reinterpret_cast<float4 *>(x + (long)b * dim);
    for (int i = threadIdx.x; i < (dim >> 2); i += blockDim.x) dst[i] = src[i];
}

// xn[b] = w * (ss * x[b]), ss = 1 / sqrt(sum(x^2) / n + 1e-5) (K/RootMeanSquare.java:25-35, K/WeightNormalizeAndScale.java:73).
// One workgroup of 1024 threads per sequence.
static __global__ void __launch_bounds__(1024) k_brms(const float *__restrict__ x, const float *__restrict__ w, float *__restrict__ xn, int n)
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
static __global__ void __launch_bounds__(1024) k_bres_rms(const float *__restrict__ part, int slices, float *__restrict__ x, const float *__restrict__ w,
                                                   float *__restrict__ xn, int n)
{
    __shared__ float red[16];
    const int b = blockIdx.x, tid = threadIdx.x, n4 = n >> 2;
    const long stride4 = (long)gridDim.x * n4;   // 16-byte words between two slices (one workgroup per sequence)
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
// grid (hidden / 256, sequences), 256 threads.
static __global__ void __launch_bounds__(256) k_bepi_swiglu(const float *__restrict__ p1, const float *__restrict__ p3, int slices, int hidden,
                                                     const float *__restrict__ silu, int exact, float *__restrict__ hb)
{
    const int b = blockIdx.y, rix = blockIdx.x * 256 + threadIdx.x;
    const long n = (long)gridDim.y * hidden, i = (long)b * hidden + rix;
    float h1 = 0.0f, h3 = 0.0f;
#pragma unroll 8
    for (int s = 0; s < slices; s++) { h1 += p1[(long)s * n + i]; h3 += p3[(long)s * n + i]; }
    const float sg = silu_sigma(silu, h1, exact);
    hb[i] = __fmul_rn(h1, __fmul_rn(sg, h3));
}

struct BAttn {
    const float *pq, *pk, *pv;   // partial products of Wq, Wk, Wv: (slices, sequences, dim | kv_dim)
    int slices;
    const float2 *rope;          // (seq_len, head_size / 2) cos, sin
    float *kc, *vc;              // this layer's part of the batch cache, head-major: + b * seq_stride + (kv head * cap + pos) * head_size
    long seq_stride;             // floats between two sequences
    int cap;                     // positions the cache holds
    float *out;                  // (sequences, dim)
    const BatchState *st;
    int n_heads, kv_mul, head_size, kv_dim, dim;
    float sqrt_hs;
    // MODE 1, 2 (the rows are consecutive positions of ONE sequence, st->pos + b, in one cache):
    long head_stride;            // floats between two kv heads of a position's row
    int row_stride;              // and between two positions
    int nrows;                   // rows in use: the others neither store nor attend
    int nseq;                    // rows of the products' partial sums (k_pflash; k_battn has them as its grid)
    // k_pflash with the keys of a (head, 16 queries) pair split over gridDim.z workgroups:
    float *pf_part;              // (head, half, z) x (16 maxima, 16 sums, 16 x head_size values): what each leaves for the last one
    unsigned *pf_cnt;            // (head, half): how many have; zero between launches
};

// Attention of one head of one sequence over positions 0..pos (K/AttentionLoop.java:29-54, K/ExpSumNormalize.java:25-38,
// K/AccumWeightedValue.java).  First q of the head and k, v of its kv head at this position: the slices of the products
// summed in order, RoPE on the pairs of q and k (K/ApplyRope.java:74-90), k and v into the cache row (J/Run.java:95-99; by
// the first head of the kv group).  Then LPR lanes per cache row (four floats of the head each): the row slots of the
// workgroup take the positions in turn with an online softmax, and the slots are folded at the end.  grid (n_heads, sequences).
constexpr int kBattnRows = 4;

// MODE 0: the sequences of a batch, all at position st->pos, each with a cache of its own (head-major).  MODE 1 and 2: the
// rows are the positions st->pos + b of one sequence sharing one cache (any layout: head_stride, row_stride): 1 only stores
// k and v of its position, 2 only attends (over the rows below its own position, which a launch in MODE 1 has stored,
// and its own).
template <int LPR, int MODE = 0>
__global__ void __launch_bounds__(256) k_battn(const BAttn a)
{
    constexpr int RPW = 64 / LPR, NSLOT = 4 * RPW;
    __shared__ float sm_m[NSLOT], sm_l[NSLOT];
    __shared__ float4 sm_acc[NSLOT * LPR];
    __shared__ __align__(16) float sm_qkv[3][4 * LPR];
    const int h = blockIdx.x, b = blockIdx.y, tid = threadIdx.x, lane = tid & 63;
    const int j = lane % LPR, slot = (tid >> 6) * RPW + lane / LPR;
    if (MODE != 0 && b >= a.nrows) return;
    if (MODE == 1 && h % a.kv_mul != 0) return;   // (one head of a group stores its kv head)
    const int pos = a.st->pos + (MODE != 0 ? b : 0), len = pos + 1, hs = a.head_size, kvh = h / a.kv_mul;
    const long hstride = MODE != 0 ? a.head_stride : (long)a.cap * hs;
    const int rs = MODE != 0 ? a.row_stride : hs;
    const int half = hs >> 1;
    for (int p = tid; p < 3 * half; p += 256) {   // one thread per pair of q, k, v
        const int which = p / half, idx = p - which * half;
        {
            const int rows = which == 0 ? a.dim : a.kv_dim, row = (which == 0 ? h : kvh) * hs + 2 * idx;
            const float *part = which == 0 ? a.pq : which == 1 ? a.pk : a.pv;
            float v0 = 0.0f, v1 = 0.0f;
#pragma unroll 8
            for (int s = 0; s < a.slices; s++) {   // (independent loads, added in slice order)
                const float2 t = *reinterpret_cast<const float2 *>(part + ((long)s * gridDim.y + b) * rows + row);
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
            if (MODE != 2 && which > 0 && h % a.kv_mul == 0)
                *reinterpret_cast<float2 *>((which == 1 ? a.kc : a.vc) + (long)b * a.seq_stride + kvh * hstride + (long)pos * rs + 2 * idx) =
                    make_float2(v0, v1);
        }
    }
    if (MODE == 1) return;
    __syncthreads();
    const bool on = 4 * j < hs;
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    const float4 q4 = on ? *reinterpret_cast<const float4 *>(&sm_qkv[0][4 * j]) : zero;
    const float4 kp = on ? *reinterpret_cast<const float4 *>(&sm_qkv[1][4 * j]) : zero;   // the row of this position
    const float4 vp = on ? *reinterpret_cast<const float4 *>(&sm_qkv[2][4 * j]) : zero;
    const long base = (long)b * a.seq_stride + kvh * hstride + 4 * j;   // (MODE 0: the head's rows lie one after the other)
    float m = -3.0e38f, l = 0.0f;
    float4 acc = zero;
    constexpr int R = kBattnRows;   // rows in flight per slot
    const int last = max(pos - 1, 0);
    for (int tb = slot; tb < len; tb += R * NSLOT) {
        // (unconditional loads from the global address space: a row past the cache's last is that last row again and is
        // left out below; a load chosen by a condition became a flat load from one of two addresses)
        float4 kk[R], vv[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const long at = base + (long)min(tb + r * NSLOT, last) * rs;
            kk[r] = *reinterpret_cast<const float4 *>(a.kc + at);
            vv[r] = *reinterpret_cast<const float4 *>(a.vc + at);
        }
        float sv[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int t = tb + r * NSLOT;
            const bool cached = on && t < pos;
            // (component by component: a choice between whole float4s went through scratch memory)
            kk[r].x = t == pos ? kp.x : cached ? kk[r].x : 0.0f; kk[r].y = t == pos ? kp.y : cached ? kk[r].y : 0.0f;
            kk[r].z = t == pos ? kp.z : cached ? kk[r].z : 0.0f; kk[r].w = t == pos ? kp.w : cached ? kk[r].w : 0.0f;
            vv[r].x = t == pos ? vp.x : cached ? vv[r].x : 0.0f; vv[r].y = t == pos ? vp.y : cached ? vv[r].y : 0.0f;
            vv[r].z = t == pos ? vp.z : cached ? vv[r].z : 0.0f; vv[r].w = t == pos ? vp.w : cached ? vv[r].w : 0.0f;
            sv[r] = (q4.x * kk[r].x + q4.y * kk[r].y) + (q4.z * kk[r].z + q4.w * kk[r].w);
        }
#pragma unroll
        for (int off = LPR / 2; off > 0; off >>= 1) {
#pragma unroll
            for (int r = 0; r < R; r++) sv[r] += __shfl_xor(sv[r], off);
        }
        float mb = m;
#pragma unroll
        for (int r = 0; r < R; r++) {
            sv[r] = tb + r * NSLOT < len ? __fdiv_rn(sv[r], a.sqrt_hs) : -3.0e38f;
            mb = fmaxf(mb, sv[r]);
        }
        const float sc = expf(m - mb);
        l *= sc;
        acc.x *= sc; acc.y *= sc; acc.z *= sc; acc.w *= sc;
#pragma unroll
        for (int r = 0; r < R; r++) {
            const float p = tb + r * NSLOT < len ? expf(sv[r] - mb) : 0.0f;
            l += p;
            acc.x += p * vv[r].x; acc.y += p * vv[r].y; acc.z += p * vv[r].z; acc.w += p * vv[r].w;
        }
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
    const float *part;    // (slices, sequences, vocab) partial logits
    int slices, vocab;
    float *logits;        // (sequences, vocab)
    BatchState *st;
    const int *prompts;   // (sequences, prompt_stride)
    int prompt_stride;
    int *out_tokens;      // (sequences, out_stride): `next` of every step
    int out_stride;
};

// Logits of every sequence (the slices summed in order), first index of the maximum (J/Sampler.java:46-57) and the step of
// the token loop (J/Run.java:635-642, 668, 680): forced prompt id or argmax.  One workgroup per sequence; the last
// workgroup to finish advances the position.
static __global__ void __launch_bounds__(1024) k_bnext(const BNext a, unsigned *done)
{
    __shared__ float bval[16];
    __shared__ int bidx[16];
    const int b = blockIdx.x, tid = threadIdx.x;
    const long n = (long)gridDim.x * a.vocab;
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
        if (atomicAdd(done, 1u) == gridDim.x - 1) {   // every sequence has its token: the step is over
            *done = 0u;
            a.st->pos = pos + 1;
        }
    }
}

// y[b][r] = sum over the slices, in slice order
// Attention of 16 consecutive positions of one sequence for one head on the fp32 matrix cores (after k_battn<LPR, 1> has
// stored their k and v): every cache row is fetched once for the 16 queries, instead of once per query.
//   scores, transposed: S^T (16 keys x 16 queries) = K (16 keys x HS) . Q^T (HS x 16 queries), HS / 4 v_mfma_f32_16x16x4_f32;
//     a lane (c = lane % 16, g = lane / 16) then holds S^T[key 4 g + e][query c], e = 0..3: the keys of a query lie in four
//     lanes, so a query's maximum is two cross-lane steps, and the same registers are the B operand of
//   values, transposed: O^T (HS x 16 queries) += V^T (HS x 16 keys) . P^T (16 keys x 16 queries), HS / 4 more;
//   online softmax over the tiles of 16 keys (K/AttentionLoop.java:29-54, K/ExpSumNormalize.java:25-38,
//     K/AccumWeightedValue.java restated as in k_battn), a query seeing the keys up to its own position.
// The waves of the workgroup take every WAVES-th tile of keys and merge their (maximum, sum, values) through LDS.
// The k index of a product may be permuted if both operands are: lane group g supplies the dimensions 16 u + 4 g + e
// (one 16-byte load per u) and the keys 4 g + e.
// grid: (n_heads, 2, 1..4): z splits the tiles of keys over that many workgroups, the last of which to finish merges what the
// others left in device memory.  64 * WAVES threads; dynamic LDS: (16 (HS + 4) + 32 WAVES + 16 WAVES HS) floats.
template <int HS, int WAVES>
__global__ void __launch_bounds__(64 * WAVES) k_pflash(const BAttn a)
{
    constexpr int U = HS / 16;
    extern __shared__ __align__(16) float pf_lds[];
    constexpr int SQ = HS + 4;           // (a row of q four floats longer: the sixteen rows a wave reads together start in different banks)
    float *sq = pf_lds;                  // [16 queries][SQ]
    float *wm = pf_lds + 16 * SQ;        // [WAVES][16]
    float *wl = wm + WAVES * 16;         // [WAVES][16]
    float *wo = wl + WAVES * 16;         // [WAVES][HS / 4][16 queries][4]: dimension d of query q at (d / 4) * 64 + 4 q + d % 4
    __shared__ float ww[WAVES * 16], wM[16];
    __shared__ int s_last;
    const int h = blockIdx.x, qb = blockIdx.y * 16, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = lane & 15, g = lane >> 4;
    if (qb >= a.nrows) return;
    const int vrows = min(16, a.nrows - qb);   // (rows past the end repeat the last one: their output is not used)
    const int pos0 = a.st->pos + qb, kvh = h / a.kv_mul, half = HS / 2;
    for (int p = tid; p < 16 * half; p += 64 * WAVES) {   // q of the rows: the slices of the product added up, RoPE at the row's position
        const int r = p / half, idx = p - r * half, b = qb + min(r, vrows - 1);
        float v0 = 0.0f, v1 = 0.0f;
#pragma unroll 8
        for (int s = 0; s < a.slices; s++) {
            const float2 t = *reinterpret_cast<const float2 *>(a.pq + ((long)s * a.nseq + b) * a.dim + h * HS + 2 * idx);
            v0 += t.x; v1 += t.y;
        }
        const float2 cs = a.rope[(long)(a.st->pos + b) * half + idx];
        sq[r * SQ + 2 * idx] = __fsub_rn(__fmul_rn(v0, cs.x), __fmul_rn(v1, cs.y));
        sq[r * SQ + 2 * idx + 1] = __fadd_rn(__fmul_rn(v0, cs.y), __fmul_rn(v1, cs.x));
    }
    __syncthreads();
    float4 qv[U];
#pragma unroll
    for (int u = 0; u < U; u++) qv[u] = *reinterpret_cast<const float4 *>(&sq[c * SQ + 16 * u + 4 * g]);
    const int qpos = pos0 + min(c, vrows - 1), lastkey = pos0 + vrows - 1, ntiles = lastkey / 16 + 1;
    const float *kc = a.kc + kvh * a.head_stride, *vc = a.vc + kvh * a.head_stride;
    const long rs = a.row_stride;
    v4f32 o[U];
#pragma unroll
    for (int u = 0; u < U; u++) o[u] = v4f32{0.f, 0.f, 0.f, 0.f};
    float m = -3.0e38f, l = 0.0f;
    // tile t of the keys goes to workgroup t % NS (z) and there to wave (t / NS) % WAVES: few tiles spread over the workgroups first
    const int NS = gridDim.z;
    const int mytiles = (ntiles - (int)blockIdx.z + NS - 1) / NS;   // of this workgroup
    const int nw = min(WAVES, mytiles);                              // waves that have any
    for (int t = blockIdx.z + NS * wave; t < ntiles; t += NS * WAVES) {
        const int k0 = t * 16;
        const float *krow = kc + (long)min(k0 + c, lastkey) * rs + 4 * g;   // (past the last key: that key again, left out below)
        float4 kf[U];
#pragma unroll
        for (int u = 0; u < U; u++) kf[u] = *reinterpret_cast<const float4 *>(krow + 16 * u);
        v4f32 st = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < U; u++) {
            st = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[u].x, qv[u].x, st, 0, 0, 0);
            st = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[u].y, qv[u].y, st, 0, 0, 0);
            st = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[u].z, qv[u].z, st, 0, 0, 0);
            st = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[u].w, qv[u].w, st, 0, 0, 0);
        }
        float sv[4], tmax = -3.0e38f;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            sv[e] = k0 + 4 * g + e <= qpos ? __fdiv_rn(st[e], a.sqrt_hs) : -3.0e38f;   // (a query sees the keys up to its own position)
            tmax = fmaxf(tmax, sv[e]);
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
        const float mb = fmaxf(m, tmax), sc = expf(m - mb);
        float pr[4];
        l *= sc;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            pr[e] = k0 + 4 * g + e <= qpos ? expf(sv[e] - mb) : 0.0f;
            l += pr[e];
        }
#pragma unroll
        for (int u = 0; u < U; u++) o[u] *= sc;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float *vrow = vc + (long)min(k0 + 4 * g + e, lastkey) * rs + c;
#pragma unroll
            for (int u = 0; u < U; u++) o[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(vrow[16 * u], pr[e], o[u], 0, 0, 0);
        }
        m = mb;
    }
    l += __shfl_xor(l, 16);
    l += __shfl_xor(l, 32);
    if (g == 0) { wm[wave * 16 + c] = m; wl[wave * 16 + c] = l; }
    if (wave < nw) {   // (the waves without a tile have nothing to add)
#pragma unroll
        for (int u = 0; u < U; u++)   // (a lane's four dimensions 16 u + 4 g + e of query c as one 16-byte store, a wave's stores 1 KB in a row)
            *reinterpret_cast<v4f32 *>(&wo[wave * HS * 16 + (4 * u + g) * 64 + 4 * c]) = o[u];
    }
    __syncthreads();
    if (tid < 16 * WAVES) {   // weight of wave w's part in query q's sum: tid = w * 16 + q (a workgroup without any tile leaves
        const int q = tid & 15;   // maximum -3e38, sum 0 and values 0)
        float M = wm[q];
#pragma unroll
        for (int w = 1; w < WAVES; w++) M = fmaxf(M, wm[w * 16 + q]);
        ww[tid] = expf(wm[tid] - M);
        if (tid < 16) wM[tid] = M;
    }
    __syncthreads();
    if (NS == 1) {
        for (int idx = tid; idx < HS * 16; idx += 64 * WAVES) {   // the waves' parts of a query merged
            const int d = (idx >> 6) * 4 + (idx & 3), q = (idx >> 2) & 15;   // (neighbouring lanes read neighbouring words of LDS)
            float L = 0.0f, O = 0.0f;
#pragma unroll
            for (int w = 0; w < WAVES; w++) {
                if (w < nw) {
                    const float wt = ww[w * 16 + q];
                    L += wt * wl[w * 16 + q];
                    O += wt * wo[w * HS * 16 + idx];
                }
            }
            if (q < vrows) a.out[(long)(qb + q) * a.dim + h * HS + d] = __fdiv_rn(O, L);
        }
        return;
    }
    // The keys are split over NS workgroups: each leaves its maxima, sums and values (not yet divided) in device memory, and
    // the last one to do so merges them all.
    constexpr int PER = 32 + 16 * HS;
    const int pair = h * gridDim.y + blockIdx.y;
    float *mine = a.pf_part + ((long)pair * NS + blockIdx.z) * PER;
    for (int idx = tid; idx < HS * 16; idx += 64 * WAVES) {   // (values in the order they have in LDS)
        const int d = (idx >> 6) * 4 + (idx & 3), q = (idx >> 2) & 15;
        float L = 0.0f, O = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; w++) {
            if (w < nw) {
                const float wt = ww[w * 16 + q];
                L += wt * wl[w * 16 + q];
                O += wt * wo[w * HS * 16 + idx];
            }
        }
        st_coh(mine + 32 + idx, O);
        if (d == 0) { st_coh(mine + q, wM[q]); st_coh(mine + 16 + q, L); }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // (this thread's stores have arrived where the other workgroups read)
    __syncthreads();
    if (tid == 0) {
        const unsigned old = __hip_atomic_fetch_add(a.pf_cnt + pair, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = old + 1u == (unsigned)NS;
        if (s_last) __hip_atomic_store(a.pf_cnt + pair, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // (for the next launch)
    }
    __syncthreads();
    if (!s_last) return;
    const float *all = a.pf_part + (long)pair * NS * PER;
    for (int idx = tid; idx < HS * 16; idx += 64 * WAVES) {
        const int q = (idx >> 2) & 15;
        float mz[4], M = -3.0e38f;
#pragma unroll
        for (int z = 0; z < 4; z++) {
            mz[z] = z < NS ? ld_coh(all + (long)z * PER + q) : -3.0e38f;
            M = fmaxf(M, mz[z]);
        }
        float L = 0.0f, O = 0.0f;
#pragma unroll
        for (int z = 0; z < 4; z++) {
            if (z < NS) {
                const float wt = expf(mz[z] - M);
                L += wt * ld_coh(all + (long)z * PER + 16 + q);
                O += wt * ld_coh(all + (long)z * PER + 32 + idx);
            }
        }
        if (q < vrows) a.out[(long)(qb + q) * a.dim + h * HS + (idx >> 6) * 4 + (idx & 3)] = __fdiv_rn(O, L);
    }
}

// y[0..rows) = row `row` of the product whose slices lie in part, (slices, nseq, rows)
static __global__ void __launch_bounds__(256) k_brow(const float *__restrict__ part, float *__restrict__ y, int rows, int slices, int nseq, int row)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < rows; i += gridDim.x * blockDim.x) {
        float t = 0.0f;
        for (int sl = 0; sl < slices; sl++) t += part[((long)sl * nseq + row) * rows + i];
        y[i] = t;
    }
}

static __global__ void __launch_bounds__(256) k_breduce(const float *__restrict__ part, float *__restrict__ y, int rows, int slices)
{
    const long n = (long)kBatch * rows;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        float t = 0.0f;
        for (int sl = 0; sl < slices; sl++) t += part[(long)sl * n + i];
        y[i] = t;
    }
}

}  // namespace l2j
