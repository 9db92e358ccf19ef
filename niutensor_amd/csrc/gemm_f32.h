/*
 * fp32 GEMM for gfx950: c = alpha * op(a) op(b) + beta * c (+ bias), fp32 MFMA.
 * Replaces the cublasSgemm / cublasSgemmStridedBatched / cublasSgemmBatched calls of
 * the reference (source/tensor/core/arithmetic/XTensorBLAS.cu:61-72,133-145,204-216).
 *
 * One workgroup computes a BM x BN tile of c; its WGM x WGN waves each own a
 * (BM/WGM) x (BN/WGN) sub-tile held as 32x32 accumulator blocks of
 * v_mfma_f32_32x32x2_f32 (lane l feeds row/column l%32 at k slot l/32).
 *
 * Operand staging in LDS, chosen per operand by how it lies in memory:
 *   MN-contiguous (a with X_TRANS, b with X_NOTRANS): rows of k, S[k][mn].
 *       16-byte global loads and 16-byte LDS writes along mn; a fragment is
 *       32 consecutive floats per half-wave: no bank conflicts, no padding.
 *   K-contiguous (a with X_NOTRANS, b with X_TRANS): rows of mn, S[mn][k], row
 *       pitch BKT+4 floats. 16-byte global loads and 16-byte LDS writes along
 *       k; a lane fetches FOUR k values of its row with one 16-byte read, and
 *       the pitch of 80 bytes puts the eight lanes of a 128-byte LDS phase in
 *       eight different 16-byte bank groups.
 * The order in which k values meet inside a slab is free as long as both
 * operands agree, so MFMA step t of a slab takes k = 8*(t/4) + 4*(l/32) + t%4:
 * that is what makes the four-at-once fetch of the K-contiguous layout line up
 * with single-row fetches of the other layout.
 *
 * Pipeline, per slab of BKT values of k: the wave holds all its fragments of
 * the current slab in registers and issues MFMAs only from them; the next
 * slab travels global -> registers (one slab ahead) -> the other LDS stage
 * (first half of the MFMAs) -> one barrier -> the second register set (second
 * half of the MFMAs). The 16-byte global loads are buffer loads: the slab's
 * base address lives in scalar registers and advances by a scalar add, the
 * per-lane offset never changes, and reads past the end of the matrix return
 * zero in hardware, so the steady-state loop has no address arithmetic and no
 * predication on the vector side.
 */
#pragma once
#include "gemm_common.h"
#include <type_traits>

namespace ntsamd {

template <int N>
struct IntC {
    static constexpr int value = N;
};

/* a raw buffer descriptor over [base, base + bytes): dword 3 selects 32-bit data, no swizzle */
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void * base, long long bytes)
{
    /* bytes > 0 always: the base is inside the matrix */
    int n = (unsigned long long)bytes >> 31 ? 0x7fffffff : (int)bytes;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, n, 0x00020000);
}

/* a byte offset no descriptor made by make_rsrc covers: the load returns zero */
#define NTSAMD_OOB_OFFSET 0x7fffffff

__device__ __forceinline__ f32x4 buffer_load_f32x4(__amdgpu_buffer_rsrc_t rsrc, int byteOffset)
{
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, byteOffset, 0, 0);
    return __builtin_bit_cast(f32x4, v);
}

/* R16 (products with at most 16 rows, on the 32 x 128 tile): a wave multiplies only the first 16 rows of the
   tile, as two 16 x 16 blocks of v_mfma_f32_16x16x4_f32 side by side (lane l feeds row/column l % 16 at k slot
   l / 16; step t of a group of 16 k takes k = 4 * (l / 16) + t, so a K-contiguous operand is still one 16-byte
   read per group): half the MFMA work of 32 padded rows, and a chain of dependent MFMAs half as long. */
template <int BM, int BN, int BKT, int WGM, int WGN, bool AKC, bool BKC, bool VEC, bool CS, typename PT, bool R16 = false>
__global__ void __launch_bounds__(WGM * WGN * 64, 2)
gemm_f32_kernel(const GemmParams p, const PT tab)
{
    static_assert(!R16 || (BM == 32 && WGM == 1 && VEC && !CS), "16-row MFMAs: one row of waves on a 32-row tile");
    constexpr int NT = WGM * WGN * 64;
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int BS = R16 ? 16 : 32;                      /* rows and columns of an accumulator block */
    constexpr int TI = R16 ? 1 : WM / 32, TJ = WN / BS;
    constexpr int KPM = R16 ? 4 : 2;                       /* k per MFMA */
    constexpr int KG = 4 * KPM;                            /* k per group of four MFMA steps */
    constexpr int ACCN = R16 ? 4 : 16;                     /* accumulator registers per block */
    constexpr int KK = BKT / KPM;         /* MFMA steps per slab */
    /* K-contiguous operand in LDS. Slab of 32: rows BKT + 4 floats apart. Slab of 16: rows of 64 bytes with no
       padding, four to a 256-byte line of the 64 banks, and the four 16-byte pieces of row r stored permuted,
       piece u at position u ^ ((r >> 2) & 3): rows r, r+4, r+8, r+12 share their 64 bytes of the line, and both the
       sixteen lanes that write four rows and the sixteen that read one piece of sixteen rows cover the whole line
       (the 80-byte pitch this replaces made the writes of a fourth row wrap into the first: 17 % of the LDS
       cycles were bank conflicts) */
    constexpr bool SWZ = BKT == 16;
    constexpr int LDK = SWZ ? BKT : BKT + 4;
    constexpr int NA = BM * BKT / 4 / NT;
    constexpr int NB = BN * BKT / 4 / NT;
    constexpr int ASIZE = AKC ? BM * LDK : BKT * BM;
    constexpr int BSIZE = BKC ? BN * LDK : BKT * BN;
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be made of 32x32 blocks");
    static_assert((BM * BKT / 4) % NT == 0 && (BN * BKT / 4) % NT == 0, "loads must divide evenly");
    static_assert(BKT % 8 == 0, "slab depth");

    __shared__ __attribute__((aligned(16))) float As[2][ASIZE];
    __shared__ __attribute__((aligned(16))) float Bs[2][BSIZE];

    const TileCoord tc = tile_of_workgroup(p);
    const float * __restrict__ A;
    const float * __restrict__ B;
    float * __restrict__ C;
    if constexpr (sizeof(PT) > 1) {
        A = static_cast<const float *>(tab.a[tc.batch]);
        B = static_cast<const float *>(tab.b[tc.batch]);
        C = static_cast<float *>(tab.c[tc.batch]);
    }
    else {
        A = static_cast<const float *>(p.a) + batch_offset(tc.batch, p.batchInner, p.strideA, p.strideA1);
        B = static_cast<const float *>(p.b) + batch_offset(tc.batch, p.batchInner, p.strideB, p.strideB1);
        C = static_cast<float *>(p.c) + batch_offset(tc.batch, p.batchInner, p.strideC, p.strideC1);
    }

    const int M = p.M, N = p.N, K = p.K;
    /* R16: a workgroup multiplies the first 16 rows of what it stages, and the workgroups stand 16 rows apart */
    const int m0 = tc.tm * (R16 ? 16 : BM), n0 = tc.tn * BN;
    const int tid = threadIdx.x;
    /* the wave number is the same in every lane: said explicitly, or every buffer access whose descriptor is built
       from it (the epilogue's 64 stores per lane) is wrapped in a loop that tests the descriptor lane by lane */
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave / WGN) * WM, wn0 = (wave % WGN) * WN;
    const int l32 = R16 ? (lane & 15) : (lane & 31);      /* row / column inside a block */
    const int lh = R16 ? (lane >> 4) : (lane >> 5);        /* k slot */

    /* ---- staging slots: which 4 elements of the slab each thread moves ------ */
    int aOff[NA], bOff[NB];        /* 16-byte path: byte offset from the slab base */
    int aLds[NA], bLds[NB];        /* float index in the LDS stage */
    int aK[NA], bK[NB];            /* k of the slot's first element inside the slab */
    int aMN[NA], bMN[NB];          /* row (K-contiguous) or first column (MN-contiguous) inside the tile */
#pragma unroll
    for (int s = 0; s < NA; s++) {
        int g = tid + s * NT;
        if (AKC) {
            int row = g / (BKT / 4);
            aK[s] = (g % (BKT / 4)) * 4;
            aMN[s] = row;
            aLds[s] = SWZ ? row * LDK + (((aK[s] >> 2) ^ ((row >> 2) & 3)) << 2) : row * LDK + aK[s];
            int r = m0 + row < M - 1 ? row : M - 1 - m0;        /* rows past the edge repeat the last one */
            aOff[s] = (r * p.lda + aK[s]) * 4;
        }
        else {
            aK[s] = g / (BM / 4);
            aMN[s] = (g % (BM / 4)) * 4;
            aLds[s] = aK[s] * BM + aMN[s];
            /* four columns from aMN[s] on. A run that starts inside the row may end in the next one (rows
               need not be multiples of four long): what it brings from there lands in columns past M,
               whose results are never stored. A run that starts past the row reads as zero. */
            aOff[s] = m0 + aMN[s] < M ? (aK[s] * p.lda + aMN[s]) * 4 : NTSAMD_OOB_OFFSET;
        }
    }
#pragma unroll
    for (int s = 0; s < NB; s++) {
        int g = tid + s * NT;
        if (BKC) {
            int row = g / (BKT / 4);
            bK[s] = (g % (BKT / 4)) * 4;
            bMN[s] = row;
            bLds[s] = SWZ ? row * LDK + (((bK[s] >> 2) ^ ((row >> 2) & 3)) << 2) : row * LDK + bK[s];
            int r = n0 + row < N - 1 ? row : N - 1 - n0;
            bOff[s] = (r * p.ldb + bK[s]) * 4;
        }
        else {
            bK[s] = g / (BN / 4);
            bMN[s] = (g % (BN / 4)) * 4;
            bLds[s] = bK[s] * BN + bMN[s];
            bOff[s] = n0 + bMN[s] < N ? (bK[s] * p.ldb + bMN[s]) * 4 : NTSAMD_OOB_OFFSET;
        }
    }

    /* first element of the tile's operand panels, and one past the end of each matrix */
    const float * aTile = AKC ? A + (size_t)m0 * p.lda : A + m0;
    const float * bTile = BKC ? B + (size_t)n0 * p.ldb : B + n0;
    const float * aEnd = A + (size_t)((AKC ? M : K) - 1) * p.lda + (AKC ? K : M);
    const float * bEnd = B + (size_t)((BKC ? N : K) - 1) * p.ldb + (BKC ? K : N);

    f32x4 ra[NA], rb[NB];

    auto load_global = [&](auto TAIL, int k0) {
        constexpr bool mayHangOver = decltype(TAIL)::value != 0;
        if constexpr (VEC) {
            const float * ab = AKC ? aTile + k0 : aTile + (size_t)k0 * p.lda;
            const float * bb = BKC ? bTile + k0 : bTile + (size_t)k0 * p.ldb;
            __amdgpu_buffer_rsrc_t ar = make_rsrc(ab, (long long)(aEnd - ab) * 4);
            __amdgpu_buffer_rsrc_t br = make_rsrc(bb, (long long)(bEnd - bb) * 4);
            /* only the last slab can hang over K. Rows of k past the end of an MN-contiguous
               matrix are past the end of the buffer and read as zero by themselves; a
               K-contiguous row would run on into the next row instead, so those lanes are
               sent out of range explicitly */
            const bool tail = mayHangOver && k0 + BKT > K;
#pragma unroll
            for (int s = 0; s < NA; s++) {
                int off = aOff[s];
                if (AKC && tail && k0 + aK[s] >= K)
                    off = NTSAMD_OOB_OFFSET;
                ra[s] = buffer_load_f32x4(ar, off);
            }
#pragma unroll
            for (int s = 0; s < NB; s++) {
                int off = bOff[s];
                if (BKC && tail && k0 + bK[s] >= K)
                    off = NTSAMD_OOB_OFFSET;
                rb[s] = buffer_load_f32x4(br, off);
            }
            /* K need not be a multiple of four: the run that straddles it keeps its k < K only */
            if constexpr (mayHangOver && AKC) {
                if (tail) {
#pragma unroll
                    for (int s = 0; s < NA; s++)
#pragma unroll
                        for (int e = 1; e < 4; e++)
                            if (k0 + aK[s] + e >= K)
                                ra[s][e] = 0.f;
                }
            }
            if constexpr (mayHangOver && BKC) {
                if (tail) {
#pragma unroll
                    for (int s = 0; s < NB; s++)
#pragma unroll
                        for (int e = 1; e < 4; e++)
                            if (k0 + bK[s] + e >= K)
                                rb[s][e] = 0.f;
                }
            }
        }
        else {
            /* generic path: any alignment, element by element, predicated */
#pragma unroll
            for (int s = 0; s < NA; s++) {
                f32x4 v = {0.f, 0.f, 0.f, 0.f};
                if (AKC) {
                    int r = m0 + aMN[s] < M - 1 ? m0 + aMN[s] : M - 1;
                    const float * rp = A + (size_t)r * p.lda;
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (k0 + aK[s] + e < K)
                            v[e] = rp[k0 + aK[s] + e];
                }
                else if (k0 + aK[s] < K) {
                    const float * rp = A + (size_t)(k0 + aK[s]) * p.lda;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        int c = m0 + aMN[s] + e < M - 1 ? m0 + aMN[s] + e : M - 1;
                        v[e] = rp[c];
                    }
                }
                ra[s] = v;
            }
#pragma unroll
            for (int s = 0; s < NB; s++) {
                f32x4 v = {0.f, 0.f, 0.f, 0.f};
                if (BKC) {
                    int r = n0 + bMN[s] < N - 1 ? n0 + bMN[s] : N - 1;
                    const float * rp = B + (size_t)r * p.ldb;
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (k0 + bK[s] + e < K)
                            v[e] = rp[k0 + bK[s] + e];
                }
                else if (k0 + bK[s] < K) {
                    const float * rp = B + (size_t)(k0 + bK[s]) * p.ldb;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        int c = n0 + bMN[s] + e < N - 1 ? n0 + bMN[s] + e : N - 1;
                        v[e] = rp[c];
                    }
                }
                rb[s] = v;
            }
        }
    };

    auto store_lds = [&](int buf) {
#pragma unroll
        for (int s = 0; s < NA; s++)
            *reinterpret_cast<f32x4 *>(&As[buf][aLds[s]]) = ra[s];
#pragma unroll
        for (int s = 0; s < NB; s++)
            *reinterpret_cast<f32x4 *>(&Bs[buf][bLds[s]]) = rb[s];
    };

    /* ---- fragments: two register sets, [set][...] ----------------------------
       K-contiguous operand: one f32x4 per block and per group of four steps;
       MN-contiguous operand: one float per block and per step */
    f32x4 fa4[2][AKC ? KK / 4 : 1][TI];
    float fa1[2][AKC ? 1 : KK][TI];
    f32x4 fb4[2][BKC ? KK / 4 : 1][TJ];
    float fb1[2][BKC ? 1 : KK][TJ];

    auto read_frags = [&](auto SET, int buf) {
        constexpr int set = decltype(SET)::value;
        if constexpr (AKC) {
            const float * as = &As[buf][(wm0 + l32) * LDK + (SWZ ? 0 : 4 * lh)];
#pragma unroll
            for (int q = 0; q < KK / 4; q++)
#pragma unroll
                for (int i = 0; i < TI; i++)
                    fa4[set][q][i] = *reinterpret_cast<const f32x4 *>(
                        as + i * 32 * LDK + (SWZ ? (((lh + (KG / 4) * q) ^ ((l32 >> 2) & 3)) << 2) : KG * q));
        }
        else {
            const float * as = &As[buf][4 * lh * BM + wm0 + l32];
#pragma unroll
            for (int t = 0; t < KK; t++)
#pragma unroll
                for (int i = 0; i < TI; i++)
                    fa1[set][t][i] = as[(KG * (t / 4) + (t % 4)) * BM + i * 32];
        }
        if constexpr (BKC) {
            const float * bs = &Bs[buf][(wn0 + l32) * LDK + (SWZ ? 0 : 4 * lh)];
#pragma unroll
            for (int q = 0; q < KK / 4; q++)
#pragma unroll
                for (int j = 0; j < TJ; j++)
                    fb4[set][q][j] = *reinterpret_cast<const f32x4 *>(
                        bs + j * BS * LDK + (SWZ ? (((lh + (KG / 4) * q) ^ ((l32 >> 2) & 3)) << 2) : KG * q));
        }
        else {
            const float * bs = &Bs[buf][4 * lh * BN + wn0 + l32];
#pragma unroll
            for (int t = 0; t < KK; t++)
#pragma unroll
                for (int j = 0; j < TJ; j++)
                    fb1[set][t][j] = bs[(KG * (t / 4) + (t % 4)) * BN + j * BS];
        }
    };

    typedef typename std::conditional<R16, f32x4, f32x16>::type Acc;
    Acc acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; i++)
#pragma unroll
        for (int j = 0; j < TJ; j++)
#pragma unroll
            for (int r = 0; r < ACCN; r++)
                acc[i][j][r] = 0.f;

    /* CS: every lane also adds up the op(b) values that pass through its fragments: lane
       (l32, lh) of a wave sees, for each of its columns, every k of the slab that its half
       of the wave feeds to the MFMAs; the two halves are added at the end */
    float colSum[CS ? TJ : 1];
#pragma unroll
    for (int j = 0; j < (CS ? TJ : 1); j++)
        colSum[j] = 0.f;

    auto mfma_steps = [&](auto SET, int first, int last) {
        constexpr int set = decltype(SET)::value;
#pragma unroll
        for (int t = first; t < last; t++)
#pragma unroll
            for (int i = 0; i < TI; i++)
#pragma unroll
                for (int j = 0; j < TJ; j++) {
                    float av = AKC ? fa4[set][t / 4][i][t % 4] : fa1[set][t][i];
                    float bv = BKC ? fb4[set][t / 4][j][t % 4] : fb1[set][t][j];
                    if constexpr (R16)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, bv, acc[i][j], 0, 0, 0);
                    else
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[i][j], 0, 0, 0);
                    if constexpr (CS)
                        if (i == 0)
                            colSum[j] += bv;
                }
    };

    /* this workgroup's k range: all of K, or one of p.splits pieces */
    const int kBeg = tc.split * p.kPerSplit;
    const int kLen = (p.splits > 1 && kBeg + p.kPerSplit < K ? p.kPerSplit : K - kBeg);
    const int nk = (kLen + BKT - 1) / BKT;

    /* One slab: fragments of slab kt are in register set SET and came from LDS stage SET.
       FULL: slabs kt+1 and kt+2 exist and are complete, so nothing is conditional and the
       slab is one straight run of instructions that the scheduler can interleave. */
    auto slab = [&](auto SET, auto FULL, int kt) {
        constexpr int set = decltype(SET)::value;
        constexpr bool full = decltype(FULL)::value != 0;
        if (full || kt + 1 < nk)
            store_lds(set ^ 1);                  /* slab kt+1, fetched during slab kt-1 */
        if (full)
            load_global(IntC<0>(), kBeg + (kt + 2) * BKT);
        else if (kt + 2 < nk)
            load_global(IntC<1>(), kBeg + (kt + 2) * BKT);
        mfma_steps(SET, 0, KK / 2);
        if constexpr (full) {
            /* An MFMA keeps the matrix pipe busy for 64 cycles but takes one issue slot:
               spread the LDS writes, the buffer loads and their scalar bookkeeping
               between the MFMAs instead of in front of them, so the pipe never waits
               for this wave to get through a block of other work. */
#pragma unroll
            for (int g = 0; g < KK / 2 * TI * TJ; g++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);     /* one MFMA */
                __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);     /* one LDS write */
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);     /* one global read */
                __builtin_amdgcn_sched_group_barrier(0x006, 4, 0);     /* some scalar / vector ALU */
            }
        }
        /* keep the compiler from sliding MFMAs across the barrier: the point of
           the first half is to be in flight while the wave waits here */
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();                         /* stage set^1 complete; stage set no longer read by anyone */
        __builtin_amdgcn_sched_barrier(0);
        if (full || kt + 1 < nk)
            read_frags(IntC<set ^ 1>(), set ^ 1);
        mfma_steps(SET, KK / 2, KK);
        if constexpr (full) {
#pragma unroll
            for (int g = 0; g < KK / 2 * TI * TJ; g++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);     /* one MFMA */
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);     /* one LDS read */
                __builtin_amdgcn_sched_group_barrier(0x006, 2, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    if (nk > 0) {
        load_global(IntC<1>(), kBeg);
        store_lds(0);
        if (nk > 1)
            load_global(IntC<1>(), kBeg + BKT);
        __syncthreads();
        read_frags(IntC<0>(), 0);
        const int nkFull = kLen / BKT;           /* slabs that lie entirely inside the k range */
        int kt = 0;
        for (; kt + 3 < nkFull; kt += 2) {
            slab(IntC<0>(), IntC<1>(), kt);
            slab(IntC<1>(), IntC<1>(), kt + 1);
        }
        for (; kt < nk; kt += 2) {
            slab(IntC<0>(), IntC<0>(), kt);
            if (kt + 1 < nk)
                slab(IntC<1>(), IntC<0>(), kt + 1);
        }
    }

    /* ---- epilogue: accumulator register r of lane l is element
       (8*(r/4) + 4*(l/32) + r%4, l%32) of its 32x32 block, so a store covers
       two rows of 32 consecutive floats and needs no alignment of ldc
       (16x16 blocks: element (4*(l/16) + r, l%16), four rows of 16 floats) ---------- */
    const float alpha = p.alpha, beta = p.beta;
    const float * __restrict__ bias = static_cast<const float *>(p.bias);
    const int biasMode = p.biasMode;
    const int act = p.act;

    if constexpr (VEC) {
        /* The wave's rows of c as one buffer that ends where c ends: rows past M drop
           off its end and columns past N are sent out of range, so the stores (and the
           loads for beta != 0) need no predicates. Row-indexed bias is not handled here. */
        if (m0 + wm0 >= M)
            return;
        float * cw = C + (size_t)(m0 + wm0) * p.ldc;
        __amdgpu_buffer_rsrc_t cr = make_rsrc(cw, (long long)(M - m0 - wm0) * p.ldc * 4);
        const unsigned rowPitch = (unsigned)p.ldc * 4u;
        unsigned cOff[TJ];
        float bcol[TJ];
#pragma unroll
        for (int j = 0; j < TJ; j++) {
            const int col = n0 + wn0 + j * BS + l32;
            cOff[j] = col < N ? (unsigned)(4 * lh * p.ldc + col) * 4u : (unsigned)NTSAMD_OOB_OFFSET;
            bcol[j] = biasMode == BIAS_COL && col < N ? bias[col] : 0.f;
        }
        if constexpr (CS) {
            /* the first tile row's first wave row has seen every k of its columns */
            if (tc.tm == 0 && wm0 == 0) {
                float * cs = static_cast<float *>(p.colSum);
#pragma unroll
                for (int j = 0; j < TJ; j++) {
                    const float v = colSum[j] + __shfl_xor(colSum[j], 32);
                    const int col = n0 + wn0 + j * BS + l32;
                    if (lh == 0 && col < N) {
                        if (p.splits > 1)
                            unsafeAtomicAdd(cs + col, v);      /* the caller has applied colSumBeta */
                        else
                            cs[col] = p.colSumBeta != 0.f ? p.colSumBeta * cs[col] + v : v;
                    }
                }
            }
        }
        if (p.splits > 1 && p.splitWork != NULL) {
            /* one of several workgroups that share this tile, and a workspace for them to meet in: the partial
               tile goes there as it is (splits x batch dense M x N matrices), and split_reduce.hip adds the pieces
               in their order, the same bits on every run, and applies alpha, beta, bias and activation */
            float * w = p.splitWork + ((size_t)tc.split * p.batch + tc.batch) * M * N;
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                const int col = n0 + wn0 + j * BS + l32;
                if (col < N) {
#pragma unroll
                    for (int i = 0; i < TI; i++)
#pragma unroll
                        for (int r = 0; r < ACCN; r++) {
                            const int row = m0 + wm0 + i * 32 + (R16 ? r : 8 * (r / 4) + (r % 4)) + 4 * lh;
                            if (row < M)
                                w[(size_t)row * N + col] = acc[i][j][r];
                        }
                }
            }
            return;
        }
        if (p.splits > 1) {
            /* no workspace: add the partial product to c,
               which already holds beta * c; the bias rides on the first piece. Every add is
               predicated on its own row and column: an atomic must never be issued out of range
               (loads and stores past the end of a buffer are dropped by the hardware; this path
               does not rely on the same for atomics and uses plain global atomics). */
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                const int col = n0 + wn0 + j * BS + l32;
                if (col < N) {
                    const float bj = tc.split == 0 ? bcol[j] : 0.f;
#pragma unroll
                    for (int i = 0; i < TI; i++)
#pragma unroll
                        for (int r = 0; r < ACCN; r++) {
                            const int row = m0 + wm0 + i * 32 + (R16 ? r : 8 * (r / 4) + (r % 4)) + 4 * lh;
                            if (row < M)
                                unsafeAtomicAdd(C + (size_t)row * p.ldc + col, alpha * acc[i][j][r] + bj);
                        }
                }
            }
            return;
        }
        /* beta is tested once, outside the loops: inside them the test would fence every
           load of c off in a block of its own, one memory round trip after the other; the cache policy of the
           stores is a constant of the instruction, so it is chosen out here too */
        auto store_all = [&](auto BETAC, auto AUXC) {
            constexpr bool useOld = decltype(BETAC)::value != 0;
            constexpr int aux = decltype(AUXC)::value;
            float old[useOld ? TI : 1][useOld ? TJ : 1][ACCN];
            if constexpr (useOld) {
#pragma unroll
                for (int i = 0; i < TI; i++)
#pragma unroll
                    for (int j = 0; j < TJ; j++)
#pragma unroll
                        for (int r = 0; r < ACCN; r++) {
                            const unsigned off = cOff[j] + (unsigned)(i * 32 + (R16 ? r : 8 * (r / 4) + (r % 4))) * rowPitch;
                            old[i][j][r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(cr, (int)off, 0, 0));
                        }
            }
#pragma unroll
            for (int i = 0; i < TI; i++)
#pragma unroll
                for (int j = 0; j < TJ; j++)
#pragma unroll
                    for (int r = 0; r < ACCN; r++) {
                        const unsigned off = cOff[j] + (unsigned)(i * 32 + (R16 ? r : 8 * (r / 4) + (r % 4))) * rowPitch;
                        float v = alpha * acc[i][j][r] + bcol[j];
                        if constexpr (useOld)
                            v += beta * old[i][j][r];
                        v = activate(v, act);
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), cr, (int)off, 0, aux);
                    }
        };
        if (beta != 0.f) {
            if (p.storeHint)
                store_all(IntC<1>(), IntC<STORE_WRITE_THROUGH>());
            else
                store_all(IntC<1>(), IntC<STORE_DEFAULT>());
        }
        else {
            if (p.storeHint)
                store_all(IntC<0>(), IntC<STORE_WRITE_THROUGH>());
            else
                store_all(IntC<0>(), IntC<STORE_DEFAULT>());
        }
    }
    else {
        /* generic path: plain pointers, per-element bounds, every bias mode */
#pragma unroll
        for (int j = 0; j < TJ; j++) {
            const int col = n0 + wn0 + j * BS + l32;
            if (col >= N)
                continue;
            float bcol = 0.f;
            if (biasMode == BIAS_COL)
                bcol = bias[col];
#pragma unroll
            for (int i = 0; i < TI; i++) {
                const int rowBase = m0 + wm0 + i * 32 + 4 * lh;
                float * cb = C + (size_t)rowBase * p.ldc + col;
#pragma unroll
                for (int r = 0; r < ACCN; r++) {
                    const int dr = R16 ? r : 8 * (r / 4) + (r % 4);
                    if (rowBase + dr < M) {
                        float * cp = cb + (size_t)dr * p.ldc;
                        float v = alpha * acc[i][j][r];
                        if (beta != 0.f)
                            v += beta * (*cp);
                        if (biasMode == BIAS_ROW)
                            v += bias[((rowBase + dr) / p.biasRowDiv) % p.biasLen];
                        else
                            v += bcol;
                        *cp = activate(v, act);
                    }
                }
            }
        }
    }
}

template <int CFG, bool AKC, bool BKC, bool VEC, bool CS, typename PT, bool R16 = false>
static int launch_f32_one(const GemmParams & p0, const PT & tab, hipStream_t stream)
{
    typedef TileShape<CFG> S;
    GemmParams p = p0;
    p.tilesM = R16 ? (p.M + 15) / 16 : (p.M + S::BM - 1) / S::BM;
    p.tilesN = (p.N + S::BN - 1) / S::BN;
    if (p.splits < 1 || !VEC)
        p.splits = 1;
    dim3 grid((unsigned)(p.tilesM * p.tilesN * p.batch * p.splits));
    hipLaunchKernelGGL((gemm_f32_kernel<S::BM, S::BN, S::BKT32, S::WGM, S::WGN, AKC, BKC, VEC, CS, PT, R16>),
                       grid, dim3(S::WGM * S::WGN * 64), 0, stream, p, tab);
    return (int)hipGetLastError();
}

template <bool AKC, bool BKC>
static int launch_f32_trans(const GemmParams & p, const PtrBatch * ptrs, bool vec, int cfg, hipStream_t stream)
{
    NoPtrs none = {0};
    if (ptrs) {
        /* a list of matrices: the same kernels, each workgroup looks its matrices up in the argument block */
        if (!vec)
            return launch_f32_one<CFG_64x64, AKC, BKC, false, false, PtrBatch>(p, *ptrs, stream);
        if (cfg == CFG_128x128)
            return launch_f32_one<CFG_128x128, AKC, BKC, true, false, PtrBatch>(p, *ptrs, stream);
        return launch_f32_one<CFG_64x64, AKC, BKC, true, false, PtrBatch>(p, *ptrs, stream);
    }
    if (!vec)
        return launch_f32_one<CFG_64x64, AKC, BKC, false, false, NoPtrs>(p, none, stream);
    /* column sums and split k ranges exist on the 16-byte path only; the caller checks that */
    if (p.colSum != NULL) {
        if (cfg == CFG_128x128)
            return launch_f32_one<CFG_128x128, AKC, BKC, true, true, NoPtrs>(p, none, stream);
        return launch_f32_one<CFG_64x64, AKC, BKC, true, true, NoPtrs>(p, none, stream);
    }
    if (cfg == CFG_128x128)
        return launch_f32_one<CFG_128x128, AKC, BKC, true, false, NoPtrs>(p, none, stream);
    if (cfg == CFG_32x128 || cfg == CFG_16x128) {
        /* at most 16 rows, or 16 rows per workgroup asked for: 16-row MFMAs on the same tile (p.wideRowsOnly
           keeps the 32-row ones for products of at most 16 rows: for measurements) */
        if (cfg == CFG_16x128 || (p.M <= 16 && !p.wideRowsOnly))
            return launch_f32_one<CFG_32x128, AKC, BKC, true, false, NoPtrs, true>(p, none, stream);
        return launch_f32_one<CFG_32x128, AKC, BKC, true, false, NoPtrs>(p, none, stream);
    }
    return launch_f32_one<CFG_64x64, AKC, BKC, true, false, NoPtrs>(p, none, stream);
}

}  // namespace ntsamd
