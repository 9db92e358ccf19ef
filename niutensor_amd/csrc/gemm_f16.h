/*
 * fp16 GEMM for gfx950 with fp32 accumulation: c = alpha * op(a) op(b) + beta * c (+ bias).
 * Replaces the cublasGemmEx / cublasGemmStridedBatchedEx / cublasGemmBatchedEx calls
 * of the reference (source/tensor/core/arithmetic/XTensorBLAS.cu:73-100,146-173,217-243).
 * The reference asks cuBLAS for fp16 accumulation and rounds alpha and beta to
 * half (:74-78); this kernel keeps alpha, beta and the accumulator in fp32 and
 * rounds once, to nearest even, when it stores a half result.
 *
 * v_mfma_f32_32x32x16_f16 takes, per lane, eight consecutive k of one row (A) or
 * one column (B): lane l holds row/column l%32 and k = 8*(l/32) .. +7 of the step.
 * Operand staging in LDS, chosen per operand by how it lies in memory:
 *   K-contiguous (a with X_NOTRANS, b with X_TRANS): rows of mn, S[mn][k], 64 bytes
 *       each without padding, the four 16-byte pieces of a row permuted by
 *       (row >> 2) & 3. 16-byte global loads and LDS writes along k; a fragment is
 *       one 16-byte LDS read. Neither the writes (sixteen lanes: four rows) nor the
 *       reads (sixteen lanes: one piece of sixteen rows) meet in a bank.
 *   MN-contiguous (a with X_TRANS, b with X_NOTRANS): rows of k, S[k][mn], pitch
 *       BMN+32 halves. 16-byte global loads and LDS writes along mn; a fragment is
 *       two ds_read_b64_tr_b16: within 16 lanes the instruction hands lane c the
 *       c-th half of each of the four rows that lanes 0-3, 4-7, 8-11, 12-15 point
 *       at, which is exactly "four consecutive k of column c" when those lane
 *       groups point at four consecutive k rows. Thirty-two lanes take 64 bytes of
 *       each of four k rows in one cycle of the 64 banks: the pitch of 64 bytes
 *       mod 256 keeps those apart.
 *
 * Pipeline per slab of BKT values of k, as in the fp32 kernel: all fragments of
 * the current slab sit in registers; a later slab goes global -> registers ->
 * the other LDS stage -> one barrier -> the second register set, and every one
 * of those instructions is interleaved between MFMAs. The registers between
 * global memory and LDS are a ring of RING slabs: a slab is requested RING
 * slabs before its turn and written to LDS one slab before it, so RING - 1
 * slabs are on their way at any time (a trip to memory takes several slabs'
 * worth of MFMAs, and nothing else covers it where a workgroup has its CU to
 * itself: 4096 x 512 x 30011 with rows of 30011 halves took 642 us with one slab
 * on its way).
 */
#pragma once
#include "gemm_common.h"
#include "gemm_f32.h"   /* make_rsrc, IntC, NTSAMD_OOB_OFFSET */
#include <type_traits>

namespace ntsamd {

typedef _Float16 half_t;

__device__ __forceinline__ f16x8 buffer_load_f16x8(__amdgpu_buffer_rsrc_t rsrc, int byteOffset)
{
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, byteOffset, 0, 0);
    return __builtin_bit_cast(f16x8, v);
}

/* Eight halves from any 2-byte aligned place in a buffer of `bytes` bytes. A 16-byte buffer load may start on any
   even address, but its range check works on whole dwords: where the eight halves hang over the end of the buffer
   the dword that straddles the end is dropped with its valid half. Such a piece (the last of the matrix, at most)
   is fetched half by half instead. The test is a branch around the load, and a loop body cut up by branches waits
   for ALL loads in flight at every turn: only the loads of the last slabs go through here. */
__device__ __forceinline__ f16x8 buffer_load_f16x8_any(__amdgpu_buffer_rsrc_t rsrc, int byteOffset, int bytes)
{
    f16x8 v;
    if ((unsigned)byteOffset < (unsigned)bytes && (unsigned)byteOffset + 16u > (unsigned)bytes) {
#pragma unroll
        for (int e = 0; e < 8; e++)
            v[e] = __builtin_bit_cast(_Float16, __builtin_amdgcn_raw_buffer_load_b16(rsrc, byteOffset + 2 * e, 0, 0));
    }
    else
        v = buffer_load_f16x8(rsrc, byteOffset);
    return v;
}

/* transposing LDS read: see the header comment for what each lane receives */
__device__ __forceinline__ f16x4 lds_read_tr16(const half_t * p)
{
    typedef __fp16 hv4 __attribute__((__vector_size__(4 * sizeof(__fp16))));
    hv4 v = __builtin_amdgcn_ds_read_tr16_b64_v4f16((__attribute__((address_space(3))) hv4 *)(p));
    return __builtin_bit_cast(f16x4, v);
}

template <typename OutT>
__device__ __forceinline__ void buffer_store_out(OutT v, __amdgpu_buffer_rsrc_t rsrc, int byteOffset);
template <>
__device__ __forceinline__ void buffer_store_out<float>(float v, __amdgpu_buffer_rsrc_t rsrc, int byteOffset)
{
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), rsrc, byteOffset, 0, 0);
}
template <>
__device__ __forceinline__ void buffer_store_out<half_t>(half_t v, __amdgpu_buffer_rsrc_t rsrc, int byteOffset)
{
    __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, v), rsrc, byteOffset, 0, 0);
}
template <typename OutT>
__device__ __forceinline__ float buffer_load_out(__amdgpu_buffer_rsrc_t rsrc, int byteOffset);
template <>
__device__ __forceinline__ float buffer_load_out<float>(__amdgpu_buffer_rsrc_t rsrc, int byteOffset)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, byteOffset, 0, 0));
}
template <>
__device__ __forceinline__ float buffer_load_out<half_t>(__amdgpu_buffer_rsrc_t rsrc, int byteOffset)
{
    return (float)__builtin_bit_cast(half_t, __builtin_amdgcn_raw_buffer_load_b16(rsrc, byteOffset, 0, 0));
}

/* AT: the element type of a in memory. With float, a is rounded to half (to nearest even, as
   _CudaConvertDataType does, core/getandset/ConvertDataType.cu:31-38) on its way from the registers into LDS: the
   product of float probabilities with half values needs no converted copy of the probabilities
   (source/sample/transformer/submodel/Attention.cpp:231-237). */
template <typename OutT, int BM, int BN, int BKT, int WGM, int WGN, int MINW, bool AKC, bool BKC, bool VEC, typename PT, typename AT = half_t>
__global__ void __launch_bounds__(WGM * WGN * 64, MINW)
gemm_f16_kernel(const GemmParams p, const PT tab)
{
    constexpr int NT = WGM * WGN * 64;
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int TI = WM / 32, TJ = WN / 32;
    constexpr int KS = BKT / 16;          /* MFMA k steps per slab */
    /* LDS, 64 banks (256 bytes a cycle). K-contiguous operand: rows of 64 bytes, no padding, four to a 256-byte line,
       the four 16-byte pieces of row r stored at piece ^ ((r >> 2) & 3): the sixteen lanes that write four rows
       cover a whole line, and so do the sixteen that read one piece of sixteen rows (the 80-byte pitch this replaces
       made the fourth row of a write wrap into the first: SQ_LDS_BANK_CONFLICT at a third of the LDS cycles).
       MN-contiguous operand: a transposing read takes 64 bytes from each of four k rows at a time, so the rows
       stand 64 bytes (mod 256) apart: BM + 32 halves (with + 16 two neighbouring rows shared 32 bytes of banks). */
    static_assert(BKT == 32, "the permutation of a K-contiguous row is laid out for rows of four 16-byte pieces");
    constexpr int LDK = BKT;
    constexpr int LDA = BM + 32;
    constexpr int LDB = BN + 32;
    constexpr int NA = BM * BKT / 8 / NT;
    constexpr int NB = BN * BKT / 8 / NT;
    constexpr int ASIZE = AKC ? BM * LDK : BKT * LDA;
    constexpr int BSIZE = BKC ? BN * LDK : BKT * LDB;
    constexpr int RING = 4;               /* slabs between global memory and LDS, in registers */
    constexpr int NMFMA = KS * TI * TJ;   /* MFMAs per slab */
    constexpr int PRE = NMFMA / 4;        /* MFMAs issued before the slab's barrier */
    constexpr int PREG = PRE > 0 ? PRE : 1;
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be made of 32x32 blocks");
    static_assert((BM * BKT / 8) % NT == 0 && (BN * BKT / 8) % NT == 0, "loads must divide evenly");
    static_assert(BKT % 16 == 0, "slab depth");

    __shared__ __attribute__((aligned(16))) half_t As[2][ASIZE];
    __shared__ __attribute__((aligned(16))) half_t Bs[2][BSIZE];

    const TileCoord tc = tile_of_workgroup(p);
    constexpr bool AF32 = std::is_same<AT, float>::value;
    constexpr int ASZ = (int)sizeof(AT);
    const AT * __restrict__ A;
    const half_t * __restrict__ B;
    OutT * __restrict__ C;
    if constexpr (sizeof(PT) > 1) {
        A = static_cast<const AT *>(tab.a[tc.batch]);
        B = static_cast<const half_t *>(tab.b[tc.batch]);
        C = static_cast<OutT *>(tab.c[tc.batch]);
    }
    else {
        A = static_cast<const AT *>(p.a) + batch_offset(tc.batch, p.batchInner, p.strideA, p.strideA1);
        B = static_cast<const half_t *>(p.b) + batch_offset(tc.batch, p.batchInner, p.strideB, p.strideB1);
        C = static_cast<OutT *>(p.c) + batch_offset(tc.batch, p.batchInner, p.strideC, p.strideC1);
    }

    /* K: the k range of this workgroup, all of p.K or one of p.splits pieces that begins at kBeg (p.kPerSplit is a
       multiple of the slab depth, so only the last piece has a ragged end, and that is where the operands end too) */
    const int kBeg = p.splits > 1 ? tc.split * p.kPerSplit : 0;
    const int M = p.M, N = p.N, K = p.splits > 1 && kBeg + p.kPerSplit < p.K ? p.kPerSplit : p.K - kBeg;
    const int m0 = tc.tm * BM, n0 = tc.tn * BN;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);      /* the same in every lane: said explicitly, so that descriptors built from it are scalars */
    const int wm0 = (wave / WGN) * WM, wn0 = (wave % WGN) * WN;
    const int l32 = lane & 31, lh = lane >> 5;

    /* ---- staging slots: which 8 halves of the slab each thread moves --------- */
    int aOff[NA], bOff[NB];        /* 16-byte path: byte offset from the slab base */
    int aLds[NA], bLds[NB];        /* half index in the LDS stage */
    int aK[NA], bK[NB];            /* k of the slot's first element inside the slab */
    int aMN[NA], bMN[NB];          /* row (K-contiguous) or first column (MN-contiguous) inside the tile */
#pragma unroll
    for (int s = 0; s < NA; s++) {
        int g = tid + s * NT;
        if (AKC) {
            int row = g / (BKT / 8);
            aK[s] = (g % (BKT / 8)) * 8;
            aMN[s] = row;
            aLds[s] = row * LDK + (((aK[s] >> 3) ^ ((row >> 2) & 3)) << 3);
            int r = m0 + row < M - 1 ? row : M - 1 - m0;
            aOff[s] = (r * p.lda + aK[s]) * ASZ;
        }
        else {
            aK[s] = g / (BM / 8);
            aMN[s] = (g % (BM / 8)) * 8;
            aLds[s] = aK[s] * LDA + aMN[s];
            /* columns past M are fetched from nowhere (zeros); a piece that straddles M runs on into the next
               row of k, into columns of the tile that are never stored */
            aOff[s] = m0 + aMN[s] < M ? (aK[s] * p.lda + aMN[s]) * ASZ : NTSAMD_OOB_OFFSET;
        }
    }
#pragma unroll
    for (int s = 0; s < NB; s++) {
        int g = tid + s * NT;
        if (BKC) {
            int row = g / (BKT / 8);
            bK[s] = (g % (BKT / 8)) * 8;
            bMN[s] = row;
            bLds[s] = row * LDK + (((bK[s] >> 3) ^ ((row >> 2) & 3)) << 3);
            int r = n0 + row < N - 1 ? row : N - 1 - n0;
            bOff[s] = (r * p.ldb + bK[s]) * 2;
        }
        else {
            bK[s] = g / (BN / 8);
            bMN[s] = (g % (BN / 8)) * 8;
            bLds[s] = bK[s] * LDB + bMN[s];
            bOff[s] = n0 + bMN[s] < N ? (bK[s] * p.ldb + bMN[s]) * 2 : NTSAMD_OOB_OFFSET;
        }
    }

    const AT * aTile = AKC ? A + (size_t)m0 * p.lda + kBeg : A + m0 + (size_t)kBeg * p.lda;
    const half_t * bTile = BKC ? B + (size_t)n0 * p.ldb + kBeg : B + n0 + (size_t)kBeg * p.ldb;
    const AT * aEnd = A + (size_t)((AKC ? M : p.K) - 1) * p.lda + (AKC ? p.K : M);
    const half_t * bEnd = B + (size_t)((BKC ? N : p.K) - 1) * p.ldb + (BKC ? p.K : N);

    /* a float a waits in the ring as it came (two registers of four floats per piece) and is rounded when it moves on to LDS */
    f16x8 ra[AF32 ? 1 : RING][AF32 ? 1 : NA], rb[RING][NB];
    f32x4 raF[AF32 ? RING : 1][AF32 ? NA : 1][2];

    auto load_global = [&](auto RINGC, auto TAIL, int k0) {
        constexpr int rg = decltype(RINGC)::value;
        constexpr bool mayHangOver = decltype(TAIL)::value != 0;
        if constexpr (VEC) {
            const AT * ab = AKC ? aTile + k0 : aTile + (size_t)k0 * p.lda;
            const half_t * bb = BKC ? bTile + k0 : bTile + (size_t)k0 * p.ldb;
            const long long aLeft = (long long)(aEnd - ab) * ASZ, bLeft = (long long)(bEnd - bb) * 2;
            const int aBytes = aLeft >> 31 ? 0x7fffffff : (int)aLeft, bBytes = bLeft >> 31 ? 0x7fffffff : (int)bLeft;
            __amdgpu_buffer_rsrc_t ar = make_rsrc(ab, aLeft);
            __amdgpu_buffer_rsrc_t br = make_rsrc(bb, bLeft);
            /* The one piece that can hang over the end of a buffer lies in the last slab (the last row of k of an
               MN-contiguous operand, the end of the last row of a K-contiguous one): only the loads of the last
               slabs (mayHangOver) look for it.
               Rows of k past the end of an MN-contiguous matrix read as zero by themselves;
               a K-contiguous row would run on into the next row, so those lanes are sent
               out of range explicitly, and the halves of a piece that straddles K are set to zero
               (last slab only) */
            const bool tail = mayHangOver && k0 + BKT > K;
#pragma unroll
            for (int s = 0; s < NA; s++) {
                int off = aOff[s];
                if (AKC && tail && k0 + aK[s] >= K)
                    off = NTSAMD_OOB_OFFSET;
                if constexpr (AF32) {
                    /* floats start on dwords, and a 16-byte buffer load is range-checked dword by dword: nothing
                       hangs over the end of the buffer half-way */
                    (void)aBytes;
                    raF[rg][s][0] = buffer_load_f32x4(ar, off);
                    raF[rg][s][1] = buffer_load_f32x4(ar, off == NTSAMD_OOB_OFFSET ? off : off + 16);
                    if constexpr (mayHangOver && AKC)
                        if (tail) {
#pragma unroll
                            for (int e = 1; e < 8; e++)
                                raF[rg][s][e / 4][e % 4] = k0 + aK[s] + e < K ? raF[rg][s][e / 4][e % 4] : 0.f;
                        }
                }
                else {
                    if constexpr (mayHangOver)
                        ra[rg][s] = buffer_load_f16x8_any(ar, off, aBytes);
                    else
                        ra[rg][s] = buffer_load_f16x8(ar, off);
                    if constexpr (mayHangOver && AKC)
                        if (tail) {
#pragma unroll
                            for (int e = 1; e < 8; e++)
                                ra[rg][s][e] = k0 + aK[s] + e < K ? ra[rg][s][e] : (half_t)0;
                        }
                }
            }
#pragma unroll
            for (int s = 0; s < NB; s++) {
                int off = bOff[s];
                if (BKC && tail && k0 + bK[s] >= K)
                    off = NTSAMD_OOB_OFFSET;
                if constexpr (mayHangOver)
                    rb[rg][s] = buffer_load_f16x8_any(br, off, bBytes);
                else
                    rb[rg][s] = buffer_load_f16x8(br, off);
                if constexpr (mayHangOver && BKC)
                    if (tail) {
#pragma unroll
                        for (int e = 1; e < 8; e++)
                            rb[rg][s][e] = k0 + bK[s] + e < K ? rb[rg][s][e] : (half_t)0;
                    }
            }
        }
        else {
            /* generic path: any alignment, element by element, predicated */
#pragma unroll
            for (int s = 0; s < NA; s++) {
                f16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
                f32x4 w[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
                if (AKC) {
                    int r = m0 + aMN[s] < M - 1 ? m0 + aMN[s] : M - 1;
                    const AT * rp = A + (size_t)r * p.lda;
#pragma unroll
                    for (int e = 0; e < 8; e++)
                        if (k0 + aK[s] + e < K) {
                            if constexpr (AF32) w[e / 4][e % 4] = rp[k0 + aK[s] + e];
                            else v[e] = rp[k0 + aK[s] + e];
                        }
                }
                else if (k0 + aK[s] < K) {
                    const AT * rp = A + (size_t)(k0 + aK[s]) * p.lda;
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        int c = m0 + aMN[s] + e < M - 1 ? m0 + aMN[s] + e : M - 1;
                        if constexpr (AF32) w[e / 4][e % 4] = rp[c];
                        else v[e] = rp[c];
                    }
                }
                if constexpr (AF32) {
                    raF[rg][s][0] = w[0];
                    raF[rg][s][1] = w[1];
                }
                else
                    ra[rg][s] = v;
            }
#pragma unroll
            for (int s = 0; s < NB; s++) {
                f16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
                if (BKC) {
                    int r = n0 + bMN[s] < N - 1 ? n0 + bMN[s] : N - 1;
                    const half_t * rp = B + (size_t)r * p.ldb;
#pragma unroll
                    for (int e = 0; e < 8; e++)
                        if (k0 + bK[s] + e < K)
                            v[e] = rp[k0 + bK[s] + e];
                }
                else if (k0 + bK[s] < K) {
                    const half_t * rp = B + (size_t)(k0 + bK[s]) * p.ldb;
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        int c = n0 + bMN[s] + e < N - 1 ? n0 + bMN[s] + e : N - 1;
                        v[e] = rp[c];
                    }
                }
                rb[rg][s] = v;
            }
        }
    };

    auto store_lds = [&](auto RINGC, int buf) {
        constexpr int rg = decltype(RINGC)::value;
#pragma unroll
        for (int s = 0; s < NA; s++) {
            if constexpr (AF32) {
                f16x8 v;
#pragma unroll
                for (int e = 0; e < 8; e++)
                    v[e] = (half_t)raF[rg][s][e / 4][e % 4];          /* v_cvt_f16_f32: to nearest even */
                *reinterpret_cast<f16x8 *>(&As[buf][aLds[s]]) = v;
            }
            else
                *reinterpret_cast<f16x8 *>(&As[buf][aLds[s]]) = ra[rg][s];
        }
#pragma unroll
        for (int s = 0; s < NB; s++)
            *reinterpret_cast<f16x8 *>(&Bs[buf][bLds[s]]) = rb[rg][s];
    };

    /* ---- fragments: two register sets, [set][k step][block] ------------------- */
    f16x8 fa[2][KS][TI], fb[2][KS][TJ];

    /* lane's place in a transposing read: which of the four k rows, which 4 columns */
    const int trRow = (lane & 15) >> 2;
    const int trCol = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

    auto read_frags = [&](auto SET, int buf) {
        constexpr int set = decltype(SET)::value;
        if constexpr (AKC) {
            const half_t * as = &As[buf][(wm0 + l32) * LDK];
#pragma unroll
            for (int kk = 0; kk < KS; kk++)
#pragma unroll
                for (int i = 0; i < TI; i++)
                    fa[set][kk][i] = *reinterpret_cast<const f16x8 *>(as + i * 32 * LDK + (((2 * kk + lh) ^ ((l32 >> 2) & 3)) << 3));
        }
        else {
            const half_t * as = &As[buf][(8 * lh + trRow) * LDA + wm0 + trCol];
#pragma unroll
            for (int kk = 0; kk < KS; kk++)
#pragma unroll
                for (int i = 0; i < TI; i++) {
                    f16x4 lo = lds_read_tr16(as + (kk * 16) * LDA + i * 32);
                    f16x4 hi = lds_read_tr16(as + (kk * 16 + 4) * LDA + i * 32);
                    fa[set][kk][i] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                }
        }
        if constexpr (BKC) {
            const half_t * bs = &Bs[buf][(wn0 + l32) * LDK];
#pragma unroll
            for (int kk = 0; kk < KS; kk++)
#pragma unroll
                for (int j = 0; j < TJ; j++)
                    fb[set][kk][j] = *reinterpret_cast<const f16x8 *>(bs + j * 32 * LDK + (((2 * kk + lh) ^ ((l32 >> 2) & 3)) << 3));
        }
        else {
            const half_t * bs = &Bs[buf][(8 * lh + trRow) * LDB + wn0 + trCol];
#pragma unroll
            for (int kk = 0; kk < KS; kk++)
#pragma unroll
                for (int j = 0; j < TJ; j++) {
                    f16x4 lo = lds_read_tr16(bs + (kk * 16) * LDB + j * 32);
                    f16x4 hi = lds_read_tr16(bs + (kk * 16 + 4) * LDB + j * 32);
                    fb[set][kk][j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                }
        }
    };

    f32x16 acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; i++)
#pragma unroll
        for (int j = 0; j < TJ; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                acc[i][j][r] = 0.f;

    /* MFMAs number first .. last-1 of the slab, in (k step, i, j) order */
    auto mfma_range = [&](auto SET, int first, int last) {
        constexpr int set = decltype(SET)::value;
#pragma unroll
        for (int t = first; t < last; t++) {
            const int kk = t / (TI * TJ), i = (t / TJ) % TI, j = t % TJ;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[set][kk][i], fb[set][kk][j], acc[i][j], 0, 0, 0);
        }
    };

    const int nk = (K + BKT - 1) / BKT;

    /* One slab, number kt = SLOT mod RING: its fragments are in register set SLOT % 2 and came from LDS stage
       SLOT % 2. FULL: slabs kt+1 .. kt+RING exist, are complete and are followed by another, so the slab is
       straight-line code with plain loads. */
    auto slab = [&](auto SLOT, auto FULL, int kt) {
        constexpr int slot = decltype(SLOT)::value;
        constexpr int set = slot & 1;
        typedef IntC<set> SET_T;
        const SET_T SET = SET_T();
        constexpr bool full = decltype(FULL)::value != 0;
        if (full || kt + 1 < nk)
            store_lds(IntC<(slot + 1) % RING>(), set ^ 1);     /* slab kt+1, requested during slab kt+1-RING */
        mfma_range(SET, 0, PRE);
        if constexpr (full) {
#pragma unroll
            for (int g = 0; g < PRE; g++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);     /* one MFMA */
                __builtin_amdgcn_sched_group_barrier(0x200, (NA + NB + PREG - 1) / PREG, 0);   /* LDS writes */
                __builtin_amdgcn_sched_group_barrier(0x006, 2, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();                         /* stage set^1 complete; stage set no longer read by anyone */
        __builtin_amdgcn_sched_barrier(0);
        /* slab kt+RING into the registers that slab kt left for LDS one slab ago */
        if (full)
            load_global(IntC<slot>(), IntC<0>(), (kt + RING) * BKT);
        else if (kt + RING < nk)
            load_global(IntC<slot>(), IntC<1>(), (kt + RING) * BKT);
        if (full || kt + 1 < nk)
            read_frags(IntC<set ^ 1>(), set ^ 1);
        mfma_range(SET, PRE, NMFMA);
        if constexpr (full) {
            constexpr int REST = NMFMA - PRE;
            constexpr int NREAD = (AKC ? 1 : 2) * KS * TI + (BKC ? 1 : 2) * KS * TJ;
#pragma unroll
            for (int g = 0; g < REST; g++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);     /* one MFMA */
                __builtin_amdgcn_sched_group_barrier(0x100, (NREAD + REST - 1) / REST, 0);   /* LDS reads */
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);                            /* one global read */
                __builtin_amdgcn_sched_group_barrier(0x006, 3, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    static_assert(RING >= 2 && RING % 2 == 0, "the ring and the two LDS stages turn together");
    if (nk > 0) {
        /* slabs 0 .. RING-1 requested, slab 0 on to LDS (slab 0's turn then asks for slab RING) */
        auto first = [&](auto self, auto SLOT) {
            constexpr int slot = decltype(SLOT)::value;
            if constexpr (slot < RING) {
                if (slot < nk) {
                    load_global(SLOT, IntC<1>(), slot * BKT);
                    self(self, IntC<slot + 1>());
                }
            }
        };
        first(first, IntC<0>());
        store_lds(IntC<0>(), 0);
        __syncthreads();
        read_frags(IntC<0>(), 0);
        const int nkFull = K / BKT;
        /* RING slabs per turn, so that registers and stages have fixed names; kt stays a multiple of RING */
        auto turn = [&](auto self, auto SLOT, auto FULL, int kt) {
            constexpr int slot = decltype(SLOT)::value;
            constexpr bool full = decltype(FULL)::value != 0;
            if constexpr (slot < RING) {
                if (full || kt + slot < nk) {
                    slab(SLOT, FULL, kt + slot);
                    self(self, IntC<slot + 1>(), FULL, kt);
                }
            }
        };
        int kt = 0;
        /* straight-line turns: every slab they ask for is complete and is not the last one */
        for (; kt + 2 * RING < nkFull; kt += RING)
            turn(turn, IntC<0>(), IntC<1>(), kt);
        for (; kt < nk; kt += RING)
            turn(turn, IntC<0>(), IntC<0>(), kt);
    }

    /* ---- epilogue: accumulator register r of lane l is element
       (8*(r/4) + 4*(l/32) + r%4, l%32) of its 32x32 block ------------------------ */
    if (p.splits > 1) {
        /* one of several workgroups that share this tile: the partial tile goes to the workspace as it is (splits x
           batch dense M x N fp32 matrices), and split_reduce.hip adds the pieces in their order and applies alpha,
           beta, bias and activation */
        float * w = p.splitWork + ((size_t)tc.split * p.batch + tc.batch) * M * N;
#pragma unroll
        for (int j = 0; j < TJ; j++) {
            const int col = n0 + wn0 + j * 32 + l32;
            if (col < N) {
#pragma unroll
                for (int i = 0; i < TI; i++)
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int row = m0 + wm0 + i * 32 + 8 * (r / 4) + 4 * lh + (r % 4);
                        if (row < M)
                            w[(size_t)row * N + col] = acc[i][j][r];
                    }
            }
        }
        return;
    }
    const float alpha = p.alpha, beta = p.beta;
    const OutT * __restrict__ bias = static_cast<const OutT *>(p.bias);
    const int biasMode = p.biasMode;

    if constexpr (VEC) {
        /* the wave's rows of c as one buffer that ends where c ends: rows past M drop off
           its end, columns past N are sent out of range. Row-indexed bias is not handled here. */
        if (m0 + wm0 >= M)
            return;
        OutT * cw = C + (size_t)(m0 + wm0) * p.ldc;
        __amdgpu_buffer_rsrc_t cr = make_rsrc(cw, (long long)(M - m0 - wm0) * p.ldc * (long long)sizeof(OutT));
        const unsigned rowPitch = (unsigned)p.ldc * (unsigned)sizeof(OutT);
#pragma unroll
        for (int j = 0; j < TJ; j++) {
            const int col = n0 + wn0 + j * 32 + l32;
            const unsigned cOff = col < N ? (unsigned)(4 * lh * p.ldc + col) * (unsigned)sizeof(OutT)
                                          : (unsigned)NTSAMD_OOB_OFFSET;
            float bcol = 0.f;
            if (biasMode == BIAS_COL && col < N)
                bcol = (float)bias[col];
#pragma unroll
            for (int i = 0; i < TI; i++) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const unsigned off = cOff + (unsigned)(i * 32 + 8 * (r / 4) + (r % 4)) * rowPitch;
                    float v = alpha * acc[i][j][r] + bcol;
                    if (beta != 0.f)
                        v += beta * buffer_load_out<OutT>(cr, (int)off);
                    buffer_store_out<OutT>((OutT)activate(v, p.act), cr, (int)off);
                }
            }
        }
    }
    else {
        /* generic path: plain pointers, per-element bounds, every bias mode */
#pragma unroll
        for (int j = 0; j < TJ; j++) {
            const int col = n0 + wn0 + j * 32 + l32;
            if (col >= N)
                continue;
            float bcol = 0.f;
            if (biasMode == BIAS_COL)
                bcol = (float)bias[col];
#pragma unroll
            for (int i = 0; i < TI; i++) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int row = m0 + wm0 + i * 32 + 8 * (r / 4) + 4 * lh + (r % 4);
                    if (row < M) {
                        OutT * cp = C + (size_t)row * p.ldc + col;
                        float v = alpha * acc[i][j][r];
                        if (beta != 0.f)
                            v += beta * (float)(*cp);
                        if (biasMode == BIAS_ROW)
                            v += (float)bias[(row / p.biasRowDiv) % p.biasLen];
                        else
                            v += bcol;
                        *cp = (OutT)activate(v, p.act);
                    }
                }
            }
        }
    }
}

template <typename OutT, int CFG, bool AKC, bool BKC, bool VEC, typename PT, typename AT = half_t>
static int launch_f16_one(const GemmParams & p0, const PT & tab, hipStream_t stream)
{
    typedef TileShape<CFG> S;
    GemmParams p = p0;
    p.tilesM = (p.M + S::BM - 1) / S::BM;
    p.tilesN = (p.N + S::BN - 1) / S::BN;
    /* pieces of k meet in a workspace (the 16-byte fetch, no lists of matrices) or there are none */
    if (!(VEC && sizeof(PT) == 1 && p.splits > 1 && p.splitWork != NULL))
        p.splits = 1;
    dim3 grid((unsigned)(p.tilesM * p.tilesN * p.batch * p.splits));
    hipLaunchKernelGGL((gemm_f16_kernel<OutT, S::BM, S::BN, 32, S::WGM, S::WGN, S::MINW16, AKC, BKC, VEC, PT, AT>),
                       grid, dim3(S::WGM * S::WGN * 64), 0, stream, p, tab);
    return (int)hipGetLastError();
}

}  // namespace ntsamd
