/*
 * fp16 GEMM for gfx950, main path: global memory -> LDS without passing through
 * registers (buffer_load_dwordx4 ... lds), four LDS stages, fp32 accumulation.
 * Used for 16-byte aligned operands with a half result; everything else goes
 * through the register-staged kernel in gemm_f16.h. Same arithmetic, same
 * fragment layouts (see that file for what v_mfma_f32_32x32x16_f16 and
 * ds_read_b64_tr_b16 expect).
 *
 * An LDS-direct load writes the 64 lanes' 16 bytes to 1 KB of consecutive LDS, at
 * an address the whole wave shares; WHICH 16 bytes of global memory a lane fetches
 * is free. That freedom is what keeps the fragment reads free of bank conflicts
 * without padding inside a chunk. The LDS of this part serves 256 bytes a cycle from
 * 64 banks of 4 bytes (measured: layouts that are conflict-free on 32 banks showed
 * SQ_LDS_BANK_CONFLICT at 46 % of SQ_LDS_IDX_ACTIVE, these show 3 %): 16 lanes of a
 * 16-byte read, or 32 lanes of an 8-byte read, go together and must cover 256
 * different bytes modulo 256.
 *   K-contiguous operand (rows of mn, 32 halves = 64 bytes of k per row): a chunk
 *       is 16 rows. The four 16-byte columns of row r are stored permuted,
 *       column c at position c ^ ((r >> 2) & 3): rows r, r+4, r+8, r+12 share their
 *       64 bytes of a 256-byte line, and sixteen consecutive rows reading the same
 *       logical column hit sixteen different 16-byte bank groups.
 *       With slabs of 64 along k (BKT_ = 64, the 64 x 64 tile only) a row is a whole
 *       128-byte line, a chunk is 8 rows, and column c of row r sits at position
 *       c ^ ((r >> 1) & 7): rows of equal parity share their half of a 256-byte line.
 *   MN-contiguous operand (rows of k): a chunk holds rows k, k + NCH, k + 2 NCH ...
 *       (NCH chunks per slab), and chunks are 1 KB + 64 bytes apart, so the four
 *       consecutive k rows of one transposing read sit in four different chunks,
 *       64 bytes apart modulo 256: the 32 bytes a row gives to lanes 0-15 and the
 *       next 32 bytes it gives to lanes 16-31 fill the line.
 *
 * Pipeline: loads for slab t+4 are issued during the second k step of slab t, the
 * moment the stage of slab t is free (about 3 slabs = 3000 cycles of cover for the
 * global latency). A slab is two MFMA k steps; its fragments are double-buffered
 * per k step. The one barrier of a slab sits between the two steps: by then the
 * wave has waited for its own loads of slab t+1 (vmcnt) and for its own last reads
 * of slab t (lgkmcnt), so after the barrier every wave may read slab t+1 and
 * overwrite the stage of slab t, and the MFMAs of the second step are ready to
 * issue the moment the barrier opens, because their fragments were read before it.
 */
#pragma once
#include "gemm_common.h"
#include "gemm_f16.h"
#include <type_traits>

namespace ntsamd {

/* s_waitcnt with only the vector-memory counter set (gfx9 encoding: vmcnt in bits 3:0 and 15:14) */
template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt range");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

__device__ __forceinline__ void wait_lgkmcnt0()
{
    __builtin_amdgcn_s_waitcnt(0xC07F);     /* lgkmcnt = 0, vmcnt and expcnt left at their maxima */
}

/* A raw buffer descriptor as four scalars (base low, base high, bytes, format word), for
   the loads below that the compiler must not see as memory operations of its own. */
typedef int i32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ i32x4 make_desc(const void * base, long long bytes)
{
    const unsigned long long b = reinterpret_cast<unsigned long long>(base);
    i32x4 d;
    d[0] = (int)(unsigned)b;
    d[1] = (int)((b >> 32) & 0xffffu);
    d[2] = (unsigned long long)bytes >> 31 ? 0x7fffffff : (int)bytes;
    d[3] = 0x00020000;
    return d;
}

/* Global memory -> LDS, 16 bytes per lane: lane l's data lands at ldsAddr + 16 l (ldsAddr is the
   same for the whole wave and travels in M0). Written as inline assembly on purpose: as a
   compiler builtin, every later LDS read is made to wait for ALL outstanding loads (the compiler
   cannot tell which LDS bytes a load in flight will write), which would serialise the
   pipeline. The waits are placed by hand instead (wait_vmcnt below). */
__device__ __forceinline__ void lds_dma16(i32x4 desc, unsigned ldsAddr, int byteOffset)
{
    asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :
                 : "s"(ldsAddr), "v"(byteOffset), "s"(desc)
                 : "memory");
}

/* SPLIT: the k range is cut into p.splits pieces, one workgroup each, and every workgroup leaves its partial tile
   as plain fp32 (no alpha, beta, bias or activation) in p.splitWork, which holds p.splits x p.batch dense M x N
   matrices; split_reduce.hip adds the pieces up and does what the epilogue would have done. */
template <typename OutT, int BM, int BN, int WGM, int WGN, int MINW, bool AKC, bool BKC, bool CS, bool SPLIT = false, int NSTAGE = 4,
          bool PP = false, int BKT_ = 32>
__global__ void __launch_bounds__(WGM * WGN * 64, MINW)
gemm_f16_direct_kernel(const GemmParams p)
{
    static_assert(!CS || std::is_same<OutT, half_t>::value, "column sums have the type of b and of c");
    static_assert(!(CS && SPLIT), "column sums are not gathered from pieces of k");
    static_assert(!SPLIT || std::is_same<OutT, float>::value, "partial tiles are fp32");
    constexpr int BKT = BKT_, KS = BKT / 16;               /* slab depth, MFMA k steps per slab */
    constexpr int NW = WGM * WGN;
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int TI = WM / 32, TJ = WN / 32;
    static_assert(BKT == 32 || (BKT == 64 && TI == 1 && TJ == 1 && !PP), "slabs of 64: the one-block wave tile only");
    /* per-operand LDS geometry, bytes */
    constexpr int ROWB = BKT * 2;                          /* a K-contiguous row of a slab */
    constexpr int LPRK = BKT / 8;                          /* lanes per such row */
    constexpr int A_RPC = AKC ? 1024 / ROWB : 512 / BM;    /* rows per chunk */
    constexpr int B_RPC = BKC ? 1024 / ROWB : 512 / BN;
    constexpr int A_NCH = AKC ? BM / A_RPC : BKT / A_RPC;  /* chunks per slab */
    constexpr int B_NCH = BKC ? BN / B_RPC : BKT / B_RPC;
    constexpr int A_CP = AKC ? 1024 : 1088;                /* chunk pitch */
    constexpr int B_CP = BKC ? 1024 : 1088;
    constexpr int A_BYTES = A_NCH * A_CP;
    constexpr int B_BYTES = B_NCH * B_CP;
    constexpr int STAGE = A_BYTES + B_BYTES;
    constexpr int NLA = A_NCH / NW, NLB = B_NCH / NW;      /* load instructions per wave and slab */
    constexpr int NL = NLA + NLB;
    static_assert(A_NCH % NW == 0 && B_NCH % NW == 0, "chunks must divide among the waves");
    static_assert(AKC || A_NCH >= 4, "transposing reads need four chunks");
    static_assert(BKC || B_NCH >= 4, "transposing reads need four chunks");

    __shared__ __attribute__((aligned(1024))) char lds[NSTAGE * STAGE];

    const TileCoord tc = tile_of_workgroup(p);
    const half_t * __restrict__ A = static_cast<const half_t *>(p.a) + batch_offset(tc.batch, p.batchInner, p.strideA, p.strideA1);
    const half_t * __restrict__ B = static_cast<const half_t *>(p.b) + batch_offset(tc.batch, p.batchInner, p.strideB, p.strideB1);
    OutT * __restrict__ C;
    if constexpr (SPLIT)
        C = reinterpret_cast<OutT *>(p.splitWork) + ((size_t)tc.split * p.batch + tc.batch) * p.M * p.N;
    else
        C = static_cast<OutT *>(p.c) + batch_offset(tc.batch, p.batchInner, p.strideC, p.strideC1);

    /* K: the k range of this workgroup, which starts at kBeg (p.kPerSplit is a multiple of the slab depth, so only
       the last piece has a ragged end, and that is where the operands end too) */
    const int kBeg = SPLIT ? tc.split * p.kPerSplit : 0;
    const int M = p.M, N = p.N, K = SPLIT && kBeg + p.kPerSplit < p.K ? p.kPerSplit : p.K - kBeg;
    const int m0 = tc.tm * BM, n0 = tc.tn * BN;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave / WGN) * WM, wn0 = (wave % WGN) * WN;
    const int l32 = lane & 31, lh = lane >> 5;

    /* ---- what each lane fetches for each of its wave's chunks -------------------- */
    int aOff[NLA], bOff[NLB];      /* byte offset from the slab base */
    int aKc[NLA], bKc[NLB];        /* K-contiguous: first k of the lane's 16 bytes inside the slab */
#pragma unroll
    for (int q = 0; q < NLA; q++) {
        const int ch = wave * NLA + q;
        if (AKC) {
            int row = ch * A_RPC + lane / LPRK;
            int col = (lane % LPRK) ^ (BKT == 32 ? (row >> 2) & 3 : (row >> 1) & 7);
            aKc[q] = col * 8;
            int r = m0 + row < M - 1 ? row : M - 1 - m0;
            aOff[q] = (r * p.lda + col * 8) * 2;
        }
        else {
            constexpr int LPR = 64 / A_RPC;                  /* lanes per row */
            int krow = ch + A_NCH * (lane / LPR);
            int c = (lane % LPR) * 8;
            c = m0 + c < p.mOper - 8 ? c : p.mOper - 8 - m0;
            aKc[q] = 0;
            aOff[q] = (krow * p.lda + c) * 2;
        }
    }
#pragma unroll
    for (int q = 0; q < NLB; q++) {
        const int ch = wave * NLB + q;
        if (BKC) {
            int row = ch * B_RPC + lane / LPRK;
            int col = (lane % LPRK) ^ (BKT == 32 ? (row >> 2) & 3 : (row >> 1) & 7);
            bKc[q] = col * 8;
            int r = n0 + row < N - 1 ? row : N - 1 - n0;
            bOff[q] = (r * p.ldb + col * 8) * 2;
        }
        else {
            constexpr int LPR = 64 / B_RPC;
            int krow = ch + B_NCH * (lane / LPR);
            int c = (lane % LPR) * 8;
            c = n0 + c < p.nOper - 8 ? c : p.nOper - 8 - n0;
            bKc[q] = 0;
            bOff[q] = (krow * p.ldb + c) * 2;
        }
    }

    const half_t * aTile = AKC ? A + (size_t)m0 * p.lda + kBeg : A + m0 + (size_t)kBeg * p.lda;
    const half_t * bTile = BKC ? B + (size_t)n0 * p.ldb + kBeg : B + n0 + (size_t)kBeg * p.ldb;
    const half_t * aEnd = A + (size_t)((AKC ? M : p.K) - 1) * p.lda + p.mOper;
    const half_t * bEnd = B + (size_t)((BKC ? N : p.K) - 1) * p.ldb + p.nOper;

    const unsigned ldsBase = (unsigned)(size_t)((__attribute__((address_space(3))) char *)lds);

    /* issue load number q (0 .. NL-1) of this wave for slab kt */
    auto issue_load = [&](auto TAIL, int kt, int q) {
        constexpr bool mayHangOver = decltype(TAIL)::value != 0;
        const int k0 = kt * BKT;
        const unsigned stage = ldsBase + (unsigned)((kt % NSTAGE) * STAGE);
        const bool tail = mayHangOver && k0 + BKT > K;
        if (q < NLA) {
            const half_t * ab = AKC ? aTile + k0 : aTile + (size_t)k0 * p.lda;
            int off = aOff[q];
            if (AKC && tail && k0 + aKc[q] >= K)
                off = NTSAMD_OOB_OFFSET;
            lds_dma16(make_desc(ab, (long long)(aEnd - ab) * 2), stage + (unsigned)((wave * NLA + q) * A_CP), off);
        }
        else {
            const half_t * bb = BKC ? bTile + k0 : bTile + (size_t)k0 * p.ldb;
            int off = bOff[q - NLA];
            if (BKC && tail && k0 + bKc[q - NLA] >= K)
                off = NTSAMD_OOB_OFFSET;
            lds_dma16(make_desc(bb, (long long)(bEnd - bb) * 2), stage + (unsigned)(A_BYTES + (wave * NLB + (q - NLA)) * B_CP), off);
        }
    };

    auto issue_loads = [&](auto TAIL, int kt) {
#pragma unroll
        for (int q = 0; q < NL; q++)
            issue_load(TAIL, kt, q);
    };

    /* ---- fragment addresses (byte offsets inside a stage) ---------------------------- */
    const int trRow = (lane & 15) >> 2;
    const int trCol = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    int aFrag[KS], bFrag[KS];      /* K-contiguous: offset for k step kk, block 0 */
    int aTr[KS][2], bTr[KS][2];    /* MN-contiguous: offset for k step kk, half h, block 0 */
#pragma unroll
    for (int kk = 0; kk < KS; kk++) {
        const int sw = BKT == 32 ? (l32 >> 2) & 3 : (l32 >> 1) & 7;
        aFrag[kk] = (wm0 + l32) * ROWB + ((kk * 2 + lh) ^ sw) * 16;
        bFrag[kk] = A_BYTES + (wn0 + l32) * ROWB + ((kk * 2 + lh) ^ sw) * 16;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int kr = 16 * kk + 8 * lh + 4 * h + trRow;
            aTr[kk][h] = (kr % A_NCH) * A_CP + (kr / A_NCH) * (BM * 2) + (wm0 + trCol) * 2;
            bTr[kk][h] = A_BYTES + (kr % B_NCH) * B_CP + (kr / B_NCH) * (BN * 2) + (wn0 + trCol) * 2;
        }
    }

    f16x8 fa[2][TI], fb[2][TJ];

    /* fragment number f (a blocks first, then b blocks) of k step KK of the slab in `stage` */
    auto read_frag = [&](auto KKC, const char * stage, int f) {
        constexpr int kk = decltype(KKC)::value;
        if (f < TI) {
            const int i = f;
            if constexpr (AKC)
                fa[kk][i] = *reinterpret_cast<const f16x8 *>(stage + aFrag[kk] + i * 32 * ROWB);
            else {
                f16x4 lo = lds_read_tr16(reinterpret_cast<const half_t *>(stage + aTr[kk][0] + i * 64));
                f16x4 hi = lds_read_tr16(reinterpret_cast<const half_t *>(stage + aTr[kk][1] + i * 64));
                fa[kk][i] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
        }
        else {
            const int j = f - TI;
            if constexpr (BKC)
                fb[kk][j] = *reinterpret_cast<const f16x8 *>(stage + bFrag[kk] + j * 32 * ROWB);
            else {
                f16x4 lo = lds_read_tr16(reinterpret_cast<const half_t *>(stage + bTr[kk][0] + j * 64));
                f16x4 hi = lds_read_tr16(reinterpret_cast<const half_t *>(stage + bTr[kk][1] + j * 64));
                fb[kk][j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
        }
    };

    auto read_frags = [&](auto KKC, const char * stage) {
#pragma unroll
        for (int f = 0; f < TI + TJ; f++)
            read_frag(KKC, stage, f);
    };

    f32x16 acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; i++)
#pragma unroll
        for (int j = 0; j < TJ; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                acc[i][j][r] = 0.f;

    /* CS: column sums of op(b), gathered from the b fragments on their way to the MFMAs
       (v_dot2_f32_f16 against ones: exact products, fp32 sums). Lane (l32, lh) sees, for each
       of its columns, the k values its half of the wave feeds in; the halves meet at the end. */
    float colSum[CS ? TJ : 1];
#pragma unroll
    for (int j = 0; j < (CS ? TJ : 1); j++)
        colSum[j] = 0.f;

    constexpr int NM = TI * TJ;                                       /* MFMAs per k step */
    constexpr int NF = TI + TJ;                                       /* fragments per k step */
    constexpr int RPF = (AKC ? 1 : 2);                                /* LDS reads per a fragment */

    const int nk = (K + BKT - 1) / BKT;

    /* One k step: its NM MFMAs, with the reads of the OTHER register set (from `src`, if
       READ) and this wave's loads of slab `loadKt` (if LOAD) dealt out between them, in
       program order AND pinned there: an MFMA holds the matrix pipe for 32 cycles but
       takes one issue slot, so the other instructions ride in its shadow. */
    auto k_step = [&](auto KKC, auto READC, auto LOADC, auto TAILC, const char * src, int loadKt) {
        constexpr int kk = decltype(KKC)::value;
        constexpr bool doRead = decltype(READC)::value != 0;
        constexpr bool doLoad = decltype(LOADC)::value != 0;
#pragma unroll
        for (int g = 0; g < NM; g++) {
            const int i = g / TJ, j = g % TJ;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[kk][i], fb[kk][j], acc[i][j], 0, 0, 0);
            if constexpr (CS) {
                if (i == 0) {
                    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
                    const h2 ones = {(_Float16)1, (_Float16)1};
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const h2 pr = {fb[kk][j][2 * e], fb[kk][j][2 * e + 1]};
                        colSum[j] = __builtin_amdgcn_fdot2(pr, ones, colSum[j], false);
                    }
                }
            }
            if (doRead) {
                /* fragments f with f * NM / NF == g: spread evenly over the MFMAs */
#pragma unroll
                for (int f = 0; f < NF; f++)
                    if (f * NM / NF == g)
                        read_frag(IntC<kk ^ 1>(), src, f);
            }
            if (doLoad) {
#pragma unroll
                for (int q = 0; q < NL; q++)
                    if (q * NM / NL == g)
                        issue_load(TAILC, loadKt, q);
            }
        }
    };

    /* One slab. AHEAD = how many later slabs exist (capped at 4): decides which loads are
       issued and how many may still be in flight at the barrier. */
    auto slab = [&](auto AHEADC, auto TAILC, int kt) {
        constexpr int ahead = decltype(AHEADC)::value;
        const char * stage = lds + (kt % NSTAGE) * STAGE;
        const char * next = lds + ((kt + 1) % NSTAGE) * STAGE;

        /* k step 0: multiply it, fetch step 1 of this slab */
        k_step(IntC<0>(), IntC<1>(), IntC<0>(), TAILC, stage, 0);
        __builtin_amdgcn_sched_barrier(0);

        /* slab kt+1 must have landed: at most the loads of slabs kt+2 and kt+3 stay in flight */
        if constexpr (ahead >= 3)
            wait_vmcnt<2 * NL>();
        else if constexpr (ahead == 2)
            wait_vmcnt<NL>();
        else
            wait_vmcnt<0>();
        wait_lgkmcnt0();
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);

        /* k step 1: multiply it, fetch step 0 of the next slab. Every wave has read the last fragment of
           this slab's stage before the barrier (its second step's fragments were fetched during the first),
           so the stage is free from here on: the loads of slab kt+4 go into it now, half a slab earlier
           than if they waited for the next slab to begin */
        k_step(IntC<1>(), IntC<(ahead >= 1)>(), IntC<(ahead >= 4)>(), TAILC, next, kt + 4);
        __builtin_amdgcn_sched_barrier(0);
    };

    /* A wave with one accumulator block (the 64 x 64 tile) has one MFMA per k step to wait behind, and an LDS
       read takes four times as long to come back: with its fragments requested one k step ahead, as below, such a
       wave spends its time waiting for them (0.16 us per slab for a workgroup alone on its CU). It asks for the
       fragments of a whole slab at once instead, one slab ahead, into a second set of registers (0.14 us per slab).
       The loop is written for any number of stages; eight instead of four gain nothing (measured: a lone
       workgroup is not waiting for memory either), and four leave room for four workgroups on a CU. */
    constexpr bool DEEP = TI == 1 && TJ == 1;
    if constexpr (DEEP) {
        f16x8 da[2][KS], db[2][KS];                  /* [set][k step] */
        f32x16 accOdd;
#pragma unroll
        for (int r = 0; r < 16; r++)
            accOdd[r] = 0.f;
        auto read_set = [&](auto SETC, const char * stage) {
            constexpr int S = decltype(SETC)::value;
#pragma unroll
            for (int kk = 0; kk < KS; kk++) {
                if constexpr (AKC)
                    da[S][kk] = *reinterpret_cast<const f16x8 *>(stage + aFrag[kk]);
                else {
                    f16x4 lo = lds_read_tr16(reinterpret_cast<const half_t *>(stage + aTr[kk][0]));
                    f16x4 hi = lds_read_tr16(reinterpret_cast<const half_t *>(stage + aTr[kk][1]));
                    da[S][kk] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                }
                if constexpr (BKC)
                    db[S][kk] = *reinterpret_cast<const f16x8 *>(stage + bFrag[kk]);
                else {
                    f16x4 lo = lds_read_tr16(reinterpret_cast<const half_t *>(stage + bTr[kk][0]));
                    f16x4 hi = lds_read_tr16(reinterpret_cast<const half_t *>(stage + bTr[kk][1]));
                    db[S][kk] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                }
            }
        };
        /* Slab kt, whose fragments are in set S. AHEAD = how many later slabs exist (capped at NSTAGE). */
        auto deep_slab = [&](auto SETC, auto AHEADC, auto TAILC, int kt) {
            constexpr int S = decltype(SETC)::value;
            constexpr int ahead = decltype(AHEADC)::value;
            if constexpr (ahead >= 1) {
                /* slab kt+1 must have landed: at most the loads of slabs kt+2 .. kt+NSTAGE-1 stay in flight. Every
                   wave's reads of this slab's stage have come back by the barrier (they are what the MFMAs below
                   wait for anyway), so the stage is free after it. */
                wait_vmcnt<((ahead < NSTAGE - 1 ? ahead : NSTAGE - 1) - 1) * NL>();
                wait_lgkmcnt0();
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_sched_barrier(0);
                read_set(IntC<S ^ 1>(), lds + ((kt + 1) % NSTAGE) * STAGE);
                if constexpr (ahead >= NSTAGE)
                    issue_loads(TAILC, kt + NSTAGE);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int kk = 0; kk < KS; kk++) {
                /* slabs of four k steps: odd steps add into a second accumulator, so that no MFMA waits for the
                   one before it (a lone wave on its SIMD has nobody to fill that wait) */
                if (KS == 4 && (kk & 1))
                    accOdd = __builtin_amdgcn_mfma_f32_32x32x16_f16(da[S][kk], db[S][kk], accOdd, 0, 0, 0);
                else
                    acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(da[S][kk], db[S][kk], acc[0][0], 0, 0, 0);
                if constexpr (CS) {
                    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
                    const h2 ones = {(_Float16)1, (_Float16)1};
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const h2 pr = {db[S][kk][2 * e], db[S][kk][2 * e + 1]};
                        colSum[0] = __builtin_amdgcn_fdot2(pr, ones, colSum[0], false);
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        };
        static_assert((NSTAGE - 1) * NL < 64, "the wait counter has six bits");
        if (nk > 0) {
            /* prologue: every stage in flight, then wait for the first */
            auto issue_first = [&](auto self, auto NC) {
                constexpr int n = decltype(NC)::value;
                if constexpr (n < NSTAGE) {
                    if (nk > n) {
                        issue_loads(IntC<1>(), n);
                        self(self, IntC<n + 1>());
                    }
                }
            };
            issue_first(issue_first, IntC<0>());
            auto wait_first = [&](auto self, auto NC) {
                constexpr int n = decltype(NC)::value;          /* slabs in flight besides the first */
                if (nk > n)
                    wait_vmcnt<n * NL>();
                else if constexpr (n > 0)
                    self(self, IntC<n - 1>());
            };
            wait_first(wait_first, IntC<NSTAGE - 1>());
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
            read_set(IntC<0>(), lds);

            /* two slabs per turn, so that the register sets have fixed names; kt stays even */
            const int nkFull = K / BKT;
            int kt = 0;
            for (; kt + NSTAGE + 1 < nkFull; kt += 2) {  /* the slabs to fetch are complete: no tail handling */
                deep_slab(IntC<0>(), IntC<NSTAGE>(), IntC<0>(), kt);
                deep_slab(IntC<1>(), IntC<NSTAGE>(), IntC<0>(), kt + 1);
            }
            for (; kt + NSTAGE + 1 < nk; kt += 2) {
                deep_slab(IntC<0>(), IntC<NSTAGE>(), IntC<1>(), kt);
                deep_slab(IntC<1>(), IntC<NSTAGE>(), IntC<1>(), kt + 1);
            }
            /* one to NSTAGE + 1 slabs are left, the first of them in set 0: the one with R slabs to go (itself
               included) is in set (left - R) & 1 */
            const int left = nk - kt;
            auto rest = [&](auto self, auto RC, auto PARC) {
                constexpr int R = decltype(RC)::value, P = decltype(PARC)::value;
                if constexpr (R >= 1) {
                    if (nk - kt == R) {
                        deep_slab(IntC<((P + R) & 1)>(), IntC<(R - 1 < NSTAGE ? R - 1 : NSTAGE)>(), IntC<1>(), kt);
                        kt++;
                    }
                    self(self, IntC<R - 1>(), PARC);
                }
            };
            if (left & 1)
                rest(rest, IntC<NSTAGE + 1>(), IntC<1>());
            else
                rest(rest, IntC<NSTAGE + 1>(), IntC<0>());
        }
        if constexpr (KS == 4) {
#pragma unroll
            for (int r = 0; r < 16; r++)
                acc[0][0][r] += accOdd[r];
        }
    }
    else if constexpr (PP) {
        /* Ping-pong: the eight waves form two groups, waves 0-3 and waves 4-7, one wave of each on every SIMD.
           A slab is two phases for a wave: a MEMORY phase (this wave's loads of the slab three ahead go out, all
           the fragments of the slab come in from LDS) and a COMPUTE phase (the slab's 2 x NM MFMAs back to back,
           at raised priority), each closed by a workgroup barrier. The second group runs one phase behind the
           first (it passes one barrier more before it starts and the first one more at the end), so on every
           SIMD one wave is in its compute phase while the other is in its memory phase: the matrix pipe sees one
           unbroken run of MFMAs from alternating waves, and the LDS latency, the waits and the barriers of one
           wave lie under the MFMAs of the other, instead of both waves of a SIMD meeting the same barrier at
           the same time. Number the barriers b = 0, 1, 2 ... after the one that ends the prologue. The first
           group reads slab t between barriers 2t-1 and 2t, the second between 2t and 2t+1. Every wave has waited
           for its own loads of slab t+1 before it leaves the memory phase of slab t (before barrier 2t for the
           first group, 2t+1 for the second), so slab t+1 is whole in LDS for everybody after barrier 2t+1, which
           is where its earliest reader starts. A wave overwrites the stage of slab t-1 (with slab t+3) at the
           start of its memory phase of slab t, after barrier 2t-1 (2t for the second group); the last reads of
           slab t-1 finished before barrier 2t-1. */
        static_assert(NSTAGE == 4 && NW == 8 && !CS, "ping-pong: eight waves, four stages, no column sums");
        if (nk > 0) {
            const bool follower = wave >= NW / 2;
            issue_loads(IntC<1>(), 0);
            if (nk > 1)
                issue_loads(IntC<1>(), 1);
            if (nk > 2)
                issue_loads(IntC<1>(), 2);
            if (nk > 3)
                issue_loads(IntC<1>(), 3);
            if (nk > 3)
                wait_vmcnt<3 * NL>();
            else if (nk > 2)
                wait_vmcnt<2 * NL>();
            else if (nk > 1)
                wait_vmcnt<NL>();
            else
                wait_vmcnt<0>();
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
            if (follower)
                __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);

            /* AHEAD = how many later slabs exist (capped at 3); ISSUE: slab kt+3 exists and is not in flight yet */
            auto pp_slab = [&](auto AHEADC, auto ISSUEC, auto TAILC, int kt) {
                constexpr int ahead = decltype(AHEADC)::value;
                const char * stage = lds + (kt % NSTAGE) * STAGE;
                if constexpr (decltype(ISSUEC)::value != 0)
                    issue_loads(TAILC, kt + 3);
                read_frags(IntC<0>(), stage);
                read_frags(IntC<1>(), stage);
                wait_vmcnt<(ahead >= 3 ? 2 : (ahead == 2 ? 1 : 0)) * NL>();
                wait_lgkmcnt0();
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_sched_barrier(0);
                __builtin_amdgcn_s_setprio(1);
#pragma unroll
                for (int kk = 0; kk < KS; kk++)
#pragma unroll
                    for (int g = 0; g < NM; g++) {
                        const int i = g / TJ, j = g % TJ;
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[kk][i], fb[kk][j], acc[i][j], 0, 0, 0);
                    }
                __builtin_amdgcn_s_setprio(0);
                __builtin_amdgcn_sched_barrier(0);
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_sched_barrier(0);
            };

            const int nkFull = K / BKT;
            int kt = 0;
            /* the first slab issues nothing: the prologue has slabs 0 to 3 in flight */
            if (nk > 3)
                pp_slab(IntC<3>(), IntC<0>(), IntC<0>(), 0);
            else if (nk > 2)
                pp_slab(IntC<2>(), IntC<0>(), IntC<0>(), 0);
            else if (nk > 1)
                pp_slab(IntC<1>(), IntC<0>(), IntC<0>(), 0);
            else
                pp_slab(IntC<0>(), IntC<0>(), IntC<0>(), 0);
            kt = 1;
            for (; kt + 3 < nkFull; kt++)
                pp_slab(IntC<3>(), IntC<1>(), IntC<0>(), kt);      /* slab kt+3 is complete: no tail handling */
            for (; kt + 3 < nk; kt++)
                pp_slab(IntC<3>(), IntC<1>(), IntC<1>(), kt);
            if (kt + 2 < nk) {
                pp_slab(IntC<2>(), IntC<0>(), IntC<0>(), kt);
                kt++;
            }
            if (kt + 1 < nk) {
                pp_slab(IntC<1>(), IntC<0>(), IntC<0>(), kt);
                kt++;
            }
            if (kt < nk)
                pp_slab(IntC<0>(), IntC<0>(), IntC<0>(), kt);
            if (!follower)
                __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    else if (nk > 0) {
        static_assert(DEEP || NSTAGE == 4, "this loop is written for four stages");
        /* prologue: all four stages in flight, then wait for the first */
        issue_loads(IntC<1>(), 0);
        if (nk > 1)
            issue_loads(IntC<1>(), 1);
        if (nk > 2)
            issue_loads(IntC<1>(), 2);
        if (nk > 3)
            issue_loads(IntC<1>(), 3);
        if (nk > 3)
            wait_vmcnt<3 * NL>();
        else if (nk > 2)
            wait_vmcnt<2 * NL>();
        else if (nk > 1)
            wait_vmcnt<NL>();
        else
            wait_vmcnt<0>();
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        read_frags(IntC<0>(), lds);

        const int nkFull = K / BKT;              /* slabs entirely inside K */
        int kt = 0;
        for (; kt + 4 < nkFull; kt++)
            slab(IntC<4>(), IntC<0>(), kt);      /* slab kt+4 is complete: no tail handling */
        for (; kt + 4 < nk; kt++)
            slab(IntC<4>(), IntC<1>(), kt);
        if (kt + 3 < nk) {
            slab(IntC<3>(), IntC<0>(), kt);
            kt++;
        }
        if (kt + 2 < nk) {
            slab(IntC<2>(), IntC<0>(), kt);
            kt++;
        }
        if (kt + 1 < nk) {
            slab(IntC<1>(), IntC<0>(), kt);
            kt++;
        }
        if (kt < nk)
            slab(IntC<0>(), IntC<0>(), kt);
    }

    /* ---- epilogue: accumulator register r of lane l is element
       (8*(r/4) + 4*(l/32) + r%4, l%32) of its 32x32 block. The wave's rows of c are one
       buffer that ends where c ends: rows past M drop off it, columns past N are sent
       out of range. ------------------------------------------------------------------- */
    /* the lane number again, from the hardware rather than from threadIdx: a value that
       would otherwise have to stay in a register (or be spilled) across the whole main loop */
    const int laneE = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    const int l32E = laneE & 31, lhE = laneE >> 5;
    const float alpha = SPLIT ? 1.f : p.alpha, beta = SPLIT ? 0.f : p.beta;
    const OutT * __restrict__ bias = static_cast<const OutT *>(p.bias);     /* the bias has the type of c */
    const int biasMode = SPLIT ? (int)BIAS_NONE : p.biasMode;
    const int act = SPLIT ? (int)ACT_NONE : p.act;
    const int ldc = SPLIT ? N : p.ldc;
    OutT * cw = C + (size_t)(m0 + wm0) * ldc;
    const unsigned rowPitch = (unsigned)ldc * (unsigned)sizeof(OutT);

    if constexpr (CS) {
        /* the first tile row's first wave row has seen every k of its columns */
        if (tc.tm == 0 && wm0 == 0) {
            half_t * cs = static_cast<half_t *>(p.colSum);
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                const float v = colSum[j] + __shfl_xor(colSum[j], 32);
                const int col = n0 + wn0 + j * 32 + l32E;
                if (lhE == 0 && col < N)
                    cs[col] = (half_t)(p.colSumBeta != 0.f ? p.colSumBeta * (float)cs[col] + v : v);
            }
        }
    }

    /* Wide path (rows of c 16-byte aligned): a lane owns one COLUMN of each block, so storing
       straight from the accumulators means 2-byte stores, 64 contiguous bytes per row and
       instruction, and the store instruction count (16 per block) bounds the epilogue.
       Instead each wave turns 32 rows at a time through its own piece of LDS (the stages are
       free by now) and moves 16 bytes per lane: whole rows of the wave's tile, whole cache
       lines, an eighth of the instructions. With beta == 0 the values cross LDS as halves;
       with beta != 0 they cross as fp32 and meet the old c (one 16-byte load per lane) on the
       far side, so the result is still rounded once. */
    const bool wide = std::is_same<OutT, half_t>::value &&
                      (p.ldc & 7) == 0 && (N & 7) == 0 && (reinterpret_cast<size_t>(C) & 15) == 0;
    if constexpr (std::is_same<OutT, half_t>::value) if (wide) {
        constexpr int LPR = TJ * 4;                  /* lanes that cover one row of the wave's tile */
        constexpr int RPI = 64 / LPR;                /* rows per 16-byte store instruction */
        __syncthreads();                             /* every wave has read its last fragments */
        if (m0 + wm0 >= M)
            return;
        __amdgpu_buffer_rsrc_t cr = make_rsrc(cw, (long long)(M - m0 - wm0) * p.ldc * 2);
        float bcol[TJ];
#pragma unroll
        for (int j = 0; j < TJ; j++) {
            const int col = n0 + wn0 + j * 32 + l32E;
            bcol[j] = biasMode == BIAS_COL && col < N ? (float)bias[col] : 0.f;
        }
        const int rdRow = laneE / LPR, rdChunk = laneE % LPR;
        const int colW = n0 + wn0 + rdChunk * 8;
        const unsigned cOffW = colW + 8 <= N ? (unsigned)(rdRow * p.ldc + colW) * 2u : (unsigned)NTSAMD_OOB_OFFSET;

        auto turn = [&](auto BETAC, auto AUXC) {
            constexpr bool useOld = decltype(BETAC)::value != 0;
            constexpr int aux = decltype(AUXC)::value;
            typedef typename std::conditional<useOld, float, half_t>::type StageT;
            /* row pitch: the two half-waves write rows 4 apart; keep them in different banks */
            constexpr int PITCH = TJ * 32 * (int)sizeof(StageT) + (useOld ? 32 : 16);
            constexpr int GROUP = 32 * PITCH;
            constexpr int NBUF = useOld ? 1 : 2;
            static_assert(NBUF * GROUP * NW <= NSTAGE * STAGE, "epilogue staging must fit the stages");
            char * mine = lds + wave * NBUF * GROUP;
#pragma unroll
            for (int i = 0; i < TI; i++) {
                char * buf = mine + (i % NBUF) * GROUP;
                f32x4 old[32 / RPI];
                if constexpr (useOld) {
#pragma unroll
                    for (int q = 0; q < 32 / RPI; q++)
                        old[q] = buffer_load_f32x4(cr, (int)(cOffW + (unsigned)(i * 32 + q * RPI) * rowPitch));
                }
#pragma unroll
                for (int j = 0; j < TJ; j++)
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int row = 8 * (r / 4) + 4 * lhE + (r % 4);
                        *reinterpret_cast<StageT *>(buf + row * PITCH + (j * 32 + l32E) * (int)sizeof(StageT)) =
                            (StageT)(useOld ? alpha * acc[i][j][r] + bcol[j] : activate(alpha * acc[i][j][r] + bcol[j], act));
                    }
                /* the wave's own lanes exchange data through LDS: LDS executes one wave's
                   instructions in order, the fences only keep the compiler from reordering */
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
                for (int q = 0; q < 32 / RPI; q++) {
                    const char * src = buf + (q * RPI + rdRow) * PITCH + rdChunk * 8 * (int)sizeof(StageT);
                    const unsigned off = cOffW + (unsigned)(i * 32 + q * RPI) * rowPitch;
                    if constexpr (useOld) {
                        const f32x4 lo = *reinterpret_cast<const f32x4 *>(src);
                        const f32x4 hi = *reinterpret_cast<const f32x4 *>(src + 16);
                        const f16x8 o = __builtin_bit_cast(f16x8, old[q]);
                        f16x8 v;
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            v[e] = (half_t)activate(lo[e] + beta * (float)o[e], act);
                            v[4 + e] = (half_t)activate(hi[e] + beta * (float)o[4 + e], act);
                        }
                        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(f32x4, v), cr, (int)off, 0, aux);
                    }
                    else {
                        const f32x4 v = *reinterpret_cast<const f32x4 *>(src);
                        __builtin_amdgcn_raw_buffer_store_b128(v, cr, (int)off, 0, aux);
                    }
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
            }
        };
        if (beta != 0.f) {
            if (p.storeHint)
                turn(IntC<1>(), IntC<STORE_WRITE_THROUGH>());
            else
                turn(IntC<1>(), IntC<STORE_DEFAULT>());
        }
        else {
            if (p.storeHint)
                turn(IntC<0>(), IntC<STORE_WRITE_THROUGH>());
            else
                turn(IntC<0>(), IntC<STORE_DEFAULT>());
        }
        return;
    }

    /* Narrow path: element-wise stores straight from the accumulators, any alignment of c; also the
       path of a float result (half products whose result feeds a softmax: no separate conversion pass),
       where an instruction covers two rows of 128 contiguous bytes. beta is tested outside the loops:
       inside them every load of c would sit in a block of its own, one memory round trip after the other. */
    if (m0 + wm0 >= M)
        return;
    __amdgpu_buffer_rsrc_t cr = make_rsrc(cw, (long long)(M - m0 - wm0) * ldc * (long long)sizeof(OutT));
    auto narrow = [&](auto BETAC) {
        constexpr bool useOld = decltype(BETAC)::value != 0;
#pragma unroll
        for (int j = 0; j < TJ; j++) {
            const int col = n0 + wn0 + j * 32 + l32E;
            const unsigned cOff = col < N ? (unsigned)(4 * lhE * ldc + col) * (unsigned)sizeof(OutT)
                                          : (unsigned)NTSAMD_OOB_OFFSET;
            float bcol = 0.f;
            if (biasMode == BIAS_COL && col < N)
                bcol = (float)bias[col];
#pragma unroll
            for (int i = 0; i < TI; i++) {
                float old[16];
                if constexpr (useOld) {
#pragma unroll
                    for (int r = 0; r < 16; r++)
                        old[r] = buffer_load_out<OutT>(cr, (int)(cOff + (unsigned)(i * 32 + 8 * (r / 4) + (r % 4)) * rowPitch));
                }
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const unsigned off = cOff + (unsigned)(i * 32 + 8 * (r / 4) + (r % 4)) * rowPitch;
                    float v = alpha * acc[i][j][r] + bcol;
                    if constexpr (useOld)
                        v += beta * old[r];
                    buffer_store_out<OutT>((OutT)activate(v, act), cr, (int)off);
                }
            }
        }
    };
    if (beta != 0.f)
        narrow(IntC<1>());
    else
        narrow(IntC<0>());
}

template <typename OutT, int BM, int BN, int WGM, int WGN, int MINW, bool AKC, bool BKC, bool CS, bool SPLIT = false, int NSTAGE = 4,
          bool PP = false, int BKT = 32>
static int launch_f16_direct_shape(const GemmParams & p0, hipStream_t stream)
{
    GemmParams p = p0;
    p.tilesM = (p.M + BM - 1) / BM;
    p.tilesN = (p.N + BN - 1) / BN;
    if (!SPLIT)
        p.splits = 1;
    dim3 grid((unsigned)(p.tilesM * p.tilesN * p.batch * p.splits));
    hipLaunchKernelGGL((gemm_f16_direct_kernel<OutT, BM, BN, WGM, WGN, MINW, AKC, BKC, CS, SPLIT, NSTAGE, PP, BKT>),
                       grid, dim3(WGM * WGN * 64), 0, stream, p);
    return (int)hipGetLastError();
}

template <typename OutT, int CFG, bool AKC, bool BKC, bool CS>
static int launch_f16_direct(const GemmParams & p, hipStream_t stream)
{
    typedef TileShape<CFG> S;
    if constexpr (CFG == CFG_256x256) {
        /* The big tile on eight waves (wave tile 128 x 64, two waves per SIMD that cover each other's waits at
           the barrier and for LDS) instead of four (wave tile 128 x 128, half the LDS reads per MFMA): measured
           15-20 % faster at k = 512, 3-8 % at k = 1024, level at k = 4096 and 0-4 % slower at k = 8192. */
        if constexpr (!CS) {
            if (p.f16PingPong)
                return launch_f16_direct_shape<OutT, S::BM, S::BN, 2, 4, 1, AKC, BKC, false, false, 4, true>(p, stream);
        }
        if (p.K <= 2048)
            return launch_f16_direct_shape<OutT, S::BM, S::BN, 2, 4, 1, AKC, BKC, CS>(p, stream);
    }
    else if constexpr (!CS) {
        /* pieces of k leave fp32 partial tiles, whatever the type of c */
        if (p.splits > 1 && p.splitWork != NULL) {
            if constexpr (CFG == CFG_64x64)
                if (p.f16Slab64)
                    return launch_f16_direct_shape<float, S::BM, S::BN, S::WGM, S::WGN, S::MINW16, AKC, BKC, CS, true, 4, false, 64>(p, stream);
            return launch_f16_direct_shape<float, S::BM, S::BN, S::WGM, S::WGN, S::MINW16, AKC, BKC, CS, true>(p, stream);
        }
    }
    /* the small tile with slabs of 64: whole 128-byte lines of a K-contiguous operand per load, half the barriers
       and waits per k, four stages of 16-17 KB (three or six stages cost a division by a number that is no power
       of two where a stage's address is worked out, and ran slower than four; eight leave one workgroup to a CU) */
    if constexpr (CFG == CFG_64x64)
        if (p.f16Slab64)
            return launch_f16_direct_shape<OutT, S::BM, S::BN, S::WGM, S::WGN, S::MINW16, AKC, BKC, CS, false, 4, false, 64>(p, stream);
    return launch_f16_direct_shape<OutT, S::BM, S::BN, S::WGM, S::WGN, S::MINW16, AKC, BKC, CS>(p, stream);
}

/* a in float, rounded to half on its way to LDS (no lists of matrices) */
template <typename OutT, bool AKC, bool BKC, bool VEC>
static int launch_f16_staged_a32(const GemmParams & p, int cfg, hipStream_t stream)
{
    NoPtrs none = {0};
    if constexpr (VEC) if (cfg != CFG_64x64)
        return launch_f16_one<OutT, CFG_128x128, AKC, BKC, VEC, NoPtrs, float>(p, none, stream);
    return launch_f16_one<OutT, CFG_64x64, AKC, BKC, VEC, NoPtrs, float>(p, none, stream);
}

template <typename OutT, bool AKC, bool BKC, bool VEC>
static int launch_f16_staged(const GemmParams & p, const PtrBatch * ptrs, int cfg, hipStream_t stream)
{
    NoPtrs none = {0};
    if constexpr (VEC) if (cfg != CFG_64x64) {
        if (ptrs)
            return launch_f16_one<OutT, CFG_128x128, AKC, BKC, VEC, PtrBatch>(p, *ptrs, stream);
        return launch_f16_one<OutT, CFG_128x128, AKC, BKC, VEC, NoPtrs>(p, none, stream);
    }
    if (ptrs)
        return launch_f16_one<OutT, CFG_64x64, AKC, BKC, VEC, PtrBatch>(p, *ptrs, stream);
    return launch_f16_one<OutT, CFG_64x64, AKC, BKC, VEC, NoPtrs>(p, none, stream);
}

template <bool AKC, bool BKC>
static int launch_f16_persistent(const GemmParams & p0, hipStream_t stream);     /* gemm_f16_persist.h */

template <bool AKC, bool BKC>
static int launch_f16_trans(const GemmParams & p, const PtrBatch * ptrs, int vec, bool outF32, int cfg,
                            hipStream_t stream)
{
    if (p.aF32) {
        if (vec == F16_STAGED)
            return outF32 ? launch_f16_staged_a32<float, AKC, BKC, true>(p, cfg, stream)
                          : launch_f16_staged_a32<half_t, AKC, BKC, true>(p, cfg, stream);
        return outF32 ? launch_f16_staged_a32<float, AKC, BKC, false>(p, cfg, stream)
                      : launch_f16_staged_a32<half_t, AKC, BKC, false>(p, cfg, stream);
    }
    if (vec == F16_STAGED)
        return outF32 ? launch_f16_staged<float, AKC, BKC, true>(p, ptrs, cfg, stream)
                      : launch_f16_staged<half_t, AKC, BKC, true>(p, ptrs, cfg, stream);
    if (vec == F16_SCALAR || ptrs)
        return outF32 ? launch_f16_staged<float, AKC, BKC, false>(p, ptrs, cfg, stream)
                      : launch_f16_staged<half_t, AKC, BKC, false>(p, ptrs, cfg, stream);
    /* many tiles of 256 x 256 with nothing to read in the epilogue: one workgroup per CU walks over them */
    if (cfg == CFG_256x256 && p.persistGrid > 0 && !outF32)
        return launch_f16_persistent<AKC, BKC>(p, stream);
    /* a float result: the same main loop, 4-byte stores from the accumulators */
    if (outF32) {
        if (cfg == CFG_256x256)
            return launch_f16_direct<float, CFG_256x256, AKC, BKC, false>(p, stream);
        if (cfg == CFG_128x128)
            return launch_f16_direct<float, CFG_128x128, AKC, BKC, false>(p, stream);
        return launch_f16_direct<float, CFG_64x64, AKC, BKC, false>(p, stream);
    }
    /* column sums: the 256x256 tile has no registers to spare, and products that want column
       sums (weight gradients) are too small for it anyway */
    if (p.colSum != NULL) {
        if (cfg == CFG_64x64)
            return launch_f16_direct<half_t, CFG_64x64, AKC, BKC, true>(p, stream);
        return launch_f16_direct<half_t, CFG_128x128, AKC, BKC, true>(p, stream);
    }
    if (cfg == CFG_256x256)
        return launch_f16_direct<half_t, CFG_256x256, AKC, BKC, false>(p, stream);
    if (cfg == CFG_128x128)
        return launch_f16_direct<half_t, CFG_128x128, AKC, BKC, false>(p, stream);
    return launch_f16_direct<half_t, CFG_64x64, AKC, BKC, false>(p, stream);
}

}  // namespace ntsamd
