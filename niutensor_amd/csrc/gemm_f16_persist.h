/*
 * fp16 GEMM for gfx950, 256 x 256 tile (128 x 256 where the result is small), persistent form: one workgroup per
 * CU walks over several tiles of c, and the first four slabs of the NEXT tile are on their way to LDS before the
 * finished tile's results leave. The LDS layout of mn-contiguous operands and the ping-pong main loop (two wave
 * groups one phase apart, one barrier pair per slab) are those of gemm_f16_direct_kernel<..., PP = true> (see
 * gemm_f16_direct.h); the MFMA is v_mfma_f32_16x16x32_f16 here, which adds the 32 products of a k step in another
 * order than the 32 x 32 x 16 form of the other kernels: the two agree to the last half bit or one step apart.
 *
 * Why: a 256 x 256 tile ends with 128 KB of stores per CU. When every CU runs one tile per workgroup, all CUs of a
 * round finish together, 33 MB leave at once (about 6 us at the rate the fabric takes stores), nothing is
 * multiplied meanwhile, and the next round of workgroups starts cold: launch, four slabs to fetch before the first
 * MFMA. Here the next tile's main loop starts with its operands already in LDS.
 *
 * What that takes:
 *   - The epilogue must be short and must write whole 128-byte lines. The b fragment goes into the MFMA as the
 *     FIRST operand, so result register r of lane l is row l % 16 of its 16 x 16 block and column 4 (l / 16) + r:
 *     a lane holds four consecutive columns of one row, 8 bytes of c. Block row by block row the wave writes those
 *     8-byte pieces to its own piece of LDS and reads whole rows back, 8 lanes to a row of the wave's 64 columns:
 *     a store instruction covers 8 rows of 128 contiguous bytes. Activation and cache policy of the stores are
 *     compile-time constants of the epilogue's code (tested per value they cost four vector instructions each,
 *     3.6 us per tile); the turn through LDS is double-buffered.
 *   - The staging area lies where slabs 2 and 3 go, so the next tile's slabs 0 and 1 are requested before the
 *     epilogue and slabs 2 and 3 after it, behind a barrier (a wave's loads land anywhere in a stage, also where
 *     another wave is still staging).
 *   - Vector-memory operations complete in issue order, loads and stores alike, and one counter (vmcnt) counts
 *     them all. A follow-on tile's slabs 0 and 1 are requested BEFORE the finished tile's NST stores and slabs 2
 *     and 3 after them; the waits of the first two slabs count the stores in (see main_loop), from slab 2 on the
 *     stores are older than every load still awaited.
 *   - A k-contiguous operand is fetched TWO slabs at a time: a slab of 32 k is 64 bytes of a row, half a cache
 *     line, and fetched slab by slab every line crossed the path from L2 twice (measured with the same kernel
 *     fetching whole lines of the wrong bytes: 8192 x 4096 x 1024 with both operands k-contiguous 68.5 -> 63.4 us,
 *     8192^3 903 -> 845 us). So the eight lanes that fetch a row's 128 bytes sit in one load instruction: a chunk
 *     of 1 KB is 8 rows x (64 bytes of the even slab, then 64 bytes of the odd slab), the four stages of such an
 *     operand are two pair slots, and a pair is requested at the start of an even slab, two slabs before its
 *     first half is read. An mn-contiguous operand keeps its slab-by-slab fetch three slabs ahead (its rows are
 *     whole lines already). The two operands have their own regions of LDS for that.
 *   - The only loads besides the operands' are the bias (HASB): four 8-byte loads per lane and tile, requested
 *     between the finished tile's stores and the next tile's slabs 2 and 3 and counted with the stores; their
 *     first use is pinned behind the main loop, where nothing is in flight, because the compiler cannot see the
 *     LDS-direct loads (inline assembly) and would otherwise wait for ALL of them wherever it first touched the
 *     bias.
 *   - Old c (HASC, beta != 0) is read in the epilogue, a block row ahead, as the lane's own 8-byte pieces, and added
 *     in fp32 before the one rounding. Those loads are the compiler's, and it waits for them by counting what IT
 *     has issued: so in this form nothing of the next tile is requested before the epilogue is over (the
 *     accounting of the first slab is then that of a workgroup's first tile).
 */
#pragma once
#include "gemm_f16_direct.h"

namespace ntsamd {

template <bool AKC, bool BKC, bool HASB, int BM = 256, bool HASC = false>
__global__ void __launch_bounds__(512, 1)
gemm_f16_persistent_kernel(const GemmParams p)
{
    /* HASC: beta != 0, the old c is read on the way out. Its loads come from the compiler (it places their waits), so
       nothing of the next tile may be in flight behind the compiler's back while they are: the next tile's first
       slabs are requested after the epilogue, not before it (about 2 us per tile that the other form hides). */
    /* BM = 128 (k-contiguous a only): a tile of 128 x 256 for results with fewer 256 x 256 tiles than the part has
       CUs; the waves stand 2 x 4 as before, each with 64 x 64 of the tile */
    static_assert(BM == 256 || (BM == 128 && AKC), "the 128-row tile takes a k-contiguous a");
    constexpr int BN = 256, WGN = 4, NW = 8, BKT = 32;
    constexpr int WM = BM / 2, WN = 64, TI = WM / 16, TJ = WN / 16;      /* 16 x 16 blocks of v_mfma_f32_16x16x32_f16: a slab is ONE k step */
    /* LDS, one region per operand, four slabs each.
       k-contiguous: two pair slots of 32 KB; a chunk of 1 KB holds 8 rows x [slab parity][64 bytes], the four 16-byte
           columns of a row's 64 bytes permuted by (row >> 1) & 3. A fragment read has lane l at row l % 16, column
           l / 16; measured with SQ_LDS_BANK_CONFLICT on that address pattern: none with this permutation, one
           conflict cycle per cycle with (row >> 2) & 3 (the permutation that is free of conflicts where lane l reads
           row l % 32, column l / 32, as the 32 x 32 x 16 fragments of the other half kernels do).
       mn-contiguous: four stages of 16 chunks (k rows c and c+16, 512 bytes each), chunks 1088 bytes apart and
           chunks 8-15 another 32 bytes on: a transposing read of lanes 0-31 takes 32 bytes from each of k rows s and
           8 + s (s = 0..3), i.e. from chunks s and 8 + s, which then lie 64 s and 64 s + 32 bytes into a 256-byte
           line of the 64 banks. */
    constexpr int KC_SLOT = 32 * 1024, KC_REGION = 2 * KC_SLOT;
    constexpr int A_SLOT = BM * 128;                /* a pair of slabs of a k-contiguous a: BM rows of 128 bytes */
    constexpr int MN_CP = 1088, MN_STAGE = 69 * 256, MN_REGION = 4 * MN_STAGE;
    static_assert(15 * MN_CP + 32 + 1024 <= MN_STAGE, "sixteen chunks must fit a stage");
    constexpr int A_REGION = AKC ? 2 * A_SLOT : MN_REGION, B_REGION = BKC ? KC_REGION : MN_REGION;
    constexpr int A_HALF = AKC ? A_SLOT : 2 * MN_STAGE, B_HALF = BKC ? KC_SLOT : 2 * MN_STAGE;   /* where slabs 2 and 3 begin */
    /* load instructions per wave: KA, KB per PAIR of slabs (k-contiguous), MA, MB per slab (mn-contiguous) */
    constexpr int KA = AKC ? BM / 64 : 0, KB = BKC ? 4 : 0, MA = AKC ? 0 : 2, MB = BKC ? 0 : 2;
    constexpr int KK = KA + KB, MM = MA + MB;
    /* the epilogue's turn through LDS: 16 rows of the wave's 64 columns as halves, rows 144 bytes apart (32 lanes
       that write 8 bytes each, 16 rows x 2 pieces, then cover all 64 banks) */
    constexpr int EPI_PITCH = WN * 2 + 16, EPI_WAVE = 16 * EPI_PITCH;
    constexpr int NST = TI * 2;                     /* store instructions per wave and tile: 8 rows of 128 bytes each */
    /* HASB: a bias by column, of c's type. The 16 values that a lane's columns take (four 8-byte loads) are requested
       after the previous tile's stores and before slabs 2 and 3, so the waits of the first two slabs count them with
       the stores; the first tile's are requested before anything else. */
    constexpr int NB = HASB ? TJ : 0;
    constexpr int NSB = NST + NB;                   /* what lies between a later tile's slabs 0-1 and 2-3 */
    /* the staging of the epilogue: waves 0 .. EPI_IN_A - 1 in the second half of a's region, the others in b's */
    constexpr int EPI_IN_A = BM == 256 ? 4 : 2;
    static_assert(EPI_IN_A * 2 * EPI_WAVE <= A_REGION - A_HALF && (NW - EPI_IN_A) * 2 * EPI_WAVE <= B_REGION - B_HALF, "the epilogue's staging must fit the second halves");
    static_assert(A_REGION + B_REGION <= 160 * 1024, "the stages must fit LDS");
    static_assert(MM + NSB + KK + 2 * MM < 64, "the wait counter has six bits");

    __shared__ __attribute__((aligned(1024))) char lds[A_REGION + B_REGION];

    /* profiling builds (-DNTSAMD_PROBE) leave time stamps of the 100 MHz clock in LDS (thread 0 only) and write
       them, 16 per workgroup, to where p.bias points when the kernel ends */
#ifdef NTSAMD_PROBE
    __shared__ unsigned long long stampLds[16];
#define NTSAMD_STAMP(n) do { const unsigned long long t_ = __builtin_amdgcn_s_memrealtime(); if (threadIdx.x == 0) stampLds[(n)] = t_; } while (0)
#else
#define NTSAMD_STAMP(n) do { } while (0)
#endif
#define NTSAMD_FINE(n) do { } while (0)

    const int M = p.M, N = p.N, K = p.K;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave / WGN) * WM, wn0 = (wave % WGN) * WN;
    const bool follower = wave >= NW / 2;
    const int nk = (K + BKT - 1) / BKT;                        /* the launcher guarantees nk >= 8 */
    const int total = p.tilesM * p.tilesN * p.batch;
    f16x4 bv[HASB ? TJ : 1];
    /* the bias of the tile whose columns begin at bn0: columns 16 j + 4 (lane / 16) .. + 3 of the wave's 64, what
       result registers 0-3 of block column j hold; past N the buffer ends and the loads bring zeros */
    auto load_bias = [&](int bn0) {
        if constexpr (HASB) {
            const __amdgpu_buffer_rsrc_t br = make_rsrc(const_cast<half_t *>(static_cast<const half_t *>(p.bias)), (long long)N * 2);
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
                const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(br, (bn0 + wn0 + 16 * j + 4 * (lane >> 4)) * 2, 0, 0);
                bv[j] = __builtin_bit_cast(f16x4, v);
            }
        }
    };

    /* ---- the tile whose operands are being fetched ---------------------------------- */
    /* Where a tile lies is scalar arithmetic with divisions in it (a microsecond of it, measured, when it sat
       between one tile's last slab and its epilogue): locate() works it out for the NEXT tile while the current
       tile waits for its first slab, adopt() then only has the per-lane offsets left to do. */
    struct Loc {
        int m0, n0;
        half_t * C;
        const half_t * A, * B;
    };
    auto locate = [&](int id) {
        const TileCoord tc = tile_of_id(p, id);
        Loc l;
        l.A = static_cast<const half_t *>(p.a) + batch_offset(tc.batch, p.batchInner, p.strideA, p.strideA1);
        l.B = static_cast<const half_t *>(p.b) + batch_offset(tc.batch, p.batchInner, p.strideB, p.strideB1);
        l.C = static_cast<half_t *>(p.c) + batch_offset(tc.batch, p.batchInner, p.strideC, p.strideC1);
        l.m0 = tc.tm * BM;
        l.n0 = tc.tn * BN;
        return l;
    };
    int m0 = 0, n0 = 0;
    half_t * C = NULL;
    const half_t * aTile = NULL, * bTile = NULL, * aEnd = NULL, * bEnd = NULL;
    /* a lane's share of its wave's chunks: byte offset from the first element of the slab (of the pair's even slab),
       and, k-contiguous, the first k of its 16 bytes inside the pair */
    constexpr int NQA = AKC ? KA : MA, NQB = BKC ? KB : MB;
    int aOff[NQA], bOff[NQB];
    int aKc[NQA], bKc[NQB];
    auto adopt = [&](const Loc & l) {
        const half_t * A = l.A, * B = l.B;
        C = l.C;
        m0 = l.m0;
        n0 = l.n0;
#pragma unroll
        for (int q = 0; q < NQA; q++) {
            const int ch = wave * NQA + q;
            if (AKC) {
                const int row = ch * 8 + ((lane >> 2) & 7);
                const int col = (lane & 3) ^ ((row >> 1) & 3);
                aKc[q] = (lane >> 5) * 32 + col * 8;
                const int r = m0 + row < M - 1 ? row : M - 1 - m0;
                aOff[q] = (r * p.lda + aKc[q]) * 2;
            }
            else {
                const int krow = ch + 16 * (lane >> 5);
                int c = (lane & 31) * 8;
                c = m0 + c < p.mOper - 8 ? c : p.mOper - 8 - m0;
                aKc[q] = 0;
                aOff[q] = (krow * p.lda + c) * 2;
            }
        }
#pragma unroll
        for (int q = 0; q < NQB; q++) {
            const int ch = wave * NQB + q;
            if (BKC) {
                const int row = ch * 8 + ((lane >> 2) & 7);
                const int col = (lane & 3) ^ ((row >> 1) & 3);
                bKc[q] = (lane >> 5) * 32 + col * 8;
                const int r = n0 + row < N - 1 ? row : N - 1 - n0;
                bOff[q] = (r * p.ldb + bKc[q]) * 2;
            }
            else {
                const int krow = ch + 16 * (lane >> 5);
                int c = (lane & 31) * 8;
                c = n0 + c < p.nOper - 8 ? c : p.nOper - 8 - n0;
                bKc[q] = 0;
                bOff[q] = (krow * p.ldb + c) * 2;
            }
        }
        aTile = AKC ? A + (size_t)m0 * p.lda : A + m0;
        bTile = BKC ? B + (size_t)n0 * p.ldb : B + n0;
        aEnd = A + (size_t)((AKC ? M : K) - 1) * p.lda + p.mOper;
        bEnd = B + (size_t)((BKC ? N : K) - 1) * p.ldb + p.nOper;
    };

    const unsigned ldsBase = (unsigned)(size_t)((__attribute__((address_space(3))) char *)lds);

    /* the pair of slabs (kt, kt + 1), kt even, of the k-contiguous operands; the pieces that begin at or past K
       are sent out of range (they read as zero) */
    auto issue_pair = [&](int kt) {
        const int k0 = kt * BKT;
        const bool tail = k0 + 2 * BKT > K;
        const unsigned slot = (unsigned)(((kt >> 1) & 1) * KC_SLOT), slotA = (unsigned)(((kt >> 1) & 1) * A_SLOT);
        if constexpr (AKC) {
            const half_t * ab = aTile + k0;
            const i32x4 ad = make_desc(ab, (long long)(aEnd - ab) * 2);
#pragma unroll
            for (int q = 0; q < KA; q++) {
                int off = aOff[q];
                if (tail && k0 + aKc[q] >= K)
                    off = NTSAMD_OOB_OFFSET;
                lds_dma16(ad, ldsBase + slotA + (unsigned)((wave * KA + q) * 1024), off);
            }
        }
        if constexpr (BKC) {
            const half_t * bb = bTile + k0;
            const i32x4 bd = make_desc(bb, (long long)(bEnd - bb) * 2);
#pragma unroll
            for (int q = 0; q < KB; q++) {
                int off = bOff[q];
                if (tail && k0 + bKc[q] >= K)
                    off = NTSAMD_OOB_OFFSET;
                lds_dma16(bd, ldsBase + (unsigned)A_REGION + slot + (unsigned)((wave * KB + q) * 1024), off);
            }
        }
    };
    /* slab kt of the mn-contiguous operands (rows of k past K lie past the end of the descriptor: they read as zero) */
    auto issue_slab = [&](int kt) {
        const int k0 = kt * BKT;
        const unsigned stage = (unsigned)((kt & 3) * MN_STAGE);
        if constexpr (!AKC) {
            const half_t * ab = aTile + (size_t)k0 * p.lda;
            const i32x4 ad = make_desc(ab, (long long)(aEnd - ab) * 2);
#pragma unroll
            for (int q = 0; q < MA; q++)
                lds_dma16(ad, ldsBase + stage + (unsigned)((wave * MA + q) * MN_CP + 32 * ((wave * MA + q) >> 3)), aOff[q]);
        }
        if constexpr (!BKC) {
            const half_t * bb = bTile + (size_t)k0 * p.ldb;
            const i32x4 bd = make_desc(bb, (long long)(bEnd - bb) * 2);
#pragma unroll
            for (int q = 0; q < MB; q++)
                lds_dma16(bd, ldsBase + (unsigned)A_REGION + stage + (unsigned)((wave * MB + q) * MN_CP + 32 * ((wave * MB + q) >> 3)), bOff[q]);
        }
    };
    /* slabs kt and kt + 1 (kt even) of both operands, in the order the waits below count on: the pair, then the
       mn-contiguous operands' slab kt, then their slab kt + 1 */
    auto issue_two = [&](int kt) {
        issue_pair(kt);
        issue_slab(kt);
        issue_slab(kt + 1);
    };

    /* ---- fragment addresses (byte offsets inside the operand's region, slab 0) ----------- */
    /* v_mfma_f32_16x16x32_f16: lane l of either operand holds index l % 16 of its block and k = 8 (l / 16) .. + 7; the
       b fragment is the FIRST operand here, so that result register r of lane l is row l % 16 of the block of c (the
       a fragment's index) and column 4 (l / 16) + r (the b fragment's index): a lane holds four consecutive columns
       of one row, 8 bytes of c.
       k-contiguous: row + 16-byte column of a pair chunk, the column permuted by (row >> 1) & 3.
       mn-contiguous: two transposing reads, each of which hands a lane four consecutive k (k rows 8 g + 4 h + s,
       s = 0..3, pointed at by address lanes 4 s + q with their four columns 4 q .. 4 q + 3). */
    const int rho = lane & 15, g4 = lane >> 4;
    int aFrag = 0, bFrag = 0, aTr[2] = {0, 0}, bTr[2] = {0, 0};
    {
        const int ra = wm0 + rho, rb = wn0 + rho;
        const int sw = (rho >> 1) & 3;
        aFrag = (ra >> 3) * 1024 + (ra & 7) * 64 + ((g4 ^ sw) * 16);
        bFrag = A_REGION + (rb >> 3) * 1024 + (rb & 7) * 64 + ((g4 ^ sw) * 16);
        const int s4 = rho >> 2, q4 = rho & 3;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int kr = 8 * g4 + 4 * h + s4, ch = kr & 15;
            aTr[h] = ch * MN_CP + 32 * (ch >> 3) + (kr >> 4) * (BM * 2) + (wm0 + 4 * q4) * 2;
            bTr[h] = A_REGION + ch * MN_CP + 32 * (ch >> 3) + (kr >> 4) * (BN * 2) + (wn0 + 4 * q4) * 2;
        }
    }
    /* where slab kt of an operand begins inside its region */
    auto slab_base = [&](bool kc, int slotBytes, int kt) {
        return kc ? ((kt >> 1) & 1) * slotBytes + (kt & 1) * 512 : (kt & 3) * MN_STAGE;
    };

    f16x8 fa[TI], fb[TJ];
    auto read_frags = [&](int kt) {
        const char * sa = lds + slab_base(AKC, A_SLOT, kt), * sb = lds + slab_base(BKC, KC_SLOT, kt);
#pragma unroll
        for (int i = 0; i < TI; i++) {
            if constexpr (AKC)
                fa[i] = *reinterpret_cast<const f16x8 *>(sa + aFrag + i * 2048);
            else {
                f16x4 lo = lds_read_tr16(reinterpret_cast<const half_t *>(sa + aTr[0] + i * 32));
                f16x4 hi = lds_read_tr16(reinterpret_cast<const half_t *>(sa + aTr[1] + i * 32));
                fa[i] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
        }
#pragma unroll
        for (int j = 0; j < TJ; j++) {
            if constexpr (BKC)
                fb[j] = *reinterpret_cast<const f16x8 *>(sb + bFrag + j * 2048);
            else {
                f16x4 lo = lds_read_tr16(reinterpret_cast<const half_t *>(sb + bTr[0] + j * 32));
                f16x4 hi = lds_read_tr16(reinterpret_cast<const half_t *>(sb + bTr[1] + j * 32));
                fb[j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
        }
    };

    f32x4 acc[TI][TJ];

    /* s_waitcnt takes its count as a constant: the handful of counts the loop below asks for, picked by a scalar
       branch (once per slab and wave) */
    auto wait_vm = [&](int n) {
        if (n == 0) wait_vmcnt<0>();
        else if (n == MM) wait_vmcnt<MM>();
        else if (n == 2 * MM) wait_vmcnt<2 * MM>();
        else if (n == KK + MM) wait_vmcnt<KK + MM>();
        else if (n == KK + 2 * MM) wait_vmcnt<KK + 2 * MM>();
        else if (n == NSB + KK + 2 * MM) wait_vmcnt<NSB + KK + 2 * MM>();
        else if (n == MM + KK + 2 * MM) wait_vmcnt<MM + KK + 2 * MM>();
        else if (n == MM + NSB + KK + 2 * MM) wait_vmcnt<MM + NSB + KK + 2 * MM>();
        else wait_vmcnt<0>();
    };

    /* The main loop of one tile whose first four slabs are in flight, requested as issue_two(0), `extra` other
       operations (the previous tile's stores), issue_two(2). One slab is a memory phase, a barrier, a compute phase
       and a barrier (see the ping-pong loop of gemm_f16_direct_kernel). At the start of its memory phase a wave may
       overwrite the slabs before kt: an even slab (from 2 on) requests the pair (kt + 2, kt + 3) of the
       k-contiguous operands, every slab (from 1 on) requests slab kt + 3 of the others, where they exist. When the
       phase ends slab kt + 1 must be whole; what may still be in flight is what was requested after its last piece:
         slab 0:  the previous tile's stores and slabs 2 and 3                                  extra + KK + 2 MM
         even kt: the mn-contiguous slab kt + 2 (requested in slab kt - 1), the pair (kt + 2, kt + 3) and the
                  mn-contiguous slab kt + 3 (both requested in slab kt)                          KK + 2 MM
         odd kt:  the mn-contiguous slabs kt + 2 and kt + 3 (the pair that holds slab kt + 1 was requested in slab
                  kt - 1, before them)                                                           2 MM
         slab nk - 3: nothing comes after slab nk - 1: the pair (nk - 1, nk) if kt is even, and the mn-contiguous
                  slab nk - 1                                                                    (KK +) MM
         the last two slabs: nothing.
       The loop is ONE copy of the slab's code whatever kt is (the compiler spilled accumulators when the first and
       last slabs had copies of their own: fourteen of them). */
    auto main_loop = [&](int extra) {
#pragma unroll
        for (int i = 0; i < TI; i++)
#pragma unroll
            for (int j = 0; j < TJ; j++)
                acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
        /* slab 0 is whole: after its last piece came its neighbour's mn-contiguous part, the stores, and slabs 2 and 3 */
        wait_vm(MM + extra + KK + 2 * MM);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        if (follower)
            __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        NTSAMD_STAMP(extra ? 7 : 1);
        /* the second half of a slab: barrier, the slab's MFMAs at raised priority, barrier */
        auto compute = [&](int kt) {
            (void)kt;
            wait_lgkmcnt0();
            NTSAMD_FINE(2);
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
            NTSAMD_FINE(3);
            __builtin_amdgcn_s_setprio(1);
            /* block rows forth and back: every second row keeps the b fragment of the MFMA before it (a little less
               switching at the matrix pipe's inputs: 1-2 % of the run time on random data) */
#pragma unroll
            for (int i = 0; i < TI; i++)
#pragma unroll
                for (int jj = 0; jj < TJ; jj++) {
                    const int j = (i & 1) ? TJ - 1 - jj : jj;
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[j], fa[i], acc[i][j], 0, 0, 0);
                }
            __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_sched_barrier(0);
            NTSAMD_FINE(4);
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
            NTSAMD_FINE(5);
        };
        /* One slab. ISSUE: 2 = it requests the pair (kt + 2, kt + 3) if kt is even and slab kt + 3 of the
           mn-contiguous operands, 1 = the pair only, 0 = nothing. What may stay in flight is a constant for odd kt
           and one for even kt. (Written with the slab's place in the tile as compile-time flags and few copies: a
           single loop over all slabs with everything tested at run time, and a copy per distinct slab, both made
           the compiler move or spill accumulators.) */
        auto slab = [&](auto ISSUEC, auto ODDC, auto EVENC, int kt) {
            constexpr int ISSUE = decltype(ISSUEC)::value;
            const bool odd = (kt & 1) != 0;
            if constexpr (ISSUE >= 1 && KK > 0) {
                if (!odd)
                    issue_pair(kt + 2);
            }
            if constexpr (ISSUE >= 2 && MM > 0)
                issue_slab(kt + 3);
            read_frags(kt);
            if constexpr (decltype(ODDC)::value == decltype(EVENC)::value)
                wait_vmcnt<decltype(ODDC)::value>();
            else {
                if (odd)
                    wait_vmcnt<decltype(ODDC)::value>();
                else
                    wait_vmcnt<decltype(EVENC)::value>();
            }
            compute(kt);
        };
        /* slab 0 requests nothing (slabs 2 and 3 are in flight) and counts the previous tile's stores */
        read_frags(0);
        if (extra)
            wait_vmcnt<NSB + KK + 2 * MM>();
        else
            wait_vmcnt<KK + 2 * MM>();
        compute(0);
        int kt = 1;
        for (; kt + 3 < nk; kt++)
            slab(IntC<2>(), IntC<2 * MM>(), IntC<KK + 2 * MM>(), kt);
        slab(IntC<1>(), IntC<MM>(), IntC<KK + MM>(), kt);          /* slab nk - 3: after slab nk - 1 of the mn-contiguous operands nothing is requested */
        slab(IntC<0>(), IntC<0>(), IntC<0>(), kt + 1);
        slab(IntC<0>(), IntC<0>(), IntC<0>(), kt + 2);
        if (!follower)
            __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    };

    /* ---- epilogue of the tile at (em0, en0) of eC: accumulator register r of lane (rho, g4) is row rho of its block
       of c and column 4 g4 + r. Block row by block row (16 rows) the wave writes its 8-byte pieces to its own piece
       of LDS as rows of 64 halves and reads whole rows back, 8 lanes to a row: every store instruction covers 8 rows
       of 128 contiguous bytes. The wave's rows of c are one buffer that ends where c ends: rows past M drop off it,
       columns past N are sent out of range (N is a multiple of 8 here). ---------------------------------------- */
    auto epilogue_as = [&](auto ACTC, auto THROUGHC, int em0, int en0, half_t * eC) {
        /* whether there is an activation and how the stores treat the caches are constants of this copy of the code:
           tested per element, the activation made the epilogue four vector instructions per value, 512 per lane,
           and with two waves to a SIMD that, not the stores, was what the 3.6 us between two tiles were made of */
        constexpr int act = decltype(ACTC)::value;
        constexpr int aux = decltype(THROUGHC)::value ? STORE_WRITE_THROUGH : STORE_DEFAULT;
        const float alpha = p.alpha;
        /* a wave whose rows lie past M stores into a buffer of no bytes: every store is dropped, but every store is
           ISSUED, so that all waves have the same number of operations in flight (the waits count them) */
        const int rowsLeft = M - em0 - wm0 > 0 ? M - em0 - wm0 : 0;
        half_t * cw = eC + (size_t)(rowsLeft > 0 ? em0 + wm0 : 0) * p.ldc;
        __amdgpu_buffer_rsrc_t cr = make_rsrc(cw, (long long)rowsLeft * p.ldc * 2);
        const unsigned rowPitch = (unsigned)p.ldc * 2u;
        const int rdRow = lane >> 3, rdChunk = lane & 7;
        const int colW = en0 + wn0 + rdChunk * 8;
        const unsigned cOffW = colW + 8 <= N ? (unsigned)(rdRow * p.ldc + colW) * 2u : (unsigned)NTSAMD_OOB_OFFSET;
        /* the staging lies where slabs 2 and 3 go: four waves in a's region, four in b's; two buffers per wave, so
           that block row i + 1 is on its way into LDS while block row i comes back out */
        char * mine = lds + (wave < EPI_IN_A ? A_HALF + wave * (2 * EPI_WAVE) : A_REGION + B_HALF + (wave - EPI_IN_A) * (2 * EPI_WAVE));
        /* HASC: the old values of a lane's own pieces (row rho of block row i, columns 16 j + 4 g4 .. + 3: 8 bytes),
           fetched one block row ahead and added in fp32 before the one rounding */
        const float beta = p.beta;
        f16x4 cold[HASC ? 2 : 1][HASC ? TJ : 1];
        auto load_c = [&](int i) {
            if constexpr (HASC) {
#pragma unroll
                for (int j = 0; j < TJ; j++) {
                    typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
                    const int col = en0 + wn0 + 16 * j + 4 * g4;
                    const unsigned off = col < N ? (unsigned)(i * 16 + rho) * rowPitch + (unsigned)col * 2u : (unsigned)NTSAMD_OOB_OFFSET;
                    const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(cr, (int)off, 0, 0);
                    cold[i & 1][j] = __builtin_bit_cast(f16x4, v);
                }
            }
        };
        auto put = [&](int i) {
            char * wr = mine + (i & 1) * EPI_WAVE + rho * EPI_PITCH + g4 * 8;
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                f16x4 v;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float x = alpha * acc[i][j][e];
                    if constexpr (HASB)
                        x += (float)bv[j][e];
                    if constexpr (HASC)
                        x += beta * (float)cold[i & 1][j][e];
                    v[e] = (half_t)activate(x, act);
                }
                *reinterpret_cast<f16x4 *>(wr + j * 32) = v;
            }
        };
        load_c(0);
        put(0);
        if (TI > 1)
            load_c(1);
#pragma unroll
        for (int i = 0; i < TI; i++) {
            /* the wave's own lanes exchange data through LDS: LDS executes one wave's instructions in order, the
               fences only keep the compiler from reordering */
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            const char * rd = mine + (i & 1) * EPI_WAVE + rdRow * EPI_PITCH + rdChunk * 16;
            f32x4 v[2];
#pragma unroll
            for (int q = 0; q < 2; q++)
                v[q] = *reinterpret_cast<const f32x4 *>(rd + q * 8 * EPI_PITCH);
            if (i + 1 < TI)
                put(i + 1);
            if (i + 2 < TI)
                load_c(i + 2);
#pragma unroll
            for (int q = 0; q < 2; q++)
                __builtin_amdgcn_raw_buffer_store_b128(v[q], cr, (int)(cOffW + (unsigned)(i * 16 + q * 8) * rowPitch), 0, aux);
        }
    };
    auto epilogue = [&](int em0, int en0, half_t * eC) {
        if (p.act == ACT_RECTIFY) {
            if (p.storeHint)
                epilogue_as(IntC<ACT_RECTIFY>(), IntC<1>(), em0, en0, eC);
            else
                epilogue_as(IntC<ACT_RECTIFY>(), IntC<0>(), em0, en0, eC);
        }
        else {
            if (p.storeHint)
                epilogue_as(IntC<ACT_NONE>(), IntC<1>(), em0, en0, eC);
            else
                epilogue_as(IntC<ACT_NONE>(), IntC<0>(), em0, en0, eC);
        }
    };

    /* ---- the walk over this workgroup's tiles ------------------------------------------ */
    int id = (int)blockIdx.x;
    if (id >= total)
        return;
    NTSAMD_STAMP(0);
    adopt(locate(id));
    load_bias(n0);
    issue_two(0);
    issue_two(2);
    int extra = 0;
    for (;;) {
        id += (int)gridDim.x;
        const bool more = id < total;
        const Loc next = locate(more ? id : 0);          /* while the first slab is on its way */
        main_loop(extra);
        NTSAMD_STAMP(extra ? 10 : 4);
        /* every wave has passed the last barrier of the main loop: nobody reads the stages any more */
        const int em0 = m0, en0 = n0;
        half_t * eC = C;
        if constexpr (HASB) {
            /* the bias is used from here on: whatever wait the compiler puts before its first use lands here, where
               nothing is in flight, and not behind the next tile's first slabs */
#pragma unroll
            for (int j = 0; j < TJ; j++)
                asm volatile("" : "+v"(bv[j]));
        }
        if constexpr (!HASC) {
            if (more) {
                adopt(next);
                issue_two(0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        NTSAMD_STAMP(more ? 5 : 11);
        epilogue(em0, en0, eC);
        __builtin_amdgcn_sched_barrier(0);
        NTSAMD_STAMP(more ? 6 : 12);
        if (!more)
            break;
        if constexpr (HASC)
            adopt(next);
        load_bias(n0);
        /* where slabs 2 and 3 go is free once every wave has read its staged rows back */
        wait_lgkmcnt0();
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (HASC) {
            /* the stores and the loads of old c lie before all four slabs, as before a workgroup's first tile */
            issue_two(0);
            issue_two(2);
            extra = 0;
        }
        else {
            issue_two(2);
            extra = NSB;
        }
    }
#ifdef NTSAMD_PROBE
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    NTSAMD_STAMP(13);
    if (tid == 0) {
        unsigned long long * out = const_cast<unsigned long long *>(static_cast<const unsigned long long *>(p.bias)) + (size_t)blockIdx.x * 16;
        for (int n = 0; n < 16; n++)
            out[n] = stampLds[n];
    }
#endif
}

template <bool AKC, bool BKC>
static int launch_f16_persistent(const GemmParams & p0, hipStream_t stream)
{
    GemmParams p = p0;
    /* p.persistRows: 128 = tiles of 128 x 256 (a k-contiguous), otherwise 256 x 256 */
    const int bm = AKC && p.persistRows == 128 ? 128 : 256;
    p.tilesM = (p.M + bm - 1) / bm;
    p.tilesN = (p.N + 255) / 256;
    p.splits = 1;
    const long long total = (long long)p.tilesM * p.tilesN * p.batch;
    const unsigned groups = (unsigned)(total < p.persistGrid ? total : p.persistGrid);
#ifdef NTSAMD_PROBE
    const bool hasBias = false;         /* a profiling build: the bias pointer is where the time stamps go */
#else
    const bool hasBias = p.bias != NULL;
#endif
    const bool hasC = p.beta != 0.f;
    auto go = [&](auto BMC) {
        constexpr int bmc = decltype(BMC)::value;
        if (hasC)       /* (never with a bias as well: that combination has no registers left, the dispatcher keeps it away) */
            hipLaunchKernelGGL((gemm_f16_persistent_kernel<AKC, BKC, false, bmc, true>), dim3(groups), dim3(512), 0, stream, p);
        else {
            if (hasBias)
                hipLaunchKernelGGL((gemm_f16_persistent_kernel<AKC, BKC, true, bmc, false>), dim3(groups), dim3(512), 0, stream, p);
            else
                hipLaunchKernelGGL((gemm_f16_persistent_kernel<AKC, BKC, false, bmc, false>), dim3(groups), dim3(512), 0, stream, p);
        }
    };
    if constexpr (AKC) {
        if (bm == 128) {
            go(IntC<128>());
            return (int)hipGetLastError();
        }
    }
    go(IntC<256>());
    return (int)hipGetLastError();
}

}  // namespace ntsamd
