/*
 * fp16 GEMM for gfx950, 256 x 256 tile, persistent form: one workgroup per CU walks over
 * several tiles of c, and the first four slabs of the NEXT tile are on their way to LDS
 * before the finished tile's results leave. Same arithmetic, same LDS layouts and the same
 * ping-pong main loop as gemm_f16_direct_kernel<..., PP = true> (see gemm_f16_direct.h for
 * both); the results are the same bits.
 *
 * Why: a 256 x 256 tile ends with 128 KB of stores per CU. When every CU runs one tile per
 * workgroup, all CUs of a round finish together, 33 MB leave at once (about 7 us at the rate
 * the part sustains for stores alone), nothing is multiplied meanwhile, and the next round of
 * workgroups starts cold: launch, four slabs to fetch before the first MFMA. Here the store
 * burst of a tile overlaps the main loop of the next one, and that loop starts with its
 * operands already in LDS. Only the last tile's stores stay exposed.
 *
 * What that takes:
 *   - The epilogue must be short and must write whole 128-byte lines. Turning the accumulators
 *     through LDS two bytes at a time (a lane of v_mfma_f32_32x32x16_f16's result holds one
 *     COLUMN of its block) took 3.9 us per tile in this kernel, measured with time stamps: more
 *     than the stores themselves. Here the MFMA computes the TRANSPOSED block instead (the b
 *     fragment goes in as the first operand, the a fragment as the second: the fragment layouts
 *     of the two operands are the same), so a lane holds one ROW of c, and the columns of the b
 *     tile are dealt to the lanes of its fragment in a permuted order (groups of four columns,
 *     see `pcol`) chosen so that eight consecutive accumulator registers of a lane are eight
 *     consecutive columns: 16 bytes. Storing those straight to memory was measured too: 32
 *     rows x 32 bytes per instruction, four times the cache lines touched, 4.8 us per tile and
 *     the next tile's loads held up behind them. So the 16-byte pieces still cross LDS, 32
 *     rows of the wave's 64 columns at a time (4 writes and 4 reads of 16 bytes per lane where
 *     there were 32 writes of 2 bytes), and leave as whole lines, 8 rows per instruction. The
 *     order of the sum over k is unchanged: the results are the same bits.
 *   - The staging area lies in stages 2 and 3, so the next tile's slabs 0 and 1 are requested
 *     before the epilogue and slabs 2 and 3 after it, behind a barrier (a wave's loads land
 *     anywhere in a stage, also where another wave is still staging).
 *   - Vector-memory operations complete in issue order, loads and stores alike, and one
 *     counter (vmcnt) counts them all. A follow-on tile's slabs 0 and 1 are requested BEFORE
 *     the finished tile's NST stores and slabs 2 and 3 after them, so "slab 0 has landed" is
 *     vmcnt <= 3 NL + NST and "slab 1 has landed" is vmcnt <= 2 NL + NST; from slab 2 on the
 *     stores are older than every load still awaited.
 *   - No loads in the epilogue: the compiler cannot see the LDS-direct loads (inline
 *     assembly) and would wait for ALL of them before using a loaded value. Hence beta == 0
 *     and no bias here; products with either run on the one-tile-per-workgroup kernels.
 */
#pragma once
#include "gemm_f16_direct.h"

namespace ntsamd {

template <bool AKC, bool BKC>
__global__ void __launch_bounds__(512, 1)
gemm_f16_persistent_kernel(const GemmParams p)
{
    constexpr int BM = 256, BN = 256, WGN = 4, NW = 8, BKT = 32, KS = 2, NSTAGE = 4;
    constexpr int WM = 128, WN = 64, TI = 4, TJ = 2, NM = TI * TJ;
    /* per-operand LDS geometry, bytes: as in gemm_f16_direct_kernel */
    constexpr int A_RPC = AKC ? 16 : 512 / BM;
    constexpr int B_RPC = BKC ? 16 : 512 / BN;
    constexpr int A_NCH = AKC ? BM / 16 : BKT / A_RPC;
    constexpr int B_NCH = BKC ? BN / 16 : BKT / B_RPC;
    constexpr int A_CP = AKC ? 1024 : 1088;
    constexpr int B_CP = BKC ? 1024 : 1088;
    constexpr int A_BYTES = A_NCH * A_CP;
    constexpr int B_BYTES = B_NCH * B_CP;
    constexpr int STAGE = A_BYTES + B_BYTES;
    constexpr int NLA = A_NCH / NW, NLB = B_NCH / NW;
    constexpr int NL = NLA + NLB;
    /* the epilogue's turn through LDS: 32 rows of the wave's 64 columns as halves, rows 144 bytes apart (sixteen
       lanes that write 16 bytes each to sixteen consecutive rows then cover all 64 banks) */
    constexpr int EPI_PITCH = WN * 2 + 16, EPI_WAVE = 32 * EPI_PITCH;
    constexpr int NST = TI * 4;                     /* store instructions per wave and tile: 8 rows of 128 bytes each */
    static_assert(NW * EPI_WAVE <= 2 * STAGE, "the epilogue's staging must fit stages 2 and 3");
    static_assert(NSTAGE * STAGE <= 160 * 1024, "the stages must fit LDS");
    static_assert(3 * NL + NST < 64, "the wait counter has six bits");

    __shared__ __attribute__((aligned(1024))) char lds[NSTAGE * STAGE];

    /* profiling builds (-DNTSAMD_PROBE) keep time stamps of the 100 MHz clock in registers and write them, 16 per
       workgroup, to where p.bias points when the kernel ends */
#ifdef NTSAMD_PROBE
    unsigned long long st[16] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#define NTSAMD_STAMP(n) do { st[(n)] = __builtin_amdgcn_s_memrealtime(); } while (0)
    /* and, of slab 8 of every tile, the shader clock at six points of the slab, waves 0 and 4 */
    unsigned long long fine[6] = {0, 0, 0, 0, 0, 0};
#define NTSAMD_FINE(n) do { if (kt == 8) fine[(n)] = __builtin_amdgcn_s_memtime(); } while (0)
#else
#define NTSAMD_STAMP(n) do { } while (0)
#define NTSAMD_FINE(n) do { } while (0)
#endif

    const int M = p.M, N = p.N, K = p.K;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave / WGN) * WM, wn0 = (wave % WGN) * WN;
    const int l32 = lane & 31, lh = lane >> 5;
    const bool follower = wave >= NW / 2;
    const int nk = (K + BKT - 1) / BKT, nkFull = K / BKT;     /* the launcher guarantees nk >= 8 */
    const int total = p.tilesM * p.tilesN * p.batch;

    /* ---- the tile whose operands are being fetched ---------------------------------- */
    int m0 = 0, n0 = 0;
    half_t * C = NULL;
    const half_t * aTile = NULL, * bTile = NULL, * aEnd = NULL, * bEnd = NULL;
    int aOff[NLA], bOff[NLB];
    int aKc[NLA], bKc[NLB];
    auto setup = [&](int id) {
        const TileCoord tc = tile_of_id(p, id);
        const half_t * A = static_cast<const half_t *>(p.a) + batch_offset(tc.batch, p.batchInner, p.strideA, p.strideA1);
        const half_t * B = static_cast<const half_t *>(p.b) + batch_offset(tc.batch, p.batchInner, p.strideB, p.strideB1);
        C = static_cast<half_t *>(p.c) + batch_offset(tc.batch, p.batchInner, p.strideC, p.strideC1);
        m0 = tc.tm * BM;
        n0 = tc.tn * BN;
#pragma unroll
        for (int q = 0; q < NLA; q++) {
            const int ch = wave * NLA + q;
            if (AKC) {
                int row = ch * 16 + (lane >> 2);
                int col = (lane & 3) ^ ((row >> 2) & 3);
                aKc[q] = col * 8;
                int r = m0 + row < M - 1 ? row : M - 1 - m0;
                aOff[q] = (r * p.lda + col * 8) * 2;
            }
            else {
                constexpr int LPRA = 64 / A_RPC;
                int krow = ch + A_NCH * (lane / LPRA);
                int c = (lane % LPRA) * 8;
                c = m0 + c < M - 8 ? c : M - 8 - m0;
                aKc[q] = 0;
                aOff[q] = (krow * p.lda + c) * 2;
            }
        }
#pragma unroll
        for (int q = 0; q < NLB; q++) {
            const int ch = wave * NLB + q;
            if (BKC) {
                int row = ch * 16 + (lane >> 2);
                int col = (lane & 3) ^ ((row >> 2) & 3);
                bKc[q] = col * 8;
                int r = n0 + row < N - 1 ? row : N - 1 - n0;
                bOff[q] = (r * p.ldb + col * 8) * 2;
            }
            else {
                constexpr int LPRB = 64 / B_RPC;
                int krow = ch + B_NCH * (lane / LPRB);
                int c = (lane % LPRB) * 8;
                c = n0 + c < N - 8 ? c : N - 8 - n0;
                bKc[q] = 0;
                bOff[q] = (krow * p.ldb + c) * 2;
            }
        }
        aTile = AKC ? A + (size_t)m0 * p.lda : A + m0;
        bTile = BKC ? B + (size_t)n0 * p.ldb : B + n0;
        aEnd = A + (size_t)((AKC ? M : K) - 1) * p.lda + (AKC ? K : M);
        bEnd = B + (size_t)((BKC ? N : K) - 1) * p.ldb + (BKC ? K : N);
    };

    const unsigned ldsBase = (unsigned)(size_t)((__attribute__((address_space(3))) char *)lds);

    auto issue_loads = [&](auto TAIL, int kt) {
        constexpr bool mayHangOver = decltype(TAIL)::value != 0;
        const int k0 = kt * BKT;
        const unsigned stage = ldsBase + (unsigned)((kt % NSTAGE) * STAGE);
        const bool tail = mayHangOver && k0 + BKT > K;
        const half_t * ab = AKC ? aTile + k0 : aTile + (size_t)k0 * p.lda;
        const half_t * bb = BKC ? bTile + k0 : bTile + (size_t)k0 * p.ldb;
        const i32x4 ad = make_desc(ab, (long long)(aEnd - ab) * 2), bd = make_desc(bb, (long long)(bEnd - bb) * 2);
#pragma unroll
        for (int q = 0; q < NLA; q++) {
            int off = aOff[q];
            if (AKC && tail && k0 + aKc[q] >= K)
                off = NTSAMD_OOB_OFFSET;
            lds_dma16(ad, stage + (unsigned)((wave * NLA + q) * A_CP), off);
        }
#pragma unroll
        for (int q = 0; q < NLB; q++) {
            int off = bOff[q];
            if (BKC && tail && k0 + bKc[q] >= K)
                off = NTSAMD_OOB_OFFSET;
            lds_dma16(bd, stage + (unsigned)(A_BYTES + (wave * NLB + q) * B_CP), off);
        }
    };

    /* ---- fragment addresses (byte offsets inside a stage) ---------------------------- */
    /* The b fragment is the FIRST operand of the MFMA here: its lane rho (0..31) supplies the result's ROW rho, and
       result register r of a lane with half-wave h holds row 8 (r/4) + 4 h + r%4. Column pcol(rho) of the b block
       goes to fragment lane rho, with groups of four columns dealt out as
           group q = rho / 4 = (q2 q1 q0)  ->  columns 4 (q2 q0 q1) .. + 3   (the two low bits of the group swap)
       so that registers 8 g .. 8 g + 7 of a lane are columns 16 g + 8 h .. + 7 of the block. */
    const int q3 = l32 >> 2;
    const int pcol = 4 * ((q3 & 4) | ((q3 & 1) << 1) | ((q3 >> 1) & 1)) + (l32 & 3);
    const int trRow = (lane & 15) >> 2;
    const int trCol = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    /* a transposing read hands result lane c the piece of four columns that address lanes with (lane & 3) == c / 4
       point at: the same exchange of the two low bits of the group number, on the addresses */
    const int trColB = 16 * ((lane >> 4) & 1) + 8 * (lane & 1) + 4 * ((lane >> 1) & 1);
    int aFrag[KS], bFrag[KS];
    int aTr[KS][2], bTr[KS][2];
#pragma unroll
    for (int kk = 0; kk < KS; kk++) {
        const int sw = (l32 >> 2) & 3, swB = (pcol >> 2) & 3;
        aFrag[kk] = (wm0 + l32) * 64 + ((kk * 2 + lh) ^ sw) * 16;
        bFrag[kk] = A_BYTES + (wn0 + pcol) * 64 + ((kk * 2 + lh) ^ swB) * 16;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int kr = 16 * kk + 8 * lh + 4 * h + trRow;
            aTr[kk][h] = (kr % A_NCH) * A_CP + (kr / A_NCH) * (BM * 2) + (wm0 + trCol) * 2;
            bTr[kk][h] = A_BYTES + (kr % B_NCH) * B_CP + (kr / B_NCH) * (BN * 2) + (wn0 + trColB) * 2;
        }
    }

    f16x8 fa[KS][TI], fb[KS][TJ];
    auto read_frags = [&](const char * stage) {
#pragma unroll
        for (int kk = 0; kk < KS; kk++) {
#pragma unroll
            for (int i = 0; i < TI; i++) {
                if constexpr (AKC)
                    fa[kk][i] = *reinterpret_cast<const f16x8 *>(stage + aFrag[kk] + i * 32 * 64);
                else {
                    f16x4 lo = lds_read_tr16(reinterpret_cast<const half_t *>(stage + aTr[kk][0] + i * 64));
                    f16x4 hi = lds_read_tr16(reinterpret_cast<const half_t *>(stage + aTr[kk][1] + i * 64));
                    fa[kk][i] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                }
            }
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                if constexpr (BKC)
                    fb[kk][j] = *reinterpret_cast<const f16x8 *>(stage + bFrag[kk] + j * 32 * 64);
                else {
                    f16x4 lo = lds_read_tr16(reinterpret_cast<const half_t *>(stage + bTr[kk][0] + j * 64));
                    f16x4 hi = lds_read_tr16(reinterpret_cast<const half_t *>(stage + bTr[kk][1] + j * 64));
                    fb[kk][j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                }
            }
        }
    };

    f32x16 acc[TI][TJ];

    /* One slab: memory phase, barrier, compute phase, barrier (see the ping-pong loop of gemm_f16_direct_kernel).
       AHEAD = how many later slabs exist (capped at 3); ISSUE: slab kt+3 exists and is not in flight yet; EXTRA:
       stores of the previous tile that may still be in flight behind the loads this slab waits for. */
    auto pp_slab = [&](auto AHEADC, auto ISSUEC, auto TAILC, auto EXTRAC, int kt) {
        constexpr int ahead = decltype(AHEADC)::value;
        const char * stage = lds + (kt % NSTAGE) * STAGE;
        NTSAMD_FINE(0);
        if constexpr (decltype(ISSUEC)::value != 0)
            issue_loads(TAILC, kt + 3);
        read_frags(stage);
        NTSAMD_FINE(1);
        wait_vmcnt<(ahead >= 3 ? 2 : (ahead == 2 ? 1 : 0)) * NL + decltype(EXTRAC)::value>();
        wait_lgkmcnt0();
        NTSAMD_FINE(2);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        NTSAMD_FINE(3);
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int kk = 0; kk < KS; kk++)
#pragma unroll
            for (int g = 0; g < NM; g++) {
                const int i = g / TJ, j = g % TJ;
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[kk][j], fa[kk][i], acc[i][j], 0, 0, 0);
            }
        __builtin_amdgcn_s_setprio(0);
        __builtin_amdgcn_sched_barrier(0);
        NTSAMD_FINE(4);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        NTSAMD_FINE(5);
    };

    /* The main loop of one tile whose first four slabs are in flight. EXTRA: stores issued after those loads. */
    auto main_loop = [&](auto EXTRAC, auto PROBEC) {
        constexpr int pb = decltype(PROBEC)::value;      /* first time stamp of this tile */
        (void)pb;
#pragma unroll
        for (int i = 0; i < TI; i++)
#pragma unroll
            for (int j = 0; j < TJ; j++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    acc[i][j][r] = 0.f;
        wait_vmcnt<3 * NL + decltype(EXTRAC)::value>();
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        if (follower)
            __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        NTSAMD_STAMP(pb);
        pp_slab(IntC<3>(), IntC<0>(), IntC<0>(), EXTRAC, 0);
        pp_slab(IntC<3>(), IntC<1>(), IntC<0>(), IntC<0>(), 1);   /* nk >= 8: slabs 4 and 5 are complete */
        pp_slab(IntC<3>(), IntC<1>(), IntC<0>(), IntC<0>(), 2);
        NTSAMD_STAMP(pb + 1);
        int kt = 3;
#ifdef NTSAMD_PROBE
        pp_slab(IntC<3>(), IntC<1>(), IntC<0>(), IntC<0>(), kt);
        kt++;
        NTSAMD_STAMP(pb + 2);
#endif
        for (; kt + 3 < nkFull; kt++)
            pp_slab(IntC<3>(), IntC<1>(), IntC<0>(), IntC<0>(), kt);
        for (; kt + 3 < nk; kt++)
            pp_slab(IntC<3>(), IntC<1>(), IntC<1>(), IntC<0>(), kt);
        pp_slab(IntC<2>(), IntC<0>(), IntC<0>(), IntC<0>(), kt);
        pp_slab(IntC<1>(), IntC<0>(), IntC<0>(), IntC<0>(), kt + 1);
        pp_slab(IntC<0>(), IntC<0>(), IntC<0>(), IntC<0>(), kt + 2);
        if (!follower)
            __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    };

    /* ---- epilogue of the tile at (em0, en0) of eC: accumulator register r of lane (l32, lh) is row l32 of its
       block of c and, by the permutation above, column 16 (r/8) + 8 lh + r%8: eight consecutive registers are 16
       bytes of one row. Block row by block row the wave writes them to its own piece of LDS as rows of 64 halves and
       reads whole rows back, 8 lanes to a row: every store instruction covers 8 rows of 128 contiguous bytes. The
       wave's rows of c are one buffer that ends where c ends: rows past M drop off it, columns past N are sent out
       of range (N is a multiple of 8 here). -------------------------------------------------------------------- */
    auto epilogue = [&](int em0, int en0, half_t * eC) {
        const float alpha = p.alpha;
        const int act = p.act;
        /* a wave whose rows lie past M stores into a buffer of no bytes: every store is dropped, but every store is
           ISSUED, so that all waves have the same number of operations in flight (the waits count them) */
        const int rowsLeft = M - em0 - wm0 > 0 ? M - em0 - wm0 : 0;
        half_t * cw = eC + (size_t)(rowsLeft > 0 ? em0 + wm0 : 0) * p.ldc;
        __amdgpu_buffer_rsrc_t cr = make_rsrc(cw, (long long)rowsLeft * p.ldc * 2);
        const unsigned rowPitch = (unsigned)p.ldc * 2u;
        const int rdRow = lane >> 3, rdChunk = lane & 7;
        const int colW = en0 + wn0 + rdChunk * 8;
        const unsigned cOffW = colW + 8 <= N ? (unsigned)(rdRow * p.ldc + colW) * 2u : (unsigned)NTSAMD_OOB_OFFSET;
        char * mine = lds + 2 * STAGE + wave * EPI_WAVE;
        char * wr = mine + l32 * EPI_PITCH + lh * 16;
        const char * rd = mine + rdRow * EPI_PITCH + rdChunk * 16;
#pragma unroll
        for (int i = 0; i < TI; i++) {
#pragma unroll
            for (int j = 0; j < TJ; j++)
#pragma unroll
                for (int g = 0; g < 2; g++) {
                    f16x8 v;
#pragma unroll
                    for (int e = 0; e < 8; e++)
                        v[e] = (half_t)activate(alpha * acc[i][j][8 * g + e], act);
                    *reinterpret_cast<f16x8 *>(wr + (j * 32 + 16 * g) * 2) = v;
                }
            /* the wave's own lanes exchange data through LDS: LDS executes one wave's instructions in order, the
               fences only keep the compiler from reordering */
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const f32x4 v = *reinterpret_cast<const f32x4 *>(rd + q * 8 * EPI_PITCH);
                const int off = (int)(cOffW + (unsigned)(i * 32 + q * 8) * rowPitch);
                if (p.storeHint)
                    __builtin_amdgcn_raw_buffer_store_b128(v, cr, off, 0, STORE_WRITE_THROUGH);
                else
                    __builtin_amdgcn_raw_buffer_store_b128(v, cr, off, 0, STORE_DEFAULT);
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
    };

    /* ---- the walk over this workgroup's tiles ------------------------------------------ */
    int id = (int)blockIdx.x;
    if (id >= total)
        return;
    NTSAMD_STAMP(0);
    setup(id);
    issue_loads(IntC<0>(), 0);
    issue_loads(IntC<0>(), 1);
    issue_loads(IntC<0>(), 2);
    issue_loads(IntC<0>(), 3);
    main_loop(IntC<0>(), IntC<1>());
    NTSAMD_STAMP(4);
    for (;;) {
        /* every wave has passed the last barrier of the main loop: nobody reads the stages any more */
        const int em0 = m0, en0 = n0;
        half_t * eC = C;
        id += (int)gridDim.x;
        const bool more = id < total;
        if (more) {
            setup(id);
            issue_loads(IntC<0>(), 0);
            issue_loads(IntC<0>(), 1);
        }
        __builtin_amdgcn_sched_barrier(0);
        NTSAMD_STAMP(more ? 5 : 11);
        epilogue(em0, en0, eC);
        __builtin_amdgcn_sched_barrier(0);
        NTSAMD_STAMP(more ? 6 : 12);
        if (!more)
            break;
        /* stages 2 and 3 are free once every wave has read its staged rows back */
        wait_lgkmcnt0();
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        issue_loads(IntC<0>(), 2);
        issue_loads(IntC<0>(), 3);
        main_loop(IntC<NST>(), IntC<7>());
        NTSAMD_STAMP(10);
    }
#ifdef NTSAMD_PROBE
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    NTSAMD_STAMP(13);
    if (tid == 0) {
        unsigned long long * out = const_cast<unsigned long long *>(static_cast<const unsigned long long *>(p.bias)) + (size_t)blockIdx.x * 16;
#pragma unroll
        for (int n = 0; n < 16; n++)
            out[n] = st[n];
    }
    if (lane == 0 && (wave == 0 || wave == 4)) {
        unsigned long long * out = const_cast<unsigned long long *>(static_cast<const unsigned long long *>(p.bias)) +
                                   (size_t)gridDim.x * 16 + ((size_t)blockIdx.x * 2 + wave / 4) * 8;
#pragma unroll
        for (int n = 0; n < 6; n++)
            out[n] = fine[n];
        out[6] = __builtin_amdgcn_s_memtime();
        out[7] = __builtin_amdgcn_s_memrealtime();
    }
#endif
}

template <bool AKC, bool BKC>
static int launch_f16_persistent(const GemmParams & p0, hipStream_t stream)
{
    GemmParams p = p0;
    p.tilesM = (p.M + 255) / 256;
    p.tilesN = (p.N + 255) / 256;
    p.splits = 1;
    const long long total = (long long)p.tilesM * p.tilesN * p.batch;
    const unsigned groups = (unsigned)(total < p.persistGrid ? total : p.persistGrid);
    hipLaunchKernelGGL((gemm_f16_persistent_kernel<AKC, BKC>), dim3(groups), dim3(512), 0, stream, p);
    return (int)hipGetLastError();
}

}  // namespace ntsamd
