/*
 * out = softmax(scale * Q K^T + mask) V per head, fp32, in one kernel for gfx950.
 *
 * Stands where the reference's attention runs a chain of operators
 * (source/sample/transformer/submodel/Attention.cpp:186-237): Split of q, k, v
 * into heads, Scale of q, BMMul(q, k^T), Sum with the mask, Softmax over the
 * last dimension, BMMul with v, Merge of the heads. Here the head split and
 * merge are strides and the scores never leave the registers.
 *
 * Work split: a workgroup of 4 waves takes 64 query rows of one (head, batch
 * item), 16 rows per wave; two workgroups share a CU, so each SIMD holds two
 * waves and one wave's softmax arithmetic runs under the other's MFMAs. Keys
 * and values stream through LDS in blocks of KB keys; row maxima and sums are
 * carried from block to block and the running result is rescaled when a later
 * block raises a row's maximum, so any number of keys takes one pass over k, v.
 *
 * Both products are computed TRANSPOSED with v_mfma_f32_16x16x4_f32
 * (D = A B + C, A: lane l holds A[l%16][l/16], B: lane l holds B[l/16][l%16],
 * D: register r of lane l holds D[4*(l/16) + r][l%16]):
 *   S^T = K Q^T   A = key block from LDS (one 16-byte read feeds four steps),
 *                 B = Q fragments, in registers for the whole kernel;
 *                 lane (m, g) = (l%16, l/16) ends up with the scores of query m
 *                 against keys 16 j + 4 g + r of every 16-key block j.
 *   O^T = V^T P^T B = P^T: lane (m, g) must supply, for query m, one key per
 *                 step out of its group g - which is exactly a score register
 *                 it already holds (the order in which a sum runs over the keys
 *                 is free), A = value rows from LDS.
 * So the probabilities go from accumulator to operand without any exchange, a
 * query row's maximum and sum are reductions inside a lane plus two cross-lane
 * steps (lanes m, m+16, m+32, m+48), and every per-row quantity is one register.
 */
#include "gemm_common.h"
#include "gemm_f32.h"
#include "attention.h"

namespace ntsamd {

/* DHM: head size the kernel is built for (dh <= DHM; columns past dh are zero in LDS and in the
   q fragments, and are multiplied like the others: the launcher picks the smallest DHM that holds dh);
   KB: keys per block */
template <int DHM, int KB>
__global__ void __launch_bounds__(256, 2)
attention_f32_kernel(const AttnParams p)
{
    constexpr int KP = DHM + 4;          /* row pitch of the value block in floats: 4 mod 64, so the 4-byte reads of
                                            rows 4 apart spread over all banks */
    constexpr int KPK = DHM + 8;         /* the same for the keys: a 16-byte read takes lanes 0-7 and 16-23 together
                                            (rows m = 0..7, columns g = 0, 1), then 8-15 with 24-31 and so on: with a
                                            pitch of 2 mod 16 pieces of 16 bytes those sixteen lanes hit sixteen
                                            different pieces of the 256 bytes a cycle serves; with the pitch of the
                                            values every such read took two turns (counted: SQ_LDS_BANK_CONFLICT) */
    constexpr int NT = DHM / 16;         /* groups of four MFMA steps over dh; also 16-column blocks of the result */
    constexpr int NJ = KB / 16;          /* 16-key blocks */
    constexpr int LOADS = KB * DHM / 4 / 256;
    constexpr float LOG2E = 1.4426950408889634f;

    __shared__ __attribute__((aligned(16))) float Ks[KB * KPK];
    __shared__ __attribute__((aligned(16))) float Vs[KB * KP];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = lane & 15, g = lane >> 4;

    /* workgroups of one (head, batch item) are neighbours on one XCD: they share k and v in its L2 */
    const int id = xcd_contiguous_id((int)blockIdx.x, (int)gridDim.x);
    const int qt = id % p.qTiles;
    const int pair = id / p.qTiles;
    const int h = pair / p.batch, b = pair - h * p.batch;
    const int lq = p.lq, lk = p.lk, dh = p.dh;

    const float * Q = static_cast<const float *>(p.q) + h * p.qH + b * p.qB;
    const float * K = static_cast<const float *>(p.k) + h * p.kH + b * p.kB;
    const float * V = static_cast<const float *>(p.v) + h * p.vH + b * p.vB;
    float * O = static_cast<float *>(p.out) + h * p.oH + b * p.oB;

    const int row = qt * 64 + wave * 16 + m;              /* this lane's query row */
    const int rowc = row < lq ? row : lq - 1;             /* rows past the end repeat the last one; never stored */
    const float * MK = p.mask ? p.mask + ((long long)pair * lq + rowc) * lk : nullptr;

    /* ---- key / value staging: 16 bytes per thread and step through buffer loads whose descriptor ends
       with the last key, so keys past lk read as zero; columns past dh get an offset outside every
       descriptor. A thread's column never changes, its rows are RSTEP apart from step to step. ---- */
    constexpr int TPR = DHM / 4;         /* threads per row */
    constexpr int RSTEP = 256 / TPR;     /* rows per step */
    const int sr0 = tid / TPR, sc = (tid % TPR) * 4;
    const int sLds = sr0 * KP + sc, sLdsK = sr0 * KPK + sc;
    const __amdgpu_buffer_rsrc_t kRsrc = make_rsrc(K, ((long long)(lk - 1) * p.kL + dh) * 4);
    const __amdgpu_buffer_rsrc_t vRsrc = make_rsrc(V, ((long long)(lk - 1) * p.vL + dh) * 4);
    const int kL4 = (int)p.kL * 4, vL4 = (int)p.vL * 4;
    const int kOff0 = sc < dh ? sr0 * kL4 + sc * 4 : NTSAMD_OOB_OFFSET;
    const int vOff0 = sc < dh ? sr0 * vL4 + sc * 4 : NTSAMD_OOB_OFFSET;
    f32x4 kreg[LOADS], vreg[LOADS];
    auto load_k = [&](int kb0, int first, int last) {
#pragma unroll
        for (int s = 0; s < LOADS; s++)
            if (s >= first && s < last)
                kreg[s] = buffer_load_f32x4(kRsrc, sc < dh ? kOff0 + (kb0 + s * RSTEP) * kL4 : NTSAMD_OOB_OFFSET);
    };
    auto load_v = [&](int kb0) {
#pragma unroll
        for (int s = 0; s < LOADS; s++)
            vreg[s] = buffer_load_f32x4(vRsrc, sc < dh ? vOff0 + (kb0 + s * RSTEP) * vL4 : NTSAMD_OOB_OFFSET);
    };
    load_k(0, 0, LOADS / 2);     /* the second half of the first keys is asked for when the first has arrived */

    /* ---- Q fragments: lane (m, g) feeds query m with columns 16 t + 4 g + e in step e of group t ---- */
    f32x4 qf[NT];
    {
        const float * qr = Q + (long long)rowc * p.qL;
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const int c = 16 * t + 4 * g;
            f32x4 z = {0.f, 0.f, 0.f, 0.f};
            qf[t] = c < dh ? *reinterpret_cast<const f32x4 *>(qr + c) : z;
        }
    }

    f32x4 accO[NT];
#pragma unroll
    for (int d = 0; d < NT; d++)
        accO[d] = f32x4{0.f, 0.f, 0.f, 0.f};
    float rowMax = -INFINITY, rowSum = 0.f;              /* in units of log2: the scores are scaled by log2(e) */
    const float scale2 = p.scale * LOG2E;

    /* The keys of a block reach LDS in two halves, and the first product begins when the first half is there:
           keys of half 1 -> LDS | barrier | S1 = K1 Q^T | keys of half 2, values -> LDS | barrier | S2 = K2 Q^T |
           softmax of the block | O += P V
       At the start of the kernel every workgroup of the grid waits for its queries and keys at once, at the rate the
       memory delivers them: the second half of the first keys (and then the values) are asked for only when the
       first half has arrived, so that everybody's first halves travel first. The first barrier also says that every
       wave has finished the previous block's second half and its values, the second that every wave has finished
       this block's first half. (Measured against it at the benchmark shape: the softmax of one half between the
       MFMAs of the other half's products, 13.0 us where this order takes 12.8: the matrix pipe of a SIMD is kept busy
       by its two waves either way.) */
    constexpr int HJ = NJ / 2;           /* 16-key blocks per half */
    constexpr int HL = LOADS / 2;        /* staging steps per half */
    constexpr int PAIRS = HJ / 2;        /* the key fragments come from LDS two blocks of 16 keys at a time */
    constexpr int STEPS = NT * PAIRS;    /* steps of 8 MFMAs of a half's first product */
    static_assert(NJ % 4 == 0 && LOADS % 2 == 0, "two halves of pairs of 16-key blocks");

    for (int kb0 = 0; kb0 < lk; kb0 += KB) {
        const bool more = kb0 + KB < lk;
        const bool second = kb0 + 16 * HJ < lk;          /* the second half holds a key: else it is not multiplied */

#pragma unroll
        for (int s = 0; s < HL; s++)
            *reinterpret_cast<f32x4 *>(&Ks[sLdsK + s * RSTEP * KPK]) = kreg[s];
        __syncthreads();
        if (kb0 == 0) {
            load_k(0, HL, LOADS);
            load_v(0);
        }

        f32x4 accS[NJ];
#pragma unroll
        for (int j = 0; j < NJ; j++)
            accS[j] = f32x4{0.f, 0.f, 0.f, 0.f};
        /* a mask that moves 16 bytes at a time is asked for, half a block at a time, before the product begins and
           without a branch (keys past the end read the row's last ones and are overwritten below), so that its loads
           travel together and behind the product */
        const bool maskEarly = MK != nullptr && p.maskVec;
        f32x4 kf[2][2], mk[HJ];
        auto load_mask = [&](const int jb) {
            if (maskEarly) {
#pragma unroll
                for (int j = 0; j < HJ; j++) {
                    const int key = kb0 + 16 * (jb + j) + 4 * g;   /* lk is a multiple of 4 here: all four or none */
                    mk[j] = *reinterpret_cast<const f32x4 *>(MK + (key < lk ? key : lk - 4));
                }
            }
        };
        /* scale, mask and the end of the keys for the half that begins with block jb */
        auto scale_and_mask = [&](const int jb) {
            if (MK != nullptr) {
                if (p.maskVec) {
#pragma unroll
                    for (int j = jb; j < jb + HJ; j++)
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            accS[j][r] = fmaf(mk[j - jb][r], LOG2E, accS[j][r] * scale2);
                }
                else {
#pragma unroll
                    for (int j = jb; j < jb + HJ; j++)
#pragma unroll
                        for (int r = 0; r < 4; r++) {
                            int key = kb0 + 16 * j + 4 * g + r;
                            key = key < lk ? key : lk - 1;
                            accS[j][r] = fmaf(MK[key], LOG2E, accS[j][r] * scale2);
                        }
                }
            }
            else {
#pragma unroll
                for (int j = jb; j < jb + HJ; j++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        accS[j][r] *= scale2;
            }
            if (kb0 + KB > lk) {                               /* last, partial block: keys past the end count for nothing */
#pragma unroll
                for (int j = jb; j < jb + HJ; j++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (kb0 + 16 * j + 4 * g + r >= lk)
                            accS[j][r] = -INFINITY;
            }
        };
        /* ---- S^T = K Q^T for the half that begins with block jb; the key fragments of a step are asked for one step
           ahead (16 registers; the scheduling fences keep the compiler from fetching further ahead); the second half
           carries the first half's scale and mask behind its first step ---- */
        auto scores = [&](const int jb) {
#pragma unroll
            for (int i = 0; i < 2; i++)
                kf[0][i] = *reinterpret_cast<const f32x4 *>(&Ks[(16 * (jb + i) + m) * KPK + 4 * g]);
#pragma unroll
            for (int st = 0; st < STEPS; st++) {
                const int t = st / PAIRS, j0 = jb + 2 * (st % PAIRS);
                if (st + 1 < STEPS) {
                    const int t1 = (st + 1) / PAIRS, j1 = jb + 2 * ((st + 1) % PAIRS);
#pragma unroll
                    for (int i = 0; i < 2; i++)
                        kf[(st + 1) & 1][i] = *reinterpret_cast<const f32x4 *>(&Ks[(16 * (j1 + i) + m) * KPK + 16 * t1 + 4 * g]);
                }
                {
#pragma unroll
                    for (int e = 0; e < 4; e++)
#pragma unroll
                        for (int i = 0; i < 2; i++)
                            accS[j0 + i] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[st & 1][i][e], qf[t][e], accS[j0 + i], 0, 0, 0);
                }
                if (jb > 0 && st == 0) {
                    scale_and_mask(0);
                    load_mask(HJ);                           /* the first half has used its own */
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        load_mask(0);
        scores(0);

        /* ---- the second half of the keys and the values into LDS ---- */
#pragma unroll
        for (int s = HL; s < LOADS; s++)
            *reinterpret_cast<f32x4 *>(&Ks[sLdsK + s * RSTEP * KPK]) = kreg[s];
#pragma unroll
        for (int s = 0; s < LOADS; s++)
            *reinterpret_cast<f32x4 *>(&Vs[sLds + s * RSTEP * KP]) = vreg[s];
        __syncthreads();
        if (more)
            load_k(kb0 + KB, 0, LOADS);

        if (second)
            scores(HJ);
        else {
            scale_and_mask(0);
            load_mask(HJ);
        }
        if (more)
            load_v(kb0 + KB);
        scale_and_mask(HJ);

        /* ---- running softmax of this lane's query row ------------------------------------------------ */
        float mx = accS[0][0];
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                mx = fmaxf(mx, accS[j][r]);
        mx = lane_groups_max(mx);
        const float newMax = fmaxf(rowMax, mx);
        const float shift = newMax == -INFINITY ? 0.f : newMax;      /* a row with nothing to see yet */
        const float corr = __builtin_amdgcn_exp2f(rowMax - shift);     /* 2^-inf = 0 on the first block */
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float e = __builtin_amdgcn_exp2f(accS[j][r] - shift);
                accS[j][r] = e;
                sum += e;
            }
        rowSum = rowSum * corr + sum;                    /* this lane's keys only: the four lanes of a row meet at the end */
        rowMax = newMax;
#pragma unroll
        for (int d = 0; d < NT; d++)
            accO[d] *= corr;

        /* ---- O^T += V^T P^T: the probabilities are operands as they lie ---------------------------------- */
        float vf[2][4][NT];
#pragma unroll
        for (int r = 0; r < 4; r++)
#pragma unroll
            for (int d = 0; d < NT; d++)
                vf[0][r][d] = Vs[(4 * g + r) * KP + m + 16 * d];
        auto context = [&](const int jb) {
#pragma unroll
            for (int j = jb; j < jb + HJ; j++) {
                if (j + 1 < NJ) {
#pragma unroll
                    for (int r = 0; r < 4; r++)
#pragma unroll
                        for (int d = 0; d < NT; d++)
                            vf[(j + 1) & 1][r][d] = Vs[(16 * (j + 1) + 4 * g + r) * KP + m + 16 * d];
                }
#pragma unroll
                for (int r = 0; r < 4; r++)
#pragma unroll
                    for (int d = 0; d < NT; d++)
                        accO[d] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[j & 1][r][d], accS[j][r], accO[d], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        context(0);
        if (second)
            context(HJ);
    }

    /* ---- out = result / row sum: register r of block d is column 16 d + 4 g + r of the lane's row ---- */
    rowSum = lane_groups_sum(rowSum);
    if (row < lq) {
        const float inv = rowSum > 0.f ? 1.f / rowSum : 0.f;
        float * orow = O + (long long)row * p.oL;
#pragma unroll
        for (int d = 0; d < NT; d++) {
            const int c = 16 * d + 4 * g;
            if (c < dh)
                *reinterpret_cast<f32x4 *>(orow + c) = accO[d] * inv;
        }
    }
}

int launch_attention_f32(const AttnParams & p0, hipStream_t stream)
{
    AttnParams p = p0;
    p.qTiles = (p.lq + 63) / 64;
    p.maskVec = (p.mask != nullptr && p.lk % 4 == 0 && (reinterpret_cast<uintptr_t>(p.mask) & 15) == 0) ? 1 : 0;
    dim3 grid((unsigned)(p.heads * p.batch * p.qTiles));
    if (p.dh <= 16)
        hipLaunchKernelGGL((attention_f32_kernel<16, 128>), grid, dim3(256), 0, stream, p);
    else if (p.dh <= 32)
        hipLaunchKernelGGL((attention_f32_kernel<32, 128>), grid, dim3(256), 0, stream, p);
    else if (p.dh <= 64)
        hipLaunchKernelGGL((attention_f32_kernel<64, 128>), grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL((attention_f32_kernel<128, 64>), grid, dim3(256), 0, stream, p);
    return (int)hipGetLastError();
}

}  // namespace ntsamd
