/*
 * The attention of the reference's TRAINING path in one kernel, fp32, for gfx950
 * (source/sample/transformer/submodel/Attention.cpp:194-242 with isTraining set): Split of q, k, v into heads,
 * Scale of q, BMMul(q, k^T), Sum with the mask, Softmax, Dropout, BMMul with v, Merge of the heads. Dropout there
 * is a mask tensor of the probabilities' shape, filled with 0 and 1 / (1 - p) by the caller's random number
 * generator, and an element-wise Multiply (source/tensor/function/Dropout.cpp:148-162); the backward step needs the
 * softmax's result (its own gradient) and the product's first operand (the gradient of v), so both are tensors of
 * the graph. Here, per launch:
 *     probs   = softmax(scale q k^T + mask)          written once, [heads][batch][lq][lk]
 *     dropped = probs * dropMask                     written once if asked for (dropMask given)
 *     out     = dropped v  (probs v without a mask)  merged layout, as attention_f32.hip writes it
 * The scores never reach memory, the probabilities are not read back, the head split and merge are strides.
 * The training path otherwise takes three launches of this library (attention_probs_f32.hip, the caller's Multiply,
 * the product on merged tensors) and moves the probabilities five times instead of twice.
 *
 * Layout of the work and of both products: attention_f32.hip (64 query rows per workgroup, 16 per wave; S^T = K Q^T
 * and O^T = V^T P^T with v_mfma_f32_16x16x4_f32, lane (m, g) holds query m against keys 16 j + 4 g + r: four
 * neighbours of a row of probs, and exactly the operand the second product wants from that lane). The
 * probabilities leave normalised, so a row's maximum and sum must be final before its first probability is
 * written: with more keys than one block holds, a first pass over the keys finds them (the first product only) and
 * the second pass computes the scores again, as attention_probs_f32.hip does.
 */
#include "gemm_common.h"
#include "gemm_f32.h"
#include "attention.h"

namespace ntsamd {

template <int DHM, int KB>
__global__ void __launch_bounds__(256, 2)
attention_train_f32_kernel(const AttnParams p)
{
    constexpr int KP = DHM + 4;
    constexpr int KPK = DHM + 8;         /* the same for the keys: a 16-byte read takes lanes 0-7 and 16-23 together
                                            (rows m = 0..7, columns g = 0, 1), then 8-15 with 24-31 and so on: with a
                                            pitch of 2 mod 16 pieces of 16 bytes those sixteen lanes hit sixteen
                                            different pieces of the 256 bytes a cycle serves; with the pitch of the
                                            values every such read took two turns (counted: SQ_LDS_BANK_CONFLICT) */
    constexpr int NT = DHM / 16;
    constexpr int NJ = KB / 16;
    constexpr int LOADS = KB * DHM / 4 / 256;
    constexpr float LOG2E = 1.4426950408889634f;

    __shared__ __attribute__((aligned(16))) float Ks[KB * KPK];
    __shared__ __attribute__((aligned(16))) float Vs[KB * KP];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = lane & 15, g = lane >> 4;

    const int id = xcd_contiguous_id((int)blockIdx.x, (int)gridDim.x);
    const int qt = id % p.qTiles;
    const int pair = id / p.qTiles;
    const int h = pair / p.batch, b = pair - h * p.batch;
    const int lq = p.lq, lk = p.lk, dh = p.dh;

    const float * Q = static_cast<const float *>(p.q) + h * p.qH + b * p.qB;
    const float * K = static_cast<const float *>(p.k) + h * p.kH + b * p.kB;
    const float * V = static_cast<const float *>(p.v) + h * p.vH + b * p.vB;
    float * O = static_cast<float *>(p.out) + h * p.oH + b * p.oB;

    const int row = qt * 64 + wave * 16 + m;
    const int rowc = row < lq ? row : lq - 1;             /* rows past the end repeat the last one; never stored */
    /* where this lane's row begins in the four [heads][batch][lq][lk] tensors: one offset, added to whichever base
       (a scalar) is wanted at the time (four pointers per lane are eight registers the first product does not have) */
    const long long rowAt = ((long long)pair * lq + rowc) * lk;
    const float * const MK = p.mask;
    const float * const DM = p.dropMask;
    float * const PR = p.probs;
    float * const DR = p.dropped;

    /* ---- key / value staging, as in attention_f32.hip ---- */
    constexpr int TPR = DHM / 4;
    constexpr int RSTEP = 256 / TPR;
    const int sr0 = tid / TPR, sc = (tid % TPR) * 4;
    const int sLds = sr0 * KP + sc, sLdsK = sr0 * KPK + sc;
    const __amdgpu_buffer_rsrc_t kRsrc = make_rsrc(K, ((long long)(lk - 1) * p.kL + dh) * 4);
    const __amdgpu_buffer_rsrc_t vRsrc = make_rsrc(V, ((long long)(lk - 1) * p.vL + dh) * 4);
    const int kL4 = (int)p.kL * 4, vL4 = (int)p.vL * 4;
    const int kOff0 = sc < dh ? sr0 * kL4 + sc * 4 : NTSAMD_OOB_OFFSET;
    const int vOff0 = sc < dh ? sr0 * vL4 + sc * 4 : NTSAMD_OOB_OFFSET;
    f32x4 kreg[LOADS], vreg[LOADS];
    auto load_k = [&](int kb0) {
#pragma unroll
        for (int s = 0; s < LOADS; s++)
            kreg[s] = buffer_load_f32x4(kRsrc, sc < dh ? kOff0 + (kb0 + s * RSTEP) * kL4 : NTSAMD_OOB_OFFSET);
    };
    auto load_v = [&](int kb0) {
#pragma unroll
        for (int s = 0; s < LOADS; s++)
            vreg[s] = buffer_load_f32x4(vRsrc, sc < dh ? vOff0 + (kb0 + s * RSTEP) * vL4 : NTSAMD_OOB_OFFSET);
    };
    load_k(0);

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

    const float scale2 = p.scale * LOG2E;
    const bool oneBlock = lk <= KB;
    float rowMax = -INFINITY, rowSum = 0.f;              /* in units of log2: the scores are scaled by log2(e) */

    /* the scaled and masked scores (times log2 e) of this wave's rows against the block of keys in LDS */
    /* The key fragments come from LDS two blocks of 16 keys at a time, one step ahead of the eight products that
       use them: 16 registers, where fragments for a whole slice of the head dimension would be 64. What that frees
       holds the loads that travel behind this product: the first values (firstV) from its start, with them a mask
       that moves 16 bytes at a time, or else the dropout mask (dropMask); with such a mask the dropout mask follows
       from the start of the product's last slice. The mask is read without a branch (keys past the end read the
       row's last ones and are overwritten below), so that its loads travel together. */
    const bool maskEarly = MK != nullptr && p.maskVec;
    auto scores = [&](int kb0, f32x4 (&accS)[NJ], auto && firstV, auto && dropMask) {
        constexpr int PAIRS = NJ / 2, STEPS = NT * PAIRS;
#pragma unroll
        for (int j = 0; j < NJ; j++)
            accS[j] = f32x4{0.f, 0.f, 0.f, 0.f};
        f32x4 kf[2][2], mk[NJ];
        if (maskEarly) {
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                const int key = kb0 + 16 * j + 4 * g;
                mk[j] = *reinterpret_cast<const f32x4 *>(MK + rowAt + (key < lk ? key : lk - 4));
            }
        }
        firstV();
        if (!maskEarly)
            dropMask();
#pragma unroll
        for (int i = 0; i < 2; i++)
            kf[0][i] = *reinterpret_cast<const f32x4 *>(&Ks[(16 * i + m) * KPK + 4 * g]);
#pragma unroll
        for (int st = 0; st < STEPS; st++) {
            const int t = st / PAIRS, j0 = 2 * (st % PAIRS);
            if (st + 1 < STEPS) {
                const int t1 = (st + 1) / PAIRS, j1 = 2 * ((st + 1) % PAIRS);
#pragma unroll
                for (int i = 0; i < 2; i++)
                    kf[(st + 1) & 1][i] = *reinterpret_cast<const f32x4 *>(&Ks[(16 * (j1 + i) + m) * KPK + 16 * t1 + 4 * g]);
            }
            if (maskEarly && st == STEPS - PAIRS)
                dropMask();
#pragma unroll
            for (int e = 0; e < 4; e++)
#pragma unroll
                for (int i = 0; i < 2; i++)
                    accS[j0 + i] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[st & 1][i][e], qf[t][e], accS[j0 + i], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (MK != nullptr) {
            if (p.maskVec) {
#pragma unroll
                for (int j = 0; j < NJ; j++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        accS[j][r] = fmaf(mk[j][r], LOG2E, accS[j][r] * scale2);
            }
            else {
#pragma unroll
                for (int j = 0; j < NJ; j++)
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        int key = kb0 + 16 * j + 4 * g + r;
                        key = key < lk ? key : lk - 1;
                        accS[j][r] = fmaf(MK[rowAt + key], LOG2E, accS[j][r] * scale2);
                    }
            }
        }
        else {
#pragma unroll
            for (int j = 0; j < NJ; j++)
#pragma unroll
                for (int r = 0; r < 4; r++)
                    accS[j][r] *= scale2;
        }
        if (kb0 + KB > lk) {
#pragma unroll
            for (int j = 0; j < NJ; j++)
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (kb0 + 16 * j + 4 * g + r >= lk)
                        accS[j][r] = -INFINITY;
        }
    };
    /* a block's part in the row's maximum and sum */
    auto fold = [&](const f32x4 (&accS)[NJ]) {
        float mx = accS[0][0];
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                mx = fmaxf(mx, accS[j][r]);
        mx = lane_groups_max(mx);
        const float newMax = fmaxf(rowMax, mx);
        const float shift = newMax == -INFINITY ? 0.f : newMax;
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                sum += __builtin_amdgcn_exp2f(accS[j][r] - shift);
        sum = lane_groups_sum(sum);
        rowSum = rowSum * __builtin_amdgcn_exp2f(rowMax - shift) + sum;
        rowMax = newMax;
    };

    /* ---- more keys than one block holds: a first pass for every row's maximum and sum ---- */
    if (!oneBlock) {
        for (int kb0 = 0; kb0 < lk; kb0 += KB) {
#pragma unroll
            for (int s = 0; s < LOADS; s++)
                *reinterpret_cast<f32x4 *>(&Ks[sLdsK + s * RSTEP * KPK]) = kreg[s];
            __syncthreads();
            load_k(kb0 + KB < lk ? kb0 + KB : 0);            /* the next block, or the first again for the second pass */
            f32x4 accS[NJ];
            scores(kb0, accS, [] {}, [] {});
            fold(accS);
            __syncthreads();                                 /* every wave is done with this block of keys */
        }
    }

    /* ---- the pass that writes: probabilities out, dropout, second product ---- */
    f32x4 accO[NT];
#pragma unroll
    for (int d = 0; d < NT; d++)
        accO[d] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int kb0 = 0; kb0 < lk; kb0 += KB) {
        const bool more = kb0 + KB < lk;
#pragma unroll
        for (int s = 0; s < LOADS; s++)
            *reinterpret_cast<f32x4 *>(&Ks[sLdsK + s * RSTEP * KPK]) = kreg[s];
        __syncthreads();                                 /* also: every wave has finished the previous block's Vs */
        if (more)
            load_k(kb0 + KB);

        f32x4 accS[NJ], dm[NJ];
        scores(kb0, accS, [&] {
            if (kb0 == 0)
                load_v(0);
        }, [&] {
            if (DM == nullptr)
                return;
            if (p.probsVec) {                  /* (keys past the end: any finite value, their probabilities are 0) */
#pragma unroll
                for (int j = 0; j < NJ; j++) {
                    const int key = kb0 + 16 * j + 4 * g;
                    dm[j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(DM + rowAt + (key < lk ? key : lk - 4)));
                }
            }
            else {
#pragma unroll
                for (int j = 0; j < NJ; j++)
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const int key = kb0 + 16 * j + 4 * g + r;
                        dm[j][r] = DM[rowAt + (key < lk ? key : lk - 1)];
                    }
            }
        });
        if (oneBlock)
            fold(accS);
        const float shift = rowMax == -INFINITY ? 0.f : rowMax;
        const float inv = rowSum > 0.f ? 1.f / rowSum : 0.f;
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                accS[j][r] = __builtin_amdgcn_exp2f(accS[j][r] - shift) * inv;
        auto store = [&](float * base, const f32x4 (&val)[NJ]) {
            if (row >= lq)
                return;
            float * to = base + rowAt;
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                const int key = kb0 + 16 * j + 4 * g;
                if (p.probsVec) {
                    if (key < lk)
                        *reinterpret_cast<f32x4 *>(to + key) = val[j];
                }
                else {
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (key + r < lk)
                            to[key + r] = val[j][r];
                }
            }
        };
        store(PR, accS);
        if (DM != nullptr) {
#pragma unroll
            for (int j = 0; j < NJ; j++)
                accS[j] *= dm[j];
            if (DR != nullptr)
                store(DR, accS);
        }
        /* keys past the end of a partial block: their probabilities are exp2(-inf) = 0 and multiply rows of zeros */

        /* ---- values into LDS, second product (attention_f32.hip) ---- */
#pragma unroll
        for (int s = 0; s < LOADS; s++)
            *reinterpret_cast<f32x4 *>(&Vs[sLds + s * RSTEP * KP]) = vreg[s];
        __syncthreads();                                 /* also: every wave has finished this block's Ks */
        if (more)
            load_v(kb0 + KB);
        float vf[2][4][NT];
#pragma unroll
        for (int r = 0; r < 4; r++)
#pragma unroll
            for (int d = 0; d < NT; d++)
                vf[0][r][d] = Vs[(4 * g + r) * KP + m + 16 * d];
#pragma unroll
        for (int j = 0; j < NJ; j++) {
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
    }

    /* ---- the probabilities were normalised: the result is the sum itself ---- */
    if (row < lq) {
        float * orow = O + (long long)row * p.oL;
#pragma unroll
        for (int d = 0; d < NT; d++) {
            const int c = 16 * d + 4 * g;
            if (c < dh)
                *reinterpret_cast<f32x4 *>(orow + c) = accO[d];
        }
    }
}

int launch_attention_train_f32(const AttnParams & p0, hipStream_t stream)
{
    AttnParams p = p0;
    p.qTiles = (p.lq + 63) / 64;
    p.maskVec = (p.mask != nullptr && p.lk % 4 == 0 && (reinterpret_cast<uintptr_t>(p.mask) & 15) == 0) ? 1 : 0;
    /* probabilities, dropout mask and dropped probabilities move 16 bytes at a time if all of them can */
    p.probsVec = (p.lk % 4 == 0 && (reinterpret_cast<uintptr_t>(p.probs) & 15) == 0 &&
                  (reinterpret_cast<uintptr_t>(p.dropMask) & 15) == 0 && (reinterpret_cast<uintptr_t>(p.dropped) & 15) == 0) ? 1 : 0;
    dim3 grid((unsigned)(p.heads * p.batch * p.qTiles));
    /* at most 64 keys (short sentences): blocks of 64, so that no product multiplies 16-key blocks without a key */
    const bool few = p.lk <= 64;
    if (p.dh <= 16) {
        if (few)
            hipLaunchKernelGGL((attention_train_f32_kernel<16, 64>), grid, dim3(256), 0, stream, p);
        else
            hipLaunchKernelGGL((attention_train_f32_kernel<16, 128>), grid, dim3(256), 0, stream, p);
    }
    else if (p.dh <= 32) {
        if (few)
            hipLaunchKernelGGL((attention_train_f32_kernel<32, 64>), grid, dim3(256), 0, stream, p);
        else
            hipLaunchKernelGGL((attention_train_f32_kernel<32, 128>), grid, dim3(256), 0, stream, p);
    }
    else if (p.dh <= 64) {
        if (few)
            hipLaunchKernelGGL((attention_train_f32_kernel<64, 64>), grid, dim3(256), 0, stream, p);
        else
            hipLaunchKernelGGL((attention_train_f32_kernel<64, 128>), grid, dim3(256), 0, stream, p);
    }
    else
        hipLaunchKernelGGL((attention_train_f32_kernel<128, 64>), grid, dim3(256), 0, stream, p);
    return (int)hipGetLastError();
}

}  // namespace ntsamd
