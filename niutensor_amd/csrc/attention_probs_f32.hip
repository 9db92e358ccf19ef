/*
 * probs = softmax(scale * Q K^T + mask) per head, fp32, in one kernel for gfx950: the first half of the
 * attention, as far as the reference's training path shares it with inference
 * (source/sample/transformer/submodel/Attention.cpp:194-224): Split of q and k into heads, Scale of q,
 * BMMul(q, k^T), Sum with the mask, Softmax over the last dimension. The training path then applies
 * Dropout to the probabilities and multiplies them with v (:226-235), and its backward step needs them,
 * so they are the output here: a dense [heads][batch][lq][lk] tensor, written once. The scores never
 * reach memory and the head split of q and k is strides.
 *
 * Same layout of the work as attention_f32.hip (64 query rows per workgroup, 16 per wave, the product
 * computed transposed with v_mfma_f32_16x16x4_f32 so that lane (m, g) holds query m against keys
 * 16 j + 4 g + r: four neighbours of a row of probs, one 16-byte store). With more keys than one block
 * holds, a first pass over the keys finds every row's maximum and sum and a second pass computes the
 * scores again and writes them out normalised: twice the first product, still no intermediate tensor.
 */
#include "gemm_common.h"
#include "gemm_f32.h"
#include "attention.h"

namespace ntsamd {

template <int DHM, int KB>
__global__ void __launch_bounds__(256, 2)
attention_probs_f32_kernel(const AttnParams p)
{
    constexpr int KPK = DHM + 8;         /* row pitch of the key block in floats: a 16-byte read takes lanes 0-7 and 16-23 together
                                            (rows m = 0..7, columns g = 0, 1), then 8-15 with 24-31 and so on: with a
                                            pitch of 2 mod 16 pieces of 16 bytes those sixteen lanes hit sixteen
                                            different pieces of the 256 bytes a cycle serves; with a pitch of 1 mod 16
                                            pieces every such read took two turns (counted: SQ_LDS_BANK_CONFLICT) */
    constexpr int NT = DHM / 16;
    constexpr int NJ = KB / 16;
    constexpr int LOADS = KB * DHM / 4 / 256;
    constexpr float LOG2E = 1.4426950408889634f;

    __shared__ __attribute__((aligned(16))) float Ks[KB * KPK];

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

    const int row = qt * 64 + wave * 16 + m;
    const int rowc = row < lq ? row : lq - 1;
    const float * MK = p.mask ? p.mask + ((long long)pair * lq + rowc) * lk : nullptr;
    float * PR = static_cast<float *>(p.out) + ((long long)pair * lq + rowc) * lk;

    constexpr int TPR = DHM / 4;
    constexpr int RSTEP = 256 / TPR;
    const int sr0 = tid / TPR, sc = (tid % TPR) * 4;
    const int sLdsK = sr0 * KPK + sc;
    const __amdgpu_buffer_rsrc_t kRsrc = make_rsrc(K, ((long long)(lk - 1) * p.kL + dh) * 4);
    const int kL4 = (int)p.kL * 4;
    const int kOff0 = sc < dh ? sr0 * kL4 + sc * 4 : NTSAMD_OOB_OFFSET;
    f32x4 kreg[LOADS];
    auto load_k = [&](int kb0) {
#pragma unroll
        for (int s = 0; s < LOADS; s++)
            kreg[s] = buffer_load_f32x4(kRsrc, sc < dh ? kOff0 + (kb0 + s * RSTEP) * kL4 : NTSAMD_OOB_OFFSET);
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
    auto scores = [&](int kb0, f32x4 (&accS)[NJ]) {
#pragma unroll
        for (int j = 0; j < NJ; j++)
            accS[j] = f32x4{0.f, 0.f, 0.f, 0.f};
        /* The key fragments come from LDS two blocks of 16 keys at a time, one step ahead of the eight products
           that use them (16 registers, where fragments for a whole group would be 64). What that frees holds a mask
           that moves 16 bytes at a time, asked for before the product begins and without a branch (keys past the
           end read the row's last ones and are overwritten below), so that its loads travel together and behind
           the product. */
        constexpr int PAIRS = NJ / 2, STEPS = NT * PAIRS;
        const bool maskEarly = MK != nullptr && p.maskVec;
        f32x4 kf[2][2], mk[NJ];
        if (maskEarly) {
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                const int key = kb0 + 16 * j + 4 * g;
                mk[j] = *reinterpret_cast<const f32x4 *>(MK + (key < lk ? key : lk - 4));
            }
        }
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
                        accS[j][r] = fmaf(MK[key], LOG2E, accS[j][r] * scale2);
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

    /* probabilities of one block out to memory: four neighbours per register group */
    auto store = [&](int kb0, const f32x4 (&accS)[NJ], float shift, float inv) {
        if (row >= lq)
            return;
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const int key = kb0 + 16 * j + 4 * g;
            f32x4 pr;
#pragma unroll
            for (int r = 0; r < 4; r++)
                pr[r] = __builtin_amdgcn_exp2f(accS[j][r] - shift) * inv;
            if (p.probsVec) {
                if (key < lk)
                    *reinterpret_cast<f32x4 *>(PR + key) = pr;
            }
            else {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (key + r < lk)
                        PR[key + r] = pr[r];
            }
        }
    };

    /* ---- first pass: maximum and sum of every row ---- */
    for (int kb0 = 0; kb0 < lk; kb0 += KB) {
#pragma unroll
        for (int s = 0; s < LOADS; s++)
            *reinterpret_cast<f32x4 *>(&Ks[sLdsK + s * RSTEP * KPK]) = kreg[s];
        __syncthreads();
        /* the next block of this pass, or the first block again for the second pass */
        if (kb0 + KB < lk)
            load_k(kb0 + KB);
        else if (!oneBlock)
            load_k(0);

        f32x4 accS[NJ];
        scores(kb0, accS);
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
        if (oneBlock) {
            store(0, accS, shift, rowSum > 0.f ? 1.f / rowSum : 0.f);
            return;
        }
        __syncthreads();                                 /* every wave is done with this block of keys */
    }

    /* ---- second pass: the scores again, written out normalised ---- */
    const float shift = rowMax == -INFINITY ? 0.f : rowMax;
    const float inv = rowSum > 0.f ? 1.f / rowSum : 0.f;
    for (int kb0 = 0; kb0 < lk; kb0 += KB) {
#pragma unroll
        for (int s = 0; s < LOADS; s++)
            *reinterpret_cast<f32x4 *>(&Ks[sLdsK + s * RSTEP * KPK]) = kreg[s];
        __syncthreads();
        if (kb0 + KB < lk)
            load_k(kb0 + KB);
        f32x4 accS[NJ];
        scores(kb0, accS);
        store(kb0, accS, shift, inv);
        __syncthreads();
    }
}

int launch_attention_probs_f32(const AttnParams & p0, hipStream_t stream)
{
    AttnParams p = p0;
    p.qTiles = (p.lq + 63) / 64;
    p.maskVec = (p.mask != nullptr && p.lk % 4 == 0 && (reinterpret_cast<uintptr_t>(p.mask) & 15) == 0) ? 1 : 0;
    p.probsVec = (p.lk % 4 == 0 && (reinterpret_cast<uintptr_t>(p.out) & 15) == 0) ? 1 : 0;
    dim3 grid((unsigned)(p.heads * p.batch * p.qTiles));
    /* at most 64 keys (short sentences): blocks of 64, so that no product multiplies 16-key blocks without a key */
    const bool few = p.lk <= 64;
    if (p.dh <= 16) {
        if (few)
            hipLaunchKernelGGL((attention_probs_f32_kernel<16, 64>), grid, dim3(256), 0, stream, p);
        else
            hipLaunchKernelGGL((attention_probs_f32_kernel<16, 128>), grid, dim3(256), 0, stream, p);
    }
    else if (p.dh <= 32) {
        if (few)
            hipLaunchKernelGGL((attention_probs_f32_kernel<32, 64>), grid, dim3(256), 0, stream, p);
        else
            hipLaunchKernelGGL((attention_probs_f32_kernel<32, 128>), grid, dim3(256), 0, stream, p);
    }
    else if (p.dh <= 64) {
        if (few)
            hipLaunchKernelGGL((attention_probs_f32_kernel<64, 64>), grid, dim3(256), 0, stream, p);
        else
            hipLaunchKernelGGL((attention_probs_f32_kernel<64, 128>), grid, dim3(256), 0, stream, p);
    }
    else
        hipLaunchKernelGGL((attention_probs_f32_kernel<128, 64>), grid, dim3(256), 0, stream, p);
    return (int)hipGetLastError();
}

}  // namespace ntsamd
