/*
 * out = softmax(scale * Q K^T + mask) V per head for half tensors, in one kernel for gfx950:
 * half products with fp32 accumulation, the softmax in fp32, one rounding of the
 * probabilities to half before the second product and one of the result.
 *
 * Stands where the reference's attention, run with half tensors, issues
 * (source/sample/transformer/submodel/Attention.cpp:186-237) Split, ScaleMe,
 * BMMul(q, k^T) in half, ConvertDataType to float (:216-218), the mask add and the Softmax
 * in float, ConvertDataType back to half (:229-230), BMMul with v in half, Merge. The scores
 * stay in fp32 registers from the first product to the softmax (the reference rounds them to
 * half in between), so the two conversion passes and their tensors disappear.
 *
 * Same plan as the fp32 kernel (attention_f32.hip): 64 query rows of one (head, batch item)
 * per workgroup, 16 per wave; keys and values stream through LDS in blocks of 128; both
 * products are computed transposed so that the probabilities pass from accumulator to
 * operand inside a lane:
 *   S^T = K Q^T   v_mfma_f32_16x16x32_f16: lane (m, g) = (l%16, l/16) feeds key m / query m with the
 *                 eight columns 32 t + 8 g .. + 7 (one 16-byte read) and receives the scores of query m
 *                 against keys 16 j + 4 g + r, r = 0..3.
 *   O^T = V^T P^T v_mfma_f32_16x16x32_f16 over pairs of 16-key blocks: B wants eight k per lane: the four
 *                 scores above of either block, rounded to half. A wants V[key 16 j + 4 g + r][column m],
 *                 four values one LDS row apart per block: a transposing read (ds_read_b64_tr_b16) of the
 *                 4 x 16 block whose rows the lane groups 0-3, 4-7, 8-11, 12-15 of every 16 lanes point at.
 */
#include "gemm_common.h"
#include "gemm_f16.h"       /* half_t, make_rsrc, buffer_load_f16x8, lds_read_tr16 */
#include "attention.h"

namespace ntsamd {

/* DHM: head size the kernel is built for (dh <= DHM, a multiple of 8; columns past dh are zero).
   QR: blocks of 16 query rows per wave. With two, a key or value fragment that a wave reads from LDS feeds two MFMAs
   instead of one: every wave of a workgroup reads every key and every value of a block, and at long sequences those
   reads, not the matrix pipe, are what the kernel waits for (LDS busy 53 % of the kernel's cycles with one block per
   wave). A workgroup then takes 128 query rows, so short sequences, which need the workgroups, keep one block.
   Two blocks of query rows go with blocks of 64 keys: scores and probabilities of 2 x 128 keys at once spilled 37
   registers and ran slower than one block of rows; with 64 keys the kernel fits 168 registers, three waves to a SIMD
   (heads of 128: 242 registers, two waves, as with one block of rows). */
template <int DHM, int QR, int KB = (QR == 2 ? 64 : 128)>   /* KB: keys per block in LDS */
__global__ void __launch_bounds__(256, QR == 2 && DHM <= 64 ? 3 : 2)
attention_f16_kernel(const AttnParams p)
{
    constexpr int PITCH = DHM * 2 + 16;      /* bytes per LDS row: 16 mod 128, so 16-byte reads of consecutive rows
                                                walk through the banks */
    constexpr int NT = DHM / 32;             /* k steps of the first product */
    constexpr int ND = DHM / 16;             /* 16-column blocks of the result */
    constexpr int NJ = KB / 16;              /* 16-key blocks */
    constexpr int TPR = DHM / 8;             /* threads per row when staging (16 bytes each) */
    constexpr int RSTEP = 256 / TPR;
    constexpr int LOADS = KB / RSTEP;
    constexpr float LOG2E = 1.4426950408889634f;

    __shared__ __attribute__((aligned(16))) char Ks[KB * PITCH];
    __shared__ __attribute__((aligned(16))) char Vs[KB * PITCH];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m = lane & 15, g = lane >> 4;

    const int id = xcd_contiguous_id((int)blockIdx.x, (int)gridDim.x);
    const int qt = id % p.qTiles;
    const int pair = id / p.qTiles;
    const int h = pair / p.batch, b = pair - h * p.batch;
    const int lq = p.lq, lk = p.lk, dh = p.dh;

    const half_t * Q = static_cast<const half_t *>(p.q) + h * p.qH + b * p.qB;
    const half_t * K = static_cast<const half_t *>(p.k) + h * p.kH + b * p.kB;
    const half_t * V = static_cast<const half_t *>(p.v) + h * p.vH + b * p.vB;
    half_t * O = static_cast<half_t *>(p.out) + h * p.oH + b * p.oB;

    /* this lane's query rows, one per block of 16 */
    int row[QR];
    const float * MK[QR];
#pragma unroll
    for (int q = 0; q < QR; q++) {
        row[q] = qt * (64 * QR) + wave * (16 * QR) + 16 * q + m;
        const int rowc = row[q] < lq ? row[q] : lq - 1;
        MK[q] = p.mask ? p.mask + ((long long)pair * lq + rowc) * lk : nullptr;
    }
    const bool masked = p.mask != nullptr;

    /* ---- staging of keys and values, as in the fp32 kernel ---- */
    const int sr0 = tid / TPR, sc = (tid % TPR) * 8;
    const int sLds = sr0 * PITCH + sc * 2;
    const __amdgpu_buffer_rsrc_t kRsrc = make_rsrc(K, ((long long)(lk - 1) * p.kL + dh) * 2);
    const __amdgpu_buffer_rsrc_t vRsrc = make_rsrc(V, ((long long)(lk - 1) * p.vL + dh) * 2);
    const int kL2 = (int)p.kL * 2, vL2 = (int)p.vL * 2;
    const int kOff0 = sr0 * kL2 + sc * 2, vOff0 = sr0 * vL2 + sc * 2;
    f16x8 kreg[LOADS], vreg[LOADS];
    auto load_k = [&](int kb0) {
#pragma unroll
        for (int s = 0; s < LOADS; s++)
            kreg[s] = buffer_load_f16x8(kRsrc, sc < dh ? kOff0 + (kb0 + s * RSTEP) * kL2 : NTSAMD_OOB_OFFSET);
    };
    auto load_v = [&](int kb0) {
#pragma unroll
        for (int s = 0; s < LOADS; s++)
            vreg[s] = buffer_load_f16x8(vRsrc, sc < dh ? vOff0 + (kb0 + s * RSTEP) * vL2 : NTSAMD_OOB_OFFSET);
    };
    load_k(0);

    /* ---- Q fragments ---- */
    f16x8 qf[QR][NT];
#pragma unroll
    for (int q = 0; q < QR; q++) {
        const half_t * qr = Q + (long long)(row[q] < lq ? row[q] : lq - 1) * p.qL;
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const int c = 32 * t + 8 * g;
            f16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
            qf[q][t] = c < dh ? *reinterpret_cast<const f16x8 *>(qr + c) : z;
        }
    }

    f32x4 accO[QR][ND];
    float rowMax[QR], rowSum[QR];
#pragma unroll
    for (int q = 0; q < QR; q++) {
#pragma unroll
        for (int d = 0; d < ND; d++)
            accO[q][d] = f32x4{0.f, 0.f, 0.f, 0.f};
        rowMax[q] = -INFINITY;
        rowSum[q] = 0.f;
    }
    const float scale2 = p.scale * LOG2E;

    /* where this lane points for the transposing reads: row 4 g + (m / 4) of a 16-key block, columns 4 (m % 4) .. + 3 */
    const int trOff = (4 * g + (m >> 2)) * PITCH + (m & 3) * 8;

    for (int kb0 = 0; kb0 < lk; kb0 += KB) {
        const bool more = kb0 + KB < lk;

#pragma unroll
        for (int s = 0; s < LOADS; s++)
            *reinterpret_cast<f16x8 *>(&Ks[sLds + s * RSTEP * PITCH]) = kreg[s];
        __syncthreads();
        /* the first values are asked for only now: at the start every workgroup of the grid wants its keys and
           queries at once, and values queued among them would hold back the keys of the workgroups that start later */
        if (kb0 == 0)
            load_v(0);
        if (more)
            load_k(kb0 + KB);

        /* ---- S^T = K Q^T: a key fragment feeds the products of all of the lane's query rows ---- */
        f32x4 accS[QR][NJ];
#pragma unroll
        for (int q = 0; q < QR; q++)
#pragma unroll
            for (int j = 0; j < NJ; j++)
                accS[q][j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < NT; t++) {
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                const f16x8 kf = *reinterpret_cast<const f16x8 *>(&Ks[(16 * j + m) * PITCH + 64 * t + 16 * g]);
#pragma unroll
                for (int q = 0; q < QR; q++)
                    accS[q][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[q][t], accS[q][j], 0, 0, 0);
            }
        }

        f16x4 pf[QR][NJ];                                /* the probabilities as the second product's operand */
#pragma unroll
        for (int q = 0; q < QR; q++) {
            /* ---- scale and mask ---- */
            if (masked) {
                if (p.maskVec) {
#pragma unroll
                    for (int j = 0; j < NJ; j++) {
                        const int key = kb0 + 16 * j + 4 * g;
                        f32x4 z = {0.f, 0.f, 0.f, 0.f};
                        const f32x4 mk = key < lk ? *reinterpret_cast<const f32x4 *>(MK[q] + key) : z;
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            accS[q][j][r] = fmaf(mk[r], LOG2E, accS[q][j][r] * scale2);
                    }
                }
                else {
#pragma unroll
                    for (int j = 0; j < NJ; j++)
#pragma unroll
                        for (int r = 0; r < 4; r++) {
                            int key = kb0 + 16 * j + 4 * g + r;
                            key = key < lk ? key : lk - 1;
                            accS[q][j][r] = fmaf(MK[q][key], LOG2E, accS[q][j][r] * scale2);
                        }
                }
            }
            else {
#pragma unroll
                for (int j = 0; j < NJ; j++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        accS[q][j][r] *= scale2;
            }
            if (kb0 + KB > lk) {
#pragma unroll
                for (int j = 0; j < NJ; j++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (kb0 + 16 * j + 4 * g + r >= lk)
                            accS[q][j][r] = -INFINITY;
            }

            /* ---- running softmax of this lane's query row, in fp32 ---- */
            float mx = accS[q][0][0];
#pragma unroll
            for (int j = 0; j < NJ; j++)
#pragma unroll
                for (int r = 0; r < 4; r++)
                    mx = fmaxf(mx, accS[q][j][r]);
            mx = lane_groups_max(mx);
            const float newMax = fmaxf(rowMax[q], mx);
            const float shift = newMax == -INFINITY ? 0.f : newMax;
            const float corr = __builtin_amdgcn_exp2f(rowMax[q] - shift);
            float sum = 0.f;
#pragma unroll
            for (int j = 0; j < NJ; j++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const float e = __builtin_amdgcn_exp2f(accS[q][j][r] - shift);
                    sum += e;
                    pf[q][j][r] = (half_t)e;
                }
            rowSum[q] = rowSum[q] * corr + sum;          /* this lane's keys only: the four lanes of a row meet at the end */
            rowMax[q] = newMax;
#pragma unroll
            for (int d = 0; d < ND; d++)
                accO[q][d] *= corr;
        }

#pragma unroll
        for (int s = 0; s < LOADS; s++)
            *reinterpret_cast<f16x8 *>(&Vs[sLds + s * RSTEP * PITCH]) = vreg[s];
        __syncthreads();
        if (more)
            load_v(kb0 + KB);

        /* ---- O^T += V^T P^T, 32 keys per MFMA: the k index 8 g + e of v_mfma_f32_16x16x32_f16 stands for key
           4 g + e of the first 16-key block of a pair for e < 4 and for key 4 g + e - 4 of the second for e >= 4 (the
           order in which a sum runs over the keys is free), so a lane's operands are its two blocks' four
           probabilities and two transposing reads side by side. (The 16x16x16 form runs at half the rate.) A
           value fragment feeds the products of all of the lane's query rows. ---- */
#pragma unroll
        for (int j = 0; j < NJ; j += 2)
#pragma unroll
            for (int d = 0; d < ND; d++) {
                const f16x4 lo = lds_read_tr16(reinterpret_cast<const half_t *>(&Vs[16 * j * PITCH + trOff + 32 * d]));
                const f16x4 hi = lds_read_tr16(reinterpret_cast<const half_t *>(&Vs[16 * (j + 1) * PITCH + trOff + 32 * d]));
                const f16x8 vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
                for (int q = 0; q < QR; q++) {
                    const f16x8 pp = __builtin_shufflevector(pf[q][j], pf[q][j + 1], 0, 1, 2, 3, 4, 5, 6, 7);
                    accO[q][d] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, pp, accO[q][d], 0, 0, 0);
                }
            }
    }

    /* ---- out = result / row sum: register r of block d is column 16 d + 4 g + r of the lane's row ---- */
#pragma unroll
    for (int q = 0; q < QR; q++) {
        const float total = lane_groups_sum(rowSum[q]);
        if (row[q] < lq) {
            const float inv = total > 0.f ? 1.f / total : 0.f;
            half_t * orow = O + (long long)row[q] * p.oL;
#pragma unroll
            for (int d = 0; d < ND; d++) {
                const int c = 16 * d + 4 * g;
                if (c < dh) {
                    f16x4 o;
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        o[r] = (half_t)(accO[q][d][r] * inv);
                    *reinterpret_cast<f16x4 *>(orow + c) = o;
                }
            }
        }
    }
}

int launch_attention_f16(const AttnParams & p0, hipStream_t stream)
{
    AttnParams p = p0;
    p.maskVec = (p.mask != nullptr && p.lk % 4 == 0 && (reinterpret_cast<uintptr_t>(p.mask) & 15) == 0) ? 1 : 0;
    /* 128 query rows per workgroup (two blocks of 16 per wave) where that still leaves two workgroups for every CU
       of the part */
    const long long groups128 = (long long)p.heads * p.batch * ((p.lq + 127) / 128);
    const bool two = p.lq > 64 && groups128 >= 512;
    p.qTiles = two ? (p.lq + 127) / 128 : (p.lq + 63) / 64;
    dim3 grid((unsigned)(p.heads * p.batch * p.qTiles));
    if (two) {
        if (p.dh <= 32)
            hipLaunchKernelGGL((attention_f16_kernel<32, 2>), grid, dim3(256), 0, stream, p);
        else if (p.dh <= 64)
            hipLaunchKernelGGL((attention_f16_kernel<64, 2>), grid, dim3(256), 0, stream, p);
        else
            hipLaunchKernelGGL((attention_f16_kernel<128, 2>), grid, dim3(256), 0, stream, p);
    }
    else if (p.lk <= 64) {          /* short sentences: blocks of 64 keys, so that no product multiplies 16-key blocks without a key */
        if (p.dh <= 32)
            hipLaunchKernelGGL((attention_f16_kernel<32, 1, 64>), grid, dim3(256), 0, stream, p);
        else if (p.dh <= 64)
            hipLaunchKernelGGL((attention_f16_kernel<64, 1, 64>), grid, dim3(256), 0, stream, p);
        else
            hipLaunchKernelGGL((attention_f16_kernel<128, 1, 64>), grid, dim3(256), 0, stream, p);
    }
    else if (p.dh <= 32)
        hipLaunchKernelGGL((attention_f16_kernel<32, 1>), grid, dim3(256), 0, stream, p);
    else if (p.dh <= 64)
        hipLaunchKernelGGL((attention_f16_kernel<64, 1>), grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL((attention_f16_kernel<128, 1>), grid, dim3(256), 0, stream, p);
    return (int)hipGetLastError();
}

}  // namespace ntsamd
