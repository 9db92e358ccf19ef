/*
 * out = softmax(scale * Q K^T + mask) V per head, fp32, in one kernel for gfx950.
 *
 * Stands where the reference's attention runs a chain of operators
 * (source/sample/transformer/submodel/Attention.cpp:186-237): Split of q, k, v
 * into heads, Scale of q, BMMul(q, k^T), Sum with the mask, Softmax over the
 * last dimension, BMMul with v, Merge of the heads. Here the head split and
 * merge are strides, and the scores never leave the CU: per workgroup 128 query
 * rows of one (head, batch item), one wave per 32 rows; the keys stream through
 * LDS in blocks; row maxima and sums are carried along and the running result
 * is rescaled when a later block raises a row's maximum, so any number of keys
 * is handled with one pass over k and v.
 *
 * MFMA v_mfma_f32_32x32x2_f32 twice per key block:
 *   scores  = Q (rows x dh, fragments held in registers for the whole kernel)
 *             times the key block (K-contiguous rows in LDS),
 *   result += P (the wave's 32 x KB probabilities, turned through the wave's own
 *             piece of LDS from accumulator layout to operand layout) times the
 *             value block (rows of keys in LDS).
 * Accumulator register r of lane l is element (8*(r/4) + 4*(l/32) + r%4, l%32) of a
 * 32x32 block: a lane holds ONE key column of 16 rows, so a row's maximum and sum are
 * a butterfly over the 32 lanes of a half-wave, after which every lane of the half
 * knows them.
 */
#include "gemm_common.h"
#include "gemm_f32.h"

namespace ntsamd {

struct AttnParams {
    const float * q;
    const float * k;
    const float * v;
    const float * mask;                 /* NULL, or dense [heads][batch][lq][lk] added to the scaled scores */
    float * out;
    int heads, batch, lq, lk, dh;
    long long qH, qB, qL;               /* element strides: head, batch item, row (columns are contiguous) */
    long long kH, kB, kL;
    long long vH, vB, vL;
    long long oH, oB, oL;
    float scale;
    int qTiles;
};

__device__ __forceinline__ float half_wave_max(float x)
{
#pragma unroll
    for (int m = 1; m < 32; m <<= 1)
        x = fmaxf(x, __shfl_xor(x, m));
    return x;
}

__device__ __forceinline__ float half_wave_sum(float x)
{
#pragma unroll
    for (int m = 1; m < 32; m <<= 1)
        x += __shfl_xor(x, m);
    return x;
}

/* DHM: head size the kernel is built for (dh <= DHM, columns past dh are zero);
   KB: keys per block */
template <int DHM, int KB>
__global__ void __launch_bounds__(256, 1)
attention_f32_kernel(const AttnParams p)
{
    constexpr int KP = DHM + 4;          /* row pitch of the key and value blocks, floats */
    constexpr int PP = KB + 4;           /* row pitch of a wave's probabilities */
    constexpr int NQ = DHM / 8;          /* groups of four MFMA steps over dh */
    constexpr int NJ = KB / 32;          /* 32-key blocks of scores per wave */
    constexpr int NO = DHM / 32;         /* 32-column blocks of the result per wave */
    constexpr int LOADS = KB * DHM / 4 / 256;

    __shared__ __attribute__((aligned(16))) float Ks[KB * KP];
    __shared__ __attribute__((aligned(16))) float Vs[KB * KP];
    __shared__ __attribute__((aligned(16))) float Ps[4 * 32 * PP];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, lh = lane >> 5;

    const int qt = (int)blockIdx.x % p.qTiles;
    const int pair = (int)blockIdx.x / p.qTiles;
    const int h = pair / p.batch, b = pair - h * p.batch;
    const int lq = p.lq, lk = p.lk, dh = p.dh;

    const float * Q = p.q + h * p.qH + b * p.qB;
    const float * K = p.k + h * p.kH + b * p.kB;
    const float * V = p.v + h * p.vH + b * p.vB;
    float * O = p.out + h * p.oH + b * p.oB;
    const float * MK = p.mask ? p.mask + ((long long)pair * lq) * lk : nullptr;

    const int row0 = qt * 128 + wave * 32;          /* first query row of this wave */

    /* ---- Q fragments: lane (l32, lh) feeds row l32, k = 8 g + 4 lh + e of group g ---- */
    f32x4 qf[NQ];
    {
        int r = row0 + l32;
        r = r < lq ? r : lq - 1;                    /* rows past the end repeat the last one; never stored */
        const float * qr = Q + (long long)r * p.qL;
#pragma unroll
        for (int g = 0; g < NQ; g++) {
            const int c = 8 * g + 4 * lh;
            f32x4 z = {0.f, 0.f, 0.f, 0.f};
            qf[g] = c < dh ? *reinterpret_cast<const f32x4 *>(qr + c) : z;
        }
    }

    f32x16 accO[NO];
#pragma unroll
    for (int j = 0; j < NO; j++)
#pragma unroll
        for (int r = 0; r < 16; r++)
            accO[j][r] = 0.f;
    float rowMax[16], rowSum[16];
#pragma unroll
    for (int r = 0; r < 16; r++) {
        rowMax[r] = -INFINITY;
        rowSum[r] = 0.f;
    }

    float * myP = Ps + wave * 32 * PP;

    for (int kb0 = 0; kb0 < lk; kb0 += KB) {
        /* ---- key and value block into LDS: 16 bytes per thread and step; rows past lk and
           columns past dh are zero ------------------------------------------------------ */
        __syncthreads();                            /* the previous block is no longer read */
#pragma unroll
        for (int s = 0; s < LOADS; s++) {
            const int idx = tid + s * 256;
            const int row = idx / (DHM / 4), c = (idx % (DHM / 4)) * 4;
            const int key = kb0 + row;
            f32x4 kv = {0.f, 0.f, 0.f, 0.f}, vv = {0.f, 0.f, 0.f, 0.f};
            if (key < lk && c < dh) {
                kv = *reinterpret_cast<const f32x4 *>(K + (long long)key * p.kL + c);
                vv = *reinterpret_cast<const f32x4 *>(V + (long long)key * p.vL + c);
            }
            *reinterpret_cast<f32x4 *>(&Ks[row * KP + c]) = kv;
            *reinterpret_cast<f32x4 *>(&Vs[row * KP + c]) = vv;
        }
        __syncthreads();

        /* ---- scores of the wave's 32 rows against the block's keys ---------------------- */
        f32x16 accS[NJ];
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                accS[j][r] = 0.f;
#pragma unroll
        for (int g = 0; g < NQ; g++) {
            if (8 * g < dh) {
#pragma unroll
                for (int j = 0; j < NJ; j++) {
                    const f32x4 kf = *reinterpret_cast<const f32x4 *>(&Ks[(j * 32 + l32) * KP + 8 * g + 4 * lh]);
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        accS[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(qf[g][e], kf[e], accS[j], 0, 0, 0);
                }
            }
        }

        /* ---- scale and mask: the mask test sits outside the loops so that the loads are not
           fenced off one by one; rows and keys past the end read the last valid element ------ */
        if (MK != nullptr) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                int row = row0 + 8 * (r / 4) + 4 * lh + (r % 4);
                row = row < lq ? row : lq - 1;
#pragma unroll
                for (int j = 0; j < NJ; j++) {
                    int key = kb0 + j * 32 + l32;
                    key = key < lk ? key : lk - 1;
                    accS[j][r] = accS[j][r] * p.scale + MK[(long long)row * lk + key];
                }
            }
        }
        else {
#pragma unroll
            for (int r = 0; r < 16; r++)
#pragma unroll
                for (int j = 0; j < NJ; j++)
                    accS[j][r] *= p.scale;
        }

        /* ---- running softmax ------------------------------------------------------------------- */
#pragma unroll
        for (int r = 0; r < 16; r++) {
            float mx = -INFINITY;
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                const int key = kb0 + j * 32 + l32;
                const float s = key < lk ? accS[j][r] : -INFINITY;
                accS[j][r] = s;
                mx = fmaxf(mx, s);
            }
            mx = half_wave_max(mx);
            const float newMax = fmaxf(rowMax[r], mx);
            const float shift = newMax == -INFINITY ? 0.f : newMax;     /* a row with nothing to see yet */
            const float corr = expf(rowMax[r] - shift);               /* exp(-inf) = 0 on the first block */
            float sum = 0.f;
#pragma unroll
            for (int j = 0; j < NJ; j++) {
                const float e = expf(accS[j][r] - shift);
                accS[j][r] = e;
                sum += e;
            }
            sum = half_wave_sum(sum);
            rowSum[r] = rowSum[r] * corr + sum;
            rowMax[r] = newMax;
#pragma unroll
            for (int j = 0; j < NO; j++)
                accO[j][r] *= corr;
        }

        /* ---- probabilities: accumulator layout -> operand layout through the wave's LDS ------ */
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                myP[(8 * (r / 4) + 4 * lh + (r % 4)) * PP + j * 32 + l32] = accS[j][r];
        /* the wave's own lanes exchange data: LDS runs one wave's instructions in order, the
           fences keep the compiler from reordering */
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        /* ---- result += P times the value block ------------------------------------------------- */
#pragma unroll
        for (int g = 0; g < KB / 8; g++) {
            const f32x4 pf = *reinterpret_cast<const f32x4 *>(&myP[l32 * PP + 8 * g + 4 * lh]);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int kk = 8 * g + 4 * lh + e;
#pragma unroll
                for (int j = 0; j < NO; j++)
                    if (j * 32 < dh)
                        accO[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(pf[e], Vs[kk * KP + j * 32 + l32], accO[j], 0, 0, 0);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }

    /* ---- out = result / row sum; a lane stores one column of 16 rows: 128 contiguous bytes per row ---- */
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int row = row0 + 8 * (r / 4) + 4 * lh + (r % 4);
        if (row < lq) {
            const float inv = rowSum[r] > 0.f ? 1.f / rowSum[r] : 0.f;
            float * orow = O + (long long)row * p.oL;
#pragma unroll
            for (int j = 0; j < NO; j++) {
                const int col = j * 32 + l32;
                if (col < dh)
                    orow[col] = accO[j][r] * inv;
            }
        }
    }
}

int launch_attention_f32(const AttnParams & p0, hipStream_t stream)
{
    AttnParams p = p0;
    p.qTiles = (p.lq + 127) / 128;
    dim3 grid((unsigned)(p.heads * p.batch * p.qTiles));
    if (p.dh <= 64)
        hipLaunchKernelGGL((attention_f32_kernel<64, 128>), grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL((attention_f32_kernel<128, 64>), grid, dim3(256), 0, stream, p);
    return (int)hipGetLastError();
}

}  // namespace ntsamd
