/*
 * fp32 GEMM for gfx950: c = alpha * op(a) op(b) + beta * c (+ bias), fp32 MFMA.
 * Replaces the cublasSgemm / cublasSgemmStridedBatched / cublasSgemmBatched calls of
 * the reference (source/tensor/core/arithmetic/XTensorBLAS.cu:61-72,133-145,204-216).
 *
 * One workgroup computes a BM x BN tile of c; its WGM x WGN waves each own a
 * (BM/WGM) x (BN/WGN) sub-tile held as 32x32 accumulator blocks of
 * v_mfma_f32_32x32x2_f32. Both operands are staged through LDS in k-major
 * rows (S[k][mn]), so a wave's operand fetch is 32 consecutive floats per
 * half-wave whatever the transpose flags are; K-contiguous sources are
 * transposed on the way into LDS. Two LDS stages: global loads for slab t+1
 * are issued before the MFMA work on slab t and parked in registers.
 */
#pragma once
#include "gemm_common.h"

namespace ntsamd {

/* four elements (row, k..k+3) of a K-contiguous operand; zero beyond K */
template <bool VEC>
__device__ __forceinline__ f32x4 ld4_kcontig(const float * __restrict__ rowPtr, int k, int K)
{
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (VEC) {
        /* K % 4 == 0 here: the group is entirely inside or entirely outside */
        if (k < K)
            v = *reinterpret_cast<const f32x4 *>(rowPtr + k);
    }
    else {
#pragma unroll
        for (int e = 0; e < 4; e++)
            if (k + e < K)
                v[e] = rowPtr[k + e];
    }
    return v;
}

/* four elements (k, m..m+3) of an MN-contiguous operand; zero beyond K,
   indices beyond the matrix edge are clamped (those outputs are never stored) */
template <bool VEC>
__device__ __forceinline__ f32x4 ld4_mncontig(const float * __restrict__ base, int ld, int k, int K, int m, int M)
{
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (k < K) {
        const float * r = base + (size_t)k * ld;
        if (VEC) {
            /* M % 4 == 0 here */
            int mm = m < M - 4 ? m : M - 4;
            v = *reinterpret_cast<const f32x4 *>(r + mm);
        }
        else {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                int mm = m + e < M - 1 ? m + e : M - 1;
                v[e] = r[mm];
            }
        }
    }
    return v;
}

template <int BM, int BN, int BKT, int WGM, int WGN, bool AKC, bool BKC, bool VEC, typename PT>
__global__ void __launch_bounds__(WGM * WGN * 64)
gemm_f32_kernel(const GemmParams p, const PT tab)
{
    constexpr int NT = WGM * WGN * 64;
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int TI = WM / 32, TJ = WN / 32;
    /* K-contiguous sources are written to LDS one float at a time, four k-rows
       per lane; a row pitch of 2 mod 8 spreads those writes over all banks */
    constexpr int LDA = AKC ? BM + 2 : BM;
    constexpr int LDB = BKC ? BN + 2 : BN;
    constexpr int NA = BM * BKT / 4 / NT;
    constexpr int NB = BN * BKT / 4 / NT;
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be made of 32x32 blocks");
    static_assert((BM * BKT / 4) % NT == 0 && (BN * BKT / 4) % NT == 0, "loads must divide evenly");
    static_assert(BKT % 4 == 0, "slab depth");

    __shared__ __attribute__((aligned(16))) float As[2][BKT * LDA];
    __shared__ __attribute__((aligned(16))) float Bs[2][BKT * LDB];

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
        A = static_cast<const float *>(p.a) + (long long)tc.batch * p.strideA;
        B = static_cast<const float *>(p.b) + (long long)tc.batch * p.strideB;
        C = static_cast<float *>(p.c) + (long long)tc.batch * p.strideC;
    }

    const int M = p.M, N = p.N, K = p.K;
    const int m0 = tc.tm * BM, n0 = tc.tn * BN;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm0 = (wave / WGN) * WM, wn0 = (wave % WGN) * WN;
    const int l32 = lane & 31, lh = lane >> 5;

    /* per-thread staging slots */
    const float * aRow[NA];
    const float * bRow[NB];
    int aK[NA], aMN[NA], bK[NB], bMN[NB];
#pragma unroll
    for (int s = 0; s < NA; s++) {
        int g = tid + s * NT;
        if (AKC) {
            aMN[s] = g / (BKT / 4);
            aK[s] = (g % (BKT / 4)) * 4;
            int row = m0 + aMN[s];
            row = row < M - 1 ? row : M - 1;
            aRow[s] = A + (size_t)row * p.lda;
        }
        else {
            aK[s] = g / (BM / 4);
            aMN[s] = (g % (BM / 4)) * 4;
            aRow[s] = A;
        }
    }
#pragma unroll
    for (int s = 0; s < NB; s++) {
        int g = tid + s * NT;
        if (BKC) {
            bMN[s] = g / (BKT / 4);
            bK[s] = (g % (BKT / 4)) * 4;
            int row = n0 + bMN[s];
            row = row < N - 1 ? row : N - 1;
            bRow[s] = B + (size_t)row * p.ldb;
        }
        else {
            bK[s] = g / (BN / 4);
            bMN[s] = (g % (BN / 4)) * 4;
            bRow[s] = B;
        }
    }

    f32x4 ra[NA], rb[NB];

    auto load_global = [&](int k0) {
#pragma unroll
        for (int s = 0; s < NA; s++) {
            if (AKC)
                ra[s] = ld4_kcontig<VEC>(aRow[s], k0 + aK[s], K);
            else
                ra[s] = ld4_mncontig<VEC>(aRow[s], p.lda, k0 + aK[s], K, m0 + aMN[s], M);
        }
#pragma unroll
        for (int s = 0; s < NB; s++) {
            if (BKC)
                rb[s] = ld4_kcontig<VEC>(bRow[s], k0 + bK[s], K);
            else
                rb[s] = ld4_mncontig<VEC>(bRow[s], p.ldb, k0 + bK[s], K, n0 + bMN[s], N);
        }
    };

    auto store_lds = [&](int buf) {
#pragma unroll
        for (int s = 0; s < NA; s++) {
            if (AKC) {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    As[buf][(aK[s] + e) * LDA + aMN[s]] = ra[s][e];
            }
            else
                *reinterpret_cast<f32x4 *>(&As[buf][aK[s] * LDA + aMN[s]]) = ra[s];
        }
#pragma unroll
        for (int s = 0; s < NB; s++) {
            if (BKC) {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    Bs[buf][(bK[s] + e) * LDB + bMN[s]] = rb[s][e];
            }
            else
                *reinterpret_cast<f32x4 *>(&Bs[buf][bK[s] * LDB + bMN[s]]) = rb[s];
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

    const int nk = (K + BKT - 1) / BKT;
    if (nk > 0) {
        load_global(0);
        store_lds(0);
    }
    __syncthreads();

    for (int kt = 0; kt < nk; kt++) {
        const int buf = kt & 1;
        if (kt + 1 < nk)
            load_global((kt + 1) * BKT);

        const float * as = &As[buf][lh * LDA + wm0 + l32];
        const float * bs = &Bs[buf][lh * LDB + wn0 + l32];
#pragma unroll
        for (int kk = 0; kk < BKT / 2; kk++) {
            float af[TI], bf[TJ];
#pragma unroll
            for (int i = 0; i < TI; i++)
                af[i] = as[kk * 2 * LDA + i * 32];
#pragma unroll
            for (int j = 0; j < TJ; j++)
                bf[j] = bs[kk * 2 * LDB + j * 32];
#pragma unroll
            for (int i = 0; i < TI; i++)
#pragma unroll
                for (int j = 0; j < TJ; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bf[j], acc[i][j], 0, 0, 0);
        }

        if (kt + 1 < nk)
            store_lds(buf ^ 1);
        __syncthreads();
    }

    /* epilogue: accumulator register r of lane l is element
       (8*(r/4) + 4*(l/32) + r%4, l%32) of its 32x32 block, so a store covers
       two rows of 32 consecutive floats and needs no alignment of ldc */
    const float alpha = p.alpha, beta = p.beta;
    const float * __restrict__ bias = static_cast<const float *>(p.bias);
#pragma unroll
    for (int j = 0; j < TJ; j++) {
        const int col = n0 + wn0 + j * 32 + l32;
        if (col >= N)
            continue;
        float bcol = 0.f;
        if (p.biasMode == BIAS_COL)
            bcol = bias[col];
#pragma unroll
        for (int i = 0; i < TI; i++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = m0 + wm0 + i * 32 + 8 * (r / 4) + 4 * lh + (r % 4);
                if (row < M) {
                    float * cp = C + (size_t)row * p.ldc + col;
                    float v = alpha * acc[i][j][r];
                    if (beta != 0.f)
                        v += beta * (*cp);
                    if (p.biasMode == BIAS_ROW)
                        v += bias[(row / p.biasRowDiv) % p.biasLen];
                    else
                        v += bcol;
                    *cp = v;
                }
            }
        }
    }
}

template <int CFG, bool AKC, bool BKC, bool VEC, typename PT>
static int launch_f32_one(const GemmParams & p0, const PT & tab, hipStream_t stream)
{
    typedef TileShape<CFG> S;
    GemmParams p = p0;
    p.tilesM = (p.M + S::BM - 1) / S::BM;
    p.tilesN = (p.N + S::BN - 1) / S::BN;
    dim3 grid((unsigned)(p.tilesM * p.tilesN * p.batch));
    hipLaunchKernelGGL((gemm_f32_kernel<S::BM, S::BN, 16, S::WGM, S::WGN, AKC, BKC, VEC, PT>),
                       grid, dim3(S::WGM * S::WGN * 64), 0, stream, p, tab);
    return (int)hipGetLastError();
}

template <bool AKC, bool BKC>
static int launch_f32_trans(const GemmParams & p, const PtrBatch * ptrs, bool vec, int cfg, hipStream_t stream)
{
    NoPtrs none = {0};
    if (ptrs) {
        /* pointer lists are the rare path: one instantiation, element-wise loads */
        return launch_f32_one<CFG_64x64, AKC, BKC, false, PtrBatch>(p, *ptrs, stream);
    }
    if (!vec)
        return launch_f32_one<CFG_64x64, AKC, BKC, false, NoPtrs>(p, none, stream);
    if (cfg == CFG_128x128)
        return launch_f32_one<CFG_128x128, AKC, BKC, true, NoPtrs>(p, none, stream);
    return launch_f32_one<CFG_64x64, AKC, BKC, true, NoPtrs>(p, none, stream);
}

}  // namespace ntsamd
