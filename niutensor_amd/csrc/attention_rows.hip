/*
 * Attention for a handful of query rows per head (a decoding step: one new position against the
 * cached keys and values, source/sample/transformer/submodel/Attention.cpp:120-171 with the cache
 * of :143-160): out = softmax(scale q k^T + mask) v for lq <= 8.
 *
 * With so few rows the 64-row MFMA tiles of the one-kernel attention multiply padding (B = 128 x 8
 * heads, lk = 128, one row: 27 us in float where the keys and values take 8.4 us to read). Here
 * every key and value element is read once, 16 bytes per lane, and meets the query rows in the
 * vector ALU: one workgroup per (head, batch item); a group of LPR lanes covers one row of k
 * (then of v), the groups take the rows in turn. Scores and probabilities live in LDS.
 *   1. score[r][j] = scale * <q[r], k[j]> + mask: LPR lanes hold 4 columns each of
 *      the row of k and of every query row, multiply, and add up across the group.
 *   2. one wave per query row: maximum, exp2 of the scaled difference, sum (as in the MFMA
 *      kernels: exp(x) = exp2(x log2 e)); the probabilities stay unnormalised, 1 / sum beside them.
 *   3. out[r] = sum_j p[r][j] v[j] / sum: each group adds up the rows of v it takes, the groups'
 *      partial rows meet in LDS.
 * Float only: half tensors stay on the MFMA kernel, whose padding costs little at sixteen times the rate.
 */
#include "attention.h"
#include <stdint.h>

namespace ntsamd {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int ROWS_MAX = 8;         /* query rows per head this kernel takes */
constexpr int NT = 256;

template <typename T> struct Piece;                       /* what one lane moves: 16 bytes */
template <> struct Piece<float> {
    static constexpr int N = 4;
    static __device__ __forceinline__ void load(const float * p, float (&x)[8])
    {
        const f32x4 v = *reinterpret_cast<const f32x4 *>(p);
        for (int e = 0; e < 4; e++)
            x[e] = v[e];
    }
    static __device__ __forceinline__ void store(float * p, const float (&x)[8])
    {
        f32x4 v;
        for (int e = 0; e < 4; e++)
            v[e] = x[e];
        *reinterpret_cast<f32x4 *>(p) = v;
    }
};
/* LPR: lanes per row of k / v (a power of two, LPR * Piece::N >= dh) */
template <typename T, int LPR>
__global__ void __launch_bounds__(NT) attention_rows_kernel(const AttnParams p)
{
    constexpr int PN = Piece<T>::N;
    constexpr int G = NT / LPR;                      /* groups of lanes: rows of k in flight */
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int lq = p.lq, lk = p.lk, dh = p.dh;
    float * sc = smem;                               /* [lq][lk] scores, then unnormalised probabilities */
    float * inv = sc + lq * lk;                      /* [ROWS_MAX] 1 / sum */
    float * red = inv + ROWS_MAX;                    /* [G][lq][LPR * PN] partial result rows */

    const int h = (int)blockIdx.x / p.batch, b = (int)blockIdx.x - h * p.batch;
    const T * q = static_cast<const T *>(p.q) + h * p.qH + b * p.qB;
    const T * k = static_cast<const T *>(p.k) + h * p.kH + b * p.kB;
    const T * v = static_cast<const T *>(p.v) + h * p.vH + b * p.vB;
    T * out = static_cast<T *>(p.out) + h * p.oH + b * p.oB;
    const float * mask = p.mask ? p.mask + ((long long)h * p.batch + b) * lq * lk : nullptr;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int g = tid / LPR, lr = tid % LPR;
    const int col = lr * PN;
    const bool live = col < dh;                      /* dh is a multiple of PN: a lane has all of its columns or none */

    /* this lane's columns of every query row */
    float qr[ROWS_MAX][8];
#pragma unroll
    for (int r = 0; r < ROWS_MAX; r++) {
#pragma unroll
        for (int e = 0; e < 8; e++)
            qr[r][e] = 0.f;
        if (r < lq && live)
            Piece<T>::load(q + r * p.qL + col, qr[r]);
    }

    /* ---- 1. scores ------------------------------------------------------------------------ */
    for (int j0 = 0; j0 < lk; j0 += G) {
        const int j = j0 + g;
        float kv[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (j < lk && live)
            Piece<T>::load(k + j * p.kL + col, kv);
#pragma unroll
        for (int r = 0; r < ROWS_MAX; r++) {
            if (r < lq) {                            /* the same for the whole workgroup */
                float s = 0.f;
#pragma unroll
                for (int e = 0; e < PN; e++)
                    s += kv[e] * qr[r][e];
#pragma unroll
                for (int d = LPR / 2; d >= 1; d >>= 1)
                    s += __shfl_xor(s, d);
                if (lr == 0 && j < lk) {
                    s *= p.scale;
                    if (mask)
                        s += mask[r * lk + j];
                    sc[r * lk + j] = s;
                }
            }
        }
    }
    __syncthreads();

    /* ---- 2. softmax, one wave per row -------------------------------------------------------- */
    for (int r = wave; r < lq; r += NT / 64) {
        float m = -3.0e38f;
        for (int j = lane; j < lk; j += 64)
            m = fmaxf(m, sc[r * lk + j]);
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1)
            m = fmaxf(m, __shfl_xor(m, d));
        float sum = 0.f;
        for (int j = lane; j < lk; j += 64) {
            const float e = __builtin_amdgcn_exp2f((sc[r * lk + j] - m) * 1.4426950408889634f);
            sc[r * lk + j] = e;
            sum += e;
        }
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1)
            sum += __shfl_xor(sum, d);
        if (lane == 0)
            inv[r] = 1.f / sum;
    }
    __syncthreads();

    /* ---- 3. probabilities times v --------------------------------------------------------------- */
    float acc[ROWS_MAX][8];
#pragma unroll
    for (int r = 0; r < ROWS_MAX; r++)
#pragma unroll
        for (int e = 0; e < 8; e++)
            acc[r][e] = 0.f;
    for (int j0 = 0; j0 < lk; j0 += G) {
        const int j = j0 + g;
        if (j < lk && live) {
            float vv[8];
            Piece<T>::load(v + j * p.vL + col, vv);
#pragma unroll
            for (int r = 0; r < ROWS_MAX; r++)
                if (r < lq) {
                    const float pr = sc[r * lk + j];
#pragma unroll
                    for (int e = 0; e < PN; e++)
                        acc[r][e] += pr * vv[e];
                }
        }
    }
    constexpr int W = LPR * PN;                      /* columns a group covers */
#pragma unroll
    for (int r = 0; r < ROWS_MAX; r++)
        if (r < lq) {
#pragma unroll
            for (int e = 0; e < PN; e++)
                red[(g * lq + r) * W + col + e] = acc[r][e];
        }
    __syncthreads();
    /* one lane per 16 bytes of the result */
    for (int x = tid; x < lq * LPR; x += NT) {
        const int r = x / LPR, c = (x - r * LPR) * PN;
        if (c < dh) {
            float o[8];
#pragma unroll
            for (int e = 0; e < 8; e++)
                o[e] = 0.f;
            for (int gg = 0; gg < G; gg++)
#pragma unroll
                for (int e = 0; e < PN; e++)
                    o[e] += red[(gg * lq + r) * W + c + e];
#pragma unroll
            for (int e = 0; e < PN; e++)
                o[e] *= inv[r];
            Piece<T>::store(out + r * p.oL + c, o);
        }
    }
}

template <typename T, int LPR>
int launch_rows(const AttnParams & p, hipStream_t stream)
{
    constexpr int PN = Piece<T>::N;
    const size_t lds = ((size_t)p.lq * p.lk + ROWS_MAX + (size_t)(NT / LPR) * p.lq * LPR * PN) * sizeof(float);
    hipLaunchKernelGGL((attention_rows_kernel<T, LPR>), dim3((unsigned)(p.heads * p.batch)), dim3(NT), lds, stream, p);
    return (int)hipGetLastError();
}

}  // namespace

/* LDS the kernel would need, or 0 if the problem is not its kind */
size_t attention_rows_lds(const AttnParams & p, bool half)
{
    /* float only: in half the MFMA tiles of padding cost less than widening every element in the vector ALU
       (measured: 128 x 8 heads, 128 keys, one row: 8.0 us on the MFMA kernel, 11.4 us here) */
    if (p.lq > ROWS_MAX || half)
        return 0;
    const int pn = 4;
    int lpr = 4;
    while (lpr * pn < p.dh)
        lpr *= 2;
    return ((size_t)p.lq * p.lk + ROWS_MAX + (size_t)(NT / lpr) * p.lq * lpr * pn) * sizeof(float);
}

int launch_attention_rows(const AttnParams & p, bool half, hipStream_t stream)
{
    if (half)
        return (int)hipErrorInvalidValue;            /* not taken: attention_rows_lds says 0 for half */
    if (p.dh <= 16)
        return launch_rows<float, 4>(p, stream);
    if (p.dh <= 32)
        return launch_rows<float, 8>(p, stream);
    if (p.dh <= 64)
        return launch_rows<float, 16>(p, stream);
    return launch_rows<float, 32>(p, stream);
}

}  // namespace ntsamd
