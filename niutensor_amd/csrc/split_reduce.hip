/*
 * Second half of a half-precision product whose k range was cut into pieces (the weight gradients of
 * source/network/XBackwardMath.cpp:1160-1280 and the few-row products of a decoding step: few tiles of c, a long
 * k): the product kernel left `splits` partial results, each `batch` dense M x N fp32 matrices, one set after the
 * other; this kernel adds them up, in the order of the pieces (the same bits on every run), and does what the
 * product kernel's epilogue does in one piece:
 *     c = f(alpha * sum + bias[col] + beta * c)
 * on c's own leading dimension, batch strides and type. Memory-bound: splits x 4 bytes read per element.
 */
#include "gemm_common.h"
#include "gemm_f16.h"       /* half_t */
#include <type_traits>

namespace ntsamd {

namespace {

constexpr int SPLITS_MAX = 16;      /* the most pieces the dispatcher cuts k into */

/* V consecutive columns per thread: 4 where c's rows allow 16-byte (float) or 8-byte (half) accesses, else 1 */
template <typename OutT, int V>
__global__ void __launch_bounds__(256)
split_reduce_kernel(const GemmParams p)
{
    const int M = p.M, N = p.N;
    const int perRow = N / V;
    const long long total = (long long)p.batch * M * perRow;
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total)
        return;
    const int cg = (int)(idx % perRow);
    const long long rest = idx / perRow;
    const int row = (int)(rest % M), item = (int)(rest / M);
    const int col = cg * V;

    const size_t piece = (size_t)p.batch * M * N;
    const float * w = p.splitWork + ((size_t)item * M + row) * N + col;
    /* every piece's load is issued before the first sum waits: one trip to memory, not one per piece */
    float part[SPLITS_MAX][V];
#pragma unroll
    for (int s = 0; s < SPLITS_MAX; s++) {
        if (s < p.splits) {
            if constexpr (V == 4) {
                const float4 v = *reinterpret_cast<const float4 *>(w + s * piece);
                part[s][0] = v.x;
                part[s][1] = v.y;
                part[s][2] = v.z;
                part[s][3] = v.w;
            }
            else
                part[s][0] = w[s * piece];
        }
    }
    float sum[V];
#pragma unroll
    for (int e = 0; e < V; e++)
        sum[e] = 0.f;
#pragma unroll
    for (int s = 0; s < SPLITS_MAX; s++)
        if (s < p.splits) {
#pragma unroll
            for (int e = 0; e < V; e++)
                sum[e] += part[s][e];
        }

    OutT * c = static_cast<OutT *>(p.c) + batch_offset(item, p.batchInner, p.strideC, p.strideC1) + (size_t)row * p.ldc + col;
    const OutT * bias = static_cast<const OutT *>(p.bias);
    OutT out[V];
#pragma unroll
    for (int e = 0; e < V; e++) {
        float v = p.alpha * sum[e];
        if (p.biasMode == BIAS_COL)
            v += (float)bias[col + e];
        if (p.beta != 0.f)
            v += p.beta * (float)c[e];
        out[e] = (OutT)activate(v, p.act);
    }
    if constexpr (V == 4) {
        typedef OutT Vec __attribute__((ext_vector_type(4)));
        Vec o = {out[0], out[1], out[2], out[3]};
        *reinterpret_cast<Vec *>(c) = o;
    }
    else
        c[0] = out[0];
}

template <typename OutT>
int launch_typed(const GemmParams & p, hipStream_t stream)
{
    const bool wide = p.N % 4 == 0 && p.ldc % 4 == 0 && p.strideC % 4 == 0 && p.strideC1 % 4 == 0 &&
                      (reinterpret_cast<size_t>(p.c) & (4 * sizeof(OutT) - 1)) == 0 &&
                      (reinterpret_cast<size_t>(p.splitWork) & 15) == 0;
    if (p.splits > SPLITS_MAX)
        return (int)hipErrorInvalidValue;
    const long long total = (long long)p.batch * p.M * (wide ? p.N / 4 : p.N);
    const long long groups = (total + 255) / 256;
    if (groups > 0x7fffffffLL)
        return (int)hipErrorInvalidValue;
    if (wide)
        hipLaunchKernelGGL((split_reduce_kernel<OutT, 4>), dim3((unsigned)groups), dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL((split_reduce_kernel<OutT, 1>), dim3((unsigned)groups), dim3(256), 0, stream, p);
    return (int)hipGetLastError();
}

}  // namespace

int launch_split_reduce(const GemmParams & p, bool outF32, hipStream_t stream)
{
    return outF32 ? launch_typed<float>(p, stream) : launch_typed<half_t>(p, stream);
}

}  // namespace ntsamd
