/*
 * Sums over the outer and inner dimensions of a dense [X][Y][Z] tensor:
 *     out[y] = beta * out[y] + sum_x sum_z in[x][y][z]
 * which is what the bias gradient of MulAndShift needs
 * (source/network/XBackwardMath.cpp:1793-1846: _ReduceSum over the last
 * dimension, _ReduceSum over the first, _Sum into the gradient). With Z == 1
 * it is the column sum of an [X][Y] matrix. The matrix-multiplication kernels
 * produce the same column sums as a by-product when they can; these kernels
 * serve the shapes and layouts where they cannot. Also here: the scaling pass
 * that applies beta ahead of kernels that add to their result with atomics.
 * Memory-bound, fp32 accumulation for both data types. Float column sums over
 * many rows are cut into pieces of the rows: with a workspace the pieces leave
 * their sums there and split_reduce.hip adds them in their order (the same bits
 * on every run); without one they add to the result with atomics.
 */
#include "gemm_common.h"
#include "gemm_f16.h"       /* half_t */

namespace ntsamd {

/* Z == 1. A workgroup owns 64 columns and one piece of the rows: 16 threads side by side
   read 4 columns each (256 contiguous bytes of a row for fp32), 16 such rows per step. */
enum { SUM_WHOLE = 0, SUM_ATOMIC = 1, SUM_PIECE = 2 };   /* what a workgroup does with its sums */

/* WIDE: rows are whole groups of four columns and start on 4-column boundaries of memory (one load per thread and row) */
template <typename T, int MODE, bool WIDE = false>
__global__ void __launch_bounds__(256)
column_sum_kernel(const T * __restrict__ in, int X, int Y, int rowsPerPiece, T * __restrict__ out, float beta)
{
    __shared__ float part[16][64];
    const int cg = threadIdx.x & 15, rl = threadIdx.x >> 4;
    const int col0 = blockIdx.x * 64 + cg * 4;
    const int xBeg = blockIdx.y * rowsPerPiece;
    const int xEnd = xBeg + rowsPerPiece < X ? xBeg + rowsPerPiece : X;
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    if (WIDE && col0 + 3 < Y) {
        typedef T vec_t __attribute__((ext_vector_type(4)));
#pragma unroll 4
        for (int x = xBeg + rl; x < xEnd; x += 16) {
            const vec_t v = *reinterpret_cast<const vec_t *>(in + (size_t)x * Y + col0);
#pragma unroll
            for (int e = 0; e < 4; e++)
                s[e] += (float)v[e];
        }
    }
    else if (col0 + 3 < Y) {
#pragma unroll 4
        for (int x = xBeg + rl; x < xEnd; x += 16) {
            const T * rp = in + (size_t)x * Y + col0;
#pragma unroll
            for (int e = 0; e < 4; e++)
                s[e] += (float)rp[e];
        }
    }
    else {
        for (int x = xBeg + rl; x < xEnd; x += 16) {
            const T * rp = in + (size_t)x * Y + col0;
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (col0 + e < Y)
                    s[e] += (float)rp[e];
        }
    }
#pragma unroll
    for (int e = 0; e < 4; e++)
        part[rl][cg * 4 + e] = s[e];
    __syncthreads();
    if (threadIdx.x < 64) {
        float v = 0.f;
#pragma unroll
        for (int r = 0; r < 16; r++)
            v += part[r][threadIdx.x];
        const int col = blockIdx.x * 64 + threadIdx.x;
        if (col < Y) {
            if constexpr (MODE == SUM_ATOMIC)
                unsafeAtomicAdd(reinterpret_cast<float *>(out) + col, v);     /* beta already applied */
            else if constexpr (MODE == SUM_PIECE)
                reinterpret_cast<float *>(out)[(size_t)blockIdx.y * Y + col] = v;   /* out: pieces x Y partial sums */
            else
                out[col] = (T)(beta != 0.f ? beta * (float)out[col] + v : v);
        }
    }
}

/* any Z: one workgroup per y, its threads stride over the (x, z) pairs */
template <typename T>
__global__ void __launch_bounds__(256)
outer_inner_sum_kernel(const T * __restrict__ in, int X, int Y, int Z, T * __restrict__ out, float beta)
{
    __shared__ float part[256];
    const int y = blockIdx.x;
    const long long total = (long long)X * Z;
    float s = 0.f;
    for (long long e = threadIdx.x; e < total; e += 256) {
        const long long x = e / Z, z = e - x * Z;
        s += (float)in[(x * Y + y) * Z + z];
    }
    part[threadIdx.x] = s;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w)
            part[threadIdx.x] += part[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0)
        out[y] = (T)(beta != 0.f ? beta * (float)out[y] + part[0] : part[0]);
}

/* v[i] = beta * v[i] (beta == 0 stores zeros whatever v held) */
template <typename T>
__global__ void __launch_bounds__(256)
scale_kernel(T * __restrict__ v, long long n, float beta)
{
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i < n)
        v[i] = (T)(beta != 0.f ? beta * (float)v[i] : 0.f);
}

int launch_scale(bool half, void * v, long long n, float beta, hipStream_t stream)
{
    if (n <= 0 || beta == 1.f)
        return 0;
    dim3 grid((unsigned)((n + 255) / 256));
    if (half)
        hipLaunchKernelGGL(scale_kernel<half_t>, grid, dim3(256), 0, stream, static_cast<half_t *>(v), n, beta);
    else
        hipLaunchKernelGGL(scale_kernel<float>, grid, dim3(256), 0, stream, static_cast<float *>(v), n, beta);
    return (int)hipGetLastError();
}

/* c[row][col] = f(c[row][col] + bias[(row / div) % len]): the broadcast add along a dimension that is not the last,
   as a pass of its own behind the product, which is how the reference does it (_SumDim with KernelAddWithCol,
   source/tensor/core/arithmetic/SumDim.cu:79-105, called from MulAndShift.cpp:88); f is the activation */
template <typename T, int VEC>
__global__ void __launch_bounds__(256)
row_bias_kernel(T * __restrict__ c, int M, int colsV, int ldc, const T * __restrict__ bias, int div, int len, int act)
{
    /* a block is 64 pieces of VEC columns by 4 rows; rows beyond what the grid's second dimension holds are
       reached by striding */
    typedef T vec_t __attribute__((ext_vector_type(VEC)));
    const int col = blockIdx.x * 64 + (threadIdx.x & 63);
    if (col >= colsV)
        return;
    for (int row = blockIdx.y * 4 + (threadIdx.x >> 6); row < M; row += gridDim.y * 4) {
        const float bv = (float)bias[(row / div) % len];
        T * at = c + (long long)row * ldc + col * VEC;
        if constexpr (VEC == 1)
            *at = (T)activate((float)*at + bv, act);
        else {
            vec_t v = *reinterpret_cast<const vec_t *>(at);
#pragma unroll
            for (int e = 0; e < VEC; e++)
                v[e] = (T)activate((float)v[e] + bv, act);
            *reinterpret_cast<vec_t *>(at) = v;
        }
    }
}

template <typename T>
static void launch_row_bias_t(T * c, int M, int N, int ldc, const T * bias, int div, int len, int act, hipStream_t stream)
{
    constexpr int VEC = 16 / (int)sizeof(T);
    const bool wide = N % VEC == 0 && ldc % VEC == 0 && (reinterpret_cast<uintptr_t>(c) & 15) == 0;
    const int colsV = wide ? N / VEC : N;
    const int rowBlocks = (M + 3) / 4;
    dim3 grid((unsigned)((colsV + 63) / 64), (unsigned)(rowBlocks < 65535 ? rowBlocks : 65535));
    if (wide)
        hipLaunchKernelGGL((row_bias_kernel<T, VEC>), grid, dim3(256), 0, stream, c, M, colsV, ldc, bias, div, len, act);
    else
        hipLaunchKernelGGL((row_bias_kernel<T, 1>), grid, dim3(256), 0, stream, c, M, colsV, ldc, bias, div, len, act);
}

int launch_row_bias(bool half, void * c, int M, int N, int ldc, const void * bias, int div, int len, int act, hipStream_t stream)
{
    if (M <= 0 || N <= 0)
        return 0;
    if (half)
        launch_row_bias_t(static_cast<half_t *>(c), M, N, ldc, static_cast<const half_t *>(bias), div, len, act, stream);
    else
        launch_row_bias_t(static_cast<float *>(c), M, N, ldc, static_cast<const float *>(bias), div, len, act, stream);
    return (int)hipGetLastError();
}

/* work: NULL, or workFloats floats of device memory that this stream's launches may use until the call's last
   kernel has run */
int launch_reduce_sum_xz(bool half, const void * in, int X, int Y, int Z, void * out, float beta, hipStream_t stream,
                         float * work, size_t workFloats)
{
    if (Y <= 0)
        return 0;
    if (Z != 1) {
        if (half)
            hipLaunchKernelGGL(outer_inner_sum_kernel<half_t>, dim3((unsigned)Y), dim3(256), 0, stream,
                               static_cast<const half_t *>(in), X, Y, Z, static_cast<half_t *>(out), beta);
        else
            hipLaunchKernelGGL(outer_inner_sum_kernel<float>, dim3((unsigned)Y), dim3(256), 0, stream,
                               static_cast<const float *>(in), X, Y, Z, static_cast<float *>(out), beta);
        return (int)hipGetLastError();
    }
    const int colGroups = (Y + 63) / 64;
    /* enough pieces to give every CU a few workgroups, at least 64 rows each */
    int pieces = (1024 + colGroups - 1) / colGroups;
    if (pieces > (X + 63) / 64)
        pieces = (X + 63) / 64;
    const bool wide = Y % 4 == 0 && (reinterpret_cast<uintptr_t>(in) & (half ? 7 : 15)) == 0;
    if (work != NULL && pieces > 1 && (size_t)Y * 2 <= workFloats) {
        /* the pieces meet in the workspace as fp32 and are added in their order; a half result is rounded once,
           from the fp32 total */
        const int most = (size_t)Y * 16 <= workFloats ? 16 : (int)(workFloats / (size_t)Y);
        if (pieces > most)
            pieces = most;
        const int rows = (X + pieces - 1) / pieces;
        pieces = (X + rows - 1) / rows;
        const dim3 grid((unsigned)colGroups, (unsigned)pieces);
        if (half && wide)
            hipLaunchKernelGGL((column_sum_kernel<half_t, SUM_PIECE, true>), grid, dim3(256), 0, stream,
                               static_cast<const half_t *>(in), X, Y, rows, reinterpret_cast<half_t *>(work), 1.f);
        else if (half)
            hipLaunchKernelGGL((column_sum_kernel<half_t, SUM_PIECE>), grid, dim3(256), 0, stream,
                               static_cast<const half_t *>(in), X, Y, rows, reinterpret_cast<half_t *>(work), 1.f);
        else if (wide)
            hipLaunchKernelGGL((column_sum_kernel<float, SUM_PIECE, true>), grid, dim3(256), 0, stream,
                               static_cast<const float *>(in), X, Y, rows, reinterpret_cast<float *>(work), 1.f);
        else
            hipLaunchKernelGGL((column_sum_kernel<float, SUM_PIECE>), grid, dim3(256), 0, stream,
                               static_cast<const float *>(in), X, Y, rows, reinterpret_cast<float *>(work), 1.f);
        int rc = (int)hipGetLastError();
        if (rc != 0)
            return rc;
        GemmParams p = {};
        p.c = out;
        p.M = 1;
        p.N = Y;
        p.ldc = Y;
        p.batch = 1;
        p.alpha = 1.f;
        p.beta = beta;
        p.splits = pieces;
        p.splitWork = work;
        return launch_split_reduce(p, !half, stream);
    }
    if (half || pieces <= 1) {
        /* one piece (half without a workspace: the sums are rounded once, from the fp32 total) */
        const dim3 grid((unsigned)colGroups, 1);
        if (half && wide)
            hipLaunchKernelGGL((column_sum_kernel<half_t, SUM_WHOLE, true>), grid, dim3(256), 0, stream,
                               static_cast<const half_t *>(in), X, Y, X > 0 ? X : 1, static_cast<half_t *>(out), beta);
        else if (half)
            hipLaunchKernelGGL((column_sum_kernel<half_t, SUM_WHOLE>), grid, dim3(256), 0, stream,
                               static_cast<const half_t *>(in), X, Y, X > 0 ? X : 1, static_cast<half_t *>(out), beta);
        else if (wide)
            hipLaunchKernelGGL((column_sum_kernel<float, SUM_WHOLE, true>), grid, dim3(256), 0, stream,
                               static_cast<const float *>(in), X, Y, X > 0 ? X : 1, static_cast<float *>(out), beta);
        else
            hipLaunchKernelGGL((column_sum_kernel<float, SUM_WHOLE>), grid, dim3(256), 0, stream,
                               static_cast<const float *>(in), X, Y, X > 0 ? X : 1, static_cast<float *>(out), beta);
        return (int)hipGetLastError();
    }
    int rc = launch_scale(false, out, Y, beta, stream);
    if (rc != 0)
        return rc;
    const int rowsPerPiece = (X + pieces - 1) / pieces;
    pieces = (X + rowsPerPiece - 1) / rowsPerPiece;
    hipLaunchKernelGGL((column_sum_kernel<float, SUM_ATOMIC>), dim3((unsigned)colGroups, (unsigned)pieces), dim3(256), 0, stream,
                       static_cast<const float *>(in), X, Y, rowsPerPiece, static_cast<float *>(out), 1.f);
    return (int)hipGetLastError();
}

}  // namespace ntsamd
