/*
 * Element-wise data type conversion for gfx950, standing where the reference runs
 * KernelFloatToFloat16 / KernelFloat16ToFloat / KernelFloatToInt / KernelIntToFloat
 * (source/tensor/core/getandset/ConvertDataType.cu:31-66, dispatched at :78-99 and
 * :106-137):
 *     float -> half   round to nearest even (what __float2half does)
 *     half  -> float  exact
 *     float -> int    toward zero; values beyond the int range saturate, NaN gives 0
 *                     (what a float-to-int cast does on the reference's GPU path)
 *     int   -> float  round to nearest even
 * Memory-bound: a lane moves 8 elements per step with 16- and 32-byte accesses when
 * both arrays are 16-byte aligned, and a grid of a few workgroups per CU strides over
 * the array so that every access of a wave is one contiguous run.
 */
#include "gemm_common.h"
#include "gemm_f16.h"       /* half_t */

namespace ntsamd {

template <typename S, typename T>
__device__ __forceinline__ T convert_one(S x)
{
    return (T)x;            /* float -> _Float16 is v_cvt_f16_f32 (RNE) */
}

/* the cast alone leaves values outside the int range undefined: spell the saturation out */
template <>
__device__ __forceinline__ int convert_one<float, int>(float x)
{
    if (x != x)
        return 0;
    if (x >= 2147483648.f)
        return 0x7fffffff;
    if (x <= -2147483648.f)
        return (int)0x80000000;
    return (int)x;
}

template <typename S, typename T>
__global__ void __launch_bounds__(256)
convert_kernel(const S * __restrict__ s, T * __restrict__ t, long long n, int vec)
{
    typedef S SV __attribute__((ext_vector_type(8)));
    typedef T TV __attribute__((ext_vector_type(8)));
    const long long tid = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long nthreads = (long long)gridDim.x * 256;
    long long done = 0;
    if (vec) {
        const long long groups = n / 8;
        for (long long i = tid; i < groups; i += nthreads) {
            const SV x = reinterpret_cast<const SV *>(s)[i];
            TV y;
#pragma unroll
            for (int e = 0; e < 8; e++)
                y[e] = convert_one<S, T>(x[e]);
            reinterpret_cast<TV *>(t)[i] = y;
        }
        done = groups * 8;
    }
    for (long long i = done + tid; i < n; i += nthreads)
        t[i] = convert_one<S, T>(s[i]);
}

template <typename S, typename T>
static int launch_convert_t(const void * s, void * t, long long n, hipStream_t stream)
{
    /* both arrays 16-byte aligned: 8 elements per lane and step (the wider of the two types moves 32 bytes) */
    const int vec = ((reinterpret_cast<uintptr_t>(s) | reinterpret_cast<uintptr_t>(t)) & 15) == 0 ? 1 : 0;
    long long work = vec ? (n + 7) / 8 : n;
    long long blocks = (work + 255) / 256;
    if (blocks > 256 * 8)
        blocks = 256 * 8;                       /* 8 workgroups per CU, each striding over the array */
    if (blocks < 1)
        blocks = 1;
    hipLaunchKernelGGL((convert_kernel<S, T>), dim3((unsigned)blocks), dim3(256), 0, stream,
                       static_cast<const S *>(s), static_cast<T *>(t), n, vec);
    return (int)hipGetLastError();
}

/* rows x cols halves whose rows stand srcPitch elements apart (any even address) copied to rows dstPitch apart
   (a multiple of 8, 16-byte aligned), the columns from cols to dstPitch filled with zeros: what lets a half operand
   with rows of odd length travel the 16-byte path afterwards. A lane moves one 16-byte piece of a destination row. */
__global__ void __launch_bounds__(256)
repitch_f16_kernel(const half_t * __restrict__ s, long long srcPitch, half_t * __restrict__ t, int dstPitch, long long rows, int cols)
{
    typedef half_t HV __attribute__((ext_vector_type(8)));
    const int perRow = dstPitch / 8;
    const long long pieces = rows * perRow;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < pieces; i += (long long)gridDim.x * 256) {
        const long long row = i / perRow;
        const int c = (int)(i - row * perRow) * 8;
        const half_t * src = s + row * srcPitch + c;
        HV v;
#pragma unroll
        for (int e = 0; e < 8; e++)
            v[e] = c + e < cols ? src[e] : (half_t)0.f;
        *reinterpret_cast<HV *>(t + row * dstPitch + c) = v;
    }
}

int launch_repitch_f16(const void * s, long long srcPitch, void * t, int dstPitch, long long rows, int cols, hipStream_t stream)
{
    long long blocks = (rows * (dstPitch / 8) + 255) / 256;
    if (blocks > 256 * 8)
        blocks = 256 * 8;
    if (blocks < 1)
        blocks = 1;
    hipLaunchKernelGGL(repitch_f16_kernel, dim3((unsigned)blocks), dim3(256), 0, stream,
                       static_cast<const half_t *>(s), srcPitch, static_cast<half_t *>(t), dstPitch, rows, cols);
    return (int)hipGetLastError();
}

/* kinds: 0 float -> half, 1 half -> float, 2 float -> int, 3 int -> float */
int launch_convert(int kind, const void * s, void * t, long long n, hipStream_t stream)
{
    switch (kind) {
    case 0: return launch_convert_t<float, half_t>(s, t, n, stream);
    case 1: return launch_convert_t<half_t, float>(s, t, n, stream);
    case 2: return launch_convert_t<float, int>(s, t, n, stream);
    default: return launch_convert_t<int, float>(s, t, n, stream);
    }
}

}  // namespace ntsamd
