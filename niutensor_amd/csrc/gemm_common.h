/*
 * Shared definitions of the gfx950 GEMM kernels: problem descriptor, vector
 * types, workgroup-to-tile mapping.
 *
 * All matrices are dense and row-major. A "K-contiguous" operand stores the
 * reduction index fastest (a with X_NOTRANS, b with X_TRANS); an
 * "MN-contiguous" operand stores the output index fastest (a with X_TRANS,
 * b with X_NOTRANS). The leading dimension is the stored column count in the
 * reference's BLAS calls (XTensorBLAS.cu:64-71: lda=ma, ldb=mb, ldc=mc); the kernels
 * take any leading dimension of at least that, which is how the heads of a merged
 * [batch, length, heads * width] tensor are multiplied where they stand.
 */
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ntsamd {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

/* Cache policy of the stores that write c through the fast epilogues (the last argument of the buffer store
   builtins: sc0 = 1, nt = 2, sc1 = 16). WRITE_THROUGH (sc0 sc1) sends the lines on to memory as they are written
   instead of leaving them dirty in the XCD's L2: a kernel that ends with its result dirty in L2 is followed by
   the write-back of all of it before the next kernel on the stream may start (measured: about 5 us after 67 MB
   of half results, 1.4 of 10.4 us on the attention-shaped batches), while lines written through leave during the
   kernel. Only for results whose rows are whole 128-byte lines: written through in pieces of lines (rows of
   30011 floats) the same stores were 4 % slower than the default. */
constexpr int STORE_DEFAULT = 0, STORE_WRITE_THROUGH = 17, STORE_STREAM = 2;      /* nt = 2: the line is the first to leave the cache again */

enum BiasMode { BIAS_NONE = 0, BIAS_COL = 1, BIAS_ROW = 2 };

/* applied to a result element on its way out: y = x < 0 ? 0 : x is the reference's Rectify
   (source/tensor/function/Rectify.cpp:47-55, Rectify.cu:39-49; a NaN stays a NaN) */
enum Activation { ACT_NONE = 0, ACT_RECTIFY = 1 };
__device__ __forceinline__ float activate(float v, int act)
{
    return (act == ACT_RECTIFY && v < 0.f) ? 0.f : v;
}

/* pointer-array batches travel in the kernel argument block: no device
   allocation, no host-to-device copy. One launch covers PTR_BATCH_MAX items. */
#define NTSAMD_PTR_BATCH_MAX 128
struct PtrBatch {
    const void * a[NTSAMD_PTR_BATCH_MAX];
    const void * b[NTSAMD_PTR_BATCH_MAX];
    void * c[NTSAMD_PTR_BATCH_MAX];
};
struct NoPtrs {
    char unused;
};

struct GemmParams {
    const void * a;
    const void * b;
    void * c;
    const void * bias;
    int M, N, K;
    int lda, ldb, ldc;
    long long strideA, strideB, strideC;   /* elements between batch items; 0 = shared operand */
    /* a batch laid out as a grid: item i stands at (i % batchInner) * stride + (i / batchInner) * stride1
       (heads of a [batch, length, heads * width] tensor, say). batchInner == 0: items `stride` apart. */
    int batchInner;
    long long strideA1, strideB1, strideC1;
    float alpha, beta;
    int biasMode;                          /* BiasMode */
    int biasRowDiv, biasLen;               /* BIAS_ROW: index = (row / biasRowDiv) % biasLen */
    int tilesM, tilesN;
    int batch;
    int groupM;                            /* tile rows that share a pass over the tile columns */
    /* column sums of op(b) in the same pass: colSum[j] = colSumBeta * colSum[j] + sum_k op(b)[k][j]
       (NULL = none); written by the workgroups of the first tile row */
    void * colSum;
    float colSumBeta;
    /* The k range is cut into `splits` pieces of kPerSplit (a multiple of every slab depth), one workgroup
       each; 1 = one workgroup per tile, plain stores. The pieces go to splitWork (splits x batch dense M x N
       fp32 matrices) as plain products, and launch_split_reduce adds them up in their order and writes c
       (fp16: 16-byte path, 64 x 64 and 128 x 128 tiles). fp32 with splitWork == NULL: the pieces ADD alpha *
       (their partial product) to c with atomics, in no fixed order, and the caller has already applied beta
       to c. */
    int splits, kPerSplit;
    float * splitWork;
    int act;                               /* Activation of the epilogue */
    int wideRowsOnly;                      /* fp32, measurements: no 16-row MFMAs for products of at most 16 rows */
    int f16Slab64;                         /* half, 64 x 64 tile on the LDS-direct path: slabs of 64 along k */
    int f16PingPong;                       /* half, 256 x 256 tile: the two wave groups run one phase apart */
    int storeHint;                         /* != 0: the fast epilogues write c through (STORE_WRITE_THROUGH) */
    int persistGrid;                       /* half, 256 x 256 tile: > 0 = that many workgroups walk over all tiles */
    int persistRows;                       /* rows of the tiles they walk over: 128 (a k-contiguous) or 256 */
    int aF32;                              /* half product whose a is stored as float: rounded to half on its way to LDS */
    /* half, 16-byte path: the number of columns a stored row of a / b really has (the operand's row length, rounded
       up to 8 where the operand is a re-pitched copy whose padding holds zeros) */
    int mOper, nOper;
};

/* The dispatcher hands consecutive workgroup ids to the 8 XCDs in turn, and
   every XCD has its own L2. Renumber so that each XCD works on one contiguous
   range of tiles and the operand panels those tiles share stay in that L2. */
__device__ __forceinline__ int xcd_contiguous_id(int id, int total)
{
    const int X = 8;
    int per = total / X, rem = total % X;
    int xcd = id % X, idx = id / X;
    return xcd * per + (xcd < rem ? xcd : rem) + idx;
}

/* first element of batch item `item` of an operand */
__device__ __forceinline__ long long batch_offset(int item, int inner, long long stride0, long long stride1)
{
    if (inner <= 0)
        return (long long)item * stride0;
    const int outer = item / inner;
    return (long long)(item - outer * inner) * stride0 + (long long)outer * stride1;
}

struct TileCoord {
    int batch, tm, tn, split;
};

/* the tile with number `raw` in the order workgroups are dispatched in (consecutive numbers go to the XCDs in turn) */
__device__ __forceinline__ TileCoord tile_of_id(const GemmParams & p, int raw)
{
    int perBatch = p.tilesM * p.tilesN;
    int perSplit = perBatch * p.batch;
    int id = xcd_contiguous_id(raw, perSplit * p.splits);
    TileCoord t;
    t.split = id / perSplit;
    id -= t.split * perSplit;
    t.batch = id / perBatch;
    int r = id - t.batch * perBatch;
    int perGroup = p.groupM * p.tilesN;
    int g = r / perGroup;
    int firstM = g * p.groupM;
    int gsz = p.tilesM - firstM < p.groupM ? p.tilesM - firstM : p.groupM;
    int q = r - g * perGroup;
    t.tm = firstM + q % gsz;
    t.tn = q / gsz;
    return t;
}

__device__ __forceinline__ TileCoord tile_of_workgroup(const GemmParams & p)
{
    return tile_of_id(p, (int)blockIdx.x);
}

/* tile shapes the dispatcher can pick from */
/* CFG_16x128 (float): the 32 x 128 tile's kernel on 16-row MFMAs, one workgroup per 16 rows of c */
enum TileCfg { CFG_128x128 = 0, CFG_64x64 = 1, CFG_256x256 = 2, CFG_32x128 = 3, CFG_16x128 = 4, CFG_COUNT = 5 };

/* BM x BN tile per workgroup of WGM x WGN waves; BKT32: slab depth of the fp32 kernel
   (small tiles serve small, latency-bound products: a deeper slab means fewer round trips
   to memory); MINW16: waves per SIMD the fp16 kernel is
   built for (its 256x256 tile keeps 256 accumulator registers per lane: one wave per SIMD) */
template <int CFG> struct TileShape;
template <> struct TileShape<CFG_128x128> { static constexpr int BM = 128, BN = 128, WGM = 2, WGN = 2, MINW16 = 2, BKT32 = 16; };
template <> struct TileShape<CFG_64x64> { static constexpr int BM = 64, BN = 64, WGM = 2, WGN = 2, MINW16 = 2, BKT32 = 32; };
/* fp32 only, for products with at most 32 rows (a decoding step): no rows of padding to multiply */
template <> struct TileShape<CFG_32x128> { static constexpr int BM = 32, BN = 128, WGM = 1, WGN = 4, MINW16 = 2, BKT32 = 32; };
template <> struct TileShape<CFG_256x256> { static constexpr int BM = 256, BN = 256, WGM = 2, WGN = 2, MINW16 = 1, BKT32 = 16; };

int launch_f32(const GemmParams & p, const PtrBatch * ptrs, bool aKContig, bool bKContig,
               bool vec, int cfg, hipStream_t stream);
/* vec: how a and b are fetched. F16_SCALAR: element by element, every bias mode; F16_DIRECT: 16 bytes per lane
   straight to LDS (16-byte aligned rows of whole 16-byte pieces); F16_STAGED: 16 bytes per lane through
   registers, any alignment and row length */
enum F16Fetch { F16_SCALAR = 0, F16_DIRECT = 1, F16_STAGED = 2 };
int launch_f16(const GemmParams & p, const PtrBatch * ptrs, bool aKContig, bool bKContig,
               int vec, bool outF32, int cfg, hipStream_t stream);
/* c = f(alpha * (sum of the p.splits partial products in p.splitWork) + bias + beta * c) */
int launch_split_reduce(const GemmParams & p, bool outF32, hipStream_t stream);

}  // namespace ntsamd
