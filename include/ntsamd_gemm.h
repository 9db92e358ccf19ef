/*
 * ntsamd_gemm.h - C ABI of the gfx950 (MI355X) matrix-multiplication library
 * for NiuTensor.
 *
 * These entry points stand where the reference's `USE_CUDA` branch calls
 * cuBLAS: each one receives exactly what the corresponding
 * `_CudaBLASMatrixMUL*` function of source/tensor/core/arithmetic/XTensorBLAS.h
 * receives, minus the cuBLAS handle, plus the device id and a stream.
 *
 * Conventions (all taken from the reference):
 *   - matrices are dense, row-major; na,ma / nb,mb / nc,mc are the STORED row
 *     and column counts, so lda = ma, ldb = mb, ldc = mc (XTensorBLAS.cu:64-71);
 *   - transposedA / transposedB use MATRIX_TRANS_TYPE values: X_TRANS = 0,
 *     X_NOTRANS = 1 (XDataType.h:36);
 *   - data types use TENSOR_DATA_TYPE values: X_FLOAT = 2, X_FLOAT16 = 3
 *     (XDataType.h:33). Supported triples (a, b, c): (X_FLOAT, X_FLOAT, X_FLOAT),
 *     (X_FLOAT16, X_FLOAT16, X_FLOAT16) and (X_FLOAT16, X_FLOAT16, X_FLOAT);
 *     anything else fails with "Unsupported data type!" (XTensorBLAS.cu:101-103).
 *     Beyond the reference: (X_FLOAT, X_FLOAT16, X_FLOAT16) and (X_FLOAT, X_FLOAT16,
 *     X_FLOAT) give the result of ConvertDataType(a, X_FLOAT16) followed by the half
 *     product, bit for bit, without the conversion pass or its temporary where the
 *     product is short (the probabilities of the half attention,
 *     source/sample/transformer/submodel/Attention.cpp:231-237): a is rounded to half,
 *     to nearest even, where the kernel fetches it. Long products round a once, into
 *     the stream's workspace, and run as all-half products (ntsamd_matrix_mul_static
 *     and ntsamd_matrix_mul_batched_grid never do: they always round in the fetch).
 *     Not offered by the pointer-list and column-sum entry points;
 *   - the result is c = alpha * op(a) * op(b) + beta * c. With beta == 0 the
 *     kernels never read c, so the caller does not have to zero it first (the
 *     reference calls SetZeroAll before every beta == 0 product,
 *     MatrixMul2D.cu:154-155; that pass is no longer needed);
 *   - alpha and beta arrive as float for every data type; half products
 *     accumulate in fp32;
 *   - c must not overlap a or b; all pointers are device pointers on `devID`.
 *
 * Every function returns 0 on success and a non-zero code on failure; the
 * message of the last failure on the calling thread is available from
 * ntsamd_last_error(). Nothing is thrown across this boundary. The library
 * restores the caller's current device before returning and issues its work
 * on `stream` (NULL = the default stream, which is what the reference uses)
 * without synchronising. Its only state beyond a per-device flag, and the only
 * device memory it allocates, is a 32 MiB workspace per device and stream for
 * products with few tiles and a long k, which are cut along k (partial
 * products in fp32, added up in a fixed order by a second kernel, so results
 * are the same bits on every run): allocated at the first such product on that
 * stream, kept until ntsamd_release_workspaces or the end of the process. At
 * most 64 workspaces are alive at a time; a stream that cannot have one (that
 * limit, or no memory) gets its products in one piece, float and half alike:
 * slower for those shapes, the same arithmetic as the single piece of any
 * other product.
 *
 * Threads and streams: every entry point may be called from any host thread.
 * Calls that use a workspace hold its lock from before their first launch
 * until after their last, so two host threads that issue to ONE stream (every
 * caller of the NULL stream does) get their kernels queued call by call and
 * cannot read each other's partial products. Launches on different streams
 * have different workspaces. Kernels recorded into a graph keep the workspace
 * of the stream they were captured on, so graphs captured on one stream and
 * that stream's own launches must not run concurrently; such a graph holds
 * the workspace's ADDRESS, so it must be destroyed (or captured again) once
 * ntsamd_release_workspaces has freed that workspace, and must not be replayed
 * afterwards. NTSAMD_SPLIT_K=1 in
 * the environment (read once, at the library's first call) keeps every product
 * in one piece and the library from allocating.
 */
#ifndef NTSAMD_GEMM_H
#define NTSAMD_GEMM_H

#ifdef __cplusplus
extern "C" {
#endif

#define NTSAMD_X_TRANS 0
#define NTSAMD_X_NOTRANS 1
#define NTSAMD_X_INT 0
#define NTSAMD_X_FLOAT 2
#define NTSAMD_X_FLOAT16 3

/* return codes */
#define NTSAMD_OK 0
#define NTSAMD_ERR_ARGUMENT 1     /* bad shape, pointer, flag or count */
#define NTSAMD_ERR_DATATYPE 2     /* "Unsupported data type!" */
#define NTSAMD_ERR_DEVICE 3       /* no such device, or not a gfx950 device */
#define NTSAMD_ERR_LAUNCH 4       /* the HIP runtime refused the launch */

/* bias broadcast of the fused epilogue */
#define NTSAMD_BIAS_NONE 0
#define NTSAMD_BIAS_COL 1         /* c[i][j] += bias[j]                      */
#define NTSAMD_BIAS_ROW 2         /* c[i][j] += bias[(i / rowDiv) % biasLen] */

/* function applied to every result element of ntsamd_matrix_mul_bias_act */
#define NTSAMD_ACT_NONE 0
#define NTSAMD_ACT_RECTIFY 1      /* y = x < 0 ? 0 : x */

/* Message of the last failure on this thread ("" if none). */
const char * ntsamd_last_error(void);

/* Library version, "major.minor". */
const char * ntsamd_version(void);

/* Checks that `devID` exists and is a gfx950 device and loads the kernels'
   code object on it. Optional: every entry point does this on first use.
   Takes the place of GDevs.GetCudaHandle(devID) (XDevice.cpp:207-224); there
   is no handle to create. */
int ntsamd_init(int devID);

/*
 * One product. Replaces
 *   _CudaBLASMatrixMUL(handle, a, transposedA, dataTypeA, b, transposedB, dataTypeB,
 *                      c, dataTypeC, na, ma, nb, mb, nc, mc, alpha, beta)
 * source/tensor/core/arithmetic/XTensorBLAS.h:36-40, XTensorBLAS.cu:38-104.
 */
int ntsamd_matrix_mul(int devID, void * stream,
                      const void * a, int transposedA, int dataTypeA,
                      const void * b, int transposedB, int dataTypeB,
                      void * c, int dataTypeC,
                      int na, int ma, int nb, int mb, int nc, int mc,
                      float alpha, float beta);

/*
 * One product with the bias add fused into the epilogue:
 *   c = alpha * op(a) * op(b) + beta * c + broadcast(bias).
 * Replaces the pair the reference's MulAndShift issues (MulAndShift.cpp:69,88):
 * _CudaBLASMatrixMUL into a temporary followed by _CudaSumDim
 * (SumDim.cu:120-211; KernelAddWithRow :43-64 is NTSAMD_BIAS_COL,
 * KernelAddWithCol :79-105 is NTSAMD_BIAS_ROW with rowDiv = the product of
 * the result's dimensions after the broadcast one, last excluded).
 * `bias` has the data type of c and `biasLen` elements; for NTSAMD_BIAS_COL
 * biasLen must equal mc.
 */
int ntsamd_matrix_mul_bias(int devID, void * stream,
                           const void * a, int transposedA, int dataTypeA,
                           const void * b, int transposedB, int dataTypeB,
                           void * c, int dataTypeC,
                           int na, int ma, int nb, int mb, int nc, int mc,
                           float alpha, float beta,
                           const void * bias, int biasMode, int biasLen, int biasRowDiv);

/*
 * The same with a function applied to the result on its way out:
 *   c = f(alpha * op(a) * op(b) + beta * c + broadcast(bias)).
 * NTSAMD_ACT_RECTIFY is the reference's Rectify (source/tensor/function/Rectify.cpp:34-56,
 * _CudaRectify Rectify.cu:39-83): the feed-forward block computes
 * Rectify(MulAndShift(input, w1, b1)) (source/sample/transformer/submodel/FFN.cpp:94), which
 * in the reference is the product, the broadcast add and then a third pass that reads and
 * writes the whole hidden activation once more. A negative zero and a NaN pass unchanged, as
 * in the reference's kernel (x < 0 is false for both).
 */
int ntsamd_matrix_mul_bias_act(int devID, void * stream,
                               const void * a, int transposedA, int dataTypeA,
                               const void * b, int transposedB, int dataTypeB,
                               void * c, int dataTypeC,
                               int na, int ma, int nb, int mb, int nc, int mc,
                               float alpha, float beta,
                               const void * bias, int biasMode, int biasLen, int biasRowDiv, int activation);

/*
 * One product that also returns the column sums of op(b), gathered from the
 * operand on its way through the kernel:
 *   c = alpha * op(a) * op(b) + beta * c
 *   colSum[j] = colSumBeta * colSum[j] + sum_k op(b)[k][j],   j < mc.
 * This is the weight-gradient step of a linear layer: for c = x * w + bias the
 * reference's GradMulAndShift (source/network/XBackwardMath.cpp:1774-1884)
 * computes dE/dw = x^T * dE/dc with _MatrixMul (:635-637 via :1857-1879) and
 * dE/dbias = column sums of dE/dc with _ReduceSum + _Sum into the gradient
 * (:1805-1810), two passes over dE/dc. Here op(b) = dE/dc is read once.
 * colSum has the data type of c and mc elements and must not overlap c.
 * (X_FLOAT16, X_FLOAT16, X_FLOAT) is not accepted here.
 */
int ntsamd_matrix_mul_colsum(int devID, void * stream,
                             const void * a, int transposedA, int dataTypeA,
                             const void * b, int transposedB, int dataTypeB,
                             void * c, int dataTypeC,
                             int na, int ma, int nb, int mb, int nc, int mc,
                             float alpha, float beta,
                             void * colSum, float colSumBeta);

/*
 * out[j] = beta * out[j] + sum_i sum_k in[i][j][k] over a dense [x][y][z]
 * tensor (z == 1: the column sums of an x by y matrix). Replaces what
 * GradMulAndShift does for the bias gradient when it is not a by-product of
 * the weight gradient (source/network/XBackwardMath.cpp:1793-1846):
 * _CudaReduceSum over the last dimension into a temporary, _CudaReduceSum
 * over the first into a second temporary, _CudaSum into the gradient
 * (source/tensor/core/reduce/ReduceSum.cu, core/arithmetic/Sum.cu). No
 * temporaries here. dataType is X_FLOAT or X_FLOAT16 for both tensors.
 */
int ntsamd_reduce_sum_xz(int devID, void * stream, const void * in, int dataType,
                         int x, int y, int z, void * out, float beta);

/*
 * `count` products over equally spaced matrices; strides are in ELEMENTS and
 * a stride of 0 shares one a or b among all products. Replaces
 *   _CudaBLASMatrixMULBatchedStrided(handle, a, transposedA, dataTypeA, strideA, ...)
 * source/tensor/core/arithmetic/XTensorBLAS.h:51-56, XTensorBLAS.cu:181-247.
 */
int ntsamd_matrix_mul_batched_strided(int devID, void * stream,
                                      const void * a, int transposedA, int dataTypeA, long long strideA,
                                      const void * b, int transposedB, int dataTypeB, long long strideB,
                                      void * c, int dataTypeC, long long strideC,
                                      int count, int na, int ma, int nb, int mb, int nc, int mc,
                                      float alpha, float beta);

/*
 * count0 x count1 products whose matrices stand inside larger tensors: item
 * (i0, i1), i0 < count0, i1 < count1, is the na x ma matrix whose rows are
 * lda >= ma elements apart and whose first element is a + i0 * strideA0 +
 * i1 * strideA1 (likewise b and c; strides in ELEMENTS, 0 shares an operand).
 * This is how the heads of a merged [batch, length, heads * width] tensor are
 * multiplied where they stand, and how the result is written in merged form:
 * it replaces _CudaBLASMatrixMULBatchedStrided (source/tensor/core/arithmetic/
 * XTensorBLAS.cu:181-247, where cuBLAS's lda/ldb/ldc are fixed to ma/mb/mc)
 * TOGETHER WITH the Split before it and the Merge after it, which copy
 * every tensor once (source/tensor/core/shape/Split.cpp:42-150, Merge.cpp:47-165;
 * used so in source/sample/transformer/submodel/Attention.cpp:197-201 and :241-242).
 * The result matrices may interleave but must not overlap.
 */
int ntsamd_matrix_mul_batched_grid(int devID, void * stream,
                                   const void * a, int transposedA, int dataTypeA, int lda,
                                   long long strideA0, long long strideA1,
                                   const void * b, int transposedB, int dataTypeB, int ldb,
                                   long long strideB0, long long strideB1,
                                   void * c, int dataTypeC, int ldc,
                                   long long strideC0, long long strideC1,
                                   int count0, int count1, int na, int ma, int nb, int mb, int nc, int mc,
                                   float alpha, float beta);

/*
 * `count` products over arbitrary same-shaped matrices. a, b and c are HOST
 * arrays of `count` DEVICE pointers. Replaces
 *   _CudaBLASMatrixMULBatched(handle, a, ..., count, na, ma, nb, mb, nc, mc, alpha, beta)
 * source/tensor/core/arithmetic/XTensorBLAS.h:43-48, XTensorBLAS.cu:109-178,
 * together with the staging the reference does before calling it
 * (XTensorBLAS.cu:315-368: three device arrays allocated, filled by cudaMemcpy,
 * freed afterwards). Here the pointers ride in the kernel arguments, so there
 * is no allocation and no copy.
 */
int ntsamd_matrix_mul_batched(int devID, void * stream,
                              const void * const * a, int transposedA, int dataTypeA,
                              const void * const * b, int transposedB, int dataTypeB,
                              void * const * c, int dataTypeC,
                              int count, int na, int ma, int nb, int mb, int nc, int mc,
                              float alpha, float beta);

/*
 * Attention for every head in one kernel:
 *   out[h][b] = softmax(scale * q[h][b] * k[h][b]^T + mask[h][b]) * v[h][b],   softmax over the keys.
 * Replaces the operator chain of the reference's Attention::MakeAttention in inference
 * (source/sample/transformer/submodel/Attention.cpp:186-237): Split of q, k and v into
 * heads (core/shape/Split.cpp), ScaleMe of q (:202-205), BMMul(q, X_NOTRANS, k, X_TRANS)
 * (:208-211), SumMe with the mask (:217-222), Softmax(att, -1) (:224, function/Softmax.cu),
 * BMMul(att, v) (:232-235) and Merge of the heads (:239, core/shape/Merge.cpp). The scores
 * are never written to memory, and the head split and merge are addressing:
 *   element (h, b, row, col) of q is q[h * strides[0] + b * strides[1] + row * strides[2] + col],
 *   likewise strides[3..5] for k, [6..8] for v, [9..11] for out (in elements).
 * For tensors stored [batch][rows][heads * dh], as before Split and after Merge, the strides
 * are (dh, rows * heads * dh, heads * dh); for tensors stored [heads][batch][rows][dh], as
 * after Split, they are (batch * rows * dh, rows * dh, dh).
 * q and out have lq rows, k and v have lk rows, every row has dh columns (at most 128).
 * mask is NULL or a dense X_FLOAT tensor [heads][batch][lq][lk] added to the scaled scores
 * (the reference's masks hold 0 and -1e9). dataType is the type of q, k, v and out:
 *   X_FLOAT    fp32 throughout; dh and the strides are multiples of 4.
 *   X_FLOAT16  half products with fp32 accumulation, the softmax in fp32 on the unrounded scores,
 *              probabilities and result rounded to half once each: the reference's half path
 *              (:216-218 scores converted to float for the mask and the softmax, :229-230 back to
 *              half) without its two conversion passes; dh and the strides are multiples of 8.
 * The training path of the reference applies dropout between the softmax and the second
 * product (:226-227) and keeps the probabilities for the backward step: it stays on the
 * batched-product entry points above.
 */
int ntsamd_attention(int devID, void * stream,
                     const void * q, const void * k, const void * v, const void * mask, void * out, int dataType,
                     int heads, int batch, int lq, int lk, int dh,
                     const long long * strides, float scale);

/*
 * The first half of the attention, for callers that need the probabilities themselves:
 *   probs[h][b] = softmax(scale * q[h][b] * k[h][b]^T + mask[h][b])   (dense [heads][batch][lq][lk], X_FLOAT).
 * Replaces Split of q and k, ScaleMe, BMMul(q, X_NOTRANS, k, X_TRANS), SumMe with the mask and Softmax(att, -1)
 * (source/sample/transformer/submodel/Attention.cpp:194-224) with one launch; the training path of the
 * reference goes on from here with Dropout and BMMul(att, v) (:226-235), and its backward step reads the
 * probabilities. strides[0..2] address q and strides[3..5] address k as in ntsamd_attention; dataType is
 * X_FLOAT; dh is a multiple of 4, at most 128.
 */
int ntsamd_attention_probs(int devID, void * stream,
                           const void * q, const void * k, const void * mask, void * probs, int dataType,
                           int heads, int batch, int lq, int lk, int dh,
                           const long long * strides, float scale);

/*
 * The attention of the reference's TRAINING path in one launch: the operator chain of Attention::MakeAttention with
 * isTraining set (source/sample/transformer/submodel/Attention.cpp:194-242): Split x3, Scale, BMMul(q, k^T), Sum with
 * the mask, Softmax, Dropout, BMMul with v, Merge. Dropout in the reference is a mask tensor of the probabilities'
 * shape, filled by the caller's random number generator with 0 and 1 / (1 - p), and an element-wise Multiply
 * (source/tensor/function/Dropout.cpp:148-162); the backward step reads the softmax's result and the product's
 * first operand, so both are written:
 *     probs   = softmax(scale q k^T + mask)     dense float [heads][batch][lq][lk], as ntsamd_attention_probs
 *     dropped = probs * dropMask                the same shape; written only if `dropped` is not NULL
 *     out     = (dropMask ? dropped : probs) v  laid out by strides[9..11], as ntsamd_attention
 * mask and dropMask may be NULL (no mask; no dropout, then `dropped` must be NULL too). q, k, v, out and strides
 * as for ntsamd_attention; X_FLOAT only (the reference converts half scores to float for its softmax, and its
 * dropout mask is a float tensor). Replaces, of this library's own entry points, ntsamd_attention_probs, the
 * caller's Multiply and ntsamd_matrix_mul_batched_grid: the probabilities cross memory twice instead of five times.
 */
int ntsamd_attention_train(int devID, void * stream,
                           const void * q, const void * k, const void * v, const void * mask, const void * dropMask,
                           void * probs, void * dropped, void * out, int dataType,
                           int heads, int batch, int lq, int lk, int dh,
                           const long long * strides, float scale);

/*
 * Element-wise data type conversion t[i] = (typeT) s[i], i < size.
 * Replaces _CudaConvertDataType(devID, s, typeS, t, typeT, size) and the tensor form
 * _CudaConvertDataType(input, output) (source/tensor/core/getandset/ConvertDataType.cu:78-99,
 * :106-137) with their kernels (:31-66):
 *   X_FLOAT -> X_FLOAT16  round to nearest even;  X_FLOAT16 -> X_FLOAT  exact;
 *   X_FLOAT -> X_INT      toward zero, saturating, NaN -> 0;  X_INT -> X_FLOAT  round to nearest even.
 * Equal types: nothing is done and nothing is copied, as in the reference (:81-82, :108-109).
 * Every other pair: NTSAMD_ERR_DATATYPE, "Unsupported data types for conversion!".
 * s and t must not overlap.
 */
int ntsamd_convert_data_type(int devID, void * stream, const void * s, int typeS, void * t, int typeT,
                             long long size);

/*
 * Frees the workspaces the library allocated on `devID` (every device if devID < 0): one of 32 MiB per stream on
 * which a product was ever cut along k. Waits for the device's work first; the next product that wants a
 * workspace allocates it again, most likely at another address. HIP graphs that recorded products which used a
 * workspace (products cut along k, a float a rounded once before a long half product, half operands copied with
 * padded rows) hold the old address: destroy or re-capture them around a release, never replay them after it
 * (they would read and write freed memory). Do not call this while any stream of the process is being captured:
 * hipFree is not allowed then. Has no counterpart among the reference's cuBLAS calls (cuBLAS keeps its own
 * workspace inside the handle, released by cublasDestroy, which the reference never calls: XDevice.cpp:100-108).
 */
int ntsamd_release_workspaces(int devID);

/*
 * ntsamd_matrix_mul for callers that cannot allocate: it calls no hipMalloc, no hipFree and no allocating
 * library routine, ever. HAS NO COUNTERPART IN THE REFERENCE; it is for code under HIP graph capture,
 * tight serving loops and harnesses that forbid allocation, where ntsamd_matrix_mul's first product cut along
 * k on a stream would allocate that stream's workspace. Same arguments, same result, same kernels; the partial
 * products of a k cut into pieces go to a static array in device memory of NTSAMD_STATIC_SCRATCH_BYTES, which
 * is part of the library's code object: every GPU the library runs on holds one copy from the moment the code
 * is loaded there until the process ends. ntsamd_init(devID) looks the array's address up and is the place to
 * do that before a capture begins; the product kernels themselves are separate code objects that the runtime
 * loads at their first launch, so a product of each kind that will be captured should have run once, eagerly,
 * before the capture (one warm-up call per data type and transpose pair).
 *   splits = 0           the library chooses, among the ways to cut k whose partial products fit the array
 *                        (one piece, and no scratch at all, for most shapes: see ntsamd_matrix_mul);
 *   splits = 2, 4, 8, 16 k is cut into that many pieces (fewer where rounding a piece up to whole slabs of 32
 *                        makes the last ones empty). NTSAMD_ERR_ARGUMENT, with the sizes in the message,
 *                        if splits x nc x mc x 4 bytes exceed NTSAMD_STATIC_SCRATCH_BYTES, if a piece would
 *                        be shorter than 128 (half) or 64 (float) values of k, if a row of an operand or of
 *                        c has 2097152 elements or more, or if a measurement knob (NTSAMD_TILE_CFG) holds
 *                        the product to a tile shape that has no kernel for pieces. Half operands of any
 *                        even address and row length, and a float a with a half b, can be cut.
 * All calls on one GPU share that GPU's array, on whatever stream: calls that may overlap on one GPU (different
 * streams, or graphs replayed side by side) race on it and must be ordered by the caller. The array keeps the
 * last call's partial products; every call overwrites all it reads, so nothing has to be cleared.
 */
#define NTSAMD_STATIC_SCRATCH_BYTES (16 << 20)
int ntsamd_matrix_mul_static(int devID, void * stream,
                             const void * a, int transposedA, int dataTypeA,
                             const void * b, int transposedB, int dataTypeB,
                             void * c, int dataTypeC,
                             int na, int ma, int nb, int mb, int nc, int mc,
                             float alpha, float beta, int splits);

#ifdef __cplusplus
}
#endif
#endif
