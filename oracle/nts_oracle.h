/*
 * TEST INFRASTRUCTURE - not part of the shipped library.
 *
 * CPU restatement of the NiuTensor matrix-multiplication family, used only as
 * the checker for the gfx950 kernels (tests, smoke check, CPU baseline timing).
 * Nothing in the product library may include or link this.
 *
 * Every function names the reference source (relative to the NiuTensor tree)
 * whose arithmetic and loop order it follows.
 */
#ifndef NTS_ORACLE_H
#define NTS_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* enum values of the reference, source/tensor/XDataType.h:33,36 */
#define ORACLE_X_TRANS 0
#define ORACLE_X_NOTRANS 1
#define ORACLE_X_FLOAT 2
#define ORACLE_X_FLOAT16 3

/* 2-D: c = op(a) op(b) alpha + c beta, fp32, single accumulator, ascending k.
   na,ma / nb,mb / nc,mc are the STORED row and column counts.
   Follows MatrixMul2DParallel.cpp:43-129 (TN, NT, TT) and the FAST_MATRIX
   branch of MatrixMul2DMultiTheading.cpp:59-145 (NN).
   Returns 0, or -1 when the shapes do not match (MatrixMul2D.cpp:56-67). */
int oracle_matmul2d(const float *a, int transA, const float *b, int transB, float *c,
                    int na, int ma, int nb, int mb, int nc, int mc,
                    float alpha, float beta);

/* Same-order batched product, block i of a times block i of b.
   Follows MatrixMulBatched.cpp:157-218. dims arrays hold `order` sizes each. */
int oracle_matmul_batched(const float *a, int transA, const int *aDims,
                          const float *b, int transB, const int *bDims,
                          float *c, const int *cDims, int order,
                          float alpha, float beta);

/* N-D product: flatten rule and (p,q) block pairing of MatrixMul.cpp:52-208. */
int oracle_matmul(const float *a, int transA, const int *aDims, int aOrder,
                  const float *b, int transB, const int *bDims, int bOrder,
                  float *c, const int *cDims, int cOrder,
                  float alpha, float beta);

/* Sum.cpp:233-260 */
int oracle_broadcast_dim_index(const int *aDims, int aOrder, const int *bDims, int bOrder);

/* c = a + b*beta, b broadcast along dimension n. CPU branch of SumDim.cpp:49-126. */
int oracle_sumdim(const float *a, const int *aDims, int aOrder,
                  const float *b, int bUnitNum, float *c, int n, float beta);

/* c = alpha * op(x) op(w) + bias; MulAndShift.cpp:38-110 and :120-188.
   cDims/cOrder are outputs (cDims must hold 8 ints). Returns the broadcast
   dimension n (>=0), or a negative value where the reference aborts. */
int oracle_mulandshift(const float *x, int transX, const int *xDims, int xOrder,
                       const float *w, int transW, const int *wDims, int wOrder,
                       const float *bias, const int *bDims, int bOrder,
                       float *c, int *cDims, int *cOrder, float alpha);

/* out = sum of `in` along dimension dim; the CPU branch of ReduceSum.cpp:47-232 with
   power 1, no shift, no exp (how GradMulAndShift calls it), including the order in which
   its 32-lane buffers fold when the reduced dimension is the last one. */
int oracle_reduce_sum(const float *in, const int *dims, int order, int dim, float *out);

/* The products XMathGrad::GradMatrixMul issues for c = op(a) op(b) alpha on 2-D tensors
   (source/network/XBackwardMath.cpp:636-696): deda += ..., dedb += ... (beta = 1); a NULL
   gradient is skipped, as for a tensor that needs none. dedc is [rows of op(a)] x [cols of op(b)]. */
int oracle_grad_matmul2d(const float *a, float *deda, int transA,
                         const float *b, float *dedb, int transB,
                         const float *dedc, int na, int ma, int nb, int mb, float alpha);

/* XMathGrad::GradMatrixMul(node) (XBackwardMath.cpp:584-633): 2-D x 2-D, or the flatten
   rule for an untransposed N-D a; -2 where the reference aborts with "TODO!". */
int oracle_grad_matmul(const float *a, float *deda, int transA, const int *aDims, int aOrder,
                       const float *b, float *dedb, int transB, const int *bDims, int bOrder,
                       const float *dedc, float alpha);

/* XMathGrad::GradMatrixMulBatched (XBackwardMath.cpp:709-786) */
int oracle_grad_matmul_batched(const float *a, float *deda, int transA, const int *aDims,
                               const float *b, float *dedb, int transB, const int *bDims,
                               const float *dedc, const int *cDims, int order, float alpha);

/* XMathGrad::GradMulAndShift (XBackwardMath.cpp:1774-1884) for c = alpha op(x) op(w) + bias with
   the bias broadcast along dimension n of c: dedbias += sums of dedc, then GradMatrixMul.
   transX / transW are the flags as that function holds them in its local variables. */
int oracle_grad_mulandshift(const float *x, float *dedx, int transX, const int *xDims, int xOrder,
                            const float *w, float *dedw, int transW, const int *wDims, int wOrder,
                            float *dedbias, int biasNum,
                            const float *dedc, const int *cDims, int cOrder, int n, float alpha);

/* y = softmax over the last dimension of a [rows][n] tensor: the CPU branch of
   source/tensor/function/Softmax.cpp:38-117 with its _ReduceMax and its
   _ReduceSum(x, sum, dim, max, 1, true), sums in the reference's order. */
int oracle_softmax(const float *x, long rows, int n, float *y);

/* The inference path of Attention::MakeAttention (source/sample/transformer/submodel/
   Attention.cpp:186-239) on q [batch][lq][hidden], k and v [batch][lk][hidden], mask NULL or
   [heads][batch][lq][lk]: Split into heads, scale q, BMMul(q, k^T), add the mask, Softmax,
   BMMul with v, Merge. out is [batch][lq][hidden]. */
int oracle_attention(const float *q, const float *k, const float *v, const float *mask, float *out,
                     int batch, int lq, int lk, int hidden, int heads, float scale);

/* The first half of the same chain, as far as the training path shares it with inference (:194-224): Split, scale of
   q, BMMul(q, k^T), the mask, Softmax. probs is [heads][batch][lq][lk]: what the reference then passes through Dropout
   and multiplies with v, and what its backward step needs. */
int oracle_attention_probs(const float *q, const float *k, const float *mask, float *probs,
                           int batch, int lq, int lk, int hidden, int heads, float scale);

/* y = max(0, x) as _Rectify computes it (source/tensor/function/Rectify.cpp:47-55): a value below zero
   becomes 0, everything else (negative zero and NaN included) passes */
void oracle_rectify(const float *x, long n, float *y);

/* t[i] = (typeT) s[i] as the reference's GPU kernels convert (source/tensor/core/getandset/
   ConvertDataType.cu:31-66): X_FLOAT -> X_FLOAT16 round to nearest even (__float2half), X_FLOAT16 -> X_FLOAT
   exact, X_FLOAT -> X_INT toward zero (saturating, NaN -> 0: the GPU's cast), X_INT -> X_FLOAT round to
   nearest even. float <-> int is also what the CPU branch computes for values inside the int range
   (ConvertDataType.cpp:83-94); the CPU branch for half (:95-106) casts the VALUE to an integer and is not
   followed. Types are the reference's TENSOR_DATA_TYPE values (X_INT 0, X_FLOAT 2, X_FLOAT16 3).
   Returns 0, or -1 for a pair of types the reference refuses; equal types do nothing (:81-82). */
int oracle_convert_data_type(const void *s, int typeS, void *t, int typeT, long n);

/* comparator of the reference tests, CheckData.cpp:29-39 */
int oracle_is_float_equal(float a, float b, float absError, float relError);
/* CheckData.cpp:78-97 with its fixed relative bound 1e-4 */
int oracle_check_data(const float *value, const float *answer, int num, float tolerance);

/* IEEE binary16 conversion, round to nearest even. The reference's own CPU
   conversion is an integer cast (ConvertDataType.cpp:95-106), so this follows
   IEEE 754 instead and is pinned against numpy.float16 in the tests. */
uint16_t oracle_f32_to_f16(float f);
float oracle_f16_to_f32(uint16_t h);
void oracle_f32_to_f16_array(const float *src, uint16_t *dst, long n);
void oracle_f16_to_f32_array(const uint16_t *src, float *dst, long n);

/* portable seeded fills (splitmix64); the reference fills with libc rand()
   (SetData.cpp:484), which is not reproducible across C libraries. */
void oracle_fill_uniform(float *x, long n, uint64_t seed, float lo, float hi);
void oracle_fill_normal(float *x, long n, uint64_t seed, float mean, float std);

#ifdef __cplusplus
}
#endif
#endif
