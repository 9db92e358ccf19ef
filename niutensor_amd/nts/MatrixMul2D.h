/* c = trans(a) * trans(b) * alpha + c * beta for matrices; signature of
   source/tensor/core/arithmetic/MatrixMul2D.h:31-35 */
#ifndef NTSAMD_MATRIXMUL2D_H
#define NTSAMD_MATRIXMUL2D_H

#include "XTensor.h"

namespace nts {

void _MatrixMul2D(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                  XTensor * c, DTYPE alpha = (DTYPE)1.0, DTYPE beta = 0, XPRunner * parallelRunner = NULL);

/* Host tensors (devID < 0). The reference multiplies them with its own CPU code: _MatrixMul2D falls to
   _MatrixMul2DParallel when none of a, b, c is on a GPU (source/tensor/core/arithmetic/MatrixMul2D.cpp:77-94), the
   batched and list forms loop over their items and come down to the same function (MatrixMulBatched.cpp:157-271),
   and MulAndShift adds the bias with _SumDim (MulAndShift.cpp:88). This library holds no CPU arithmetic; a tree
   that takes this layer hands its own functions in once, at start-up:
       nts::SetHostMatrixMul2D(_MatrixMul2DParallel);      (MatrixMul2DParallel.h)
       nts::SetHostSumDim(_SumDim);                        (SumDim.h)
   Without them a product of host tensors ends in the fatal error it always ended in here. NULL takes a hook out
   again; setting a hook is not synchronised with products that run at the same time. */
typedef void (*HostMatrixMul2DFn)(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                                  XTensor * c, DTYPE alpha, DTYPE beta, XPRunner * parallelRunner);
typedef void (*HostSumDimFn)(const XTensor * a, const XTensor * b, XTensor * c, int n, DTYPE beta);
void SetHostMatrixMul2D(HostMatrixMul2DFn fn);
void SetHostSumDim(HostSumDimFn fn);
HostMatrixMul2DFn GetHostMatrixMul2D();
HostSumDimFn GetHostSumDim();

/* the GPU half of _MatrixMul2D; stands where _CudaMatrixMul2D does (MatrixMul2D.cuh) */
void _AmdMatrixMul2D(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                     XTensor * c, DTYPE alpha = (DTYPE)1.0, DTYPE beta = 0);

/* what the fused epilogue of MulAndShift needs to know about the bias */
struct BiasSpec {
    const void * data;
    int mode;      /* 1: bias[column]; 2: bias[(row / rowDiv) % len] */
    int len;
    int rowDiv;
    int act;       /* 0: nothing; 1: Rectify applied to the result (NTSAMD_ACT_RECTIFY) */
};

void _AmdMatrixMul2DBias(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                         XTensor * c, DTYPE alpha, DTYPE beta, const BiasSpec * bias);

/* _AmdMatrixMul2D that also adds the column sums of op(b) to colSum (an order-1 tensor,
   or any tensor with as many elements as c has columns): colSum = colSum * colSumBeta + sums */
void _AmdMatrixMul2DColSum(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                           XTensor * c, DTYPE alpha, DTYPE beta, XTensor * colSum, DTYPE colSumBeta);

}  // namespace nts
#endif
