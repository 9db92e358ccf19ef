/* c = trans(a) * trans(b) * alpha + c * beta for matrices; signature of
   source/tensor/core/arithmetic/MatrixMul2D.h:31-35 */
#ifndef NTSAMD_MATRIXMUL2D_H
#define NTSAMD_MATRIXMUL2D_H

#include "XTensor.h"

namespace nts {

void _MatrixMul2D(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                  XTensor * c, DTYPE alpha = (DTYPE)1.0, DTYPE beta = 0, XPRunner * parallelRunner = NULL);

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
