/*
 * Batched product of two same-order tensors: block i of a times block i of b.
 * Declarations of source/tensor/core/arithmetic/MatrixMulBatched.h:37-83.
 */
#ifndef NTSAMD_MATRIXMULBATCHED_H
#define NTSAMD_MATRIXMULBATCHED_H

#include "XTensor.h"
#include "XTensorBLAS.h"

namespace nts {

#define BMMul MatrixMulBatched

void _MatrixMulBatched(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                       XTensor * c, DTYPE alpha = (DTYPE)1.0, DTYPE beta = 0, XPRunner * parallelRunner = NULL);

void _MatrixMulBatchedGPU(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                          XTensor * c, DTYPE alpha = (DTYPE)1.0, DTYPE beta = 0);

/* host tensors: one _MatrixMul2D per block / per list item, which ends in the function handed in with
   SetHostMatrixMul2D (the loops of MatrixMulBatched.cpp:157-218 and :231-271 in a build without BLAS) */
void _MatrixMulBatchedCPU(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                          XTensor * c, DTYPE alpha = (DTYPE)1.0, DTYPE beta = 0);
void _MatrixMulBatchedCPU(const TensorList * a, MATRIX_TRANS_TYPE transposedA, const TensorList * b, MATRIX_TRANS_TYPE transposedB,
                          TensorList * c, DTYPE alpha = (DTYPE)1.0, DTYPE beta = 0);

XTensor MatrixMulBatched(const XTensor & a, MATRIX_TRANS_TYPE transposedA, const XTensor & b, MATRIX_TRANS_TYPE transposedB,
                         DTYPE alpha = (DTYPE)1.0, XPRunner * parallelRunner = NULL);

XTensor MatrixMulBatched(const XTensor & a, const XTensor & b, DTYPE alpha = (DTYPE)1.0, XPRunner * parallelRunner = NULL);

}  // namespace nts
#endif
