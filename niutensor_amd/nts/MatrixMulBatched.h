/*
 * Batched product of two same-order tensors: block i of a times block i of b.
 * Declarations of source/tensor/core/arithmetic/MatrixMulBatched.h:37-83
 * (the CPU entry points are not part of this library).
 */
#ifndef NTSAMD_MATRIXMULBATCHED_H
#define NTSAMD_MATRIXMULBATCHED_H

#include "XTensor.h"

namespace nts {

#define BMMul MatrixMulBatched

void _MatrixMulBatched(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                       XTensor * c, DTYPE alpha = (DTYPE)1.0, DTYPE beta = 0, XPRunner * parallelRunner = NULL);

void _MatrixMulBatchedGPU(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                          XTensor * c, DTYPE alpha = (DTYPE)1.0, DTYPE beta = 0);

XTensor MatrixMulBatched(const XTensor & a, MATRIX_TRANS_TYPE transposedA, const XTensor & b, MATRIX_TRANS_TYPE transposedB,
                         DTYPE alpha = (DTYPE)1.0, XPRunner * parallelRunner = NULL);

XTensor MatrixMulBatched(const XTensor & a, const XTensor & b, DTYPE alpha = (DTYPE)1.0, XPRunner * parallelRunner = NULL);

}  // namespace nts
#endif
