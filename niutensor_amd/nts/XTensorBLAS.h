/*
 * The GPU matrix-multiplication back end of the nts:: layer on gfx950.
 * These four functions stand where the reference declares the cuBLAS-backed
 * _CudaBLASMatrixMUL, _CudaBLASMatrixMULBatched, _CudaBLASMatrixMULBatchedStrided and
 * _CudaBLASMatrixMULList (source/tensor/core/arithmetic/XTensorBLAS.h:36-61). The
 * argument lists are the same apart from the cuBLAS handle, which is replaced
 * by the device id; they forward to the C ABI of include/ntsamd_gemm.h.
 */
#ifndef NTSAMD_XTENSORBLAS_H
#define NTSAMD_XTENSORBLAS_H

#include "XTensor.h"

namespace nts {

/* a list of tensors, as the reference's TensorList (source/tensor/XList.h:179-187), reduced to what the path uses */
struct TensorList {
    XTensor ** items;
    int count;
    int maxNum;
    explicit TensorList(int myMaxNum = 16);
    ~TensorList();
    void Add(XTensor * t);
    XTensor * GetItem(int i) const { return items[i]; }
};

void _AmdMatrixMUL(int devID,
                   const void * a, MATRIX_TRANS_TYPE transposedA, TENSOR_DATA_TYPE dataTypeA,
                   const void * b, MATRIX_TRANS_TYPE transposedB, TENSOR_DATA_TYPE dataTypeB,
                   void * c, TENSOR_DATA_TYPE dataTypeC,
                   int na, int ma, int nb, int mb, int nc, int mc, DTYPE alpha = (DTYPE)1.0, DTYPE beta = 1.0);

void _AmdMatrixMULBatched(int devID,
                          const void ** a, MATRIX_TRANS_TYPE transposedA, TENSOR_DATA_TYPE dataTypeA,
                          const void ** b, MATRIX_TRANS_TYPE transposedB, TENSOR_DATA_TYPE dataTypeB,
                          void ** c, TENSOR_DATA_TYPE dataTypeC,
                          int count, int na, int ma, int nb, int mb, int nc, int mc,
                          DTYPE alpha = (DTYPE)1.0, DTYPE beta = 1.0);

void _AmdMatrixMULBatchedStrided(int devID,
                                 const void * a, MATRIX_TRANS_TYPE transposedA, TENSOR_DATA_TYPE dataTypeA, long long int strideA,
                                 const void * b, MATRIX_TRANS_TYPE transposedB, TENSOR_DATA_TYPE dataTypeB, long long int strideB,
                                 void * c, TENSOR_DATA_TYPE dataTypeC, long long int strideC,
                                 int count, int na, int ma, int nb, int mb, int nc, int mc,
                                 DTYPE alpha = (DTYPE)1.0, DTYPE beta = 1.0);

void _AmdMatrixMULList(int devID, const TensorList * a, MATRIX_TRANS_TYPE transposedA,
                       const TensorList * b, MATRIX_TRANS_TYPE transposedB, TensorList * c,
                       int count, DTYPE alpha = (DTYPE)1.0, DTYPE beta = 1.0);

/* one product with the broadcast add of MulAndShift fused into its epilogue:
   biasMode 1 adds bias[column], biasMode 2 adds bias[(row / biasRowDiv) % biasLen];
   activation 1 applies Rectify to the result as well */
void _AmdMatrixMULBias(int devID,
                       const void * a, MATRIX_TRANS_TYPE transposedA, TENSOR_DATA_TYPE dataTypeA,
                       const void * b, MATRIX_TRANS_TYPE transposedB, TENSOR_DATA_TYPE dataTypeB,
                       void * c, TENSOR_DATA_TYPE dataTypeC,
                       int na, int ma, int nb, int mb, int nc, int mc, DTYPE alpha, DTYPE beta,
                       const void * bias, int biasMode, int biasLen, int biasRowDiv, int activation = 0);

/* one product that also returns the column sums of op(b):
   colSum[j] = colSumBeta * colSum[j] + sum_k op(b)[k][j]; for the backward step of MulAndShift,
   where the reference runs _CudaBLASMatrixMUL, _CudaReduceSum and _CudaSum one after the other
   (source/network/XBackwardMath.cpp:1805-1810, 1857-1879) */
void _AmdMatrixMULColSum(int devID,
                         const void * a, MATRIX_TRANS_TYPE transposedA, TENSOR_DATA_TYPE dataTypeA,
                         const void * b, MATRIX_TRANS_TYPE transposedB, TENSOR_DATA_TYPE dataTypeB,
                         void * c, TENSOR_DATA_TYPE dataTypeC,
                         int na, int ma, int nb, int mb, int nc, int mc, DTYPE alpha, DTYPE beta,
                         void * colSum, DTYPE colSumBeta);

/* out[j] = beta * out[j] + sum_i sum_k in[i][j][k] over a dense [x][y][z] tensor */
void _AmdReduceSumXZ(int devID, const void * in, TENSOR_DATA_TYPE dataType, int x, int y, int z,
                     void * out, DTYPE beta);

}  // namespace nts
#endif
