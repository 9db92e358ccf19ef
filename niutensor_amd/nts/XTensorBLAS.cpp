/*
 * GPU back end of the nts:: matrix products on gfx950: forwards to the C ABI
 * (include/ntsamd_gemm.h). Written in place of the cuBLAS calls of
 * source/tensor/core/arithmetic/XTensorBLAS.cu; the list dispatcher keeps the
 * reference's three-way choice (:252-387): equally spaced items go out as one
 * strided batch, same-shaped items as one pointer batch, anything else one by one.
 */
#include "XTensorBLAS.h"
#include "../../include/ntsamd_gemm.h"

#include <stdint.h>

namespace nts {

TensorList::TensorList(int myMaxNum) : items(NULL), count(0), maxNum(myMaxNum > 0 ? myMaxNum : 1)
{
    items = new XTensor *[maxNum];
}

TensorList::~TensorList()
{
    delete[] items;
}

void TensorList::Add(XTensor * t)
{
    if (count == maxNum) {
        XTensor ** bigger = new XTensor *[maxNum * 2];
        for (int i = 0; i < count; i++)
            bigger[i] = items[i];
        delete[] items;
        items = bigger;
        maxNum *= 2;
    }
    items[count++] = t;
}

/* a failure of the library is fatal, like every error of the reference's path;
   "Unsupported data type!" is what XTensorBLAS.cu:101-103 prints */
static void Check(int rc)
{
    if (rc == NTSAMD_ERR_DATATYPE) {
        ShowNTErrors("Unsupported data type!");
    }
    else if (rc != NTSAMD_OK) {
        ShowNTErrors(ntsamd_last_error());
    }
}

void _AmdMatrixMUL(int devID,
                   const void * a, MATRIX_TRANS_TYPE transposedA, TENSOR_DATA_TYPE dataTypeA,
                   const void * b, MATRIX_TRANS_TYPE transposedB, TENSOR_DATA_TYPE dataTypeB,
                   void * c, TENSOR_DATA_TYPE dataTypeC,
                   int na, int ma, int nb, int mb, int nc, int mc, DTYPE alpha, DTYPE beta)
{
    Check(ntsamd_matrix_mul(devID, NULL, a, transposedA, dataTypeA, b, transposedB, dataTypeB, c, dataTypeC,
                            na, ma, nb, mb, nc, mc, alpha, beta));
}

void _AmdMatrixMULBias(int devID,
                       const void * a, MATRIX_TRANS_TYPE transposedA, TENSOR_DATA_TYPE dataTypeA,
                       const void * b, MATRIX_TRANS_TYPE transposedB, TENSOR_DATA_TYPE dataTypeB,
                       void * c, TENSOR_DATA_TYPE dataTypeC,
                       int na, int ma, int nb, int mb, int nc, int mc, DTYPE alpha, DTYPE beta,
                       const void * bias, int biasMode, int biasLen, int biasRowDiv, int activation)
{
    Check(ntsamd_matrix_mul_bias_act(devID, NULL, a, transposedA, dataTypeA, b, transposedB, dataTypeB, c, dataTypeC,
                                     na, ma, nb, mb, nc, mc, alpha, beta, bias, biasMode, biasLen, biasRowDiv, activation));
}

void _AmdMatrixMULColSum(int devID,
                         const void * a, MATRIX_TRANS_TYPE transposedA, TENSOR_DATA_TYPE dataTypeA,
                         const void * b, MATRIX_TRANS_TYPE transposedB, TENSOR_DATA_TYPE dataTypeB,
                         void * c, TENSOR_DATA_TYPE dataTypeC,
                         int na, int ma, int nb, int mb, int nc, int mc, DTYPE alpha, DTYPE beta,
                         void * colSum, DTYPE colSumBeta)
{
    Check(ntsamd_matrix_mul_colsum(devID, NULL, a, transposedA, dataTypeA, b, transposedB, dataTypeB, c, dataTypeC,
                                   na, ma, nb, mb, nc, mc, alpha, beta, colSum, colSumBeta));
}

void _AmdReduceSumXZ(int devID, const void * in, TENSOR_DATA_TYPE dataType, int x, int y, int z,
                     void * out, DTYPE beta)
{
    Check(ntsamd_reduce_sum_xz(devID, NULL, in, dataType, x, y, z, out, beta));
}

void _AmdMatrixMULBatched(int devID,
                          const void ** a, MATRIX_TRANS_TYPE transposedA, TENSOR_DATA_TYPE dataTypeA,
                          const void ** b, MATRIX_TRANS_TYPE transposedB, TENSOR_DATA_TYPE dataTypeB,
                          void ** c, TENSOR_DATA_TYPE dataTypeC,
                          int count, int na, int ma, int nb, int mb, int nc, int mc, DTYPE alpha, DTYPE beta)
{
    Check(ntsamd_matrix_mul_batched(devID, NULL, a, transposedA, dataTypeA, b, transposedB, dataTypeB,
                                    c, dataTypeC, count, na, ma, nb, mb, nc, mc, alpha, beta));
}

void _AmdMatrixMULBatchedStrided(int devID,
                                 const void * a, MATRIX_TRANS_TYPE transposedA, TENSOR_DATA_TYPE dataTypeA, long long int strideA,
                                 const void * b, MATRIX_TRANS_TYPE transposedB, TENSOR_DATA_TYPE dataTypeB, long long int strideB,
                                 void * c, TENSOR_DATA_TYPE dataTypeC, long long int strideC,
                                 int count, int na, int ma, int nb, int mb, int nc, int mc, DTYPE alpha, DTYPE beta)
{
    Check(ntsamd_matrix_mul_batched_strided(devID, NULL, a, transposedA, dataTypeA, strideA,
                                            b, transposedB, dataTypeB, strideB, c, dataTypeC, strideC,
                                            count, na, ma, nb, mb, nc, mc, alpha, beta));
}

void _AmdMatrixMULList(int devID, const TensorList * a, MATRIX_TRANS_TYPE transposedA,
                       const TensorList * b, MATRIX_TRANS_TYPE transposedB, TensorList * c,
                       int count, DTYPE alpha, DTYPE beta)
{
    CheckNTErrors((a && b && c), "Empty input lists!");
    CheckNTErrors((a->count == b->count && a->count == c->count), "Input lists must be of the same size!");
    (void)count;

    if (a->count == 0)
        return;

    /* uniform: every item has the shape of the first; strided: the byte gaps between
       neighbours are constant for a, for b and for c */
    bool isUniform = true;
    bool isStrided = true;
    bool haveGap = false;
    intptr_t gapA = 0, gapB = 0, gapC = 0;
    for (int i = 1; i < a->count && isUniform; i++) {
        if (!_IsSameShaped(a->GetItem(i - 1), a->GetItem(i)) ||
            !_IsSameShaped(b->GetItem(i - 1), b->GetItem(i)) ||
            !_IsSameShaped(c->GetItem(i - 1), c->GetItem(i))) {
            isUniform = false;
            break;
        }
        intptr_t ga = (intptr_t)a->GetItem(i)->data - (intptr_t)a->GetItem(i - 1)->data;
        intptr_t gb = (intptr_t)b->GetItem(i)->data - (intptr_t)b->GetItem(i - 1)->data;
        intptr_t gc = (intptr_t)c->GetItem(i)->data - (intptr_t)c->GetItem(i - 1)->data;
        if (!haveGap) {
            gapA = ga;
            gapB = gb;
            gapC = gc;
            haveGap = true;
        }
        else if (ga != gapA || gb != gapB || gc != gapC)
            isStrided = false;
    }
    /* a batch walks forward through memory; anything else goes through the pointer list */
    if (gapA < 0 || gapB < 0 || gapC < 0)
        isStrided = false;

    XTensor * a0 = a->GetItem(0);
    XTensor * b0 = b->GetItem(0);
    XTensor * c0 = c->GetItem(0);

    if (isUniform && isStrided) {
        _AmdMatrixMULBatchedStrided(devID,
                                    a0->data, transposedA, a0->dataType, gapA / a0->unitSize,
                                    b0->data, transposedB, b0->dataType, gapB / b0->unitSize,
                                    c0->data, c0->dataType, gapC / c0->unitSize, a->count,
                                    a0->dimSize[0], a0->dimSize[1], b0->dimSize[0], b0->dimSize[1],
                                    c0->dimSize[0], c0->dimSize[1], alpha, beta);
    }
    else if (isUniform) {
        const void ** ap = new const void *[a->count];
        const void ** bp = new const void *[a->count];
        void ** cp = new void *[a->count];
        for (int i = 0; i < a->count; i++) {
            ap[i] = a->GetItem(i)->data;
            bp[i] = b->GetItem(i)->data;
            cp[i] = c->GetItem(i)->data;
        }
        _AmdMatrixMULBatched(devID, ap, transposedA, a0->dataType, bp, transposedB, b0->dataType,
                             cp, c0->dataType, a->count,
                             a0->dimSize[0], a0->dimSize[1], b0->dimSize[0], b0->dimSize[1],
                             c0->dimSize[0], c0->dimSize[1], alpha, beta);
        delete[] ap;
        delete[] bp;
        delete[] cp;
    }
    else {
        for (int i = 0; i < a->count; i++) {
            XTensor * ai = a->GetItem(i);
            XTensor * bi = b->GetItem(i);
            XTensor * ci = c->GetItem(i);
            _AmdMatrixMUL(devID, ai->data, transposedA, ai->dataType, bi->data, transposedB, bi->dataType,
                          ci->data, ci->dataType,
                          ai->dimSize[0], ai->dimSize[1], bi->dimSize[0], bi->dimSize[1],
                          ci->dimSize[0], ci->dimSize[1], alpha, beta);
        }
    }
}

}  // namespace nts
