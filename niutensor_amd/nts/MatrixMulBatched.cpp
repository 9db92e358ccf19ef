/*
 * Same-order batched matrix product on a gfx950 GPU.
 * Host logic of source/tensor/core/arithmetic/MatrixMulBatched.cpp:49-138
 * (checks, block count, one strided-batched call with the per-matrix element
 * counts as strides) and of its allocating wrappers (:291-390). c is not zeroed
 * before a beta == 0 product (:121-122 does that): the kernels do not read it.
 */
#include "MatrixMulBatched.h"
#include "MatrixMul2D.h"
#include "XTensorBLAS.h"

namespace nts {

void _MatrixMulBatched(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                       XTensor * c, DTYPE alpha, DTYPE beta, XPRunner * parallelRunner)
{
    (void)parallelRunner;
    CheckNTErrors((a && b && c), "Empty input tensors!");
    CheckNTErrors((a->dataType == b->dataType && a->dataType == c->dataType),
                  "Input tensors should have the same data type!");
    CheckNTErrors((a->order >= 2 && b->order >= 2 && c->order >= 2), "Input tensors must have a order >= 2!");
    CheckNTErrors((a->order == b->order && a->order == c->order), "Input tensor and output tensor must have same order!");

    if (a->devID >= 0 || b->devID >= 0 || c->devID >= 0)
        _MatrixMulBatchedGPU(a, transposedA, b, transposedB, c, alpha, beta);
    else
        _MatrixMulBatchedCPU(a, transposedA, b, transposedB, c, alpha, beta);
}

void _MatrixMulBatchedCPU(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                          XTensor * c, DTYPE alpha, DTYPE beta)
{
    CheckNTErrors((a && b && c), "Empty input tensors!");
    CheckNTErrors((a->dataType == b->dataType && a->dataType == c->dataType),
                  "Input tensors should have the same data type!");
    CheckNTErrors((a->order >= 2 && b->order >= 2 && c->order >= 2), "Input tensors must have a order >= 2!");
    CheckNTErrors((a->order == b->order && a->order == c->order), "Input tensor and output tensor must have same order!");

    const int order = a->order;
    const XTensor * t[3] = {a, b, c};
    int rows[3], cols[3];
    for (int k = 0; k < 3; k++) {
        rows[k] = t[k]->dimSize[order - 2];
        cols[k] = t[k]->dimSize[order - 1];
    }
    const int an = transposedA == X_TRANS ? cols[0] : rows[0], am = transposedA == X_TRANS ? rows[0] : cols[0];
    const int bn = transposedB == X_TRANS ? cols[1] : rows[1], bm = transposedB == X_TRANS ? rows[1] : cols[1];
    CheckNTErrors((am == bn && an == rows[2] && bm == cols[2]), "Unmatched tensors in multiplication!");

    int blockNum = 1;
    for (int i = 0; i < order - 2; i++) {
        CheckNTErrors((a->dimSize[i] == c->dimSize[i]), "Incorrect tensor sizes!");
        CheckNTErrors((b->dimSize[i] == c->dimSize[i]), "Incorrect tensor sizes!");
        blockNum *= a->dimSize[i];
    }

    /* one matrix-shaped view per operand (a negative size: the shape and no storage), moved from block to block */
    XTensor * view[3];
    for (int k = 0; k < 3; k++)
        view[k] = NewTensor2DV2(-rows[k], cols[k], t[k]->dataType, t[k]->devID, t[k]->mem);
    for (int i = 0; i < blockNum; i++) {
        for (int k = 0; k < 3; k++)
            view[k]->data = (char *)t[k]->data + (size_t)i * rows[k] * cols[k] * t[k]->unitSize;
        _MatrixMul2D(view[0], transposedA, view[1], transposedB, view[2], alpha, beta);
    }
    for (int k = 0; k < 3; k++) {
        view[k]->data = NULL;
        delete view[k];
    }
}

void _MatrixMulBatchedCPU(const TensorList * a, MATRIX_TRANS_TYPE transposedA, const TensorList * b, MATRIX_TRANS_TYPE transposedB,
                          TensorList * c, DTYPE alpha, DTYPE beta)
{
    CheckNTErrors((a && b && c), "Empty input lists!");
    CheckNTErrors((a->count == b->count && a->count == c->count), "Input lists must be of the same size!");
    for (int i = 0; i < a->count; i++) {
        XTensor * ai = a->GetItem(i), * bi = b->GetItem(i), * ci = c->GetItem(i);
        CheckNTErrors((ai->order == 2 && bi->order == 2 && ci->order == 2), "2d tensor (i.e., matrix) is required!");
        _MatrixMul2D(ai, transposedA, bi, transposedB, ci, alpha, beta);
    }
}

void _MatrixMulBatchedGPU(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                          XTensor * c, DTYPE alpha, DTYPE beta)
{
    CheckNTErrors((a && b && c), "Empty input tensors!");
    CheckNTErrors((a->dataType == b->dataType && a->dataType == c->dataType),
                  "Input tensors should have the same data type!");
    CheckNTErrors((a->order >= 2 && b->order >= 2 && c->order >= 2), "Input tensors must have a order >= 2!");
    CheckNTErrors((a->order == b->order && a->order == c->order), "Input tensor and output tensor must have same order!");
    CheckNTErrors(a->devID >= 0 && b->devID >= 0 && c->devID >= 0, "The tensors must be on GPUs");
    CheckNTErrors(a->devID == b->devID && a->devID == c->devID, "The code must be run on the same GPU!");

    const int order = a->order;
    int aRows = a->dimSize[order - 2], aCols = a->dimSize[order - 1];
    int bRows = b->dimSize[order - 2], bCols = b->dimSize[order - 1];
    int cn = c->dimSize[order - 2], cm = c->dimSize[order - 1];
    int an = transposedA == X_TRANS ? aCols : aRows;
    int am = transposedA == X_TRANS ? aRows : aCols;
    int bn = transposedB == X_TRANS ? bCols : bRows;
    int bm = transposedB == X_TRANS ? bRows : bCols;

    CheckNTErrors((am == bn && an == cn && bm == cm), "Unmatched tensors in multiplication!");

    int blockNum = 1;
    for (int i = 0; i < order - 2; i++) {
        CheckNTErrors((a->dimSize[i] == c->dimSize[i]), "Incorrect tensor sizes!");
        CheckNTErrors((b->dimSize[i] == c->dimSize[i]), "Incorrect tensor sizes!");
        blockNum *= a->dimSize[i];
    }

    _AmdMatrixMULBatchedStrided(a->devID,
                                a->data, transposedA, a->dataType, (long long)aRows * aCols,
                                b->data, transposedB, b->dataType, (long long)bRows * bCols,
                                c->data, c->dataType, (long long)cn * cm, blockNum,
                                aRows, aCols, bRows, bCols, cn, cm, alpha, beta);
}

XTensor MatrixMulBatched(const XTensor & a, MATRIX_TRANS_TYPE transposedA, const XTensor & b, MATRIX_TRANS_TYPE transposedB,
                         DTYPE alpha, XPRunner * parallelRunner)
{
    CheckNTErrors(a.dataType == b.dataType, "Input tensors should have the same data type!");
    CheckNTErrors(a.order >= 2 && b.order >= 2, "Input tensors must have a order >= 2!");
    CheckNTErrors(a.order == b.order, "Input tensor and output tensor must have same order!");

    int an = transposedA == X_TRANS ? a.dimSize[a.order - 1] : a.dimSize[a.order - 2];
    int am = transposedA == X_TRANS ? a.dimSize[a.order - 2] : a.dimSize[a.order - 1];
    int bn = transposedB == X_TRANS ? b.dimSize[b.order - 1] : b.dimSize[b.order - 2];
    int bm = transposedB == X_TRANS ? b.dimSize[b.order - 2] : b.dimSize[b.order - 1];

    CheckNTErrors(am == bn, "Unmatched tensors in multiplication!");

    /* a's leading dimensions, then the matrix dimensions of the product */
    int dimSize[MAX_TENSOR_DIM_NUM];
    for (int i = 0; i < a.order - 2; i++)
        dimSize[i] = a.dimSize[i];
    dimSize[a.order - 2] = an;
    dimSize[a.order - 1] = bm;

    XTensor c(a.order, dimSize, a.dataType, 1.0F, a.devID, a.mem);
    c.SetTMPFlag();

    _MatrixMulBatched(&a, transposedA, &b, transposedB, &c, alpha, 0, parallelRunner);

    /* autograd edge: tails a and b, then transposedA, transposedB, alpha (:321-326) */
    if (a.enableGrad && b.enableGrad) {
        XLink::MakeLink(&a, &b, &c, MATH_MATRIXMULBATCHED);
        XLink::AddParamToHeadTrans(&c, transposedA);
        XLink::AddParamToHeadTrans(&c, transposedB);
        XLink::AddParamToHead(&c, alpha);
    }
    return c;
}

XTensor MatrixMulBatched(const XTensor & a, const XTensor & b, DTYPE alpha, XPRunner * parallelRunner)
{
    return MatrixMulBatched(a, X_NOTRANS, b, X_NOTRANS, alpha, parallelRunner);
}

}  // namespace nts
