/*
 * Matrix product of two 2-D tensors on a gfx950 GPU.
 * Host logic of source/tensor/core/arithmetic/MatrixMul2D.cpp:46-94 (shape
 * rule, "any tensor on a GPU selects the GPU path") and MatrixMul2D.cu:123-164
 * (same-GPU rule, accepted data types). Two things differ on purpose: c is not
 * zeroed before a beta == 0 product, because the kernels do not read c then;
 * and host tensors go to the function the host tree handed in with SetHostMatrixMul2D
 * (its own _MatrixMul2DParallel), because this library holds no CPU arithmetic: without
 * such a function they are refused.
 */
#include "MatrixMul2D.h"
#include "XTensorBLAS.h"

namespace nts {

static HostMatrixMul2DFn hostMatrixMul2D = NULL;
static HostSumDimFn hostSumDim = NULL;

void SetHostMatrixMul2D(HostMatrixMul2DFn fn) { hostMatrixMul2D = fn; }
void SetHostSumDim(HostSumDimFn fn) { hostSumDim = fn; }
HostMatrixMul2DFn GetHostMatrixMul2D() { return hostMatrixMul2D; }
HostSumDimFn GetHostSumDim() { return hostSumDim; }

void _MatrixMul2D(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                  XTensor * c, DTYPE alpha, DTYPE beta, XPRunner * parallelRunner)
{
    CheckNTErrors((a && b && c), "Empty input tensors!");
    CheckNTErrors((a->dataType == b->dataType), "Input tensors should have the same data type!");
    CheckNTErrors((a->order == 2 && b->order == 2 && c->order == 2), "Input tensors must have a order = 2!");

    int an = a->dimSize[0], am = a->dimSize[1];
    int bn = b->dimSize[0], bm = b->dimSize[1];
    int cn = c->dimSize[0], cm = c->dimSize[1];
    int am2 = transposedA == X_TRANS ? an : am;
    int an2 = transposedA == X_TRANS ? am : an;
    int bm2 = transposedB == X_TRANS ? bn : bm;
    int bn2 = transposedB == X_TRANS ? bm : bn;

    CheckNTErrors((am2 == bn2 && an2 == cn && bm2 == cm), "Unmatched tensors in multiplication!");

    if (a->devID >= 0 || b->devID >= 0 || c->devID >= 0) {
        _AmdMatrixMul2D(a, transposedA, b, transposedB, c, alpha, beta);
        return;
    }

    /* none of the three on a GPU: the host tree's dense float product (MatrixMul2D.cpp:77-94) */
    CheckNTErrors((!a->isSparse && !b->isSparse && !c->isSparse), "Sparse matrices are outside this library.");
    if (hostMatrixMul2D == NULL) {
        ShowNTErrors("Host tensors are multiplied by NiuTensor's own CPU path, which this library does not replace!");
    }
    if (a->dataType == DEFAULT_DTYPE && b->dataType == DEFAULT_DTYPE && c->dataType == DEFAULT_DTYPE)
        hostMatrixMul2D(a, transposedA, b, transposedB, c, alpha, beta, parallelRunner);
    else {
        ShowNTErrors("TODO!");
    }
}

void _AmdMatrixMul2DBias(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                         XTensor * c, DTYPE alpha, DTYPE beta, const BiasSpec * bias)
{
    CheckNTErrors((a && b && c), "Empty matrices in multiplication!");

    int an = transposedA == X_TRANS ? a->dimSize[1] : a->dimSize[0];
    int am = transposedA == X_TRANS ? a->dimSize[0] : a->dimSize[1];
    int bn = transposedB == X_TRANS ? b->dimSize[1] : b->dimSize[0];
    int bm = transposedB == X_TRANS ? b->dimSize[0] : b->dimSize[1];

    CheckNTErrors((am == bn && an == c->dimSize[0] && bm == c->dimSize[1]), "Unmatched matrices in multiplication!");
    CheckNTErrors((a->devID >= 0), "Cuda version matrix mutiplication must be run on GPUs.");
    CheckNTErrors(a->devID == b->devID && a->devID == c->devID,
                  "Matrices used in multiplication are not on the same GPU.");
    CheckNTErrors((!a->isSparse && !b->isSparse && !c->isSparse), "Sparse matrices are outside this library.");

    if ((a->dataType == X_FLOAT && b->dataType == X_FLOAT && c->dataType == X_FLOAT) ||
        (a->dataType == X_FLOAT16 && b->dataType == X_FLOAT16 && c->dataType == X_FLOAT16)) {
        if (bias == NULL)
            _AmdMatrixMUL(a->devID, a->data, transposedA, a->dataType, b->data, transposedB, a->dataType,
                          c->data, c->dataType,
                          a->dimSize[0], a->dimSize[1], b->dimSize[0], b->dimSize[1], c->dimSize[0], c->dimSize[1],
                          alpha, beta);
        else
            _AmdMatrixMULBias(a->devID, a->data, transposedA, a->dataType, b->data, transposedB, a->dataType,
                              c->data, c->dataType,
                              a->dimSize[0], a->dimSize[1], b->dimSize[0], b->dimSize[1], c->dimSize[0], c->dimSize[1],
                              alpha, beta, bias->data, bias->mode, bias->len, bias->rowDiv, bias->act);
    }
    else {
        ShowNTErrors("TODO!");
    }
}

void _AmdMatrixMul2DColSum(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                           XTensor * c, DTYPE alpha, DTYPE beta, XTensor * colSum, DTYPE colSumBeta)
{
    CheckNTErrors((a && b && c && colSum), "Empty matrices in multiplication!");
    CheckNTErrors((a->order == 2 && b->order == 2 && c->order == 2), "Input tensors must have a order = 2!");

    int an = transposedA == X_TRANS ? a->dimSize[1] : a->dimSize[0];
    int am = transposedA == X_TRANS ? a->dimSize[0] : a->dimSize[1];
    int bn = transposedB == X_TRANS ? b->dimSize[1] : b->dimSize[0];
    int bm = transposedB == X_TRANS ? b->dimSize[0] : b->dimSize[1];

    CheckNTErrors((am == bn && an == c->dimSize[0] && bm == c->dimSize[1]), "Unmatched matrices in multiplication!");
    CheckNTErrors((colSum->unitNum == bm), "Wrong tensor size!");
    CheckNTErrors((a->devID >= 0), "Cuda version matrix mutiplication must be run on GPUs.");
    CheckNTErrors(a->devID == b->devID && a->devID == c->devID && a->devID == colSum->devID,
                  "Matrices used in multiplication are not on the same GPU.");
    CheckNTErrors((a->dataType == b->dataType && a->dataType == c->dataType && a->dataType == colSum->dataType),
                  "Input tensors should have the same data type!");
    CheckNTErrors((a->dataType == X_FLOAT || a->dataType == X_FLOAT16), "TODO!");

    _AmdMatrixMULColSum(a->devID, a->data, transposedA, a->dataType, b->data, transposedB, b->dataType,
                        c->data, c->dataType,
                        a->dimSize[0], a->dimSize[1], b->dimSize[0], b->dimSize[1], c->dimSize[0], c->dimSize[1],
                        alpha, beta, colSum->data, colSumBeta);
}

void _AmdMatrixMul2D(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                     XTensor * c, DTYPE alpha, DTYPE beta)
{
    _AmdMatrixMul2DBias(a, transposedA, b, transposedB, c, alpha, beta, NULL);
}

}  // namespace nts
