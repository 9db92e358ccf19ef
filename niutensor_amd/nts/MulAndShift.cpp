/*
 * MulAndShift on a gfx950 GPU: one kernel launch for product and bias.
 *
 * The reference (source/tensor/core/arithmetic/MulAndShift.cpp:38-110, :120-188)
 * computes the product into a temporary, zeroing it first, then adds the bias
 * in a second pass into a second tensor (_SumDim, SumDim.cu:120-211). Here the
 * add happens in the epilogue of the product, on the accumulators: no temporary,
 * no zeroing, one write of the result. What is kept: the result shape, the
 * dimension rule of GetBroadcastDimIndex, the cases that abort, the autograd
 * edge with its parameters.
 */
#include "MulAndShift.h"
#include "MatrixMul.h"

namespace nts {

int GetBroadcastDimIndex(const XTensor & a, const XTensor & b)
{
    /* source/tensor/core/arithmetic/Sum.cpp:233-260 */
    if (a.order < b.order)
        return -1;
    if (IsSameShaped(a, b))
        return -1;

    /* b may have one dimension that is not 1; the answer is the LAST dimension of a of that size */
    int hitDim = -1;
    bool isHit = false;
    for (int i = b.order - 1; i >= 0; i--) {
        if (b.dimSize[i] == 1)
            continue;
        if (isHit)
            return -1;
        isHit = true;
        for (int j = a.order - 1; j >= 0; j--) {
            if (b.dimSize[i] == a.dimSize[j]) {
                hitDim = j;
                break;
            }
        }
    }
    return hitDim;
}

static XTensor MulAndShiftCore(const XTensor & x, MATRIX_TRANS_TYPE transposedX,
                               const XTensor & w, MATRIX_TRANS_TYPE transposedW,
                               const XTensor & b, DTYPE alpha, bool firstOverload, int act = 0)
{
    CheckNTErrors(x.dataType == w.dataType, "Input tensors should have the same data type!");
    CheckNTErrors(x.order >= 2 && w.order >= 2, "Input tensors must have a order >= 2!");

    int xn = transposedX == X_TRANS ? x.dimSize[x.order - 1] : x.dimSize[x.order - 2];
    int xm = transposedX == X_TRANS ? x.dimSize[x.order - 2] : x.dimSize[x.order - 1];
    int wn = transposedW == X_TRANS ? w.dimSize[w.order - 1] : w.dimSize[w.order - 2];
    int wm = transposedW == X_TRANS ? w.dimSize[w.order - 2] : w.dimSize[w.order - 1];

    CheckNTErrors(xm == wn, "Unmatched tensors in multiplication!");

    int order = x.order + w.order - 2;
    CheckNTErrors(order <= MAX_TENSOR_DIM_NUM, "The result has too many dimensions!");
    int dimSize[MAX_TENSOR_DIM_NUM];
    int sub = 0;
    for (int i = 0; i < x.order - 2; i++)
        dimSize[sub++] = x.dimSize[i];
    for (int i = 0; i < w.order - 2; i++)
        dimSize[sub++] = w.dimSize[i];
    dimSize[sub++] = xn;
    dimSize[sub++] = wm;

    /* decide along which dimension the bias goes before anything is allocated;
       a tensor made with a negative size has the shape and no storage */
    int shapeOnly[MAX_TENSOR_DIM_NUM];
    for (int i = 0; i < order; i++)
        shapeOnly[i] = dimSize[i];
    shapeOnly[0] = -shapeOnly[0];
    XTensor shape(order, shapeOnly, x.dataType, 1.0F, x.devID, x.mem);

    int n;
    if (b.order == 0) {
        /* a scalar bias: the first overload shifts every element by it (:74-75); the
           second one has no such case and ends in "Something is wrong!" */
        CheckNTErrors(firstOverload, "Something is wrong!");
        n = SCALAR_BIAS;
    }
    else {
        n = GetBroadcastDimIndex(shape, b);
        if (n == -1) {
            /* the reference aborts here too, after an element-wise sum (:79-84) */
            ShowNTErrors("TODO!");
        }
        else if (!(n >= 0 && n < order)) {
            ShowNTErrors("Something is wrong!");
        }
    }

    XTensor c(order, dimSize, x.dataType, 1.0F, x.devID, x.mem);
    c.SetTMPFlag();

    _MatrixMulBias(&x, transposedX, &w, transposedW, &c, alpha, 0, &b, n, act);

    if (n == SCALAR_BIAS || act != 0)
        return c;

    /* autograd edge: tails x, w, b, then n, transposedX, transposedW and, in the
       first overload only, alpha (:94-100 and :174-179) */
    if (w.enableGrad && b.enableGrad) {
        XLink::MakeLink(&x, &w, &b, &c, MATH_MULANDSHIFT);
        XLink::AddParamToHeadInt(&c, n);
        XLink::AddParamToHeadTrans(&c, transposedX);
        XLink::AddParamToHeadTrans(&c, transposedW);
        if (firstOverload)
            XLink::AddParamToHead(&c, alpha);
    }

    return c;
}

XTensor MulAndShift(const XTensor & x, const XTensor & w, const XTensor & b, DTYPE alpha, XPRunner * parallelRunner)
{
    (void)parallelRunner;
    return MulAndShiftCore(x, X_NOTRANS, w, X_NOTRANS, b, alpha, true);
}

XTensor MulAndShiftRectify(const XTensor & x, const XTensor & w, const XTensor & b, DTYPE alpha)
{
    return MulAndShiftCore(x, X_NOTRANS, w, X_NOTRANS, b, alpha, true, 1);
}

XTensor MulAndShift(const XTensor & x, MATRIX_TRANS_TYPE transposedX, const XTensor & w, MATRIX_TRANS_TYPE transposedW,
                    const XTensor & b, DTYPE alpha, XPRunner * parallelRunner)
{
    (void)parallelRunner;
    return MulAndShiftCore(x, transposedX, w, transposedW, b, alpha, false);
}

}  // namespace nts
