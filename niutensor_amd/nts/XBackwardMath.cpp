/*
 * Backward step of MatrixMul, MatrixMulBatched and MulAndShift on gfx950.
 * Host logic of source/network/XBackwardMath.cpp:584-786 and :1774-1884.
 *
 * Differences from the reference, on purpose:
 *  - the bias gradient of MulAndShift needs the sums of dE/dc over every
 *    dimension but the broadcast one. The reference reduces dE/dc into one or
 *    two temporaries and adds the last to the gradient (three or four kernels
 *    and a second pass over dE/dc). Here the sums are a by-product of the
 *    dE/dw product when dE/dc is its second, untransposed operand, and one
 *    kernel without temporaries otherwise.
 *  - an edge recorded by the second MulAndShift overload holds three
 *    parameters (n, transposedX, transposedW) and no alpha
 *    (MulAndShift.cpp:174-179); the reference's backward reads a fourth one
 *    past the end and takes the two flags in the opposite order
 *    (XBackwardMath.cpp:1791-1794). Here alpha is 1 for such an edge and the
 *    flags are taken in the order they were recorded.
 */
#include "XBackwardMath.h"
#include "MatrixMul.h"
#include "MatrixMul2D.h"
#include "MatrixMulBatched.h"
#include "XTensorBLAS.h"

namespace nts {

void XNoder::MakeGrad(XTensor * node)
{
    if (node == NULL)
        return;
    if (node->grad == NULL || !_IsSameShaped(node, node->grad)) {
        delete node->grad;
        node->grad = NewTensor(node);
        node->grad->SetZeroAll();
    }
}

bool XMathGrad::IsMathOP(XTensor * node)
{
    int id = node->income.typeID;
    return id == MATH_MATRIXMUL || id == MATH_MATRIXMULBATCHED || id == MATH_MULANDSHIFT;
}

void XMathGrad::MakeGrad(XTensor * node, bool isEfficient)
{
    CheckNTErrors(node != NULL, "No gradient found!");
    if (!isEfficient) {
        CheckNTErrors(node->grad != NULL, "No gradient found!");
    }
    else {
        CheckNTErrors(!node->isGrad || node->grad != NULL, "No gradient found!");
    }

    int operID = node->income.typeID;
    if (operID == MATH_MATRIXMUL)
        GradMatrixMul(node, isEfficient);
    else if (operID == MATH_MATRIXMULBATCHED)
        GradMatrixMulBatched(node, isEfficient);
    else if (operID == MATH_MULANDSHIFT)
        GradMulAndShift(node, isEfficient);
    else {
        ShowNTErrors("Unsupported backward computation! TODO!");
    }
}

/* the tails of an edge are recorded as const; the backward step owns their gradients */
static XTensor * Tail(XLink & income, int i)
{
    return const_cast<XTensor *>(income.tails[i]);
}

/* shapes of a and c (and of their gradients) folded to matrices for the duration of a call:
   the flatten rule of _MatrixMul for an untransposed a of order > 2 (XBackwardMath.cpp:611-629) */
struct Flattened {
    XTensor * t;
    int order;
    int dims[MAX_TENSOR_DIM_NUM];
    explicit Flattened(XTensor * tensor) : t(tensor), order(0)
    {
        if (t == NULL)
            return;
        order = t->order;
        memcpy(dims, t->dimSize, sizeof(int) * MAX_TENSOR_DIM_NUM);
        t->Reshape(t->unitNum / t->GetDim(-1), t->GetDim(-1));
    }
    ~Flattened()
    {
        if (t != NULL)
            t->Reshape(order, dims);
    }
};

void XMathGrad::GradMatrixMul(XTensor * node, bool isEfficient)
{
    XLink & income = node->income;
    CheckNTErrors(income.tailNum == 2, "Wrong input tensor number for MULTIPLY!");
    CheckNTErrors(income.paramNum == 3, "Wrong parameter number for MULTIPLY!");

    XTensor * a = Tail(income, 0);
    XTensor * b = Tail(income, 1);
    MATRIX_TRANS_TYPE transA = income.GetParamTrans(0);
    MATRIX_TRANS_TYPE transB = income.GetParamTrans(1);
    DTYPE alpha = income.GetParam(2);

    if (!isEfficient || a->isGrad)
        XNoder::MakeGrad(a);
    if (!isEfficient || b->isGrad)
        XNoder::MakeGrad(b);

    XTensor * c = node;
    XTensor * dedc = node->grad;
    XTensor * deda = a->grad;
    XTensor * dedb = b->grad;

    if (a->order == 2 && b->order == 2)
        GradMatrixMul(a, deda, transA, b, dedb, transB, dedc, alpha, isEfficient);
    else if (transA == X_NOTRANS && a->order > 2 && b->order == 2) {
        Flattened fa(a), fc(c), fda((!isEfficient || a->isGrad) ? deda : NULL), fdc(dedc);
        GradMatrixMul(a, deda, transA, b, dedb, transB, dedc, alpha, isEfficient);
    }
    else {
        ShowNTErrors("TODO!");
    }
}

void XMathGrad::GradMatrixMul(XTensor * a, XTensor * deda, MATRIX_TRANS_TYPE transA,
                              XTensor * b, XTensor * dedb, MATRIX_TRANS_TYPE transB,
                              XTensor * dedc, DTYPE alpha, bool isEfficient)
{
    GradMatrixMulColSum(a, deda, transA, b, dedb, transB, dedc, alpha, isEfficient, NULL);
}

bool XMathGrad::GradMatrixMulColSum(XTensor * a, XTensor * deda, MATRIX_TRANS_TYPE transA,
                                    XTensor * b, XTensor * dedb, MATRIX_TRANS_TYPE transB,
                                    XTensor * dedc, DTYPE alpha, bool isEfficient, XTensor * colSum)
{
    const bool wantA = !isEfficient || a->isGrad;
    const bool wantB = !isEfficient || b->isGrad;
    bool summed = false;

    /* c = a * b * alpha */
    if (transA == X_NOTRANS && transB == X_NOTRANS) {
        /* dE/da = dE/dc * b^T * alpha */
        if (wantA)
            _MatrixMul(dedc, X_NOTRANS, b, X_TRANS, deda, alpha, 1.0F);
        /* dE/db = a^T * dE/dc * alpha */
        if (wantB) {
            if (colSum != NULL) {
                _AmdMatrixMul2DColSum(a, X_TRANS, dedc, X_NOTRANS, dedb, alpha, 1.0F, colSum, 1.0F);
                summed = true;
            }
            else
                _MatrixMul(a, X_TRANS, dedc, X_NOTRANS, dedb, alpha, 1.0F);
        }
    }
    /* c = a^T * b * alpha */
    else if (transA == X_TRANS && transB == X_NOTRANS) {
        /* dE/da = b * dE/dc^T * alpha */
        if (wantA)
            _MatrixMul(b, X_NOTRANS, dedc, X_TRANS, deda, alpha, 1.0F);
        /* dE/db = a * dE/dc * alpha */
        if (wantB) {
            if (colSum != NULL) {
                _AmdMatrixMul2DColSum(a, X_NOTRANS, dedc, X_NOTRANS, dedb, alpha, 1.0F, colSum, 1.0F);
                summed = true;
            }
            else
                _MatrixMul(a, X_NOTRANS, dedc, X_NOTRANS, dedb, alpha, 1.0F);
        }
    }
    /* c = a * b^T * alpha */
    else if (transA == X_NOTRANS && transB == X_TRANS) {
        /* dE/da = dE/dc * b * alpha */
        if (wantA)
            _MatrixMul(dedc, X_NOTRANS, b, X_NOTRANS, deda, alpha, 1.0F);
        /* dE/db = dE/dc^T * a * alpha */
        if (wantB)
            _MatrixMul(dedc, X_TRANS, a, X_NOTRANS, dedb, alpha, 1.0F);
    }
    /* c = a^T * b^T * alpha */
    else if (transA == X_TRANS && transB == X_TRANS) {
        /* dE/da = b^T * dE/dc^T * alpha */
        if (wantA)
            _MatrixMul(b, X_TRANS, dedc, X_TRANS, deda, alpha, 1.0F);
        /* dE/db = dE/dc^T * a^T * alpha */
        if (wantB)
            _MatrixMul(dedc, X_TRANS, a, X_TRANS, dedb, alpha, 1.0F);
    }
    return summed;
}

void XMathGrad::GradMatrixMulBatched(XTensor * node, bool isEfficient)
{
    XLink & income = node->income;
    CheckNTErrors(income.tailNum == 2, "Wrong input tensor number for MULTIPLY!");
    CheckNTErrors(income.paramNum == 3, "Wrong parameter number for MULTIPLY!");

    XTensor * a = Tail(income, 0);
    XTensor * b = Tail(income, 1);
    MATRIX_TRANS_TYPE transA = income.GetParamTrans(0);
    MATRIX_TRANS_TYPE transB = income.GetParamTrans(1);
    DTYPE alpha = income.GetParam(2);

    const bool wantA = !isEfficient || a->isGrad;
    const bool wantB = !isEfficient || b->isGrad;
    if (wantA)
        XNoder::MakeGrad(a);
    if (wantB)
        XNoder::MakeGrad(b);

    XTensor * dedc = node->grad;
    XTensor * deda = a->grad;
    XTensor * dedb = b->grad;

    if (transA == X_NOTRANS && transB == X_NOTRANS) {
        if (wantA)
            _MatrixMulBatched(dedc, X_NOTRANS, b, X_TRANS, deda, alpha, 1.0F);
        if (wantB)
            _MatrixMulBatched(a, X_TRANS, dedc, X_NOTRANS, dedb, alpha, 1.0F);
    }
    else if (transA == X_TRANS && transB == X_NOTRANS) {
        if (wantA)
            _MatrixMulBatched(b, X_NOTRANS, dedc, X_TRANS, deda, alpha, 1.0F);
        if (wantB)
            _MatrixMulBatched(a, X_NOTRANS, dedc, X_NOTRANS, dedb, alpha, 1.0F);
    }
    else if (transA == X_NOTRANS && transB == X_TRANS) {
        if (wantA)
            _MatrixMulBatched(dedc, X_NOTRANS, b, X_NOTRANS, deda, alpha, 1.0F);
        if (wantB)
            _MatrixMulBatched(dedc, X_TRANS, a, X_NOTRANS, dedb, alpha, 1.0F);
    }
    else if (transA == X_TRANS && transB == X_TRANS) {
        if (wantA)
            _MatrixMulBatched(b, X_TRANS, dedc, X_TRANS, deda, alpha, 1.0F);
        if (wantB)
            _MatrixMulBatched(dedc, X_TRANS, a, X_TRANS, dedb, alpha, 1.0F);
    }
}

void XMathGrad::GradMulAndShift(XTensor * node, bool isEfficient)
{
    XLink & income = node->income;
    CheckNTErrors(income.tailNum == 3, "wrong input tensor number");
    CheckNTErrors(income.paramNum == 3 || income.paramNum == 4, "wrong parameter number");

    XTensor * x = Tail(income, 0);
    XTensor * w = Tail(income, 1);
    XTensor * b = Tail(income, 2);

    int n = income.GetParamInt(0);
    MATRIX_TRANS_TYPE transX = income.GetParamTrans(1);
    MATRIX_TRANS_TYPE transW = income.GetParamTrans(2);
    DTYPE alpha = income.paramNum == 4 ? income.GetParam(3) : (DTYPE)1.0;

    const bool wantB = !isEfficient || b->isGrad;
    const bool wantW = !isEfficient || w->isGrad;
    const bool wantX = !isEfficient || x->isGrad;
    if (wantB)
        XNoder::MakeGrad(b);
    if (wantW)
        XNoder::MakeGrad(w);
    if (wantX)
        XNoder::MakeGrad(x);

    XTensor * c = node;
    XTensor * dedc = node->grad;
    const int order = node->order;
    CheckNTErrors(n >= 0 && n < order, "Wrong dimension!");

    /* the sums ride on the dE/dw product when the bias runs along the last dimension of c
       (dE/dc is then a matrix with |b| columns) and that product exists and has dE/dc as
       its untransposed second operand */
    bool sumsOwed = wantB;
    const bool canRide = wantB && wantW && n == order - 1 && transW == X_NOTRANS &&
                         (dedc->dataType == X_FLOAT || dedc->dataType == X_FLOAT16);

    if (x->order == 2 && w->order == 2) {
        if (GradMatrixMulColSum(x, x->grad, transX, w, w->grad, transW, dedc, alpha, isEfficient,
                                canRide ? b->grad : NULL))
            sumsOwed = false;
    }
    else if (transX == X_NOTRANS && x->order > 2 && w->order == 2) {
        Flattened fx(x), fc(c), fdx(wantX ? x->grad : NULL), fdc(dedc);
        if (GradMatrixMulColSum(x, x->grad, transX, w, w->grad, transW, dedc, alpha, isEfficient,
                                canRide ? b->grad : NULL))
            sumsOwed = false;
    }
    /* other shapes: the reference computes no dE/dx and dE/dw either (XBackwardMath.cpp:1857-1883) */

    if (sumsOwed) {
        /* dE/dc as (x, |b|, z): everything before dimension n, dimension n, everything after */
        int xs = 1, zs = 1;
        for (int i = 0; i < n; i++)
            xs *= dedc->dimSize[i];
        for (int i = n + 1; i < order; i++)
            zs *= dedc->dimSize[i];
        CheckNTErrors(b->grad->unitNum == dedc->dimSize[n], "Wrong tensor size!");
        CheckNTErrors(dedc->devID >= 0 && dedc->devID == b->grad->devID,
                      "Host tensors are reduced by NiuTensor's own CPU path, which this library does not replace!");
        _AmdReduceSumXZ(dedc->devID, dedc->data, dedc->dataType, xs, dedc->dimSize[n], zs, b->grad->data, 1.0F);
    }
}

}  // namespace nts
