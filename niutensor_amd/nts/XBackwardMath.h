/*
 * The backward step of the matrix-multiplication family on gfx950: what the
 * reference's autograd runs for the edges MATH_MATRIXMUL, MATH_MATRIXMULBATCHED
 * and MATH_MULANDSHIFT (source/network/XBackwardMath.h:31-44, 88-101, 200-202;
 * XBackwardMath.cpp:584-786, 1774-1884), plus XNoder::MakeGrad
 * (source/network/XNoder.cpp:27-37). Every gradient is ADDED to what the
 * gradient tensor holds, through products with beta = 1.
 */
#ifndef NTSAMD_XBACKWARDMATH_H
#define NTSAMD_XBACKWARDMATH_H

#include "XTensor.h"

namespace nts {

class XNoder
{
public:
    /* gives the node a zeroed gradient of its own shape unless it has one */
    static void MakeGrad(XTensor * node);
};

class XMathGrad
{
public:
    /* compute dE/dx of the tails of a node from node->grad; isEfficient: only
       tails with isGrad set receive a gradient */
    static void MakeGrad(XTensor * node, bool isEfficient);

    /* whether the node was produced by one of the three operations handled here */
    static bool IsMathOP(XTensor * node);

    /* c = matmul(a, b) * alpha on matrices: dE/da and dE/db from dE/dc */
    static void GradMatrixMul(XTensor * a, XTensor * deda, MATRIX_TRANS_TYPE transA,
                              XTensor * b, XTensor * dedb, MATRIX_TRANS_TYPE transB,
                              XTensor * dedc, DTYPE alpha, bool isEfficient);

private:
    static void GradMatrixMul(XTensor * node, bool isEfficient);
    static void GradMatrixMulBatched(XTensor * node, bool isEfficient);
    static void GradMulAndShift(XTensor * node, bool isEfficient);

    /* GradMatrixMul that, where dE/db is a product with dE/dc as its second, untransposed
       operand, also adds the column sums of dE/dc to colSum in the same kernel; returns
       whether it did (false: the caller still owes the sums) */
    static bool GradMatrixMulColSum(XTensor * a, XTensor * deda, MATRIX_TRANS_TYPE transA,
                                    XTensor * b, XTensor * dedb, MATRIX_TRANS_TYPE transB,
                                    XTensor * dedc, DTYPE alpha, bool isEfficient, XTensor * colSum);
};

}  // namespace nts
#endif
