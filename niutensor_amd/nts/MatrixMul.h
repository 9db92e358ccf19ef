/*
 * c = trans(a) * trans(b) * alpha + c * beta over the last two dimensions of a and b.
 * Declarations of source/tensor/core/arithmetic/MatrixMul.h:43-78, unchanged.
 */
#ifndef NTSAMD_MATRIXMUL_H
#define NTSAMD_MATRIXMUL_H

#include "XTensor.h"

namespace nts {

#define MMul MatrixMul

/* Every order-2 block a_p of a is multiplied with every order-2 block b_q of b;
   the result block (p, q) is stored at index p * (number of b blocks) + q, so c
   has a's leading dimensions, then b's, then the matrix dimensions. */
void _MatrixMul(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                XTensor * c, DTYPE alpha = (DTYPE)1.0, DTYPE beta = 0, XPRunner * parallelRunner = NULL);

/* makes a new tensor for the result and returns it */
XTensor MatrixMul(const XTensor & a, MATRIX_TRANS_TYPE transposedA, const XTensor & b, MATRIX_TRANS_TYPE transposedB,
                  DTYPE alpha = (DTYPE)1.0, XPRunner * parallelRunner = NULL);

void MatrixMul(const XTensor & a, MATRIX_TRANS_TYPE transposedA, const XTensor & b, MATRIX_TRANS_TYPE transposedB,
               XTensor & c, DTYPE alpha = (DTYPE)1.0, DTYPE beta = 0, XPRunner * parallelRunner = NULL);

/* no transposition: c = a * b * alpha */
XTensor MatrixMul(const XTensor & a, const XTensor & b, DTYPE alpha = (DTYPE)1.0, XPRunner * parallelRunner = NULL);

void MatrixMul(const XTensor & a, const XTensor & b, XTensor & c, DTYPE alpha = (DTYPE)1.0,
               XPRunner * parallelRunner = NULL);

bool CheckMMulShape(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                    XTensor * c);

/* _MatrixMul with the broadcast add of `bias` along dimension n of c fused into
   the product (bias == NULL: plain _MatrixMul; n == SCALAR_BIAS: a one-element
   bias added to every element). act == 1 applies Rectify to the result on its way out (needs a
   bias: the epilogue is the fused one). Used by MulAndShift and MulAndShiftRectify. */
#define SCALAR_BIAS (-2)
void _MatrixMulBias(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                    XTensor * c, DTYPE alpha, DTYPE beta, const XTensor * bias, int n, int act = 0);

}  // namespace nts
#endif
