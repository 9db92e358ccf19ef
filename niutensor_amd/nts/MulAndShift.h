/*
 * c = x * w * alpha + b, the linear layer. Declarations of
 * source/tensor/core/arithmetic/MulAndShift.h:32-37, plus GetBroadcastDimIndex
 * (source/tensor/core/arithmetic/Sum.h), which picks the dimension the bias is added along.
 */
#ifndef NTSAMD_MULANDSHIFT_H
#define NTSAMD_MULANDSHIFT_H

#include "XTensor.h"

namespace nts {

XTensor MulAndShift(const XTensor & x, const XTensor & w, const XTensor & b,
                    DTYPE alpha = (DTYPE)1.0, XPRunner * parallelRunner = NULL);

XTensor MulAndShift(const XTensor & x, MATRIX_TRANS_TYPE transposedX,
                    const XTensor & w, MATRIX_TRANS_TYPE transposedW,
                    const XTensor & b, DTYPE alpha = (DTYPE)1.0, XPRunner * parallelRunner = NULL);

/* Rectify(MulAndShift(x, w, b, alpha)) as ONE kernel: what the feed-forward block of the transformer sample
   computes first (source/sample/transformer/submodel/FFN.cpp:94, Rectify: source/tensor/function/Rectify.cpp:34-56).
   For inference: no autograd edge is recorded (the reference links Rectify to the product's output, which does
   not exist here). */
XTensor MulAndShiftRectify(const XTensor & x, const XTensor & w, const XTensor & b, DTYPE alpha = (DTYPE)1.0);

/* the dimension of a that b is broadcast along, or -1 */
int GetBroadcastDimIndex(const XTensor & a, const XTensor & b);

}  // namespace nts
#endif
