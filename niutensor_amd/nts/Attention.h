/*
 * Multi-head attention of the reference's transformer sample as one call on a gfx950 GPU:
 * what Attention::MakeAttention (source/sample/transformer/submodel/Attention.cpp:186-239)
 * computes between the input projections and the output projection when it is not training.
 */
#ifndef NTSAMD_ATTENTION_H
#define NTSAMD_ATTENTION_H

#include "XTensor.h"

namespace nts {

/* out = Merge(Softmax(Split(q) * scale x Split(k)^T + mask, -1) x Split(v))
   q, out: (batch..., lq, hidden); k, v: (batch..., lk, hidden); nhead divides hidden;
   mask: NULL or an X_FLOAT tensor (nhead, batch..., lq, lk), added to the scaled scores.
   q, k, v, out: all X_FLOAT or all X_FLOAT16 (half products, fp32 softmax); one GPU. */
void _AmdAttention(const XTensor * q, const XTensor * k, const XTensor * v, const XTensor * mask,
                   XTensor * out, int nhead, DTYPE scale);

/* the same into a new tensor shaped like q */
XTensor AmdAttention(const XTensor & q, const XTensor & k, const XTensor & v, const XTensor * mask,
                     int nhead, DTYPE scale);

/* probs = Softmax(Split(q) * scale x Split(k)^T + mask, -1) as a (nhead, batch..., lq, lk) tensor: the part of
   MakeAttention that training shares with inference (:194-224); Dropout and BMMul(probs, Split(v)) follow in the
   caller, and the backward step reads probs. X_FLOAT. */
void _AmdAttentionProbs(const XTensor * q, const XTensor * k, const XTensor * mask, XTensor * probs, int nhead, DTYPE scale);
XTensor AmdAttentionProbs(const XTensor & q, const XTensor & k, const XTensor * mask, int nhead, DTYPE scale);

/* out = Merge(probs x Split(v)): the end of MakeAttention (:235-242) after Softmax and Dropout, as one batched
   product that reads the heads of v where they stand in (batch..., lk, hidden) and writes out in merged form
   (batch..., lq, hidden); neither Split nor Merge copies anything. probs: (nhead, batch..., lq, lk).
   All X_FLOAT or all X_FLOAT16. */
void _AmdAttentionContext(const XTensor * probs, const XTensor * v, XTensor * out, int nhead);
XTensor AmdAttentionContext(const XTensor & probs, const XTensor & v, int nhead);

/* The whole of MakeAttention between the projections when it IS training (:194-242), one launch:
       probs   = Softmax(Split(q) * scale x Split(k)^T + mask, -1)      (nhead, batch..., lq, lk), written
       dropped = probs * dropMask                                        the same shape, written if not NULL
       out     = Merge((dropMask ? dropped : probs) x Split(v))          (batch..., lq, hidden)
   dropMask is the tensor Dropout multiplies with (0 and 1 / (1 - p), filled by the caller's generator,
   source/tensor/function/Dropout.cpp:148-162); the backward step reads probs (the softmax's gradient) and dropped
   (the gradient of v). All X_FLOAT. */
void _AmdAttentionTrain(const XTensor * q, const XTensor * k, const XTensor * v, const XTensor * mask, const XTensor * dropMask,
                        XTensor * probs, XTensor * dropped, XTensor * out, int nhead, DTYPE scale);

}  // namespace nts
#endif
