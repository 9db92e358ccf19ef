/*
 * Multi-head attention as one kernel launch.
 * Shape rules follow the operators it stands for: Split(x, order - 1, nhead) turns (batch..., l, hidden)
 * into (nhead, batch..., l, hidden / nhead) (source/tensor/core/shape/Split.cpp:39-124), the batched
 * products pair equal leading dimensions (core/arithmetic/MatrixMulBatched.cpp:49-138), Softmax runs over
 * the last dimension, Merge(x, order - 1) undoes the split (core/shape/Merge.cpp:41-150).
 */
#include "Attention.h"
#include "../../include/ntsamd_gemm.h"

namespace nts {

void _AmdAttention(const XTensor * q, const XTensor * k, const XTensor * v, const XTensor * mask,
                   XTensor * out, int nhead, DTYPE scale)
{
    CheckNTErrors((q && k && v && out), "Empty input tensors!");
    CheckNTErrors((q->dataType == X_FLOAT || q->dataType == X_FLOAT16), "TODO!");
    CheckNTErrors((k->dataType == q->dataType && v->dataType == q->dataType && out->dataType == q->dataType),
                  "Input tensors should have the same data type!");
    CheckNTErrors((q->order >= 2 && q->order == k->order && q->order == v->order && q->order == out->order),
                  "Input tensors must have the same order >= 2!");
    CheckNTErrors((q->devID >= 0), "This code must be run on GPUs!");
    CheckNTErrors((q->devID == k->devID && q->devID == v->devID && q->devID == out->devID),
                  "The tensors must be on the same GPU!");
    CheckNTErrors((_IsSameShaped(k, v) && _IsSameShaped(q, out)), "Unmatched tensors in attention!");

    const int order = q->order;
    const int hidden = q->dimSize[order - 1];
    const int lq = q->dimSize[order - 2], lk = k->dimSize[order - 2];
    CheckNTErrors((nhead > 0 && hidden % nhead == 0), "The hidden size must be a multiple of the number of heads!");
    CheckNTErrors((k->dimSize[order - 1] == hidden), "Unmatched tensors in attention!");
    int batch = 1;
    for (int i = 0; i < order - 2; i++) {
        CheckNTErrors((q->dimSize[i] == k->dimSize[i]), "Unmatched tensors in attention!");
        batch *= q->dimSize[i];
    }
    if (mask != NULL) {
        CheckNTErrors((mask->dataType == X_FLOAT && mask->devID == q->devID), "Unmatched tensors in attention!");
        CheckNTErrors((mask->unitNum == nhead * batch * lq * lk), "Unmatched tensors in attention!");
    }

    const int dh = hidden / nhead;
    /* head h of row r of batch item b starts at element b * rows * hidden + r * hidden + h * dh */
    long long strides[12] = {dh, (long long)lq * hidden, hidden,
                             dh, (long long)lk * hidden, hidden,
                             dh, (long long)lk * hidden, hidden,
                             dh, (long long)lq * hidden, hidden};
    int rc = ntsamd_attention(q->devID, NULL, q->data, k->data, v->data, mask != NULL ? mask->data : NULL, out->data,
                              q->dataType, nhead, batch, lq, lk, dh, strides, scale);
    if (rc != NTSAMD_OK) {
        ShowNTErrors(ntsamd_last_error());
    }
}

XTensor AmdAttention(const XTensor & q, const XTensor & k, const XTensor & v, const XTensor * mask,
                     int nhead, DTYPE scale)
{
    XTensor out(q.order, q.dimSize, q.dataType, 1.0F, q.devID, q.mem);
    out.SetTMPFlag();
    _AmdAttention(&q, &k, &v, mask, &out, nhead, scale);
    return out;
}

void _AmdAttentionProbs(const XTensor * q, const XTensor * k, const XTensor * mask, XTensor * probs, int nhead, DTYPE scale)
{
    CheckNTErrors((q && k && probs), "Empty input tensors!");
    CheckNTErrors((q->dataType == X_FLOAT && k->dataType == X_FLOAT && probs->dataType == X_FLOAT), "TODO!");
    CheckNTErrors((q->order >= 2 && q->order == k->order && probs->order == q->order + 1),
                  "Input tensors must have the same order >= 2!");
    CheckNTErrors((q->devID >= 0), "This code must be run on GPUs!");
    CheckNTErrors((q->devID == k->devID && q->devID == probs->devID), "The tensors must be on the same GPU!");

    const int order = q->order;
    const int hidden = q->dimSize[order - 1];
    const int lq = q->dimSize[order - 2], lk = k->dimSize[order - 2];
    CheckNTErrors((nhead > 0 && hidden % nhead == 0), "The hidden size must be a multiple of the number of heads!");
    CheckNTErrors((k->dimSize[order - 1] == hidden), "Unmatched tensors in attention!");
    int batch = 1;
    for (int i = 0; i < order - 2; i++) {
        CheckNTErrors((q->dimSize[i] == k->dimSize[i]), "Unmatched tensors in attention!");
        batch *= q->dimSize[i];
    }
    CheckNTErrors((probs->unitNum == nhead * batch * lq * lk), "Unmatched tensors in attention!");
    if (mask != NULL) {
        CheckNTErrors((mask->dataType == X_FLOAT && mask->devID == q->devID), "Unmatched tensors in attention!");
        CheckNTErrors((mask->unitNum == probs->unitNum), "Unmatched tensors in attention!");
    }
    const int dh = hidden / nhead;
    long long strides[6] = {dh, (long long)lq * hidden, hidden, dh, (long long)lk * hidden, hidden};
    int rc = ntsamd_attention_probs(q->devID, NULL, q->data, k->data, mask != NULL ? mask->data : NULL, probs->data,
                                    X_FLOAT, nhead, batch, lq, lk, dh, strides, scale);
    if (rc != NTSAMD_OK) {
        ShowNTErrors(ntsamd_last_error());
    }
}

XTensor AmdAttentionProbs(const XTensor & q, const XTensor & k, const XTensor * mask, int nhead, DTYPE scale)
{
    CheckNTErrors((q.order >= 2 && q.order + 1 <= MAX_TENSOR_DIM_NUM), "Input tensors must have the same order >= 2!");
    /* (nhead, batch..., lq, lk): the shape BMMul(Split(q), Split(k)^T) has in the reference */
    int dims[MAX_TENSOR_DIM_NUM];
    dims[0] = nhead;
    for (int i = 0; i < q.order - 1; i++)
        dims[i + 1] = q.dimSize[i];
    dims[q.order] = k.dimSize[k.order - 2];
    XTensor probs(q.order + 1, dims, q.dataType, 1.0F, q.devID, q.mem);
    probs.SetTMPFlag();
    _AmdAttentionProbs(&q, &k, mask, &probs, nhead, scale);
    return probs;
}

void _AmdAttentionContext(const XTensor * probs, const XTensor * v, XTensor * out, int nhead)
{
    CheckNTErrors((probs && v && out), "Empty input tensors!");
    /* float probabilities may meet half values (the half training path keeps the softmax and its dropout in float,
       source/sample/transformer/submodel/Attention.cpp:215-232, and converts before the product): the kernel rounds
       them to half where it fetches them, the ConvertDataType pass and its temporary are not needed */
    CheckNTErrors((v->dataType == out->dataType &&
                   (probs->dataType == v->dataType || (probs->dataType == X_FLOAT && v->dataType == X_FLOAT16))),
                  "Unmatched data types!");
    CheckNTErrors((v->dataType == X_FLOAT || v->dataType == X_FLOAT16), "TODO!");
    CheckNTErrors((v->order >= 2 && out->order == v->order && probs->order == v->order + 1),
                  "Input tensors must have the same order >= 2!");
    CheckNTErrors((v->devID >= 0), "This code must be run on GPUs!");
    CheckNTErrors((v->devID == probs->devID && v->devID == out->devID), "The tensors must be on the same GPU!");

    const int order = v->order;
    const int hidden = v->dimSize[order - 1];
    const int lk = v->dimSize[order - 2], lq = out->dimSize[order - 2];
    CheckNTErrors((nhead > 0 && hidden % nhead == 0), "The hidden size must be a multiple of the number of heads!");
    CheckNTErrors((out->dimSize[order - 1] == hidden), "Unmatched tensors in attention!");
    int batch = 1;
    for (int i = 0; i < order - 2; i++) {
        CheckNTErrors((v->dimSize[i] == out->dimSize[i]), "Unmatched tensors in attention!");
        batch *= v->dimSize[i];
    }
    CheckNTErrors((probs->dimSize[0] == nhead && probs->dimSize[order] == lk && probs->dimSize[order - 1] == lq &&
                   probs->unitNum == nhead * batch * lq * lk), "Unmatched tensors in attention!");
    const int dh = hidden / nhead;
    /* item (b, h): probs[h][b] is dense, the heads of v and out are dh columns of rows `hidden` long */
    int rc = ntsamd_matrix_mul_batched_grid(v->devID, NULL,
                                            probs->data, X_NOTRANS, probs->dataType, lk, (long long)lq * lk, (long long)batch * lq * lk,
                                            v->data, X_NOTRANS, v->dataType, hidden, (long long)lk * hidden, dh,
                                            out->data, out->dataType, hidden, (long long)lq * hidden, dh,
                                            batch, nhead, lq, lk, lk, dh, lq, dh, 1.0F, 0.0F);
    if (rc != NTSAMD_OK) {
        ShowNTErrors(ntsamd_last_error());
    }
}

XTensor AmdAttentionContext(const XTensor & probs, const XTensor & v, int nhead)
{
    CheckNTErrors((v.order >= 2 && probs.order == v.order + 1), "Input tensors must have the same order >= 2!");
    int dims[MAX_TENSOR_DIM_NUM];
    for (int i = 0; i < v.order; i++)
        dims[i] = v.dimSize[i];
    dims[v.order - 2] = probs.dimSize[probs.order - 2];
    XTensor out(v.order, dims, v.dataType, 1.0F, v.devID, v.mem);
    out.SetTMPFlag();
    _AmdAttentionContext(&probs, &v, &out, nhead);
    return out;
}

void _AmdAttentionTrain(const XTensor * q, const XTensor * k, const XTensor * v, const XTensor * mask, const XTensor * dropMask,
                        XTensor * probs, XTensor * dropped, XTensor * out, int nhead, DTYPE scale)
{
    CheckNTErrors((q && k && v && probs && out), "Empty input tensors!");
    CheckNTErrors((q->dataType == X_FLOAT && k->dataType == X_FLOAT && v->dataType == X_FLOAT &&
                   probs->dataType == X_FLOAT && out->dataType == X_FLOAT), "TODO!");
    CheckNTErrors((q->order >= 2 && q->order == k->order && q->order == v->order && q->order == out->order &&
                   probs->order == q->order + 1), "Input tensors must have the same order >= 2!");
    CheckNTErrors((q->devID >= 0), "This code must be run on GPUs!");
    CheckNTErrors((q->devID == k->devID && q->devID == v->devID && q->devID == out->devID && q->devID == probs->devID),
                  "The tensors must be on the same GPU!");
    CheckNTErrors((_IsSameShaped(k, v) && _IsSameShaped(q, out)), "Unmatched tensors in attention!");
    CheckNTErrors((dropped == NULL || dropMask != NULL), "Unmatched tensors in attention!");

    const int order = q->order;
    const int hidden = q->dimSize[order - 1];
    const int lq = q->dimSize[order - 2], lk = k->dimSize[order - 2];
    CheckNTErrors((nhead > 0 && hidden % nhead == 0), "The hidden size must be a multiple of the number of heads!");
    CheckNTErrors((k->dimSize[order - 1] == hidden), "Unmatched tensors in attention!");
    int batch = 1;
    for (int i = 0; i < order - 2; i++) {
        CheckNTErrors((q->dimSize[i] == k->dimSize[i]), "Unmatched tensors in attention!");
        batch *= q->dimSize[i];
    }
    CheckNTErrors((probs->unitNum == nhead * batch * lq * lk), "Unmatched tensors in attention!");
    const XTensor * like[3] = {mask, dropMask, dropped};
    for (int i = 0; i < 3; i++)
        if (like[i] != NULL) {
            CheckNTErrors((like[i]->dataType == X_FLOAT && like[i]->devID == q->devID && like[i]->unitNum == probs->unitNum),
                          "Unmatched tensors in attention!");
        }
    const int dh = hidden / nhead;
    long long strides[12] = {dh, (long long)lq * hidden, hidden,
                             dh, (long long)lk * hidden, hidden,
                             dh, (long long)lk * hidden, hidden,
                             dh, (long long)lq * hidden, hidden};
    int rc = ntsamd_attention_train(q->devID, NULL, q->data, k->data, v->data, mask != NULL ? mask->data : NULL,
                                    dropMask != NULL ? dropMask->data : NULL, probs->data,
                                    dropped != NULL ? dropped->data : NULL, out->data, X_FLOAT,
                                    nhead, batch, lq, lk, dh, strides, scale);
    if (rc != NTSAMD_OK) {
        ShowNTErrors(ntsamd_last_error());
    }
}

}  // namespace nts
