/*
 * Problem descriptor of the one-kernel attention (attention_f32.hip), shared with
 * the C ABI (ntsamd_capi.hip).
 */
#pragma once
#include <hip/hip_runtime.h>

namespace ntsamd {

struct AttnParams {
    const void * q;                     /* q, k, v, out: float or half, one type for all four */
    const void * k;
    const void * v;
    const float * mask;                 /* NULL, or dense float [heads][batch][lq][lk] added to the scaled scores */
    void * out;
    int heads, batch, lq, lk, dh;
    long long qH, qB, qL;               /* element strides: head, batch item, row (columns are contiguous) */
    long long kH, kB, kL;
    long long vH, vB, vL;
    long long oH, oB, oL;
    float scale;
    int qTiles;                         /* filled in by the launcher */
    int maskVec;                        /* filled in by the launcher: 16-byte mask loads are possible */
    int probsVec;                       /* filled in by the launcher (attention_probs, attention_train): 16-byte stores are possible */
    /* the training form (attention_train_f32.hip): dense float [heads][batch][lq][lk] tensors */
    float * probs;                      /* the softmax's result, written */
    const float * dropMask;             /* NULL, or what the probabilities are multiplied with before the second product */
    float * dropped;                    /* NULL, or where probs * dropMask is written */
};

int launch_attention_f32(const AttnParams & p, hipStream_t stream);
int launch_attention_f16(const AttnParams & p, hipStream_t stream);
/* a handful of query rows per head (a decoding step): every key and value read once, no MFMA tiles of padding.
   attention_rows_lds: the LDS that kernel would need for the problem, 0 if it does not take it */
size_t attention_rows_lds(const AttnParams & p, bool half);
int launch_attention_rows(const AttnParams & p, bool half, hipStream_t stream);
/* probabilities only: out is the dense [heads][batch][lq][lk] tensor, v is not used */
int launch_attention_probs_f32(const AttnParams & p, hipStream_t stream);
/* the training path in one launch: probs, probs * dropMask and the merged context */
int launch_attention_train_f32(const AttnParams & p, hipStream_t stream);

}  // namespace ntsamd
