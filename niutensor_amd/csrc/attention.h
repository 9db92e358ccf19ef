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

/* A query row's scores sit in the four lanes l % 16 + 16 g of a wave. The largest and the sum over those four lanes,
   delivered to all four, by two exchanges inside the vector ALU: v_permlane16_swap gives the rows of 16 lanes
   [x0 x0 x2 x2] and [x1 x1 x3 x3] from two copies of [x0 x1 x2 x3], v_permlane32_swap the halves [y_lo y_lo] and
   [y_hi y_hi]. (__shfl_xor takes each step through LDS: ds_bpermute and a wait for it, four times per row and block
   of keys.) The pairs are added in the order the shuffles added them. */
typedef unsigned lanes_u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void lane_rows_exchanged(float x, float & a, float & b)
{
    const unsigned u = __builtin_bit_cast(unsigned, x);
    const lanes_u32x2 r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    a = __builtin_bit_cast(float, (unsigned)r[0]);
    b = __builtin_bit_cast(float, (unsigned)r[1]);
}

__device__ __forceinline__ void lane_halves_exchanged(float x, float & a, float & b)
{
    const unsigned u = __builtin_bit_cast(unsigned, x);
    const lanes_u32x2 r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    a = __builtin_bit_cast(float, (unsigned)r[0]);
    b = __builtin_bit_cast(float, (unsigned)r[1]);
}

__device__ __forceinline__ float lane_groups_max(float x)
{
    float a, b;
    lane_rows_exchanged(x, a, b);
    lane_halves_exchanged(fmaxf(a, b), a, b);
    return fmaxf(a, b);
}

__device__ __forceinline__ float lane_groups_sum(float x)
{
    float a, b;
    lane_rows_exchanged(x, a, b);
    lane_halves_exchanged(a + b, a, b);
    return a + b;
}

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
