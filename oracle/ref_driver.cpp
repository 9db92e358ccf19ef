/*
 * TEST INFRASTRUCTURE - not part of the shipped library.
 *
 * C entry points around the REAL NiuTensor CPU implementation, compiled from
 * the reference tree where it lies (see the Makefile beside this file). The
 * resulting library is only used to validate the C restatement in
 * nts_oracle.c and, optionally, as the CPU baseline. Every tensor here lives
 * on the host (devID = -1), so the reference takes its naive CPU path
 * (_MatrixMul2DParallel; no BLAS is linked). The backward entry points run the
 * reference's own autograd step (source/network/XBackwardMath.cpp) on the edge
 * that its forward operator recorded.
 */
#include "XTensor.h"
#include "XCall.h"
#include "core/CHeader.h"
#include "test/TMatrixMul.h"
#include "test/TMatrixMul2D.h"
#include "test/TMatrixMul2DParallel.h"
#include "test/TMatrixMulBatched.h"
#include "test/TSumDim.h"
#include "../network/XBackwardMath.h"
#include "function/FHeader.h"

#include <string.h>

using namespace nts;

static XTensor * Make(const int * dims, int order, const float * data)
{
    XTensor * t = NewTensorV2(order, dims, X_FLOAT, 1.0F, -1, NULL);
    if (data != NULL)
        t->SetData(data, t->unitNum);
    return t;
}

extern "C" {

int ref_matmul2d(const float * a, int transA, const float * b, int transB, float * c,
                 int na, int ma, int nb, int mb, int nc, int mc, float alpha, float beta)
{
    int ad[2] = {na, ma}, bd[2] = {nb, mb}, cd[2] = {nc, mc};
    XTensor * ta = Make(ad, 2, a);
    XTensor * tb = Make(bd, 2, b);
    XTensor * tc = Make(cd, 2, c);
    _MatrixMul2D(ta, (MATRIX_TRANS_TYPE)transA, tb, (MATRIX_TRANS_TYPE)transB, tc, alpha, beta);
    memcpy(c, tc->data, sizeof(float) * (size_t)tc->unitNum);
    delete ta; delete tb; delete tc;
    return 0;
}

int ref_matmul(const float * a, int transA, const int * aDims, int aOrder,
               const float * b, int transB, const int * bDims, int bOrder,
               float * c, const int * cDims, int cOrder, float alpha, float beta)
{
    XTensor * ta = Make(aDims, aOrder, a);
    XTensor * tb = Make(bDims, bOrder, b);
    XTensor * tc = Make(cDims, cOrder, c);
    _MatrixMul(ta, (MATRIX_TRANS_TYPE)transA, tb, (MATRIX_TRANS_TYPE)transB, tc, alpha, beta);
    memcpy(c, tc->data, sizeof(float) * (size_t)tc->unitNum);
    delete ta; delete tb; delete tc;
    return 0;
}

int ref_matmul_batched(const float * a, int transA, const int * aDims,
                       const float * b, int transB, const int * bDims,
                       float * c, const int * cDims, int order, float alpha, float beta)
{
    XTensor * ta = Make(aDims, order, a);
    XTensor * tb = Make(bDims, order, b);
    XTensor * tc = Make(cDims, order, c);
    _MatrixMulBatched(ta, (MATRIX_TRANS_TYPE)transA, tb, (MATRIX_TRANS_TYPE)transB, tc, alpha, beta);
    memcpy(c, tc->data, sizeof(float) * (size_t)tc->unitNum);
    delete ta; delete tb; delete tc;
    return 0;
}

/* the allocating wrapper: returns the order of the result, fills cDims and c */
int ref_matmul_alloc(const float * a, int transA, const int * aDims, int aOrder,
                     const float * b, int transB, const int * bDims, int bOrder,
                     float * c, int * cDims, float alpha)
{
    XTensor * ta = Make(aDims, aOrder, a);
    XTensor * tb = Make(bDims, bOrder, b);
    XTensor tc = MatrixMul(*ta, (MATRIX_TRANS_TYPE)transA, *tb, (MATRIX_TRANS_TYPE)transB, alpha);
    for (int i = 0; i < tc.order; i++)
        cDims[i] = tc.dimSize[i];
    memcpy(c, tc.data, sizeof(float) * (size_t)tc.unitNum);
    int order = tc.order;
    delete ta; delete tb;
    return order;
}

int ref_broadcast_dim_index(const int * aDims, int aOrder, const int * bDims, int bOrder)
{
    XTensor * ta = Make(aDims, aOrder, NULL);
    XTensor * tb = Make(bDims, bOrder, NULL);
    int n = GetBroadcastDimIndex(*ta, *tb);
    delete ta; delete tb;
    return n;
}

int ref_sumdim(const float * a, const int * aDims, int aOrder,
               const float * b, const int * bDims, int bOrder, float * c, int n, float beta)
{
    XTensor * ta = Make(aDims, aOrder, a);
    XTensor * tb = Make(bDims, bOrder, b);
    XTensor * tc = Make(aDims, aOrder, NULL);
    _SumDim(ta, tb, tc, n, beta);
    memcpy(c, tc->data, sizeof(float) * (size_t)tc->unitNum);
    delete ta; delete tb; delete tc;
    return 0;
}

/* overload == 1: MulAndShift(x, w, b, alpha); overload == 2: with transpose flags.
   Returns the order of the result. */
int ref_mulandshift(int overload,
                    const float * x, int transX, const int * xDims, int xOrder,
                    const float * w, int transW, const int * wDims, int wOrder,
                    const float * bias, const int * bDims, int bOrder,
                    float * c, int * cDims, float alpha)
{
    XTensor * tx = Make(xDims, xOrder, x);
    XTensor * tw = Make(wDims, wOrder, w);
    XTensor * tb = Make(bDims, bOrder, bias);
    XTensor tc;
    if (overload == 1)
        tc = MulAndShift(*tx, *tw, *tb, alpha);
    else
        tc = MulAndShift(*tx, (MATRIX_TRANS_TYPE)transX, *tw, (MATRIX_TRANS_TYPE)transW, *tb, alpha);
    for (int i = 0; i < tc.order; i++)
        cDims[i] = tc.dimSize[i];
    memcpy(c, tc.data, sizeof(float) * (size_t)tc.unitNum);
    int order = tc.order;
    delete tx; delete tw; delete tb;
    return order;
}

int ref_reduce_sum(const float * in, const int * dims, int order, int dim, float * out)
{
    XTensor * ti = Make(dims, order, in);
    int od[MAX_TENSOR_DIM_NUM];
    int n = 0;
    for (int i = 0; i < order; i++)
        if (i != dim)
            od[n++] = dims[i];
    XTensor * to = Make(od, order - 1, NULL);
    _ReduceSum(ti, to, dim);
    memcpy(out, to->data, sizeof(float) * (size_t)to->unitNum);
    delete ti; delete to;
    return 0;
}

/* Forward with the reference's operator (kind 0: MatrixMul, 1: MatrixMulBatched,
   2: MulAndShift(x, w, b, alpha)) with gradients enabled, so that the result carries the
   edge; then dE/dc is set and XMathGrad::MakeGrad runs the backward step for that edge.
   deda / dedb / dedbias hold the gradients' starting values on entry (the step adds to
   them) and the results on return. Returns the order of c. */
int ref_grad(int kind,
             const float * a, const int * aDims, int aOrder, int transA,
             const float * b, const int * bDims, int bOrder, int transB,
             const float * bias, const int * biasDims, int biasOrder,
             float alpha, const float * dedc,
             float * deda, float * dedb, float * dedbias)
{
    bool backup = X_ENABLE_GRAD;
    X_ENABLE_GRAD = true;
    XTensor * ta = Make(aDims, aOrder, a);
    XTensor * tb = Make(bDims, bOrder, b);
    XTensor * tbias = kind == 2 ? Make(biasDims, biasOrder, bias) : NULL;
    int order;
    {
        XTensor tc;
        if (kind == 0)
            tc = MatrixMul(*ta, (MATRIX_TRANS_TYPE)transA, *tb, (MATRIX_TRANS_TYPE)transB, alpha);
        else if (kind == 1)
            tc = MatrixMulBatched(*ta, (MATRIX_TRANS_TYPE)transA, *tb, (MATRIX_TRANS_TYPE)transB, alpha);
        else
            tc = MulAndShift(*ta, *tb, *tbias, alpha);
        order = tc.order;
        tc.grad = NewTensor(&tc);
        tc.grad->SetData(dedc, tc.unitNum);
        ta->grad = NewTensor(ta);
        ta->grad->SetData(deda, ta->unitNum);
        tb->grad = NewTensor(tb);
        tb->grad->SetData(dedb, tb->unitNum);
        if (tbias != NULL) {
            tbias->grad = NewTensor(tbias);
            tbias->grad->SetData(dedbias, tbias->unitNum);
        }
        XMathGrad::MakeGrad(&tc, false);
        memcpy(deda, ta->grad->data, sizeof(float) * (size_t)ta->unitNum);
        memcpy(dedb, tb->grad->data, sizeof(float) * (size_t)tb->unitNum);
        if (tbias != NULL)
            memcpy(dedbias, tbias->grad->data, sizeof(float) * (size_t)tbias->unitNum);
    }
    delete ta; delete tb;
    if (tbias != NULL)
        delete tbias;
    X_ENABLE_GRAD = backup;
    return order;
}

int ref_softmax(const float * x, const int * dims, int order, float * y)
{
    XTensor * tx = Make(dims, order, x);
    XTensor * ty = Make(dims, order, NULL);
    _Softmax(tx, ty, order - 1);
    memcpy(y, ty->data, sizeof(float) * (size_t)ty->unitNum);
    delete tx; delete ty;
    return 0;
}

/* the operator chain of Attention::MakeAttention in inference, with the reference's own operators:
   q [batch][lq][hidden], k, v [batch][lk][hidden], mask NULL or [heads][batch][lq][lk] */
int ref_attention(const float * q, const float * k, const float * v, const float * mask, float * out,
                  int batch, int lq, int lk, int hidden, int heads, float scale)
{
    int dq[3] = {batch, lq, hidden}, dk[3] = {batch, lk, hidden}, dm[4] = {heads, batch, lq, lk};
    XTensor * tq = Make(dq, 3, q);
    XTensor * tk = Make(dk, 3, k);
    XTensor * tv = Make(dk, 3, v);
    XTensor * tm = mask != NULL ? Make(dm, 4, mask) : NULL;
    /* inference: no autograd edges, as the sample's translator runs it (DISABLE_GRAD) */
    bool backup = X_ENABLE_GRAD;
    X_ENABLE_GRAD = false;
    {
        XTensor qh = Split(*tq, 2, heads);
        XTensor kh = Split(*tk, 2, heads);
        XTensor vh = Split(*tv, 2, heads);
        ScaleAndShiftMe(qh, scale, 0.0F);
        XTensor att = BMMul(qh, X_NOTRANS, kh, X_TRANS);
        if (tm != NULL)
            SumMe(att, *tm);
        att = Softmax(att, -1);
        att = BMMul(att, vh);
        XTensor merged = Merge(att, att.order - 1);
        memcpy(out, merged.data, sizeof(float) * (size_t)merged.unitNum);
    }
    delete tq; delete tk; delete tv;
    if (tm != NULL)
        delete tm;
    X_ENABLE_GRAD = backup;
    return 0;
}

/* the same chain up to the Softmax: probs [heads][batch][lq][lk] */
int ref_attention_probs(const float * q, const float * k, const float * mask, float * probs,
                        int batch, int lq, int lk, int hidden, int heads, float scale)
{
    int dq[3] = {batch, lq, hidden}, dk[3] = {batch, lk, hidden}, dm[4] = {heads, batch, lq, lk};
    XTensor * tq = Make(dq, 3, q);
    XTensor * tk = Make(dk, 3, k);
    XTensor * tm = mask != NULL ? Make(dm, 4, mask) : NULL;
    bool backup = X_ENABLE_GRAD;
    X_ENABLE_GRAD = false;
    {
        XTensor qh = Split(*tq, 2, heads);
        XTensor kh = Split(*tk, 2, heads);
        ScaleAndShiftMe(qh, scale, 0.0F);
        XTensor att = BMMul(qh, X_NOTRANS, kh, X_TRANS);
        if (tm != NULL)
            SumMe(att, *tm);
        att = Softmax(att, -1);
        memcpy(probs, att.data, sizeof(float) * (size_t)att.unitNum);
    }
    delete tq; delete tk;
    if (tm != NULL)
        delete tm;
    X_ENABLE_GRAD = backup;
    return 0;
}

int ref_rectify(const float * x, int n, float * y)
{
    int dims[1] = {n};
    XTensor * tx = Make(dims, 1, x);
    XTensor * ty = Make(dims, 1, NULL);
    _Rectify(tx, ty);
    memcpy(y, ty->data, sizeof(float) * (size_t)n);
    delete tx; delete ty;
    return 0;
}

/* _ConvertDataType between X_FLOAT (2) and X_INT (0) on the host (ConvertDataType.cpp:83-94); the
   half branches of the host code cast the value to an integer and are of no use as a reference */
int ref_convert(const void * s, int typeS, void * t, int typeT, int n)
{
    int dims[1] = {n};
    XTensor * ts = NewTensorV2(1, dims, (TENSOR_DATA_TYPE)typeS, 1.0F, -1);
    XTensor * tt = NewTensorV2(1, dims, (TENSOR_DATA_TYPE)typeT, 1.0F, -1);
    memcpy(ts->data, s, (size_t)n * ts->unitSize);
    _ConvertDataType(ts, tt);
    memcpy(t, tt->data, (size_t)n * tt->unitSize);
    delete ts; delete tt;
    return 0;
}

/* the reference's own known-answer tests for this path; bit i set = suite i passed */
int ref_run_matmul_tests()
{
    int ok = 0;
    if (TestMatrixMul()) ok |= 1;
    if (TestMatrixMul2D()) ok |= 2;
    if (TestMatrixMul2DParallel()) ok |= 4;
    if (TestMatrixMulBatched()) ok |= 8;
    if (TestSumDim()) ok |= 16;
    return ok;
}

int ref_enum_values(int * out)
{
    out[0] = (int)X_TRANS; out[1] = (int)X_NOTRANS;
    out[2] = (int)X_FLOAT; out[3] = (int)X_FLOAT16;
    out[4] = (int)sizeof(XTensor);
    return 0;
}

}
