/*
 * TEST INFRASTRUCTURE - not part of the shipped library (see nts_oracle.h).
 *
 * Plain-C restatement of the CPU path of the NiuTensor matrix-multiplication
 * family. Build with -ffp-contract=off: the reference is compiled without FMA
 * contraction for baseline x86-64, and the single fp32 accumulator with
 * ascending k is what fixes the rounding of every output element.
 */
#include "nts_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ---- 2-D product -------------------------------------------------------- */

/* NN kernel: MatrixMul2DMultiTheading.cpp:59-145 (FAST_MATRIX branch) run as
   one job over the whole of c (XMatrixSegment.cpp:44-49: no runner => 1 job).
   Four loop bodies there differ only in whether alpha is multiplied per term
   (alpha != 1) and whether c*beta is added (beta != 0). */
static void mm_nn(const float *a, const float *b, float *c,
                  int am, int bm, int cn, int cm, float alpha, float beta)
{
    int num = am;
    for (int i = 0; i < cn; i++) {
        float *p3 = c + (long)i * cm;
        for (int j = 0; j < cm; j++) {
            float r = 0;
            const float *p1 = a + (long)i * am;
            const float *p2 = b + j;
            if (alpha == 1) {
                for (int k = 0; k < num; k++) {
                    r += (*p1) * (*p2);
                    p1 += 1;
                    p2 += bm;
                }
            }
            else {
                for (int k = 0; k < num; k++) {
                    r += (*p1) * (*p2) * alpha;
                    p1 += 1;
                    p2 += bm;
                }
            }
            if (beta == 0)
                *p3 = r;
            else
                *p3 = *p3 * beta + r;
            p3 += 1;
        }
    }
}

/* TN / NT / TT: MatrixMul2DParallel.cpp:67-128. alpha is always multiplied
   inside the sum; the output is always c*beta + r (c was zeroed for beta==0). */
static void mm_strided(const float *a, long aRowStep, long aKStep,
                       const float *b, long bColStep, long bKStep,
                       float *c, int cn, int cm, int num, float alpha, float beta)
{
    for (int i = 0; i < cn; i++) {
        float *p3 = c + (long)i * cm;
        for (int j = 0; j < cm; j++) {
            float r = 0;
            const float *p1 = a + i * aRowStep;
            const float *p2 = b + j * bColStep;
            for (int k = 0; k < num; k++) {
                r += (*p1) * (*p2) * alpha;
                p1 += aKStep;
                p2 += bKStep;
            }
            *p3 = *p3 * beta + r;
            p3 += 1;
        }
    }
}

int oracle_matmul2d(const float *a, int transA, const float *b, int transB, float *c,
                    int na, int ma, int nb, int mb, int nc, int mc,
                    float alpha, float beta)
{
    /* shape rule of MatrixMul2D.cpp:56-67 */
    int am2 = transA == ORACLE_X_TRANS ? na : ma;
    int an2 = transA == ORACLE_X_TRANS ? ma : na;
    int bm2 = transB == ORACLE_X_TRANS ? nb : mb;
    int bn2 = transB == ORACLE_X_TRANS ? mb : nb;
    if (!(am2 == bn2 && an2 == nc && bm2 == mc))
        return -1;

    /* MatrixMul2DParallel.cpp:57-58: beta == 0 zeroes c first, so whatever c
       held (NaN included) never reaches the result */
    if (beta == 0)
        memset(c, 0, sizeof(float) * (size_t)nc * (size_t)mc);

    if (nc == 0 || mc == 0)
        return 0;

    if (transA == ORACLE_X_NOTRANS && transB == ORACLE_X_NOTRANS)
        mm_nn(a, b, c, ma, mb, nc, mc, alpha, beta);
    else if (transA == ORACLE_X_TRANS && transB == ORACLE_X_NOTRANS)
        mm_strided(a, 1, ma, b, 1, mb, c, nc, mc, na, alpha, beta);   /* :67-86 */
    else if (transA == ORACLE_X_NOTRANS && transB == ORACLE_X_TRANS)
        mm_strided(a, ma, 1, b, mb, 1, c, nc, mc, ma, alpha, beta);   /* :88-107 */
    else
        mm_strided(a, 1, ma, b, mb, 1, c, nc, mc, na, alpha, beta);   /* :109-128 */
    return 0;
}

/* ---- batched and N-D products ------------------------------------------- */

int oracle_matmul_batched(const float *a, int transA, const int *aDims,
                          const float *b, int transB, const int *bDims,
                          float *c, const int *cDims, int order,
                          float alpha, float beta)
{
    /* MatrixMulBatched.cpp:171-191 */
    if (order < 2)
        return -1;
    int an = transA == ORACLE_X_TRANS ? aDims[order - 1] : aDims[order - 2];
    int am = transA == ORACLE_X_TRANS ? aDims[order - 2] : aDims[order - 1];
    int bn = transB == ORACLE_X_TRANS ? bDims[order - 1] : bDims[order - 2];
    int bm = transB == ORACLE_X_TRANS ? bDims[order - 2] : bDims[order - 1];
    int cn = cDims[order - 2];
    int cm = cDims[order - 1];
    if (!(am == bn && an == cn && bm == cm))
        return -1;

    long aBlock = (long)aDims[order - 1] * aDims[order - 2];
    long bBlock = (long)bDims[order - 1] * bDims[order - 2];
    long cBlock = (long)cDims[order - 1] * cDims[order - 2];
    int blockNum = 1;
    for (int i = 0; i < order - 2; i++) {
        if (aDims[i] != cDims[i] || bDims[i] != cDims[i])
            return -1;
        blockNum *= aDims[i];
    }

    /* :201-210, one _MatrixMul2D per block */
    for (int i = 0; i < blockNum; i++) {
        int r = oracle_matmul2d(a + i * aBlock, transA, b + i * bBlock, transB, c + i * cBlock,
                                aDims[order - 2], aDims[order - 1],
                                bDims[order - 2], bDims[order - 1],
                                cn, cm, alpha, beta);
        if (r != 0)
            return r;
    }
    return 0;
}

static long unit_num(const int *dims, int order)
{
    long n = 1;
    for (int i = 0; i < order; i++)
        n *= dims[i];
    return n;
}

int oracle_matmul(const float *a, int transA, const int *aDims, int aOrder,
                  const float *b, int transB, const int *bDims, int bOrder,
                  float *c, const int *cDims, int cOrder,
                  float alpha, float beta)
{
    /* MatrixMul.cpp:56-61 */
    if (aOrder < 2 || bOrder < 2 || cOrder < 2)
        return -1;
    if (cOrder != aOrder + bOrder - 2)
        return -1;

    /* MatrixMul.cpp:65-78: a higher-order, untransposed a times a matrix b is
       one 2-D product over the flattened leading dimensions */
    if (transA == ORACLE_X_NOTRANS && aOrder > 2 && bOrder == 2) {
        int ncolA = aDims[aOrder - 1];
        int ncolC = cDims[cOrder - 1];
        return oracle_matmul2d(a, transA, b, transB, c,
                               (int)(unit_num(aDims, aOrder) / ncolA), ncolA,
                               bDims[0], bDims[1],
                               (int)(unit_num(cDims, cOrder) / ncolC), ncolC,
                               alpha, beta);
    }

    /* MatrixMul.cpp:80-110 */
    int an = transA == ORACLE_X_TRANS ? aDims[aOrder - 1] : aDims[aOrder - 2];
    int am = transA == ORACLE_X_TRANS ? aDims[aOrder - 2] : aDims[aOrder - 1];
    int bn = transB == ORACLE_X_TRANS ? bDims[bOrder - 1] : bDims[bOrder - 2];
    int bm = transB == ORACLE_X_TRANS ? bDims[bOrder - 2] : bDims[bOrder - 1];
    int cn = cDims[cOrder - 2];
    int cm = cDims[cOrder - 1];
    if (!(am == bn && an == cn && bm == cm))
        return -1;

    long aBlock = (long)aDims[aOrder - 1] * aDims[aOrder - 2];
    long bBlock = (long)bDims[bOrder - 1] * bDims[bOrder - 2];
    long cBlock = (long)cDims[cOrder - 1] * cDims[cOrder - 2];
    int aBlockNum = 1, bBlockNum = 1;
    for (int i = 0; i < aOrder - 2; i++) {
        if (aDims[i] != cDims[i])
            return -1;
        aBlockNum *= aDims[i];
    }
    for (int i = 0; i < bOrder - 2; i++) {
        if (bDims[i] != cDims[i - 2 + aOrder])
            return -1;
        bBlockNum *= bDims[i];
    }

    /* MatrixMul.cpp:121-146 pairs every block p of a with every block q of b;
       the result block sits at p * bBlockNum + q. The CPU list path then runs
       one _MatrixMul2D per pair (MatrixMulBatched.cpp:257-270). */
    for (int p = 0; p < aBlockNum; p++) {
        for (int q = 0; q < bBlockNum; q++) {
            int r = oracle_matmul2d(a + p * aBlock, transA, b + q * bBlock, transB,
                                    c + ((long)p * bBlockNum + q) * cBlock,
                                    aDims[aOrder - 2], aDims[aOrder - 1],
                                    bDims[bOrder - 2], bDims[bOrder - 1],
                                    cn, cm, alpha, beta);
            if (r != 0)
                return r;
        }
    }
    return 0;
}

/* ---- bias broadcast ------------------------------------------------------ */

int oracle_broadcast_dim_index(const int *aDims, int aOrder, const int *bDims, int bOrder)
{
    /* Sum.cpp:235-238 */
    if (aOrder < bOrder)
        return -1;
    if (aOrder == bOrder) {
        int same = 1;
        for (int i = 0; i < aOrder; i++)
            if (aDims[i] != bDims[i])
                same = 0;
        if (same)
            return -1;
    }

    /* Sum.cpp:240-259: b may have one dimension that is not 1; the answer is
       the LAST dimension of a with that size */
    int hitDim = -1;
    int isHit = 0;
    for (int i = 0; i < bOrder; i++) {
        if (bDims[bOrder - 1 - i] == 1)
            continue;
        if (isHit)
            return -1;
        isHit = 1;
        for (int j = 0; j < aOrder; j++) {
            if (bDims[bOrder - 1 - i] == aDims[aOrder - 1 - j]) {
                hitDim = aOrder - 1 - j;
                break;
            }
        }
    }
    return hitDim;
}

int oracle_sumdim(const float *a, const int *aDims, int aOrder,
                  const float *b, int bUnitNum, float *c, int n, float beta)
{
    /* SumDim.cpp:51 MODX */
    if (aOrder != 0)
        n = (int)(n - floor((double)n / aOrder) * aOrder);
    if (aDims[n] != bUnitNum)
        return -1;

    long num = unit_num(aDims, aOrder);

    /* SumDim.cpp:63-66 */
    if (beta == 0) {
        memmove(c, a, sizeof(float) * (size_t)num);
        return 0;
    }

    /* SumDim.cpp:81-91 */
    int stride = 1;
    int blockSize = aDims[n];
    for (int i = aOrder - 1; i >= 0; i--) {
        if (i > n)
            stride *= aDims[i];
    }

    if (stride > 1) {
        /* SumDim.cpp:95-102 */
        long j = 0;
        for (long i = 0; i < num; i += stride, j++) {
            const float *ap = a + i;
            float bv = b[j % blockSize] * beta;
            float *cp = c + i;
            for (int k = 0; k < stride; k++)
                cp[k] = ap[k] + bv;
        }
    }
    else {
        /* SumDim.cpp:103-117 */
        for (long i = 0; i < num; i += blockSize) {
            const float *ap = a + i;
            float *cp = c + i;
            if (beta == 1.0F) {
                for (int j = 0; j < blockSize; j++)
                    cp[j] = ap[j] + b[j];
            }
            else {
                for (int j = 0; j < blockSize; j++)
                    cp[j] = ap[j] + b[j] * beta;
            }
        }
    }
    return 0;
}

int oracle_mulandshift(const float *x, int transX, const int *xDims, int xOrder,
                       const float *w, int transW, const int *wDims, int wOrder,
                       const float *bias, const int *bDims, int bOrder,
                       float *c, int *cDims, int *cOrder, float alpha)
{
    if (xOrder < 2 || wOrder < 2)
        return -1;

    /* MulAndShift.cpp:44-60 and :128-142 */
    int xn = transX == ORACLE_X_TRANS ? xDims[xOrder - 1] : xDims[xOrder - 2];
    int wm = transW == ORACLE_X_TRANS ? wDims[wOrder - 2] : wDims[wOrder - 1];
    int order = xOrder + wOrder - 2;
    int sub = 0;
    for (int i = 0; i < xOrder - 2; i++)
        cDims[sub++] = xDims[i];
    for (int i = 0; i < wOrder - 2; i++)
        cDims[sub++] = wDims[i];
    cDims[sub++] = xn;
    cDims[sub++] = wm;
    *cOrder = order;

    long num = unit_num(cDims, order);
    float *tmp = (float *)malloc(sizeof(float) * (size_t)(num > 0 ? num : 1));
    if (!tmp)
        return -1;

    /* :69 / :151 */
    int r = oracle_matmul(x, transX, xDims, xOrder, w, transW, wDims, wOrder,
                          tmp, cDims, order, alpha, 0);
    if (r != 0) {
        free(tmp);
        return -1;
    }

    int n;
    if (bOrder == 0) {
        /* :74-75 (first overload only): ScaleAndShift(tmp, c, 1, b) */
        if (transX != ORACLE_X_NOTRANS || transW != ORACLE_X_NOTRANS) {
            free(tmp);
            return -2;
        }
        for (long i = 0; i < num; i++)
            c[i] = tmp[i] * 1.0F + bias[0];
        n = order;   /* no broadcast dimension */
    }
    else {
        /* :77-92 */
        n = oracle_broadcast_dim_index(cDims, order, bDims, bOrder);
        if (n < 0 || n >= order) {
            free(tmp);
            return -2;   /* the reference aborts here ("TODO!") */
        }
        if (oracle_sumdim(tmp, cDims, order, bias, (int)unit_num(bDims, bOrder), c, n, 1.0F) != 0) {
            free(tmp);
            return -2;
        }
    }
    free(tmp);
    return n;
}

/* ---- backward: the products and sums the autograd issues for this path ------ */

int oracle_reduce_sum(const float *in, const int *dims, int order, int dim, float *out)
{
    /* ReduceSum.cpp:47-80 */
    if (order < 1 || dim < 0 || dim >= order)
        return -1;
    int stride = 1, strideNum = dims[dim], blockNum = 1;
    for (int i = 0; i < order; i++) {
        if (i < dim)
            blockNum *= dims[i];
        else if (i > dim)
            stride *= dims[i];
    }
    long blockSize = (long)stride * strideNum;
    int last = dims[order - 1];

    if (last % 32 == 0 && last >= 32 && dim == order - 1) {
        /* ReduceSum.cpp:83-116: 32 running sums (four buffers of eight lanes) over the
           contiguous items, folded as (b0 + b1) + (b2 + b3) and then lane by lane from 0 */
        for (int i = 0; i < blockNum; i++) {
            const float *ip = in + blockSize * i;
            float buf[4][8];
            for (int k = 0; k < 4; k++)
                for (int l = 0; l < 8; l++)
                    buf[k][l] = ip[k * 8 + l] - 0.0F;
            for (int j = 1; j < strideNum / 32; j++)
                for (int k = 0; k < 4; k++)
                    for (int l = 0; l < 8; l++)
                        buf[k][l] = (ip[j * 32 + k * 8 + l] - 0.0F) + buf[k][l];
            float sum = 0.0F;
            for (int l = 0; l < 8; l++) {
                /* operator+ computes a[i] + this[i]: the right operand comes first */
                float b01 = buf[1][l] + buf[0][l];
                float b23 = buf[3][l] + buf[2][l];
                sum = sum + (b23 + b01);
            }
            out[i] = sum;
        }
        return 0;
    }
    /* ReduceSum.cpp:117-143 (buffers over columns) and :146-228 (scalar loop) both add the
       items of one output element one after the other, in ascending position along dim;
       the first starts from the first item, the second from 0 */
    int vector = last % 32 == 0 && last >= 32;
    for (int k = 0; k < blockNum; k++) {
        const float *ip = in + blockSize * k;
        float *op = out + (long)stride * k;
        for (int i = 0; i < stride; i++) {
            float sum;
            int first;
            if (vector) {
                sum = ip[i] - 0.0F;
                first = 1;
            }
            else {
                sum = 0;
                first = 0;
            }
            for (int j = first; j < strideNum; j++) {
                if (vector)
                    sum = (ip[(long)j * stride + i] - 0.0F) + sum;
                else
                    sum += ip[(long)j * stride + i];
            }
            op[i] = sum;
        }
    }
    return 0;
}

int oracle_grad_matmul2d(const float *a, float *deda, int transA,
                         const float *b, float *dedb, int transB,
                         const float *dedc, int na, int ma, int nb, int mb, float alpha)
{
    /* shape of c as _MatrixMul2D sees it (MatrixMul2D.cpp:56-67) */
    int cn = transA == ORACLE_X_TRANS ? ma : na;
    int cm = transB == ORACLE_X_TRANS ? nb : mb;
    int r = 0;
    const int T = ORACLE_X_TRANS, NT = ORACLE_X_NOTRANS;
    /* XBackwardMath.cpp:636-696: every gradient is ADDED to what the tensor holds (beta = 1) */
    if (transA == NT && transB == NT) {
        if (deda)
            r |= oracle_matmul2d(dedc, NT, b, T, deda, cn, cm, nb, mb, na, ma, alpha, 1.0F);
        if (dedb)
            r |= oracle_matmul2d(a, T, dedc, NT, dedb, na, ma, cn, cm, nb, mb, alpha, 1.0F);
    }
    else if (transA == T && transB == NT) {
        if (deda)
            r |= oracle_matmul2d(b, NT, dedc, T, deda, nb, mb, cn, cm, na, ma, alpha, 1.0F);
        if (dedb)
            r |= oracle_matmul2d(a, NT, dedc, NT, dedb, na, ma, cn, cm, nb, mb, alpha, 1.0F);
    }
    else if (transA == NT && transB == T) {
        if (deda)
            r |= oracle_matmul2d(dedc, NT, b, NT, deda, cn, cm, nb, mb, na, ma, alpha, 1.0F);
        if (dedb)
            r |= oracle_matmul2d(dedc, T, a, NT, dedb, cn, cm, na, ma, nb, mb, alpha, 1.0F);
    }
    else {
        if (deda)
            r |= oracle_matmul2d(b, T, dedc, T, deda, nb, mb, cn, cm, na, ma, alpha, 1.0F);
        if (dedb)
            r |= oracle_matmul2d(dedc, T, a, T, dedb, cn, cm, na, ma, nb, mb, alpha, 1.0F);
    }
    return r;
}

int oracle_grad_matmul(const float *a, float *deda, int transA, const int *aDims, int aOrder,
                       const float *b, float *dedb, int transB, const int *bDims, int bOrder,
                       const float *dedc, float alpha)
{
    /* XBackwardMath.cpp:608-633 */
    if (aOrder == 2 && bOrder == 2)
        return oracle_grad_matmul2d(a, deda, transA, b, dedb, transB, dedc,
                                    aDims[0], aDims[1], bDims[0], bDims[1], alpha);
    if (transA == ORACLE_X_NOTRANS && aOrder > 2 && bOrder == 2) {
        int ncolA = aDims[aOrder - 1];
        return oracle_grad_matmul2d(a, deda, transA, b, dedb, transB, dedc,
                                    (int)(unit_num(aDims, aOrder) / ncolA), ncolA, bDims[0], bDims[1], alpha);
    }
    return -2;      /* ShowNTErrors("TODO!") */
}

int oracle_grad_matmul_batched(const float *a, float *deda, int transA, const int *aDims,
                               const float *b, float *dedb, int transB, const int *bDims,
                               const float *dedc, const int *cDims, int order, float alpha)
{
    const int T = ORACLE_X_TRANS, NT = ORACLE_X_NOTRANS;
    int r = 0;
    /* XBackwardMath.cpp:731-786: the same eight products, batched */
    if (transA == NT && transB == NT) {
        if (deda)
            r |= oracle_matmul_batched(dedc, NT, cDims, b, T, bDims, deda, aDims, order, alpha, 1.0F);
        if (dedb)
            r |= oracle_matmul_batched(a, T, aDims, dedc, NT, cDims, dedb, bDims, order, alpha, 1.0F);
    }
    else if (transA == T && transB == NT) {
        if (deda)
            r |= oracle_matmul_batched(b, NT, bDims, dedc, T, cDims, deda, aDims, order, alpha, 1.0F);
        if (dedb)
            r |= oracle_matmul_batched(a, NT, aDims, dedc, NT, cDims, dedb, bDims, order, alpha, 1.0F);
    }
    else if (transA == NT && transB == T) {
        if (deda)
            r |= oracle_matmul_batched(dedc, NT, cDims, b, NT, bDims, deda, aDims, order, alpha, 1.0F);
        if (dedb)
            r |= oracle_matmul_batched(dedc, T, cDims, a, NT, aDims, dedb, bDims, order, alpha, 1.0F);
    }
    else {
        if (deda)
            r |= oracle_matmul_batched(b, T, bDims, dedc, T, cDims, deda, aDims, order, alpha, 1.0F);
        if (dedb)
            r |= oracle_matmul_batched(dedc, T, cDims, a, T, aDims, dedb, bDims, order, alpha, 1.0F);
    }
    return r;
}

int oracle_grad_mulandshift(const float *x, float *dedx, int transX, const int *xDims, int xOrder,
                            const float *w, float *dedw, int transW, const int *wDims, int wOrder,
                            float *dedbias, int biasNum,
                            const float *dedc, const int *cDims, int cOrder, int n, float alpha)
{
    long num = unit_num(cDims, cOrder);
    if (dedbias) {
        float *tmp = (float *)malloc(sizeof(float) * (size_t)(biasNum > 0 ? biasNum : 1));
        if (!tmp)
            return -1;
        if (n == cOrder - 1) {
            /* XBackwardMath.cpp:1797-1814: dE/dc as a matrix with |b| columns, summed over its
               rows into a temporary, which _Sum then adds to the gradient (c = a + b * 1) */
            int d2[2] = {(int)(num / cDims[cOrder - 1]), cDims[cOrder - 1]};
            if (d2[1] != biasNum || oracle_reduce_sum(dedc, d2, 2, 0, tmp) != 0) {
                free(tmp);
                return -1;
            }
        }
        else {
            /* :1816-1846: dE/dc as (x, |b|, z), summed over z, then over x */
            int d3[3] = {1, cDims[n], 1};
            for (int i = 0; i < n; i++)
                d3[0] *= cDims[i];
            d3[2] = (int)(num / ((long)d3[0] * d3[1]));
            float *inter = (float *)malloc(sizeof(float) * (size_t)d3[0] * d3[1]);
            if (!inter || d3[1] != biasNum) {
                free(inter);
                free(tmp);
                return -1;
            }
            oracle_reduce_sum(dedc, d3, 3, 2, inter);
            oracle_reduce_sum(inter, d3, 2, 0, tmp);
            free(inter);
        }
        for (int i = 0; i < biasNum; i++)
            dedbias[i] = tmp[i] + dedbias[i];
        free(tmp);
    }
    /* :1857-1879: the products of GradMatrixMul on x and w */
    return oracle_grad_matmul(x, dedx, transX, xDims, xOrder, w, dedw, transW, wDims, wOrder, dedc, alpha);
}

/* ---- attention: the operator chain of the transformer sample -------------------- */

int oracle_softmax(const float *x, long rows, int n, float *y)
{
    if (n <= 0)
        return -1;
    for (long i = 0; i < rows; i++) {
        const float *ip = x + i * n;
        float *op = y + i * n;
        /* _ReduceMax over the row (ReduceMax.cpp): the maximum does not depend on the order */
        float mx = ip[0];
        for (int j = 1; j < n; j++)
            mx = ip[j] > mx ? ip[j] : mx;
        /* _ReduceSum(x, sum, leadDim, max, 1.0F, true): sum of (DTYPE)exp(x - max), in the
           order of ReduceSum.cpp. Which exp runs depends on the file: ReduceSum.cpp and Softmax.cpp call
           exp on a float and get C++'s float overload; VectorBuffer.cpp (the 32-lane path) gets the
           double one and rounds the result to float (both established against the compiled reference): 32 running sums folded at the end when the row length is a
           multiple of 32 (:83-116), one running sum from 0 otherwise (:146-228) */
        float sum;
        if (n % 32 == 0 && n >= 32) {
            float buf[4][8];
            for (int k = 0; k < 4; k++)
                for (int l = 0; l < 8; l++)
                    buf[k][l] = (float)exp(ip[k * 8 + l] - mx);
            for (int j = 1; j < n / 32; j++)
                for (int k = 0; k < 4; k++)
                    for (int l = 0; l < 8; l++)
                        buf[k][l] = (float)exp(ip[j * 32 + k * 8 + l] - mx) + buf[k][l];
            sum = 0.0F;
            for (int l = 0; l < 8; l++) {
                float b01 = buf[1][l] + buf[0][l];
                float b23 = buf[3][l] + buf[2][l];
                sum = sum + (b23 + b01);
            }
        }
        else {
            sum = 0;
            for (int j = 0; j < n; j++)
                sum += expf(ip[j] - mx);
        }
        /* Softmax.cpp:92-109 */
        if (sum == 0) {
            for (int j = 0; j < n; j++)
                op[j] = 0;
        }
        else {
            for (int j = 0; j < n; j++) {
                float r = expf(ip[j] - mx) / sum;
                if (r > 1.0F)
                    r = 1.0F;
                else if (r < 0)
                    r = 0;
                op[j] = r;
            }
        }
    }
    return 0;
}

/* shared by the two entry points below: probs (may be NULL) receives Softmax(...), out (may be NULL, then v may be) the result */
static int attention_chain(const float *q, const float *k, const float *v, const float *mask, float *probs, float *out,
                           int batch, int lq, int lk, int hidden, int heads, float scale)
{
    if (heads <= 0 || hidden % heads != 0)
        return -1;
    const int dh = hidden / heads;
    const long nq = (long)heads * batch * lq * dh, nk = (long)heads * batch * lk * dh;
    const long na = (long)heads * batch * lq * lk;
    float *qh = (float *)malloc(sizeof(float) * (size_t)(nq > 0 ? nq : 1));
    float *kh = (float *)malloc(sizeof(float) * (size_t)(nk > 0 ? nk : 1));
    float *vh = (float *)malloc(sizeof(float) * (size_t)(nk > 0 ? nk : 1));
    float *att = (float *)malloc(sizeof(float) * (size_t)(na > 0 ? na : 1));
    float *prob = (float *)malloc(sizeof(float) * (size_t)(na > 0 ? na : 1));
    float *oh = (float *)malloc(sizeof(float) * (size_t)(nq > 0 ? nq : 1));
    int r = -1;
    if (qh && kh && vh && att && prob && oh) {
        /* Attention.cpp:194-198: Split(x, order - 1, nhead): head h takes columns h*dh .. of every row
           and becomes block h of a [heads][batch][rows][dh] tensor (Split.cpp) */
        for (int h = 0; h < heads; h++)
            for (int b = 0; b < batch; b++) {
                for (int l = 0; l < lq; l++)
                    for (int j = 0; j < dh; j++)
                        /* :202-205 Scale / ScaleMe of q: v * scale + 0 (ScaleAndShift.cpp:70-75) */
                        qh[(((long)h * batch + b) * lq + l) * dh + j] = q[((long)b * lq + l) * hidden + h * dh + j] * scale + 0.0F;
                for (int l = 0; l < lk; l++)
                    for (int j = 0; j < dh; j++) {
                        kh[(((long)h * batch + b) * lk + l) * dh + j] = k[((long)b * lk + l) * hidden + h * dh + j];
                        if (v)
                            vh[(((long)h * batch + b) * lk + l) * dh + j] = v[((long)b * lk + l) * hidden + h * dh + j];
                    }
            }
        int dq[4] = {heads, batch, lq, dh}, dk[4] = {heads, batch, lk, dh}, da[4] = {heads, batch, lq, lk};
        /* :208-211 BMMul(q, X_NOTRANS, kheads, X_TRANS) */
        r = oracle_matmul_batched(qh, ORACLE_X_NOTRANS, dq, kh, ORACLE_X_TRANS, dk, att, da, 4, 1.0F, 0.0F);
        /* :217-222 Sum / SumMe with the mask: c = a + b */
        if (r == 0 && mask)
            for (long i = 0; i < na; i++)
                att[i] = att[i] + mask[i];
        /* :224 Softmax(att, -1) */
        if (r == 0)
            r = oracle_softmax(att, (long)heads * batch * lq, lk, prob);
        if (r == 0 && probs)
            memcpy(probs, prob, sizeof(float) * (size_t)na);
        /* :232-235 BMMul(att, vheads) */
        if (r == 0 && out)
            r = oracle_matmul_batched(prob, ORACLE_X_NOTRANS, da, vh, ORACLE_X_NOTRANS, dk, oh, dq, 4, 1.0F, 0.0F);
        /* :239 Merge(att, order - 1): block h goes back to columns h*dh .. (Merge.cpp) */
        if (r == 0 && out)
            for (int h = 0; h < heads; h++)
                for (int b = 0; b < batch; b++)
                    for (int l = 0; l < lq; l++)
                        for (int j = 0; j < dh; j++)
                            out[((long)b * lq + l) * hidden + h * dh + j] = oh[(((long)h * batch + b) * lq + l) * dh + j];
    }
    free(qh); free(kh); free(vh); free(att); free(prob); free(oh);
    return r;
}

int oracle_attention(const float *q, const float *k, const float *v, const float *mask, float *out,
                     int batch, int lq, int lk, int hidden, int heads, float scale)
{
    return attention_chain(q, k, v, mask, NULL, out, batch, lq, lk, hidden, heads, scale);
}

int oracle_attention_probs(const float *q, const float *k, const float *mask, float *probs,
                           int batch, int lq, int lk, int hidden, int heads, float scale)
{
    return attention_chain(q, k, NULL, mask, probs, NULL, batch, lq, lk, hidden, heads, scale);
}

/* ---- rectify ------------------------------------------------------------------ */

void oracle_rectify(const float *x, long n, float *y)
{
    for (long i = 0; i < n; i++) {
        float p = x[i];
        if (p < 0)
            p = 0;
        y[i] = p;
    }
}

/* ---- data type conversion ------------------------------------------------- */

int oracle_convert_data_type(const void *s, int typeS, void *t, int typeT, long n)
{
    if (typeS == typeT)
        return 0;
    if (typeS == 2 && typeT == 3)
        oracle_f32_to_f16_array((const float *)s, (uint16_t *)t, n);
    else if (typeS == 3 && typeT == 2)
        oracle_f16_to_f32_array((const uint16_t *)s, (float *)t, n);
    else if (typeS == 2 && typeT == 0) {
        const float *in = (const float *)s;
        int *out = (int *)t;
        for (long i = 0; i < n; i++) {
            float x = in[i];
            if (x != x)
                out[i] = 0;
            else if (x >= 2147483648.0F)
                out[i] = 0x7fffffff;
            else if (x <= -2147483648.0F)
                out[i] = (int)0x80000000;
            else
                out[i] = (int)x;
        }
    }
    else if (typeS == 0 && typeT == 2) {
        const int *in = (const int *)s;
        float *out = (float *)t;
        for (long i = 0; i < n; i++)
            out[i] = (float)in[i];
    }
    else
        return -1;
    return 0;
}

/* ---- comparator ---------------------------------------------------------- */

int oracle_is_float_equal(float a, float b, float absError, float relError)
{
    /* CheckData.cpp:29-39 */
    if (a == b)
        return 1;
    if (fabs(a - b) < absError)
        return 1;
    if (fabs(a) < fabs(b))
        return fabs((a - b) / b) < relError ? 1 : 0;
    else
        return fabs((a - b) / a) < relError ? 1 : 0;
}

int oracle_check_data(const float *value, const float *answer, int num, float tolerance)
{
    for (int i = 0; i < num; i++)
        if (!oracle_is_float_equal(value[i], answer[i], tolerance, 1e-4F))
            return 0;
    return 1;
}

/* ---- binary16 ------------------------------------------------------------ */

uint16_t oracle_f32_to_f16(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t absx = x & 0x7fffffffu;

    if (absx >= 0x7f800000u)                      /* Inf or NaN */
        return (uint16_t)(sign | 0x7c00u | (absx > 0x7f800000u ? 0x0200u | ((absx >> 13) & 0x3ffu) : 0));
    if (absx >= 0x477ff000u)                      /* rounds to >= 65520 => Inf */
        return (uint16_t)(sign | 0x7c00u);
    if (absx < 0x33000001u)                       /* <= 2^-25 => 0 (ties to even) */
        return (uint16_t)sign;

    int exp = (int)(absx >> 23) - 127;
    uint32_t man = (absx & 0x7fffffu) | 0x800000u;   /* 24-bit significand */
    int shift;
    uint32_t base;
    if (exp < -14) {                              /* sub-normal half */
        shift = 13 + (-14 - exp);
        base = 0;
    }
    else {
        shift = 13;
        base = (uint32_t)(exp + 15) << 10;
        man &= 0x7fffffu;
    }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u)))
        q++;                                      /* a carry moves into the exponent */
    return (uint16_t)(sign | (base + q));
}

float oracle_f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t x;
    if (exp == 0) {
        if (man == 0)
            x = sign;
        else {
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while (!(man & 0x400u));
            x = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
        }
    }
    else if (exp == 31)
        x = sign | 0x7f800000u | (man << 13);
    else
        x = sign | ((exp + 112u) << 23) | (man << 13);
    float f;
    memcpy(&f, &x, 4);
    return f;
}

void oracle_f32_to_f16_array(const float *src, uint16_t *dst, long n)
{
    for (long i = 0; i < n; i++)
        dst[i] = oracle_f32_to_f16(src[i]);
}

void oracle_f16_to_f32_array(const uint16_t *src, float *dst, long n)
{
    for (long i = 0; i < n; i++)
        dst[i] = oracle_f16_to_f32(src[i]);
}

/* ---- seeded fills -------------------------------------------------------- */

static uint64_t splitmix64(uint64_t *s)
{
    uint64_t z = (*s += 0x9e3779b97f4a7c15ull);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

/* 53 random bits -> [0,1) */
static double u01(uint64_t *s)
{
    return (double)(splitmix64(s) >> 11) * (1.0 / 9007199254740992.0);
}

void oracle_fill_uniform(float *x, long n, uint64_t seed, float lo, float hi)
{
    uint64_t s = seed;
    for (long i = 0; i < n; i++)
        x[i] = (float)(lo + (hi - lo) * u01(&s));
}

void oracle_fill_normal(float *x, long n, uint64_t seed, float mean, float std)
{
    uint64_t s = seed;
    for (long i = 0; i < n; i += 2) {
        double u1 = 1.0 - u01(&s);   /* (0,1] */
        double u2 = u01(&s);
        double r = sqrt(-2.0 * log(u1));
        double t = 6.283185307179586476925286766559 * u2;
        x[i] = (float)(mean + std * r * cos(t));
        if (i + 1 < n)
            x[i + 1] = (float)(mean + std * r * sin(t));
    }
}
