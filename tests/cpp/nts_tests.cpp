/*
 * Tests of the nts:: host layer on a gfx950 GPU, written the way the reference
 * writes its own (source/tensor/test/TMatrixMul.cpp, TMatrixMul2D.cpp,
 * TMatrixMulBatched.cpp): literal inputs, the operation, a comparison with the
 * known answer through the reference's comparator (abs 1e-4 or rel 1e-4,
 * core/utilities/CheckData.cpp:29-39). The GPU halves of those tests are what is
 * reproduced here; cases the reference does not have (NT/TT, alpha/beta, fp16,
 * MulAndShift, lists, the backward step) are checked against the CPU oracle on seeded inputs.
 *
 *   nts_tests                run everything on device 0, exit 0 if all passed
 *   nts_tests --alloc-bench  time an allocating call with and without reuse of device blocks
 *   nts_tests --bench        time the operators of the baseline's configurations 2 to 5 through this layer
 *                            (MulAndShift, MatrixMulBatched twice, MatrixMul twice): one JSON line each
 *   nts_tests --host         the dispatch of host tensors to the functions a host tree hands in (no GPU needed)
 *   nts_tests --abort NAME   provoke one fatal error (no GPU needed): the process
 *                            must print the reference's message and abort
 */
#include "../../niutensor_amd/nts/XTensor.h"
#include "../../niutensor_amd/nts/MatrixMul.h"
#include "../../niutensor_amd/nts/MatrixMul2D.h"
#include "../../niutensor_amd/nts/MatrixMulBatched.h"
#include "../../niutensor_amd/nts/MulAndShift.h"
#include "../../niutensor_amd/nts/XBackwardMath.h"
#include "../../niutensor_amd/nts/ConvertDataType.h"
#include "../../niutensor_amd/nts/Attention.h"
#include "../../oracle/nts_oracle.h"

#include "../../include/ntsamd_gemm.h"
#include <hip/hip_runtime_api.h>

#include <chrono>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <thread>
#include <vector>

using namespace nts;

static const int DEV = 0;

/* _CheckData of the reference for a device tensor: read back, compare element-wise */
static bool CheckData(const XTensor * t, const void * answer, int num, float tolerance)
{
    if (t->data == NULL || answer == NULL || num != t->unitNum)
        return false;
    std::vector<float> host(num);
    t->GetData(host.data());
    return oracle_check_data(host.data(), (const float *)answer, num, tolerance) != 0;
}

static XTensor * NewGPU(int order, const int * dims, const float * data, TENSOR_DATA_TYPE type = X_FLOAT)
{
    XTensor * t = NewTensorV2(order, dims, type, 1.0F, DEV);
    if (data != NULL) {
        if (type == X_FLOAT)
            t->SetData(data, t->unitNum);
        else {
            std::vector<uint16_t> h(t->unitNum);
            oracle_f32_to_f16_array(data, h.data(), t->unitNum);
            t->SetData(h.data(), t->unitNum);
        }
    }
    return t;
}

/* ---- the reference's known-answer cases, GPU halves ------------------------- */

/* TMatrixMul.cpp case 1 / TMatrixMul2D.cpp case 1 / TMatrixMulBatched.cpp case 1: (2,3) x (3,2) */
static bool TestMatrixMul1()
{
    int d1[2] = {2, 3}, d2[2] = {3, 2}, dt[2] = {2, 2};
    DTYPE sData1[2][3] = {{1.0F, 2.0F, 3.0F}, {-4.0F, 5.0F, 6.0F}};
    DTYPE sData2[3][2] = {{0.0F, -1.0F}, {1.0F, 2.0F}, {2.0F, 1.0F}};
    DTYPE answer[2][2] = {{8.0F, 6.0F}, {17.0F, 20.0F}};

    XTensor * s1 = NewGPU(2, d1, &sData1[0][0]);
    XTensor * s2 = NewGPU(2, d2, &sData2[0][0]);
    XTensor * t = NewGPU(2, dt, NULL);
    XTensor * t2 = NewGPU(2, dt, NULL);
    XTensor * t3 = NewGPU(2, dt, NULL);
    XTensor tUser, tUserB;
    t->SetZeroAll();

    _MatrixMul(s1, X_NOTRANS, s2, X_NOTRANS, t);
    tUser = MatrixMul(*s1, X_NOTRANS, *s2, X_NOTRANS);
    _MatrixMul2D(s1, X_NOTRANS, s2, X_NOTRANS, t2);
    _MatrixMulBatched(s1, X_NOTRANS, s2, X_NOTRANS, t3);
    tUserB = MatrixMulBatched(*s1, X_NOTRANS, *s2, X_NOTRANS);

    bool ok = CheckData(t, answer, 4, 1e-4F) && CheckData(&tUser, answer, 4, 1e-4F) &&
              CheckData(t2, answer, 4, 1e-4F) && CheckData(t3, answer, 4, 1e-4F) &&
              CheckData(&tUserB, answer, 4, 1e-4F);
    delete s1; delete s2; delete t; delete t2; delete t3;
    return ok;
}

/* TMatrixMul.cpp case 2 / TMatrixMul2D.cpp case 2: a stored (3,2), X_TRANS */
static bool TestMatrixMul2()
{
    int d1[2] = {3, 2}, d2[2] = {3, 2}, dt[2] = {2, 2};
    DTYPE sData1[3][2] = {{1.0F, -4.0F}, {2.0F, 5.0F}, {3.0F, 6.0F}};
    DTYPE sData2[3][2] = {{0.0F, -1.0F}, {1.0F, 2.0F}, {2.0F, 1.0F}};
    DTYPE answer[2][2] = {{8.0F, 6.0F}, {17.0F, 20.0F}};

    XTensor * s1 = NewGPU(2, d1, &sData1[0][0]);
    XTensor * s2 = NewGPU(2, d2, &sData2[0][0]);
    XTensor * t = NewGPU(2, dt, NULL);
    XTensor * t2 = NewGPU(2, dt, NULL);
    XTensor tUser;

    _MatrixMul(s1, X_TRANS, s2, X_NOTRANS, t);
    tUser = MatrixMul(*s1, X_TRANS, *s2, X_NOTRANS);
    _MatrixMul2D(s1, X_TRANS, s2, X_NOTRANS, t2);

    bool ok = CheckData(t, answer, 4, 1e-4F) && CheckData(&tUser, answer, 4, 1e-4F) && CheckData(t2, answer, 4, 1e-4F);
    delete s1; delete s2; delete t; delete t2;
    return ok;
}

static DTYPE sData323[3][2][3] = {{{0.0F, -1.0F, 2.0F}, {2.0F, 1.0F, 3.0F}},
                                  {{1.0F, 2.0F, 4.0F}, {3.0F, 1.0F, 2.0F}},
                                  {{-1.0F, 3.0F, 2.0F}, {1.0F, -1.0F, 0.0F}}};
static DTYPE sData232[2][3][2] = {{{1.0F, 2.0F}, {-4.0F, 3.0F}, {2.0F, 6.0F}},
                                  {{1.0F, 2.0F}, {3.0F, 4.0F}, {5.0F, 6.0F}}};

/* TMatrixMul.cpp case 3: (3,2,3) x (2,3,2) -> (3,2,2,2), every block of a with every block of b */
static bool TestMatrixMul3()
{
    int d1[3] = {3, 2, 3}, d2[3] = {2, 3, 2}, dt[4] = {3, 2, 2, 2};
    DTYPE answer[3][2][2][2] = {{{{8.0F, 9.0F}, {4.0F, 25.0F}}, {{7.0F, 8.0F}, {20.0F, 26.0F}}},
                                {{{1.0F, 32.0F}, {3.0F, 21.0F}}, {{27.0F, 34.0F}, {16.0F, 22.0F}}},
                                {{{-9.0F, 19.0F}, {5.0F, -1.0F}}, {{18.0F, 22.0F}, {-2.0F, -2.0F}}}};
    XTensor * s1 = NewGPU(3, d1, &sData323[0][0][0]);
    XTensor * s2 = NewGPU(3, d2, &sData232[0][0][0]);
    XTensor * t = NewGPU(4, dt, NULL);
    XTensor tUser;

    _MatrixMul(s1, X_NOTRANS, s2, X_NOTRANS, t);
    tUser = MatrixMul(*s1, X_NOTRANS, *s2, X_NOTRANS);

    bool ok = CheckData(t, answer, 24, 1e-4F) && CheckData(&tUser, answer, 24, 1e-4F) &&
              tUser.order == 4 && tUser.dimSize[0] == 3 && tUser.dimSize[1] == 2;
    delete s1; delete s2; delete t;
    return ok;
}

/* TMatrixMul.cpp case 4: (3,2,3) x (3,2) -> (3,2,2), the flattened product */
static bool TestMatrixMul4()
{
    int d1[3] = {3, 2, 3}, d2[2] = {3, 2}, dt[3] = {3, 2, 2};
    DTYPE sData2[3][2] = {{1.0F, 2.0F}, {3.0F, 4.0F}, {5.0F, 6.0F}};
    DTYPE answer[3][2][2] = {{{7.0F, 8.0F}, {20.0F, 26.0F}}, {{27.0F, 34.0F}, {16.0F, 22.0F}}, {{18.0F, 22.0F}, {-2.0F, -2.0F}}};
    XTensor * s1 = NewGPU(3, d1, &sData323[0][0][0]);
    XTensor * s2 = NewGPU(2, d2, &sData2[0][0]);
    XTensor * t = NewGPU(3, dt, NULL);
    XTensor tUser;

    _MatrixMul(s1, X_NOTRANS, s2, X_NOTRANS, t);
    tUser = MatrixMul(*s1, X_NOTRANS, *s2, X_NOTRANS);

    bool ok = CheckData(t, answer, 12, 1e-4F) && CheckData(&tUser, answer, 12, 1e-4F);
    delete s1; delete s2; delete t;
    return ok;
}

/* TMatrixMulBatched.cpp case 2: (2,2,3) x (2,3,2) -> (2,2,2), block i with block i */
static bool TestMatrixMulBatched2()
{
    int d1[3] = {2, 2, 3}, d2[3] = {2, 3, 2}, dt[3] = {2, 2, 2};
    DTYPE answer[2][2][2] = {{{8.0F, 9.0F}, {4.0F, 25.0F}}, {{27.0F, 34.0F}, {16.0F, 22.0F}}};
    XTensor * s1 = NewGPU(3, d1, &sData323[0][0][0]);
    XTensor * s2 = NewGPU(3, d2, &sData232[0][0][0]);
    XTensor * t = NewGPU(3, dt, NULL);
    XTensor tUser;

    _MatrixMulBatched(s1, X_NOTRANS, s2, X_NOTRANS, t);
    tUser = MatrixMulBatched(*s1, X_NOTRANS, *s2, X_NOTRANS);

    bool ok = CheckData(t, answer, 8, 1e-4F) && CheckData(&tUser, answer, 8, 1e-4F);
    delete s1; delete s2; delete t;
    return ok;
}

/* ---- seeded cases against the CPU oracle ------------------------------------- */

static float MaxRelErr(const std::vector<float> & got, const std::vector<float> & ref)
{
    float mx = 0;
    for (size_t i = 0; i < ref.size(); i++)
        mx = fmaxf(mx, fabsf(ref[i]));
    float e = 0;
    for (size_t i = 0; i < ref.size(); i++)
        e = fmaxf(e, fabsf(got[i] - ref[i]) / mx);
    return e;
}

static int Prod(const int * d, int n)
{
    int p = 1;
    for (int i = 0; i < n; i++)
        p *= d[i];
    return p;
}

/* all four transposes with alpha, beta and ragged sizes: fp32 within 1e-5 * sqrt(K) of the oracle */
static bool TestMatrixMulSeeded()
{
    bool ok = true;
    int sizes[4][3] = {{37, 29, 53}, {130, 70, 33}, {256, 128, 64}, {5, 300, 17}};
    for (int s = 0; s < 4; s++) {
        int M = sizes[s][0], N = sizes[s][1], K = sizes[s][2];
        for (int ta = 0; ta < 2; ta++) {
            for (int tb = 0; tb < 2; tb++) {
                int da[2] = {ta == X_TRANS ? K : M, ta == X_TRANS ? M : K};
                int db[2] = {tb == X_TRANS ? N : K, tb == X_TRANS ? K : N};
                int dc[2] = {M, N};
                std::vector<float> a(M * K), b(K * N), c0(M * N), ref(M * N), got(M * N);
                oracle_fill_uniform(a.data(), M * K, 100 + s, -1, 1);
                oracle_fill_uniform(b.data(), K * N, 200 + s, -1, 1);
                oracle_fill_uniform(c0.data(), M * N, 300 + s, -1, 1);
                ref = c0;
                oracle_matmul2d(a.data(), ta, b.data(), tb, ref.data(), da[0], da[1], db[0], db[1], M, N, 0.5F, 1.0F);
                XTensor * ga = NewGPU(2, da, a.data());
                XTensor * gb = NewGPU(2, db, b.data());
                XTensor * gc = NewGPU(2, dc, c0.data());
                _MatrixMul(ga, (MATRIX_TRANS_TYPE)ta, gb, (MATRIX_TRANS_TYPE)tb, gc, 0.5F, 1.0F);
                gc->GetData(got.data());
                float e = MaxRelErr(got, ref);
                if (!(e <= 1e-5F * sqrtf((float)K))) {
                    fprintf(stderr, "seeded %dx%dx%d ta=%d tb=%d err=%g\n", M, N, K, ta, tb, e);
                    ok = false;
                }
                delete ga; delete gb; delete gc;
            }
        }
    }
    return ok;
}

/* a transposed N-D a against one matrix is NOT flattened: a batch that shares b */
static bool TestMatrixMulTransposedND()
{
    int da[3] = {4, 6, 10}, db[2] = {6, 7}, dc[3] = {4, 10, 7};
    std::vector<float> a(240), b(42), ref(280), got(280);
    oracle_fill_uniform(a.data(), 240, 1, -1, 1);
    oracle_fill_uniform(b.data(), 42, 2, -1, 1);
    oracle_matmul(a.data(), X_TRANS, da, 3, b.data(), X_NOTRANS, db, 2, ref.data(), dc, 3, 1.0F, 0.0F);
    XTensor * ga = NewGPU(3, da, a.data());
    XTensor * gb = NewGPU(2, db, b.data());
    XTensor tUser = MatrixMul(*ga, X_TRANS, *gb, X_NOTRANS);
    bool ok = tUser.order == 3 && tUser.dimSize[0] == 4 && tUser.dimSize[1] == 10 && tUser.dimSize[2] == 7;
    tUser.GetData(got.data());
    ok = ok && MaxRelErr(got, ref) < 1e-5F;
    delete ga; delete gb;
    return ok;
}

/* attention-shaped batch: S = Q K^T / 8, then S V */
static bool TestMatrixMulBatchedAttention()
{
    int dq[3] = {6, 50, 24}, dk[3] = {6, 40, 24}, ds[3] = {6, 50, 40}, dv[3] = {6, 40, 24}, dout[3] = {6, 50, 24};
    std::vector<float> q(Prod(dq, 3)), k(Prod(dk, 3)), v(Prod(dv, 3)), s(Prod(ds, 3)), o(Prod(dout, 3));
    oracle_fill_normal(q.data(), q.size(), 1, 0, 1);
    oracle_fill_normal(k.data(), k.size(), 2, 0, 1);
    oracle_fill_normal(v.data(), v.size(), 3, 0, 1);
    oracle_matmul_batched(q.data(), X_NOTRANS, dq, k.data(), X_TRANS, dk, s.data(), ds, 3, 0.125F, 0.0F);
    oracle_matmul_batched(s.data(), X_NOTRANS, ds, v.data(), X_NOTRANS, dv, o.data(), dout, 3, 1.0F, 0.0F);
    XTensor * gq = NewGPU(3, dq, q.data());
    XTensor * gk = NewGPU(3, dk, k.data());
    XTensor * gv = NewGPU(3, dv, v.data());
    XTensor gs = BMMul(*gq, X_NOTRANS, *gk, X_TRANS, 0.125F);
    XTensor go = BMMul(gs, *gv);
    std::vector<float> hs(s.size()), ho(o.size());
    gs.GetData(hs.data());
    go.GetData(ho.data());
    bool ok = MaxRelErr(hs, s) < 8e-5F && MaxRelErr(ho, o) < 8e-5F;
    delete gq; delete gk; delete gv;
    return ok;
}

/* MulAndShift: last-dimension bias (fused column add), an earlier-dimension bias,
   the transposed overload, a scalar bias; and the autograd edge it records */
static bool TestMulAndShift()
{
    bool ok = true;
    int dx[3] = {4, 6, 10}, dw[2] = {10, 8};
    std::vector<float> x(240), w(80), ref(192), got(192);
    oracle_fill_uniform(x.data(), 240, 21, -1, 1);
    oracle_fill_normal(w.data(), 80, 22, 0, 0.02F);
    XTensor * gx = NewGPU(3, dx, x.data());
    XTensor * gw = NewGPU(2, dw, w.data());
    gw->enableGrad = true;

    int biasShapes[4][3] = {{8, 0, 0}, {1, 8, 0}, {6, 0, 0}, {4, 1, 1}};
    int biasOrders[4] = {1, 2, 1, 3};
    int expectN[4] = {2, 2, 1, 0};
    for (int i = 0; i < 4; i++) {
        int nb = Prod(biasShapes[i], biasOrders[i]);
        std::vector<float> bias(nb);
        oracle_fill_normal(bias.data(), nb, 23 + i, 0, 0.02F);
        int cd[8], co = 0;
        int n = oracle_mulandshift(x.data(), X_NOTRANS, dx, 3, w.data(), X_NOTRANS, dw, 2,
                                   bias.data(), biasShapes[i], biasOrders[i], ref.data(), cd, &co, 0.5F);
        XTensor * gb = NewGPU(biasOrders[i], biasShapes[i], bias.data());
        gb->enableGrad = true;
        XTensor c = MulAndShift(*gx, *gw, *gb, 0.5F);
        c.GetData(got.data());
        bool shape = c.order == 3 && c.dimSize[0] == 4 && c.dimSize[1] == 6 && c.dimSize[2] == 8;
        bool edge = c.income.typeID == MATH_MULANDSHIFT && c.income.tailNum == 3 && c.income.paramNum == 4 &&
                    c.income.params[0].i == n && c.income.params[1].i == X_NOTRANS && c.income.params[3].f == 0.5F;
        float e = MaxRelErr(got, ref);
        if (!(shape && edge && n == expectN[i] && e < 4e-5F)) {
            fprintf(stderr, "mulandshift bias %d: n=%d shape=%d edge=%d err=%g\n", i, n, shape, edge, e);
            ok = false;
        }
        delete gb;
    }

    /* the overload with transpose flags: w stored (8, 10) */
    {
        std::vector<float> wt(80), bias(8);
        for (int i = 0; i < 10; i++)
            for (int j = 0; j < 8; j++)
                wt[j * 10 + i] = w[i * 8 + j];
        oracle_fill_normal(bias.data(), 8, 30, 0, 0.02F);
        int dwt[2] = {8, 10}, dbias[1] = {8}, cd[8], co = 0;
        oracle_mulandshift(x.data(), X_NOTRANS, dx, 3, wt.data(), X_TRANS, dwt, 2, bias.data(), dbias, 1, ref.data(), cd, &co, 1.0F);
        XTensor * gwt = NewGPU(2, dwt, wt.data());
        XTensor * gb = NewGPU(1, dbias, bias.data());
        XTensor c = MulAndShift(*gx, X_NOTRANS, *gwt, X_TRANS, *gb);
        c.GetData(got.data());
        if (!(MaxRelErr(got, ref) < 4e-5F && c.income.tailNum == 0))
            ok = false;
        delete gwt; delete gb;
    }

    /* scalar bias (order 0), first overload only */
    {
        float shift = 0.25F;
        int none[1] = {0};
        XTensor * gb = NewGPU(0, none, &shift);
        int cd[8], co = 0;
        oracle_mulandshift(x.data(), X_NOTRANS, dx, 3, w.data(), X_NOTRANS, dw, 2, &shift, none, 0, ref.data(), cd, &co, 1.0F);
        XTensor c = MulAndShift(*gx, *gw, *gb);
        c.GetData(got.data());
        if (!(MaxRelErr(got, ref) < 4e-5F))
            ok = false;
        delete gb;
    }
    delete gx; delete gw;
    return ok;
}

/* fp16 tensors: fp32 accumulation, result within 1e-2 of the fp32 oracle on the rounded inputs */
static bool TestMatrixMulHalf()
{
    bool ok = true;
    int M = 96, N = 80, K = 72;
    for (int ta = 0; ta < 2; ta++) {
        for (int tb = 0; tb < 2; tb++) {
            int da[2] = {ta == X_TRANS ? K : M, ta == X_TRANS ? M : K};
            int db[2] = {tb == X_TRANS ? N : K, tb == X_TRANS ? K : N};
            int dc[2] = {M, N};
            std::vector<float> a(M * K), b(K * N), ref(M * N), got(M * N);
            std::vector<uint16_t> h(M * N);
            oracle_fill_normal(a.data(), M * K, 41, 0, 0.5F);
            oracle_fill_normal(b.data(), K * N, 42, 0, 0.5F);
            /* round the inputs to half first: both sides then multiply the same numbers */
            std::vector<uint16_t> ha(M * K), hb(K * N);
            oracle_f32_to_f16_array(a.data(), ha.data(), M * K);
            oracle_f16_to_f32_array(ha.data(), a.data(), M * K);
            oracle_f32_to_f16_array(b.data(), hb.data(), K * N);
            oracle_f16_to_f32_array(hb.data(), b.data(), K * N);
            oracle_matmul2d(a.data(), ta, b.data(), tb, ref.data(), da[0], da[1], db[0], db[1], M, N, 1.0F, 0.0F);
            XTensor * ga = NewGPU(2, da, a.data(), X_FLOAT16);
            XTensor * gb = NewGPU(2, db, b.data(), X_FLOAT16);
            XTensor * gc = NewGPU(2, dc, NULL, X_FLOAT16);
            _MatrixMul2D(ga, (MATRIX_TRANS_TYPE)ta, gb, (MATRIX_TRANS_TYPE)tb, gc);
            gc->GetData(h.data());
            oracle_f16_to_f32_array(h.data(), got.data(), M * N);
            float e = MaxRelErr(got, ref);
            if (!(e < 1e-2F)) {
                fprintf(stderr, "half ta=%d tb=%d err=%g\n", ta, tb, e);
                ok = false;
            }
            delete ga; delete gb; delete gc;
        }
    }
    return ok;
}

/* the edge a product records for autograd, and the wrapper that reuses a formed c */
static bool TestMatrixMulLinkAndReuse()
{
    int d1[2] = {2, 3}, d2[2] = {3, 2};
    DTYPE sData1[2][3] = {{1.0F, 2.0F, 3.0F}, {-4.0F, 5.0F, 6.0F}};
    DTYPE sData2[3][2] = {{0.0F, -1.0F}, {1.0F, 2.0F}, {2.0F, 1.0F}};
    DTYPE twice[2][2] = {{16.0F, 12.0F}, {34.0F, 40.0F}};
    XTensor * s1 = NewGPU(2, d1, &sData1[0][0]);
    XTensor * s2 = NewGPU(2, d2, &sData2[0][0]);
    s1->enableGrad = true;
    s2->enableGrad = true;
    XTensor c;
    MatrixMul(*s1, X_NOTRANS, *s2, X_NOTRANS, c, 1.0F, 0.0F);     /* forms c */
    MatrixMul(*s1, X_NOTRANS, *s2, X_NOTRANS, c, 1.0F, 1.0F);     /* accumulates into it */
    bool ok = CheckData(&c, twice, 4, 1e-4F);
    ok = ok && c.income.typeID == MATH_MATRIXMUL && c.income.tailNum == 2 && c.income.tails[0] == s1 &&
         c.income.paramNum == 3 && c.income.params[0].i == X_NOTRANS && c.income.params[2].f == 1.0F;
    XTensor d = MatrixMulBatched(*s1, X_NOTRANS, *s2, X_NOTRANS, 2.0F);
    ok = ok && d.income.typeID == MATH_MATRIXMULBATCHED && d.income.params[2].f == 2.0F && CheckData(&d, twice, 4, 1e-4F);
    s1->enableGrad = false;
    XTensor e = MatrixMul(*s1, *s2);
    ok = ok && e.income.tailNum == 0;
    delete s1; delete s2;
    return ok;
}

/* beta == 0 must not let the old contents of c through (the reference zeroes c first) */
static bool TestBetaZeroIgnoresOldContents()
{
    int d1[2] = {64, 32}, d2[2] = {32, 48}, dt[2] = {64, 48};
    std::vector<float> a(64 * 32), b(32 * 48), junk(64 * 48, NAN), ref(64 * 48), got(64 * 48);
    oracle_fill_uniform(a.data(), a.size(), 51, -1, 1);
    oracle_fill_uniform(b.data(), b.size(), 52, -1, 1);
    oracle_matmul2d(a.data(), X_NOTRANS, b.data(), X_NOTRANS, ref.data(), 64, 32, 32, 48, 64, 48, 1.0F, 0.0F);
    XTensor * ga = NewGPU(2, d1, a.data());
    XTensor * gb = NewGPU(2, d2, b.data());
    XTensor * gc = NewGPU(2, dt, junk.data());
    _MatrixMul(ga, X_NOTRANS, gb, X_NOTRANS, gc);
    gc->GetData(got.data());
    bool ok = MaxRelErr(got, ref) < 6e-5F;
    delete ga; delete gb; delete gc;
    return ok;
}

/* ---- backward: XMathGrad on the edges the forward operators record ------------ */

static std::vector<float> Filled(int n, uint64_t seed)
{
    std::vector<float> v(n);
    oracle_fill_uniform(v.data(), n, seed, -1, 1);
    return v;
}

static void SetGrad(XTensor * t, const std::vector<float> & g)
{
    t->grad = NewTensor(t);
    t->grad->SetData(g.data(), t->unitNum);
}

static float GradErr(const XTensor * t, const std::vector<float> & ref)
{
    std::vector<float> got(ref.size());
    t->grad->GetData(got.data());
    return MaxRelErr(got, ref);
}

/* MatrixMul, 2-D, every transpose pair; gradients start non-zero: the step must ADD */
static bool TestGradMatrixMul()
{
    bool ok = true;
    const int M = 70, K = 45, N = 52;
    for (int ta = 0; ta < 2; ta++)
        for (int tb = 0; tb < 2; tb++) {
            int da[2] = {ta == X_TRANS ? K : M, ta == X_TRANS ? M : K};
            int db[2] = {tb == X_TRANS ? N : K, tb == X_TRANS ? K : N};
            std::vector<float> a = Filled(M * K, 1), b = Filled(K * N, 2), dedc = Filled(M * N, 3);
            std::vector<float> deda = Filled(M * K, 4), dedb = Filled(K * N, 5);
            XTensor * ga = NewGPU(2, da, a.data());
            XTensor * gb = NewGPU(2, db, b.data());
            ga->enableGrad = gb->enableGrad = true;
            SetGrad(ga, deda);
            SetGrad(gb, dedb);
            {
                XTensor c = MatrixMul(*ga, (MATRIX_TRANS_TYPE)ta, *gb, (MATRIX_TRANS_TYPE)tb, 0.75F);
                SetGrad(&c, dedc);
                ok = ok && XMathGrad::IsMathOP(&c);
                XMathGrad::MakeGrad(&c, false);
            }
            oracle_grad_matmul(a.data(), deda.data(), ta, da, 2, b.data(), dedb.data(), tb, db, 2, dedc.data(), 0.75F);
            float ea = GradErr(ga, deda), eb = GradErr(gb, dedb);
            if (!(ea < 8e-5F && eb < 8e-5F)) {
                fprintf(stderr, "grad matmul ta=%d tb=%d: %g %g\n", ta, tb, ea, eb);
                ok = false;
            }
            delete ga; delete gb;
        }
    return ok;
}

/* the flatten rule (an untransposed a of order 3 against a matrix), and the "efficient" mode:
   only tensors with isGrad set receive a gradient */
static bool TestGradMatrixMulFlattenAndEfficient()
{
    int da[3] = {5, 9, 20}, db[2] = {20, 16};
    std::vector<float> a = Filled(900, 11), b = Filled(320, 12), dedc = Filled(5 * 9 * 16, 13);
    std::vector<float> deda(900, 0.f), dedb(320, 0.f);
    XTensor * ga = NewGPU(3, da, a.data());
    XTensor * gb = NewGPU(2, db, b.data());
    ga->enableGrad = gb->enableGrad = true;
    gb->isGrad = true;                       /* a does not want a gradient */
    bool ok = true;
    {
        XTensor c = MatrixMul(*ga, X_NOTRANS, *gb, X_NOTRANS);
        SetGrad(&c, dedc);
        XMathGrad::MakeGrad(&c, true);
        ok = ok && c.order == 3 && c.grad->order == 3 && ga->order == 3;     /* shapes restored */
    }
    ok = ok && ga->grad == NULL && gb->grad != NULL;
    oracle_grad_matmul(a.data(), NULL, X_NOTRANS, da, 3, b.data(), dedb.data(), X_NOTRANS, db, 2, dedc.data(), 1.0F);
    ok = ok && GradErr(gb, dedb) < 8e-5F;
    /* the full mode gives a its gradient too */
    {
        XTensor c = MatrixMul(*ga, X_NOTRANS, *gb, X_NOTRANS);
        SetGrad(&c, dedc);
        XMathGrad::MakeGrad(&c, false);
    }
    oracle_grad_matmul(a.data(), deda.data(), X_NOTRANS, da, 3, b.data(), dedb.data(), X_NOTRANS, db, 2, dedc.data(), 1.0F);
    ok = ok && ga->grad != NULL && ga->grad->order == 3 && GradErr(ga, deda) < 8e-5F && GradErr(gb, dedb) < 8e-5F;
    delete ga; delete gb;
    return ok;
}

static bool TestGradMatrixMulBatched()
{
    bool ok = true;
    const int B = 6, M = 40, K = 24, N = 50;
    for (int ta = 0; ta < 2; ta++)
        for (int tb = 0; tb < 2; tb++) {
            int da[3] = {B, ta == X_TRANS ? K : M, ta == X_TRANS ? M : K};
            int db[3] = {B, tb == X_TRANS ? N : K, tb == X_TRANS ? K : N};
            int dc[3] = {B, M, N};
            std::vector<float> a = Filled(B * M * K, 21), b = Filled(B * K * N, 22), dedc = Filled(B * M * N, 23);
            std::vector<float> deda = Filled(B * M * K, 24), dedb = Filled(B * K * N, 25);
            XTensor * ga = NewGPU(3, da, a.data());
            XTensor * gb = NewGPU(3, db, b.data());
            ga->enableGrad = gb->enableGrad = true;
            SetGrad(ga, deda);
            SetGrad(gb, dedb);
            {
                XTensor c = MatrixMulBatched(*ga, (MATRIX_TRANS_TYPE)ta, *gb, (MATRIX_TRANS_TYPE)tb, 0.125F);
                SetGrad(&c, dedc);
                XMathGrad::MakeGrad(&c, false);
            }
            oracle_grad_matmul_batched(a.data(), deda.data(), ta, da, b.data(), dedb.data(), tb, db, dedc.data(), dc, 3, 0.125F);
            float ea = GradErr(ga, deda), eb = GradErr(gb, dedb);
            if (!(ea < 8e-5F && eb < 8e-5F)) {
                fprintf(stderr, "grad batched ta=%d tb=%d: %g %g\n", ta, tb, ea, eb);
                ok = false;
            }
            delete ga; delete gb;
        }
    return ok;
}

/* MulAndShift: bias along the last dimension (its gradient rides on the dE/dw product), along a
   middle one and along the first (a reduction of its own); fp32 and fp16 */
static bool TestGradMulAndShift()
{
    bool ok = true;
    int dx[3] = {4, 6, 40}, dw[2] = {40, 32};
    int biasShapes[3][3] = {{32, 0, 0}, {6, 0, 0}, {4, 1, 1}};
    int biasOrders[3] = {1, 1, 3};
    for (int half = 0; half < 2; half++)
        for (int i = 0; i < 3; i++) {
            const TENSOR_DATA_TYPE type = half ? X_FLOAT16 : X_FLOAT;
            const int nb = Prod(biasShapes[i], biasOrders[i]);
            std::vector<float> x = Filled(960, 31), w = Filled(1280, 32), bias = Filled(nb, 33), dedc = Filled(4 * 6 * 32, 34);
            std::vector<float> dedx = Filled(960, 35), dedw = Filled(1280, 36), dedb = Filled(nb, 37);
            std::vector<float> * all[7] = {&x, &w, &bias, &dedc, &dedx, &dedw, &dedb};
            if (half)
                for (int k = 0; k < 7; k++) {           /* the checker works on the values the GPU holds */
                    std::vector<uint16_t> h(all[k]->size());
                    oracle_f32_to_f16_array(all[k]->data(), h.data(), (long)h.size());
                    oracle_f16_to_f32_array(h.data(), all[k]->data(), (long)h.size());
                }
            XTensor * gx = NewGPU(3, dx, x.data(), type);
            XTensor * gw = NewGPU(2, dw, w.data(), type);
            XTensor * gb = NewGPU(biasOrders[i], biasShapes[i], bias.data(), type);
            gx->enableGrad = gw->enableGrad = gb->enableGrad = true;
            gx->grad = NewGPU(3, dx, dedx.data(), type);
            gw->grad = NewGPU(2, dw, dedw.data(), type);
            gb->grad = NewGPU(biasOrders[i], biasShapes[i], dedb.data(), type);
            int n;
            {
                XTensor c = MulAndShift(*gx, *gw, *gb, 0.5F);
                n = c.income.GetParamInt(0);
                int dc[3] = {4, 6, 32};
                c.grad = NewGPU(3, dc, dedc.data(), type);
                XMathGrad::MakeGrad(&c, false);
                ok = ok && c.grad->order == 3 && gx->grad->order == 3;
            }
            int dc[3] = {4, 6, 32};
            oracle_grad_mulandshift(x.data(), dedx.data(), X_NOTRANS, dx, 3, w.data(), dedw.data(), X_NOTRANS, dw, 2,
                                    dedb.data(), nb, dedc.data(), dc, 3, n, 0.5F);
            std::vector<float> got;
            float errs[3];
            XTensor * grads[3] = {gx->grad, gw->grad, gb->grad};
            std::vector<float> * refs[3] = {&dedx, &dedw, &dedb};
            for (int k = 0; k < 3; k++) {
                got.resize(refs[k]->size());
                if (half) {
                    std::vector<uint16_t> h(got.size());
                    grads[k]->GetData(h.data());
                    oracle_f16_to_f32_array(h.data(), got.data(), (long)h.size());
                }
                else
                    grads[k]->GetData(got.data());
                errs[k] = MaxRelErr(got, *refs[k]);
            }
            const float lim = half ? 1e-2F : 8e-5F;
            if (!(errs[0] < lim && errs[1] < lim && errs[2] < lim)) {
                fprintf(stderr, "grad mulandshift half=%d bias %d (n=%d): %g %g %g\n", half, i, n, errs[0], errs[1], errs[2]);
                ok = false;
            }
            delete gx; delete gw; delete gb;
        }
    return ok;
}

/* ---- data type conversion: the reference's TConvertDataType, GPU halves ------------------ */

/* TConvertDataType.cpp case 1 (:36-90) float -> int and case 2 (:111-165) int -> float */
static bool TestConvertDataType12()
{
    int dims[2] = {3, 2};
    DTYPE aData[3][2] = {{1.0F, 2.0F}, {0.5F, 4.0F}, {5.0F, 6.0F}};
    int answer[3][2] = {{1, 2}, {0, 4}, {5, 6}};
    XTensor * a = NewTensorV2(2, dims, X_FLOAT, 1.0F, DEV);
    XTensor * b = NewTensorV2(2, dims, X_INT, 1.0F, DEV);
    a->SetData(aData, 6);
    b->SetZeroAll();
    _ConvertDataType(a, b);
    int got[6];
    b->GetData(got);
    bool ok = memcmp(got, answer, sizeof(got)) == 0;

    DTYPE answer2[3][2] = {{1.0F, 2.0F}, {0.0F, 4.0F}, {5.0F, 6.0F}};
    XTensor * c = NewTensorV2(2, dims, X_FLOAT, 1.0F, DEV);
    c->SetZeroAll();
    _ConvertDataType(b, c);
    ok = ok && CheckData(c, answer2, 6, 1e-4F);
    delete a; delete b; delete c;
    return ok;
}

/* TConvertDataType.cpp case 3 (:185-268): float -> half for both operands, the half product, half -> float;
   the answer stands in the reference's test (:243-245) with its comparison commented out (:270) */
static bool TestConvertDataType3()
{
    int d1[2] = {3, 2}, d2[2] = {2, 3}, d3[2] = {3, 3};
    DTYPE data1[3][2] = {{1.0F, -2.0F}, {0.5F, -4.0F}, {0.0F, 6.0F}};
    DTYPE data2[2][3] = {{1.0F, 2.0F, 3.0F}, {0.0F, 4.0F, 5.0F}};
    DTYPE answer[3][3] = {{1.0F, -6.0F, -7.0F}, {0.5F, -15.0F, -18.5F}, {0.0F, 24.0F, 30.0F}};
    XTensor * a = NewTensorV2(2, d1, X_FLOAT, 1.0F, DEV);
    XTensor * b = NewTensorV2(2, d2, X_FLOAT, 1.0F, DEV);
    XTensor * c = NewTensorV2(2, d1, X_FLOAT16, 1.0F, DEV);
    XTensor * d = NewTensorV2(2, d2, X_FLOAT16, 1.0F, DEV);
    XTensor * e = NewTensorV2(2, d3, X_FLOAT16, 1.0F, DEV);
    XTensor * f = NewTensorV2(2, d3, X_FLOAT, 1.0F, DEV);
    a->SetData(data1, 6);
    b->SetData(data2, 6);
    _ConvertDataType(a, c);
    _ConvertDataType(b, d);
    _MatrixMul(c, X_NOTRANS, d, X_NOTRANS, e);
    _ConvertDataType(e, f);
    bool ok = CheckData(f, answer, 9, 1e-4F);
    /* the round trip of the test's CPU half (:229-235) */
    XTensor back = ConvertDataType(ConvertDataType(*a, X_FLOAT16), X_FLOAT);
    ok = ok && back.dataType == X_FLOAT && CheckData(&back, data1, 6, 1e-4F);
    /* the allocating form records its edge only for a tensor that takes part in autograd */
    a->enableGrad = true;
    XTensor linked = ConvertDataType(*a, X_FLOAT16);
    ok = ok && linked.income.typeID == GETANDSET_CONVERTDATATYPE && linked.income.tailNum == 1 && linked.income.tails[0] == a;
    ok = ok && back.income.tailNum == 0;
    delete a; delete b; delete c; delete d; delete e; delete f;
    return ok;
}

/* ---- attention in one call against the oracle's restatement of the operator chain ------------- */

static bool TestAttention()
{
    bool ok = true;
    const int cases[3][5] = {{2, 37, 53, 64, 4}, {3, 128, 128, 96, 2}, {1, 70, 200, 128, 1}};   /* batch, lq, lk, hidden, heads */
    for (int ci = 0; ci < 3; ci++)
        for (int masked = 0; masked < 2; masked++) {
            const int B = cases[ci][0], lq = cases[ci][1], lk = cases[ci][2], H = cases[ci][3], nh = cases[ci][4];
            int dq[3] = {B, lq, H}, dk[3] = {B, lk, H}, dm[4] = {nh, B, lq, lk};
            std::vector<float> q(B * lq * H), k(B * lk * H), v(B * lk * H), m(nh * B * lq * lk), ref(B * lq * H), got(B * lq * H);
            oracle_fill_normal(q.data(), (long)q.size(), 71 + ci, 0, 1.0F);
            oracle_fill_normal(k.data(), (long)k.size(), 72 + ci, 0, 1.0F);
            oracle_fill_normal(v.data(), (long)v.size(), 73 + ci, 0, 1.0F);
            oracle_fill_uniform(m.data(), (long)m.size(), 74 + ci, 0.0F, 1.0F);
            for (size_t i = 0; i < m.size(); i++)
                m[i] = (m[i] < 0.3F && i % lk != 0) ? -1e9F : 0.0F;
            const float scale = 1.0F / sqrtf((float)(H / nh));
            oracle_attention(q.data(), k.data(), v.data(), masked ? m.data() : NULL, ref.data(), B, lq, lk, H, nh, scale);
            XTensor * gq = NewGPU(3, dq, q.data());
            XTensor * gk = NewGPU(3, dk, k.data());
            XTensor * gv = NewGPU(3, dk, v.data());
            XTensor * gm = masked ? NewGPU(4, dm, m.data()) : NULL;
            XTensor out = AmdAttention(*gq, *gk, *gv, gm, nh, scale);
            out.GetData(got.data());
            /* the probabilities on their own, as the training path keeps them */
            {
                std::vector<float> pref(nh * B * lq * lk), pgot(nh * B * lq * lk);
                oracle_attention_probs(q.data(), k.data(), masked ? m.data() : NULL, pref.data(), B, lq, lk, H, nh, scale);
                XTensor probs = AmdAttentionProbs(*gq, *gk, gm, nh, scale);
                probs.GetData(pgot.data());
                ok = ok && probs.order == 4 && probs.dimSize[0] == nh && probs.dimSize[1] == B && probs.dimSize[2] == lq && probs.dimSize[3] == lk;
                float pe = 0;
                for (size_t i = 0; i < pgot.size(); i++)
                    pe = fmaxf(pe, fabsf(pgot[i] - pref[i]));
                if (!(pe < 1e-5F * sqrtf((float)(H / nh)))) {
                    fprintf(stderr, "attention probabilities case %d masked %d err=%g\n", ci, masked, pe);
                    ok = false;
                }
                /* ... and the product with the heads of v where they stand, written in merged form: the two
                   calls together are the whole chain */
                std::vector<float> cgot(B * lq * H);
                XTensor ctx = AmdAttentionContext(probs, *gv, nh);
                ctx.GetData(cgot.data());
                ok = ok && ctx.order == 3 && ctx.dimSize[0] == B && ctx.dimSize[1] == lq && ctx.dimSize[2] == H;
                float ce = MaxRelErr(cgot, ref);
                if (!(ce < 1e-5F * sqrtf((float)(H / nh + lk)))) {
                    fprintf(stderr, "attention context case %d masked %d err=%g\n", ci, masked, ce);
                    ok = false;
                }
                /* the half model's form of the same step: the float probabilities straight against half values
                   (no ConvertDataType of the probabilities), a half context */
                XTensor vHalf = ConvertDataType(*gv, X_FLOAT16);
                XTensor ctxHalf = AmdAttentionContext(probs, vHalf, nh);
                ok = ok && ctxHalf.dataType == X_FLOAT16 && ctxHalf.order == 3 && ctxHalf.dimSize[2] == H;
                XTensor ctxBack = ConvertDataType(ctxHalf, X_FLOAT);
                std::vector<float> hgot(B * lq * H);
                ctxBack.GetData(hgot.data());
                float he = MaxRelErr(hgot, ref);
                if (!(he < 1e-2F)) {
                    fprintf(stderr, "attention context with half values case %d masked %d err=%g\n", ci, masked, he);
                    ok = false;
                }
            }
            float e = MaxRelErr(got, ref);
            if (!(e < 1e-5F * sqrtf((float)(H / nh + lk)))) {
                fprintf(stderr, "attention case %d masked %d err=%g\n", ci, masked, e);
                ok = false;
            }
            delete gq; delete gk; delete gv;
            if (gm != NULL)
                delete gm;
        }
    return ok;
}

/* ---- Rectify(MulAndShift(x, w, b)) in one kernel: the reference's TRectify values through a unit product, and a
   seeded feed-forward layer against the oracle ------------------------------------------------------------ */

static bool TestMulAndShiftRectify()
{
    bool ok = true;
    {
        /* TRectify.cpp:43-46: x times the identity plus a zero bias, rectified */
        int dx[2] = {2, 3}, dw[2] = {3, 3}, db[1] = {3};
        DTYPE xData[2][3] = {{0.0F, -1.0F, 2.0F}, {3.0F, -4.0F, -5.0F}};
        DTYPE eye[3][3] = {{1, 0, 0}, {0, 1, 0}, {0, 0, 1}};
        DTYPE zero[3] = {0, 0, 0};
        DTYPE answer[2][3] = {{0.0F, 0.0F, 2.0F}, {3.0F, 0.0F, 0.0F}};
        XTensor * x = NewGPU(2, dx, &xData[0][0]);
        XTensor * w = NewGPU(2, dw, &eye[0][0]);
        XTensor * b = NewGPU(1, db, zero);
        XTensor y = MulAndShiftRectify(*x, *w, *b);
        ok = ok && CheckData(&y, answer, 6, 1e-4F);
        delete x; delete w; delete b;
    }
    int dx[3] = {4, 33, 96}, dw[2] = {96, 200}, db[1] = {200};
    std::vector<float> x(4 * 33 * 96), w(96 * 200), b(200), pre(4 * 33 * 200), ref(4 * 33 * 200), got(4 * 33 * 200);
    oracle_fill_uniform(x.data(), (long)x.size(), 501, -1.0F, 1.0F);
    oracle_fill_normal(w.data(), (long)w.size(), 502, 0, 0.1F);
    oracle_fill_normal(b.data(), (long)b.size(), 503, 0, 0.1F);
    int dc[8], cOrder = 0;
    oracle_mulandshift(x.data(), X_NOTRANS, dx, 3, w.data(), X_NOTRANS, dw, 2, b.data(), db, 1, pre.data(), dc, &cOrder, 1.0F);
    oracle_rectify(pre.data(), (long)pre.size(), ref.data());
    XTensor * gx = NewGPU(3, dx, x.data());
    XTensor * gw = NewGPU(2, dw, w.data());
    XTensor * gb = NewGPU(1, db, b.data());
    XTensor y = MulAndShiftRectify(*gx, *gw, *gb);
    y.GetData(got.data());
    ok = ok && y.order == 3 && y.dimSize[0] == 4 && y.dimSize[1] == 33 && y.dimSize[2] == 200 && y.income.tailNum == 0;
    float e = MaxRelErr(got, ref);
    if (!(e < 1e-5F * sqrtf(96.0F))) {
        fprintf(stderr, "mulandshift+rectify err=%g\n", e);
        ok = false;
    }
    delete gx; delete gw; delete gb;
    return ok;
}

/* ---- the C ABI from several host threads at once, each on a stream of its own (the reference runs one worker
   thread per device and more than one model replica per process): same bits as a single-threaded run --------- */

static void ThreadBody(int id, const float * a, const float * b, const float * bias, float * out, int * status)
{
    const int M = 200, N = 136, K = 96;
    hipStream_t stream;
    *status = 1;
    if (hipSetDevice(DEV) != hipSuccess || hipStreamCreate(&stream) != hipSuccess)
        return;
    float *da, *db, *dbias, *dc;
    if (hipMalloc((void **)&da, M * K * 4) != hipSuccess || hipMalloc((void **)&db, K * N * 4) != hipSuccess ||
        hipMalloc((void **)&dbias, N * 4) != hipSuccess || hipMalloc((void **)&dc, M * N * 4) != hipSuccess)
        return;
    hipMemcpy(da, a, M * K * 4, hipMemcpyHostToDevice);
    hipMemcpy(db, b, K * N * 4, hipMemcpyHostToDevice);
    hipMemcpy(dbias, bias, N * 4, hipMemcpyHostToDevice);
    int rc = 0;
    for (int it = 0; it < 40 && rc == 0; it++) {
        /* every thread asks for something else in between, so that the calls really interleave */
        if ((it + id) % 3 == 0)
            rc = ntsamd_matrix_mul(DEV, stream, da, X_NOTRANS, X_FLOAT, db, X_NOTRANS, X_FLOAT, dc, X_FLOAT, M, K, K, N, M, N, 0.5F, 0.0F);
        rc = rc != 0 ? rc : ntsamd_matrix_mul_bias_act(DEV, stream, da, X_NOTRANS, X_FLOAT, db, X_NOTRANS, X_FLOAT, dc, X_FLOAT,
                                                       M, K, K, N, M, N, 1.0F + id, 0.0F, dbias, NTSAMD_BIAS_COL, N, 1, NTSAMD_ACT_RECTIFY);
        /* a call that must fail leaves its message with THIS thread only */
        int bad = ntsamd_matrix_mul(DEV, stream, da, X_NOTRANS, 4, db, X_NOTRANS, 4, dc, 4, M, K, K, N, M, N, 1.0F, 0.0F);
        if (bad != NTSAMD_ERR_DATATYPE || strcmp(ntsamd_last_error(), "Unsupported data type!") != 0)
            rc = -1;
    }
    hipStreamSynchronize(stream);
    hipMemcpy(out, dc, M * N * 4, hipMemcpyDeviceToHost);
    hipFree(da); hipFree(db); hipFree(dbias); hipFree(dc);
    hipStreamDestroy(stream);
    *status = rc;
}

static bool TestThreads()
{
    const int M = 200, N = 136, K = 96, T = 4;
    std::vector<float> a(M * K), b(K * N), bias(N), pre(M * N), ref(M * N);
    oracle_fill_uniform(a.data(), M * K, 601, -1.0F, 1.0F);
    oracle_fill_uniform(b.data(), K * N, 602, -1.0F, 1.0F);
    oracle_fill_normal(bias.data(), N, 603, 0, 1.0F);
    std::vector<std::vector<float> > out(T, std::vector<float>(M * N));
    int status[T];
    std::vector<std::thread> threads;
    for (int t = 0; t < T; t++)
        threads.push_back(std::thread(ThreadBody, t, a.data(), b.data(), bias.data(), out[t].data(), &status[t]));
    for (int t = 0; t < T; t++)
        threads[t].join();
    bool ok = true;
    for (int t = 0; t < T; t++) {
        ok = ok && status[t] == 0;
        oracle_matmul2d(a.data(), X_NOTRANS, b.data(), X_NOTRANS, pre.data(), M, K, K, N, M, N, 1.0F + t, 0.0F);
        for (int i = 0; i < M * N; i++)
            pre[i] += bias[i % N];
        oracle_rectify(pre.data(), M * N, ref.data());
        float e = MaxRelErr(out[t], ref);
        if (!(e < 1e-5F * sqrtf((float)K))) {
            fprintf(stderr, "thread %d err=%g\n", t, e);
            ok = false;
        }
    }
    return ok;
}

/* ---- device blocks are handed out again: same results, no growth --------------------------------- */

static bool TestMemoryReuse()
{
    bool ok = true;
    int dq[3] = {16, 64, 32};
    std::vector<float> q(16 * 64 * 32), k(16 * 64 * 32), first(16 * 64 * 64), again(16 * 64 * 64);
    oracle_fill_normal(q.data(), (long)q.size(), 91, 0, 1.0F);
    oracle_fill_normal(k.data(), (long)k.size(), 92, 0, 1.0F);
    XTensor * gq = NewGPU(3, dq, q.data());
    XTensor * gk = NewGPU(3, dq, k.data());
    {
        XTensor s = MatrixMulBatched(*gq, X_NOTRANS, *gk, X_TRANS, 0.125F);
        s.GetData(first.data());
    }
    long long h0, m0, h1, m1;
    size_t spare0, spare1;
    XMemCacheStats(DEV, &spare0, &h0, &m0);
    void * seen = NULL;
    for (int i = 0; i < 50; i++) {
        XTensor s = MatrixMulBatched(*gq, X_NOTRANS, *gk, X_TRANS, 0.125F);
        if (i == 0)
            seen = s.data;
        ok = ok && s.data == seen;                     /* the block the previous result gave up */
        if (i == 49)
            s.GetData(again.data());
    }
    XMemCacheStats(DEV, &spare1, &h1, &m1);
    ok = ok && h1 - h0 == 50 && m1 == m0 && spare1 == spare0;
    ok = ok && memcmp(first.data(), again.data(), first.size() * sizeof(float)) == 0;
    /* requests of another size class do not take that block; releasing empties the lists */
    int dsmall[2] = {5, 7};
    XTensor * t = NewTensorV2(2, dsmall, X_FLOAT, 1.0F, DEV);
    ok = ok && t->data != seen;
    delete t;
    XMemCacheRelease(DEV);
    XMemCacheStats(DEV, &spare1, NULL, NULL);
    ok = ok && spare1 == 0;
    /* switched off, a request goes to the runtime and a release goes back to it */
    XMemCacheEnable(false);
    {
        XTensor s = MatrixMulBatched(*gq, X_NOTRANS, *gk, X_TRANS, 0.125F);
        s.GetData(again.data());
        ok = ok && memcmp(first.data(), again.data(), first.size() * sizeof(float)) == 0;
    }
    XMemCacheStats(DEV, &spare1, NULL, NULL);
    ok = ok && spare1 == 0;
    XMemCacheEnable(true);
    delete gq; delete gk;
    return ok;
}

/* time per allocating call at the attention shape of the benchmark, with and without block reuse */
static int AllocBench()
{
    int dq[3] = {256, 128, 64};
    std::vector<float> q(256 * 128 * 64);
    oracle_fill_normal(q.data(), (long)q.size(), 5, 0, 1.0F);
    XTensor * gq = NewGPU(3, dq, q.data());
    XTensor * gk = NewGPU(3, dq, q.data());
    float sink;
    for (int mode = 0; mode < 2; mode++) {
        XMemCacheEnable(mode == 0);
        for (int i = 0; i < 20; i++)
            XTensor s = MatrixMulBatched(*gq, X_NOTRANS, *gk, X_TRANS, 0.125F);
        gq->GetData(q.data());                          /* a blocking copy: the queue is empty */
        const int n = 500;
        auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < n; i++)
            XTensor s = MatrixMulBatched(*gq, X_NOTRANS, *gk, X_TRANS, 0.125F);
        XTensor last = MatrixMulBatched(*gq, X_NOTRANS, *gk, X_TRANS, 0.125F);
        XMemCopy(&sink, -1, last.data, DEV, sizeof(float));
        auto t1 = std::chrono::steady_clock::now();
        printf("MatrixMulBatched [256x128x64] x [256x128x64]^T, new result tensor per call, blocks %s: %.1f us per call\n",
               mode == 0 ? "handed out again" : "from hipMalloc / hipFree",
               std::chrono::duration<double, std::micro>(t1 - t0).count() / (n + 1));
    }
    XMemCacheEnable(true);
    delete gq; delete gk;
    return 0;
}


/* ---- host tensors: the layer hands them to the host tree's functions --------------- */

/* stand-ins for the host tree's _MatrixMul2DParallel and _SumDim: plain loops of this file (never the oracle
   library, which the layer must not depend on), enough to show that the right blocks arrive in the right order */
static int hostProducts = 0, hostSums = 0;
static void HostProduct(const XTensor * a, MATRIX_TRANS_TYPE ta, const XTensor * b, MATRIX_TRANS_TYPE tb,
                        XTensor * c, DTYPE alpha, DTYPE beta, XPRunner *)
{
    hostProducts++;
    const int M = c->dimSize[0], N = c->dimSize[1], K = ta == X_TRANS ? a->dimSize[0] : a->dimSize[1];
    const float * A = (const float *)a->data, * B = (const float *)b->data;
    float * C = (float *)c->data;
    for (int i = 0; i < M; i++)
        for (int j = 0; j < N; j++) {
            double sum = 0;
            for (int k = 0; k < K; k++)
                sum += (double)(ta == X_TRANS ? A[k * M + i] : A[i * K + k]) * (tb == X_TRANS ? B[j * K + k] : B[k * N + j]);
            C[i * N + j] = (float)(alpha * sum + (beta != 0 ? beta * C[i * N + j] : 0.0));
        }
}
static void HostSumLastDim(const XTensor * a, const XTensor * b, XTensor * c, int n, DTYPE beta)
{
    hostSums++;
    if (n != a->order - 1)
        return;
    const int cols = a->dimSize[n];
    for (int i = 0; i < a->unitNum; i++)
        ((float *)c->data)[i] = ((const float *)a->data)[i] + ((const float *)b->data)[i % cols] * beta;
}

static XTensor * NewHost(int order, const int * dims, const float * data)
{
    XTensor * t = NewTensorV2(order, dims, X_FLOAT, 1.0F, -1);
    if (data != NULL)
        memcpy(t->data, data, sizeof(float) * t->unitNum);
    return t;
}
static bool SameAs(const XTensor * t, const void * answer, int num)
{
    return t->devID < 0 && t->unitNum == num && oracle_check_data((const float *)t->data, (const float *)answer, num, 1e-4F) != 0;
}

/* The reference's known answers again, on host tensors: _MatrixMul2D, the flattened product and the (p, q) list of
   _MatrixMul, the blocks of _MatrixMulBatched, the allocating wrappers and MulAndShift all reach the two functions
   the host tree handed in (source/tensor/core/arithmetic/MatrixMul2D.cpp:77-94, MatrixMul.cpp:180-185,
   MatrixMulBatched.cpp:157-271, MulAndShift.cpp:69-88). */
static bool TestHostDispatch()
{
    SetHostMatrixMul2D(HostProduct);
    SetHostSumDim(HostSumLastDim);
    hostProducts = hostSums = 0;
    bool ok = GetHostMatrixMul2D() == HostProduct && GetHostSumDim() == HostSumLastDim;

    int d23[2] = {2, 3}, d32[2] = {3, 2}, d22[2] = {2, 2};
    DTYPE a23[2][3] = {{1.0F, 2.0F, 3.0F}, {-4.0F, 5.0F, 6.0F}};
    DTYPE a32t[3][2] = {{1.0F, -4.0F}, {2.0F, 5.0F}, {3.0F, 6.0F}};
    DTYPE b32[3][2] = {{0.0F, -1.0F}, {1.0F, 2.0F}, {2.0F, 1.0F}};
    DTYPE want22[2][2] = {{8.0F, 6.0F}, {17.0F, 20.0F}};
    XTensor * s1 = NewHost(2, d23, &a23[0][0]), * s1t = NewHost(2, d32, &a32t[0][0]), * s2 = NewHost(2, d32, &b32[0][0]);
    XTensor * t = NewHost(2, d22, NULL), * t2 = NewHost(2, d22, NULL);
    _MatrixMul2D(s1, X_NOTRANS, s2, X_NOTRANS, t);
    _MatrixMul(s1t, X_TRANS, s2, X_NOTRANS, t2);
    XTensor user = MatrixMul(*s1, X_NOTRANS, *s2, X_NOTRANS);
    ok = ok && SameAs(t, want22, 4) && SameAs(t2, want22, 4) && SameAs(&user, want22, 4) && hostProducts == 3;

    /* (3,2,3) x (2,3,2): six pairs of blocks, result block (p, q) at p * 2 + q */
    int d323[3] = {3, 2, 3}, d232[3] = {2, 3, 2}, d3222[4] = {3, 2, 2, 2}, d322[3] = {3, 2, 2}, d222[3] = {2, 2, 2}, d223[3] = {2, 2, 3};
    DTYPE want3222[3][2][2][2] = {{{{8.0F, 9.0F}, {4.0F, 25.0F}}, {{7.0F, 8.0F}, {20.0F, 26.0F}}},
                                  {{{1.0F, 32.0F}, {3.0F, 21.0F}}, {{27.0F, 34.0F}, {16.0F, 22.0F}}},
                                  {{{-9.0F, 19.0F}, {5.0F, -1.0F}}, {{18.0F, 22.0F}, {-2.0F, -2.0F}}}};
    XTensor * n1 = NewHost(3, d323, &sData323[0][0][0]), * n2 = NewHost(3, d232, &sData232[0][0][0]);
    XTensor * t4 = NewHost(4, d3222, NULL);
    hostProducts = 0;
    _MatrixMul(n1, X_NOTRANS, n2, X_NOTRANS, t4);
    ok = ok && SameAs(t4, want3222, 24) && hostProducts == 6;

    /* (3,2,3) x (3,2): one product over the flattened rows */
    DTYPE b32b[3][2] = {{1.0F, 2.0F}, {3.0F, 4.0F}, {5.0F, 6.0F}};
    DTYPE want322[3][2][2] = {{{7.0F, 8.0F}, {20.0F, 26.0F}}, {{27.0F, 34.0F}, {16.0F, 22.0F}}, {{18.0F, 22.0F}, {-2.0F, -2.0F}}};
    XTensor * w = NewHost(2, d32, &b32b[0][0]), * t3 = NewHost(3, d322, NULL);
    hostProducts = 0;
    _MatrixMul(n1, X_NOTRANS, w, X_NOTRANS, t3);
    ok = ok && SameAs(t3, want322, 12) && hostProducts == 1;

    /* (2,2,3) x (2,3,2), block i with block i */
    DTYPE want222[2][2][2] = {{{8.0F, 9.0F}, {4.0F, 25.0F}}, {{27.0F, 34.0F}, {16.0F, 22.0F}}};
    XTensor * m1 = NewHost(3, d223, &sData323[0][0][0]), * tb = NewHost(3, d222, NULL);
    hostProducts = 0;
    _MatrixMulBatched(m1, X_NOTRANS, n2, X_NOTRANS, tb);
    XTensor userB = MatrixMulBatched(*m1, X_NOTRANS, *n2, X_NOTRANS);
    ok = ok && SameAs(tb, want222, 8) && SameAs(&userB, want222, 8) && hostProducts == 4;

    /* MulAndShift: the product, then the host tree's broadcast add along the last dimension, in place */
    int d2[1] = {2};
    DTYPE bias2[2] = {0.5F, -1.0F};
    DTYPE wantShift[3][2][2] = {{{7.5F, 7.0F}, {20.5F, 25.0F}}, {{27.5F, 33.0F}, {16.5F, 21.0F}}, {{18.5F, 21.0F}, {-1.5F, -3.0F}}};
    XTensor * bs = NewHost(1, d2, bias2);
    hostProducts = 0;
    XTensor shifted = MulAndShift(*n1, *w, *bs);
    ok = ok && SameAs(&shifted, wantShift, 12) && hostProducts == 1 && hostSums == 1 && shifted.order == 3;

    SetHostMatrixMul2D(NULL);
    SetHostSumDim(NULL);
    ok = ok && GetHostMatrixMul2D() == NULL;
    delete s1; delete s1t; delete s2; delete t; delete t2; delete n1; delete n2; delete t4; delete w; delete t3;
    delete m1; delete tb; delete bs;
    return ok;
}

/* ---- the operators of the baseline's configurations, timed through this layer ---------------- */

struct Timer {
    hipEvent_t e0, e1;
    Timer() { hipEventCreate(&e0); hipEventCreate(&e1); }
    ~Timer() { hipEventDestroy(e0); hipEventDestroy(e1); }
    template <class F> double Us(F f, int calls)
    {
        hipEventRecord(e0, NULL);
        for (int i = 0; i < calls; i++)
            f();
        hipEventRecord(e1, NULL);
        hipEventSynchronize(e1);
        float ms = 0;
        hipEventElapsedTime(&ms, e0, e1);
        return (double)ms * 1e3 / calls;
    }
    /* runs f until 0.15 s of GPU time have passed (the clocks of the part settle under load), then times `calls`
       calls five times over and returns the shortest average */
    template <class F> double Settled(F f, int calls)
    {
        double spent = 0;
        for (int n = 8; spent < 0.15e6; n = n < 256 ? n * 2 : n)
            spent += Us(f, n) * n;
        double best = 1e30;
        for (int r = 0; r < 5; r++)
            best = fmin(best, Us(f, calls));
        return best;
    }
};

static XTensor * Filled(int order, const int * dims, int seed, float sd, TENSOR_DATA_TYPE type = X_FLOAT, bool uniform = false)
{
    std::vector<float> h(Prod(dims, order));
    if (uniform)
        oracle_fill_uniform(h.data(), (long)h.size(), seed, -1.0F, 1.0F);
    else
        oracle_fill_normal(h.data(), (long)h.size(), seed, 0, sd);
    return NewGPU(order, dims, h.data(), type);
}

/* One JSON line per configuration: microseconds per operator call (HIP events on the NULL stream, which is where
   this layer issues its work, 200 calls after settling), the allocating form (a new result tensor per call, as
   the reference's callers use it) and the in-place form beside it. */
static int Bench()
{
    Timer tm;
    {
        /* configuration 2: MulAndShift(x[32x128x512], w[512x2048], b[2048]) */
        int dx[3] = {32, 128, 512}, dw[2] = {512, 2048}, db[1] = {2048}, dc[3] = {32, 128, 2048};
        XTensor * x = Filled(3, dx, 1, 0, X_FLOAT, true), * w = Filled(2, dw, 2, 0.02F), * b = Filled(1, db, 3, 0.02F);
        XTensor * c = NewGPU(3, dc, NULL);
        const double alloc = tm.Settled([&] { XTensor r = MulAndShift(*x, *w, *b); }, 200);
        const double inplace = tm.Settled([&] { _MatrixMulBias(x, X_NOTRANS, w, X_NOTRANS, c, 1.0F, 0, b, 2); }, 200);
        printf("{\"config\": 2, \"operator\": \"nts::MulAndShift(x, w, b)\", \"launches\": 1, \"us_per_call\": %.2f, \"us_per_call_into_existing_tensor\": %.2f}\n", alloc, inplace);
        delete x; delete w; delete b; delete c;
    }
    {
        /* configuration 3: BMMul(q, X_NOTRANS, k, X_TRANS, 1/8), then BMMul(s, v) */
        int dq[3] = {256, 128, 64}, ds[3] = {256, 128, 128};
        XTensor * q = Filled(3, dq, 1, 1.0F), * k = Filled(3, dq, 2, 1.0F), * v = Filled(3, dq, 3, 1.0F);
        XTensor * s = NewGPU(3, ds, NULL), * o = NewGPU(3, dq, NULL);
        const double alloc = tm.Settled([&] {
            XTensor sc = MatrixMulBatched(*q, X_NOTRANS, *k, X_TRANS, 0.125F);
            XTensor out = MatrixMulBatched(sc, X_NOTRANS, *v, X_NOTRANS);
        }, 200);
        const double inplace = tm.Settled([&] {
            _MatrixMulBatched(q, X_NOTRANS, k, X_TRANS, s, 0.125F, 0);
            _MatrixMulBatched(s, X_NOTRANS, v, X_NOTRANS, o, 1.0F, 0);
        }, 200);
        printf("{\"config\": 3, \"operator\": \"nts::MatrixMulBatched(q, k^T, 1/8) then nts::MatrixMulBatched(s, v)\", \"launches\": 2, \"us_per_call\": %.2f, \"us_per_call_into_existing_tensor\": %.2f}\n", alloc / 2, inplace / 2);
        delete q; delete k; delete v; delete s; delete o;
    }
    {
        /* configuration 4: MatrixMul(a[1024x8192], X_TRANS, b[1024x4096], X_NOTRANS), half */
        int da[2] = {1024, 8192}, db[2] = {1024, 4096}, dc[2] = {8192, 4096};
        XTensor * a = Filled(2, da, 1, 0.02F, X_FLOAT16), * b = Filled(2, db, 2, 0.02F, X_FLOAT16);
        XTensor * c = NewGPU(2, dc, NULL, X_FLOAT16);
        const double alloc = tm.Settled([&] { XTensor r = MatrixMul(*a, X_TRANS, *b, X_NOTRANS); }, 200);
        const double inplace = tm.Settled([&] { _MatrixMul(a, X_TRANS, b, X_NOTRANS, c, 1.0F, 0); }, 200);
        printf("{\"config\": 4, \"operator\": \"nts::MatrixMul(a, X_TRANS, b, X_NOTRANS), half\", \"launches\": 1, \"us_per_call\": %.2f, \"us_per_call_into_existing_tensor\": %.2f}\n", alloc, inplace);
        delete a; delete b; delete c;
    }
    {
        /* configuration 5: MatrixMul(h[4096x512], X_NOTRANS, w[30011x512], X_TRANS, c, 1, beta = 1) */
        int dh[2] = {4096, 512}, dw[2] = {30011, 512}, dc[2] = {4096, 30011};
        XTensor * h = Filled(2, dh, 1, 0, X_FLOAT, true), * w = Filled(2, dw, 2, 0.02F);
        XTensor * c = Filled(2, dc, 3, 0, X_FLOAT, true);
        const double inplace = tm.Settled([&] { MatrixMul(*h, X_NOTRANS, *w, X_TRANS, *c, 1.0F, 1.0F); }, 50);
        printf("{\"config\": 5, \"operator\": \"nts::MatrixMul(h, X_NOTRANS, w, X_TRANS, c, 1, 1)\", \"launches\": 1, \"us_per_call\": %.2f, \"us_per_call_into_existing_tensor\": %.2f}\n", inplace, inplace);
        delete h; delete w; delete c;
    }
    fflush(stdout);
    return 0;
}

/* ---- fatal errors: same message, same ending as the reference ---------------- */

static int Provoke(const char * name)
{
    /* view tensors (a negative size: shape only, no allocation) on device 0:
       every check below fires before the GPU is touched */
    int d23[2] = {-2, 3}, d32[2] = {-3, 2}, d22[2] = {-2, 2}, d223[3] = {-2, 2, 3};
    XTensor a(2, d23, X_FLOAT, 1.0F, 0, NULL), b(2, d32, X_FLOAT, 1.0F, 0, NULL), c(2, d22, X_FLOAT, 1.0F, 0, NULL);
    XTensor h(2, d32, X_FLOAT16, 1.0F, 0, NULL), t3(3, d223, X_FLOAT, 1.0F, 0, NULL);
    XTensor host(2, d22, X_FLOAT, 1.0F, -1, NULL);
    if (!strcmp(name, "unmatched"))
        _MatrixMul2D(&a, X_NOTRANS, &a, X_NOTRANS, &c);
    else if (!strcmp(name, "datatype"))
        _MatrixMul(&a, X_NOTRANS, &h, X_NOTRANS, &c);
    else if (!strcmp(name, "order"))
        _MatrixMulBatched(&t3, X_NOTRANS, &b, X_NOTRANS, &c);
    else if (!strcmp(name, "wrongorder"))
        _MatrixMul(&t3, X_NOTRANS, &b, X_NOTRANS, &c);
    else if (!strcmp(name, "empty"))
        _MatrixMul(NULL, X_NOTRANS, &b, X_NOTRANS, &c);
    else if (!strcmp(name, "host"))
        _MatrixMul2D(&host, X_NOTRANS, &host, X_NOTRANS, &host);
    else if (!strcmp(name, "nograd")) {
        /* a node without dE/dc cannot be differentiated (XBackwardMath.cpp:34-36) */
        XLink::MakeLink(&a, &b, &c, MATH_MATRIXMUL);
        XMathGrad::MakeGrad(&c, false);
    }
    else if (!strcmp(name, "gradtodo")) {
        /* a transposed a of order 3 has no backward in the reference either (:631-633) */
        XTensor cc(3, d223, X_FLOAT, 1.0F, 0, NULL);
        XLink::MakeLink(&t3, &b, &cc, MATH_MATRIXMUL);
        XLink::AddParamToHeadTrans(&cc, X_TRANS);
        XLink::AddParamToHeadTrans(&cc, X_NOTRANS);
        XLink::AddParamToHead(&cc, 1.0F);
        t3.isGrad = false;
        cc.grad = new XTensor(3, d223, X_FLOAT, 1.0F, 0, NULL);
        XMathGrad::MakeGrad(&cc, true);
    }
    else if (!strcmp(name, "converthost")) {
        XTensor hostHalf(2, d22, X_FLOAT16, 1.0F, -1, NULL);
        _ConvertDataType(&host, &hostHalf);              /* host tensors: the reference's CPU path, not this library */
    }
    else if (!strcmp(name, "convertsize")) {
        XTensor big(3, d223, X_FLOAT16, 1.0F, 0, NULL);
        _ConvertDataType(&a, &big);                      /* 6 elements into 12 */
    }
    else if (!strcmp(name, "attentionheads")) {
        /* a hidden size of 3 does not split into 2 heads */
        XTensor o3(3, d223, X_FLOAT, 1.0F, 0, NULL);
        _AmdAttention(&t3, &t3, &t3, NULL, &o3, 2, 1.0F);
    }
    else if (!strcmp(name, "attentiontype")) {
        XTensor o3(3, d223, X_FLOAT16, 1.0F, 0, NULL);
        _AmdAttention(&t3, &t3, &t3, NULL, &o3, 1, 1.0F);
    }
    else if (!strcmp(name, "biasshape")) {
        XTensor bias(2, d22, X_FLOAT, 1.0F, 0, NULL);
        MulAndShift(a, b, bias);
    }
    else
        return 2;
    return 0;   /* not reached when the error fires */
}

#define RUN(t) { bool r_ = t(); printf(">> %-36s %s\n", #t, r_ ? "passed" : "FAILED"); fflush(stdout); all = all && r_; }

int main(int argc, char ** argv)
{
    if (argc == 3 && !strcmp(argv[1], "--abort"))
        return Provoke(argv[2]);
    if (argc == 2 && !strcmp(argv[1], "--alloc-bench"))
        return AllocBench();
    if (argc == 2 && !strcmp(argv[1], "--bench"))
        return Bench();
    if (argc == 2 && !strcmp(argv[1], "--host")) {
        const bool ok = TestHostDispatch();
        printf(">> %-36s %s\n", "TestHostDispatch", ok ? "passed" : "FAILED");
        return ok ? 0 : 1;
    }

    bool all = true;
    RUN(TestMatrixMul1);
    RUN(TestMatrixMul2);
    RUN(TestMatrixMul3);
    RUN(TestMatrixMul4);
    RUN(TestMatrixMulBatched2);
    RUN(TestMatrixMulSeeded);
    RUN(TestMatrixMulTransposedND);
    RUN(TestMatrixMulBatchedAttention);
    RUN(TestMulAndShift);
    RUN(TestMatrixMulHalf);
    RUN(TestMatrixMulLinkAndReuse);
    RUN(TestBetaZeroIgnoresOldContents);
    RUN(TestGradMatrixMul);
    RUN(TestGradMatrixMulFlattenAndEfficient);
    RUN(TestGradMatrixMulBatched);
    RUN(TestGradMulAndShift);
    RUN(TestConvertDataType12);
    RUN(TestConvertDataType3);
    RUN(TestAttention);
    RUN(TestMulAndShiftRectify);
    RUN(TestThreads);
    RUN(TestMemoryReuse);
    RUN(TestHostDispatch);
    printf(all ? "OK! Everything is good!\n" : "Sorry, some problems happened!\n");
    return all ? 0 : 1;
}
