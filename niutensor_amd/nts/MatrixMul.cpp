/*
 * N-D matrix product on a gfx950 GPU: dispatch of
 * source/tensor/core/arithmetic/MatrixMul.cpp:52-208 and its allocating
 * wrappers (:272-459), over the kernels of libntsamd.
 *
 * Kept from the reference: the checks and their messages; the flatten rule (an
 * untransposed a of order > 2 against a matrix b is one 2-D product, :65-78);
 * the (p, q) pairing of blocks otherwise, result block at p * bBlockNum + q
 * (:121-146); the rule that the block list runs on the GPU only if a, b and c
 * are all on one (:156-159); result shape, temporary flag and autograd edge of
 * the wrappers. Dropped: SetZeroAll before a beta == 0 product (:163-164), which
 * the kernels make unnecessary, and the CPU and sparse branches.
 */
#include "MatrixMul.h"
#include "MatrixMul2D.h"
#include "MatrixMulBatched.h"
#include "XTensorBLAS.h"

namespace nts {

/* stored and logical sizes of the matrix dimensions of t */
struct MatDims {
    int rows, cols;   /* as stored: dimSize[order-2], dimSize[order-1] */
    int n, m;         /* after trans(): n rows, m columns */
};

static MatDims MatrixDims(const XTensor * t, MATRIX_TRANS_TYPE trans)
{
    MatDims d;
    d.rows = t->dimSize[t->order - 2];
    d.cols = t->dimSize[t->order - 1];
    d.n = trans == X_TRANS ? d.cols : d.rows;
    d.m = trans == X_TRANS ? d.rows : d.cols;
    return d;
}

/* shape of a (x) b: a's leading dimensions, b's leading dimensions, then n of a and m of b */
static int ResultShape(const XTensor * a, MATRIX_TRANS_TYPE transposedA,
                       const XTensor * b, MATRIX_TRANS_TYPE transposedB, int * dimSize)
{
    int sub = 0;
    for (int i = 0; i < a->order - 2; i++)
        dimSize[sub++] = a->dimSize[i];
    for (int i = 0; i < b->order - 2; i++)
        dimSize[sub++] = b->dimSize[i];
    dimSize[sub++] = MatrixDims(a, transposedA).n;
    dimSize[sub++] = MatrixDims(b, transposedB).m;
    return sub;
}

static BiasSpec RowOrColumnBias(const XTensor * c, const XTensor * bias, int n, int lastLeading)
{
    /* c is seen as a matrix whose rows run over dimensions 0..order-2. A bias on the
       last dimension is indexed by the column; a bias on dimension n < order-1 by
       (row / product of the dimensions between n and the last) mod dimSize[n] */
    BiasSpec s;
    s.data = bias->data;
    s.act = 0;
    if (n == SCALAR_BIAS) {
        s.mode = 2;
        s.len = 1;
        s.rowDiv = 1;
    }
    else if (n == c->order - 1) {
        s.mode = 1;
        s.len = c->dimSize[n];
        s.rowDiv = 1;
    }
    else {
        s.mode = 2;
        s.len = c->dimSize[n];
        s.rowDiv = 1;
        for (int i = n + 1; i <= lastLeading; i++)
            s.rowDiv *= c->dimSize[i];
    }
    return s;
}

void _MatrixMulBias(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                    XTensor * c, DTYPE alpha, DTYPE beta, const XTensor * bias, int n, int act)
{
    CheckNTErrors(a && b && c, "Empty input tensors!");
    CheckNTErrors(a->dataType == b->dataType && a->dataType == c->dataType,
                  "Input tensors should have the same data type!");
    CheckNTErrors(a->order >= 2 && b->order >= 2 && c->order >= 2, "Input tensors must have a order >= 2!");
    CheckNTErrors(c->order == a->order + b->order - 2, "wrong tensor order");
    if (bias != NULL) {
        CheckNTErrors((n >= 0 && n < c->order) || n == SCALAR_BIAS, "Something is wrong!");
        CheckNTErrors(bias->dataType == c->dataType, "Unmatched data types in addition!");
        CheckNTErrors((n == SCALAR_BIAS ? 1 : c->dimSize[n]) == bias->unitNum, "Wrong tensor size!");
        CheckNTErrors(bias->devID == c->devID, "The code must be run on the same GPU!");
    }

    /* a higher-order a against one matrix: a single product over the flattened rows */
    if (transposedA == X_NOTRANS && a->order > 2 && b->order == 2) {
        int ncolA = a->dimSize[a->order - 1];
        int ncolC = c->dimSize[c->order - 1];
        XTensor * a2 = NewTensor2DV2(a->unitNum / ncolA, -ncolA, a->dataType, a->devID, a->mem);
        XTensor * c2 = NewTensor2DV2(c->unitNum / ncolC, -ncolC, c->dataType, c->devID, c->mem);
        a2->data = a->data;
        c2->data = c->data;
        if (bias == NULL)
            _MatrixMul2D(a2, transposedA, b, transposedB, c2, alpha, beta);
        else {
            BiasSpec spec = RowOrColumnBias(c, bias, n, c->order - 2);
            spec.act = act;
            if (a2->devID >= 0 || b->devID >= 0 || c2->devID >= 0)
                _AmdMatrixMul2DBias(a2, transposedA, b, transposedB, c2, alpha, beta, &spec);
            else {
                /* host tensors: the host tree's product, then its broadcast add in place, as MulAndShift does there
                   (MulAndShift.cpp:69, :88); both through the functions the tree handed in */
                CheckNTErrors(GetHostSumDim() != NULL && n != SCALAR_BIAS && act == 0,
                              "Host tensors are multiplied by NiuTensor's own CPU path, which this library does not replace!");
                _MatrixMul2D(a2, transposedA, b, transposedB, c2, alpha, beta);
                GetHostSumDim()(c, bias, c, n, (DTYPE)1.0);
            }
        }
        a2->data = NULL;
        c2->data = NULL;
        delete a2;
        delete c2;
        return;
    }

    MatDims da = MatrixDims(a, transposedA);
    MatDims db = MatrixDims(b, transposedB);
    int cn = c->dimSize[c->order - 2];
    int cm = c->dimSize[c->order - 1];

    CheckNTErrors((da.m == db.n && da.n == cn && db.m == cm), "Unmatched tensors in multiplication!");

    size_t aBlockBytes = (size_t)da.rows * da.cols * a->unitSize;
    size_t bBlockBytes = (size_t)db.rows * db.cols * b->unitSize;
    size_t cBlockBytes = (size_t)cn * cm * c->unitSize;
    int aBlockNum = 1;
    int bBlockNum = 1;

    for (int i = 0; i < a->order - 2; i++) {
        CheckNTErrors(a->dimSize[i] == c->dimSize[i], "Incorrect tensor sizes!");
        aBlockNum *= a->dimSize[i];
    }
    for (int i = 0; i < b->order - 2; i++) {
        CheckNTErrors(b->dimSize[i] == c->dimSize[i - 2 + a->order], "Incorrect tensor sizes!");
        bBlockNum *= b->dimSize[i];
    }

    CheckNTErrors(!a->isSparse && !b->isSparse, "Sparse matrices are outside this library.");

    /* the GPU takes the list only if all three tensors are on one (MatrixMul.cpp:156-175); anything else is
       the host's loop over the items (:180-185) */
    const bool onGpu = a->devID >= 0 && b->devID >= 0 && c->devID >= 0;
    if (onGpu) {
        CheckNTErrors((a->devID == b->devID && a->devID == c->devID), "The code must be run on the same GPU!");
    }
    else {
        CheckNTErrors(bias == NULL, "Host tensors are multiplied by NiuTensor's own CPU path, which this library does not replace!");
    }

    int aDimSize[2] = {-da.rows, da.cols};
    int bDimSize[2] = {-db.rows, db.cols};
    int cDimSize[2] = {-cn, cm};

    if (bias != NULL) {
        /* rare: a fused bias on a product that is not a single matrix. One launch per
           block, each with the slice of the bias that applies to it. */
        XTensor * ai = NewTensorV2(2, aDimSize, a->dataType, a->denseRatio, a->devID, a->mem);
        XTensor * bi = NewTensorV2(2, bDimSize, b->dataType, b->denseRatio, b->devID, b->mem);
        XTensor * ci = NewTensorV2(2, cDimSize, c->dataType, c->denseRatio, c->devID, c->mem);
        int inner = 1;   /* blocks per step of dimension n, when n is a leading dimension */
        for (int i = n + 1; i < c->order - 2; i++)
            inner *= c->dimSize[i];
        for (int p = 0; p < aBlockNum; p++) {
            for (int q = 0; q < bBlockNum; q++) {
                int block = p * bBlockNum + q;
                ai->data = (char *)a->data + aBlockBytes * p;
                bi->data = (char *)b->data + bBlockBytes * q;
                ci->data = (char *)c->data + cBlockBytes * block;
                BiasSpec spec;
                if (n >= c->order - 2 || n == SCALAR_BIAS)
                    spec = RowOrColumnBias(c, bias, n, c->order - 2);
                else {
                    spec.data = (const char *)bias->data + (size_t)((block / inner) % c->dimSize[n]) * bias->unitSize;
                    spec.mode = 2;
                    spec.len = 1;
                    spec.rowDiv = 1;
                }
                spec.act = act;
                _AmdMatrixMul2DBias(ai, transposedA, bi, transposedB, ci, alpha, beta, &spec);
            }
        }
        ai->data = NULL;
        bi->data = NULL;
        ci->data = NULL;
        delete ai;
        delete bi;
        delete ci;
        return;
    }

    TensorList * aList = new TensorList(aBlockNum * bBlockNum);
    TensorList * bList = new TensorList(aBlockNum * bBlockNum);
    TensorList * cList = new TensorList(aBlockNum * bBlockNum);

    for (int p = 0; p < aBlockNum; p++) {
        for (int q = 0; q < bBlockNum; q++) {
            XTensor * ai = NewTensorV2(2, aDimSize, a->dataType, a->denseRatio, a->devID, a->mem);
            XTensor * bi = NewTensorV2(2, bDimSize, b->dataType, b->denseRatio, b->devID, b->mem);
            XTensor * ci = NewTensorV2(2, cDimSize, c->dataType, c->denseRatio, c->devID, c->mem);
            ai->data = (char *)a->data + aBlockBytes * p;
            bi->data = (char *)b->data + bBlockBytes * q;
            ci->data = (char *)c->data + cBlockBytes * ((size_t)p * bBlockNum + q);
            aList->Add(ai);
            bList->Add(bi);
            cList->Add(ci);
        }
    }

    if (onGpu)
        _AmdMatrixMULList(a->devID, aList, transposedA, bList, transposedB, cList, aList->count, alpha, beta);
    else
        _MatrixMulBatchedCPU(aList, transposedA, bList, transposedB, cList, alpha, beta);

    for (int i = 0; i < aList->count; i++) {
        XTensor * t[3] = {aList->GetItem(i), bList->GetItem(i), cList->GetItem(i)};
        for (int k = 0; k < 3; k++) {
            t[k]->data = NULL;
            delete t[k];
        }
    }
    delete aList;
    delete bList;
    delete cList;
}

void _MatrixMul(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                XTensor * c, DTYPE alpha, DTYPE beta, XPRunner * parallelRunner)
{
    (void)parallelRunner;
    _MatrixMulBias(a, transposedA, b, transposedB, c, alpha, beta, NULL, -1);
}

bool CheckMMulShape(const XTensor * a, MATRIX_TRANS_TYPE transposedA, const XTensor * b, MATRIX_TRANS_TYPE transposedB,
                    XTensor * c)
{
    if (!(a && b && c))
        return false;
    if (!(a->dataType == b->dataType && a->dataType == c->dataType))
        return false;
    if (!(a->order >= 2 && b->order >= 2 && c->order >= 2))
        return false;

    CheckNTErrors(MatrixDims(a, transposedA).m == MatrixDims(b, transposedB).n, "Unmatched tensors in multiplication!");

    int dimSize[2 * MAX_TENSOR_DIM_NUM];
    int order = ResultShape(a, transposedA, b, transposedB, dimSize);
    /* as in the reference (:240-245), only c's first `order` sizes are compared */
    for (int i = 0; i < order; i++)
        if (dimSize[i] != c->dimSize[i])
            return false;
    return true;
}

static void CheckWrapperInputs(const XTensor & a, MATRIX_TRANS_TYPE transposedA, const XTensor & b, MATRIX_TRANS_TYPE transposedB)
{
    CheckNTErrors(a.dataType == b.dataType, "Input tensors should have the same data type!");
    CheckNTErrors(a.order >= 2 && b.order >= 2, "Input tensors must have a order >= 2!");
    CheckNTErrors(MatrixDims(&a, transposedA).m == MatrixDims(&b, transposedB).n, "Unmatched tensors in multiplication!");
    CheckNTErrors(a.order + b.order - 2 <= MAX_TENSOR_DIM_NUM, "The result has too many dimensions!");
}

/* autograd edge of a product: tails a and b, then transposedA, transposedB, alpha (:304-309) */
static void LinkProduct(const XTensor & a, MATRIX_TRANS_TYPE transposedA, const XTensor & b, MATRIX_TRANS_TYPE transposedB,
                        XTensor & c, DTYPE alpha)
{
    if (a.enableGrad && b.enableGrad) {
        XLink::MakeLink(&a, &b, &c, MATH_MATRIXMUL);
        XLink::AddParamToHeadTrans(&c, transposedA);
        XLink::AddParamToHeadTrans(&c, transposedB);
        XLink::AddParamToHead(&c, alpha);
    }
}

XTensor MatrixMul(const XTensor & a, MATRIX_TRANS_TYPE transposedA, const XTensor & b, MATRIX_TRANS_TYPE transposedB,
                  DTYPE alpha, XPRunner * parallelRunner)
{
    CheckWrapperInputs(a, transposedA, b, transposedB);

    int dimSize[2 * MAX_TENSOR_DIM_NUM];
    int order = ResultShape(&a, transposedA, &b, transposedB, dimSize);

    /* on a's device, with a's data type; dense (sparse operands are outside this library) */
    XTensor c(order, dimSize, a.dataType, 1.0F, a.devID, a.mem);
    c.SetTMPFlag();

    _MatrixMul(&a, transposedA, &b, transposedB, &c, alpha, 0, parallelRunner);
    LinkProduct(a, transposedA, b, transposedB, c, alpha);
    return c;
}

void MatrixMul(const XTensor & a, MATRIX_TRANS_TYPE transposedA, const XTensor & b, MATRIX_TRANS_TYPE transposedB,
               XTensor & c, DTYPE alpha, DTYPE beta, XPRunner * parallelRunner)
{
    CheckNTErrors(a.dataType == b.dataType, "Input tensors should have the same data type!");
    CheckNTErrors(a.order >= 2 && b.order >= 2, "Input tensors must have a order >= 2!");

    /* c is (re)made only if it is not initialised or does not have the product's shape (:324-348) */
    if (!c.isInit || !CheckMMulShape(&a, transposedA, &b, transposedB, &c)) {
        CheckWrapperInputs(a, transposedA, b, transposedB);
        int dimSize[2 * MAX_TENSOR_DIM_NUM];
        int order = ResultShape(&a, transposedA, &b, transposedB, dimSize);
        InitTensorV2(&c, order, dimSize, a.dataType, 1.0F, a.devID, a.mem);
        /* fresh memory is not zero here; a caller passing beta != 0 with an unformed c gets
           zero-initialised storage from the reference, so give the same */
        if (beta != 0)
            c.SetZeroAll();
    }

    _MatrixMul(&a, transposedA, &b, transposedB, &c, alpha, beta, parallelRunner);
    LinkProduct(a, transposedA, b, transposedB, c, alpha);
}

XTensor MatrixMul(const XTensor & a, const XTensor & b, DTYPE alpha, XPRunner * parallelRunner)
{
    return MatrixMul(a, X_NOTRANS, b, X_NOTRANS, alpha, parallelRunner);
}

void MatrixMul(const XTensor & a, const XTensor & b, XTensor & c, DTYPE alpha, XPRunner * parallelRunner)
{
    /* this overload always overwrites c (beta = 0, :449) */
    MatrixMul(a, X_NOTRANS, b, X_NOTRANS, c, alpha, 0, parallelRunner);
}

}  // namespace nts
