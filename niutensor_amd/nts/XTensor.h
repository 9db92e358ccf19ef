/*
 * A minimal nts::XTensor for the matrix-multiplication path on gfx950.
 *
 * It keeps the names and meaning of the fields the path reads in the reference
 * (source/tensor/XTensor.h:62-200): data, devID, order, dimSize, dataType,
 * unitSize, unitNum, isSparse, denseRatio, mem, isInit, isTmp, enableGrad, grad,
 * isGrad and the `income` edge used by autograd. It is not a re-implementation of the
 * reference's tensor class: memory pools, sparse storage, naming, gradients
 * and the 300-odd other members are outside this library. In an integration
 * the reference's own XTensor is used and only XTensorBLAS changes.
 *
 * Tensors are dense, row-major and contiguous. devID >= 0 is a GPU; devID < 0
 * is host memory, which this library only uses to stage data: the products
 * themselves refuse host tensors (the CPU path stays the reference's own).
 */
#ifndef NTSAMD_XTENSOR_H
#define NTSAMD_XTENSOR_H

#include "XGlobal.h"
#include "XDataType.h"

#include <stddef.h>

namespace nts {

#define MAX_TENSOR_DIM_NUM 8

/* operation ids recorded on autograd edges; values as in source/tensor/XName.h:32,56-57,69 */
#define MATH_BASE 0x00001000
#define MATH_MATRIXMUL (MATH_BASE + 21)
#define MATH_MATRIXMULBATCHED (MATH_BASE + 22)
#define MATH_MULANDSHIFT (MATH_BASE + 34)

struct XTensor;

/* memory pools are not part of this library: `mem` is carried, never used */
struct XMem;

/* The incoming hyper-edge of a tensor: which tensors it was computed from, by
   which operation, with which parameters (source/tensor/XLink.h:50-80). Only
   what MakeLink / AddParamToHead* record is kept. */
struct XLink {
    XTensor * head;
    const XTensor * tails[4];
    int tailNum;
    int typeID;
    /* parameters in the order they were added; each slot holds one int or one DTYPE */
    union Param {
        int i;
        DTYPE f;
    } params[8];
    bool paramIsInt[8];
    int paramNum;

    XLink();
    void Reset();

    static void MakeLink(const XTensor * t1, const XTensor * t2, XTensor * h, int id);
    static void MakeLink(const XTensor * t1, const XTensor * t2, const XTensor * t3, XTensor * h, int id);
    static void AddParamToHead(XTensor * h, DTYPE param);
    static void AddParamToHeadInt(XTensor * h, int param);
    static void AddParamToHeadTrans(XTensor * h, MATRIX_TRANS_TYPE param);

    /* parameter i as recorded (source/tensor/XLink.cpp:287-328) */
    DTYPE GetParam(int i) const;
    int GetParamInt(int i) const;
    MATRIX_TRANS_TYPE GetParamTrans(int i) const;
};

struct XTensor {
    int id;
    XMem * mem;
    void * data;
    int devID;
    int order;
    int dimSize[MAX_TENSOR_DIM_NUM];
    TENSOR_DATA_TYPE dataType;
    int unitSize;
    int unitNum;
    bool isSparse;
    int unitNumNonZero;
    float denseRatio;
    bool isInit;
    bool isTmp;
    bool enableGrad;
    /* dE/d(this tensor), owned by the tensor (source/tensor/XTensor.h:163-166); isGrad: the
       tensor wants its gradient kept when the backward pass runs in its "efficient" mode */
    XTensor * grad;
    bool isGrad;
    XLink income;

    XTensor();
    /* a tensor shaped like `reference` on the same device, values not copied (XTensor.cpp:96-102) */
    explicit XTensor(const XTensor * reference);
    /* a negative entry of myDimSize gives the shape without allocating: a view
       whose `data` the caller sets and clears (XTensor.cpp:1459-1463) */
    XTensor(const int myOrder, const int * myDimSize, const TENSOR_DATA_TYPE myDataType,
            const float myDenseRatio, int myDevID, XMem * myMem);
    /* copies the values, unless the source is a temporary, whose buffer is taken (XTensor.cpp:148-170) */
    XTensor(const XTensor & reference);
    XTensor & operator=(const XTensor & reference);
    ~XTensor();

    bool Resize(const int myOrder, const int * myDimSize, const TENSOR_DATA_TYPE myDataType = DEFAULT_DTYPE,
                const float myDenseRatio = 1.0F);
    void SetZeroAll();
    /* copy `num` elements from host memory into the tensor, starting at element `beg` */
    void SetData(const void * d, int num, int beg = 0);
    /* copy the whole tensor to host memory (a blocking copy: it also waits for the kernels before it) */
    void GetData(void * d) const;
    void SetTMPFlag(bool myIsTmp = true);
    void DestroyData();
    int GetDim(int dim) const;
    /* a new shape over the same elements (source/tensor/XTensor.cpp:618-650) */
    void Reshape(const int myOrder, const int * myDimSize);
    void Reshape(const int rowNum, const int colNum);

private:
    void Init();
    void ShallowCopy(const XTensor & reference);
};

/* creation helpers with the reference's names and defaults (source/tensor/XCall.h:39-192) */
void InitTensorV2(XTensor * tensor, const int myOrder, const int * myDimSize,
                  const TENSOR_DATA_TYPE myDataType = X_FLOAT, const float myDenseRatio = 1.0F,
                  const int myDevID = -1, XMem * myMem = NULL);
void InitTensorV2(XTensor * tensor, const XTensor * reference);
XTensor * NewTensorV2(const int myOrder, const int * myDimSize, const TENSOR_DATA_TYPE myDataType = X_FLOAT,
                      const float myDenseRatio = 1.0F, const int myDevID = -1, XMem * myMem = NULL);
XTensor * NewTensor2DV2(const int rowNum, const int colNum, const TENSOR_DATA_TYPE myDataType = X_FLOAT,
                        const int myDevID = -1, XMem * myMem = NULL);
XTensor * NewTensorBufV2(const int myOrder, const int * myDimSize, const TENSOR_DATA_TYPE myDataType = X_FLOAT,
                         const float myDenseRatio = 1.0F, const int myDevID = -1, XMem * myMem = NULL);
void DelTensorBuf(XTensor * tensor);
/* a tensor shaped like `a` on the same device (source/tensor/XCall.cpp:770-790) */
XTensor * NewTensor(const XTensor * a, bool isFilledData = true);

/* source/tensor/core/shape/IsSameShaped.cpp:32-58 */
bool _IsSameShaped(const XTensor * a, const XTensor * b);
bool IsSameShaped(const XTensor & a, const XTensor & b);

/* raw memory on a device (>= 0) or on the host (< 0), as XMemAlloc / XMemFree / XMemCopy */
void * XMemAlloc(int devID, size_t size);
void XMemFree(int devID, void * p);
void XMemCopy(void * t, int devIDT, const void * s, int devIDS, size_t size);

/* Freed device blocks are kept per device and size class and handed out again (see XTensor.cpp).
   XMemCacheRelease returns every idle block of a device to the HIP runtime; XMemCacheStats reports the
   idle bytes of a device and how many requests were (not) served from the lists; XMemCacheEnable(false)
   makes every later request and release go straight to hipMalloc / hipFree. */
void XMemCacheRelease(int devID);
void XMemCacheStats(int devID, size_t * spareBytes, long long * hits, long long * misses);
void XMemCacheEnable(bool on);

}  // namespace nts
#endif
