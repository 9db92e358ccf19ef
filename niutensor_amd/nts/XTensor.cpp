/*
 * Minimal nts::XTensor for the gfx950 matrix-multiplication path: shape
 * bookkeeping, device memory through the HIP runtime, autograd-edge records.
 * Field meaning follows source/tensor/XTensor.h:62-200 of the reference.
 */
#include "XTensor.h"

#include <hip/hip_runtime_api.h>

#include <atomic>
#include <mutex>
#include <stdlib.h>
#include <string.h>
#include <unordered_map>
#include <vector>

namespace nts {

static std::atomic<int> tensorIDGlobal(0);

#define MAX_CACHED_DEVICES 16

#define CheckHip(call, msg) \
{ \
    hipError_t e_ = (call); \
    if (e_ != hipSuccess) { \
        fprintf(stderr, "[ERROR] HIP: %s\n", hipGetErrorString(e_)); \
        ShowNTErrors(msg); \
    } \
}

/* run `body` with devID current, then restore the caller's device
   (ProtectCudaDev / BacktoCudaDev, source/tensor/XDevice.h:233-244) */
struct DevScope {
    int backup;
    bool switched;
    explicit DevScope(int devID) : backup(-1), switched(false)
    {
        if (devID < 0)
            return;
        if (hipGetDevice(&backup) != hipSuccess)
            backup = -1;
        if (backup != devID) {
            CheckHip(hipSetDevice(devID), "Cannot set the GPU device!");
            switched = true;
        }
    }
    ~DevScope()
    {
        if (switched && backup >= 0)
            (void)hipSetDevice(backup);
    }
};

/* ---- device memory: blocks are kept and handed out again ----------------------
   The reference takes the temporaries of a forward or backward step out of a memory pool
   (XMem, source/tensor/XMem.h:150-420) when one is attached, and calls cudaMalloc / cudaFree
   per tensor when none is (XUtility.cpp XMemAlloc / XMemFree). hipFree waits for the device
   and hipMalloc costs tens of microseconds, more than an attention-sized product takes, so
   here a freed block goes onto a per-device list of its size class and the next request of
   that class takes it from there. That is safe because every kernel and copy of this layer
   is issued to the NULL stream, as in the reference: whatever still reads or writes a block
   when the host gives it up has been queued before anything that the block's next owner
   queues. Size classes keep three leading bits (at most 12.5 % slack), 256 bytes at least.
   NTSAMD_MEM_CACHE=0 switches the lists off; NTSAMD_MEM_CACHE_MB caps the bytes kept per
   device (default 32768); XMemCacheRelease gives everything back. */

struct MemCache {
    std::mutex lock;
    std::unordered_map<void *, size_t> live[MAX_CACHED_DEVICES];               /* block -> class size */
    std::unordered_map<size_t, std::vector<void *> > spare[MAX_CACHED_DEVICES];  /* class size -> free blocks */
    size_t spareBytes[MAX_CACHED_DEVICES];
    long long hits, misses;
    bool enabled;
    size_t capBytes;
    MemCache() : hits(0), misses(0)
    {
        for (int i = 0; i < MAX_CACHED_DEVICES; i++)
            spareBytes[i] = 0;
        const char * e = getenv("NTSAMD_MEM_CACHE");
        enabled = !(e != NULL && e[0] == '0');
        const char * c = getenv("NTSAMD_MEM_CACHE_MB");
        capBytes = (size_t)(c != NULL ? atoll(c) : 32768) << 20;
    }
};

static MemCache & Cache()
{
    static MemCache * c = new MemCache();      /* never destroyed: tensors with static lifetime may outlive it */
    return *c;
}

static size_t SizeClass(size_t size)
{
    if (size <= 256)
        return 256;
    int top = 63 - __builtin_clzll((unsigned long long)(size - 1));      /* highest set bit of size - 1 */
    size_t step = (size_t)1 << (top >= 3 ? top - 2 : 0);                  /* keep three leading bits */
    if (step < 256)
        step = 256;
    return (size + step - 1) / step * step;
}

void * XMemAlloc(int devID, size_t size)
{
    void * p = NULL;
    if (size == 0)
        return NULL;
    if (devID < 0) {
        p = malloc(size);
        CheckNTErrors(p != NULL, "Cannot allocate the memory.");
        return p;
    }
    MemCache & mc = Cache();
    if (!mc.enabled || devID >= MAX_CACHED_DEVICES) {
        DevScope scope(devID);
        CheckHip(hipMalloc(&p, size), "Cannot allocate the memory.");
        return p;
    }
    const size_t cls = SizeClass(size);
    {
        std::lock_guard<std::mutex> guard(mc.lock);
        std::vector<void *> & list = mc.spare[devID][cls];
        if (!list.empty()) {
            p = list.back();
            list.pop_back();
            mc.spareBytes[devID] -= cls;
            mc.live[devID][p] = cls;
            mc.hits++;
            return p;
        }
        mc.misses++;
    }
    DevScope scope(devID);
    hipError_t e = hipMalloc(&p, cls);
    if (e != hipSuccess) {
        /* out of memory with blocks lying idle: give them back and try once more */
        (void)hipGetLastError();
        XMemCacheRelease(devID);
        CheckHip(hipMalloc(&p, cls), "Cannot allocate the memory.");
    }
    std::lock_guard<std::mutex> guard(mc.lock);
    mc.live[devID][p] = cls;
    return p;
}

void XMemFree(int devID, void * p)
{
    if (p == NULL)
        return;
    if (devID < 0) {
        free(p);
        return;
    }
    MemCache & mc = Cache();
    if (devID < MAX_CACHED_DEVICES) {
        std::lock_guard<std::mutex> guard(mc.lock);
        std::unordered_map<void *, size_t>::iterator it = mc.live[devID].find(p);
        if (it != mc.live[devID].end()) {
            const size_t cls = it->second;
            mc.live[devID].erase(it);
            if (mc.enabled && mc.spareBytes[devID] + cls <= mc.capBytes) {
                mc.spare[devID][cls].push_back(p);
                mc.spareBytes[devID] += cls;
                return;
            }
        }
    }
    DevScope scope(devID);
    CheckHip(hipFree(p), "Cannot free the memory.");
}

void XMemCacheRelease(int devID)
{
    MemCache & mc = Cache();
    if (devID < 0 || devID >= MAX_CACHED_DEVICES)
        return;
    std::vector<void *> blocks;
    {
        std::lock_guard<std::mutex> guard(mc.lock);
        for (std::unordered_map<size_t, std::vector<void *> >::iterator it = mc.spare[devID].begin();
             it != mc.spare[devID].end(); ++it)
            blocks.insert(blocks.end(), it->second.begin(), it->second.end());
        mc.spare[devID].clear();
        mc.spareBytes[devID] = 0;
    }
    if (blocks.empty())
        return;
    DevScope scope(devID);
    for (size_t i = 0; i < blocks.size(); i++)
        CheckHip(hipFree(blocks[i]), "Cannot free the memory.");
}

void XMemCacheStats(int devID, size_t * spareBytes, long long * hits, long long * misses)
{
    MemCache & mc = Cache();
    std::lock_guard<std::mutex> guard(mc.lock);
    if (spareBytes != NULL)
        *spareBytes = devID >= 0 && devID < MAX_CACHED_DEVICES ? mc.spareBytes[devID] : 0;
    if (hits != NULL)
        *hits = mc.hits;
    if (misses != NULL)
        *misses = mc.misses;
}

void XMemCacheEnable(bool on)
{
    MemCache & mc = Cache();
    std::lock_guard<std::mutex> guard(mc.lock);
    mc.enabled = on;
}

void XMemCopy(void * t, int devIDT, const void * s, int devIDS, size_t size)
{
    if (t == s || size == 0)
        return;
    if (devIDT < 0 && devIDS < 0) {
        memcpy(t, s, size);
        return;
    }
    DevScope scope(devIDT >= 0 ? devIDT : devIDS);
    hipMemcpyKind kind = devIDT < 0 ? hipMemcpyDeviceToHost
                       : devIDS < 0 ? hipMemcpyHostToDevice : hipMemcpyDeviceToDevice;
    CheckHip(hipMemcpy(t, s, size, kind), "hipMemcpy error");
}

/* ---- XLink ---------------------------------------------------------------- */

XLink::XLink()
{
    Reset();
}

void XLink::Reset()
{
    head = NULL;
    tailNum = 0;
    typeID = 0;
    paramNum = 0;
    for (int i = 0; i < 4; i++)
        tails[i] = NULL;
}

void XLink::MakeLink(const XTensor * t1, const XTensor * t2, XTensor * h, int id)
{
    CheckNTErrors(h != NULL, "head tensor cannot be empty!");
    h->income.Reset();
    h->income.head = h;
    h->income.typeID = id;
    h->income.tails[0] = t1;
    h->income.tails[1] = t2;
    h->income.tailNum = t2 != NULL ? 2 : 1;
}

void XLink::MakeLink(const XTensor * t1, const XTensor * t2, const XTensor * t3, XTensor * h, int id)
{
    MakeLink(t1, t2, h, id);
    h->income.tails[2] = t3;
    h->income.tailNum = 3;
}

void XLink::AddParamToHead(XTensor * h, DTYPE param)
{
    CheckNTErrors(h != NULL, "head tensor cannot be empty!");
    CheckNTErrors(h->income.paramNum < 8, "too many parameters");
    h->income.paramIsInt[h->income.paramNum] = false;
    h->income.params[h->income.paramNum++].f = param;
}

void XLink::AddParamToHeadInt(XTensor * h, int param)
{
    CheckNTErrors(h != NULL, "head tensor cannot be empty!");
    CheckNTErrors(h->income.paramNum < 8, "too many parameters");
    h->income.paramIsInt[h->income.paramNum] = true;
    h->income.params[h->income.paramNum++].i = param;
}

void XLink::AddParamToHeadTrans(XTensor * h, MATRIX_TRANS_TYPE param)
{
    AddParamToHeadInt(h, (int)param);
}

DTYPE XLink::GetParam(int i) const
{
    CheckNTErrors(i >= 0 && i < paramNum, "parameter array cannot be empty!");
    return params[i].f;
}

int XLink::GetParamInt(int i) const
{
    CheckNTErrors(i >= 0 && i < paramNum, "parameter array cannot be empty!");
    return params[i].i;
}

MATRIX_TRANS_TYPE XLink::GetParamTrans(int i) const
{
    return (MATRIX_TRANS_TYPE)GetParamInt(i);
}

/* ---- XTensor -------------------------------------------------------------- */

void XTensor::Init()
{
    id = -1;
    mem = NULL;
    data = NULL;
    devID = -1;
    order = -1;
    memset(dimSize, 0, sizeof(dimSize));
    dataType = DEFAULT_DTYPE;
    unitSize = sizeof(float);
    unitNum = 0;
    isSparse = false;
    unitNumNonZero = 0;
    denseRatio = 1.0F;
    isInit = false;
    isTmp = false;
    enableGrad = false;
    grad = NULL;
    isGrad = false;
    income.Reset();
}

XTensor::XTensor()
{
    Init();
    id = ++tensorIDGlobal;
}

XTensor::XTensor(const XTensor * reference)
{
    Init();
    id = ++tensorIDGlobal;
    InitTensorV2(this, reference);
}

XTensor::XTensor(const int myOrder, const int * myDimSize, const TENSOR_DATA_TYPE myDataType,
                 const float myDenseRatio, int myDevID, XMem * myMem)
{
    Init();
    id = ++tensorIDGlobal;
    order = myOrder;
    mem = myMem;
    devID = myDevID;
    if (order >= 0)
        Resize(myOrder, myDimSize, myDataType, myDenseRatio);
}

void XTensor::ShallowCopy(const XTensor & t)
{
    order = t.order;
    memcpy(dimSize, t.dimSize, sizeof(dimSize));
    dataType = t.dataType;
    unitSize = t.unitSize;
    unitNum = t.unitNum;
    isSparse = t.isSparse;
    unitNumNonZero = t.unitNumNonZero;
    denseRatio = t.denseRatio;
    isInit = t.isInit;
    enableGrad = t.enableGrad;
}

XTensor::XTensor(const XTensor & reference)
{
    Init();
    id = ++tensorIDGlobal;
    *this = reference;
}

XTensor & XTensor::operator=(const XTensor & reference)
{
    if (this == &reference)
        return *this;
    DestroyData();
    ShallowCopy(reference);
    devID = reference.devID;
    mem = reference.mem;
    if (reference.isTmp) {
        /* a temporary hands its buffer over instead of being copied */
        data = reference.data;
        const_cast<XTensor &>(reference).data = NULL;
    }
    else if (reference.data != NULL && unitNum > 0) {
        data = XMemAlloc(devID, (size_t)unitNum * unitSize);
        XMemCopy(data, devID, reference.data, reference.devID, (size_t)unitNum * unitSize);
    }
    /* the edge that produced the source describes the copy as well */
    income = reference.income;
    if (income.head != NULL)
        income.head = this;
    isTmp = false;
    return *this;
}

XTensor::~XTensor()
{
    DestroyData();
    if (grad != NULL)
        delete grad;
}

void XTensor::DestroyData()
{
    if (data != NULL)
        XMemFree(devID, data);
    data = NULL;
}

bool XTensor::Resize(const int myOrder, const int * myDimSize, const TENSOR_DATA_TYPE myDataType,
                     const float myDenseRatio)
{
    CheckNTErrors(myOrder >= 0 && myOrder <= MAX_TENSOR_DIM_NUM, "Illegal tensor order!");
    CheckNTErrors(myDenseRatio >= 1.0F, "Sparse tensors are outside this library.");
    DestroyData();

    order = myOrder;
    unitNum = 1;
    unitNumNonZero = 0;
    isInit = true;

    bool filledData = true;
    bool zeroData = false;
    for (int i = 0; i < order; i++) {
        dimSize[i] = abs(myDimSize[i]);
        if (myDimSize[i] < 0)
            filledData = false;
        if (myDimSize[i] == 0)
            zeroData = true;
        unitNum *= dimSize[i];
    }

    denseRatio = myDenseRatio;
    isSparse = false;
    dataType = myDataType;
    unitSize = GetUnitSize(dataType);

    if (zeroData) {
        unitNum = 0;
        return false;
    }

    if (filledData) {
        data = XMemAlloc(devID, (size_t)unitNum * unitSize);
        /* the reference hands out zeroed memory (XTensor.cpp:1528-1534); the products
           never depend on that, so the fill is left to SetZeroAll */
    }
    return true;
}

void XTensor::SetZeroAll()
{
    if (data == NULL || unitNum == 0)
        return;
    if (devID < 0)
        memset(data, 0, (size_t)unitNum * unitSize);
    else {
        DevScope scope(devID);
        CheckHip(hipMemset(data, 0, (size_t)unitNum * unitSize), "hipMemset error");
    }
}

void XTensor::SetData(const void * d, int num, int beg)
{
    if (data == NULL || d == NULL)
        return;
    CheckNTErrors(beg >= 0 && num >= 0 && beg + num <= unitNum, "Illegal size!");
    XMemCopy((char *)data + (size_t)beg * unitSize, devID, d, -1, (size_t)num * unitSize);
}

void XTensor::GetData(void * d) const
{
    if (data == NULL || d == NULL)
        return;
    XMemCopy(d, -1, data, devID, (size_t)unitNum * unitSize);
}

void XTensor::SetTMPFlag(bool myIsTmp)
{
    isTmp = myIsTmp;
}

int XTensor::GetDim(int dim) const
{
    CheckNTErrors(dim < order, "dimenision is out of range!");
    int d = dim;
    if (dim < 0)
        d = order + dim;
    return dimSize[d];
}

void XTensor::Reshape(const int myOrder, const int * myDimSize)
{
    CheckNTErrors(myOrder >= 0 && myOrder <= MAX_TENSOR_DIM_NUM, "Illegal tensor order!");
    int num = 1;
    for (int i = 0; i < myOrder; i++)
        num *= myDimSize[i];
    CheckNTErrors(abs(num) == unitNum, "Wrong size for reshape!");
    order = myOrder;
    memset(dimSize, 0, sizeof(dimSize));
    for (int i = 0; i < myOrder; i++)
        dimSize[i] = abs(myDimSize[i]);
}

void XTensor::Reshape(const int rowNum, const int colNum)
{
    int dims[2] = {rowNum, colNum};
    Reshape(2, dims);
}

/* ---- creation helpers ----------------------------------------------------- */

void InitTensorV2(XTensor * tensor, const int myOrder, const int * myDimSize,
                  const TENSOR_DATA_TYPE myDataType, const float myDenseRatio,
                  const int myDevID, XMem * myMem)
{
    tensor->DestroyData();
    tensor->mem = myMem;
    tensor->devID = myDevID;
    tensor->Resize(myOrder, myDimSize, myDataType, myDenseRatio);
}

void InitTensorV2(XTensor * tensor, const XTensor * reference)
{
    if (reference->order < 0)
        return;
    tensor->enableGrad = reference->enableGrad;
    InitTensorV2(tensor, reference->order, reference->dimSize, reference->dataType, reference->denseRatio,
                 reference->devID, reference->mem);
}

XTensor * NewTensorV2(const int myOrder, const int * myDimSize, const TENSOR_DATA_TYPE myDataType,
                      const float myDenseRatio, const int myDevID, XMem * myMem)
{
    return new XTensor(myOrder, myDimSize, myDataType, myDenseRatio, myDevID, myMem);
}

XTensor * NewTensor2DV2(const int rowNum, const int colNum, const TENSOR_DATA_TYPE myDataType,
                        const int myDevID, XMem * myMem)
{
    int dims[2] = {rowNum, colNum};
    return new XTensor(2, dims, myDataType, 1.0F, myDevID, myMem);
}

/* without memory pools a buffer tensor is an ordinary one (source/tensor/XCall.cpp:510-530 falls
   back to NewTensorV2 when there is no pool) */
XTensor * NewTensorBufV2(const int myOrder, const int * myDimSize, const TENSOR_DATA_TYPE myDataType,
                         const float myDenseRatio, const int myDevID, XMem * myMem)
{
    return NewTensorV2(myOrder, myDimSize, myDataType, myDenseRatio, myDevID, myMem);
}

XTensor * NewTensor(const XTensor * a, bool isFilledData)
{
    CheckNTErrors(a != NULL, "Empty input!");
    int dims[MAX_TENSOR_DIM_NUM];
    memcpy(dims, a->dimSize, sizeof(int) * MAX_TENSOR_DIM_NUM);
    if (!isFilledData && a->order > 0)
        dims[0] = -dims[0];
    return new XTensor(a->order, dims, a->dataType, a->denseRatio, a->devID, a->mem);
}

void DelTensorBuf(XTensor * tensor)
{
    delete tensor;
}

bool _IsSameShaped(const XTensor * a, const XTensor * b)
{
    if (a == NULL || b == NULL)
        return false;
    if (a->order != b->order)
        return false;
    for (int i = 0; i < a->order; i++)
        if (a->dimSize[i] != b->dimSize[i])
            return false;
    if (a->dataType != b->dataType)
        return false;
    if (a->denseRatio != b->denseRatio)
        return false;
    if (a->isSparse != b->isSparse)
        return false;
    return true;
}

bool IsSameShaped(const XTensor & a, const XTensor & b)
{
    return _IsSameShaped(&a, &b);
}

}  // namespace nts
