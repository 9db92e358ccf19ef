/*
 * C ABI of the gfx950 matrix-multiplication library (declared in
 * include/ntsamd_gemm.h): argument checking, device handling and the choice
 * of kernel. Takes the place of source/tensor/core/arithmetic/XTensorBLAS.cu
 * in the reference.
 */
#include "../../include/ntsamd_gemm.h"
#include "gemm_common.h"

#include <atomic>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

namespace ntsamd {
int launch_f32_nn(const GemmParams &, const PtrBatch *, bool, int, hipStream_t);
int launch_f32_nt(const GemmParams &, const PtrBatch *, bool, int, hipStream_t);
int launch_f32_tn(const GemmParams &, const PtrBatch *, bool, int, hipStream_t);
int launch_f32_tt(const GemmParams &, const PtrBatch *, bool, int, hipStream_t);
int launch_f16_nn(const GemmParams &, const PtrBatch *, bool, bool, int, hipStream_t);
int launch_f16_nt(const GemmParams &, const PtrBatch *, bool, bool, int, hipStream_t);
int launch_f16_tn(const GemmParams &, const PtrBatch *, bool, bool, int, hipStream_t);
int launch_f16_tt(const GemmParams &, const PtrBatch *, bool, bool, int, hipStream_t);
}

using namespace ntsamd;

namespace {

thread_local char g_error[512] = "";

int fail(int code, const char * fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

/* devices already checked: written once per device, read-only afterwards */
constexpr int MAX_DEVICES = 64;
std::atomic<int> g_deviceState[MAX_DEVICES];   /* 0 unknown, 1 good, -1 not gfx950 */

int check_device(int devID)
{
    if (devID < 0 || devID >= MAX_DEVICES)
        return fail(NTSAMD_ERR_DEVICE, "invalid device id %d", devID);
    int st = g_deviceState[devID].load(std::memory_order_acquire);
    if (st == 1)
        return NTSAMD_OK;
    if (st == 0) {
        int n = 0;
        if (hipGetDeviceCount(&n) != hipSuccess || devID >= n)
            return fail(NTSAMD_ERR_DEVICE, "no GPU with id %d (%d visible)", devID, n);
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, devID) != hipSuccess)
            return fail(NTSAMD_ERR_DEVICE, "cannot query device %d", devID);
        st = strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : -1;
        g_deviceState[devID].store(st, std::memory_order_release);
        if (st == 1)
            return NTSAMD_OK;
    }
    return fail(NTSAMD_ERR_DEVICE, "device %d is not a gfx950 (MI355X) device; this library holds gfx950 code only", devID);
}

/* switch to devID for the duration of a call and back, as ProtectCudaDev /
   BacktoCudaDev do in the reference (XDevice.h:233-244) */
struct DeviceScope {
    int backup;
    bool switched;
    int status;
    explicit DeviceScope(int devID) : backup(-1), switched(false), status(NTSAMD_OK)
    {
        if (hipGetDevice(&backup) != hipSuccess)
            backup = -1;
        if (backup != devID) {
            if (hipSetDevice(devID) != hipSuccess)
                status = fail(NTSAMD_ERR_DEVICE, "cannot switch to device %d", devID);
            else
                switched = true;
        }
    }
    ~DeviceScope()
    {
        if (switched && backup >= 0)
            (void)hipSetDevice(backup);
    }
};

struct Shape {
    int M, N, K;
    bool aKContig, bKContig;
};

int check_shape(int transposedA, int transposedB, int na, int ma, int nb, int mb, int nc, int mc, Shape & s)
{
    if ((transposedA != NTSAMD_X_TRANS && transposedA != NTSAMD_X_NOTRANS) ||
        (transposedB != NTSAMD_X_TRANS && transposedB != NTSAMD_X_NOTRANS))
        return fail(NTSAMD_ERR_ARGUMENT, "transpose flags must be X_TRANS (0) or X_NOTRANS (1), got %d and %d",
                    transposedA, transposedB);
    if (na < 0 || ma < 0 || nb < 0 || mb < 0 || nc < 0 || mc < 0)
        return fail(NTSAMD_ERR_ARGUMENT, "negative matrix size");
    int an = transposedA == NTSAMD_X_TRANS ? ma : na;
    int am = transposedA == NTSAMD_X_TRANS ? na : ma;
    int bn = transposedB == NTSAMD_X_TRANS ? mb : nb;
    int bm = transposedB == NTSAMD_X_TRANS ? nb : mb;
    /* the test the callers of the reference make (MatrixMul2D.cu:133-134) */
    if (!(am == bn && an == nc && bm == mc))
        return fail(NTSAMD_ERR_ARGUMENT, "Unmatched matrices in multiplication!");
    s.M = nc;
    s.N = mc;
    s.K = am;
    s.aKContig = transposedA == NTSAMD_X_NOTRANS;
    s.bKContig = transposedB == NTSAMD_X_TRANS;
    return NTSAMD_OK;
}

enum Kind { KIND_F32, KIND_F16, KIND_F16_F32OUT };

int check_types(int ta, int tb, int tc, Kind & kind)
{
    if (ta == NTSAMD_X_FLOAT && tb == NTSAMD_X_FLOAT && tc == NTSAMD_X_FLOAT)
        kind = KIND_F32;
    else if (ta == NTSAMD_X_FLOAT16 && tb == NTSAMD_X_FLOAT16 && tc == NTSAMD_X_FLOAT16)
        kind = KIND_F16;
    else if (ta == NTSAMD_X_FLOAT16 && tb == NTSAMD_X_FLOAT16 && tc == NTSAMD_X_FLOAT)
        kind = KIND_F16_F32OUT;
    else
        return fail(NTSAMD_ERR_DATATYPE, "Unsupported data type!");
    return NTSAMD_OK;
}

bool aligned16(const void * p)
{
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

/* Relative run time of a product under a tile shape: rounds of workgroups (256 CUs x the
   workgroups a CU holds at once) times the work of one tile, divided by how fast the shape
   runs relative to the best one on a product that fits it (measured: small tiles re-read
   operands from LDS more often per MFMA, which costs fp16 far more than fp32). */
double tile_cost(int M, int N, int count, int bm, int bn, int perCU, double quality)
{
    long long tiles = (long long)((M + bm - 1) / bm) * ((N + bn - 1) / bn) * count;
    long long slots = 256LL * perCU;
    long long rounds = (tiles + slots - 1) / slots;
    return (double)rounds * bm * bn / quality;
}

/* NTSAMD_TILE_CFG=0|1|2 forces a tile shape (128x128, 64x64, 256x256 for half; for
   measurements); otherwise the shape with the lowest estimated run time */
int choose_cfg(int M, int N, int count, bool half)
{
    const char * e = getenv("NTSAMD_TILE_CFG");
    if (e && e[0] >= '0' && e[0] < '0' + CFG_COUNT && e[1] == 0) {
        int cfg = e[0] - '0';
        if (cfg == CFG_256x256 && !half)
            cfg = CFG_128x128;
        return cfg;
    }
    int best = CFG_64x64;
    double bestCost = tile_cost(M, N, count, 64, 64, 2, half ? 0.2 : 0.8);
    double c128 = tile_cost(M, N, count, 128, 128, 2, half ? 0.45 : 1.0);
    if (c128 <= bestCost) {
        best = CFG_128x128;
        bestCost = c128;
    }
    if (half) {
        double c256 = tile_cost(M, N, count, 256, 256, 1, 1.0);
        if (c256 <= bestCost)
            best = CFG_256x256;
    }
    return best;
}

int run(int devID, void * stream, Kind kind, const Shape & s,
        const void * a, const void * b, void * c,
        int lda, int ldb, int ldc,
        long long strideA, long long strideB, long long strideC, int count,
        const PtrBatch * ptrs,
        float alpha, float beta,
        const void * bias, int biasMode, int biasLen, int biasRowDiv)
{
    if (count == 0 || s.M == 0 || s.N == 0)
        return NTSAMD_OK;

    int st = check_device(devID);
    if (st != NTSAMD_OK)
        return st;
    DeviceScope scope(devID);
    if (scope.status != NTSAMD_OK)
        return scope.status;

    GemmParams p;
    memset(&p, 0, sizeof(p));
    p.a = a;
    p.b = b;
    p.c = c;
    p.bias = bias;
    p.M = s.M;
    p.N = s.N;
    p.K = s.K;
    p.lda = lda;
    p.ldb = ldb;
    p.ldc = ldc;
    p.strideA = strideA;
    p.strideB = strideB;
    p.strideC = strideC;
    p.alpha = alpha;
    p.beta = beta;
    p.biasMode = biasMode;
    p.biasRowDiv = biasRowDiv > 0 ? biasRowDiv : 1;
    p.biasLen = biasLen > 0 ? biasLen : 1;
    p.batch = count;
    p.groupM = 8;

    const int vecElems = kind == KIND_F32 ? 4 : 8;
    /* the fast path: 16-byte buffer loads of a and b, buffer stores of c, bias by column
       only. It keeps a tile's byte offsets in 31 bits, so rows longer than 2M elements
       go through the generic path, like everything unaligned and row-indexed bias */
    bool vec = !ptrs && kind != KIND_F16_F32OUT &&
               lda % vecElems == 0 && ldb % vecElems == 0 && aligned16(a) && aligned16(b) &&
               strideA % vecElems == 0 && strideB % vecElems == 0 &&
               lda < (1 << 21) && ldb < (1 << 21) && ldc < (1 << 21) &&
               biasMode != NTSAMD_BIAS_ROW;
    int cfg = choose_cfg(s.M, s.N, count, kind != KIND_F32);
    hipStream_t hs = static_cast<hipStream_t>(stream);

    int rc;
    if (kind == KIND_F32) {
        if (s.aKContig)
            rc = s.bKContig ? launch_f32_nt(p, ptrs, vec, cfg, hs) : launch_f32_nn(p, ptrs, vec, cfg, hs);
        else
            rc = s.bKContig ? launch_f32_tt(p, ptrs, vec, cfg, hs) : launch_f32_tn(p, ptrs, vec, cfg, hs);
    }
    else {
        bool outF32 = kind == KIND_F16_F32OUT;
        if (s.aKContig)
            rc = s.bKContig ? launch_f16_nt(p, ptrs, vec, outF32, cfg, hs) : launch_f16_nn(p, ptrs, vec, outF32, cfg, hs);
        else
            rc = s.bKContig ? launch_f16_tt(p, ptrs, vec, outF32, cfg, hs) : launch_f16_tn(p, ptrs, vec, outF32, cfg, hs);
    }
    if (rc != 0)
        return fail(NTSAMD_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString((hipError_t)rc));
    return NTSAMD_OK;
}

int check_pointers(const void * a, const void * b, const void * c)
{
    if (!a || !b || !c)
        return fail(NTSAMD_ERR_ARGUMENT, "Empty matrices in multiplication!");
    return NTSAMD_OK;
}

}  // namespace

extern "C" {

const char * ntsamd_last_error(void)
{
    return g_error;
}

const char * ntsamd_version(void)
{
    return "0.1";
}

int ntsamd_init(int devID)
{
    int st = check_device(devID);
    if (st != NTSAMD_OK)
        return st;
    DeviceScope scope(devID);
    if (scope.status != NTSAMD_OK)
        return scope.status;
    return NTSAMD_OK;
}

int ntsamd_matrix_mul_bias(int devID, void * stream,
                           const void * a, int transposedA, int dataTypeA,
                           const void * b, int transposedB, int dataTypeB,
                           void * c, int dataTypeC,
                           int na, int ma, int nb, int mb, int nc, int mc,
                           float alpha, float beta,
                           const void * bias, int biasMode, int biasLen, int biasRowDiv)
{
    Kind kind;
    Shape s;
    int st = check_types(dataTypeA, dataTypeB, dataTypeC, kind);
    if (st == NTSAMD_OK)
        st = check_shape(transposedA, transposedB, na, ma, nb, mb, nc, mc, s);
    if (st != NTSAMD_OK)
        return st;
    if (s.M == 0 || s.N == 0)
        return NTSAMD_OK;
    st = check_pointers(a, b, c);
    if (st != NTSAMD_OK)
        return st;
    if (biasMode != NTSAMD_BIAS_NONE) {
        if (biasMode != NTSAMD_BIAS_COL && biasMode != NTSAMD_BIAS_ROW)
            return fail(NTSAMD_ERR_ARGUMENT, "unknown bias mode %d", biasMode);
        if (!bias || biasLen <= 0)
            return fail(NTSAMD_ERR_ARGUMENT, "bias requested but empty");
        if (biasMode == NTSAMD_BIAS_COL && biasLen != mc)
            return fail(NTSAMD_ERR_ARGUMENT, "Wrong tensor size!");   /* SumDim.cpp:59 */
        if (biasMode == NTSAMD_BIAS_ROW && biasRowDiv <= 0)
            return fail(NTSAMD_ERR_ARGUMENT, "bias row divisor must be positive");
    }
    return run(devID, stream, kind, s, a, b, c, ma, mb, mc, 0, 0, 0, 1, NULL, alpha, beta,
               biasMode == NTSAMD_BIAS_NONE ? NULL : bias, biasMode, biasLen, biasRowDiv);
}

int ntsamd_matrix_mul(int devID, void * stream,
                      const void * a, int transposedA, int dataTypeA,
                      const void * b, int transposedB, int dataTypeB,
                      void * c, int dataTypeC,
                      int na, int ma, int nb, int mb, int nc, int mc,
                      float alpha, float beta)
{
    return ntsamd_matrix_mul_bias(devID, stream, a, transposedA, dataTypeA, b, transposedB, dataTypeB,
                                  c, dataTypeC, na, ma, nb, mb, nc, mc, alpha, beta,
                                  NULL, NTSAMD_BIAS_NONE, 0, 1);
}

int ntsamd_matrix_mul_batched_strided(int devID, void * stream,
                                      const void * a, int transposedA, int dataTypeA, long long strideA,
                                      const void * b, int transposedB, int dataTypeB, long long strideB,
                                      void * c, int dataTypeC, long long strideC,
                                      int count, int na, int ma, int nb, int mb, int nc, int mc,
                                      float alpha, float beta)
{
    Kind kind;
    Shape s;
    int st = check_types(dataTypeA, dataTypeB, dataTypeC, kind);
    if (st == NTSAMD_OK)
        st = check_shape(transposedA, transposedB, na, ma, nb, mb, nc, mc, s);
    if (st != NTSAMD_OK)
        return st;
    if (count < 0)
        return fail(NTSAMD_ERR_ARGUMENT, "negative batch count");
    if (count == 0 || s.M == 0 || s.N == 0)
        return NTSAMD_OK;
    st = check_pointers(a, b, c);
    if (st != NTSAMD_OK)
        return st;
    if (strideA < 0 || strideB < 0 || strideC < 0)
        return fail(NTSAMD_ERR_ARGUMENT, "negative batch stride");
    if (count > 1 && strideC < (long long)nc * mc)
        return fail(NTSAMD_ERR_ARGUMENT, "result matrices of the batch overlap");
    return run(devID, stream, kind, s, a, b, c, ma, mb, mc, strideA, strideB, strideC, count, NULL,
               alpha, beta, NULL, NTSAMD_BIAS_NONE, 0, 1);
}

int ntsamd_matrix_mul_batched(int devID, void * stream,
                              const void * const * a, int transposedA, int dataTypeA,
                              const void * const * b, int transposedB, int dataTypeB,
                              void * const * c, int dataTypeC,
                              int count, int na, int ma, int nb, int mb, int nc, int mc,
                              float alpha, float beta)
{
    Kind kind;
    Shape s;
    int st = check_types(dataTypeA, dataTypeB, dataTypeC, kind);
    if (st == NTSAMD_OK)
        st = check_shape(transposedA, transposedB, na, ma, nb, mb, nc, mc, s);
    if (st != NTSAMD_OK)
        return st;
    if (count < 0)
        return fail(NTSAMD_ERR_ARGUMENT, "negative batch count");
    if (count == 0 || s.M == 0 || s.N == 0)
        return NTSAMD_OK;
    if (!a || !b || !c)
        return fail(NTSAMD_ERR_ARGUMENT, "Empty input lists!");
    for (int i = 0; i < count; i++)
        if (!a[i] || !b[i] || !c[i])
            return fail(NTSAMD_ERR_ARGUMENT, "Empty matrices in multiplication!");

    PtrBatch tab;
    for (int first = 0; first < count; first += NTSAMD_PTR_BATCH_MAX) {
        int n = count - first < NTSAMD_PTR_BATCH_MAX ? count - first : NTSAMD_PTR_BATCH_MAX;
        for (int i = 0; i < n; i++) {
            tab.a[i] = a[first + i];
            tab.b[i] = b[first + i];
            tab.c[i] = c[first + i];
        }
        for (int i = n; i < NTSAMD_PTR_BATCH_MAX; i++) {
            tab.a[i] = NULL;
            tab.b[i] = NULL;
            tab.c[i] = NULL;
        }
        st = run(devID, stream, kind, s, NULL, NULL, NULL, ma, mb, mc, 0, 0, 0, n, &tab,
                 alpha, beta, NULL, NTSAMD_BIAS_NONE, 0, 1);
        if (st != NTSAMD_OK)
            return st;
    }
    return NTSAMD_OK;
}

}  /* extern "C" */
