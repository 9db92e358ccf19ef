/*
 * C ABI of the gfx950 matrix-multiplication library (declared in
 * include/ntsamd_gemm.h): argument checking, device handling and the choice
 * of kernel. Takes the place of source/tensor/core/arithmetic/XTensorBLAS.cu
 * in the reference.
 */
#include "../../include/ntsamd_gemm.h"
#include "gemm_common.h"
#include "attention.h"

#include <atomic>
#include <map>
#include <mutex>
#include <utility>
#include <vector>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

namespace ntsamd {
int launch_f32_nn(const GemmParams &, const PtrBatch *, bool, int, hipStream_t);
int launch_f32_nt(const GemmParams &, const PtrBatch *, bool, int, hipStream_t);
int launch_f32_tn(const GemmParams &, const PtrBatch *, bool, int, hipStream_t);
int launch_f32_tt(const GemmParams &, const PtrBatch *, bool, int, hipStream_t);
int launch_f16_nn(const GemmParams &, const PtrBatch *, int, bool, int, hipStream_t);
int launch_f16_nt(const GemmParams &, const PtrBatch *, int, bool, int, hipStream_t);
int launch_f16_tn(const GemmParams &, const PtrBatch *, int, bool, int, hipStream_t);
int launch_f16_tt(const GemmParams &, const PtrBatch *, int, bool, int, hipStream_t);
int launch_scale(bool half, void * v, long long n, float beta, hipStream_t stream);
int launch_reduce_sum_xz(bool half, const void * in, int X, int Y, int Z, void * out, float beta, hipStream_t stream,
                         float * work, size_t workFloats);
int launch_convert(int kind, const void * s, void * t, long long n, hipStream_t stream);
int launch_repitch_f16(const void * s, long long srcPitch, void * t, int dstPitch, long long rows, int cols, hipStream_t stream);
int launch_row_bias(bool half, void * c, int M, int N, int ldc, const void * bias, int div, int len, int act, hipStream_t stream);
}

using namespace ntsamd;

namespace {

thread_local char g_error[512] = "";

/* What the last product issued from this thread was planned as (the kernel family, tile shape, pieces of k, how
   the operands are fetched, the passes around it): for the benchmark, which records it beside its timings so that
   a profile's kernel rows can be matched to what ran, and for the tests of the dispatcher. With g_planOnly set
   (ntsamd_plan_only, tests) a call stops there: nothing is looked up on a device, nothing allocated or launched,
   no pointer followed. */
thread_local char g_plan[512] = "";
thread_local bool g_planOnly = false;

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
std::atomic<int> g_deviceCUs[MAX_DEVICES];     /* compute units, known once the state is */

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
        g_deviceCUs[devID].store(prop.multiProcessorCount, std::memory_order_relaxed);
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
    explicit DeviceScope(int devID, bool planOnly = false) : backup(-1), switched(false), status(NTSAMD_OK)
    {
        if (planOnly)
            return;
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

/* KIND_A32_*: a half product whose a is stored as float and rounded to half on its way into the kernel's LDS */
enum Kind { KIND_F32, KIND_F16, KIND_F16_F32OUT, KIND_A32_F16, KIND_A32_F16_F32OUT };
inline bool kind_a32(Kind k) { return k == KIND_A32_F16 || k == KIND_A32_F16_F32OUT; }
inline bool kind_out_f32(Kind k) { return k == KIND_F16_F32OUT || k == KIND_A32_F16_F32OUT; }
inline bool kind_c_half(Kind k) { return k == KIND_F16 || k == KIND_A32_F16; }

int check_types(int ta, int tb, int tc, Kind & kind)
{
    if (ta == NTSAMD_X_FLOAT && tb == NTSAMD_X_FLOAT && tc == NTSAMD_X_FLOAT)
        kind = KIND_F32;
    else if (ta == NTSAMD_X_FLOAT16 && tb == NTSAMD_X_FLOAT16 && tc == NTSAMD_X_FLOAT16)
        kind = KIND_F16;
    else if (ta == NTSAMD_X_FLOAT16 && tb == NTSAMD_X_FLOAT16 && tc == NTSAMD_X_FLOAT)
        kind = KIND_F16_F32OUT;
    else if (ta == NTSAMD_X_FLOAT && tb == NTSAMD_X_FLOAT16 && tc == NTSAMD_X_FLOAT16)
        kind = KIND_A32_F16;
    else if (ta == NTSAMD_X_FLOAT && tb == NTSAMD_X_FLOAT16 && tc == NTSAMD_X_FLOAT)
        kind = KIND_A32_F16_F32OUT;
    else
        return fail(NTSAMD_ERR_DATATYPE, "Unsupported data type!");
    return NTSAMD_OK;
}

bool aligned16(const void * p)
{
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

/* Estimated run time of an fp32 product under a tile shape and a number of k pieces, in microseconds, fitted to
   graph-replayed measurements of both tile shapes with 1 to 8 pieces of k on two dozen products (512^3 to 4096 x 2048 x 512, 640 x 512 x 30011): the fp32 matrix pipe of a SIMD is kept busy
   by ONE wave, so what counts is how many workgroups the busiest CU runs one after the other (a second
   workgroup on a CU hides latencies but takes its own turn on the pipe): rounds = ceil(workgroups / 256). A
   workgroup's MFMAs take tile area x k x 3.48e-6 us on a 128 x 128 tile; the 64 x 64 tile (one accumulator
   block per wave: a dependent chain) runs at 0.89 of that rate alone on its CU and at 0.965 with company. What
   a workgroup spends before its first and after its last MFMA (4 us; 1.5 us for the small tile) is exposed
   once and partly hidden behind the other workgroups of the CU after that. Cutting k sends the fp32 partial
   products across memory once (about 5 TB/s, much of it behind the multiplications) on their way to a second
   launch that adds them up in a fixed order. The constants of the 16-row shape (0.55 of the rate, 1 us of ends) and of the
   cut (4.5 us) are those of a second fit, over 102 products from 64 x 512 x 512 to
   2048 x 2048 x 2048 with every shape and 1 to 16 pieces measured: the plan they choose is within 3.5 % of the best
   measured plan on every one of them (the first fit's: 24 % off on the worst, small products that it cut into
   pieces where the 16-row shape in one piece is faster). Without a workspace the pieces add to c with atomics
   instead (about 2.7 TB/s) and, unless beta is 1, a pass over c applies beta first: a launch (2.5 us) and c
   read and written. */
constexpr double SPLIT_FIXED_US = 2.3, SPLIT_FIXED_F32_US = 4.5, SPLIT_BYTES_PER_US = 5.0e6;

double tile_cost_f32(int M, int N, int K, int count, int bm, int bn, int splits, bool betaPass, bool viaWork)
{
    const bool big = bm >= 128;
    const long long groups = (long long)((M + bm - 1) / bm) * ((N + bn - 1) / bn) * count * splits;
    const long long rounds = (groups + 255) / 256;
    /* 16 rows per workgroup: every workgroup stages 128 columns of b for 16 rows of c, twice what the others move
       per MFMA (fitted: 0.55 of the rate) */
    const double rate = big ? 1.0 : (bm == 16 ? 0.55 : (rounds > 1 ? 0.965 : 0.89));
    /* the 32-row tile multiplies only 16 rows when there are no more (16-row MFMAs) */
    const double mfma = (double)(bm == 32 && M <= 16 ? 16 : bm) * bn * ((K + splits - 1) / splits) * 3.48e-6 / rate;
    const double ends = (big ? 4.0 : (bm == 16 ? 1.0 : 1.5)) * (1.0 + (double)(rounds - 1) * (big ? 0.5 : 0.25));
    const double cBytes = 4.0 * M * N * count;
    double cut = 0.0;
    if (splits > 1 && viaWork)
        cut = SPLIT_FIXED_F32_US + 2.0 * cBytes * splits / SPLIT_BYTES_PER_US;
    else if (splits > 1)
        cut = cBytes * splits / 2.7e6 + (betaPass ? 2.5 + cBytes * 2 / 2.7e6 : 0.0);
    return (double)rounds * mfma + ends + cut;
}

/* The same for fp16, fitted to graph-replayed measurements of each tile shape on 8 to 4096 workgroups with k from
   256 to 4096. Up to 256 workgroups every workgroup has a CU to itself and the time is one workgroup's chain of
   slabs, nearly whatever their number; beyond, what counts is how many the busiest CU runs (rounds), and the
   workgroups that share a CU hide each other's waits: per k and round 0.00368 us (64 x 64, against 0.0045 us
   alone), 0.0086 us (128 x 128, against 0.0078 to 0.0094 us alone), 0.0275 us (256 x 256, which always runs
   alone on its CU: four slabs to fetch before the first MFMA, 128 KB to store after the last, paid every round:
   7.2 us on eight waves, which is how it runs up to k = 2048, 3.4 us on four). Short k and many rounds favour
   the 128 x 128 tile, long k the big one. The clock under fp16 MFMA
   load depends on how much of the chip is busy, which is why the big tile is faster per k on a product that
   fills a fraction of the CUs.
   Cutting k into pieces (few tiles, long k: weight gradients, the few rows of a decoding step) makes as many
   products of a shorter k, whose fp32 results cross memory once (about 5 TB/s, much of it behind the
   multiplications) on their way to a second launch (2.3 us) that adds them up. */

double tile_cost_f16(int M, int N, int K, int count, int bm, int splits)
{
    if (splits > 1) {
        const int kPiece = ((K + splits - 1) / splits + 63) / 64 * 64;
        return tile_cost_f16(M, N, kPiece, count * splits, bm, 1) + SPLIT_FIXED_US +
               8.0 * M * N * count * splits / SPLIT_BYTES_PER_US;
    }
    const long long groups = (long long)((M + bm - 1) / bm) * ((N + bm - 1) / bm) * count;
    const long long rounds = (groups + 255) / 256;
    const bool alone = groups <= 256;
    if (bm >= 256) {
        /* the fewer CUs are busy, the higher the clock (down to 0.7 of the time) */
        const double busy = alone ? (groups < 180 ? 0.7 : (double)groups / 256.0) : 1.0;
        return K <= 2048 ? (double)rounds * (0.0275 * busy * K + 7.2) + 3.0        /* eight waves */
                         : (double)rounds * (0.02816 * busy * K + 3.4) + 4.0;      /* four */
    }
    if (bm >= 128) {
        if (alone) {
            const double full = groups <= 128 ? 0.0 : (double)(groups - 128) / 128.0;
            return (0.0078 + 0.0016 * full) * K + 4.5 + 0.6 * full;
        }
        return (double)rounds * 0.0086 * K + 4.3 + 1.4 * (double)(rounds - 1);
    }
    /* up to two workgroups to a CU run with slabs of 64 (see where f16Slab64 is set) */
    if (alone)
        return 0.0034 * K + (groups <= 128 ? 3.15 : 3.45);
    return (double)rounds * (rounds <= 2 ? 0.0026 : 0.00368) * K + 3.5 + 0.47 * (double)(rounds - 1);
}

struct Plan {
    int cfg;
    int splits;
};

/* Knobs for measurements and tests, none of them part of the documented interface: the environment is read ONCE,
   at the first call that looks (never again on the way to a launch), and ntsamd_tuning_set changes a knob in a
   running process. -1 = the library decides.
     NTSAMD_TILE_CFG=0|1|2|3|4   force a tile shape (128x128, 64x64, 256x256 for half, 32x128 and 16x128 for float)
     NTSAMD_SPLIT_K=n            force the number of pieces k is cut into (1 = never cut, and never a workspace)
     NTSAMD_F16_FETCH=0|2        keep half products off the main path (element-wise / register-staged fetch)
     NTSAMD_ATTN_ROWS=0          keep attention with a handful of query rows on the MFMA kernels
     NTSAMD_F32_R16=0            no 16-row MFMAs for float products of at most 16 rows
     NTSAMD_F32_SPLIT_ATOMIC=1   float pieces of k add to c with atomics (no workspace, no fixed order)
     NTSAMD_F16_PINGPONG=0       half, 256 x 256 tile: the main loop in which both waves of a SIMD meet one barrier
     NTSAMD_F16_PERSIST=0|2|3|4  half: never one workgroup per CU that walks over tiles / always over 256 x 256 tiles / never
                                 over 128 x 256 tiles / always over 128 x 256 tiles (where the kernel can take the product)
     NTSAMD_STORE_HINT=0|1       results never / always written through, whatever their alignment
     NTSAMD_GROUP_M=n            tile rows that share a sweep over the tile columns (8 if unset)
     NTSAMD_A32_CONVERT=0|1      float a with half b: never / whenever it fits the workspace, round a to half in a pass
                                 of its own before the product
     NTSAMD_F16_PERSIST_BETA=0   half products that read the old c keep to the one-tile kernels
     NTSAMD_F16_SLAB64=0|1       half, 64 x 64 tile on the 16-byte path: slabs of 32 / of 64 along k, however many
                                 workgroups share a CU
     NTSAMD_F16_REPITCH=0|1      half operands with rows that are no whole 16-byte pieces: never / whenever they fit the
                                 workspace, copied there with padded rows so that the product takes the 16-byte path */
struct Tuning {
    std::atomic<int> tileCfg, splitK, f16Fetch, attnRows, f32R16, f32SplitAtomic, f16PingPong, f16Persist, storeHint, groupM, a32Convert, f16Repitch, f16PersistBeta, f16Slab64;
};
Tuning g_tuning;
std::once_flag g_tuningOnce;

struct Knob {
    const char * name;
    std::atomic<int> Tuning::* field;
};
const Knob g_knobs[] = {
    {"NTSAMD_TILE_CFG", &Tuning::tileCfg},   {"NTSAMD_SPLIT_K", &Tuning::splitK},
    {"NTSAMD_F16_FETCH", &Tuning::f16Fetch}, {"NTSAMD_ATTN_ROWS", &Tuning::attnRows},
    {"NTSAMD_F32_R16", &Tuning::f32R16},     {"NTSAMD_F32_SPLIT_ATOMIC", &Tuning::f32SplitAtomic},
    {"NTSAMD_F16_PINGPONG", &Tuning::f16PingPong}, {"NTSAMD_F16_PERSIST", &Tuning::f16Persist},
    {"NTSAMD_STORE_HINT", &Tuning::storeHint}, {"NTSAMD_GROUP_M", &Tuning::groupM},
    {"NTSAMD_A32_CONVERT", &Tuning::a32Convert}, {"NTSAMD_F16_REPITCH", &Tuning::f16Repitch},
    {"NTSAMD_F16_PERSIST_BETA", &Tuning::f16PersistBeta}, {"NTSAMD_F16_SLAB64", &Tuning::f16Slab64},
};

const Tuning & tuning()
{
    std::call_once(g_tuningOnce, [] {
        for (const Knob & k : g_knobs) {
            const char * e = getenv(k.name);
            (g_tuning.*(k.field)).store(e && e[0] >= '0' && e[0] <= '9' ? atoi(e) : -1, std::memory_order_relaxed);
        }
    });
    return g_tuning;
}

/* Where the pieces of a product whose k is cut meet: one workspace per device and stream (launches on one
   stream run one after the other, so they can share; launches on different streams may overlap, so they must
   not), allocated at the first product that wants it and kept until ntsamd_release_workspaces or the end of the
   process. A call holds its workspace's mutex from before its first launch until after its last: two host
   threads that issue to one stream (every caller of the NULL stream does) cannot interleave their product and
   summing kernels. A kernel recorded into a graph keeps the workspace of the stream it was captured on: graphs
   captured on one stream, and that stream's own launches, must not run at the same time. */
constexpr size_t SPLIT_WORK_BYTES = (size_t)32 << 20;
constexpr int SPLIT_STREAMS_MAX = 64;               /* workspaces alive per process, over all devices */
struct SplitWork {
    float * mem;
    std::mutex inUse;
};
std::mutex g_splitMutex;                            /* guards the map, not the workspaces */
std::map<std::pair<int, hipStream_t>, SplitWork *> g_splitWork;   /* entries are never removed */
std::atomic<int> g_splitAlive;

/* The entry point that allocates nothing keeps its partial products here instead: part of the code object, so
   every device the library runs on holds its own copy from the moment the code is loaded there until the process
   ends. In host code the array's name is only a handle for hipGetSymbolAddress; the address on each device is
   looked up once, with that device current, and kept in g_scratch. */
constexpr size_t STATIC_SCRATCH_BYTES = (size_t)NTSAMD_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];
struct StaticScratch {
    std::atomic<float *> ptr;
    std::mutex inUse;
};
StaticScratch g_scratch[MAX_DEVICES];
std::mutex g_scratchMutex;

/* the static scratch of devID, which is current; NULL with the message set if the runtime cannot name it */
float * static_scratch(int devID)
{
    float * ptr = g_scratch[devID].ptr.load(std::memory_order_acquire);
    if (ptr != NULL)
        return ptr;
    std::lock_guard<std::mutex> lock(g_scratchMutex);
    ptr = g_scratch[devID].ptr.load(std::memory_order_acquire);
    if (ptr != NULL)
        return ptr;
    void * found = NULL;
    const hipError_t err = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
    if (err != hipSuccess || found == NULL) {
        (void)hipGetLastError();
        fail(NTSAMD_ERR_DEVICE, "cannot locate the static scratch on device %d: %s", devID, hipGetErrorString(err));
        return NULL;
    }
    g_scratch[devID].ptr.store(static_cast<float *>(found), std::memory_order_release);
    return static_cast<float *>(found);
}

/* A workspace held for the launches of one call; released when the call returns. */
struct WorkHold {
    float * mem;
    size_t bytes;
    std::mutex * held;
    WorkHold() : mem(NULL), bytes(0), held(NULL) {}
    ~WorkHold()
    {
        if (held)
            held->unlock();
    }
    /* the workspace of (devID, stream), allocated now if need be; mem stays NULL if there is none to be had (no
       memory, too many streams): the product then runs in one piece. Device devID is current. */
    void take_stream(int devID, hipStream_t stream)
    {
        if (mem != NULL)
            return;
        if (g_planOnly) {
            /* planning only: as if the workspace were there (never dereferenced) */
            mem = reinterpret_cast<float *>(static_cast<uintptr_t>(256));
            bytes = SPLIT_WORK_BYTES;
            return;
        }
        SplitWork * w;
        {
            std::lock_guard<std::mutex> lock(g_splitMutex);
            SplitWork *& slot = g_splitWork[std::make_pair(devID, stream)];
            if (slot == NULL) {
                slot = new SplitWork;
                slot->mem = NULL;
            }
            w = slot;
        }
        w->inUse.lock();
        /* a place among the SPLIT_STREAMS_MAX is taken before the allocation and given back if that fails, so that two
           threads cannot both pass the test on the last one */
        const bool place = w->mem == NULL && g_splitAlive.fetch_add(1) < SPLIT_STREAMS_MAX;
        if (w->mem == NULL && !place)
            g_splitAlive.fetch_sub(1);
        if (place) {
            /* the stream may be recording a graph: allocating is allowed then only in the relaxed mode, which is
               how allocators that serve captures do it; the allocation itself is no part of the graph */
            hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
            const bool exchanged = hipThreadExchangeStreamCaptureMode(&mode) == hipSuccess;
            void * got = NULL;
            const hipError_t err = hipMalloc(&got, SPLIT_WORK_BYTES);
            if (exchanged)
                (void)hipThreadExchangeStreamCaptureMode(&mode);
            if (err == hipSuccess && got != NULL)
                w->mem = static_cast<float *>(got);
            else {
                (void)hipGetLastError();
                g_splitAlive.fetch_sub(1);
            }
        }
        if (w->mem == NULL) {
            w->inUse.unlock();
            return;
        }
        mem = w->mem;
        bytes = SPLIT_WORK_BYTES;
        held = &w->inUse;
    }
    /* the static scratch of devID (current); false with the message set if it cannot be found */
    bool take_static(int devID)
    {
        if (g_planOnly) {
            mem = reinterpret_cast<float *>(static_cast<uintptr_t>(256));
            bytes = STATIC_SCRATCH_BYTES;
            return true;
        }
        float * ptr = static_scratch(devID);
        if (ptr == NULL)
            return false;
        g_scratch[devID].inUse.lock();
        mem = ptr;
        bytes = STATIC_SCRATCH_BYTES;
        held = &g_scratch[devID].inUse;
        return true;
    }
};

/* The tile shape and the number of k pieces with the lowest estimated run time. workBytes: what the partial
   products of a cut k may take (0: no limit, the float pieces add to c with atomics). forcedSplits >= 1: that many
   pieces or, where no shape can take them, one; otherwise the NTSAMD_SPLIT_K knob, otherwise the estimate. */
Plan choose_plan(int M, int N, int K, int count, bool half, bool maySplit, bool betaPass, size_t workBytes,
                 double cutExtra = 0.0, bool fast32 = false, int forcedSplits = -1)
{
    static const int bms[CFG_COUNT] = {128, 64, 256, 32, 16};
    static const int bns[CFG_COUNT] = {128, 64, 256, 128, 128};
    const Tuning & tn = tuning();
    int forcedCfg = tn.tileCfg.load(std::memory_order_relaxed);
    if (forcedCfg < 0 || forcedCfg >= CFG_COUNT)
        forcedCfg = -1;
    if (forcedCfg == CFG_256x256 && !half)
        forcedCfg = CFG_128x128;
    if ((forcedCfg == CFG_32x128 || forcedCfg == CFG_16x128) && half)
        forcedCfg = CFG_64x64;
    if (forcedSplits < 1)
        forcedSplits = tn.splitK.load(std::memory_order_relaxed);
    if (forcedSplits != 1 && forcedSplits != 2 && forcedSplits != 4 && forcedSplits != 8 && forcedSplits != 16)
        forcedSplits = -1;
    if (forcedSplits > 1 && (!maySplit || K / forcedSplits < 64))
        forcedSplits = 1;
    Plan best = {CFG_64x64, 1};
    double bestCost = -1.0;
    /* a forced number of pieces that no shape can take gives way: second turn */
    for (int turn = 0; turn < 2 && bestCost < 0.0; turn++) {
    if (turn == 1)
        forcedSplits = 1;
    for (int cfg = 0; cfg < CFG_COUNT; cfg++) {
        if ((cfg == CFG_256x256 && !half) || (cfg == CFG_32x128 && (half || M > 32)) ||
            (cfg == CFG_16x128 && (half || !fast32 || M <= 16)) || (forcedCfg >= 0 && cfg != forcedCfg))
            continue;
        for (int splits = 1; splits <= 16; splits *= 2) {
            if (splits > 1 && (!maySplit || K / splits < 64))
                break;
            /* the partial products must fit the workspace */
            if (splits > 1 && workBytes > 0 && (long long)M * N * count * splits * 4 > (long long)workBytes)
                break;
            /* half: the big tile has no such kernel */
            if (splits > 1 && half && (cfg == CFG_256x256 || K / splits < 128))
                break;
            if (forcedSplits >= 1 && splits != forcedSplits)
                continue;
            double c = half ? tile_cost_f16(M, N, K, count, bms[cfg], splits)
                            : tile_cost_f32(M, N, K, count, bms[cfg], bns[cfg], splits, betaPass, workBytes > 0);
            if (splits > 1)
                c += cutExtra;
            if (bestCost < 0.0 || c < bestCost) {
                bestCost = c;
                best.cfg = cfg;
                best.splits = splits;
            }
        }
    }
    }
    return best;
}

/* a batch laid out as a grid of `inner` x (count / inner) items: the second set of strides */
struct Grid {
    int inner;
    long long strideA1, strideB1, strideC1;
};

/* The entry point that allocates nothing: partial products go to the static scratch; splits = 0 lets the estimate
   choose among what fits there, 2, 4, 8 or 16 asks for that many pieces */
struct NoAlloc {
    int splits;
};

int run(int devID, void * stream, Kind kind, const Shape & s,
        const void * a, const void * b, void * c,
        int lda, int ldb, int ldc,
        long long strideA, long long strideB, long long strideC, int count,
        const PtrBatch * ptrs,
        float alpha, float beta,
        const void * bias, int biasMode, int biasLen, int biasRowDiv,
        void * colSum = NULL, float colSumBeta = 0.f, int act = ACT_NONE, const Grid * grid = NULL,
        const NoAlloc * noAlloc = NULL)
{
    if (count == 0 || s.M == 0 || s.N == 0)
        return NTSAMD_OK;

    const bool planOnly = g_planOnly;
    g_plan[0] = 0;
    if (!planOnly) {
        int st = check_device(devID);
        if (st != NTSAMD_OK)
            return st;
    }
    else if (devID < 0 || devID >= MAX_DEVICES)
        return fail(NTSAMD_ERR_DEVICE, "invalid device id %d", devID);
    DeviceScope scope(devID, planOnly);
    if (scope.status != NTSAMD_OK)
        return scope.status;
    char pre[160] = "";                 /* the passes that run before the product kernel, for the plan's text */
    auto note = [&pre](const char * what) {
        const size_t n = strlen(pre);
        snprintf(pre + n, sizeof(pre) - n, "%s%s", n ? "+" : "", what);
    };

    /* the kernels number their workgroups with 32-bit integers: the finest tiling of the largest batch,
       with k cut into the most pieces, must fit */
    if ((long long)((s.M + 15) / 16) * ((s.N + 63) / 64) * count * 16 > 0x7fffffffLL)
        return fail(NTSAMD_ERR_ARGUMENT, "the product has too many tiles for one launch (%d x %d x %d matrices)",
                    s.M, s.N, count);

    const Tuning & tn = tuning();
    hipStream_t hs = static_cast<hipStream_t>(stream);
    /* A bias along a dimension that is not the last (one value per row, or per group of rows) is added by a pass of
       its own behind the product, as the reference adds it (_SumDim with KernelAddWithCol behind the product,
       MulAndShift.cpp:69-88), and the activation with it: the product itself then runs on the fast kernels, which
       know a bias by column only. (Rows of 2^21 elements and more keep to the element-wise kernel, which adds either
       kind of bias itself.) */
    const void * rowBias = NULL;
    int rowBiasAct = ACT_NONE;
    if (bias != NULL && biasMode == NTSAMD_BIAS_ROW && !ptrs && !grid && count == 1 &&
        lda < (1 << 21) && ldb < (1 << 21) && ldc < (1 << 21)) {
        rowBias = bias;
        rowBiasAct = act;
        bias = NULL;
        biasMode = NTSAMD_BIAS_NONE;
        act = ACT_NONE;
    }
    WorkHold work;
    bool aInWork = false, repitched = false;
    if (kind_a32(kind) && !noAlloc && !ptrs && !grid && tn.a32Convert.load(std::memory_order_relaxed) != 0) {
        /* A float a is rounded to half on its way into LDS, through registers: that fetch is about half as fast again
           as the one that moves halves straight to LDS. A long product is better served by rounding a once, into
           the stream's workspace, and running the all-half product on that copy (same rounding, same bits): when
           the time the slower fetch would add exceeds one more launch and one pass over a. */
        const int rowsA = s.aKContig ? s.M : s.K, colsA = s.aKContig ? s.K : s.M;
        const long long span = (long long)(count - 1) * strideA + (long long)(rowsA - 1) * lda + colsA;
        const double slower = 0.5 * 2.0 * s.M * s.N * s.K * count / 7.0e14;
        const double pass = 2.5e-6 + (double)span * 6.0 / 5.0e12;
        const bool forced = tn.a32Convert.load(std::memory_order_relaxed) > 0;
        if (strideA >= 0 && span > 0 && (size_t)span * 2 <= SPLIT_WORK_BYTES && (forced || slower > pass)) {
            work.take_stream(devID, hs);
            if (work.mem != NULL) {
                const int rc = planOnly ? 0 : launch_convert(0, a, work.mem, span, hs);
                if (rc != 0)
                    return fail(NTSAMD_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString((hipError_t)rc));
                note("convert_kernel(a to half)");
                a = work.mem;
                kind = kind == KIND_A32_F16 ? KIND_F16 : KIND_F16_F32OUT;
                aInWork = true;
            }
        }
    }
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
    p.groupM = tn.groupM.load(std::memory_order_relaxed) > 0 ? tn.groupM.load(std::memory_order_relaxed) : 8;     /* the half walk over tiles takes 4 (see where it is chosen) */
    p.act = act;
    p.aF32 = kind_a32(kind) ? 1 : 0;
    p.wideRowsOnly = tn.f32R16.load(std::memory_order_relaxed) == 0;
    p.f16PingPong = tn.f16PingPong.load(std::memory_order_relaxed) != 0;
    {
        /* results whose rows are whole 128-byte lines are written through (see STORE_WRITE_THROUGH) */
        const long long unit = kind_c_half(kind) ? 2 : 4;
        const bool lines = (reinterpret_cast<uintptr_t>(c) & 127u) == 0 && !ptrs && (ldc * unit) % 128 == 0 &&
                           (strideC * unit) % 128 == 0 && (!grid || (grid->strideC1 * unit) % 128 == 0);
        const int knob = tn.storeHint.load(std::memory_order_relaxed);
        p.storeHint = knob >= 0 ? knob : (lines ? 1 : 0);
    }
    if (grid) {
        p.batchInner = grid->inner;
        p.strideA1 = grid->strideA1;
        p.strideB1 = grid->strideB1;
        p.strideC1 = grid->strideC1;
    }
    const int colsA = s.aKContig ? s.K : s.M, colsB = s.bKContig ? s.K : s.N;
    const bool dense = !grid && lda == colsA && ldb == colsB && ldc == s.N;

    /* the fast paths: 16-byte buffer loads of a and b, buffer stores of c, bias by column only. They keep a
       tile's byte offsets in 31 bits, so rows longer than 2M elements go through the generic path, like
       row-indexed bias. Float operands need no alignment beyond their own 4 bytes (a 16-byte buffer load may
       start on any dword, and is range-checked dword by dword). Half operands with 16-byte aligned rows of whole
       16-byte pieces travel straight to LDS (the main path); all other half operands, and lists of half
       matrices, are fetched 16 bytes at a time through registers, from any even address. */
    bool vec = lda < (1 << 21) && ldb < (1 << 21) && ldc < (1 << 21) && biasMode != NTSAMD_BIAS_ROW;
    p.mOper = colsA;
    p.nOper = colsB;
    /* b as the caller stored it: what a column-sum pass of its own reads, whatever copy the product is given */
    const void * const bStored = b;
    if ((kind == KIND_F16 || kind == KIND_F16_F32OUT) && vec && !ptrs && !grid && !noAlloc && !aInWork &&
        tn.f16Repitch.load(std::memory_order_relaxed) != 0) {
        /* A half operand whose rows are no whole 16-byte pieces (a 30011-word vocabulary) keeps the product off the
           kernels that move operands straight to LDS; fetched through registers it runs at about two thirds of
           their speed. Where the operand is small beside the product, a copy with padded rows (zeros in the
           padding) in the stream's workspace costs less than that: one launch and one pass over the operand. */
        const bool okA = lda % 8 == 0 && colsA % 8 == 0 && aligned16(a) && strideA % 8 == 0;
        const bool okB = ldb % 8 == 0 && colsB % 8 == 0 && aligned16(b) && strideB % 8 == 0;
        const int rowsA = s.aKContig ? s.M : s.K, rowsB = s.bKContig ? s.N : s.K;
        const int padA = (colsA + 7) / 8 * 8, padB = (colsB + 7) / 8 * 8;
        /* batches: items that follow each other without a gap (or one shared item) are copied as one run of rows */
        const bool runA = count == 1 || strideA == 0 || strideA == (long long)rowsA * lda;
        const bool runB = count == 1 || strideB == 0 || strideB == (long long)rowsB * ldb;
        const long long itemsA = count == 1 || strideA == 0 ? 1 : count, itemsB = count == 1 || strideB == 0 ? 1 : count;
        const long long elemsA = okA ? 0 : itemsA * rowsA * padA, elemsB = okB ? 0 : itemsB * rowsB * padB;
        const double slower = 0.4 * 2.0 * s.M * s.N * s.K * count / 7.0e14;
        const double pass = (okA ? 0.0 : 2.5e-6 + (double)elemsA * 4.0 / 3.0e12) + (okB ? 0.0 : 2.5e-6 + (double)elemsB * 4.0 / 3.0e12);
        const bool forced = tn.f16Repitch.load(std::memory_order_relaxed) > 0;
        if ((!okA || !okB) && (okA || runA) && (okB || runB) && (size_t)(elemsA + elemsB) * 2 <= SPLIT_WORK_BYTES &&
            (forced || slower > pass)) {
            work.take_stream(devID, hs);
            if (work.mem != NULL) {
                _Float16 * at = reinterpret_cast<_Float16 *>(work.mem);
                int rc = 0;
                if (!okA) {
                    rc = planOnly ? 0 : launch_repitch_f16(a, lda, at, padA, itemsA * rowsA, colsA, hs);
                    note("repitch_f16_kernel(a)");
                    p.a = a = at;
                    p.lda = lda = padA;
                    p.strideA = strideA = strideA == 0 ? 0 : (long long)rowsA * padA;
                    p.mOper = padA;
                }
                if (!okB && rc == 0) {
                    _Float16 * bt = at + elemsA;
                    rc = planOnly ? 0 : launch_repitch_f16(b, ldb, bt, padB, itemsB * rowsB, colsB, hs);
                    note("repitch_f16_kernel(b)");
                    p.b = b = bt;
                    p.ldb = ldb = padB;
                    p.strideB = strideB = strideB == 0 ? 0 : (long long)rowsB * padB;
                    p.nOper = padB;
                }
                if (rc != 0)
                    return fail(NTSAMD_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString((hipError_t)rc));
                aInWork = true;                 /* the workspace is taken: k is not cut into pieces */
                repitched = true;
            }
        }
    }
    int fetch16 = F16_SCALAR;
    if (kind != KIND_F32) {
        const bool direct = !kind_a32(kind) && vec && !ptrs && lda % 8 == 0 && ldb % 8 == 0 && (repitched || (colsA % 8 == 0 && colsB % 8 == 0)) &&
                            aligned16(a) && aligned16(b) && strideA % 8 == 0 && strideB % 8 == 0 &&
                            (!grid || (grid->strideA1 % 8 == 0 && grid->strideB1 % 8 == 0));
        fetch16 = direct ? F16_DIRECT : (vec ? F16_STAGED : F16_SCALAR);
        const int knob = tn.f16Fetch.load(std::memory_order_relaxed);   /* 0 or 2: keep off the main path */
        if (knob == F16_SCALAR || (knob == F16_STAGED && vec))
            fetch16 = knob;
        vec = fetch16 == F16_DIRECT;                               /* what the column-sum by-product needs */
    }
    const bool half = kind != KIND_F32;
    /* Cutting k into pieces pays when the result has few tiles and k is long (weight gradients, the few rows of a
       decoding step). The pieces of a product on the 16-byte path meet in a workspace and leave the ordinary way
       (any beta, bias, activation, leading dimensions; no column sums): the same bits on every run. Float pieces
       can add to c with atomics instead (in no fixed order; dense results without activation only, and c gets
       its beta first): only if the knob asks for it, or when there is no workspace to be had. */
    const bool atomicAble = !half && vec && !ptrs && act == ACT_NONE && dense;
    const bool atomicAsked = atomicAble && !noAlloc && tn.f32SplitAtomic.load(std::memory_order_relaxed) > 0;
    /* (the half copy of a float a has the workspace to itself) */
    const bool maySplit = !aInWork && (atomicAsked || ((half ? fetch16 == F16_DIRECT || fetch16 == F16_STAGED : vec) && !ptrs));
    const size_t workBytes = atomicAsked ? 0 : (noAlloc ? STATIC_SCRATCH_BYTES : SPLIT_WORK_BYTES);
    /* pieces that meet in a workspace gather no column sums: cutting costs a pass of its own over b then (a
       launch, b read once more) */
    const bool colSumAside = colSum != NULL && vec && count == 1 && !atomicAsked;
    const double cutExtra = colSumAside ? 2.3 + (half ? 2.0 : 4.0) * s.K * s.N / 4.0e6 : 0.0;
    const bool fast32 = kind == KIND_F32 && vec && !ptrs && colSum == NULL;
    int forcedSplits = -1;
    if (noAlloc && noAlloc->splits != 0) {
        forcedSplits = noAlloc->splits;
        if (forcedSplits != 2 && forcedSplits != 4 && forcedSplits != 8 && forcedSplits != 16)
            return fail(NTSAMD_ERR_ARGUMENT, "k can be cut into 2, 4, 8 or 16 pieces (or 0: the library chooses), not %d",
                        forcedSplits);
        if (!maySplit)
            return fail(NTSAMD_ERR_ARGUMENT, "this product cannot be cut along k (rows of 2097152 elements or more, or a "
                        "bias by row, keep it on the kernel that has no such form)");
        if (s.K / forcedSplits < (half ? 128 : 64))
            return fail(NTSAMD_ERR_ARGUMENT, "k = %d is too short for %d pieces (at least %d each)", s.K, forcedSplits,
                        half ? 128 : 64);
        if ((long long)s.M * s.N * count * forcedSplits * 4 > (long long)STATIC_SCRATCH_BYTES)
            return fail(NTSAMD_ERR_ARGUMENT, "%d partial products of %d x %d floats (%lld bytes) exceed the static "
                        "scratch of %lld bytes", forcedSplits, s.M, s.N, (long long)s.M * s.N * count * forcedSplits * 4,
                        (long long)STATIC_SCRATCH_BYTES);
    }
    Plan plan = choose_plan(s.M, s.N, s.K, count, half, maySplit, beta != 1.f, workBytes, cutExtra, fast32, forcedSplits);
    /* pieces that were asked for by number and that no tile shape can take (a forced tile shape without such a
       kernel) are an error, not a product in one piece */
    if (forcedSplits > 1 && plan.splits != forcedSplits)
        return fail(NTSAMD_ERR_ARGUMENT, "k cannot be cut into %d pieces under the tile shape in force (NTSAMD_TILE_CFG)",
                    forcedSplits);
    bool viaWork = false;
    if (plan.splits > 1 && !atomicAsked) {
        if (noAlloc) {
            if (!work.take_static(devID))
                return NTSAMD_ERR_DEVICE;
        }
        else
            work.take_stream(devID, hs);
        viaWork = work.mem != NULL;
        /* no workspace to be had (no memory, or too many streams hold one): the product runs in one piece, float
           and half alike, so that a result never depends on the order in which atomic adds arrive unless the
           NTSAMD_F32_SPLIT_ATOMIC knob asked for exactly that */
        if (!viaWork)
            plan = choose_plan(s.M, s.N, s.K, count, half, false, beta != 1.f, 0, 0.0, fast32);
    }
    const int cfg = plan.cfg;
    int rc = 0;
    /* More 256 x 256 tiles than CUs, a half result in whole 16-byte pieces and no old c to read on the way out (a
       bias by column rides along): one workgroup per CU walks over the tiles and fetches the next tile's first
       slabs before the finished tile's results leave */
#ifdef NTSAMD_PROBE
    const bool probeBias = true;        /* a profiling build: the bias pointer is where the time stamps go */
#else
    const bool probeBias = false;
#endif
    const bool biasFits = bias == NULL || probeBias || (biasMode == NTSAMD_BIAS_COL && aligned16(bias));
    int launchCfg = cfg;
    if (kind == KIND_F16 && fetch16 == F16_DIRECT && (beta == 0.f || (bias == NULL && tn.f16PersistBeta.load(std::memory_order_relaxed) != 0)) && biasFits && colSum == NULL && plan.splits == 1 &&
        s.K >= 256 && tn.f16Persist.load(std::memory_order_relaxed) != 0) {
        int cus = g_deviceCUs[devID].load(std::memory_order_relaxed);
        if (planOnly && cus <= 0)
            cus = 256;                  /* planning without a device: the part this library is written for */
        const long long tiles = (long long)((s.M + 255) / 256) * ((s.N + 255) / 256) * count;
        const long long tiles128 = (long long)((s.M + 127) / 128) * ((s.N + 255) / 256) * count;
        const bool wide = ldc % 8 == 0 && s.N % 8 == 0 && aligned16(c) && strideC % 8 == 0 &&
                          (!grid || grid->strideC1 % 8 == 0);
        const int knob = tn.f16Persist.load(std::memory_order_relaxed);
        /* from three tiles for four CUs on: with more CUs to spare the part is not held back by its power limit, and
           the older kernels' longer lead of the loads counts for more than the energy this one saves (measured, all
           four layouts: 192 tiles 28.1 -> 26.4 us at k = 1024 and 52.2 -> 46.7 us at k = 2048, 144 tiles 42.4 -> 43.5 us,
           128 tiles 140.8 -> 153.7 us at k = 8192) */
        if (cfg == CFG_256x256 && wide && cus > 0 && (tiles * 4 >= (long long)cus * 3 || knob == 2)) {
            p.persistGrid = cus;
            p.persistRows = 256;
        }
        /* fewer 256 x 256 tiles than CUs, but tiles of 128 x 256 give most CUs exactly one (more than one each for
           some would be a second round at a quarter of the part): the same kernel on tiles of half the height (a
           k-contiguous), whatever tile shape the estimate chose for the one-tile kernels. Measured at 256 such
           tiles: k = 4096 75 -> 66 us (b k x n) and 82 -> 67 us (b n x k), k = 2048 40 -> 36 and 43 -> 36, k = 1024
           21.7 -> 21.2 and 22.8 -> 21.2, k = 512 level or behind. */
        else if (s.aKContig && wide && cus > 0 &&
                 ((tiles < cus && tiles128 * 4 >= (long long)cus * 3 && tiles128 <= cus && s.K >= 1024 && knob != 3) || knob == 4)) {
            p.persistGrid = cus;
            p.persistRows = 128;
            launchCfg = CFG_256x256;
        }
        /* four tile rows share a sweep over the tile columns: the 32 tiles an XCD works on at a time are 4 x 8,
           the same twelve operand panels as 8 x 4, and their stores spread over twice as many columns of c
           (measured 1-2 % ahead of 8 at 8192 x 4096 x 1024, level elsewhere) */
        if (p.persistGrid > 0 && tn.groupM.load(std::memory_order_relaxed) <= 0)
            p.groupM = p.persistRows == 128 ? 8 : 4;
    }
    p.splits = 1;
    if (plan.splits > 1) {
        p.kPerSplit = ((s.K + plan.splits - 1) / plan.splits + 63) / 64 * 64;
        p.splits = (s.K + p.kPerSplit - 1) / p.kPerSplit;
        p.splitWork = viaWork ? work.mem : NULL;
    }
    {
        /* The small half tile on the LDS-direct path with slabs of 64 along k (whole 128-byte lines of a k-contiguous
           operand per load, twice the bytes on their way per workgroup) as long as a CU has at most two workgroups:
           its four stages take 68 KB of LDS, so two fit where four of the 32-deep kernel do. Measured, all layouts:
           1024 x 1024 x 4096 22.2 -> 17.1 us, 4096 x 512 x 2048 16.6 -> 14.5, 4096 x 512 x 512 6.8 -> 6.2,
           512 x 512 x 4096 in four pieces 11.8 -> 10.8; with four workgroups to a CU (8192 x 512 x 512 on this tile)
           10.3 -> 12.4. */
        const int knob = tn.f16Slab64.load(std::memory_order_relaxed);
        int cus = g_deviceCUs[devID].load(std::memory_order_relaxed);
        if (cus <= 0)
            cus = 256;
        const long long groups = (long long)((s.M + 63) / 64) * ((s.N + 63) / 64) * count * p.splits;
        p.f16Slab64 = knob >= 0 ? knob : (groups <= 2LL * cus ? 1 : 0);
    }
    if (p.splits > 1 && !viaWork && beta != 1.f) {
        /* float pieces that add to c: c is dense, count matrices of M x N, strideC apart */
        note("scale_kernel(c)");
        if (planOnly)
            rc = 0;
        else if (count == 1 || strideC == (long long)s.M * s.N)
            rc = launch_scale(false, c, (long long)s.M * s.N * count, beta, hs);
        else
            for (int i = 0; i < count && rc == 0; i++)
                rc = launch_scale(false, static_cast<float *>(c) + i * strideC, (long long)s.M * s.N, beta, hs);
        if (rc != 0)
            return fail(NTSAMD_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString((hipError_t)rc));
    }
    if (colSum != NULL) {
        /* (Float: the workgroups of the first tile row gather the sums from their b fragments and run about a fifth
           longer for it, 66.4 -> 77.9 us at 512 x 2048 over 4096 rows; a pass of its own over b before the product
           was measured against that: two launches more, 76.8 us, and b once more from memory. The by-product stays.) */
        if (vec && count == 1 && !(p.splits > 1 && viaWork)) {
            /* by-product of the product kernel */
            p.colSum = colSum;
            p.colSumBeta = colSumBeta;
            if (p.splits > 1) {
                note("scale_kernel(colSum)");
                rc = planOnly ? 0 : launch_scale(false, colSum, s.N, colSumBeta, hs);
            }
        }
        else {
            /* a pass of its own over b: rows of k for X_NOTRANS, rows of n for X_TRANS. It runs before the product
               on the same stream, so the two can share the workspace. It reads b as the caller stored it (dense
               rows), never the re-pitched copy the product may have been given. */
            if (!s.bKContig && !noAlloc && !repitched)
                work.take_stream(devID, hs);
            note(s.bKContig ? "outer_inner_sum_kernel(b)" : "column_sum_kernel(b)");
            float * const sumWork = repitched ? NULL : work.mem;
            const size_t sumFloats = repitched ? 0 : work.bytes / 4;
            if (planOnly)
                rc = 0;
            else
                rc = s.bKContig ? launch_reduce_sum_xz(half, bStored, 1, s.N, s.K, colSum, colSumBeta, hs, NULL, 0)
                                : launch_reduce_sum_xz(half, bStored, s.K, s.N, 1, colSum, colSumBeta, hs, sumWork, sumFloats);
        }
        if (rc != 0)
            return fail(NTSAMD_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString((hipError_t)rc));
    }

    {
        /* the plan in words: the kernel's family and what of its template follows from the plan */
        static const char * const tiles[CFG_COUNT] = {"128x128", "64x64", "256x256", "32x128", "16x128"};
        const char * family;
        const char * fetch;
        int tileCfg = cfg;
        if (kind == KIND_F32) {
            family = "gemm_f32_kernel";
            fetch = vec ? "vec16" : "elementwise";
            if (!vec || (ptrs && cfg != CFG_128x128) || (p.colSum != NULL && cfg != CFG_128x128))
                tileCfg = CFG_64x64;
        }
        else {
            tileCfg = launchCfg;
            const bool staged = kind_a32(kind) || fetch16 != F16_DIRECT || ptrs;
            fetch = kind_a32(kind) ? (fetch16 == F16_STAGED ? "staged16,a float" : "elementwise,a float")
                                   : (fetch16 == F16_DIRECT && !ptrs ? "lds-direct" : (fetch16 == F16_STAGED ? "staged16" : "elementwise"));
            if (staged)
                family = "gemm_f16_kernel";
            else if (launchCfg == CFG_256x256 && p.persistGrid > 0 && !kind_out_f32(kind))
                family = "gemm_f16_persistent_kernel";
            else
                family = "gemm_f16_direct_kernel";
            if (!staged && p.colSum != NULL && !kind_out_f32(kind) && tileCfg != CFG_64x64)
                tileCfg = CFG_128x128;
        }
        snprintf(g_plan, sizeof(g_plan), "%s%s%s tile=%s%s layout=%c%c fetch=%s splits=%d%s%s%s%s%s%s",
                 pre, pre[0] ? "+" : "", family,
                 family[9] == 'p' && p.persistRows == 128 ? "128x256" : tiles[tileCfg],
                 family[9] == 'p' ? ",walk" : (family[9] == 'd' && tileCfg == CFG_64x64 && p.f16Slab64 ? ",slab64" : ""),
                 s.aKContig ? 'N' : 'T', s.bKContig ? 'T' : 'N', fetch, p.splits,
                 p.splits > 1 ? (viaWork ? "+split_reduce_kernel" : ",atomic") : "",
                 p.colSum != NULL ? " colsum=in-kernel" : "",
                 rowBias != NULL ? "+row_bias_kernel" : (bias != NULL ? (biasMode == NTSAMD_BIAS_ROW ? " bias=row" : " bias=col") : ""),
                 beta != 0.f ? " beta" : "", act != ACT_NONE || rowBiasAct != ACT_NONE ? " act" : "",
                 ptrs ? " list" : (grid ? " grid" : (count > 1 ? " strided" : "")));
    }
    if (planOnly)
        return NTSAMD_OK;

    if (kind == KIND_F32) {
        if (s.aKContig)
            rc = s.bKContig ? launch_f32_nt(p, ptrs, vec, cfg, hs) : launch_f32_nn(p, ptrs, vec, cfg, hs);
        else
            rc = s.bKContig ? launch_f32_tt(p, ptrs, vec, cfg, hs) : launch_f32_tn(p, ptrs, vec, cfg, hs);
    }
    else {
        bool outF32 = kind_out_f32(kind);
        if (s.aKContig)
            rc = s.bKContig ? launch_f16_nt(p, ptrs, fetch16, outF32, launchCfg, hs) : launch_f16_nn(p, ptrs, fetch16, outF32, launchCfg, hs);
        else
            rc = s.bKContig ? launch_f16_tt(p, ptrs, fetch16, outF32, launchCfg, hs) : launch_f16_tn(p, ptrs, fetch16, outF32, launchCfg, hs);
    }
    if (rc == 0 && p.splits > 1 && viaWork)
        rc = launch_split_reduce(p, kind == KIND_F32 || kind_out_f32(kind), hs);
    if (rc == 0 && rowBias != NULL)
        rc = launch_row_bias(kind_c_half(kind), c, s.M, s.N, ldc, rowBias, biasRowDiv > 0 ? biasRowDiv : 1, biasLen > 0 ? biasLen : 1,
                             rowBiasAct, hs);
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
    (void)tuning();
    /* naming the static scratch makes the runtime load the code object on this device: here rather than at the
       first product, which may be issued where nothing may allocate */
    if (static_scratch(devID) == NULL)
        return NTSAMD_ERR_DEVICE;
    return NTSAMD_OK;
}

int ntsamd_release_workspaces(int devID)
{
    if (devID >= MAX_DEVICES)
        return fail(NTSAMD_ERR_DEVICE, "invalid device id %d", devID);
    std::vector<std::pair<int, SplitWork *> > mine;
    {
        std::lock_guard<std::mutex> lock(g_splitMutex);
        for (std::map<std::pair<int, hipStream_t>, SplitWork *>::iterator it = g_splitWork.begin();
             it != g_splitWork.end(); ++it)
            if (devID < 0 || it->first.first == devID)
                mine.push_back(std::make_pair(it->first.first, it->second));
    }
    for (size_t i = 0; i < mine.size(); i++) {
        SplitWork * w = mine[i].second;
        std::lock_guard<std::mutex> lock(w->inUse);
        if (w->mem == NULL)
            continue;
        DeviceScope scope(mine[i].first);
        if (scope.status != NTSAMD_OK)
            return scope.status;
        /* hipFree waits for the device's work, the kernels that still use the workspace included */
        const hipError_t err = hipFree(w->mem);
        if (err != hipSuccess)
            return fail(NTSAMD_ERR_DEVICE, "cannot free a workspace on device %d: %s", mine[i].first,
                        hipGetErrorString(err));
        w->mem = NULL;
        g_splitAlive.fetch_sub(1);
    }
    return NTSAMD_OK;
}

const char * ntsamd_last_plan(void)
{
    return g_plan;
}

void ntsamd_plan_only(int on)
{
    g_planOnly = on != 0;
}

int ntsamd_tuning_set(const char * name, int value)
{
    if (!name)
        return fail(NTSAMD_ERR_ARGUMENT, "no knob named");
    (void)tuning();                      /* the environment first, so that it cannot overwrite this later */
    for (const Knob & k : g_knobs)
        if (strcmp(name, k.name) == 0 || strcmp(name, k.name + 7) == 0) {
            (g_tuning.*(k.field)).store(value < 0 ? -1 : value, std::memory_order_relaxed);
            return NTSAMD_OK;
        }
    return fail(NTSAMD_ERR_ARGUMENT, "no knob named %s", name);
}

int ntsamd_matrix_mul_static(int devID, void * stream,
                             const void * a, int transposedA, int dataTypeA,
                             const void * b, int transposedB, int dataTypeB,
                             void * c, int dataTypeC,
                             int na, int ma, int nb, int mb, int nc, int mc,
                             float alpha, float beta, int splits)
{
    Kind kind;
    Shape s;
    int st = check_types(dataTypeA, dataTypeB, dataTypeC, kind);
    if (st == NTSAMD_OK)
        st = check_shape(transposedA, transposedB, na, ma, nb, mb, nc, mc, s);
    if (st != NTSAMD_OK)
        return st;
    if (splits < 0)
        return fail(NTSAMD_ERR_ARGUMENT, "negative number of pieces");
    if (s.M == 0 || s.N == 0)
        return NTSAMD_OK;
    st = check_pointers(a, b, c);
    if (st != NTSAMD_OK)
        return st;
    const NoAlloc na0 = {splits};
    return run(devID, stream, kind, s, a, b, c, ma, mb, mc, 0, 0, 0, 1, NULL, alpha, beta,
               NULL, NTSAMD_BIAS_NONE, 0, 1, NULL, 0.f, ACT_NONE, NULL, &na0);
}

int ntsamd_matrix_mul_bias(int devID, void * stream,
                           const void * a, int transposedA, int dataTypeA,
                           const void * b, int transposedB, int dataTypeB,
                           void * c, int dataTypeC,
                           int na, int ma, int nb, int mb, int nc, int mc,
                           float alpha, float beta,
                           const void * bias, int biasMode, int biasLen, int biasRowDiv)
{
    return ntsamd_matrix_mul_bias_act(devID, stream, a, transposedA, dataTypeA, b, transposedB, dataTypeB,
                                      c, dataTypeC, na, ma, nb, mb, nc, mc, alpha, beta,
                                      bias, biasMode, biasLen, biasRowDiv, NTSAMD_ACT_NONE);
}

int ntsamd_matrix_mul_bias_act(int devID, void * stream,
                               const void * a, int transposedA, int dataTypeA,
                               const void * b, int transposedB, int dataTypeB,
                               void * c, int dataTypeC,
                               int na, int ma, int nb, int mb, int nc, int mc,
                               float alpha, float beta,
                               const void * bias, int biasMode, int biasLen, int biasRowDiv, int activation)
{
    if (activation != NTSAMD_ACT_NONE && activation != NTSAMD_ACT_RECTIFY)
        return fail(NTSAMD_ERR_ARGUMENT, "unknown activation %d", activation);
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
               biasMode == NTSAMD_BIAS_NONE ? NULL : bias, biasMode, biasLen, biasRowDiv, NULL, 0.f, activation);
}

int ntsamd_matrix_mul_colsum(int devID, void * stream,
                             const void * a, int transposedA, int dataTypeA,
                             const void * b, int transposedB, int dataTypeB,
                             void * c, int dataTypeC,
                             int na, int ma, int nb, int mb, int nc, int mc,
                             float alpha, float beta,
                             void * colSum, float colSumBeta)
{
    Kind kind;
    Shape s;
    int st = check_types(dataTypeA, dataTypeB, dataTypeC, kind);
    if (st == NTSAMD_OK)
        st = check_shape(transposedA, transposedB, na, ma, nb, mb, nc, mc, s);
    if (st != NTSAMD_OK)
        return st;
    if (kind == KIND_F16_F32OUT || kind_a32(kind))
        return fail(NTSAMD_ERR_DATATYPE, "Unsupported data type!");   /* the sums have the type of b and of c */
    if (s.N == 0)
        return NTSAMD_OK;
    if (!colSum)
        return fail(NTSAMD_ERR_ARGUMENT, "column sums requested but empty");
    if (!b || (s.M > 0 && (!a || !c)))
        return fail(NTSAMD_ERR_ARGUMENT, "Empty matrices in multiplication!");
    if (s.M == 0) {
        /* no product to ride on: only the sums */
        st = check_device(devID);
        if (st != NTSAMD_OK)
            return st;
        DeviceScope scope(devID);
        if (scope.status != NTSAMD_OK)
            return scope.status;
        hipStream_t hs = static_cast<hipStream_t>(stream);
        WorkHold work;
        if (!s.bKContig && s.K >= 128)
            work.take_stream(devID, hs);
        int rc = s.bKContig ? launch_reduce_sum_xz(kind != KIND_F32, b, 1, s.N, s.K, colSum, colSumBeta, hs, NULL, 0)
                            : launch_reduce_sum_xz(kind != KIND_F32, b, s.K, s.N, 1, colSum, colSumBeta, hs,
                                                   work.mem, work.bytes / 4);
        if (rc != 0)
            return fail(NTSAMD_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString((hipError_t)rc));
        return NTSAMD_OK;
    }
    return run(devID, stream, kind, s, a, b, c, ma, mb, mc, 0, 0, 0, 1, NULL, alpha, beta,
               NULL, NTSAMD_BIAS_NONE, 0, 1, colSum, colSumBeta);
}

int ntsamd_reduce_sum_xz(int devID, void * stream, const void * in, int dataType,
                         int x, int y, int z, void * out, float beta)
{
    if (dataType != NTSAMD_X_FLOAT && dataType != NTSAMD_X_FLOAT16)
        return fail(NTSAMD_ERR_DATATYPE, "Unsupported data type!");
    if (x < 0 || y < 0 || z < 0)
        return fail(NTSAMD_ERR_ARGUMENT, "negative tensor size");
    if (y == 0)
        return NTSAMD_OK;
    if (!out || (!in && x > 0 && z > 0))
        return fail(NTSAMD_ERR_ARGUMENT, "Empty input or output tensors!");
    if ((long long)x * y * z > 0x7fffffffLL)
        return fail(NTSAMD_ERR_ARGUMENT, "tensor too large");
    int st = check_device(devID);
    if (st != NTSAMD_OK)
        return st;
    DeviceScope scope(devID);
    if (scope.status != NTSAMD_OK)
        return scope.status;
    /* column sums over many rows are cut into pieces of the rows, which meet in the stream's workspace as fp32 */
    WorkHold work;
    if (z == 1 && x >= 128)
        work.take_stream(devID, static_cast<hipStream_t>(stream));
    snprintf(g_plan, sizeof(g_plan), "%s", z > 1 ? "outer_inner_sum_kernel" : "column_sum_kernel");
    int rc = launch_reduce_sum_xz(dataType == NTSAMD_X_FLOAT16, in, x, y, z > 0 ? z : 1, out, beta,
                                  static_cast<hipStream_t>(stream), work.mem, work.bytes / 4);
    if (rc != 0)
        return fail(NTSAMD_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString((hipError_t)rc));
    return NTSAMD_OK;
}

int ntsamd_convert_data_type(int devID, void * stream, const void * s, int typeS, void * t, int typeT,
                             long long size)
{
    if (typeS == typeT)
        return NTSAMD_OK;
    int kind = -1;
    if (typeS == NTSAMD_X_FLOAT && typeT == NTSAMD_X_FLOAT16)
        kind = 0;
    else if (typeS == NTSAMD_X_FLOAT16 && typeT == NTSAMD_X_FLOAT)
        kind = 1;
    else if (typeS == NTSAMD_X_FLOAT && typeT == NTSAMD_X_INT)
        kind = 2;
    else if (typeS == NTSAMD_X_INT && typeT == NTSAMD_X_FLOAT)
        kind = 3;
    if (kind < 0)
        return fail(NTSAMD_ERR_DATATYPE, "Unsupported data types for conversion!");
    if (size < 0)
        return fail(NTSAMD_ERR_ARGUMENT, "negative tensor size");
    if (size == 0)
        return NTSAMD_OK;
    if (!s || !t)
        return fail(NTSAMD_ERR_ARGUMENT, "Empty input or output tensors!");
    const size_t unitS = kind == 1 ? 2 : 4, unitT = kind == 0 ? 2 : 4;
    if (reinterpret_cast<uintptr_t>(s) % unitS != 0 || reinterpret_cast<uintptr_t>(t) % unitT != 0)
        return fail(NTSAMD_ERR_ARGUMENT, "misaligned tensor data");
    int st = check_device(devID);
    if (st != NTSAMD_OK)
        return st;
    DeviceScope scope(devID);
    if (scope.status != NTSAMD_OK)
        return scope.status;
    snprintf(g_plan, sizeof(g_plan), "convert_kernel");
    int rc = launch_convert(kind, s, t, size, static_cast<hipStream_t>(stream));
    if (rc != 0)
        return fail(NTSAMD_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString((hipError_t)rc));
    return NTSAMD_OK;
}

int ntsamd_attention(int devID, void * stream,
                     const void * q, const void * k, const void * v, const void * mask, void * out, int dataType,
                     int heads, int batch, int lq, int lk, int dh,
                     const long long * strides, float scale)
{
    if (dataType != NTSAMD_X_FLOAT && dataType != NTSAMD_X_FLOAT16)
        return fail(NTSAMD_ERR_DATATYPE, "Unsupported data type!");
    if (heads < 0 || batch < 0 || lq < 0 || lk < 0 || dh < 0)
        return fail(NTSAMD_ERR_ARGUMENT, "negative tensor size");
    if (heads == 0 || batch == 0 || lq == 0 || dh == 0)
        return NTSAMD_OK;
    if (lk == 0)
        return fail(NTSAMD_ERR_ARGUMENT, "attention over no keys");
    if (!q || !k || !v || !out || !strides)
        return fail(NTSAMD_ERR_ARGUMENT, "Empty input tensors!");
    /* rows are moved 16 bytes at a time: 4 floats or 8 halves */
    const int vecElems = dataType == NTSAMD_X_FLOAT ? 4 : 8;
    if (dh > 128 || dh % vecElems != 0)
        return fail(NTSAMD_ERR_ARGUMENT, "head size %d is not served by the fused kernel (a multiple of %d up to 128 is)",
                    dh, vecElems);
    for (int i = 0; i < 12; i++)
        if (strides[i] < 0 || strides[i] % vecElems != 0)
            return fail(NTSAMD_ERR_ARGUMENT, "strides must be non-negative multiples of %d elements", vecElems);
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out))
        return fail(NTSAMD_ERR_ARGUMENT, "q, k, v and out must be 16-byte aligned");
    if (mask && (reinterpret_cast<uintptr_t>(mask) & 3) != 0)
        return fail(NTSAMD_ERR_ARGUMENT, "misaligned mask");
    for (int t = 0; t < 4; t++)
        if (strides[3 * t + 2] < dh)
            return fail(NTSAMD_ERR_ARGUMENT, "row stride smaller than the head size");
    if ((long long)heads * batch * ((lq + 63) / 64) > 0x7fffffffLL)
        return fail(NTSAMD_ERR_ARGUMENT, "tensor too large");
    /* the kernel addresses the rows of one head's k and v with 32-bit byte offsets, one block of keys ahead */
    for (int t = 1; t <= 2; t++)
        if (((long long)lk + 256) * strides[3 * t + 2] * 4 > 0x7fffffffLL)
            return fail(NTSAMD_ERR_ARGUMENT, "tensor too large: the keys of one head span more than 2 GiB");
    const bool planOnly = g_planOnly;
    if (!planOnly) {
        int st = check_device(devID);
        if (st != NTSAMD_OK)
            return st;
    }
    DeviceScope scope(devID, planOnly);
    if (scope.status != NTSAMD_OK)
        return scope.status;
    AttnParams p;
    memset(&p, 0, sizeof(p));
    p.q = q;
    p.k = k;
    p.v = v;
    p.mask = static_cast<const float *>(mask);
    p.out = out;
    p.heads = heads;
    p.batch = batch;
    p.lq = lq;
    p.lk = lk;
    p.dh = dh;
    p.qH = strides[0]; p.qB = strides[1]; p.qL = strides[2];
    p.kH = strides[3]; p.kB = strides[4]; p.kL = strides[5];
    p.vH = strides[6]; p.vB = strides[7]; p.vL = strides[8];
    p.oH = strides[9]; p.oB = strides[10]; p.oL = strides[11];
    p.scale = scale;
    /* up to eight query rows per head (a decoding step) go to the kernel that reads k and v once and multiplies
       in the vector ALU, as long as its scores fit in LDS; the NTSAMD_ATTN_ROWS=0 knob keeps them on the MFMA
       kernels */
    const bool halfType = dataType == NTSAMD_X_FLOAT16;
    const size_t rowsLds = attention_rows_lds(p, halfType);
    int rc;
    const bool fewRows = rowsLds > 0 && rowsLds <= 60 * 1024 && tuning().attnRows.load(std::memory_order_relaxed) != 0;
    snprintf(g_plan, sizeof(g_plan), "%s%s", fewRows ? "attention_rows_kernel" : (halfType ? "attention_f16_kernel" : "attention_f32_kernel"),
             mask ? " mask" : "");
    if (planOnly)
        return NTSAMD_OK;
    if (fewRows)
        rc = launch_attention_rows(p, halfType, static_cast<hipStream_t>(stream));
    else
        rc = halfType ? launch_attention_f16(p, static_cast<hipStream_t>(stream))
                      : launch_attention_f32(p, static_cast<hipStream_t>(stream));
    if (rc != 0)
        return fail(NTSAMD_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString((hipError_t)rc));
    return NTSAMD_OK;
}

int ntsamd_attention_probs(int devID, void * stream,
                           const void * q, const void * k, const void * mask, void * probs, int dataType,
                           int heads, int batch, int lq, int lk, int dh,
                           const long long * strides, float scale)
{
    if (dataType != NTSAMD_X_FLOAT)
        return fail(NTSAMD_ERR_DATATYPE, "Unsupported data type!");
    if (heads < 0 || batch < 0 || lq < 0 || lk < 0 || dh < 0)
        return fail(NTSAMD_ERR_ARGUMENT, "negative tensor size");
    if (heads == 0 || batch == 0 || lq == 0 || lk == 0)
        return NTSAMD_OK;
    if (!q || !k || !probs || !strides)
        return fail(NTSAMD_ERR_ARGUMENT, "Empty input tensors!");
    if (dh == 0 || dh > 128 || dh % 4 != 0)
        return fail(NTSAMD_ERR_ARGUMENT, "head size %d is not served by the fused kernel (a multiple of 4 up to 128 is)", dh);
    for (int i = 0; i < 6; i++)
        if (strides[i] < 0 || strides[i] % 4 != 0)
            return fail(NTSAMD_ERR_ARGUMENT, "strides must be non-negative multiples of 4 elements");
    if (!aligned16(q) || !aligned16(k))
        return fail(NTSAMD_ERR_ARGUMENT, "q and k must be 16-byte aligned");
    if ((mask && (reinterpret_cast<uintptr_t>(mask) & 3) != 0) || (reinterpret_cast<uintptr_t>(probs) & 3) != 0)
        return fail(NTSAMD_ERR_ARGUMENT, "misaligned mask or result");
    if (strides[2] < dh || strides[5] < dh)
        return fail(NTSAMD_ERR_ARGUMENT, "row stride smaller than the head size");
    if ((long long)heads * batch * ((lq + 63) / 64) > 0x7fffffffLL)
        return fail(NTSAMD_ERR_ARGUMENT, "tensor too large");
    if (((long long)lk + 256) * strides[5] * 4 > 0x7fffffffLL)
        return fail(NTSAMD_ERR_ARGUMENT, "tensor too large: the keys of one head span more than 2 GiB");
    const bool planOnly = g_planOnly;
    if (!planOnly) {
        int st = check_device(devID);
        if (st != NTSAMD_OK)
            return st;
    }
    DeviceScope scope(devID, planOnly);
    if (scope.status != NTSAMD_OK)
        return scope.status;
    AttnParams p;
    memset(&p, 0, sizeof(p));
    p.q = q;
    p.k = k;
    p.mask = static_cast<const float *>(mask);
    p.out = probs;
    p.heads = heads;
    p.batch = batch;
    p.lq = lq;
    p.lk = lk;
    p.dh = dh;
    p.qH = strides[0]; p.qB = strides[1]; p.qL = strides[2];
    p.kH = strides[3]; p.kB = strides[4]; p.kL = strides[5];
    p.scale = scale;
    snprintf(g_plan, sizeof(g_plan), "attention_probs_f32_kernel%s", mask ? " mask" : "");
    if (planOnly)
        return NTSAMD_OK;
    int rc = launch_attention_probs_f32(p, static_cast<hipStream_t>(stream));
    if (rc != 0)
        return fail(NTSAMD_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString((hipError_t)rc));
    return NTSAMD_OK;
}

int ntsamd_attention_train(int devID, void * stream,
                           const void * q, const void * k, const void * v, const void * mask, const void * dropMask,
                           void * probs, void * dropped, void * out, int dataType,
                           int heads, int batch, int lq, int lk, int dh,
                           const long long * strides, float scale)
{
    if (dataType != NTSAMD_X_FLOAT)
        return fail(NTSAMD_ERR_DATATYPE, "Unsupported data type!");
    if (heads < 0 || batch < 0 || lq < 0 || lk < 0 || dh < 0)
        return fail(NTSAMD_ERR_ARGUMENT, "negative tensor size");
    if (heads == 0 || batch == 0 || lq == 0)
        return NTSAMD_OK;
    if (lk == 0)
        return fail(NTSAMD_ERR_ARGUMENT, "attention over no keys");
    if (!q || !k || !v || !probs || !out || !strides)
        return fail(NTSAMD_ERR_ARGUMENT, "Empty input tensors!");
    if (dropped && !dropMask)
        return fail(NTSAMD_ERR_ARGUMENT, "dropped probabilities asked for without a dropout mask");
    if (dh == 0 || dh > 128 || dh % 4 != 0)
        return fail(NTSAMD_ERR_ARGUMENT, "head size %d is not served by the fused kernel (a multiple of 4 up to 128 is)", dh);
    for (int i = 0; i < 12; i++)
        if (strides[i] < 0 || strides[i] % 4 != 0)
            return fail(NTSAMD_ERR_ARGUMENT, "strides must be non-negative multiples of 4 elements");
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out))
        return fail(NTSAMD_ERR_ARGUMENT, "q, k, v and out must be 16-byte aligned");
    const void * four[4] = {mask, dropMask, probs, dropped};
    for (int i = 0; i < 4; i++)
        if (four[i] && (reinterpret_cast<uintptr_t>(four[i]) & 3) != 0)
            return fail(NTSAMD_ERR_ARGUMENT, "misaligned mask or probabilities");
    for (int t = 0; t < 4; t++)
        if (strides[3 * t + 2] < dh)
            return fail(NTSAMD_ERR_ARGUMENT, "row stride smaller than the head size");
    if ((long long)heads * batch * ((lq + 63) / 64) > 0x7fffffffLL)
        return fail(NTSAMD_ERR_ARGUMENT, "tensor too large");
    for (int t = 1; t <= 2; t++)
        if (((long long)lk + 256) * strides[3 * t + 2] * 4 > 0x7fffffffLL)
            return fail(NTSAMD_ERR_ARGUMENT, "tensor too large: the keys of one head span more than 2 GiB");
    const bool planOnly = g_planOnly;
    if (!planOnly) {
        int st = check_device(devID);
        if (st != NTSAMD_OK)
            return st;
    }
    DeviceScope scope(devID, planOnly);
    if (scope.status != NTSAMD_OK)
        return scope.status;
    AttnParams p;
    memset(&p, 0, sizeof(p));
    p.q = q;
    p.k = k;
    p.v = v;
    p.mask = static_cast<const float *>(mask);
    p.dropMask = static_cast<const float *>(dropMask);
    p.probs = static_cast<float *>(probs);
    p.dropped = static_cast<float *>(dropped);
    p.out = out;
    p.heads = heads;
    p.batch = batch;
    p.lq = lq;
    p.lk = lk;
    p.dh = dh;
    p.qH = strides[0]; p.qB = strides[1]; p.qL = strides[2];
    p.kH = strides[3]; p.kB = strides[4]; p.kL = strides[5];
    p.vH = strides[6]; p.vB = strides[7]; p.vL = strides[8];
    p.oH = strides[9]; p.oB = strides[10]; p.oL = strides[11];
    p.scale = scale;
    snprintf(g_plan, sizeof(g_plan), "attention_train_f32_kernel%s%s", mask ? " mask" : "", dropMask ? " dropout" : "");
    if (planOnly)
        return NTSAMD_OK;
    int rc = launch_attention_train_f32(p, static_cast<hipStream_t>(stream));
    if (rc != 0)
        return fail(NTSAMD_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString((hipError_t)rc));
    return NTSAMD_OK;
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

int ntsamd_matrix_mul_batched_grid(int devID, void * stream,
                                   const void * a, int transposedA, int dataTypeA, int lda,
                                   long long strideA0, long long strideA1,
                                   const void * b, int transposedB, int dataTypeB, int ldb,
                                   long long strideB0, long long strideB1,
                                   void * c, int dataTypeC, int ldc,
                                   long long strideC0, long long strideC1,
                                   int count0, int count1, int na, int ma, int nb, int mb, int nc, int mc,
                                   float alpha, float beta)
{
    Kind kind;
    Shape s;
    int st = check_types(dataTypeA, dataTypeB, dataTypeC, kind);
    if (st == NTSAMD_OK)
        st = check_shape(transposedA, transposedB, na, ma, nb, mb, nc, mc, s);
    if (st != NTSAMD_OK)
        return st;
    if (count0 < 0 || count1 < 0)
        return fail(NTSAMD_ERR_ARGUMENT, "negative batch count");
    if ((long long)count0 * count1 > 0x7fffffffLL)
        return fail(NTSAMD_ERR_ARGUMENT, "too many batch items");
    if (count0 == 0 || count1 == 0 || s.M == 0 || s.N == 0)
        return NTSAMD_OK;
    st = check_pointers(a, b, c);
    if (st != NTSAMD_OK)
        return st;
    if (lda < ma || ldb < mb || ldc < mc)
        return fail(NTSAMD_ERR_ARGUMENT, "leading dimension shorter than a row (lda %d for %d, ldb %d for %d, ldc %d for %d)",
                    lda, ma, ldb, mb, ldc, mc);
    if (strideA0 < 0 || strideA1 < 0 || strideB0 < 0 || strideB1 < 0 || strideC0 < 0 || strideC1 < 0)
        return fail(NTSAMD_ERR_ARGUMENT, "negative batch stride");
    /* results may interleave (heads side by side in one row of a merged tensor) but must not overlap:
       rows and the two axes of the grid, taken from the shortest stride up, must each step over
       everything the shorter ones span */
    {
        long long stride[3] = {ldc, strideC0, strideC1};
        long long count[3] = {nc, count0, count1};
        for (int i = 0; i < 3; i++)
            for (int j = i + 1; j < 3; j++)
                if (stride[j] < stride[i]) {
                    long long t = stride[i]; stride[i] = stride[j]; stride[j] = t;
                    t = count[i]; count[i] = count[j]; count[j] = t;
                }
        long long span = mc;
        for (int i = 0; i < 3; i++) {
            if (count[i] <= 1)
                continue;
            if (stride[i] < span)
                return fail(NTSAMD_ERR_ARGUMENT, "result matrices of the batch overlap");
            span += (count[i] - 1) * stride[i];
        }
    }
    Grid g = {count0, strideA1, strideB1, strideC1};
    return run(devID, stream, kind, s, a, b, c, lda, ldb, ldc, strideA0, strideB0, strideC0, count0 * count1, NULL,
               alpha, beta, NULL, NTSAMD_BIAS_NONE, 0, 1, NULL, 0.f, ACT_NONE, &g);
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
    if (kind_a32(kind))
        return fail(NTSAMD_ERR_DATATYPE, "Unsupported data type!");   /* lists of matrices: one type for a and b */
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
