/* fp16 kernels for op(a),op(b) = nt (n: X_NOTRANS, t: X_TRANS); one file per pair so they build in parallel */
#include "gemm_f16_persist.h"
namespace ntsamd {
int launch_f16_nt(const GemmParams & p, const PtrBatch * ptrs, int vec, bool outF32, int cfg, hipStream_t stream)
{
    return launch_f16_trans<true, true>(p, ptrs, vec, outF32, cfg, stream);
}
}
