/* fp32 kernels for op(a),op(b) = nt (n: X_NOTRANS, t: X_TRANS); one file per pair so they build in parallel */
#include "gemm_f32.h"
namespace ntsamd {
int launch_f32_nt(const GemmParams & p, const PtrBatch * ptrs, bool vec, int cfg, hipStream_t stream)
{
    return launch_f32_trans<true, true>(p, ptrs, vec, cfg, stream);
}
}
