// Builds the distance LUTs of all heads of one relative-attention table into a caller-provided buffer,
// (H, 4, qlen) floats: the image the attention kernel otherwise computes in LDS at the start of every
// work item.  The table is a model weight, so one build serves every launch until the table changes.
#include <hip/hip_runtime.h>

#include "lut_device.h"

namespace t5a {

namespace {

template <bool CAUSAL>
__global__ __launch_bounds__(256) void bias_lut_kernel(const FwdParams p, float* out, int window) {
    const int h = blockIdx.x, tid = threadIdx.x, lane = tid & 63;
    const int sat = window > p.bs.sat ? window : p.bs.sat;   // a folded-in window may widen the image
    const int padl = sat + LUT_PAD;
    const int qlen = 4 * lut_quads(sat, CAUSAL);
    const int nbt = p.bs.bidirectional ? 2 * p.bs.nb : p.bs.nb;
    const bool col_in_lanes = nbt <= 64;
    float tcol = 0.f;
    if (col_in_lanes && lane < nbt)
        tcol = load_table(p.table, p.table_dtype, (int64_t)lane * p.t_sbucket + (int64_t)h * p.t_shead) * 1.4426950408889634f;
    lut_fill<CAUSAL>(out + (size_t)h * (4 * qlen), p.bs, p.table, p.table_dtype, p.t_sbucket, p.t_shead, h, true, tcol,
                     col_in_lanes, padl, qlen, tid, 256, window > 0 ? window : 0x7fffffff);
}

}  // namespace

// 0: the attention kernel cannot fetch a LUT of this size (it takes at most two 16-byte pieces per thread)
int64_t bias_lut_bytes(int H, const BucketSpec& bs, bool causal, int window) {
    const int qlen = 4 * lut_quads(window > bs.sat ? window : bs.sat, causal);
    if (qlen > 512) return 0;
    return (int64_t)H * 4 * qlen * sizeof(float);
}

hipError_t launch_bias_lut(const FwdParams& p, bool causal, float* out, hipStream_t stream, int window) {
    if (causal) hipLaunchKernelGGL(bias_lut_kernel<true>, dim3(p.H), dim3(256), 0, stream, p, out, window);
    else hipLaunchKernelGGL(bias_lut_kernel<false>, dim3(p.H), dim3(256), 0, stream, p, out, window);
    return hipGetLastError();
}

}  // namespace t5a
