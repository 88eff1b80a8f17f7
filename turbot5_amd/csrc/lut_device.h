// The distance LUT of the T5 bias: layout, bucket arithmetic and the fill loop, shared by the attention
// kernel (which builds the LUT of its head in LDS) and the kernel that builds the LUTs of all heads once
// into a caller-provided buffer (lut.hip).
#pragma once
#include <hip/hip_runtime.h>

#include "t5a_internal.h"

namespace t5a {

// The distance LUT extends this far past the saturation distance on both sides.  A tile that takes
// the LUT path has at least one unsaturated (row, key) pair, and a wavefront tile spans 32 rows x
// 64 keys, so none of its distances lies more than 94 past saturation: lookups need no clamping.
constexpr int LUT_PAD = 96;

// floats per shifted copy of the distance LUT (host and device agree through this)
__host__ __device__ inline int lut_quads(int sat, bool causal) {
    const int entries = sat + LUT_PAD + (causal ? 0 : sat) + LUT_PAD + 1;   // rel = -sat-PAD .. (sat|0)+PAD
    const int quads = (entries + 3 + 3) / 4 + 1;                           // + 3 for the shifted copies
    // Four neighbouring lanes read the four copies at the same position: the copies start 16 floats apart
    // modulo the 64 LDS banks (quads = 4 mod 16), so the 16 lanes of a 16-byte read phase cover all banks.
    return quads + ((4 - quads) & 15);
}

__device__ __forceinline__ int bucket_of(const BucketSpec& s, int rel) {
    int out = 0, d;
    if (s.bidirectional) { out = rel > 0 ? s.nb : 0; d = rel < 0 ? -rel : rel; }
    else { d = rel < 0 ? -rel : 0; }
    if (d < s.max_exact) return out + d;
    // the first 16 thresholds come in with one scalar load and are compared without a loop
    // (unused slots hold INT_MAX); the loop only runs for unusually fine bucketings
    int b = s.max_exact;
#pragma unroll
    for (int t = 0; t < 16; ++t) b += (d >= s.thr[t]) ? 1 : 0;
    for (int t = 16; t < s.n_thr; ++t) b += (d >= s.thr[t]) ? 1 : 0;
    return out + b;
}

__device__ __forceinline__ float load_table(const void* table, int dtype, int64_t off) {
    if (dtype == T5A_F32) return reinterpret_cast<const float*>(table)[off];
    if (dtype == T5A_BF16) return static_cast<float>(reinterpret_cast<const __bf16*>(table)[off]);
    return static_cast<float>(reinterpret_cast<const _Float16*>(table)[off]);
}

// Fills the four shifted copies of one head's LUT: copy a, slot i holds the bias of distance i + a - padl,
// already multiplied by log2(e); future keys hold -inf when CAUSAL, distances of `window` and more hold -inf.  `tcol`: when col_in_lanes, lane b of
// every wavefront holds the table value of bucket b (times log2 e).  Every thread of the workgroup must call.
template <bool CAUSAL>
__device__ __forceinline__ void lut_fill(float* lut, const BucketSpec& bs, const void* table, int table_dtype,
                                         int64_t t_sbucket, int64_t t_shead, int h, bool has_bias, float tcol,
                                         bool col_in_lanes, int padl, int qlen, int tid, int nthreads,
                                         int window = 0x7fffffff) {
    const float log2e = 1.4426950408889634f;
    // one evaluation per distance; the value goes to all four shifted copies
    for (int e0 = 0; e0 < qlen + 3; e0 += nthreads) {   // uniform trip count: the permute needs every lane
        const int e = e0 + tid;
        const int rel = e - padl;
        float val = 0.f;
        if (has_bias) {
            const int bk = bucket_of(bs, rel);
            if (col_in_lanes)
                val = __int_as_float(__builtin_amdgcn_ds_bpermute(bk << 2, __float_as_int(tcol)));
            else
                val = load_table(table, table_dtype, (int64_t)bk * t_sbucket + (int64_t)h * t_shead) * log2e;
        }
        if (CAUSAL && rel > 0) val = -INFINITY;
        if (rel >= window || rel <= -window) val = -INFINITY;   // outside a sliding window folded into the LUT
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int i = e - a;
            if (i >= 0 && i < qlen && e < qlen + 3) lut[a * qlen + i] = val;
        }
    }
}

}  // namespace t5a
