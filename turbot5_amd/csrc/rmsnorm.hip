// T5 RMS norm (no mean subtraction, no bias) and the transient-global side-token producer
// (block sums followed by the same norm) as one HBM-bound kernel.
//
// One wavefront per output row, four rows per workgroup.  Rows of up to 4 x 64 sixteen-byte chunks stay
// in registers between the sum of squares and the scaling; longer rows are read twice (the second read
// hits cache).  Either way HBM sees one read and one write per element.  With a residual the kernel
// first forms x + residual (rounded to the input type, as torch's add leaves it), writes that sum out as
// the new residual stream and normalises it: the "add, then norm" pair between two T5 sub-layers
// (src/turbot5/model/modeling.py:159-161 followed by :113-114) as one pass.  Arithmetic follows the reference's eager path (src/turbot5/model/modules.py:51-59):
// variance and normalisation in fp32, the normalised value rounded to the weight's type when that
// is a 16-bit type, then multiplied by the weight in that type.  With group > 1 an output row is
// the norm of the SUM of `group` consecutive input rows (rounded to the input type first, as the
// reference's einsum leaves it, src/turbot5/model/utils.py:249-258); the rows left over at the end
// of a sequence join its last group (utils.py:206-212).
#include <hip/hip_runtime.h>

#include "t5a_internal.h"

namespace t5a {

template <typename T> struct Cvt;
template <> struct Cvt<float> {
    static __device__ __forceinline__ float up(float x) { return x; }
    static __device__ __forceinline__ float down(float x) { return x; }
};
template <> struct Cvt<__bf16> {
    static __device__ __forceinline__ float up(__bf16 x) { return (float)x; }
    static __device__ __forceinline__ __bf16 down(float x) { return (__bf16)x; }
};
template <> struct Cvt<_Float16> {
    static __device__ __forceinline__ float up(_Float16 x) { return (float)x; }
    static __device__ __forceinline__ _Float16 down(float x) { return (_Float16)x; }
};

template <typename T, int N> struct alignas(sizeof(T) * N) Vec { T v[N]; };

// TX input, TW weight, TY output (TY = TW for 16-bit weights, float otherwise).
// CH > 0: the row fits CH 16-byte chunks per lane and stays in registers between the sum of squares and
// the scaling (one read of the row); CH == 0: any length, the row is read twice (the second read hits cache).
template <typename TX, typename TW, typename TY, int CH>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const RmsParams p) {
    constexpr int VEC = 16 / sizeof(TX);   // elements per 16-byte load of the input
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= p.out_rows) return;
    const int64_t b = row / p.out_per_batch;
    const int g = (int)(row - b * p.out_per_batch);
    // With per-sequence lengths (and first rows) a sequence is the rows [start, end).  It has one group per group END
    // among its rows, group g taking its rows of [g * group, (g + 1) * group) and the last group every row from
    // there on (the reference's block ids for one run of tokens: min(row / group, groups - 1),
    // src/turbot5/model/utils.py:191-237); groups without a row and output rows past the groups are zero.
    // With validity bit sets (masks of any shape) the groups are counted by the caller and a group sums its valid rows.
    const unsigned* kbits = p.key_bits != nullptr ? p.key_bits + b * p.key_bits_stride : nullptr;
    const int start_b = (p.starts && !kbits) ? max(0, min(p.rows_per_batch, p.starts[b])) : 0;
    const int end_b = (p.lens && !kbits) ? min(p.rows_per_batch, start_b + max(0, p.lens[b])) : p.rows_per_batch;
    const int groups_b = kbits ? max(0, min(p.out_per_batch, p.group_counts[b]))
                               : (p.lens ? end_b / p.group - start_b / p.group : p.out_per_batch);
    const int first = max(start_b, g * p.group);
    const int count = (g == groups_b - 1 ? end_b : min((g + 1) * p.group, end_b)) - first;
    auto row_valid = [&](int r) {   // token first + r of this batch element (wavefront-uniform)
        const int tok = first + r;
        return ((kbits[kKeyBitsFront + (tok >> 5)] >> (tok & 31)) & 1u) != 0;
    };
    const TX* x = reinterpret_cast<const TX*>(p.x) + b * p.x_batch_stride + (int64_t)first * p.x_row_stride;
    const TX* res = p.residual ? reinterpret_cast<const TX*>(p.residual) + row * p.residual_row_stride : nullptr;
    TX* sum = res ? reinterpret_cast<TX*>(p.sum_out) + row * p.y_row_stride : nullptr;
    const TW* w = reinterpret_cast<const TW*>(p.weight);
    TY* y = reinterpret_cast<TY*>(p.y) + row * p.y_row_stride;
    const int nch = p.dim / VEC;
    if (g >= groups_b || count <= 0) {
        Vec<TY, VEC> zero;
#pragma unroll
        for (int i = 0; i < VEC; ++i) zero.v[i] = Cvt<TY>::down(0.f);
        for (int c = lane; c < nch; c += 64) *reinterpret_cast<Vec<TY, VEC>*>(y + c * VEC) = zero;
        return;
    }

    // chunk c of the row to normalise, as the input type holds it: the input row, or the sum of `count`
    // rows, or input + residual -- each sum rounded to the input type, as the torch expression leaves it
    auto load = [&](int c, float (&f)[VEC]) {
        if (kbits != nullptr) {   // the sum of the group's valid rows
#pragma unroll
            for (int i = 0; i < VEC; ++i) f[i] = 0.f;
            for (int r = 0; r < count; ++r) {
                if (!row_valid(r)) continue;
                const Vec<TX, VEC> u = *reinterpret_cast<const Vec<TX, VEC>*>(x + (int64_t)r * p.x_row_stride + c * VEC);
#pragma unroll
                for (int i = 0; i < VEC; ++i) f[i] += Cvt<TX>::up(u.v[i]);
            }
#pragma unroll
            for (int i = 0; i < VEC; ++i) f[i] = Cvt<TX>::up(Cvt<TX>::down(f[i]));
            return;
        }
        const Vec<TX, VEC> v = *reinterpret_cast<const Vec<TX, VEC>*>(x + c * VEC);
#pragma unroll
        for (int i = 0; i < VEC; ++i) f[i] = Cvt<TX>::up(v.v[i]);
        if (res != nullptr) {
            const Vec<TX, VEC> u = *reinterpret_cast<const Vec<TX, VEC>*>(res + c * VEC);
#pragma unroll
            for (int i = 0; i < VEC; ++i) f[i] = Cvt<TX>::up(Cvt<TX>::down(f[i] + Cvt<TX>::up(u.v[i])));
        }
        if (count > 1) {
            for (int r = 1; r < count; ++r) {
                const Vec<TX, VEC> u = *reinterpret_cast<const Vec<TX, VEC>*>(x + (int64_t)r * p.x_row_stride + c * VEC);
#pragma unroll
                for (int i = 0; i < VEC; ++i) f[i] += Cvt<TX>::up(u.v[i]);
            }
#pragma unroll
            for (int i = 0; i < VEC; ++i) f[i] = Cvt<TX>::up(Cvt<TX>::down(f[i]));
        }
    };
    auto store = [&](int c, const float (&f)[VEC], float rs) {
        if (res != nullptr) {   // the caller's new residual stream
            Vec<TX, VEC> s;
#pragma unroll
            for (int i = 0; i < VEC; ++i) s.v[i] = Cvt<TX>::down(f[i]);
            *reinterpret_cast<Vec<TX, VEC>*>(sum + c * VEC) = s;
        }
        Vec<TY, VEC> out;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const float n = f[i] * rs;
            const float wi = Cvt<TW>::up(w[c * VEC + i]);
            // 16-bit weights: the normalised value is rounded to the weight's type before the product
            out.v[i] = Cvt<TY>::down(sizeof(TW) == 2 ? Cvt<TW>::up(Cvt<TW>::down(n)) * wi : n * wi);
        }
        *reinterpret_cast<Vec<TY, VEC>*>(y + c * VEC) = out;
    };
    auto wave_rsqrt = [&](float ss) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
        return rsqrtf(ss / (float)p.dim + p.eps);
    };

    if constexpr (CH > 0) {
        float f[CH][VEC];
        float ss = 0.f;
#pragma unroll
        for (int k = 0; k < CH; ++k) {
            const int c = lane + 64 * k;
            if (c < nch) {
                load(c, f[k]);
#pragma unroll
                for (int i = 0; i < VEC; ++i) ss = fmaf(f[k][i], f[k][i], ss);
            }
        }
        const float rs = wave_rsqrt(ss);
#pragma unroll
        for (int k = 0; k < CH; ++k) {
            const int c = lane + 64 * k;
            if (c < nch) store(c, f[k], rs);
        }
    } else {
        float ss = 0.f;
        for (int c = lane; c < nch; c += 64) {
            float f[VEC];
            load(c, f);
#pragma unroll
            for (int i = 0; i < VEC; ++i) ss = fmaf(f[i], f[i], ss);
        }
        const float rs = wave_rsqrt(ss);
        for (int c = lane; c < nch; c += 64) {
            float f[VEC];
            load(c, f);
            store(c, f, rs);
        }
    }
}

template <typename TX, typename TW, typename TY>
static hipError_t launch_t(const RmsParams& p, hipStream_t s) {
    const unsigned grid = (unsigned)((p.out_rows + 3) / 4);
    const int per_lane = (p.dim / (16 / (int)sizeof(TX)) + 63) / 64;   // 16-byte chunks per lane
    if (per_lane <= 2) hipLaunchKernelGGL((rmsnorm_kernel<TX, TW, TY, 2>), dim3(grid), dim3(256), 0, s, p);
    else if (per_lane <= 4) hipLaunchKernelGGL((rmsnorm_kernel<TX, TW, TY, 4>), dim3(grid), dim3(256), 0, s, p);
    else hipLaunchKernelGGL((rmsnorm_kernel<TX, TW, TY, 0>), dim3(grid), dim3(256), 0, s, p);
    return hipGetLastError();
}

template <typename TX>
static hipError_t launch_w(const RmsParams& p, int w_dtype, hipStream_t s) {
    if (w_dtype == T5A_F32) return launch_t<TX, float, float>(p, s);
    if (w_dtype == T5A_BF16) return launch_t<TX, __bf16, __bf16>(p, s);
    if (w_dtype == T5A_F16) return launch_t<TX, _Float16, _Float16>(p, s);
    return hipErrorInvalidValue;
}

hipError_t launch_rmsnorm(const RmsParams& p, int x_dtype, int w_dtype, hipStream_t stream) {
    if (p.out_rows <= 0) return hipSuccess;
    if (x_dtype == T5A_F32) return launch_w<float>(p, w_dtype, stream);
    if (x_dtype == T5A_BF16) return launch_w<__bf16>(p, w_dtype, stream);
    if (x_dtype == T5A_F16) return launch_w<_Float16>(p, w_dtype, stream);
    return hipErrorInvalidValue;
}

}  // namespace t5a
