// T5 RMS norm (no mean subtraction, no bias) and the transient-global side-token producer
// (block sums followed by the same norm) as one HBM-bound kernel.
//
// One wavefront per output row, four rows per workgroup.  A row is read twice (sum of squares,
// then scale and store); the second read hits cache, so HBM sees one read and one write per
// element.  Arithmetic follows the reference's eager path (src/turbot5/model/modules.py:51-59):
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

// TX input, TW weight, TY output (TY = TW for 16-bit weights, float otherwise)
template <typename TX, typename TW, typename TY>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const RmsParams p) {
    constexpr int VEC = 16 / sizeof(TX);   // elements per 16-byte load of the input
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= p.out_rows) return;
    const int64_t b = row / p.out_per_batch;
    const int g = (int)(row - b * p.out_per_batch);
    const int first = g * p.group;
    const int count = g == p.out_per_batch - 1 ? p.rows_per_batch - first : p.group;
    const TX* x = reinterpret_cast<const TX*>(p.x) + b * p.x_batch_stride + (int64_t)first * p.x_row_stride;
    const TW* w = reinterpret_cast<const TW*>(p.weight);
    TY* y = reinterpret_cast<TY*>(p.y) + row * p.y_row_stride;
    const int nch = p.dim / VEC;

    auto load = [&](int c, float (&f)[VEC]) {   // chunk c of the (summed) input row, as the input type holds it
        const Vec<TX, VEC> v = *reinterpret_cast<const Vec<TX, VEC>*>(x + c * VEC);
#pragma unroll
        for (int i = 0; i < VEC; ++i) f[i] = Cvt<TX>::up(v.v[i]);
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

    float ss = 0.f;
    for (int c = lane; c < nch; c += 64) {
        float f[VEC];
        load(c, f);
#pragma unroll
        for (int i = 0; i < VEC; ++i) ss = fmaf(f[i], f[i], ss);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
    const float rs = rsqrtf(ss / (float)p.dim + p.eps);

    for (int c = lane; c < nch; c += 64) {
        float f[VEC];
        load(c, f);
        Vec<TY, VEC> out;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const float n = f[i] * rs;
            const float wi = Cvt<TW>::up(w[c * VEC + i]);
            // 16-bit weights: the normalised value is rounded to the weight's type before the product
            out.v[i] = Cvt<TY>::down(sizeof(TW) == 2 ? Cvt<TW>::up(Cvt<TW>::down(n)) * wi : n * wi);
        }
        *reinterpret_cast<Vec<TY, VEC>*>(y + c * VEC) = out;
    }
}

template <typename TX, typename TW, typename TY>
static hipError_t launch_t(const RmsParams& p, hipStream_t s) {
    const unsigned grid = (unsigned)((p.out_rows + 3) / 4);
    hipLaunchKernelGGL((rmsnorm_kernel<TX, TW, TY>), dim3(grid), dim3(256), 0, s, p);
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
