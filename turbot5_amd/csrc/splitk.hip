// Flash-decoding split-K forward for gfx950: few query rows against a long
// K/V memory.  The work is bandwidth bound (every K and V element is used once
// per query row), so it runs on the vector ALUs with 16-byte loads:
//
//   kernel 1  grid (split, head, batch x query-block): the workgroup's 256
//             threads are arranged as key slots x lanes-per-key; each slot walks
//             its keys with a private online softmax, then the slots are merged
//             through LDS into one (partial output, sum, max) per split.
//   kernel 2  merges the splits:  o = sum_s w_s o_s,  w_s = l_s e^{m_s - m} / sum.
#include "t5a_internal.h"

namespace t5a {

constexpr int SK_THREADS = 256;
constexpr float kSkNegBig = -1.0e30f;

template <typename T> struct SkLoad;
template <> struct SkLoad<__bf16> {
    static constexpr int EPL = 8;
    static __device__ __forceinline__ void load(const __bf16* p, float* out) {
        const uint4 r = *reinterpret_cast<const uint4*>(p);
        const unsigned w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            out[2 * i] = __uint_as_float(w[i] << 16);
            out[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ void widen(const unsigned __attribute__((ext_vector_type(4))) r, float* out) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            out[2 * i] = __uint_as_float(r[i] << 16);
            out[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ __bf16 cvt(float x) { return static_cast<__bf16>(x); }
};
template <> struct SkLoad<_Float16> {
    static constexpr int EPL = 8;
    static __device__ __forceinline__ void load(const _Float16* p, float* out) {
        typedef _Float16 h8 __attribute__((ext_vector_type(8)));
        const h8 r = *reinterpret_cast<const h8*>(p);
#pragma unroll
        for (int i = 0; i < 8; ++i) out[i] = static_cast<float>(r[i]);
    }
    static __device__ __forceinline__ void widen(const unsigned __attribute__((ext_vector_type(4))) r, float* out) {
        typedef _Float16 h8 __attribute__((ext_vector_type(8)));
        const h8 h = __builtin_bit_cast(h8, r);
#pragma unroll
        for (int i = 0; i < 8; ++i) out[i] = static_cast<float>(h[i]);
    }
    static __device__ __forceinline__ _Float16 cvt(float x) { return static_cast<_Float16>(x); }
};
template <> struct SkLoad<float> {
    static constexpr int EPL = 4;
    static __device__ __forceinline__ void load(const float* p, float* out) {
        const float4 r = *reinterpret_cast<const float4*>(p);
        out[0] = r.x; out[1] = r.y; out[2] = r.z; out[3] = r.w;
    }
    static __device__ __forceinline__ void widen(const unsigned __attribute__((ext_vector_type(4))) r, float* out) {
#pragma unroll
        for (int i = 0; i < 4; ++i) out[i] = __uint_as_float(r[i]);
    }
    static __device__ __forceinline__ float cvt(float x) { return x; }
};

template <typename T, int D, int MB>
__global__ __launch_bounds__(SK_THREADS) void splitk_partial_kernel(const SplitKParams p) {
    using L = SkLoad<T>;
    constexpr int EPL = L::EPL;            // elements per lane (16 bytes)
    constexpr int LPK = D / EPL;           // lanes per key row
    constexpr int KPP = SK_THREADS / LPK;  // key slots per pass
    constexpr int UNROLL = 4;

    __shared__ float sm_m[MB][KPP];
    __shared__ float sm_l[MB][KPP];
    __shared__ float sm_acc[MB][KPP][D + 1];

    const int s = blockIdx.x, h = blockIdx.y;
    const int mblocks = (p.M + MB - 1) / MB;
    const int b = blockIdx.z / mblocks;
    const int m0 = (blockIdx.z - b * mblocks) * MB;
    const int per = p.N / p.S;
    int lo = s * per;
    int hi = (s == p.S - 1) ? p.N : lo + per;
    if (p.key_lens != nullptr) {   // a padded memory: the split keeps what it holds of the valid keys (maybe nothing)
        const int first = p.key_starts != nullptr ? p.key_starts[b] : 0;
        lo = max(lo, first);
        hi = min(hi, first + p.key_lens[b]);
    }
    const int tid = threadIdx.x;
    const int c = tid % LPK, slot = tid / LPK;

    const T* qp = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.q_sb + (int64_t)h * p.q_sh;
    const T* kp = reinterpret_cast<const T*>(p.k) + (int64_t)b * p.k_sb + (int64_t)h * p.k_sh + c * EPL;
    const T* vp = reinterpret_cast<const T*>(p.v) + (int64_t)b * p.v_sb + (int64_t)h * p.v_sh + c * EPL;
    const float* bp = p.bias ? p.bias + (int64_t)b * p.b_sb + (int64_t)h * p.b_sh : nullptr;

    float qf[MB][EPL];
    float mrun[MB], lrun[MB], acc[MB][EPL];
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        if (m0 + m < p.M) {
            L::load(qp + (int64_t)(m0 + m) * p.q_sr + c * EPL, qf[m]);
#pragma unroll
            for (int x = 0; x < EPL; ++x) qf[m][x] *= p.sm_scale;
        } else {
#pragma unroll
            for (int x = 0; x < EPL; ++x) qf[m][x] = 0.f;
        }
        mrun[m] = kSkNegBig; lrun[m] = 0.f;
#pragma unroll
        for (int x = 0; x < EPL; ++x) acc[m][x] = 0.f;
    }

    // The loads of the next group of keys are in flight while the current group is reduced: the raw
    // 16-byte words wait in registers and are widened to fp32 only when consumed.
    typedef unsigned raw4 __attribute__((ext_vector_type(4)));
    raw4 kraw[UNROLL], vraw[UNROLL];
    auto fetch = [&](int j0) {
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int j = j0 + u * KPP;
            if (j < hi) {
                kraw[u] = *reinterpret_cast<const raw4*>(kp + (int64_t)j * p.k_sr);
                vraw[u] = *reinterpret_cast<const raw4*>(vp + (int64_t)j * p.v_sr);
            }
        }
    };
    if (lo + slot < hi) fetch(lo + slot);
    for (int j0 = lo + slot; j0 < hi; j0 += KPP * UNROLL) {
        float kf[UNROLL][EPL], vf[UNROLL][EPL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            if (j0 + u * KPP < hi) {
                L::widen(kraw[u], kf[u]);
                L::widen(vraw[u], vf[u]);
            }
        }
        if (j0 + KPP * UNROLL < hi) fetch(j0 + KPP * UNROLL);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int j = j0 + u * KPP;
            if (j < hi) {
#pragma unroll
                for (int m = 0; m < MB; ++m) {
                    float dot = 0.f;
#pragma unroll
                    for (int x = 0; x < EPL; ++x) dot = fmaf(qf[m][x], kf[u][x], dot);
#pragma unroll
                    for (int o = LPK / 2; o > 0; o >>= 1) dot += __shfl_xor(dot, o);
                    if (bp != nullptr && m0 + m < p.M) dot += bp[(int64_t)(m0 + m) * p.b_sr + (int64_t)j * p.b_sc];
                    const float mn = fmaxf(mrun[m], dot);
                    const float a = __expf(mrun[m] - mn);
                    const float e = __expf(dot - mn);
                    lrun[m] = lrun[m] * a + e;
#pragma unroll
                    for (int x = 0; x < EPL; ++x) acc[m][x] = fmaf(acc[m][x], a, e * vf[u][x]);
                    mrun[m] = mn;
                }
            }
        }
    }

    // merge the key slots of this workgroup
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        if (c == 0) { sm_m[m][slot] = mrun[m]; sm_l[m][slot] = lrun[m]; }
#pragma unroll
        for (int x = 0; x < EPL; ++x) sm_acc[m][slot][c * EPL + x] = acc[m][x];
    }
    __syncthreads();
    for (int idx = tid; idx < MB * D; idx += SK_THREADS) {
        const int m = idx / D, d = idx - m * D;
        if (m0 + m >= p.M) continue;
        float gm = kSkNegBig;
        for (int k = 0; k < KPP; ++k) gm = fmaxf(gm, sm_m[m][k]);
        float lt = 0.f, val = 0.f;
        for (int k = 0; k < KPP; ++k) {
            const float wgt = __expf(sm_m[m][k] - gm);
            lt = fmaf(sm_l[m][k], wgt, lt);
            val = fmaf(sm_acc[m][k][d], wgt, val);
        }
        const int64_t row = (((int64_t)b * p.H + h) * p.S + s) * p.M + (m0 + m);
        p.part_o[row * D + d] = lt > 0.f ? val / lt : 0.f;
        if (d == 0) {
            p.part_l[row] = lt;
            p.part_m[row] = lt > 0.f ? gm : -INFINITY;
        }
    }
}

// Merge over splits, one wavefront per output row.  The splits' log-sum-exps and weights are read with one
// lane per split (not one after the other), the weights go through LDS, and the weighted sum over the splits
// runs eight splits at a time so that their loads are in flight together: with 40 and more splits the serial
// version spent its time waiting for one load after the other.
template <typename T, int D>
__global__ __launch_bounds__(64) void splitk_merge_kernel(const SplitKParams p) {
    constexpr int MAXS = 256;            // weights kept in LDS; more splits fall back to recomputing them
    __shared__ float s_w[MAXS];
    const int m = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int lane = threadIdx.x;
    const int64_t base = (((int64_t)b * p.H + h) * p.S) * p.M + m;   // + s * M
    // The kernel is a chain of dependent loads for a few KB of data, so what it costs is round trips to memory:
    // a lane's first split is read once (maximum and sum of exponentials together) and kept, and the partial rows
    // are fetched eight splits at a time.
    float m_own = -INFINITY, l_own = 0.f;
    if (lane < p.S) {
        m_own = p.part_m[base + (int64_t)lane * p.M];
        l_own = p.part_l[base + (int64_t)lane * p.M];
    }
    float gm = m_own;
    for (int s = lane + 64; s < p.S; s += 64) gm = fmaxf(gm, p.part_m[base + (int64_t)s * p.M]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) gm = fmaxf(gm, __shfl_xor(gm, o, 64));
    auto weight = [&](int s) {
        const int64_t row = base + (int64_t)s * p.M;
        const float l = p.part_l[row];
        return l > 0.f ? l * __expf(p.part_m[row] - gm) : 0.f;
    };
    float wsum = 0.f;
    for (int s = lane; s < p.S; s += 64) {
        const float w = s == lane ? (l_own > 0.f ? l_own * __expf(m_own - gm) : 0.f) : weight(s);
        if (s < MAXS) s_w[s] = w;
        wsum += w;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) wsum += __shfl_xor(wsum, o, 64);
    __syncthreads();
    T* op = reinterpret_cast<T*>(p.o) + (int64_t)b * p.o_sb + (int64_t)h * p.o_sh + (int64_t)m * p.o_sr;
    const int cached = p.S < MAXS ? p.S : MAXS;
    for (int d = lane; d < D; d += 64) {
        float val = 0.f;
        int s = 0;
        for (; s < cached; s += 8) {   // (MAXS is a multiple of 8)
            float x[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) x[i] = s + i < cached ? p.part_o[(base + (int64_t)(s + i) * p.M) * D + d] : 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i)   // an empty split's row may hold anything
                if (s + i < cached) val = s_w[s + i] > 0.f ? fmaf(x[i], s_w[s + i], val) : val;
        }
        for (s = cached; s < p.S; ++s) {
            const float w = weight(s);
            if (w > 0.f) val = fmaf(p.part_o[(base + (int64_t)s * p.M) * D + d], w, val);
        }
        op[d] = SkLoad<T>::cvt(wsum > 0.f ? val / wsum : 0.f);
    }
}

template <typename T, int D>
static hipError_t launch_splitk_t(const SplitKParams& p, hipStream_t stream) {
    const int MB = p.M >= 4 ? 4 : (p.M >= 2 ? 2 : 1);
    const int mblocks = (p.M + MB - 1) / MB;
    const dim3 grid(p.S, p.H, p.B * mblocks);
    if (MB == 4) hipLaunchKernelGGL((splitk_partial_kernel<T, D, 4>), grid, dim3(SK_THREADS), 0, stream, p);
    else if (MB == 2) hipLaunchKernelGGL((splitk_partial_kernel<T, D, 2>), grid, dim3(SK_THREADS), 0, stream, p);
    else hipLaunchKernelGGL((splitk_partial_kernel<T, D, 1>), grid, dim3(SK_THREADS), 0, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((splitk_merge_kernel<T, D>), dim3(p.M, p.H, p.B), dim3(64), 0, stream, p);
    return hipGetLastError();
}

template <typename T>
static hipError_t launch_splitk_d(const SplitKParams& p, int D, hipStream_t s) {
    switch (D) {
        case 16: return launch_splitk_t<T, 16>(p, s);
        case 32: return launch_splitk_t<T, 32>(p, s);
        case 64: return launch_splitk_t<T, 64>(p, s);
        case 128: return launch_splitk_t<T, 128>(p, s);
    }
    return hipErrorInvalidValue;
}

template <typename T>
static hipError_t launch_merge_d(const SplitKParams& p, int D, hipStream_t s) {
    const dim3 grid(p.M, p.H, p.B);
    switch (D) {
        case 16: hipLaunchKernelGGL((splitk_merge_kernel<T, 16>), grid, dim3(64), 0, s, p); break;
        case 32: hipLaunchKernelGGL((splitk_merge_kernel<T, 32>), grid, dim3(64), 0, s, p); break;
        case 64: hipLaunchKernelGGL((splitk_merge_kernel<T, 64>), grid, dim3(64), 0, s, p); break;
        case 128: hipLaunchKernelGGL((splitk_merge_kernel<T, 128>), grid, dim3(64), 0, s, p); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_splitk_merge(const SplitKParams& p, int dtype, int D, hipStream_t stream) {
    if (dtype == T5A_BF16) return launch_merge_d<__bf16>(p, D, stream);
    if (dtype == T5A_F16) return launch_merge_d<_Float16>(p, D, stream);
    if (dtype == T5A_F32) return launch_merge_d<float>(p, D, stream);
    return hipErrorInvalidValue;
}

hipError_t launch_splitk(const SplitKParams& p, int dtype, int D, hipStream_t stream) {
    if (dtype == T5A_BF16) return launch_splitk_d<__bf16>(p, D, stream);
    if (dtype == T5A_F16) return launch_splitk_d<_Float16>(p, D, stream);
    if (dtype == T5A_F32) return launch_splitk_d<float>(p, D, stream);
    return hipErrorInvalidValue;
}

}  // namespace t5a
