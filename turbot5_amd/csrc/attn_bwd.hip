// Backward of the dense fused-bias attention forward for gfx950: dq, dk, dv and the gradient of the
// (num_buckets, H) bias table.  Replaces flash_attn_v2_bwd_bias of the reference
// (src/turbot5/ops/fused_bias_attention.py:397-820: _bwd_preprocess, _bwd_kv_bias_kernel with its atomics on the
// table gradient :617-619, _bwd_q_kernel).
//
// Three kernels.  The general ones do all arithmetic in fp32 (inputs of any of the three types are widened on their
// way into LDS; the products run on the fp32 matrix cores, v_mfma_f32_32x32x2_f32), so one code path serves fp32 and
// 16-bit tensors at head_dim 16, 32 and 64; 16-bit tensors at head_dim 64 have a faster pair of their own on the 16-bit
// matrix cores (bwd16_kernel, further down) unless the caller asks for fp32 arithmetic, and at head_dim 128 three
// passes of the same kind (bwd16_d128_kernel).  The general kernels:
//
//   bwd_rows_kernel   delta_i = sum_d o_id do_id and the log-sum-exp in base-2 units, per query row; also clears the
//                     table gradient
//   bwd_kernel<KV=0>  a workgroup owns 128 query rows (32 per wavefront) and walks the key tiles of 64:
//                     S^T = K Q^T, dP^T = V dO^T (key rows from LDS as the A operand, so a lane owns one query and
//                     its log-sum-exp and delta are lane scalars), P^T = exp2(c1 S^T + bias - lse),
//                     dS^T = P^T (dP^T - delta), dQ^T += K^T dS^T.  The table gradient is collected here: tiles whose
//                     distances are all saturated add their dS to one of two lane sums, the tiles around the
//                     diagonal add element by element into a per-bucket histogram in LDS; one global atomic per
//                     bucket and workgroup at the end.
//   bwd_kernel<KV=1>  a workgroup owns 128 keys and walks the query tiles of 64, the same products with the roles
//                     swapped (query rows from LDS; log-sum-exp and delta of the 64 queries staged in LDS):
//                     dV^T += dO^T P, dK^T += Q^T dS.
//
// With cu_seqlens the same kernels run a packed batch (varlen_fused_bias_attn.py:407-800): a workgroup looks up its
// sequence's first row and length and works on that sequence; the grid is sized for the longest one.
// Scores use the key position j and the query position i + N - M, as the forward does; rows whose log-sum-exp is
// -inf (no visible key) have no gradient.  Rows and keys past the end of a tensor are read as zeros and masked.
#include "lut_device.h"
#include "t5a_internal.h"

namespace t5a {

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x8 __attribute__((ext_vector_type(8)));

constexpr int kBwdThreads = 256;
constexpr int kBwdOwn = 128;     // own rows per workgroup (queries for dq, keys for dk / dv)
constexpr int kBwdOther = 64;    // rows of the other kind per tile
constexpr int kMaxBuckets = 2 * 2 * kMaxThresholds;

template <typename T> __device__ __forceinline__ float to_f32(T x) { return static_cast<float>(x); }

// four consecutive elements of a row as floats (8 or 16 bytes, aligned: head_dim and strides are multiples of 8 / 4)
template <typename T> __device__ __forceinline__ f32x4 load4(const T* p) {
    if constexpr (sizeof(T) == 4) {
        return *reinterpret_cast<const f32x4*>(p);
    } else {
        typedef T t4 __attribute__((ext_vector_type(4)));
        const t4 x = *reinterpret_cast<const t4*>(p);
        return f32x4{to_f32(x[0]), to_f32(x[1]), to_f32(x[2]), to_f32(x[3])};
    }
}
template <typename T> __device__ __forceinline__ void store4(T* p, f32x4 x) {
    if constexpr (sizeof(T) == 4) {
        *reinterpret_cast<f32x4*>(p) = x;
    } else {
        typedef T t4 __attribute__((ext_vector_type(4)));
        *reinterpret_cast<t4*>(p) = t4{(T)x[0], (T)x[1], (T)x[2], (T)x[3]};
    }
}

// rows per block of bwd_rows_kernel: up to eight threads share a row, 16 bytes per load, so that a wavefront's loads
// cover whole rows (one thread per row reads with a stride of a row and takes twice as long)
template <typename T, int D> struct RowsGeom {
    static constexpr int CH = D * (int)sizeof(T) / 16;      // 16-byte chunks per row
    static constexpr int TPR = CH < 8 ? CH : 8;             // threads per row
    static constexpr int CPT = CH / TPR;                    // chunks per thread
    static constexpr int ROWS = 256 / TPR;                  // rows per block
    static constexpr int EPC = 16 / (int)sizeof(T);         // elements per chunk
};

template <typename T, int D>
__global__ __launch_bounds__(256) void bwd_rows_kernel(const BwdParams p) {
    using G = RowsGeom<T, D>;
    // dense: row = (b, h, i) flattened, statistics (B,H,M); packed: row = (token, h) flattened, statistics (total_q, H)
    const int sub = threadIdx.x % G::TPR;
    const int64_t row = (int64_t)blockIdx.x * G::ROWS + threadIdx.x / G::TPR;
    const bool packed = p.cu_q != nullptr;
    const int64_t rows = packed ? (int64_t)p.total_q * p.H : (int64_t)p.B * p.H * p.M;
    // the table gradient is accumulated with atomics by the dq kernel: clear it here, ahead of that launch
    if (p.dtable != nullptr) {
        const int64_t n = (int64_t)p.n_buckets * p.H;
        for (int64_t x = (int64_t)blockIdx.x * 256 + threadIdx.x; x < n; x += (int64_t)gridDim.x * 256) p.dtable[x] = 0.f;
    }
    float acc = 0.f;
    if (row < rows) {
        int64_t o_off, g_off;
        if (packed) {
            const int64_t tok = row / p.H;
            const int h = (int)(row - tok * p.H);
            o_off = tok * p.o_sr + (int64_t)h * p.o_sh;
            g_off = tok * p.do_sr + (int64_t)h * p.do_sh;
        } else {
            const int i = (int)(row % p.M);
            const int64_t bh = row / p.M;
            const int h = (int)(bh % p.H), b = (int)(bh / p.H);
            o_off = (int64_t)b * p.o_sb + (int64_t)h * p.o_sh + (int64_t)i * p.o_sr;
            g_off = (int64_t)b * p.do_sb + (int64_t)h * p.do_sh + (int64_t)i * p.do_sr;
        }
        const T* o = reinterpret_cast<const T*>(p.o) + o_off;
        const T* g = reinterpret_cast<const T*>(p.dout) + g_off;
#pragma unroll
        for (int c = 0; c < G::CPT; ++c)
#pragma unroll
            for (int q4 = 0; q4 < G::EPC / 4; ++q4) {
                const int at = (sub * G::CPT + c) * G::EPC + 4 * q4;
                const f32x4 x = load4(o + at), y = load4(g + at);
                acc += x[0] * y[0] + x[1] * y[1] + x[2] * y[2] + x[3] * y[3];
            }
    }
    // (every lane takes part in the exchange; the threads of a row are neighbours in one wavefront)
#pragma unroll
    for (int off = 1; off < G::TPR; off <<= 1) acc += __shfl_xor(acc, off, 64);
    if (row >= rows || sub != 0) return;
    p.delta[row] = acc;
    const float l = p.lse[row];
    // a row without a visible key: +inf makes every exp2(score - lse2) of the row 0
    p.lse2[row] = l == -INFINITY ? INFINITY : l * 1.4426950408889634f;
}

template <typename T, int D, bool CAUSAL, bool KV>
__global__ __launch_bounds__(kBwdThreads, 2) void bwd_kernel(const BwdParams p) {
    constexpr int STR = D + 1;              // fp32 tile rows padded by one float
    constexpr int DT = (D + 31) / 32;       // 32-row blocks of the transposed gradients
    constexpr int KS = D / 2;               // k-steps of a product over head_dim
    constexpr int NT = kBwdOther / 32;
    __shared__ float ta[kBwdOther * STR + 32];     // K (dq) / Q (dk, dv) tile
    __shared__ float tb[kBwdOther * STR + 32];     // V (dq) / dO (dk, dv) tile
    __shared__ float rowstat[2 * kBwdOther];       // KV: lse2 and delta of the tile's queries
    __shared__ float lut_bias[2 * kMaxSaturation + 1];   // bias * log2(e) per clamped distance
    __shared__ int lut_bucket[KV ? 1 : 2 * kMaxSaturation + 1];
    __shared__ float hist[KV ? 1 : kMaxBuckets];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, lr = lane & 31, hh = lane >> 5;
    const int h = blockIdx.y, b = blockIdx.z;
    const int own_base = blockIdx.x * kBwdOwn;
    const int own_row = own_base + wave * 32 + lr;
    // packed batch: sequence b is the rows [cu[b], cu[b] + len) of the (total, H, D) tensors (len from seq_lens when
    // given, else up to cu[b + 1]); the batch strides are 0 and everything below works on that sequence
    int M = p.M, N = p.N;
    int64_t q_first = 0, k_first = 0;
    if (p.cu_q != nullptr) {
        q_first = p.cu_q[b]; k_first = p.cu_k[b];
        M = p.len_q != nullptr ? p.len_q[b] : p.cu_q[b + 1] - (int)q_first;
        N = p.len_k != nullptr ? p.len_k[b] : p.cu_k[b + 1] - (int)k_first;
        if (own_base >= (KV ? N : M)) return;     // (the grid is sized for the longest sequence)
    }
    const int n_own = KV ? N : M, n_other = KV ? M : N;
    const int P = N - M;                           // query i sits at key position i + P
    const bool has_bias = p.table != nullptr;
    const int sat = has_bias ? p.bs.sat : 0;

    const T* qp = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.q_sb + (int64_t)h * p.q_sh + q_first * p.q_sr;
    const T* kp = reinterpret_cast<const T*>(p.k) + (int64_t)b * p.k_sb + (int64_t)h * p.k_sh + k_first * p.k_sr;
    const T* vp = reinterpret_cast<const T*>(p.v) + (int64_t)b * p.v_sb + (int64_t)h * p.v_sh + k_first * p.v_sr;
    const T* gp = reinterpret_cast<const T*>(p.dout) + (int64_t)b * p.do_sb + (int64_t)h * p.do_sh + q_first * p.do_sr;
    // statistics of query i: index stat_base + i * stat_sr
    const int64_t stat_sr = p.cu_q != nullptr ? p.H : 1;
    const int64_t stat_base = p.cu_q != nullptr ? q_first * p.H + h : ((int64_t)b * p.H + h) * p.M;

    // bias (and bucket) per clamped distance
    if (has_bias) {
        for (int x = tid; x <= 2 * sat; x += kBwdThreads) {
            const int bk = bucket_of(p.bs, x - sat);
            lut_bias[x] = load_table(p.table, p.table_dtype, (int64_t)bk * p.t_sbucket + (int64_t)h * p.t_shead) * 1.4426950408889634f;
            if constexpr (!KV) lut_bucket[x] = bk;
        }
        if constexpr (!KV)
            for (int x = tid; x < p.n_buckets; x += kBwdThreads) hist[x] = 0.f;
    }

    // own rows as B operands of the 32x32x2 products: lane (lr, hh) holds elements 2s + hh of its row
    const bool own_ok = own_row < n_own;
    float fa[KS], fb[KS];
    {
        const T* a = (KV ? kp + (int64_t)own_row * p.k_sr : qp + (int64_t)own_row * p.q_sr);
        const T* c = (KV ? vp + (int64_t)own_row * p.v_sr : gp + (int64_t)own_row * p.do_sr);
#pragma unroll
        for (int s4 = 0; s4 < D / 4; ++s4) {
            f32x4 x = {0.f, 0.f, 0.f, 0.f}, y = {0.f, 0.f, 0.f, 0.f};
            if (own_ok) { x = load4(a + 4 * s4); y = load4(c + 4 * s4); }
            fa[2 * s4] = hh ? x[1] : x[0]; fa[2 * s4 + 1] = hh ? x[3] : x[2];
            fb[2 * s4] = hh ? y[1] : y[0]; fb[2 * s4 + 1] = hh ? y[3] : y[2];
        }
    }
    float lse2_own = INFINITY, delta_own = 0.f;
    if (!KV && own_ok) { lse2_own = p.lse2[stat_base + own_row * stat_sr]; delta_own = p.delta[stat_base + own_row * stat_sr]; }

    // tiles of the other kind that can hold a visible pair
    int t_lo = 0, t_hi = (n_other + kBwdOther - 1) / kBwdOther;
    if (CAUSAL) {
        if (!KV) t_hi = min(t_hi, max(0, (own_base + kBwdOwn - 1 + P) / kBwdOther + 1));   // keys j <= i + P
        else t_lo = max(0, own_base - P) / kBwdOther;                                      // queries i >= j - P
    }

    f32x16 acc_a[DT], acc_b[DT];     // dQ^T or dK^T; dV^T
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) { acc_a[dt][r] = 0.f; acc_b[dt][r] = 0.f; }
    float sum_lo = 0.f, sum_hi = 0.f;   // dS of the tiles saturated on the left / on the right of the diagonal

    for (int t = t_lo; t < t_hi; ++t) {
        const int o0 = t * kBwdOther;
        __syncthreads();     // the previous tile's readers are done (and the LUT is written, first time round)
        {
            const T* a = KV ? qp : kp;
            const T* c = KV ? gp : vp;
            const int64_t a_sr = KV ? p.q_sr : p.k_sr, c_sr = KV ? p.do_sr : p.v_sr;
            for (int idx = tid; idx < kBwdOther * (D / 4); idx += kBwdThreads) {
                const int row = idx / (D / 4), c4 = idx % (D / 4);
                f32x4 x = {0.f, 0.f, 0.f, 0.f}, y = {0.f, 0.f, 0.f, 0.f};
                if (o0 + row < n_other) {
                    x = load4(a + (int64_t)(o0 + row) * a_sr + 4 * c4);
                    y = load4(c + (int64_t)(o0 + row) * c_sr + 4 * c4);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) { ta[row * STR + 4 * c4 + e] = x[e]; tb[row * STR + 4 * c4 + e] = y[e]; }
            }
            if (KV && tid < 2 * kBwdOther) {
                const int row = tid & (kBwdOther - 1);
                float val = tid < kBwdOther ? INFINITY : 0.f;
                if (o0 + row < n_other)
                    val = tid < kBwdOther ? p.lse2[stat_base + (o0 + row) * stat_sr] : p.delta[stat_base + (o0 + row) * stat_sr];
                rowstat[tid] = val;
            }
        }
        __syncthreads();

        f32x16 s[NT], dp[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
            for (int r = 0; r < 16; ++r) { s[nt][r] = 0.f; dp[nt][r] = 0.f; }
            const int row = 32 * nt + lr;
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2) {
                s[nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(ta[row * STR + 2 * k2 + hh], fa[k2], s[nt], 0, 0, 0);
                dp[nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(tb[row * STR + 2 * k2 + hh], fb[k2], dp[nt], 0, 0, 0);
            }
        }

        // wavefront-uniform: every pair of this wavefront's tile lies at a saturated distance on one side
        int side = 0;
        if constexpr (!KV) {
            const int i_lo = own_base + wave * 32 + P, i_hi = i_lo + 31;    // query positions
            if (o0 + kBwdOther - 1 - i_lo <= -sat) side = 1;
            else if (o0 - i_hi >= sat) side = 2;
        }
        float tile_sum = 0.f;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int ol = 32 * nt + 8 * (r >> 2) + 4 * hh + (r & 3);   // row of the other kind inside the tile
                const int i = KV ? o0 + ol : own_row, j = KV ? own_row : o0 + ol;
                const int rel = j - (i + P);
                const bool valid = i < M && j < N && (!CAUSAL || rel <= 0);
                const int x = min(max(rel, -sat), sat) + sat;
                const float bias2 = has_bias ? lut_bias[x] : 0.f;
                const float l2 = KV ? rowstat[ol] : lse2_own;
                const float dl = KV ? rowstat[kBwdOther + ol] : delta_own;
                const float pv = valid ? __builtin_amdgcn_exp2f(__builtin_fmaf(p.c1, s[nt][r], bias2) - l2) : 0.f;
                const float ds = pv * (dp[nt][r] - dl);
                s[nt][r] = pv;
                dp[nt][r] = ds;
                if constexpr (!KV) {
                    if (has_bias) {
                        if (side != 0) tile_sum += ds;
                        else if (valid) atomicAdd(&hist[lut_bucket[x]], ds);
                    }
                }
            }
        if (side == 1) sum_lo += tile_sum; else if (side == 2) sum_hi += tile_sum;

        // dQ^T += K^T dS^T   /   dK^T += Q^T dS, dV^T += dO^T P   (contraction over the tile's 64 rows, two per product)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int ol = 32 * nt + 8 * (r >> 2) + 4 * hh + (r & 3);
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    acc_a[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(ta[ol * STR + 32 * dt + lr], dp[nt][r], acc_a[dt], 0, 0, 0);
                    if constexpr (KV)
                        acc_b[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(tb[ol * STR + 32 * dt + lr], s[nt][r], acc_b[dt], 0, 0, 0);
                }
            }
    }

    // rows: lane (lr, hh) holds, for its own row, elements 32 dt + 8 g + 4 hh .. + 3 of the transposed gradients
    const float scale = p.c1 * 0.6931471805599453f;     // d score / d (q . k), natural units
    if (own_ok) {
        T* oa = KV ? reinterpret_cast<T*>(p.dk) + (int64_t)b * p.dk_sb + (int64_t)h * p.dk_sh + (k_first + own_row) * p.dk_sr
                   : reinterpret_cast<T*>(p.dq) + (int64_t)b * p.dq_sb + (int64_t)h * p.dq_sh + (q_first + own_row) * p.dq_sr;
        T* ob = KV ? reinterpret_cast<T*>(p.dv) + (int64_t)b * p.dv_sb + (int64_t)h * p.dv_sh + (k_first + own_row) * p.dv_sr : nullptr;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d0 = 32 * dt + 8 * g + 4 * hh;
                if (d0 < D) {
                    store4(oa + d0, f32x4{acc_a[dt][4 * g] * scale, acc_a[dt][4 * g + 1] * scale,
                                          acc_a[dt][4 * g + 2] * scale, acc_a[dt][4 * g + 3] * scale});
                    if constexpr (KV)
                        store4(ob + d0, f32x4{acc_b[dt][4 * g], acc_b[dt][4 * g + 1], acc_b[dt][4 * g + 2], acc_b[dt][4 * g + 3]});
                }
            }
    }
    if constexpr (!KV) {
        if (has_bias && p.dtable != nullptr) {
            // the saturated tiles' sums: one value per wavefront and side, into the last bucket of that side
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                sum_lo += __shfl_xor(sum_lo, off, 64);
                sum_hi += __shfl_xor(sum_hi, off, 64);
            }
            if (lane == 0) {
                if (sum_lo != 0.f) atomicAdd(&hist[lut_bucket[0]], sum_lo);
                if (sum_hi != 0.f) atomicAdd(&hist[lut_bucket[2 * sat]], sum_hi);
            }
            __syncthreads();
            for (int x = tid; x < p.n_buckets; x += kBwdThreads)
                if (hist[x] != 0.f) atomicAdd(&p.dtable[(int64_t)x * p.H + h], hist[x]);
        }
    }
}


// ------------------------------------------------------------------------------------------------------------------
// 16-bit inputs at head_dim 64: the same two passes on the 16-bit matrix cores (v_mfma_f32_32x32x16_bf16 / _f16).
//
// The products over head_dim (S^T = K Q^T, dP^T = V dO^T and their counterparts of the dk / dv pass) take the inputs as
// they are; the probabilities and dS are rounded to the input type for the products over the tile's rows, as the
// reference does (fused_bias_attention.py:575-590: p.to(Q.dtype), ds.to(Q.dtype)); sums stay in fp32.  A tile of
// the other kind is 64 rows of 128 bytes in LDS and serves both kinds of product from one copy: rows are read as they
// lie (A operand, contraction over head_dim), and the contraction over the tile's rows reads it through the
// transposing LDS read (ds_read_b64_tr_b16: four rows x 16 columns per group of 16 lanes), whose k-slot order --
// rows 4h .. 4h+3 and 8+4h .. 8+4h+3 of every 16 in lane half h -- is exactly the order in which a lane holds the rows
// of a 32x32 accumulator, so P and dS go from accumulator registers to B operands with a conversion and no shuffle.
// The 16-byte chunks of a row are XOR-swizzled with a pattern that keeps both kinds of read free of bank conflicts.
// The next tile's rows are fetched into registers while the current tile is worked on.
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));

template <typename T> struct Half16;
template <> struct Half16<__bf16> {
    typedef __bf16 v8 __attribute__((ext_vector_type(8)));
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};
template <> struct Half16<_Float16> {
    typedef _Float16 v8 __attribute__((ext_vector_type(8)));
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};

// chunk swizzle of a tile row: 16 consecutive rows put a chunk into 16 different 16-byte slots of a 256-byte bank
// line (row reads), and rows 2, 3 (mod 4) swap their 64-byte halves (the transposing read touches four consecutive
// rows x 64 bytes at a time)
__device__ __forceinline__ int tile_swz(int row) { return ((row >> 1) & 7) ^ (((row >> 1) & 1) << 2); }

// LDS-DMA: a wavefront instruction fetches 64 x 16 bytes at per-lane byte offsets of a buffer (zeros past its end) and
// writes them to 1 KB of consecutive LDS addresses in lane order, without passing through registers.  Issued from
// assembly, so the wait for it (vmcnt) is the kernel's own.
__device__ __forceinline__ u32x4 dma_rsrc(const void* base, unsigned bytes) {
    const unsigned long long a = reinterpret_cast<unsigned long long>(base);
    return u32x4{(unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)a),
                 (unsigned)__builtin_amdgcn_readfirstlane((int)((unsigned)(a >> 32) & 0xffffu)),
                 (unsigned)__builtin_amdgcn_readfirstlane((int)bytes), 0x00020000u};
}
__device__ __forceinline__ void dma_16(u32x4 rs, unsigned lds_addr, int voffset) {
    const u32x4 rsrc = {(unsigned)__builtin_amdgcn_readfirstlane((int)rs[0]), (unsigned)__builtin_amdgcn_readfirstlane((int)rs[1]),
                        (unsigned)__builtin_amdgcn_readfirstlane((int)rs[2]), (unsigned)__builtin_amdgcn_readfirstlane((int)rs[3])};
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :: "s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voffset), "s"(rsrc) : "memory", "m0");
}

template <typename T, bool CAUSAL, bool KV>
__global__ __launch_bounds__(kBwdThreads, 2) void bwd16_kernel(const BwdParams p) {
    constexpr int D = 64, DT = 2, KS = 4, NT = kBwdOther / 32;
    using H16 = Half16<T>;
    using v8 = typename H16::v8;
    // two buffers of each: tile t + 1 is written while tile t is read, one barrier per tile
    __shared__ __attribute__((aligned(16))) T ta2[2][kBwdOther * D];   // K (dq) / Q (dk, dv) tiles
    __shared__ __attribute__((aligned(16))) T tb2[2][kBwdOther * D];   // V (dq) / dO (dk, dv) tiles
    __shared__ __attribute__((aligned(16))) float rowstat2[2][2 * kBwdOther];   // KV: lse2 and delta of the tiles' queries
    __shared__ float lut_bias[2 * kMaxSaturation + 1];
    __shared__ int lut_bucket[KV ? 1 : 2 * kMaxSaturation + 1];
    __shared__ float hist[KV ? 1 : kMaxBuckets];
    __shared__ float hist_rel[KV ? 1 : 2 * kMaxSaturation + 1];   // dS summed per clamped distance (tiles around the diagonal)

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, lr = lane & 31, hh = lane >> 5;
    // Grid: (own blocks, heads, batch).  With a causal mask the own blocks differ in length (a query block sees the
    // keys up to its own end, a key block the queries from its own start on), and whatever is dispatched last should
    // be short: the launch is then (heads, batch, own blocks), the slowest index walking the blocks longest first.
    const int h = CAUSAL ? blockIdx.x : blockIdx.y, b = CAUSAL ? blockIdx.y : blockIdx.z;
    const int own_block = !CAUSAL ? blockIdx.x : (KV ? blockIdx.z : gridDim.z - 1 - blockIdx.z);
    const int own_base = own_block * kBwdOwn;
    const int own_row = own_base + wave * 32 + lr;
    int M = p.M, N = p.N;
    int64_t q_first = 0, k_first = 0;
    if (p.cu_q != nullptr) {
        q_first = p.cu_q[b]; k_first = p.cu_k[b];
        M = p.len_q != nullptr ? p.len_q[b] : p.cu_q[b + 1] - (int)q_first;
        N = p.len_k != nullptr ? p.len_k[b] : p.cu_k[b + 1] - (int)k_first;
        if (own_base >= (KV ? N : M)) return;     // (the grid is sized for the longest sequence)
    }
    const int n_own = KV ? N : M, n_other = KV ? M : N;
    const int P = N - M;
    const bool has_bias = p.table != nullptr;
    const int sat = has_bias ? p.bs.sat : 0;

    const T* qp = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.q_sb + (int64_t)h * p.q_sh + q_first * p.q_sr;
    const T* kp = reinterpret_cast<const T*>(p.k) + (int64_t)b * p.k_sb + (int64_t)h * p.k_sh + k_first * p.k_sr;
    const T* vp = reinterpret_cast<const T*>(p.v) + (int64_t)b * p.v_sb + (int64_t)h * p.v_sh + k_first * p.v_sr;
    const T* gp = reinterpret_cast<const T*>(p.dout) + (int64_t)b * p.do_sb + (int64_t)h * p.do_sh + q_first * p.do_sr;
    const int64_t stat_sr = p.cu_q != nullptr ? p.H : 1;
    const int64_t stat_base = p.cu_q != nullptr ? q_first * p.H + h : ((int64_t)b * p.H + h) * p.M;

    // own rows as B operands: lane (lr, hh) holds elements 16 s + 8 hh .. + 7 of its row
    const bool own_ok = own_row < n_own;
    v8 fa[KS], fb[KS];
    {
        const T* a = (KV ? kp + (int64_t)own_row * p.k_sr : qp + (int64_t)own_row * p.q_sr);
        const T* c = (KV ? vp + (int64_t)own_row * p.v_sr : gp + (int64_t)own_row * p.do_sr);
#pragma unroll
        for (int s = 0; s < KS; ++s) {
#pragma unroll
            for (int e = 0; e < 8; ++e) { fa[s][e] = (T)0.0f; fb[s][e] = (T)0.0f; }
            if (own_ok) {
                fa[s] = *reinterpret_cast<const v8*>(a + 16 * s + 8 * hh);
                fb[s] = *reinterpret_cast<const v8*>(c + 16 * s + 8 * hh);
            }
        }
    }
    float lse2_own = INFINITY, delta_own = 0.f;
    if (!KV && own_ok) { lse2_own = p.lse2[stat_base + own_row * stat_sr]; delta_own = p.delta[stat_base + own_row * stat_sr]; }

    int t_lo = 0, t_hi = (n_other + kBwdOther - 1) / kBwdOther;
    if (CAUSAL) {
        if (!KV) t_hi = min(t_hi, max(0, (own_base + kBwdOwn - 1 + P) / kBwdOther + 1));
        else t_lo = max(0, own_base - P) / kBwdOther;
    }

    // staging by LDS-DMA: a tile is 8 slabs of 1 KB (8 rows); wavefront w requests slabs 2 w and 2 w + 1 of each of
    // the two tiles.  The chunk swizzle is applied on the source side: the lane that writes physical chunk pc of row r
    // fetches logical chunk pc ^ swizzle(r).  Rows past the end of the tensor are out of the descriptor's range and
    // arrive as zeros.  (Slices stay below 2 GiB -- checked on the host -- so 32-bit offsets do.)
    const T* src_a = KV ? qp : kp;
    const T* src_b = KV ? gp : vp;
    const int a_srb = (int)(KV ? p.q_sr : p.k_sr) * 2, b_srb = (int)(KV ? p.do_sr : p.v_sr) * 2;     // row strides in bytes
    const u32x4 rs_a = dma_rsrc(src_a, n_other > 0 ? (unsigned)(n_other - 1) * (unsigned)a_srb + D * 2 : 0u);
    const u32x4 rs_b = dma_rsrc(src_b, n_other > 0 ? (unsigned)(n_other - 1) * (unsigned)b_srb + D * 2 : 0u);
    int dma_a[2], dma_b[2];     // this lane's byte offsets inside a tile, per slab
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const int row = (2 * wave + c) * 8 + (lane >> 3), ch = (lane & 7) ^ tile_swz(row);
        dma_a[c] = row * a_srb + ch * 16;
        dma_b[c] = row * b_srb + ch * 16;
    }
    const unsigned lds_a = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)&ta2[0][0];
    const unsigned lds_b = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)&tb2[0][0];
    float rstat = 0.f;
    auto request = [&](int t, int buf) {     // tile t into buffer buf: four requests per wavefront
        const int o0 = t * kBwdOther;
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const unsigned at = (unsigned)buf * (kBwdOther * D * 2) + (2 * wave + c) * 1024u;
            dma_16(rs_a, lds_a + at, o0 * a_srb + dma_a[c]);
            dma_16(rs_b, lds_b + at, o0 * b_srb + dma_b[c]);
        }
    };
    auto fetch_stat = [&](int t) {
        const int o0 = t * kBwdOther;
        if (KV && tid < 2 * kBwdOther) {
            const int row = tid & (kBwdOther - 1);
            rstat = tid < kBwdOther ? INFINITY : 0.f;
            if (o0 + row < n_other)
                rstat = tid < kBwdOther ? p.lse2[stat_base + (o0 + row) * stat_sr] : p.delta[stat_base + (o0 + row) * stat_sr];
        }
    };
    auto stage_stat = [&](int buf) {
        if (KV && tid < 2 * kBwdOther) rowstat2[buf][tid] = rstat;
    };
    // row reads: element offsets of this lane's chunk (2 s + hh) of row 32 nt + lr
    int row_off[NT][KS];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const int row = 32 * nt + lr;
            row_off[nt][s] = row * D + (((2 * s + hh) ^ tile_swz(row)) * 8);
        }
    // transposing reads: within a group of 16 lanes, lane 4 j + a supplies the address of elements 4 a' .. of row j
    // and receives, for column (lane % 16) of the group's 16 columns, the rows j = 0 .. 3.  Group g covers the
    // columns 32 dt + 16 (g & 1) .. + 15 and the rows 4 (g >> 1) .. + 3 (first read) and 8 more (second read).
    int tr_lo[DT], tr_hi[DT];
    {
        const int g = lane >> 4, r = lane & 15, jj = r >> 2, aa = r & 3;
        const int row = 4 * (g >> 1) + jj, x = 2 * (g & 1) + (aa >> 1);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            tr_lo[dt] = row * D + (((4 * dt + x) ^ tile_swz(row)) * 8) + (aa & 1) * 4;
            tr_hi[dt] = (row + 8) * D + (((4 * dt + x) ^ tile_swz(row + 8)) * 8) + (aa & 1) * 4;
        }
    }
    auto tr_frag = [&](const T* tile, int g16, int dt) {   // columns 32 dt .. + 31 x rows 16 g16 .. + 15 of the tile, as an A operand
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(tile + tr_lo[dt] + 16 * g16 * D));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(tile + tr_hi[dt] + 16 * g16 * D));
        return __builtin_bit_cast(v8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    };

    f32x16 acc_a[DT], acc_b[DT];     // dQ^T or dK^T; dV^T
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) { acc_a[dt][r] = 0.f; acc_b[dt][r] = 0.f; }
    float sum_lo = 0.f, sum_hi = 0.f;

    // Tile t + 1 is requested when the barrier at the top of tile t has shown that every wavefront is done with the
    // buffer it goes into, and has all of tile t's work to arrive in.
    if (t_lo < t_hi) { request(t_lo, 0); fetch_stat(t_lo); stage_stat(0); }
    // the per-distance bias (and bucket) table, behind the first tile's requests and the loads of the own rows: its
    // look-ups in the bias table are one more round trip to memory, which now runs beside theirs
    if (has_bias) {
        for (int x = tid; x <= 2 * sat; x += kBwdThreads) {
            const int bk = bucket_of(p.bs, x - sat);
            lut_bias[x] = load_table(p.table, p.table_dtype, (int64_t)bk * p.t_sbucket + (int64_t)h * p.t_shead) * 1.4426950408889634f;
            if constexpr (!KV) { lut_bucket[x] = bk; hist_rel[x] = 0.f; }
        }
        if constexpr (!KV)
            for (int x = tid; x < p.n_buckets; x += kBwdThreads) hist[x] = 0.f;
    }

    for (int t = t_lo; t < t_hi; ++t) {
        const int o0 = t * kBwdOther;
        const int buf = (t - t_lo) & 1;
        __builtin_amdgcn_s_waitcnt(0x0F70);     // vmcnt(0): this wavefront's requests for tile t have landed
        __syncthreads();                        // ... and everybody's; the other buffer is free (and, first time round, the LUT written)
        if (t + 1 < t_hi) { request(t + 1, buf ^ 1); fetch_stat(t + 1); }
        const T* ta = ta2[buf]; const T* tb = tb2[buf];
        const float* rowstat = rowstat2[buf];
        (void)rowstat;

        f32x16 s[NT], dp[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            // (dP starts at -delta: the matrix core subtracts it for free)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                f32x4 d4 = {delta_own, delta_own, delta_own, delta_own};
                if constexpr (KV) d4 = *reinterpret_cast<const f32x4*>(rowstat + kBwdOther + 32 * nt + 8 * r4 + 4 * hh);
#pragma unroll
                for (int e = 0; e < 4; ++e) { s[nt][4 * r4 + e] = 0.f; dp[nt][4 * r4 + e] = -d4[e]; }
            }
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2) {
                s[nt] = H16::mfma(*reinterpret_cast<const v8*>(ta + row_off[nt][k2]), fa[k2], s[nt]);
                dp[nt] = H16::mfma(*reinterpret_cast<const v8*>(tb + row_off[nt][k2]), fb[k2], dp[nt]);
            }
        }

        // wavefront-uniform tile classes: every pair at a saturated distance on one side (constant bias); every pair
        // visible (no per-element test)
        const int w_lo = own_base + wave * 32, w_hi = w_lo + 31;            // this wavefront's own rows
        // rel = j - (i + P): dq pass j in the tile, i own; dk/dv pass i in the tile, j own
        const int rel_min = KV ? w_lo - (o0 + kBwdOther - 1 + P) : o0 - (w_hi + P);
        const int rel_max = KV ? w_hi - (o0 + P) : o0 + kBwdOther - 1 - (w_lo + P);
        int side = 0;
        if (rel_max <= -sat) side = 1; else if (rel_min >= sat) side = 2;
        const bool all_visible = o0 + kBwdOther <= n_other && w_hi < n_own && (!CAUSAL || rel_max <= 0);
        const float c1 = p.c1;
        float tile_sum = 0.f;
        // Second stage, 16 rows of the tile at a time: probabilities and dS of this lane's eight pairs, rounded to
        // the input type, then the products that contract over those rows --
        //   dQ^T += K^T dS^T   /   dK^T += Q^T dS, dV^T += dO^T P
        // -- so that the matrix cores work on one group while the vector units form the next.
        auto second_stage = [&](auto check_c, auto lut_c) {
            constexpr bool CHECK = decltype(check_c)::value, LUT = decltype(lut_c)::value;
            const float bias_c = (has_bias && !LUT) ? lut_bias[side == 1 ? 0 : 2 * sat] : 0.f;
            // Table gradient around the diagonal (dq pass, LUT variants): dS summed per distance.  Pairs at one
            // distance lie on a diagonal of the (key, query) tile, and a lane half walks its keys in ascending order:
            // each lane adds its dS to a running value that then moves one lane up (one query further) with every
            // key, so a diagonal's sum travels with it.  A lane half holds the keys 8 k + 4 hh .. + 3: five lanes up
            // between two groups.  What leaves a half at lane 31 is added to the distance's word in LDS first, and
            // at the end of the tile every lane adds what it holds: some 190 single-lane atomic adds per tile and
            // wavefront instead of 2 048 (an LDS floating-point atomic handles about one lane per cycle).
            float diag = 0.f;
            int x_last = 0;
            (void)x_last;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    f32x8 ds8, pv8;
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
                        const int r4 = 2 * u + half;
                        const int ol0 = 32 * nt + 8 * r4 + 4 * hh;     // first of four consecutive rows of the other kind
                        f32x4 l4 = {lse2_own, lse2_own, lse2_own, lse2_own};
                        if constexpr (KV) l4 = *reinterpret_cast<const f32x4*>(rowstat + ol0);
                        f32x4 bl4;   // constant bias minus log-sum-exp
#pragma unroll
                        for (int e = 0; e < 4; ++e) bl4[e] = bias_c - l4[e];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int r = 4 * r4 + e, ol = ol0 + e;
                            const int i = KV ? o0 + ol : own_row, j = KV ? own_row : o0 + ol;
                            const int rel = j - (i + P);
                            int x = 0;
                            float bias2 = bias_c;
                            if constexpr (LUT) {
                                x = min(max(rel, -sat), sat) + sat;
                                bias2 = lut_bias[x];
                            }
                            float pv = LUT ? __builtin_amdgcn_exp2f(__builtin_fmaf(c1, s[nt][r], bias2) - l4[e])
                                           : __builtin_amdgcn_exp2f(__builtin_fmaf(c1, s[nt][r], bl4[e]));
                            if constexpr (CHECK) {
                                const bool valid = i < M && j < N && (!CAUSAL || rel <= 0);
                                pv = valid ? pv : 0.f;
                            }
                            const float ds = pv * dp[nt][r];
                            pv8[4 * half + e] = pv;
                            ds8[4 * half + e] = ds;
                            if constexpr (!KV) {
                                // table gradient (no test for a table here: a branch per element would cut the
                                // loop into pieces; without one the sum is simply not used, and the LUT variants
                                // run only with one).  Per clamped distance: neighbouring lanes hold neighbouring
                                // distances, so the adds of one instruction go to different words; a pair that
                                // is not visible adds 0.
                                if constexpr (!LUT) {
                                    tile_sum += ds;
                                } else {
                                    diag += ds;      // (a pair that is not visible adds 0)
                                    x_last = x;
                                    const bool last_of_tile = nt == NT - 1 && u == 1 && half == 1 && e == 3;
                                    if (!last_of_tile) {
                                        const int out_from = e == 3 ? 27 : 31;     // lanes whose value leaves the half
                                        if (lr >= out_from) { atomicAdd(&hist_rel[x], diag); diag = 0.f; }
#pragma unroll
                                        for (int sh = 0; sh < (e == 3 ? 5 : 1); ++sh)
                                            diag = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(diag), 0x138, 0xf, 0xf, true));
                                    }
                                }
                            }
                        }
                    }
                    const v8 dsb = __builtin_convertvector(ds8, v8);
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
                        acc_a[dt] = H16::mfma(tr_frag(ta, 2 * nt + u, dt), dsb, acc_a[dt]);
                    if constexpr (KV) {
                        const v8 pb = __builtin_convertvector(pv8, v8);
#pragma unroll
                        for (int dt = 0; dt < DT; ++dt)
                            acc_b[dt] = H16::mfma(tr_frag(tb, 2 * nt + u, dt), pb, acc_b[dt]);
                    }
                }
            if constexpr (!KV && LUT) atomicAdd(&hist_rel[x_last], diag);
        };
        const bool use_lut = has_bias && side == 0;
        if (all_visible && !use_lut) second_stage(std::false_type{}, std::false_type{});
        else if (all_visible) second_stage(std::false_type{}, std::true_type{});
        else if (!use_lut) second_stage(std::true_type{}, std::false_type{});
        else second_stage(std::true_type{}, std::true_type{});
        if (side == 1) sum_lo += tile_sum; else if (side == 2) sum_hi += tile_sum;
        if (t + 1 < t_hi) stage_stat(buf ^ 1);
    }

    const float scale = p.c1 * 0.6931471805599453f;
    if (own_ok) {
        T* oa = KV ? reinterpret_cast<T*>(p.dk) + (int64_t)b * p.dk_sb + (int64_t)h * p.dk_sh + (k_first + own_row) * p.dk_sr
                   : reinterpret_cast<T*>(p.dq) + (int64_t)b * p.dq_sb + (int64_t)h * p.dq_sh + (q_first + own_row) * p.dq_sr;
        T* ob = KV ? reinterpret_cast<T*>(p.dv) + (int64_t)b * p.dv_sb + (int64_t)h * p.dv_sh + (k_first + own_row) * p.dv_sr : nullptr;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d0 = 32 * dt + 8 * g + 4 * hh;
                store4(oa + d0, f32x4{acc_a[dt][4 * g] * scale, acc_a[dt][4 * g + 1] * scale,
                                      acc_a[dt][4 * g + 2] * scale, acc_a[dt][4 * g + 3] * scale});
                if constexpr (KV)
                    store4(ob + d0, f32x4{acc_b[dt][4 * g], acc_b[dt][4 * g + 1], acc_b[dt][4 * g + 2], acc_b[dt][4 * g + 3]});
            }
    }
    if constexpr (!KV) {
        if (has_bias && p.dtable != nullptr) {
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                sum_lo += __shfl_xor(sum_lo, off, 64);
                sum_hi += __shfl_xor(sum_hi, off, 64);
            }
            if (lane == 0) {
                if (sum_lo != 0.f) atomicAdd(&hist[lut_bucket[0]], sum_lo);
                if (sum_hi != 0.f) atomicAdd(&hist[lut_bucket[2 * sat]], sum_hi);
            }
            __syncthreads();
            for (int x = tid; x <= 2 * sat; x += kBwdThreads)     // distances -> buckets
                if (hist_rel[x] != 0.f) atomicAdd(&hist[lut_bucket[x]], hist_rel[x]);
            __syncthreads();
            for (int x = tid; x < p.n_buckets; x += kBwdThreads)
                if (hist[x] != 0.f) atomicAdd(&p.dtable[(int64_t)x * p.H + h], hist[x]);
        }
    }
}

// head_dim 128 (the T5-3B / 11B head shape), 16-bit tensors: the same scheme with rows of 256 bytes.  A row's head_dim
// and two gradients of it no longer fit a wavefront's registers next to the scores, so there are three passes instead
// of two -- PASS 0: dq (and the table gradient), 2: dk, 3: dv (which needs no dP) -- each with one output accumulator;
// the tiles are single-buffered in LDS (two of 16 KB) and staged without a register prefetch.
__device__ __forceinline__ int tile_swz128(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }

template <typename T, bool CAUSAL, int PASS>
__global__ __launch_bounds__(kBwdThreads, 2) void bwd16_d128_kernel(const BwdParams p) {
    constexpr bool KV = PASS != 0;
    constexpr bool WANT_DS = PASS != 3;     // dS and the products with it (dq, dk)
    constexpr bool WANT_DV = PASS == 3;
    constexpr int D = 128, DT = 4, KS = 8, NT = kBwdOther / 32;
    using H16 = Half16<T>;
    using v8 = typename H16::v8;
    __shared__ __attribute__((aligned(16))) T ta2[1][kBwdOther * D];   // K (dq) / Q (dk, dv) tile
    __shared__ __attribute__((aligned(16))) T tb2[1][kBwdOther * D];   // V (dq) / dO (dk, dv) tile
    __shared__ __attribute__((aligned(16))) float rowstat2[1][2 * kBwdOther];   // KV: lse2 and delta of the tile's queries
    __shared__ float lut_bias[2 * kMaxSaturation + 1];
    __shared__ int lut_bucket[KV ? 1 : 2 * kMaxSaturation + 1];
    __shared__ float hist[KV ? 1 : kMaxBuckets];
    __shared__ float hist_rel[KV ? 1 : 2 * kMaxSaturation + 1];   // dS summed per clamped distance (tiles around the diagonal)

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, lr = lane & 31, hh = lane >> 5;
    // Grid: (own blocks, heads, batch).  With a causal mask the own blocks differ in length (a query block sees the
    // keys up to its own end, a key block the queries from its own start on), and whatever is dispatched last should
    // be short: the launch is then (heads, batch, own blocks), the slowest index walking the blocks longest first.
    const int h = CAUSAL ? blockIdx.x : blockIdx.y, b = CAUSAL ? blockIdx.y : blockIdx.z;
    const int own_block = !CAUSAL ? blockIdx.x : (KV ? blockIdx.z : gridDim.z - 1 - blockIdx.z);
    const int own_base = own_block * kBwdOwn;
    const int own_row = own_base + wave * 32 + lr;
    int M = p.M, N = p.N;
    int64_t q_first = 0, k_first = 0;
    if (p.cu_q != nullptr) {
        q_first = p.cu_q[b]; k_first = p.cu_k[b];
        M = p.len_q != nullptr ? p.len_q[b] : p.cu_q[b + 1] - (int)q_first;
        N = p.len_k != nullptr ? p.len_k[b] : p.cu_k[b + 1] - (int)k_first;
        if (own_base >= (KV ? N : M)) return;     // (the grid is sized for the longest sequence)
    }
    const int n_own = KV ? N : M, n_other = KV ? M : N;
    const int P = N - M;
    const bool has_bias = p.table != nullptr;
    const int sat = has_bias ? p.bs.sat : 0;

    const T* qp = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.q_sb + (int64_t)h * p.q_sh + q_first * p.q_sr;
    const T* kp = reinterpret_cast<const T*>(p.k) + (int64_t)b * p.k_sb + (int64_t)h * p.k_sh + k_first * p.k_sr;
    const T* vp = reinterpret_cast<const T*>(p.v) + (int64_t)b * p.v_sb + (int64_t)h * p.v_sh + k_first * p.v_sr;
    const T* gp = reinterpret_cast<const T*>(p.dout) + (int64_t)b * p.do_sb + (int64_t)h * p.do_sh + q_first * p.do_sr;
    const int64_t stat_sr = p.cu_q != nullptr ? p.H : 1;
    const int64_t stat_base = p.cu_q != nullptr ? q_first * p.H + h : ((int64_t)b * p.H + h) * p.M;

    if (has_bias) {
        for (int x = tid; x <= 2 * sat; x += kBwdThreads) {
            const int bk = bucket_of(p.bs, x - sat);
            lut_bias[x] = load_table(p.table, p.table_dtype, (int64_t)bk * p.t_sbucket + (int64_t)h * p.t_shead) * 1.4426950408889634f;
            if constexpr (!KV) { lut_bucket[x] = bk; hist_rel[x] = 0.f; }
        }
        if constexpr (!KV)
            for (int x = tid; x < p.n_buckets; x += kBwdThreads) hist[x] = 0.f;
    }

    // own rows as B operands: lane (lr, hh) holds elements 16 s + 8 hh .. + 7 of its row
    const bool own_ok = own_row < n_own;
    v8 fa[KS], fb[KS];
    {
        const T* a = (KV ? kp + (int64_t)own_row * p.k_sr : qp + (int64_t)own_row * p.q_sr);
        const T* c = (KV ? vp + (int64_t)own_row * p.v_sr : gp + (int64_t)own_row * p.do_sr);
#pragma unroll
        for (int s = 0; s < KS; ++s) {
#pragma unroll
            for (int e = 0; e < 8; ++e) { fa[s][e] = (T)0.0f; fb[s][e] = (T)0.0f; }
            if (own_ok) {
                fa[s] = *reinterpret_cast<const v8*>(a + 16 * s + 8 * hh);
                if constexpr (WANT_DS) fb[s] = *reinterpret_cast<const v8*>(c + 16 * s + 8 * hh);
            }
        }
    }
    float lse2_own = INFINITY, delta_own = 0.f;
    if (!KV && own_ok) { lse2_own = p.lse2[stat_base + own_row * stat_sr]; delta_own = p.delta[stat_base + own_row * stat_sr]; }

    int t_lo = 0, t_hi = (n_other + kBwdOther - 1) / kBwdOther;
    if (CAUSAL) {
        if (!KV) t_hi = min(t_hi, max(0, (own_base + kBwdOwn - 1 + P) / kBwdOther + 1));
        else t_lo = max(0, own_base - P) / kBwdOther;
    }

    // staging: thread -> four 16-byte chunks of each tile (row = idx / 16, chunk = idx % 16)
    const T* src_a = KV ? qp : kp;
    const T* src_b = KV ? gp : vp;
    const int64_t a_sr = KV ? p.q_sr : p.k_sr, b_sr = KV ? p.do_sr : p.v_sr;
    u32x4 ra[4], rb[4];
    float rstat = 0.f;
    auto fetch = [&](int t) {
        const int o0 = t * kBwdOther;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int idx = tid + c * kBwdThreads, row = idx >> 4, ch = idx & 15;
            ra[c] = u32x4{0u, 0u, 0u, 0u}; rb[c] = u32x4{0u, 0u, 0u, 0u};
            if (o0 + row < n_other) {
                ra[c] = *reinterpret_cast<const u32x4*>(src_a + (int64_t)(o0 + row) * a_sr + 8 * ch);
                rb[c] = *reinterpret_cast<const u32x4*>(src_b + (int64_t)(o0 + row) * b_sr + 8 * ch);
            }
        }
        if (KV && tid < 2 * kBwdOther) {
            const int row = tid & (kBwdOther - 1);
            rstat = tid < kBwdOther ? INFINITY : 0.f;
            if (o0 + row < n_other)
                rstat = tid < kBwdOther ? p.lse2[stat_base + (o0 + row) * stat_sr] : p.delta[stat_base + (o0 + row) * stat_sr];
        }
    };
    auto stage = [&](int buf) {
        T* ta = ta2[buf]; T* tb = tb2[buf];
        float* rowstat = rowstat2[buf];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int idx = tid + c * kBwdThreads, row = idx >> 4, ch = idx & 15;
            const int at = row * D + ((ch ^ tile_swz128(row)) * 8);
            *reinterpret_cast<u32x4*>(ta + at) = ra[c];
            *reinterpret_cast<u32x4*>(tb + at) = rb[c];
        }
        if (KV && tid < 2 * kBwdOther) rowstat[tid] = rstat;
    };
    // row reads: element offsets of this lane's chunk (2 s + hh) of row 32 nt + lr
    int row_off[NT][KS];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const int row = 32 * nt + lr;
            row_off[nt][s] = row * D + (((2 * s + hh) ^ tile_swz128(row)) * 8);
        }
    // transposing reads: within a group of 16 lanes, lane 4 j + a supplies the address of elements 4 a' .. of row j
    // and receives, for column (lane % 16) of the group's 16 columns, the rows j = 0 .. 3.  Group g covers the
    // columns 32 dt + 16 (g & 1) .. + 15 and the rows 4 (g >> 1) .. + 3 (first read) and 8 more (second read).
    int tr_lo[DT], tr_hi[DT];
    {
        const int g = lane >> 4, r = lane & 15, jj = r >> 2, aa = r & 3;
        const int row = 4 * (g >> 1) + jj, x = 2 * (g & 1) + (aa >> 1);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            tr_lo[dt] = row * D + (((4 * dt + x) ^ tile_swz128(row)) * 8) + (aa & 1) * 4;
            tr_hi[dt] = (row + 8) * D + (((4 * dt + x) ^ tile_swz128(row + 8)) * 8) + (aa & 1) * 4;
        }
    }
    auto tr_frag = [&](const T* tile, int g16, int dt) {   // columns 32 dt .. + 31 x rows 16 g16 .. + 15 of the tile, as an A operand
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(tile + tr_lo[dt] + 16 * g16 * D));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(tile + tr_hi[dt] + 16 * g16 * D));
        return __builtin_bit_cast(v8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    };

    f32x16 acc_a[DT];     // dQ^T, dK^T or dV^T
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc_a[dt][r] = 0.f;
    float sum_lo = 0.f, sum_hi = 0.f;

    for (int t = t_lo; t < t_hi; ++t) {
        const int o0 = t * kBwdOther;
        __syncthreads();     // the previous tile's readers are done (and the LUT is written, first time round)
        fetch(t);
        stage(0);
        __syncthreads();
        const T* ta = ta2[0]; const T* tb = tb2[0];
        const float* rowstat = rowstat2[0];
        (void)rowstat;

        f32x16 s[NT], dp[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            // (dP starts at -delta: the matrix core subtracts it for free)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                f32x4 d4 = {delta_own, delta_own, delta_own, delta_own};
                if constexpr (KV) d4 = *reinterpret_cast<const f32x4*>(rowstat + kBwdOther + 32 * nt + 8 * r4 + 4 * hh);
#pragma unroll
                for (int e = 0; e < 4; ++e) { s[nt][4 * r4 + e] = 0.f; dp[nt][4 * r4 + e] = WANT_DS ? -d4[e] : 0.f; }
            }
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2) {
                s[nt] = H16::mfma(*reinterpret_cast<const v8*>(ta + row_off[nt][k2]), fa[k2], s[nt]);
                if constexpr (WANT_DS) dp[nt] = H16::mfma(*reinterpret_cast<const v8*>(tb + row_off[nt][k2]), fb[k2], dp[nt]);
            }
        }

        // wavefront-uniform tile classes: every pair at a saturated distance on one side (constant bias); every pair
        // visible (no per-element test)
        const int w_lo = own_base + wave * 32, w_hi = w_lo + 31;            // this wavefront's own rows
        // rel = j - (i + P): dq pass j in the tile, i own; dk/dv pass i in the tile, j own
        const int rel_min = KV ? w_lo - (o0 + kBwdOther - 1 + P) : o0 - (w_hi + P);
        const int rel_max = KV ? w_hi - (o0 + P) : o0 + kBwdOther - 1 - (w_lo + P);
        int side = 0;
        if (rel_max <= -sat) side = 1; else if (rel_min >= sat) side = 2;
        const bool all_visible = o0 + kBwdOther <= n_other && w_hi < n_own && (!CAUSAL || rel_max <= 0);
        const float c1 = p.c1;
        float tile_sum = 0.f;
        // Second stage, 16 rows of the tile at a time: probabilities and dS of this lane's eight pairs, rounded to
        // the input type, then the products that contract over those rows --
        //   dQ^T += K^T dS^T   /   dK^T += Q^T dS, dV^T += dO^T P
        // -- so that the matrix cores work on one group while the vector units form the next.
        auto second_stage = [&](auto check_c, auto lut_c) {
            constexpr bool CHECK = decltype(check_c)::value, LUT = decltype(lut_c)::value;
            const float bias_c = (has_bias && !LUT) ? lut_bias[side == 1 ? 0 : 2 * sat] : 0.f;
            // Table gradient around the diagonal (dq pass, LUT variants): dS summed per distance.  Pairs at one
            // distance lie on a diagonal of the (key, query) tile, and a lane half walks its keys in ascending order:
            // each lane adds its dS to a running value that then moves one lane up (one query further) with every
            // key, so a diagonal's sum travels with it.  A lane half holds the keys 8 k + 4 hh .. + 3: five lanes up
            // between two groups.  What leaves a half at lane 31 is added to the distance's word in LDS first, and
            // at the end of the tile every lane adds what it holds: some 190 single-lane atomic adds per tile and
            // wavefront instead of 2 048 (an LDS floating-point atomic handles about one lane per cycle).
            float diag = 0.f;
            int x_last = 0;
            (void)x_last;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    f32x8 ds8, pv8;
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
                        const int r4 = 2 * u + half;
                        const int ol0 = 32 * nt + 8 * r4 + 4 * hh;     // first of four consecutive rows of the other kind
                        f32x4 l4 = {lse2_own, lse2_own, lse2_own, lse2_own};
                        if constexpr (KV) l4 = *reinterpret_cast<const f32x4*>(rowstat + ol0);
                        f32x4 bl4;   // constant bias minus log-sum-exp
#pragma unroll
                        for (int e = 0; e < 4; ++e) bl4[e] = bias_c - l4[e];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int r = 4 * r4 + e, ol = ol0 + e;
                            const int i = KV ? o0 + ol : own_row, j = KV ? own_row : o0 + ol;
                            const int rel = j - (i + P);
                            int x = 0;
                            float bias2 = bias_c;
                            if constexpr (LUT) {
                                x = min(max(rel, -sat), sat) + sat;
                                bias2 = lut_bias[x];
                            }
                            float pv = LUT ? __builtin_amdgcn_exp2f(__builtin_fmaf(c1, s[nt][r], bias2) - l4[e])
                                           : __builtin_amdgcn_exp2f(__builtin_fmaf(c1, s[nt][r], bl4[e]));
                            if constexpr (CHECK) {
                                const bool valid = i < M && j < N && (!CAUSAL || rel <= 0);
                                pv = valid ? pv : 0.f;
                            }
                            const float ds = pv * dp[nt][r];
                            pv8[4 * half + e] = pv;
                            ds8[4 * half + e] = ds;
                            if constexpr (!KV) {
                                // table gradient (no test for a table here: a branch per element would cut the
                                // loop into pieces; without one the sum is simply not used, and the LUT variants
                                // run only with one).  Per clamped distance: neighbouring lanes hold neighbouring
                                // distances, so the adds of one instruction go to different words; a pair that
                                // is not visible adds 0.
                                if constexpr (!LUT) {
                                    tile_sum += ds;
                                } else {
                                    diag += ds;      // (a pair that is not visible adds 0)
                                    x_last = x;
                                    const bool last_of_tile = nt == NT - 1 && u == 1 && half == 1 && e == 3;
                                    if (!last_of_tile) {
                                        const int out_from = e == 3 ? 27 : 31;     // lanes whose value leaves the half
                                        if (lr >= out_from) { atomicAdd(&hist_rel[x], diag); diag = 0.f; }
#pragma unroll
                                        for (int sh = 0; sh < (e == 3 ? 5 : 1); ++sh)
                                            diag = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(diag), 0x138, 0xf, 0xf, true));
                                    }
                                }
                            }
                        }
                    }
                    if constexpr (WANT_DS) {
                        const v8 dsb = __builtin_convertvector(ds8, v8);
#pragma unroll
                        for (int dt = 0; dt < DT; ++dt)
                            acc_a[dt] = H16::mfma(tr_frag(ta, 2 * nt + u, dt), dsb, acc_a[dt]);
                    }
                    if constexpr (WANT_DV) {
                        const v8 pb = __builtin_convertvector(pv8, v8);
#pragma unroll
                        for (int dt = 0; dt < DT; ++dt)
                            acc_a[dt] = H16::mfma(tr_frag(tb, 2 * nt + u, dt), pb, acc_a[dt]);
                    }
                }
            if constexpr (!KV && LUT) atomicAdd(&hist_rel[x_last], diag);
        };
        const bool use_lut = has_bias && side == 0;
        if (all_visible && !use_lut) second_stage(std::false_type{}, std::false_type{});
        else if (all_visible) second_stage(std::false_type{}, std::true_type{});
        else if (!use_lut) second_stage(std::true_type{}, std::false_type{});
        else second_stage(std::true_type{}, std::true_type{});
        if (side == 1) sum_lo += tile_sum; else if (side == 2) sum_hi += tile_sum;
    }

    const float scale = WANT_DV ? 1.0f : p.c1 * 0.6931471805599453f;     // d score / d (q . k), natural units; dv has none
    if (own_ok) {
        T* oa = PASS == 0 ? reinterpret_cast<T*>(p.dq) + (int64_t)b * p.dq_sb + (int64_t)h * p.dq_sh + (q_first + own_row) * p.dq_sr
              : PASS == 2 ? reinterpret_cast<T*>(p.dk) + (int64_t)b * p.dk_sb + (int64_t)h * p.dk_sh + (k_first + own_row) * p.dk_sr
                          : reinterpret_cast<T*>(p.dv) + (int64_t)b * p.dv_sb + (int64_t)h * p.dv_sh + (k_first + own_row) * p.dv_sr;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d0 = 32 * dt + 8 * g + 4 * hh;
                store4(oa + d0, f32x4{acc_a[dt][4 * g] * scale, acc_a[dt][4 * g + 1] * scale,
                                      acc_a[dt][4 * g + 2] * scale, acc_a[dt][4 * g + 3] * scale});
            }
    }
    if constexpr (!KV) {
        if (has_bias && p.dtable != nullptr) {
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                sum_lo += __shfl_xor(sum_lo, off, 64);
                sum_hi += __shfl_xor(sum_hi, off, 64);
            }
            if (lane == 0) {
                if (sum_lo != 0.f) atomicAdd(&hist[lut_bucket[0]], sum_lo);
                if (sum_hi != 0.f) atomicAdd(&hist[lut_bucket[2 * sat]], sum_hi);
            }
            __syncthreads();
            for (int x = tid; x <= 2 * sat; x += kBwdThreads)     // distances -> buckets
                if (hist_rel[x] != 0.f) atomicAdd(&hist[lut_bucket[x]], hist_rel[x]);
            __syncthreads();
            for (int x = tid; x < p.n_buckets; x += kBwdThreads)
                if (hist[x] != 0.f) atomicAdd(&p.dtable[(int64_t)x * p.H + h], hist[x]);
        }
    }
}


template <typename T, int D>
hipError_t launch_bwd_d(const BwdParams& p, bool causal, hipStream_t stream) {
    const int64_t rows = p.cu_q != nullptr ? (int64_t)p.total_q * p.H : (int64_t)p.B * p.H * p.M;
    hipLaunchKernelGGL((bwd_rows_kernel<T, D>), dim3((unsigned)((rows + RowsGeom<T, D>::ROWS - 1) / RowsGeom<T, D>::ROWS)), dim3(256), 0, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const dim3 gq((p.M + kBwdOwn - 1) / kBwdOwn, p.H, p.B), gk((p.N + kBwdOwn - 1) / kBwdOwn, p.H, p.B);
    if constexpr (sizeof(T) == 2 && D == 64) {
        if (p.fp32_math == 0) {
            if (causal) {
                const dim3 cq(p.H, p.B, gq.x), ck(p.H, p.B, gk.x);
                hipLaunchKernelGGL((bwd16_kernel<T, true, false>), cq, dim3(kBwdThreads), 0, stream, p);
                if (p.N > 0) hipLaunchKernelGGL((bwd16_kernel<T, true, true>), ck, dim3(kBwdThreads), 0, stream, p);
            } else {
                hipLaunchKernelGGL((bwd16_kernel<T, false, false>), gq, dim3(kBwdThreads), 0, stream, p);
                if (p.N > 0) hipLaunchKernelGGL((bwd16_kernel<T, false, true>), gk, dim3(kBwdThreads), 0, stream, p);
            }
            return hipGetLastError();
        }
    }
    if (causal) {
        hipLaunchKernelGGL((bwd_kernel<T, D, true, false>), gq, dim3(kBwdThreads), 0, stream, p);
        if (p.N > 0) hipLaunchKernelGGL((bwd_kernel<T, D, true, true>), gk, dim3(kBwdThreads), 0, stream, p);
    } else {
        hipLaunchKernelGGL((bwd_kernel<T, D, false, false>), gq, dim3(kBwdThreads), 0, stream, p);
        if (p.N > 0) hipLaunchKernelGGL((bwd_kernel<T, D, false, true>), gk, dim3(kBwdThreads), 0, stream, p);
    }
    return hipGetLastError();
}

// head_dim 128, 16-bit tensors: row statistics, then one pass per gradient
template <typename T>
hipError_t launch_bwd_d128(const BwdParams& p, bool causal, hipStream_t stream) {
    if constexpr (sizeof(T) != 2) {
        return hipErrorInvalidValue;
    } else {
        if (p.fp32_math != 0) return hipErrorInvalidValue;     // (the fp32 kernels hold a row's head_dim in registers: up to 64)
        const int64_t rows = p.cu_q != nullptr ? (int64_t)p.total_q * p.H : (int64_t)p.B * p.H * p.M;
        hipLaunchKernelGGL((bwd_rows_kernel<T, 128>), dim3((unsigned)((rows + RowsGeom<T, 128>::ROWS - 1) / RowsGeom<T, 128>::ROWS)), dim3(256), 0, stream, p);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        const unsigned nq = (p.M + kBwdOwn - 1) / kBwdOwn, nk = (p.N + kBwdOwn - 1) / kBwdOwn;
        if (causal) {
            const dim3 cq(p.H, p.B, nq), ck(p.H, p.B, nk);
            hipLaunchKernelGGL((bwd16_d128_kernel<T, true, 0>), cq, dim3(kBwdThreads), 0, stream, p);
            if (p.N > 0) {
                hipLaunchKernelGGL((bwd16_d128_kernel<T, true, 2>), ck, dim3(kBwdThreads), 0, stream, p);
                hipLaunchKernelGGL((bwd16_d128_kernel<T, true, 3>), ck, dim3(kBwdThreads), 0, stream, p);
            }
        } else {
            const dim3 gq(nq, p.H, p.B), gk(nk, p.H, p.B);
            hipLaunchKernelGGL((bwd16_d128_kernel<T, false, 0>), gq, dim3(kBwdThreads), 0, stream, p);
            if (p.N > 0) {
                hipLaunchKernelGGL((bwd16_d128_kernel<T, false, 2>), gk, dim3(kBwdThreads), 0, stream, p);
                hipLaunchKernelGGL((bwd16_d128_kernel<T, false, 3>), gk, dim3(kBwdThreads), 0, stream, p);
            }
        }
        return hipGetLastError();
    }
}

template <typename T>
hipError_t launch_bwd_t(const BwdParams& p, int D, bool causal, hipStream_t s) {
    switch (D) {
        case 128: return launch_bwd_d128<T>(p, causal, s);
        case 16: return launch_bwd_d<T, 16>(p, causal, s);
        case 32: return launch_bwd_d<T, 32>(p, causal, s);
        case 64: return launch_bwd_d<T, 64>(p, causal, s);
    }
    return hipErrorInvalidValue;
}

}  // namespace

hipError_t launch_bwd_dense(const BwdParams& p, int dtype, int D, bool causal, hipStream_t stream) {
    if (dtype == T5A_BF16) return launch_bwd_t<__bf16>(p, D, causal, stream);
    if (dtype == T5A_F16) return launch_bwd_t<_Float16>(p, D, causal, stream);
    if (dtype == T5A_F32) return launch_bwd_t<float>(p, D, causal, stream);
    return hipErrorInvalidValue;
}

}  // namespace t5a
