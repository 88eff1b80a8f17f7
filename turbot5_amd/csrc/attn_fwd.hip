// Fused-bias flash attention forward for gfx950 (MI355X).
//
// One kernel template serves the dense, packed (cu_seqlens), local-window,
// block+global and transient-global forwards.  A workgroup of four wavefronts
// owns 128 query rows (32 per wavefront) of one (batch, head) and walks over
// at most two key segments in tiles of 64 keys.  Per tile:
//
//   S^T = K Q^T      32x32 MFMA with K rows as the A operand, so that every
//                    lane owns ONE query column and 16 keys per 32x32 block:
//                    the softmax row reductions stay inside the lane, with one
//                    cross-half exchange per tile.
//   P   = exp2(..)   online softmax in base 2, running max / sum per lane.
//   O^T += V^T P^T   the S^T accumulators are already laid out as the B
//                    operand (for 16-bit types after a key permutation that is
//                    baked into the LDS layout of V^T), so P stays in registers.
//
// 16-bit inputs (bf16, fp16) use v_mfma_f32_32x32x16; K tiles sit row-major in
// LDS, V tiles transposed (head_dim x keys), both with an XOR swizzle on
// 16-byte chunks.  fp32 inputs use v_mfma_f32_32x32x2_f32 (one float per lane
// and operand) with K and V row-major and P kept in fp32.  Tiles are double
// buffered and filled from registers that were loaded from HBM during the
// previous tile's math.
//
// The T5 relative-position bias is not materialised.  Each workgroup expands
// its head's column of the (num_buckets, H) table into a distance-indexed LUT
// in LDS covering [-sat, sat] (sat = distance at which the buckets saturate).
// Key tiles whose distances are all beyond saturation take the FAST path where
// the bias is one scalar folded into the exp2 argument; only tiles near the
// diagonal (or needing a mask) take the GENERAL path with per-element lookups.
//
// Sparsity patterns are tile skipping: the key segments of a work item are
// computed from integer positions; nothing outside them is loaded.
#include "t5a_internal.h"

namespace t5a {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Elem;
template <> struct Elem<__bf16> {
    using v8 = bf16x8; using v4 = bf16x4;
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <> struct Elem<_Float16> {
    using v8 = f16x8; using v4 = f16x4;
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};
template <> struct Elem<float> {
    using v8 = float; using v4 = f32x4;   // operands of the fp32 MFMA are one float per lane
    static __device__ __forceinline__ f32x16 mfma(float a, float b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
    }
};

constexpr int BM = 128;      // query rows per workgroup
constexpr int BN = 64;       // keys per tile
constexpr int NTHREADS = 256;
constexpr int NT = BN / 32;  // 32-key blocks per tile
constexpr float kNegBig = -1.0e30f;

__device__ __forceinline__ int bucket_of(const BucketSpec& s, int rel) {
    int out = 0, d;
    if (s.bidirectional) { out = rel > 0 ? s.nb : 0; d = rel < 0 ? -rel : rel; }
    else { d = rel < 0 ? -rel : 0; }
    if (d < s.max_exact) return out + d;
    int b = s.max_exact;
    for (int t = 0; t < s.n_thr; ++t) b += (d >= s.thr[t]) ? 1 : 0;
    return out + b;
}

__device__ __forceinline__ float load_table(const void* table, int dtype, int64_t off) {
    if (dtype == T5A_F32) return reinterpret_cast<const float*>(table)[off];
    if (dtype == T5A_BF16) return static_cast<float>(reinterpret_cast<const __bf16*>(table)[off]);
    return static_cast<float>(reinterpret_cast<const _Float16*>(table)[off]);
}

__device__ __forceinline__ float xhalf_max(float x) { return fmaxf(x, __shfl_xor(x, 32)); }
__device__ __forceinline__ float xhalf_sum(float x) { return x + __shfl_xor(x, 32); }

template <typename T, int D>
struct Geometry {
    static constexpr bool F32 = sizeof(T) == 4;
    static constexpr int EPC = 16 / sizeof(T);         // elements per 16-byte chunk
    static constexpr int KS = F32 ? D / 2 : D / 16;    // k-steps of the S^T product
    static constexpr int DT = (D + 31) / 32;           // 32-row blocks of O^T
    static constexpr int VROWS = DT * 32;
    static constexpr int CH = D / EPC;                 // 16-byte chunks per K/V row
    static constexpr int SW = CH < 8 ? CH : 8;
    static constexpr int K_CHUNKS = BN * CH;
    static constexpr int K_PER_T = (K_CHUNKS + NTHREADS - 1) / NTHREADS;
    // 16-bit: V is staged as units of 4 keys x 4 dims and transposed; fp32: row-major chunks
    static constexpr int V_UNITS = F32 ? K_CHUNKS : (BN / 4) * (D / 4);
    static constexpr int V_PER_T = (V_UNITS + NTHREADS - 1) / NTHREADS;
    static constexpr int KSTR = F32 ? D + 1 : D;       // fp32 K rows padded by one float (bank spread)
    static constexpr int K_TILE = BN * KSTR;
    static constexpr int V_TILE = VROWS * BN;          // 16-bit: V^T (dim x key); fp32: V (key x VROWS)
    static constexpr size_t kTileBytes = (size_t)(2 * K_TILE + 2 * V_TILE) * sizeof(T);
};

template <typename T, int D, int MODE, bool CAUSAL>
__global__ __launch_bounds__(NTHREADS) void fwd_kernel(const FwdParams p) {
    using E = Elem<T>;
    using G = Geometry<T, D>;
    using v8 = typename E::v8;
    using v4 = typename E::v4;
    constexpr bool F32 = G::F32;
    constexpr int EPC = G::EPC, KS = G::KS, DT = G::DT, VROWS = G::VROWS, CH = G::CH, SW = G::SW;
    constexpr int K_CHUNKS = G::K_CHUNKS, K_PER_T = G::K_PER_T, V_UNITS = G::V_UNITS, V_PER_T = G::V_PER_T;
    constexpr int KSTR = G::KSTR, K_TILE = G::K_TILE, V_TILE = G::V_TILE;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    T* Vs = reinterpret_cast<T*>(smem);         // [2][V_TILE]
    T* Ks = Vs + 2 * V_TILE;                    // [2][K_TILE]
    float* lut = reinterpret_cast<float*>(Ks + 2 * K_TILE);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int lr = lane & 31;
    const int hh = lane >> 5;

    // ---------------------------------------------------------------- work item
    // Consecutive workgroup ids go round-robin over the 8 XCDs; give each XCD a
    // contiguous slice of the item list so that the q tiles of one (batch, head)
    // share that XCD's L2 copy of K/V.
    const int per_xcd = (p.total_items + 7) >> 3;
    int w = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (w >= p.total_items) return;

    int b = 0, h = 0, qt = 0, Mseq = 0, Nseq = 0;
    int64_t q_off, k_off, v_off, o_off, lse_off;
    if (MODE == kDense && p.cu_q != nullptr) {
        // packed batch: find (sequence, head, tile) by walking cu_seqlens
        int acc = 0, nt_b = 0, qs = 0;
        b = -1;
        for (int bb = 0; bb < p.B; ++bb) {
            qs = p.cu_q[bb];
            const int len = p.cu_q[bb + 1] - qs;
            nt_b = (len + BM - 1) / BM;
            const int cnt = nt_b * p.H;
            if (w < acc + cnt) { b = bb; Mseq = len; w -= acc; break; }
            acc += cnt;
        }
        if (b < 0) return;
        h = w / nt_b;
        qt = w - h * nt_b;
        if (CAUSAL) qt = nt_b - 1 - qt;
        const int ks = p.cu_k[b];
        Nseq = p.cu_k[b + 1] - ks;
        q_off = (int64_t)qs * p.q_sr + (int64_t)h * p.q_sh;
        o_off = (int64_t)qs * p.o_sr + (int64_t)h * p.o_sh;
        k_off = (int64_t)ks * p.k_sr + (int64_t)h * p.k_sh;
        v_off = (int64_t)ks * p.v_sr + (int64_t)h * p.v_sh;
        lse_off = (int64_t)qs * p.lse_sr + (int64_t)h * p.lse_sh;
    } else {
        const int bh = w / p.tiles_per_seq;
        qt = w - bh * p.tiles_per_seq;
        if (CAUSAL) qt = p.tiles_per_seq - 1 - qt;
        b = bh / p.H;
        h = bh - b * p.H;
        Mseq = p.M;
        Nseq = p.N;
        q_off = (int64_t)b * p.q_sb + (int64_t)h * p.q_sh;
        o_off = (int64_t)b * p.o_sb + (int64_t)h * p.o_sh;
        k_off = (int64_t)b * p.k_sb + (int64_t)h * p.k_sh;
        v_off = (int64_t)b * p.v_sb + (int64_t)h * p.v_sh;
        lse_off = (int64_t)b * p.lse_sb + (int64_t)h * p.lse_sh;
    }
    const T* qp = reinterpret_cast<const T*>(p.q) + q_off;
    T* op = reinterpret_cast<T*>(p.o) + o_off;

    // query rows of this tile: [i0, row_end); rows below row_lo are computed but not stored
    int i0, row_end, row_lo = 0, blk = 0;
    if (MODE == kBlock) {
        const int tpb = (p.block_len + BM - 1) / BM;
        blk = qt / tpb;
        i0 = blk * p.block_len + (qt - blk * tpb) * BM;
        row_end = min(Mseq, (blk + 1) * p.block_len);
        row_lo = p.aux;   // the first G rows belong to the global-query pass
    } else {
        i0 = qt * BM;
        row_end = Mseq;
    }
    const int P = p.align_end ? Nseq - Mseq : 0;

    // ---------------------------------------------------------------- key segments
    // A segment is a key range [start, end) of one K/V tensor.  Keys at or past
    // lend are read as zero vectors (they still count when below end).  The key
    // position is its index j; the query position depends on the kind:
    //   0: i + P     1: i % block_len + G (block pattern, global keys)     2: i / aux (side tokens)
    const T* seg_k[2]; const T* seg_v[2];
    int64_t seg_ksr[2], seg_vsr[2];
    int seg_start[2], seg_end[2], seg_lend[2], seg_kind[2], seg_win[2];
    int nseg = 1;
    seg_k[0] = reinterpret_cast<const T*>(p.k) + k_off;
    seg_v[0] = reinterpret_cast<const T*>(p.v) + v_off;
    seg_ksr[0] = p.k_sr; seg_vsr[0] = p.v_sr;
    seg_k[1] = seg_k[0]; seg_v[1] = seg_v[0]; seg_ksr[1] = p.k_sr; seg_vsr[1] = p.v_sr;
    seg_start[0] = 0; seg_end[0] = 0;
    seg_start[1] = seg_end[1] = seg_lend[1] = 0; seg_kind[1] = 0; seg_win[1] = 0;
    seg_kind[0] = 0; seg_win[0] = 0; seg_lend[0] = Nseq;
    if (MODE == kDense) {
        seg_end[0] = CAUSAL ? max(0, min(Nseq, i0 + BM + P)) : Nseq;
    } else if (MODE == kLocal || MODE == kTGlobal) {
        seg_start[0] = max(0, i0 - p.block_len + 1);
        seg_end[0] = min(Nseq, min(i0 + BM, Mseq) - 1 + p.block_len);
        seg_win[0] = 1;
        if (MODE == kTGlobal) {
            nseg = 2;
            seg_k[1] = reinterpret_cast<const T*>(p.side_k) + (int64_t)b * p.sk_sb + (int64_t)h * p.sk_sh;
            seg_v[1] = reinterpret_cast<const T*>(p.side_v) + (int64_t)b * p.sv_sb + (int64_t)h * p.sv_sh;
            seg_ksr[1] = p.sk_sr; seg_vsr[1] = p.sv_sr;
            seg_end[1] = p.n_side; seg_lend[1] = p.n_side; seg_kind[1] = 2;
        }
    } else {  // kBlock
        nseg = 2;
        seg_end[0] = p.aux; seg_kind[0] = 1;
        seg_start[1] = blk * p.block_len;
        seg_end[1] = blk == 0 ? p.block_len - p.aux : (blk + 1) * p.block_len;
        seg_lend[1] = Nseq;
    }
    int seg_nt[2];
    seg_nt[0] = max(0, seg_end[0] - seg_start[0] + BN - 1) / BN;
    seg_nt[1] = nseg > 1 ? max(0, seg_end[1] - seg_start[1] + BN - 1) / BN : 0;
    const int ntiles = seg_nt[0] + seg_nt[1];

    // ---------------------------------------------------------------- bias LUT
    const bool has_bias = p.table != nullptr;
    const int sat = p.bs.sat;
    if (has_bias) {
        const float log2e = 1.4426950408889634f;
        for (int idx = tid; idx <= 2 * sat; idx += NTHREADS) {
            const int bk = bucket_of(p.bs, idx - sat);
            lut[idx] = load_table(p.table, p.table_dtype, (int64_t)bk * p.t_sbucket + (int64_t)h * p.t_shead) * log2e;
        }
    }
    if (D < 32) {  // the part of V past head_dim feeds the MFMA: keep it zero
        for (int idx = tid; idx < 2 * V_TILE; idx += NTHREADS) Vs[idx] = (T)0.0f;
    }
    __syncthreads();
    const float c_neg = has_bias ? lut[0] : 0.f;
    const float c_pos = has_bias ? lut[2 * sat] : 0.f;

    // ---------------------------------------------------------------- Q fragments
    const int iw0 = i0 + wave * 32;      // first row of this wavefront
    const int iw1 = iw0 + 31;
    const int irow = iw0 + lr;           // this lane's query row
    const bool row_ok = irow < row_end;
    v8 qf[KS];
    if constexpr (F32) {
#pragma unroll
        for (int c = 0; c < D / 4; ++c) {
            f32x4 x = {0.f, 0.f, 0.f, 0.f};
            if (row_ok) x = *reinterpret_cast<const f32x4*>(qp + (int64_t)irow * p.q_sr + 4 * c);
            qf[2 * c] = hh ? x[1] : x[0];
            qf[2 * c + 1] = hh ? x[3] : x[2];
        }
    } else {
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            if (row_ok) qf[s] = *reinterpret_cast<const v8*>(qp + (int64_t)irow * p.q_sr + 16 * s + 8 * hh);
            else { for (int x = 0; x < 8; ++x) qf[s][x] = (T)0.0f; }
        }
    }

    // ---------------------------------------------------------------- tile staging
    uint4 kreg[K_PER_T];
    uint4 vreg[F32 ? V_PER_T : 2 * V_PER_T];   // 16-bit: four 8-byte rows per unit

    auto tile_of = [&](int t, int& sg, int& j0) {
        sg = t >= seg_nt[0] ? 1 : 0;
        j0 = seg_start[sg] + (t - (sg ? seg_nt[0] : 0)) * BN;
    };
    auto load_tile = [&](int t) {
        int sg, j0; tile_of(t, sg, j0);
        const T* kp = seg_k[sg]; const T* vp = seg_v[sg];
        const int64_t ksr = seg_ksr[sg], vsr = seg_vsr[sg];
        const int lend = min(seg_lend[sg], seg_end[sg]);
#pragma unroll
        for (int c = 0; c < K_PER_T; ++c) {
            const int idx = tid + c * NTHREADS;
            const int row = idx / CH, ch = idx % CH;
            const int j = j0 + row;
            kreg[c] = make_uint4(0, 0, 0, 0);
            if (idx < K_CHUNKS && j < lend) kreg[c] = *reinterpret_cast<const uint4*>(kp + (int64_t)j * ksr + ch * EPC);
        }
        if constexpr (F32) {
#pragma unroll
            for (int c = 0; c < V_PER_T; ++c) {
                const int idx = tid + c * NTHREADS;
                const int row = idx / CH, ch = idx % CH;
                const int j = j0 + row;
                vreg[c] = make_uint4(0, 0, 0, 0);
                if (idx < V_UNITS && j < lend) vreg[c] = *reinterpret_cast<const uint4*>(vp + (int64_t)j * vsr + ch * EPC);
            }
        } else {
#pragma unroll
            for (int u = 0; u < V_PER_T; ++u) {
                const int idx = tid + u * NTHREADS;
                const int dg = idx % (D / 4), kg = idx / (D / 4);
                uint2 r[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int j = j0 + 4 * kg + i;
                    r[i] = make_uint2(0, 0);
                    if (idx < V_UNITS && j < lend) r[i] = *reinterpret_cast<const uint2*>(vp + (int64_t)j * vsr + 4 * dg);
                }
                vreg[2 * u] = make_uint4(r[0].x, r[0].y, r[1].x, r[1].y);
                vreg[2 * u + 1] = make_uint4(r[2].x, r[2].y, r[3].x, r[3].y);
            }
        }
    };
    auto store_tile = [&](int buf) {
        T* ks = Ks + buf * K_TILE;
        T* vs = Vs + buf * V_TILE;
        if constexpr (F32) {
#pragma unroll
            for (int c = 0; c < K_PER_T; ++c) {
                const int idx = tid + c * NTHREADS;
                const int row = idx / CH, ch = idx % CH;
                if (idx < K_CHUNKS) {
                    float* dst = reinterpret_cast<float*>(ks) + row * KSTR + ch * 4;
                    dst[0] = __uint_as_float(kreg[c].x); dst[1] = __uint_as_float(kreg[c].y);
                    dst[2] = __uint_as_float(kreg[c].z); dst[3] = __uint_as_float(kreg[c].w);
                }
            }
#pragma unroll
            for (int c = 0; c < V_PER_T; ++c) {
                const int idx = tid + c * NTHREADS;
                const int row = idx / CH, ch = idx % CH;
                if (idx < V_UNITS) *reinterpret_cast<uint4*>(vs + row * VROWS + ch * 4) = vreg[c];
            }
        } else {
#pragma unroll
            for (int c = 0; c < K_PER_T; ++c) {
                const int idx = tid + c * NTHREADS;
                const int row = idx / CH, ch = idx % CH;
                if (idx < K_CHUNKS)
                    *reinterpret_cast<uint4*>(ks + row * D + ((ch ^ (row & (SW - 1))) * 8)) = kreg[c];
            }
#pragma unroll
            for (int u = 0; u < V_PER_T; ++u) {
                const int idx = tid + u * NTHREADS;
                const int dg = idx % (D / 4), kg = idx / (D / 4);
                if (idx < V_UNITS) {
                    // 4 keys x 4 dims -> 4 dims x 4 keys.  Key slots 4..7 and 8..11 of every 16 are
                    // swapped so that a lane's eight P values line up with one 16-byte V^T read.
                    const int pk = (kg & ~3) | ((kg & 1) << 1) | ((kg >> 1) & 1);
                    const uint4 a = vreg[2 * u], c2 = vreg[2 * u + 1];   // keys (0,1) and (2,3): {x,y | z,w}
                    uint2 y[4];
                    y[0] = make_uint2((a.x & 0xffffu) | (a.z << 16), (c2.x & 0xffffu) | (c2.z << 16));
                    y[1] = make_uint2((a.x >> 16) | (a.z & 0xffff0000u), (c2.x >> 16) | (c2.z & 0xffff0000u));
                    y[2] = make_uint2((a.y & 0xffffu) | (a.w << 16), (c2.y & 0xffffu) | (c2.w << 16));
                    y[3] = make_uint2((a.y >> 16) | (a.w & 0xffff0000u), (c2.y >> 16) | (c2.w & 0xffff0000u));
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const int d = 4 * dg + c;
                        *reinterpret_cast<uint2*>(vs + d * BN + (((pk >> 1) ^ (d & 7)) * 8) + (pk & 1) * 4) = y[c];
                    }
                }
            }
        }
    };

    // ---------------------------------------------------------------- running state
    f32x16 ot[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) ot[dt][r] = 0.f;
    float m_run = kNegBig;   // running max (base-2 units); finite, so exp2(m_run - m_new) is never NaN
    float l_run = 0.f;       // running sum over this lane's half of the keys

    if (ntiles > 0) { load_tile(0); store_tile(0); }
    __syncthreads();

    for (int t = 0; t < ntiles; ++t) {
        const int buf = t & 1;
        if (t + 1 < ntiles) load_tile(t + 1);

        int sg, j0; tile_of(t, sg, j0);
        const int kind = seg_kind[sg];
        const int s_end = seg_end[sg];
        const bool win = seg_win[sg] != 0;
        // query positions of this lane / this wavefront in the segment's bias geometry
        int qpos, qlo, qhi;
        if (kind == 0) { qpos = irow + P; qlo = iw0 + P; qhi = iw1 + P; }
        else if (kind == 1) { qpos = irow % p.block_len + p.aux; qlo = iw0 % p.block_len + p.aux; qhi = qlo + 31; }
        else { qpos = irow / p.aux; qlo = iw0 / p.aux; qhi = iw1 / p.aux; }
        const int rel_min = j0 - qhi, rel_max = j0 + BN - 1 - qlo;

        bool skip = iw0 >= row_end;                      // wavefront without live rows
        if (CAUSAL) skip = skip || rel_min > 0;          // every key is in the future of every row
        if (win) skip = skip || (rel_max <= -p.block_len) || (rel_min >= p.block_len);

        if (!skip) {
            bool general = (j0 + BN > s_end) || !(p.c1 > 0.f);
            if (CAUSAL) general = general || (rel_max > 0);
            if (win) general = general || (rel_max >= p.block_len) || (rel_min <= -p.block_len);
            float cb = 0.f;
            if (has_bias) {
                if (rel_max <= -sat) cb = c_neg;
                else if (rel_min >= sat) cb = c_pos;
                else general = true;
            }

            // ---- S^T = K Q^T
            const T* ks = Ks + buf * K_TILE;
            f32x16 st[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
                for (int r = 0; r < 16; ++r) st[nt][r] = 0.f;
                const int row = 32 * nt + lr;
#pragma unroll
                for (int s = 0; s < KS; ++s) {
                    if constexpr (F32) {
                        st[nt] = E::mfma(ks[row * KSTR + 2 * s + hh], qf[s], st[nt]);
                    } else {
                        const v8 a = *reinterpret_cast<const v8*>(ks + row * D + (((2 * s + hh) ^ (row & (SW - 1))) * 8));
                        st[nt] = E::mfma(a, qf[s], st[nt]);
                    }
                }
            }

            // ---- online softmax (base 2)
            float m_new;
            float rsum = 0.f;
            if (!general) {
                float mx = st[0][0];
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) mx = fmaxf(mx, st[nt][r]);
                mx = xhalf_max(mx);
                m_new = fmaxf(m_run, fmaf(mx, p.c1, cb));
                const float off = cb - m_new;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const float e = __builtin_amdgcn_exp2f(fmaf(st[nt][r], p.c1, off));
                        st[nt][r] = e;
                        rsum += e;
                    }
            } else {
                float mx = -INFINITY;
                const int jl = j0 + 4 * hh;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int j = jl + 32 * nt + 8 * (r >> 2) + (r & 3);
                        const int rel = j - qpos;
                        float bias = 0.f;
                        if (has_bias) bias = lut[min(max(rel, -sat), sat) + sat];
                        float tt = fmaf(st[nt][r], p.c1, bias);
                        bool ok = j < s_end;
                        if (CAUSAL) ok = ok && rel <= 0;
                        if (win) ok = ok && rel < p.block_len && rel > -p.block_len;
                        tt = ok ? tt : -INFINITY;
                        st[nt][r] = tt;
                        mx = fmaxf(mx, tt);
                    }
                mx = xhalf_max(mx);
                m_new = fmaxf(m_run, mx);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const float e = __builtin_amdgcn_exp2f(st[nt][r] - m_new);
                        st[nt][r] = e;
                        rsum += e;
                    }
            }
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
            m_run = m_new;
            l_run = l_run * alpha + rsum;
            if (__any(alpha != 1.0f)) {
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) ot[dt][r] *= alpha;
            }

            // ---- O^T += V^T P^T
            const T* vs = Vs + buf * V_TILE;
            if constexpr (F32) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        // MFMA k-slot = lane half: half 0 feeds key 8g+t, half 1 key 8g+4+t
                        const int key = 32 * nt + 8 * (r >> 2) + 4 * hh + (r & 3);
#pragma unroll
                        for (int dt = 0; dt < DT; ++dt)
                            ot[dt] = E::mfma(vs[key * VROWS + 32 * dt + lr], st[nt][r], ot[dt]);
                    }
            } else {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int u = 0; u < 2; ++u) {
                        f32x8 pv;
#pragma unroll
                        for (int x = 0; x < 8; ++x) pv[x] = st[nt][8 * u + x];
                        const v8 pb = __builtin_convertvector(pv, v8);
#pragma unroll
                        for (int dt = 0; dt < DT; ++dt) {
                            const int d = 32 * dt + lr;
                            const v8 a = *reinterpret_cast<const v8*>(vs + d * BN + (((4 * nt + 2 * u + hh) ^ (d & 7)) * 8));
                            ot[dt] = E::mfma(a, pb, ot[dt]);
                        }
                    }
            }
        }

        if (t + 1 < ntiles) store_tile(buf ^ 1);
        __syncthreads();
    }

    // ---------------------------------------------------------------- epilogue
    const float l_tot = xhalf_sum(l_run);
    const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
    if (row_ok && irow >= row_lo) {
        T* orow = op + (int64_t)irow * p.o_sr;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d0 = 32 * dt + 8 * g + 4 * hh;
                if (d0 < D) {
                    f32x4 x;
#pragma unroll
                    for (int tt = 0; tt < 4; ++tt) x[tt] = ot[dt][4 * g + tt] * inv;
                    if constexpr (F32) *reinterpret_cast<f32x4*>(orow + d0) = x;
                    else *reinterpret_cast<v4*>(orow + d0) = __builtin_convertvector(x, v4);
                }
            }
        if (p.lse != nullptr && hh == 0) {
            const float ln2 = 0.6931471805599453f;
            p.lse[lse_off + (int64_t)irow * p.lse_sr] = l_tot > 0.f ? (m_run + __builtin_log2f(l_tot)) * ln2 : -INFINITY;
        }
    }
}

// ------------------------------------------------------------------------ launch
template <typename T, int D, int MODE, bool CAUSAL>
static hipError_t launch_one(const FwdParams& p, hipStream_t stream) {
    const size_t lut_bytes = p.table != nullptr ? (size_t)(2 * p.bs.sat + 1) * sizeof(float) : sizeof(float);
    const size_t smem = Geometry<T, D>::kTileBytes + lut_bytes;
    auto kern = fwd_kernel<T, D, MODE, CAUSAL>;
    if (smem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return e;
    }
    const unsigned grid = (unsigned)(((p.total_items + 7) / 8) * 8);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(NTHREADS), smem, stream, p);
    return hipGetLastError();
}

template <typename T, int D>
static hipError_t launch_mode(const FwdParams& p, int mode, bool causal, hipStream_t s) {
    switch (mode) {
        case kDense: return causal ? launch_one<T, D, kDense, true>(p, s) : launch_one<T, D, kDense, false>(p, s);
        case kLocal: return launch_one<T, D, kLocal, false>(p, s);
        case kBlock: return launch_one<T, D, kBlock, false>(p, s);
        case kTGlobal: return launch_one<T, D, kTGlobal, false>(p, s);
    }
    return hipErrorInvalidValue;
}

template <typename T>
static hipError_t launch_dim(const FwdParams& p, int D, int mode, bool causal, hipStream_t s) {
    switch (D) {
        case 16: return launch_mode<T, 16>(p, mode, causal, s);
        case 32: return launch_mode<T, 32>(p, mode, causal, s);
        case 64: return launch_mode<T, 64>(p, mode, causal, s);
        case 128: return launch_mode<T, 128>(p, mode, causal, s);
    }
    return hipErrorInvalidValue;
}

// One translation unit per element type (selected with -DT5A_UNIT_DTYPE=<t5a_dtype>) so the
// instantiations build in parallel.
#ifndef T5A_UNIT_DTYPE
#error "compile with -DT5A_UNIT_DTYPE=0 (bf16), 1 (fp32) or 2 (fp16)"
#endif
#if T5A_UNIT_DTYPE == 0
hipError_t launch_fwd_bf16(const FwdParams& p, int D, int mode, bool causal, hipStream_t s) { return launch_dim<__bf16>(p, D, mode, causal, s); }
#elif T5A_UNIT_DTYPE == 1
hipError_t launch_fwd_f32(const FwdParams& p, int D, int mode, bool causal, hipStream_t s) { return launch_dim<float>(p, D, mode, causal, s); }
#else
hipError_t launch_fwd_f16(const FwdParams& p, int D, int mode, bool causal, hipStream_t s) { return launch_dim<_Float16>(p, D, mode, causal, s); }
#endif

}  // namespace t5a
