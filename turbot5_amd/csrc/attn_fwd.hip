// Fused-bias flash attention forward for gfx950 (MI355X).
//
// One kernel template serves the dense, packed (cu_seqlens), local-window,
// block+global and transient-global forwards.  A workgroup of four wavefronts
// owns 128 query rows (32 per wavefront) of one (batch, head) and walks over
// at most two key segments in tiles of 64 keys (32 at head_dim 128).  Per tile:
//
//   S^T = K Q^T + C  32x32 MFMA with K rows as the A operand, so that every
//                    lane owns ONE query column and 16 keys per 32x32 block:
//                    the softmax row reductions stay inside the lane, with one
//                    cross-half exchange per tile.  Q is pre-multiplied by
//                    sm_scale*log2(e); the accumulator input C carries
//                    (bias - running max), so the MFMA result is directly the
//                    exp2 argument.
//   P   = exp2(S^T)  online softmax in base 2.  The running max is only raised
//                    when a tile exceeds it by more than 2^24 (2^14 for fp16;
//                    the sums and the output are normalised by the same stale
//                    max, so the result is unchanged), which keeps the rescale
//                    off the common path.
//   O^T += V^T P^T   the S^T accumulators are already laid out as the B
//                    operand (for 16-bit types after a key permutation that is
//                    baked into the LDS layout of V^T), so P stays in registers.
//
// 16-bit inputs (bf16, fp16) use v_mfma_f32_32x32x16.  At head_dim 64 and 128
// their K and V tiles are written into four-stage LDS rings by LDS-DMA buffer
// loads (no staging registers; rows past the end of a segment arrive as
// zeros), both row-major with an XOR swizzle on 16-byte chunks applied on the
// source side, and V is transposed on the way out with ds_read_b64_tr_b16.
// Other head dims stage through registers into double buffers, V transposed
// on the LDS write.  fp32 inputs use v_mfma_f32_32x32x2_f32 (one float per
// lane and operand) with K and V row-major and P kept in fp32.  The step for
// tile t overlaps three things: the softmax head of tile t, the S product of
// tile t+1 and the exp / PV product of tile t; runs of tiles that need neither
// skipping nor masking take an unrolled fast path with compile-time stages.
//
// The T5 relative-position bias is not materialised.  Each workgroup expands
// its head's column of the (num_buckets, H) table into a distance-indexed LUT
// in LDS covering the distances at which buckets still change (or fetches the
// finished image from a per-table buffer, lut.hip); for causal
// attention the LUT holds -inf for every future key, so the diagonal needs no
// separate mask.  Four copies of the LUT, shifted by 0..3 entries, let a lane
// fetch the biases of four consecutive keys with one aligned 16-byte read,
// straight into the MFMA accumulator input.  Key tiles whose distances are all
// beyond saturation use a per-lane constant instead.  Per-element masking is
// left to the few tiles that straddle the end of a segment or a window edge.
//
// Sparsity patterns are tile skipping: the key segments of a work item are
// computed from integer positions; nothing outside them is loaded.
#include <atomic>
#include <type_traits>

#include "t5a_internal.h"
#include "lut_device.h"

namespace t5a {

// Timeline of a work item, for measurements only (build with -DT5A_TRACE, `python -m turbot5_amd.build --trace`): the
// first thread of every workgroup of the bf16 kernels stamps the shader clock at a few points; t5a_trace_read copies
// the stamps out.  Slot 0: kernel entry, 1: first key/value and query requests issued, 2: the LUT barrier passed,
// 3: first score product formed (the tile loop starts), 4..: end of each q tile's tile loop and, for runs of q tiles,
// the start of the next one's.  The shipped library has none of this.
#if defined(T5A_TRACE) && T5A_UNIT_DTYPE == 0
constexpr int kTraceSlots = 16, kTraceItems = 4096;
__device__ unsigned long long t5a_trace_buf[kTraceItems * kTraceSlots];
#define T5A_STAMP(i) do { if (threadIdx.x == 0 && blockIdx.x < kTraceItems && (i) < kTraceSlots) \
        t5a_trace_buf[(size_t)blockIdx.x * kTraceSlots + (i)] = __builtin_readcyclecounter(); } while (0)
// ... and the time of the fast steps of wavefront 0, split at the step's barrier: slot 12 holds the cycles from a
// barrier's end to the next wait (the step's own work), slot 13 the cycles in the wait for the tile requests and the
// barrier, slot 14 the number of fast steps
#define T5A_PHASE_VARS unsigned long long tr_last = 0, tr_acc[2] = {0, 0}; unsigned tr_steps = 0
#define T5A_PHASE_START() do { tr_last = __builtin_readcyclecounter(); } while (0)
#define T5A_PHASE(k) do { const unsigned long long now_ = __builtin_readcyclecounter(); tr_acc[k] += now_ - tr_last; \
        tr_last = now_; tr_steps += (k); } while (0)
#define T5A_PHASE_STORE() do { if (threadIdx.x == 0 && blockIdx.x < kTraceItems) { \
        unsigned long long* s_ = t5a_trace_buf + (size_t)blockIdx.x * kTraceSlots; \
        s_[12] = tr_acc[0]; s_[13] = tr_acc[1]; s_[14] = tr_steps; } } while (0)
#else
#define T5A_STAMP(i)
#define T5A_PHASE_VARS
#define T5A_PHASE_START()
#define T5A_PHASE(k)
#define T5A_PHASE_STORE()
#endif

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

template <typename T> struct Elem;
template <> struct Elem<__bf16> {
    using v8 = bf16x8; using v4 = bf16x4; using v2 = bf16x2;
    static __device__ __forceinline__ float sum2(v2 x, float acc) {
        const bf16x2 one = {(__bf16)1.0f, (__bf16)1.0f};
        return __builtin_amdgcn_fdot2_f32_bf16(x, one, acc, false);
    }
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    // sum of the eight values as the matrix core will see them (rounded to bf16)
    static __device__ __forceinline__ float sum8(v8 x, float acc) {
        const bf16x2 one = {(__bf16)1.0f, (__bf16)1.0f};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const bf16x2 pr = {x[2 * i], x[2 * i + 1]};
            acc = __builtin_amdgcn_fdot2_f32_bf16(pr, one, acc, false);
        }
        return acc;
    }
    static __device__ __forceinline__ float sum4(v4 x, float acc) {
        const bf16x2 one = {(__bf16)1.0f, (__bf16)1.0f};
        acc = __builtin_amdgcn_fdot2_f32_bf16(bf16x2{x[0], x[1]}, one, acc, false);
        return __builtin_amdgcn_fdot2_f32_bf16(bf16x2{x[2], x[3]}, one, acc, false);
    }
};
template <> struct Elem<_Float16> {
    using v8 = f16x8; using v4 = f16x4; using v2 = f16x2;
    static __device__ __forceinline__ float sum2(v2 x, float acc) {
        const f16x2 one = {(_Float16)1.0f, (_Float16)1.0f};
        return __builtin_amdgcn_fdot2(x, one, acc, false);
    }
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float sum8(v8 x, float acc) {
        const f16x2 one = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const f16x2 pr = {x[2 * i], x[2 * i + 1]};
            acc = __builtin_amdgcn_fdot2(pr, one, acc, false);
        }
        return acc;
    }
    static __device__ __forceinline__ float sum4(v4 x, float acc) {
        const f16x2 one = {(_Float16)1.0f, (_Float16)1.0f};
        acc = __builtin_amdgcn_fdot2(f16x2{x[0], x[1]}, one, acc, false);
        return __builtin_amdgcn_fdot2(f16x2{x[2], x[3]}, one, acc, false);
    }
};
template <> struct Elem<float> {
    using v8 = float; using v4 = f32x4; using v2 = float;   // operands of the fp32 MFMA are one float per lane
    static __device__ __forceinline__ f32x16 mfma(float a, float b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
    }
};

constexpr int BM = 128;      // query rows per workgroup
// keys per tile: 64, or 32 at head_dim 128 (16-bit types), where the halved score registers and K/V
// tiles keep two workgroups per compute unit
template <typename T, int D> constexpr int tile_keys() { return sizeof(T) == 2 && D == 128 ? 32 : 64; }
constexpr int NTHREADS = 256;
// The running max of a row is raised only when a score exceeds it by more than this many powers of
// two, so rows whose maximum creeps up over many tiles rescale their accumulators a few times, not on
// every tile.  Probabilities then reach 2^limit: bf16 and fp32 have the exponent range for 2^24 (sums
// and outputs are fp32 and are divided by the row sum at the end); fp16 tops out at 65504, hence 2^14.
template <typename T> constexpr float raise_limit() { return sizeof(T) == 2 && !__is_same(T, __bf16) ? 14.0f : 24.0f; }
// a row whose first scores (base-2 units) are at least this keeps its running max at 0 (fp16 probabilities lose
// their precision below 2^-14, so fp16 rows start at their maximum unless it is close to 0)
template <typename T> constexpr float start_floor() { return sizeof(T) == 2 && !__is_same(T, __bf16) ? -8.0f : -100.0f; }
constexpr int kWorkgroupsPerCU = 2;
   // 72 KB of LDS and 256 registers per lane each

// table element from its bits (zero-extended for the 16-bit types)
__device__ __forceinline__ float table_value(unsigned raw, int dtype) {
    if (dtype == T5A_F32) return __uint_as_float(raw);
    if (dtype == T5A_BF16) return __uint_as_float(raw << 16);
    return static_cast<float>(__builtin_bit_cast(_Float16, (unsigned short)raw));
}

// max / sum over the two lanes (l, l^32) that share a query row; the swap
// exchanges the upper half of one operand with the lower half of the other, so
// combining both results is symmetric in the halves.
// NaN-propagating maximum (v_maximum3_f32): unlike fmaxf it needs no quieting of its inputs, which
// would cost one extra instruction per matrix-core result
__device__ __forceinline__ float max_ieee(float a, float b) { return __builtin_elementwise_maximum(a, b); }
__device__ __forceinline__ float xhalf_max(float x) {
    const unsigned u = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return max_ieee(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xhalf_sum(float x) {
    const unsigned u = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Raw buffer descriptor as four dwords (for the LDS-DMA loads issued from inline assembly)
__device__ __forceinline__ u32x4 make_rsrc_words(const void* base, unsigned bytes) {
    const unsigned long long a = reinterpret_cast<unsigned long long>(base);
    // the descriptor is wavefront-uniform; say so, so that it lives in scalar registers
    return u32x4{(unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)a),
                 (unsigned)__builtin_amdgcn_readfirstlane((int)((unsigned)(a >> 32) & 0xffffu)),
                 (unsigned)__builtin_amdgcn_readfirstlane((int)bytes), 0x00020000u};
}

// One LDS-DMA request: every lane fetches 16 bytes at its byte offset `voffset` of the buffer (zeros
// when out of range) and the wavefront's 1 KB lands at LDS byte address `lds_addr` in lane order.
// Issued from assembly so that the completion wait stays under the kernel's control: the step loop
// waits with an explicit vmcnt(N) before its barrier instead of draining every request.
__device__ __forceinline__ void lds_dma_16(u32x4 rs, unsigned lds_addr, int voffset) {
    // descriptor and LDS address are wavefront-uniform; readfirstlane is free when the value already
    // sits in scalar registers and makes the "s" constraints hold when the compiler kept it in vector ones
    const u32x4 rsrc = {(unsigned)__builtin_amdgcn_readfirstlane((int)rs[0]), (unsigned)__builtin_amdgcn_readfirstlane((int)rs[1]),
                        (unsigned)__builtin_amdgcn_readfirstlane((int)rs[2]), (unsigned)__builtin_amdgcn_readfirstlane((int)rs[3])};
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :: "s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voffset), "s"(rsrc) : "memory", "m0");
}

// one dword per lane: 256 consecutive bytes of LDS
__device__ __forceinline__ void lds_dma_4(u32x4 rs, unsigned lds_addr, int voffset) {
    const u32x4 rsrc = {(unsigned)__builtin_amdgcn_readfirstlane((int)rs[0]), (unsigned)__builtin_amdgcn_readfirstlane((int)rs[1]),
                        (unsigned)__builtin_amdgcn_readfirstlane((int)rs[2]), (unsigned)__builtin_amdgcn_readfirstlane((int)rs[3])};
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, 0 offen lds"
                 :: "s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voffset), "s"(rsrc) : "memory", "m0");
}

// Two requests that share one descriptor and one LDS base: the second carries an instruction offset of
// 1024, which moves both its global and its LDS address (and takes part in the range check), so the
// caller passes its lane offset minus 1024.
__device__ __forceinline__ void lds_dma_16x2(unsigned lo, unsigned hi, unsigned bytes, unsigned lds_addr, int voff0, int voff1) {
    const u32x4 rsrc = {(unsigned)__builtin_amdgcn_readfirstlane((int)lo), (unsigned)__builtin_amdgcn_readfirstlane((int)hi),
                        (unsigned)__builtin_amdgcn_readfirstlane((int)bytes), 0x00020000u};
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %3, 0 offen lds\n\t"
                 "buffer_load_dwordx4 %2, %3, 0 offen offset:1024 lds"
                 :: "s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voff0), "v"(voff1), "s"(rsrc) : "memory", "m0");
}

// ... with the descriptor as it is (four scalar registers that the caller keeps)
__device__ __forceinline__ void lds_dma_16x2(u32x4 rsrc, unsigned lds_addr, int voff0, int voff1) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %3, 0 offen lds\n\t"
                 "buffer_load_dwordx4 %2, %3, 0 offen offset:1024 lds"
                 :: "s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voff0), "v"(voff1), "s"(rsrc) : "memory", "m0");
}

// s_waitcnt vmcnt(N) alone (six-bit count: bits 3:0 and 15:14), the other counters left open
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0F70);
}

// barrier that orders LDS traffic only (lgkmcnt), leaving LDS-DMA requests in flight
__device__ __forceinline__ void barrier_lds_only() {
    __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

template <typename T, int D>
struct Geometry {
    static constexpr bool F32 = sizeof(T) == 4;
    static constexpr int BN = tile_keys<T, D>();
    static constexpr int NT = BN / 32;                  // 32-key blocks per tile
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
    // 16-bit types with 128- or 256-byte rows are staged by LDS-DMA (buffer loads that write LDS directly):
    // no staging registers, no vector ALU work, V stays row-major and is transposed on the LDS read.
    static constexpr bool DMA = !F32 && (D == 64 || D == 128);
    // one request of a wavefront moves 1 KB: RPS whole rows of LPR lanes each; a tile is SPW such slabs per wavefront
    static constexpr int LPR = D / 8 > 0 ? D / 8 : 1;
    static constexpr int RPS = 64 / LPR;
    static constexpr int SPW = BN * D / 2048 > 0 ? BN * D / 2048 : 1;
    static constexpr int NSK = DMA ? 4 : 2;             // LDS stages of K
    static constexpr int NSV = DMA ? 4 : 2;             // LDS stages of V
    static constexpr size_t kTileBytes = (size_t)(NSK * K_TILE + NSV * V_TILE) * sizeof(T);
    // XOR swizzles of the 16-byte chunk index (16-bit types).  The LDS has 64 four-byte banks, so
    // a 16-byte read is conflict free when 16 consecutive lanes (rows) cover one 256-byte bank line.
    static constexpr int RPL = 128 / D > 1 ? 128 / D : 1;   // K rows per bank line
    static __device__ __forceinline__ int kswz(int row) { return (row / RPL) % CH; }
    // V^T rows are always 128 bytes (64 keys); the extra term spreads the transposing writes
    static __device__ __forceinline__ int vswz(int d) { return ((d >> 1) & 7) ^ ((d >> 4) & 7); }
    // row-major V (LDS-DMA path): the transposing read of a half wavefront touches 4 consecutive
    // keys x 64 bytes; flipping the 64-byte halves of keys 2,3 (mod 4) spreads them over all banks
    // (rows of 256 bytes span all banks: there the four keys of a read go to four different quarters)
    static __device__ __forceinline__ int vrow_swz(int key) { return D == 128 ? (key & 3) << 2 : ((key >> 1) & 1) << 2; }
};

template <typename T, int D, int MODE, bool CAUSAL, bool EXACT>
__global__ __launch_bounds__(NTHREADS, (D >= 128 && sizeof(T) == 4) ? 1 : kWorkgroupsPerCU) void fwd_kernel(const FwdParams p) {
    using E = Elem<T>;
    using G = Geometry<T, D>;
    using v8 = typename E::v8;
    using v4 = typename E::v4;
    constexpr bool F32 = G::F32;
    constexpr int KS = G::KS, DT = G::DT, VROWS = G::VROWS, CH = G::CH;
    constexpr int K_CHUNKS = G::K_CHUNKS, K_PER_T = G::K_PER_T, V_UNITS = G::V_UNITS, V_PER_T = G::V_PER_T;
    constexpr int KSTR = G::KSTR, K_TILE = G::K_TILE, V_TILE = G::V_TILE;
    constexpr int ES = sizeof(T);
    constexpr int BN = G::BN, NT = G::NT;
    constexpr bool DENSE = MODE == kDense || MODE == kPacked;   // one key segment starting at key 0
    constexpr bool LOCAL = MODE == kLocal || MODE == kLocalWide;   // sliding window, one segment
    constexpr bool TG = MODE == kTGlobal || MODE == kTGlobalBits;   // sliding window and side tokens
    constexpr bool BLOCK = MODE == kBlock || MODE == kBlockBits;    // own block and leading global tokens
    // Sparse patterns, LDS-DMA geometries: a work item is a RUN of consecutive q tiles of one (batch, head).  Their
    // key tiles form one stream through the LDS rings (the requests for the next q tile's first tiles go out during
    // the last steps of the current one) and the distance LUT is built once per run; a q tile of a sparse pattern
    // is only a few steps long, so that its set-up would otherwise cost as much as its steps.
    constexpr bool RUNS = (MODE == kLocal || BLOCK) && G::DMA;
    constexpr bool CURSOR = MODE == kLocal && G::DMA;   // one segment: the requests of a run advance cursors
    // head_dim 64, 16-bit types: the Q rows are staged through LDS by LDS-DMA as well (see the prologue)
    constexpr bool QDMA = G::DMA && D == 64;
    // 16-bit inputs, two ways to apply sm_scale * log2(e).  Default: Q is pre-multiplied and rounded back to the
    // input type, which puts a relative error of 2^-9 (bf16; 2^-12 for fp16) on every term of a score and costs
    // nothing per tile.  exact_scale: the Q fragments stay as loaded, the accumulator input is divided by the
    // factor and the fp32 product is multiplied by it: one more vector multiply per score (about 11 % of the
    // run time at head_dim 64).  A template parameter: as a run-time switch it cost the default path 2-3 %.
    constexpr bool exact = EXACT && !F32;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    constexpr bool DMA = G::DMA;
    constexpr int NSK = G::NSK, NSV = G::NSV;
    T* Vs = reinterpret_cast<T*>(smem);         // [NSV][V_TILE]
    T* Ks = Vs + NSV * V_TILE;                  // [NSK][K_TILE]
    float* lut = reinterpret_cast<float*>(Ks + NSK * K_TILE);   // [4][4*quads]


    // ---------------------------------------------------------------- work item
    // Consecutive workgroup ids go round-robin over the 8 XCDs; give each XCD a
    // contiguous slice of the item list so that the q tiles of one (batch, head)
    // share that XCD's L2 copy of K/V.
    // Fetch the launch parameters every path needs in one go: left alone, the compiler loads each
    // field just before its first use, which puts a chain of dependent scalar-load round trips on the
    // critical path of every workgroup.
    asm volatile("" :: "s"(p.total_items), "s"(p.tiles_per_seq), "s"(p.H), "s"(p.M), "s"(p.N), "s"(p.nsplit), "s"(p.block_items),
                 "s"(p.align_end), "s"(p.c1), "s"(p.cu_q), "s"(p.plan), "s"(p.table), "s"(p.table_dtype));
    asm volatile("" :: "s"(p.q), "s"(p.k), "s"(p.v), "s"(p.o), "s"(p.q_sb), "s"(p.q_sh), "s"(p.q_sr),
                 "s"(p.k_sb), "s"(p.k_sh), "s"(p.k_sr), "s"(p.v_sb), "s"(p.v_sh), "s"(p.v_sr));
    asm volatile("" :: "s"(p.o_sb), "s"(p.o_sh), "s"(p.o_sr), "s"(p.t_sbucket), "s"(p.t_shead),
                 "s"(p.bs.bidirectional), "s"(p.bs.nb), "s"(p.bs.max_exact), "s"(p.bs.n_thr), "s"(p.bs.sat));
    T5A_STAMP(0);
    int trace_slot = 4;
    (void)trace_slot;
    int w = 0;
    const bool planned = MODE == kPacked && p.plan != nullptr;
    if (planned) {
        // the item comes from the launch plan, below
    } else if (CAUSAL && MODE == kDense && p.xcd_lo[8] > 0) {
        // this XCD's slice [lo, hi) of the pair-major item list touches the pairs ga .. gb; walk that
        // rectangle level by level (level 0 = longest tile) and drop the cells outside the slice
        const unsigned x = blockIdx.x & 7, k = blockIdx.x >> 3;
        const unsigned lo = (unsigned)p.xcd_lo[x], hi = (unsigned)p.xcd_lo[x + 1], tps = (unsigned)p.tiles_per_seq;
        if (hi <= lo) return;
        const unsigned ga = lo / tps, gx = (hi - 1) / tps - ga + 1;
        if (k >= gx * tps) return;
        const unsigned level = k / gx;
        const unsigned wi = (ga + (k - level * gx)) * tps + level;
        if (wi < lo || wi >= hi) return;
        w = (int)wi;
    } else if (BLOCK && p.block_items > 0) {
        // (block_items > 0 marks the launch that carries the global rows' key splits, however many splits there are)
        // the key splits of the global rows are the longer items: they take the first workgroup ids, so that they
        // start first and the block items fill in around them; the block items follow in per-XCD slices
        const int n_split = p.total_items - p.block_items;
        const int lead = (n_split + 7) & ~7;
        if ((int)blockIdx.x < lead) {
            if ((int)blockIdx.x >= n_split) return;
            w = p.block_items + (int)blockIdx.x;
        } else {
            const int id = (int)blockIdx.x - lead;
            const int per_xcd = (p.block_items + 7) >> 3;
            w = (id & 7) * per_xcd + (id >> 3);
            if (w >= p.block_items) return;
        }
    } else {
        const int per_xcd = (p.total_items + 7) >> 3;
        w = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
        if (w >= p.total_items) return;
    }

    // RUNS: the work item is run_len consecutive entries of the (batch, head, q tile) list.  The part of it that
    // lies in one (batch, head) is one pass of the loop below (set-up, then its q tiles as one stream); a run that
    // crosses into the next (batch, head) starts over there with a new set-up.
    int run_left = 1, run_next = 0;
    if constexpr (RUNS) {
        run_next = w * p.run_len;
        run_left = min(p.run_len, p.tiles_per_seq * p.H * p.B - run_next);
        if (BLOCK && p.block_items > 0 && w >= p.block_items) run_left = 1;   // a key split of the global rows: one pass
    }
    for (;;) {
    // (runs of q tiles: the thread index is made opaque once per pass; otherwise every per-lane constant of the set-up
    // is computed once before this loop -- ahead of the first tile requests -- and kept, or spilled, across all passes)
    int tid = threadIdx.x;
    if constexpr (RUNS) asm volatile("" : "+v"(tid));
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lr = lane & 31;
    const int hh = lane >> 5;
    int b = 0, h = 0, qt = 0, Mseq = 0, Nseq = 0, split = 0, key0 = 0;
    bool gsplit = false;     // block pattern: this item is a key split of the global rows
    int key_lo = 0;          // windowed patterns: first key of the sequence (a batch padded on the left)
    int n_valid = 0x7fffffff;   // block pattern: valid tokens of a right-padded sequence
    int n_side = p.n_side;   // side tokens of this item's sequence (transient-global)
    int64_t q_off, k_off, v_off, o_off, lse_off;
    if (MODE == kPacked) {
        int qs = 0, ks = 0;
        if (planned) {
            // packed batch with a launch plan: entry k of this XCD's list
            const int x = blockIdx.x & 7, k = blockIdx.x >> 3;
            const int* e = p.plan + ((size_t)x * p.plan_slots + k) * 8;
            if (k >= p.plan_counts[x]) return;
            b = e[0]; h = e[1]; qt = e[2]; Mseq = e[3]; Nseq = e[4]; qs = e[5]; ks = e[6];
        } else {
            // packed batch: find (sequence, head, tile) by walking cu_seqlens
            int acc = 0, nt_b = 0;
            b = -1;
            for (int bb = 0; bb < p.B; ++bb) {
                qs = p.cu_q[bb];
                const int len = p.len_q != nullptr ? p.len_q[bb] : p.cu_q[bb + 1] - qs;
                nt_b = (len + BM - 1) / BM;
                const int cnt = nt_b * p.H;
                if (w < acc + cnt) { b = bb; Mseq = len; w -= acc; break; }
                acc += cnt;
            }
            if (b < 0) return;
            h = w / nt_b;
            qt = w - h * nt_b;
            if (CAUSAL) qt = nt_b - 1 - qt;
            ks = p.cu_k[b];
            Nseq = p.len_k != nullptr ? p.len_k[b] : p.cu_k[b + 1] - ks;
        }
        q_off = (int64_t)qs * p.q_sr + (int64_t)h * p.q_sh;
        o_off = (int64_t)qs * p.o_sr + (int64_t)h * p.o_sh;
        k_off = (int64_t)ks * p.k_sr + (int64_t)h * p.k_sh;
        v_off = (int64_t)ks * p.v_sr + (int64_t)h * p.v_sh;
        lse_off = (int64_t)qs * p.lse_sr + (int64_t)h * p.lse_sh;
    } else {
        // unsigned arithmetic: the divisions are scalar code on every workgroup's critical path
        const unsigned entry = RUNS ? (unsigned)run_next : (unsigned)w;
        // (q tiles per sequence are a power of two for the usual lengths: a shift instead of forty instructions)
        const unsigned tps = (unsigned)p.tiles_per_seq;
        unsigned bh = (tps & (tps - 1)) == 0 ? entry >> __builtin_ctz(tps | 0x80000000u) : entry / tps;
        qt = (int)(entry - bh * tps);
        if (CAUSAL) qt = p.tiles_per_seq - 1 - qt;
        if (BLOCK && p.block_items > 0 && w >= p.block_items) {
            // block pattern, behind the block items: key split `split` of the global rows of one (batch, head) --
            // its first G rows attend all keys, standard bias; the partial results are merged by a second kernel
            gsplit = true;
            const unsigned gs = (unsigned)(w - p.block_items);
            bh = gs / (unsigned)p.nsplit;
            split = (int)(gs - bh * (unsigned)p.nsplit);
            qt = 0;
        }
        if (MODE == kDense && p.nsplit > 1) {
            const unsigned g = bh / (unsigned)p.nsplit;
            split = (int)(bh - g * (unsigned)p.nsplit);
            bh = g;
        }
        b = (int)(bh / (unsigned)p.H);
        h = (int)(bh - (unsigned)b * (unsigned)p.H);
        Mseq = p.M;
        Nseq = p.N;
        // windowed patterns on a right-padded batch: the keys of a sequence end at its length; positions are
        // the row indices, so nothing else changes (rows past the length see what is left of their window).
        // Its side tokens are the full blocks of that length, the rest of its tokens joining the last one.
        if ((LOCAL || TG) && p.len_k != nullptr) {
            // the sequence's tokens are the rows [key_lo, Nseq); a token's position stays its row index
            key_lo = p.start_k != nullptr ? max(0, min(p.N, p.start_k[b])) : 0;
            Nseq = max(key_lo, min(p.N, key_lo + max(0, p.len_k[b])));
            // side tokens: one per block END among the tokens; a token's side token is min(row / aux, count - 1)
            // (what the reference's block ids come to for one run of tokens, src/turbot5/model/utils.py:191-237)
            if (TG) n_side = min(p.n_side, Nseq / p.aux - key_lo / p.aux);
        }
        // masks of any shape: the caller counts the block ENDs among the valid tokens
        if (TG && p.side_counts != nullptr) n_side = max(0, min(p.n_side, p.side_counts[b]));
        // (padded batches of the block pattern run in the instantiation for masks: the plain one knows n_valid as a constant)
        if (MODE == kBlockBits && p.len_k != nullptr) n_valid = max(0, min(p.N, p.len_k[b]));
        q_off = (int64_t)b * p.q_sb + (int64_t)h * p.q_sh;
        o_off = (int64_t)b * p.o_sb + (int64_t)h * p.o_sh;
        k_off = (int64_t)b * p.k_sb + (int64_t)h * p.k_sh;
        v_off = (int64_t)b * p.v_sb + (int64_t)h * p.v_sh;
        lse_off = (int64_t)b * p.lse_sb + (int64_t)h * p.lse_sh;
        if ((MODE == kDense && p.nsplit > 1) || gsplit) {   // this item sees only its slice of the keys
            if (gsplit) Mseq = min(p.aux, p.M);
            key0 = split * p.split_rows;
            Nseq = max(0, min(p.split_rows, p.N - key0));
            k_off += (int64_t)key0 * p.k_sr;
            v_off += (int64_t)key0 * p.v_sr;
        }
    }
    const T* qp = reinterpret_cast<const T*>(p.q) + q_off;
    T* op = reinterpret_cast<T*>(p.o) + o_off;
    // sparse patterns, masks of any shape: validity of this sequence's tokens as a bit set (the global rows'
    // key splits of the block pattern attend every key, as in the reference)
    // (the host sends such batches to instantiations of their own -- kLocalWide, kBlockBits, kTGlobalBits -- so that
    // the ones for batches without holes carry none of this)
    constexpr bool BITS = MODE == kLocalWide || MODE == kBlockBits || MODE == kTGlobalBits;
    const unsigned* kbits = (BITS && p.key_bits != nullptr && !gsplit) ? p.key_bits + (int64_t)b * p.key_bits_stride : nullptr;
    // validity of the tokens pos0 .. pos0 + 63, bit e = token pos0 + e (wavefront-uniform: scalar loads)
    auto token_bits = [&](int pos0) {
        const int w = (pos0 + 32 * kKeyBitsFront) >> 5, sh = pos0 & 31;
        const unsigned long long a = ((unsigned long long)kbits[w + 1] << 32) | kbits[w];
        return sh != 0 ? (a >> sh) | ((unsigned long long)kbits[w + 2] << (64 - sh)) : a;
    };

    // q tiles of this item: one, or a run of consecutive ones (RUNS)
    int qt_count = 1;
    if constexpr (RUNS) qt_count = min(run_left, p.tiles_per_seq - qt);
    const int qt_last = qt + qt_count;   // one past the last q tile of this pass
    // query rows of the current q tile: [i0, row_end); rows below row_lo are computed but not stored
    int i0 = 0, row_end = 0, row_lo = 0, blk = 0;
    const int tpb = BLOCK ? (p.block_len + BM - 1) / BM : 1;   // q tiles per block (block pattern)
    if (BLOCK && !gsplit) row_lo = p.aux;   // the first G rows belong to the key-split items / the global-query pass
    const int P = p.align_end ? Nseq - Mseq : -key0;   // query position minus row index, in this item's key numbering

    // ---------------------------------------------------------------- key segments
    // A segment is a key range [start, end) of one K/V tensor.  Keys at or past
    // lend are read as zero vectors (they still count when below end).  The key
    // position is its index j; the query position depends on the kind:
    //   0: i + P     1: i % block_len + G (block pattern, global keys)     2: i / aux (side tokens)
    const T* seg_k[2]; const T* seg_v[2];
    int seg_ksr[2], seg_vsr[2];      // row strides in bytes
    // (read with explicit selects, never with a run-time index: an indexed private array lives in scratch
    // memory, and a scratch load waits for every tile request in flight)
    int seg_start[2], seg_end[2], seg_lend[2], seg_kind[2], seg_win[2];
    int nseg = 1;
    seg_k[0] = reinterpret_cast<const T*>(p.k) + k_off;
    seg_v[0] = reinterpret_cast<const T*>(p.v) + v_off;
    seg_ksr[0] = (int)p.k_sr * ES; seg_vsr[0] = (int)p.v_sr * ES;
    seg_k[1] = seg_k[0]; seg_v[1] = seg_v[0]; seg_ksr[1] = seg_ksr[0]; seg_vsr[1] = seg_vsr[0];
    seg_start[0] = 0; seg_end[0] = 0;
    seg_start[1] = seg_end[1] = seg_lend[1] = 0; seg_kind[1] = 0; seg_win[1] = 0;
    seg_kind[0] = 0; seg_win[0] = 0; seg_lend[0] = Nseq;
    if (LOCAL || TG) {
        seg_win[0] = 1;
        if (TG) {
            nseg = 2;
            seg_k[1] = reinterpret_cast<const T*>(p.side_k) + (int64_t)b * p.sk_sb + (int64_t)h * p.sk_sh;
            seg_v[1] = reinterpret_cast<const T*>(p.side_v) + (int64_t)b * p.sv_sb + (int64_t)h * p.sv_sh;
            seg_ksr[1] = (int)p.sk_sr * ES; seg_vsr[1] = (int)p.sv_sr * ES;
            seg_end[1] = n_side; seg_lend[1] = n_side; seg_kind[1] = 2;
        }
    } else if (BLOCK && !gsplit) {
        nseg = 2;
        seg_end[0] = p.aux; seg_kind[0] = 1;
        seg_lend[1] = Nseq;
    } else if (BLOCK) {
        seg_end[0] = Nseq;   // one segment: this split's keys, query i at position i (P = -key0)
    }
    // The part of the geometry that changes from one q tile to the next.  RUNS: every q tile of the run has the
    // same number of tiles per segment (seg_nt): the window starts where it starts even when that is before key 0,
    // and a block's segment spans a whole block; tiles outside the keys that exist read as zeros and are skipped
    // or masked.
    int seg_nt[2] = {0, 0};
    // block pattern, right-padded sequence: the own-block keys [lo, lo + span) that the rows of block blk do not see.
    // The reference lays its additive padding mask out as [own block | global tokens] over keys that are laid out
    // [global tokens | own block] (src/turbot5/model/attentions.py:722-732 against :807-814): list column
    // c < block_len is masked iff token blk * block_len + c is padding, the last G columns never are (except in
    // block 0, where they always are).  valid = how many of the first block_len list columns stay.  (Derived from
    // n_valid where a tile is classified or masked, rather than kept: the pattern's tile loop has no registers left.)
    auto block_valid = [&]() { return max(0, min(p.block_len, n_valid - blk * p.block_len)); };
    auto block_hole = [&](int& lo, int& span) {
        const int head = max(block_valid() - p.aux, 0);   // own-block keys before the masked range
        lo = blk * p.block_len + head;
        span = blk == 0 ? 0 : max(0, p.block_len - p.aux - head);
    };
    auto set_qtile = [&](int q_tile) {
        if (BLOCK && !gsplit) {
            blk = tpb == 1 ? q_tile : q_tile / tpb;   // (a division is some forty scalar instructions)
            i0 = blk * p.block_len + (q_tile - blk * tpb) * BM;
            row_end = min(Mseq, (blk + 1) * p.block_len);
            seg_start[1] = blk * p.block_len;
            const int valid = block_valid();
            seg_end[0] = min(p.aux, valid);
            seg_end[1] = blk == 0 ? min(p.block_len - p.aux, max(valid - p.aux, 0)) : (blk + 1) * p.block_len;
        } else {
            i0 = q_tile * BM;
            row_end = Mseq;
        }
        if (DENSE) {
            seg_end[0] = CAUSAL ? max(0, min(Nseq, i0 + BM + P)) : Nseq;
        } else if (LOCAL || TG) {
            seg_start[0] = RUNS ? i0 - p.block_len + 1 : max(key_lo, i0 - p.block_len + 1);
            seg_end[0] = min(Nseq, min(i0 + BM, Mseq) - 1 + p.block_len);
        }
    };
    // first row and end of the rows of any q tile of this (batch, head)
    auto qtile_rows = [&](int q_tile, int& first, int& end) {
        if (BLOCK) {
            const int bk = tpb == 1 ? q_tile : q_tile / tpb;
            first = bk * p.block_len + (q_tile - bk * tpb) * BM;
            end = min(Mseq, (bk + 1) * p.block_len);
        } else {
            first = q_tile * BM;
            end = Mseq;
        }
    };
    set_qtile(qt);
    if constexpr (RUNS) {
        if (BLOCK && gsplit) { seg_nt[0] = (Nseq + BN - 1) / BN; seg_nt[1] = 0; }
        else if (BLOCK) { seg_nt[0] = (p.aux + BN - 1) / BN; seg_nt[1] = (p.block_len + BN - 1) / BN; }
        else { seg_nt[0] = (BM + 2 * p.block_len - 2 + BN - 1) / BN; seg_nt[1] = nseg > 1 ? (n_side + BN - 1) / BN : 0; }
    } else {
        seg_nt[0] = max(0, seg_end[0] - seg_start[0] + BN - 1) / BN;
        seg_nt[1] = nseg > 1 ? max(0, seg_end[1] - seg_start[1] + BN - 1) / BN : 0;
    }
    // an even number of tiles per q tile keeps the two score buffers of the pipeline in step from one q tile of a
    // run to the next (the extra tile lies past its segment's end and is skipped)
    // (the block pattern's q tiles are too short for fast steps anyway: no rounding there)
    if (RUNS && !BLOCK && ((seg_nt[0] + seg_nt[1]) & 1)) {   // (no run-time index: that would move the array to scratch memory)
        if (nseg > 1) seg_nt[1] += 1; else seg_nt[0] += 1;
    }
    const int ntiles = seg_nt[0] + seg_nt[1];   // tiles of one q tile
    int tbase = 0;                               // tiles of the run's earlier q tiles (the ring stages count on)
    __amdgpu_buffer_rsrc_t seg_krs[2], seg_vrs[2];
    u32x4 seg_krw[2], seg_vrw[2];
#pragma unroll
    for (int sg = 0; sg < 2; ++sg) {
        // rows at or past this read as zero.  RUNS: one descriptor per tensor for the whole run -- all the keys of
        // the (batch, head); what a q tile must not see of them is masked
        const int rows = RUNS ? (sg == 0 || BLOCK ? Nseq : n_side) : min(seg_lend[sg], seg_end[sg]);
        const unsigned kb = rows > 0 ? (unsigned)(rows - 1) * (unsigned)seg_ksr[sg] + D * ES : 0u;
        const unsigned vb = rows > 0 ? (unsigned)(rows - 1) * (unsigned)seg_vsr[sg] + D * ES : 0u;
        seg_krs[sg] = make_rsrc(seg_k[sg], kb);
        seg_vrs[sg] = make_rsrc(seg_v[sg], vb);
        seg_krw[sg] = make_rsrc_words(seg_k[sg], kb);
        seg_vrw[sg] = make_rsrc_words(seg_v[sg], vb);
    }
    const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;

    // tile t of the current q tile -> segment and first key.  RUNS: t may run past the q tile's last tile into the
    // following q tiles of the run (requests are issued up to four tiles ahead); returns false past the run's end.
    auto tile_of = [&](int t, int& sg, int& j0) {
        if constexpr (RUNS) {
            int ahead = 0;
            if (t >= ntiles) { t -= ntiles; ++ahead; }          // (requests run at most four tiles ahead: two q tiles
            if (t >= ntiles) { t -= ntiles; ++ahead; }          // further on at the very most, with q tiles of 2+ tiles)
            while (t >= ntiles) { t -= ntiles; ++ahead; }
            const int q_tile = qt + ahead;
            sg = t >= seg_nt[0] ? 1 : 0;
            const int ts = t - (sg ? seg_nt[0] : 0);
            // (a scalar division costs some forty instructions, and this runs for every request)
            if (BLOCK) j0 = sg ? (tpb == 1 ? q_tile : q_tile / tpb) * p.block_len + ts * BN : ts * BN;
            else j0 = sg ? ts * BN : q_tile * BM - p.block_len + 1 + ts * BN;
            return q_tile < qt_last;
        } else {
            sg = t >= seg_nt[0] ? 1 : 0;
            j0 = (sg ? seg_start[1] : seg_start[0]) + (t - (sg ? seg_nt[0] : 0)) * BN;
            return true;
        }
    };
    // LDS-DMA staging: a wavefront instruction writes 64 x 16 bytes to consecutive LDS addresses
    // (8 rows of 128 bytes); the XOR swizzles are applied on the SOURCE side: the lane that owns
    // physical chunk pc of row r fetches logical chunk pc ^ swizzle(r).  Rows past the end of the
    // segment are out of the buffer's range and arrive as zeros.
    auto dma_tile = [&](int t, bool is_v, int stage = -1) {
        if constexpr (DMA) {
            int sg, j0;
            const bool in_run = tile_of(t, sg, j0);
            u32x4 rs = is_v ? (sg ? seg_vrw[1] : seg_vrw[0]) : (sg ? seg_krw[1] : seg_krw[0]);
            if (!in_run) rs[2] = 0u;   // nothing is readable: the request fills its stage with zeros
            const int sr = is_v ? (sg ? seg_vsr[1] : seg_vsr[0]) : (sg ? seg_ksr[1] : seg_ksr[0]);
            if (stage < 0) stage = is_v ? (tbase + t) % NSV : (tbase + t) % NSK;
            const unsigned base = lds_base + (is_v ? (unsigned)(stage * V_TILE) : (unsigned)(NSV * V_TILE + stage * K_TILE)) * ES;
#pragma unroll
            for (int c = 0; c < G::SPW; ++c) {
                const int slab = wave * G::SPW + c;         // 1 KB = RPS rows
                const int r = slab * G::RPS + lane / G::LPR, pc = lane % G::LPR;
                const int ch = pc ^ (is_v ? G::vrow_swz(r) : G::kswz(r));
                lds_dma_16(rs, base + slab * 1024, (j0 + r) * sr + ch * 16);
            }
        }
    };
    // Runs of q tiles (one segment): the K and the V requests each walk the tiles of the run in order, so each keeps
    // a cursor -- first key, tile index inside its q tile, q tile -- that a request advances with a few scalar
    // instructions (where tile_of divides).  A request past the run's last q tile fills its stage with zeros.
    int rq_j0[2] = {0, 0}, rq_ts[2] = {0, 0}, rq_q[2] = {0, 0}, rq_stage[2] = {0, 0};   // [0]: K, [1]: V
    int rq_koff[G::SPW], rq_voff[G::SPW];   // this lane's byte offsets inside a tile
#pragma unroll
    for (int c = 0; c < G::SPW; ++c) rq_koff[c] = rq_voff[c] = 0;
    if constexpr (CURSOR) {
#pragma unroll
        for (int c = 0; c < G::SPW; ++c) {
            const int r = (wave * G::SPW + c) * G::RPS + lane / G::LPR, pc = lane % G::LPR;
            rq_koff[c] = r * seg_ksr[0] + (pc ^ G::kswz(r)) * 16;
            rq_voff[c] = r * seg_vsr[0] + (pc ^ G::vrow_swz(r)) * 16;
        }
        rq_j0[0] = rq_j0[1] = qt * BM - p.block_len + 1;
        rq_q[0] = rq_q[1] = qt;
    }
    auto dma_next = [&](bool is_v, int stage = -1) {
        if constexpr (CURSOR) {
            const int w = is_v ? 1 : 0;
            const int j0 = w ? rq_j0[1] : rq_j0[0];
            const int q_tile = w ? rq_q[1] : rq_q[0];
            u32x4 rs = is_v ? seg_vrw[0] : seg_krw[0];
            if (q_tile >= qt_last) rs[2] = 0u;
            if (stage < 0) stage = w ? rq_stage[1] : rq_stage[0];
            const unsigned base = lds_base + (is_v ? (unsigned)(stage * V_TILE) : (unsigned)(NSV * V_TILE + stage * K_TILE)) * ES;
            const int tile_off = j0 * (is_v ? seg_vsr[0] : seg_ksr[0]);
#pragma unroll
            for (int c = 0; c < G::SPW; ++c)
                lds_dma_16(rs, base + (wave * G::SPW + c) * 1024, tile_off + (is_v ? rq_voff[c] : rq_koff[c]));
            // advance (explicit selects: an indexed private array would live in scratch memory)
            int ts = (w ? rq_ts[1] : rq_ts[0]) + 1, nj0 = j0 + BN, nq = q_tile;
            if (ts == ntiles) { ts = 0; nq = q_tile + 1; nj0 += BM - ntiles * BN; }
            const int nst = ((w ? rq_stage[1] : rq_stage[0]) + 1) % (w ? NSV : NSK);
            if (w) { rq_ts[1] = ts; rq_j0[1] = nj0; rq_q[1] = nq; rq_stage[1] = nst; }
            else { rq_ts[0] = ts; rq_j0[0] = nj0; rq_q[0] = nq; rq_stage[0] = nst; }
        }
    };
    // Dense mode: the K and V requests walk the tiles in order with per-lane running byte offsets (one vector add
    // per request and step, where a descriptor moved along by scalar code costs the wavefront some twenty scalar
    // instructions: a wavefront issues one instruction of any kind every four to five cycles, so scalar bookkeeping
    // is as expensive as vector work).  The descriptors span all rows of the (batch, head): tiles past the end are
    // out of range and arrive as zeros.  Slices stay below 2 GiB (checked on the host), so 32-bit offsets do.
    const int kstep = BN * seg_ksr[0], vstep = BN * seg_vsr[0];
    int cur_koff[G::SPW], cur_voff[G::SPW];
#pragma unroll
    for (int c = 0; c < G::SPW; ++c) cur_koff[c] = cur_voff[c] = 0;
    auto cursor_seek = [&](int tk, int tv) {   // next requests: K tile tk, V tile tv
        if constexpr (DMA && DENSE) {
#pragma unroll
            for (int c = 0; c < G::SPW; ++c) {
                const int r = (wave * G::SPW + c) * G::RPS + lane / G::LPR, pc = lane % G::LPR;
                // requests go out in pairs; the second of a pair carries an instruction offset of 1024
                cur_koff[c] = r * seg_ksr[0] + (pc ^ G::kswz(r)) * 16 - (c & 1) * 1024 + tk * kstep;
                cur_voff[c] = r * seg_vsr[0] + (pc ^ G::vrow_swz(r)) * 16 - (c & 1) * 1024 + tv * vstep;
            }
        }
    };
    auto cursor_dma = [&](int kstage, int vstage) {
        if constexpr (DMA) {
            const unsigned wbase = lds_base + (unsigned)wave * (1024u * G::SPW);
            if constexpr (G::SPW == 1) {   // one request per tensor and wavefront
                lds_dma_16(seg_krw[0], wbase + (unsigned)(NSV * V_TILE + kstage * K_TILE) * ES, cur_koff[0]);
                lds_dma_16(seg_vrw[0], wbase + (unsigned)(vstage * V_TILE) * ES, cur_voff[0]);
            } else {
#pragma unroll
                for (int c = 0; c + 1 < G::SPW; c += 2) {
                    lds_dma_16x2(seg_krw[0], wbase + (unsigned)(NSV * V_TILE + kstage * K_TILE) * ES + c * 1024u,
                                 cur_koff[c], cur_koff[c + 1]);
                    lds_dma_16x2(seg_vrw[0], wbase + (unsigned)(vstage * V_TILE) * ES + c * 1024u,
                                 cur_voff[c], cur_voff[c + 1]);
                }
            }
#pragma unroll
            for (int c = 0; c < G::SPW; ++c) { cur_koff[c] += kstep; cur_voff[c] += vstep; }
        }
    };
    // ---------------------------------------------------------------- Q fragments: loads first
    int wq_lo[2] = {0, 0}, wq_hi[2] = {0, 0}, lq_pos[2] = {0, 0};   // query positions per segment, see set_positions
    int iw0 = i0 + wave * 32;      // first row of this wavefront
    int iw1 = iw0 + 31;
    int irow = iw0 + lr;           // this lane's query row
    bool row_ok = irow < row_end;
    v8 qf[KS];
    // RUNS: the Q rows of the run's NEXT q tile, requested a whole q tile ahead (plain loads: they have landed long
    // before the switch, where the only cost left is the compiler's wait for everything in flight)
    v8 qn[RUNS ? KS : 1];
    auto prefetch_q = [&](int q_tile) {
        if constexpr (RUNS) {
            // (unconditional: past the last q tile of the run it reads that one again, a lane past the last row reads
            // the last row -- such rows are computed and not stored; a conditional load makes the compiler merge
            // register sets at the loop's back edge, behind a wait for the load it has just issued)
            int first, end;
            qtile_rows(min(q_tile, qt_last - 1), first, end);
            const int row = max(0, min(first + wave * 32 + lr, end - 1));
#pragma unroll
            for (int s = 0; s < KS; ++s)
                qn[s] = *reinterpret_cast<const v8*>(qp + (int64_t)row * p.q_sr + 16 * s + 8 * hh);
        }
    };
    f32x4 qraw[F32 ? D / 4 : 1];
    if constexpr (F32) {
#pragma unroll
        for (int c = 0; c < D / 4; ++c) {
            qraw[c] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (row_ok) qraw[c] = *reinterpret_cast<const f32x4*>(qp + (int64_t)irow * p.q_sr + 4 * c);
        }
    } else if constexpr (!QDMA) {
#pragma unroll
        for (int s = 0; s < KS; ++s) {
#pragma unroll
            for (int e = 0; e < 8; ++e) qf[s][e] = (T)0.0f;
            if (row_ok) qf[s] = *reinterpret_cast<const v8*>(qp + (int64_t)irow * p.q_sr + 16 * s + 8 * hh);
        }
    }

    // ---------------------------------------------------------------- bias LUT
    const bool has_bias = p.table != nullptr;
    // Sliding window folded into the LUT (local pattern, windows up to kMaxLutWindow): the window is a function
    // of the distance alone, so the LUT holds -inf from the window's edge on and reaches LUT_PAD past it.
    // No tile then needs a per-element window mask, and every tile that is not skipped is a LUT tile.
    constexpr bool win_lut = MODE == kLocal;   // the host picks kLocal for windows up to kMaxLutWindow
    const bool has_lut = has_bias || CAUSAL || win_lut;
    const int sat_bias = has_bias ? p.bs.sat : 0;
    const int sat = win_lut ? max(sat_bias, p.block_len) : sat_bias;   // distance from which the LUT is constant
    const int padl = sat + LUT_PAD;                       // LUT index of rel = 0
    const int quads = lut_quads(sat, CAUSAL);
    const int qlen = 4 * quads;
    const float log2e = 1.4426950408889634f;
    // The head's table column: with at most 64 buckets, lane b of every wavefront fetches bucket b up
    // front and the LUT entries pick their value with a lane permute; larger tables are read per entry.
    // A caller-provided buffer may instead hold the LUTs of all heads, built once per table (lut.hip): the
    // head's image (4 * qlen floats) is then fetched as it is.
    //
    // LDS-DMA geometries fetch either of them with LDS-DMA requests of their own, issued BEFORE the first
    // K/V tiles: requests complete in order, so "at most the tile requests outstanding" means the column
    // (or this wavefront's pieces of the image) has landed, and the LUT is built while the tiles are still
    // in flight.  Nothing of this passes through vector registers: the compiler does not know that a
    // register written by a load issued from inline assembly is still in flight and may copy it too early.
    const int nbt = p.bs.bidirectional ? 2 * p.bs.nb : p.bs.nb;
    const bool col_in_lanes = nbt <= 64;
    // (the host checked qlen <= 512, and that a buffer of windowed images goes with this window)
    const bool lut_cached = has_bias && p.lut_global != nullptr && (win_lut ? p.lut_window == p.block_len : p.lut_window == 0);
    const int col_esize = p.table_dtype == T5A_F32 ? 4 : 2;
    // byte offset of this lane's bucket in the table, from the 4-byte aligned address at or below its start
    const unsigned col_misalign = (unsigned)(reinterpret_cast<uintptr_t>(p.table) & 3);
    const unsigned col_byte = col_misalign +
        (unsigned)(((int64_t)(lane < nbt ? lane : 0) * p.t_sbucket + (int64_t)h * p.t_shead) * col_esize);
    const int lut_region = (4 * qlen + 255) & ~255;   // floats: the image, rounded up to whole 1 KB requests
    float* col_stage = lut + lut_region + wave * 64;  // 64 dwords per wavefront behind it
    float tcol = 0.f;
    // With QDMA the order of the prologue's requests is  K0 V0 | Q rows | column or LUT image | K1 V1 K2 V2,
    // and K3 follows once every wavefront has taken its Q rows out of LDS: the rows are staged in the last
    // stage of the K ring (wavefronts 0, 1) and of the V ring (2, 3), 4 KB each, which the loop fills first
    // with K3 and V3.  Requests complete in order, so "at most K1 V1 K2 V2 outstanding" means that K0, V0,
    // Q and the column have landed: the LUT is built and the first product formed while the rest is in
    // flight.  (Q loaded into registers by the compiler would be waited for with "nothing outstanding".)
    static_assert(!QDMA || (K_TILE * ES == 8192 && V_TILE * ES == 8192 && NSK == 4 && NSV == 4 && NTHREADS == 256),
                  "the Q staging borrows 4 KB per wavefront from the last K and V ring stages");
    // the staged Q rows are 128 bytes: rows two apart share their banks, so the 16-byte chunks are XOR-swizzled
    // like the K tiles (on the source side of the request) and a 16-lane read phase covers all 64 banks
    auto qswz = [](int row) { return (row >> 1) & 7; };
    const unsigned q_stage = wave < 2 ? (unsigned)(NSV * V_TILE + 3 * K_TILE) * ES + wave * 4096u
                                      : (unsigned)(3 * V_TILE) * ES + (wave - 2) * 4096u;
    if constexpr (QDMA) {
        if constexpr (DENSE) { cursor_seek(0, 0); cursor_dma(0, 0); }
        else if constexpr (CURSOR) { dma_next(false); dma_next(true); }
        else { dma_tile(0, false); dma_tile(0, true); }
        const int q_row_bytes = (int)p.q_sr * ES;
        const u32x4 rs = make_rsrc_words(qp, row_end > 0 ? (unsigned)(row_end - 1) * (unsigned)q_row_bytes + D * ES : 0u);
#pragma unroll
        for (int r = 0; r < 4; ++r)   // 8 rows of 128 bytes per request; rows past the end arrive as zeros
            lds_dma_16(rs, lds_base + q_stage + r * 1024,
                       (iw0 + 8 * r + (lane >> 3)) * q_row_bytes + (((lane & 7) ^ qswz(8 * r + (lane >> 3))) * 16));
    }
    if constexpr (DMA) {
        if (lut_cached) {
            const u32x4 rs = make_rsrc_words(p.lut_global + (size_t)h * (4 * qlen), (unsigned)(qlen * 16));
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const int first = c * NTHREADS + wave * 64;   // first 16-byte piece of this request
                if (first < qlen)   // pieces past the image read as zeros into the slack behind it
                    lds_dma_16(rs, lds_base + (unsigned)(NSV * V_TILE + NSK * K_TILE) * ES + first * 16, (first + lane) * 16);
            }
        } else if (has_bias && col_in_lanes) {
            const unsigned col_bytes = col_misalign +
                (unsigned)(((int64_t)(nbt - 1) * p.t_sbucket + (int64_t)(p.H - 1) * p.t_shead + 1) * col_esize);
            const u32x4 rs = make_rsrc_words(reinterpret_cast<const char*>(p.table) - col_misalign, (col_bytes + 3) & ~3u);
            lds_dma_4(rs, lds_base + (unsigned)(NSV * V_TILE + NSK * K_TILE) * ES + (lut_region + wave * 64) * 4,
                      (int)(col_byte & ~3u));
        }
    } else if (has_bias && col_in_lanes && lane < nbt && !lut_cached) {
        tcol = load_table(p.table, p.table_dtype, (int64_t)lane * p.t_sbucket + (int64_t)h * p.t_shead) * log2e;
    }
    T5A_STAMP(1);
    // request the first tiles: they arrive while the bias LUT is built
    if constexpr (DMA) {
        if constexpr (QDMA) {
            if constexpr (DENSE) { cursor_dma(1, 1); cursor_dma(2, 2); }   // K1 V1, K2 V2
            else if constexpr (CURSOR) { dma_next(false); dma_next(true); dma_next(false); dma_next(true); }
            else { dma_tile(1, false); dma_tile(1, true); dma_tile(2, false); dma_tile(2, true); }
        } else if constexpr (DENSE) {
            cursor_seek(0, 0);
            cursor_dma(0, 0); cursor_dma(1, 1); cursor_dma(2, 2);   // K0 V0, K1 V1, K2 V2
            dma_tile(3, false);                                     // K3
        } else if constexpr (CURSOR) {
            for (int i = 0; i < 4; ++i) dma_next(false);
            for (int i = 0; i < 3; ++i) dma_next(true);
        } else {
            for (int i = 0; i < 4; ++i) dma_tile(i, false);
            for (int i = 0; i < 3; ++i) dma_tile(i, true);
        }
        // everything older than these tile requests; the clobber keeps the LDS reads below behind the wait
        asm volatile("s_waitcnt vmcnt(%0)" :: "n"((QDMA ? 4 : 7) * G::SPW) : "memory");
        if (!lut_cached && has_bias && col_in_lanes) {
            const unsigned raw = __float_as_uint(col_stage[lane]);
            const unsigned el = col_esize == 4 ? raw : ((raw >> (8 * (col_byte & 2))) & 0xffffu);
            tcol = table_value(el, p.table_dtype) * log2e;
        }
    }
    if (lut_cached) {
        if constexpr (!DMA) {
            const f32x4* src = reinterpret_cast<const f32x4*>(p.lut_global + (size_t)h * (4 * qlen));
            for (int idx = tid; idx < qlen; idx += NTHREADS) reinterpret_cast<f32x4*>(lut)[idx] = src[idx];
        }
    } else if (has_lut) {
        lut_fill<CAUSAL>(lut, p.bs, p.table, p.table_dtype, p.t_sbucket, p.t_shead, h, has_bias, tcol, col_in_lanes,
                         padl, qlen, tid, NTHREADS, win_lut ? p.block_len : 0x7fffffff);
    }
    if (D < 32) {  // the part of V past head_dim feeds the MFMA: keep it zero
        for (int idx = tid; idx < NSV * V_TILE; idx += NTHREADS) Vs[idx] = (T)0.0f;
    }
    __syncthreads();
    T5A_STAMP(2);
    const float c_neg = has_bias ? lut[0] : 0.f;                 // every key far before the query
    const float c_pos = has_bias ? lut[qlen - 1] : 0.f;          // every key far after it (non-causal)

    // ---------------------------------------------------------------- Q fragments: pre-scale by sm_scale*log2(e)
    if constexpr (QDMA) {
        const T* qs_rows = reinterpret_cast<const T*>(smem + q_stage);
#pragma unroll
        for (int s = 0; s < KS; ++s) qf[s] = *reinterpret_cast<const v8*>(qs_rows + lr * D + (((2 * s + hh) ^ qswz(lr)) * 8));
    }
    if constexpr (F32) {
#pragma unroll
        for (int c = 0; c < D / 4; ++c) {
            qf[2 * c] = (hh ? qraw[c][1] : qraw[c][0]) * p.c1;
            qf[2 * c + 1] = (hh ? qraw[c][3] : qraw[c][2]) * p.c1;
        }
    } else if (!exact) {
#pragma unroll
        for (int s = 0; s < KS; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) qf[s][e] = (T)((float)qf[s][e] * p.c1);
    }
    // exact_scale: the accumulator input is (bias - running max) / c1 and the product is multiplied by c1
    // afterwards; otherwise inv_c1 is 1 and the same instructions form (bias - running max) itself
    const float inv_c1 = exact ? 1.0f / p.c1 : 1.0f;

    // ---------------------------------------------------------------- tile staging
    u32x4 kreg[K_PER_T];
    u32x4 vreg[F32 ? V_PER_T : 2 * V_PER_T];   // 16-bit: four 8-byte rows per unit

    // V staging unit of a thread (16-bit types): 4 keys x 4 dims.  Lane bits are spread so that the
    // transposed 8-byte LDS writes of 32 consecutive lanes fall into 32 different 8-byte bank groups.
    auto v_unit = [&](int idx, int& dg, int& kg, int& rot) {
        if constexpr (D >= 64 && !F32) {
            const int kb = (idx >> 3) & 1, kgx = (idx >> 5) & 7;
            dg = (idx & 7) | (((idx >> 4) & 1) << 3) | ((idx >> 8) << 4);
            kg = ((kgx >> 1) << 2) | (kb << 1) | (kgx & 1);
            rot = (idx >> 4) & 1;
        } else {
            dg = idx % (D / 4); kg = idx / (D / 4); rot = 0;
        }
    };
    auto load_tile_k = [&](int t) {
        int sg, j0; tile_of(t, sg, j0);
        const __amdgpu_buffer_rsrc_t krs = sg ? seg_krs[1] : seg_krs[0];
        const int ksr = (sg ? seg_ksr[1] : seg_ksr[0]);
        // the whole byte offset goes into the vector operand: only that one is range checked
#pragma unroll
        for (int c = 0; c < K_PER_T; ++c) {
            const int idx = tid + c * NTHREADS;
            const int row = idx / CH, ch = idx % CH;
            if (K_CHUNKS % NTHREADS == 0 || idx < K_CHUNKS)
                kreg[c] = __builtin_amdgcn_raw_buffer_load_b128(krs, (j0 + row) * ksr + ch * 16, 0, 0);
        }
    };
    auto load_tile_v = [&](int t) {
        int sg, j0; tile_of(t, sg, j0);
        const __amdgpu_buffer_rsrc_t vrs = sg ? seg_vrs[1] : seg_vrs[0];
        const int vsr = (sg ? seg_vsr[1] : seg_vsr[0]);
        if constexpr (F32) {
#pragma unroll
            for (int c = 0; c < V_PER_T; ++c) {
                const int idx = tid + c * NTHREADS;
                const int row = idx / CH, ch = idx % CH;
                if (V_UNITS % NTHREADS == 0 || idx < V_UNITS)
                    vreg[c] = __builtin_amdgcn_raw_buffer_load_b128(vrs, (j0 + row) * vsr + ch * 16, 0, 0);
            }
        } else {
#pragma unroll
            for (int u = 0; u < V_PER_T; ++u) {
                const int idx = tid + u * NTHREADS;
                int dg, kg, rot; v_unit(idx, dg, kg, rot);
                if (V_UNITS % NTHREADS == 0 || idx < V_UNITS) {
                    u32x2 r[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        r[i] = __builtin_amdgcn_raw_buffer_load_b64(vrs, (j0 + 4 * kg + i) * vsr + dg * 8, 0, 0);
                    vreg[2 * u] = u32x4{r[0][0], r[0][1], r[1][0], r[1][1]};
                    vreg[2 * u + 1] = u32x4{r[2][0], r[2][1], r[3][0], r[3][1]};
                }
            }
        }
    };
    auto store_tile_k = [&](int buf) {
        T* ks = Ks + buf * K_TILE;
#pragma unroll
        for (int c = 0; c < K_PER_T; ++c) {
            const int idx = tid + c * NTHREADS;
            const int row = idx / CH, ch = idx % CH;
            if (K_CHUNKS % NTHREADS == 0 || idx < K_CHUNKS) {
                if constexpr (F32) {
                    float* dst = reinterpret_cast<float*>(ks) + row * KSTR + ch * 4;
                    dst[0] = __uint_as_float(kreg[c][0]); dst[1] = __uint_as_float(kreg[c][1]);
                    dst[2] = __uint_as_float(kreg[c][2]); dst[3] = __uint_as_float(kreg[c][3]);
                } else {
                    *reinterpret_cast<u32x4*>(ks + row * D + ((ch ^ G::kswz(row)) * 8)) = kreg[c];
                }
            }
        }
    };
    auto store_tile_v = [&](int buf) {
        T* vs = Vs + buf * V_TILE;
        if constexpr (F32) {
#pragma unroll
            for (int c = 0; c < V_PER_T; ++c) {
                const int idx = tid + c * NTHREADS;
                const int row = idx / CH, ch = idx % CH;
                if (V_UNITS % NTHREADS == 0 || idx < V_UNITS)
                    *reinterpret_cast<u32x4*>(vs + row * VROWS + ch * 4) = vreg[c];
            }
        } else {
#pragma unroll
            for (int u = 0; u < V_PER_T; ++u) {
                const int idx = tid + u * NTHREADS;
                int dg, kg, rot; v_unit(idx, dg, kg, rot);
                if (V_UNITS % NTHREADS == 0 || idx < V_UNITS) {
                    // 4 keys x 4 dims -> 4 dims x 4 keys.  Key slots 4..7 and 8..11 of every 16 are
                    // swapped so that a lane's eight P values line up with one 16-byte V^T read.
                    const int pk = (kg & ~3) | ((kg & 1) << 1) | ((kg >> 1) & 1);
                    const u32x4 a = vreg[2 * u], c2 = vreg[2 * u + 1];   // keys (0,1) and (2,3)
                    u32x2 y[4];
                    y[0] = u32x2{(a[0] & 0xffffu) | (a[2] << 16), (c2[0] & 0xffffu) | (c2[2] << 16)};
                    y[1] = u32x2{(a[0] >> 16) | (a[2] & 0xffff0000u), (c2[0] >> 16) | (c2[2] & 0xffff0000u)};
                    y[2] = u32x2{(a[1] & 0xffffu) | (a[3] << 16), (c2[1] & 0xffffu) | (c2[3] << 16)};
                    y[3] = u32x2{(a[1] >> 16) | (a[3] & 0xffff0000u), (c2[1] >> 16) | (c2[3] & 0xffff0000u)};
                    // half of the lanes take the dims in the order 1,0,3,2: even and odd rows
                    // (different halves of the 64 banks) are written by the same instruction
                    const bool sw = rot != 0;
                    const u32x2 z[4] = {sw ? y[1] : y[0], sw ? y[0] : y[1], sw ? y[3] : y[2], sw ? y[2] : y[3]};
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const int d = 4 * dg + (c ^ rot);
                        *reinterpret_cast<u32x2*>(vs + d * BN + (((pk >> 1) ^ G::vswz(d)) * 8) + (pk & 1) * 4) = z[c];
                    }
                }
            }
        }
    };

    // ---------------------------------------------------------------- tile classes (wavefront-uniform)
    struct TileClass { int sg, j0, side; bool skip, use_lut, need_mask; };
    // dense / packed mode: one segment starting at key 0, so the class of tile t follows from four
    // per-wavefront thresholds
    int d_tl = 0, d_tr = 0, d_ts = 0, d_tm = 0;
    if (DENSE) {
        const int qlo = iw0 + P, qhi = iw1 + P;
        const int lim = qlo - (BN - 1) - sat;                  // left-saturated tiles: BN*t <= lim
        d_tl = lim < 0 ? 0 : lim / BN + 1;
        d_tr = CAUSAL ? 0x7fffffff : (qhi + sat <= 0 ? 0 : (qhi + sat + BN - 1) / BN);   // right-saturated from here
        d_ts = iw0 >= row_end ? 0 : (CAUSAL ? (qhi < 0 ? 0 : qhi / BN + 1) : 0x7fffffff);  // skipped from here
        d_tm = seg_end[0] / BN;                                // tiles from here on straddle the segment end
    }
    // sparse patterns: the class of a tile from the geometry of the current q tile (a few dozen scalar instructions)
    // Validity of the 64 keys of a tile as the pattern's mask sees them (bit e = key j0 + e); kbits != nullptr.
    auto tile_valid = [&](int sg, int j0) {
        if (TG && sg == 1) return ~0ull;   // side tokens: the count of them is the mask
        if (!BLOCK) return token_bits(j0);
        // block pattern: list column c < block_len of [G global tokens | own block] takes the bit of token
        // blk * block_len + c (the reference's mask layout, attentions.py:722-732)
        if (sg == 0) return token_bits(blk * p.block_len + j0);            // global key j is column j
        unsigned long long m = token_bits(j0 + p.aux);                      // own key j is column G + (j - blk * block_len)
        const int e0 = (blk + 1) * p.block_len - p.aux - j0;                // tile position of the first column >= block_len:
        if (e0 < 64) m |= ~0ull << max(e0, 0);                              // never masked (block 0: cut off by the segment's end)
        return m;
    };
    auto classify_sparse = [&](int t) {
        TileClass c;
        c.sg = 0; c.j0 = 0; c.side = 0; c.skip = true; c.use_lut = false; c.need_mask = false;
        if (t >= ntiles) return c;
        tile_of(t, c.sg, c.j0);
        const int kind = (c.sg ? seg_kind[1] : seg_kind[0]);
        const bool win = (c.sg ? seg_win[1] : seg_win[0]) != 0;
        (void)kind;
        constexpr bool cached = BLOCK || TG;   // positions kept per q tile (set_positions)
        const int qlo = cached ? (c.sg ? wq_lo[1] : wq_lo[0]) : iw0 + P, qhi = cached ? (c.sg ? wq_hi[1] : wq_hi[0]) : iw1 + P;
        const int rel_min = c.j0 - qhi, rel_max = c.j0 + BN - 1 - qlo;
        c.skip = iw0 >= row_end;                              // wavefront without live rows
        if (CAUSAL) c.skip = c.skip || rel_min > 0;           // every key is in the future of every row
        if (win) c.skip = c.skip || (rel_max <= -p.block_len) || (rel_min >= p.block_len);
        const bool left_sat = rel_max <= -sat && (!CAUSAL || rel_max <= 0);
        const bool right_sat = !CAUSAL && rel_min >= sat;
        c.use_lut = has_lut && !(left_sat || right_sat);
        if constexpr (win_lut) c.use_lut = true;   // (a tile beyond the window's edge is skipped, never constant)
        const int s_end = c.sg ? seg_end[1] : seg_end[0];
        c.need_mask = c.j0 + BN > s_end;
        if constexpr (RUNS) {   // tiles before key 0 or past the end of the segment exist here (same count for every q tile)
            c.skip = c.skip || c.j0 >= s_end || c.j0 + BN <= key_lo;
            c.need_mask = c.need_mask || c.j0 < key_lo;
        }
        if (win && !win_lut) c.need_mask = c.need_mask || (rel_max >= p.block_len) || (rel_min <= -p.block_len);
        if (MODE == kBlockBits && c.sg == 1 && n_valid < Nseq) {
            int hole_lo, hole_span;
            block_hole(hole_lo, hole_span);
            c.need_mask = c.need_mask || (c.j0 < hole_lo + hole_span && c.j0 + BN > hole_lo);
        }
        if (BITS && kbits != nullptr && !c.skip) {
            const unsigned long long m = tile_valid(c.sg, c.j0);
            if (m == 0) c.skip = true;                 // no valid key in the tile
            else if (m != ~0ull) c.need_mask = true;
        }
        c.side = (has_bias && !c.use_lut && !c.skip) ? (left_sat ? 1 : 2) : 0;
        if constexpr (win_lut) c.side = 0;
        return c;
    };
    // ... evaluated once per q tile into bit sets (bit t = tile t): the steps only test bits.  Q tiles of more than
    // 64 tiles (transient-global over very long inputs) classify every tile when they reach it.
    unsigned long long cls_skip = 0, cls_mask = 0, cls_lut = 0, cls_right = 0;
    const bool cls_bits = RUNS && ntiles <= 64;   // (with many tiles per q tile, classifying them up front costs more than it saves)
    auto fill_classes = [&]() {
        cls_skip = cls_mask = cls_lut = cls_right = 0;
        if (!cls_bits) return;
        if (!(BITS && kbits != nullptr)) {
            // lane t classifies tile t: some fifty vector instructions for all tiles together instead of as many
            // scalar ones per tile, in a place where nothing else issues beside them (with validity bit sets the
            // look-ups would become vector loads, which wait for the tile requests: those go tile by tile)
            const TileClass c = classify_sparse(lane);
            const bool in = lane < ntiles;
            cls_skip = __builtin_amdgcn_ballot_w64(in && c.skip);
            cls_mask = __builtin_amdgcn_ballot_w64(in && c.need_mask);
            cls_lut = __builtin_amdgcn_ballot_w64(in && c.use_lut);
            cls_right = __builtin_amdgcn_ballot_w64(in && c.side == 2);
            return;
        }
        for (int t = 0; t < ntiles; ++t) {
            const TileClass c = classify_sparse(t);
            const unsigned long long bit = 1ull << t;
            if (c.skip) cls_skip |= bit;
            if (c.need_mask) cls_mask |= bit;
            if (c.use_lut) cls_lut |= bit;
            if (c.side == 2) cls_right |= bit;
        }
    };
    auto classify = [&](int t) {
        TileClass c;
        c.sg = 0; c.j0 = 0; c.side = 0; c.skip = true; c.use_lut = false; c.need_mask = false;
        if (t >= ntiles) return c;
        if (DENSE) {
            c.j0 = t * BN;
            c.skip = t >= d_ts;
            const bool left_sat = t < d_tl, right_sat = t >= d_tr;
            c.use_lut = has_lut && !(left_sat || right_sat);
            c.need_mask = t >= d_tm;
            c.side = (has_bias && !c.use_lut && !c.skip) ? (left_sat ? 1 : 2) : 0;
            return c;
        }
        if (!cls_bits) return classify_sparse(t);
        tile_of(t, c.sg, c.j0);
        const unsigned long long bit = 1ull << t;
        c.skip = (cls_skip & bit) != 0;
        c.need_mask = (cls_mask & bit) != 0;
        c.use_lut = win_lut || (cls_lut & bit) != 0;
        c.side = (!win_lut && has_bias && !c.use_lut && !c.skip) ? ((cls_right & bit) != 0 ? 2 : 1) : 0;
        return c;
    };

    // ---------------------------------------------------------------- running state
    f32x16 ot[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) ot[dt][r] = 0.f;
    float m_run = 0.f;       // running max (base-2 units), meaningful once `started`
    float l_run = 0.f;       // running sum over this lane's half of the keys (two partial sums)
    float l_alt = 0.f;
    bool started = false;    // a finite score has been seen for this row
    // wavefront-uniform: every row's running max is still exactly 0 (rows start there unless their first scores
    // are huge or tiny), so a LUT tile's accumulator input is the LUT entry itself, without a subtraction
    bool m_zero = true;
    // accumulator input of tiles with a constant bias: (constant - m_run) in all 16 slots.  It is
    // rewritten in ONE place per step, when the running max was raised or the tiles crossed to
    // the other saturated side, so the common path carries no copies of it.
    f32x16 cm;
    int side_cur = 0;
    float cb_cur = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) cm[r] = 0.f;

    // Query positions in each segment's bias geometry, once per q tile (they take integer divisions by run-time
    // values, some forty instructions each: not something for every tile): the wavefront's range and this lane's own.
    const int aux_shift = (TG && p.aux > 0 && (p.aux & (p.aux - 1)) == 0) ? __builtin_ctz((unsigned)p.aux) : -1;
    auto position_of = [&](int kind, int row) {
        if (kind == 0) return row + P;
        // (the rows of a q tile lie in block blk: no division; a row past the block's end is never stored)
        if (kind == 1) return (BLOCK && !gsplit) ? row - blk * p.block_len + p.aux : row % p.block_len + p.aux;
        // (side blocks of 2^k tokens, the usual case: a shift instead of a division)
        const int side = aux_shift >= 0 ? row >> aux_shift : row / p.aux;
        return min(side, n_side - 1);   // trailing tokens past the last full block join it
    };
    constexpr bool POS_CACHE = BLOCK || TG;   // (the other patterns' positions are row + P)
    auto set_positions = [&]() {
        if constexpr (!POS_CACHE) return;
        const int ir = min(irow, max(row_end - 1, iw0));   // rows past the end are never stored: keep them in range
        lq_pos[0] = position_of(seg_kind[0], ir);
        wq_lo[0] = position_of(seg_kind[0], iw0);
        wq_hi[0] = seg_kind[0] == 1 ? wq_lo[0] + 31 : position_of(seg_kind[0], iw1);
        if (nseg > 1) {
            lq_pos[1] = position_of(seg_kind[1], ir);
            wq_lo[1] = position_of(seg_kind[1], iw0);
            wq_hi[1] = seg_kind[1] == 1 ? wq_lo[1] + 31 : position_of(seg_kind[1], iw1);
        }
    };
    set_positions();
    auto lane_qpos = [&](int sg) {
        if constexpr (POS_CACHE) return sg ? lq_pos[1] : lq_pos[0];
        else return min(irow, max(row_end - 1, iw0)) + P;
    };

    // K fragments of one tile (16-bit types): issued early so that the LDS latency hides behind
    // the softmax head of the previous tile
    auto read_k = [&](int buf, v8 (&ka)[NT][KS]) {
        if constexpr (!F32) {
            const T* ks = Ks + buf * K_TILE;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const int row = 32 * nt + lr;
#pragma unroll
                for (int s = 0; s < KS; ++s)
                    ka[nt][s] = *reinterpret_cast<const v8*>(ks + row * D + (((2 * s + hh) ^ G::kswz(row)) * 8));
            }
        }
    };

    // S^T = K Q^T + C for one tile, C = bias - running max (cm must be current for constant tiles)
    auto lut_acc = [&](const TileClass& c, f32x16 (&st)[NT]) {
        const int qpos = lane_qpos(c.sg);
        {
            const float m_neg = -m_run * inv_c1;
            const int e0 = c.j0 + 4 * hh - qpos + padl;
            const float* lb = lut + (e0 & 3) * qlen;
            const int y0 = e0 >> 2;
            if (!DENSE && m_zero && !exact) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const f32x4 bq = *reinterpret_cast<const f32x4*>(lb + 4 * (y0 + 8 * nt + 2 * g));
#pragma unroll
                        for (int x = 0; x < 4; ++x) st[nt][4 * g + x] = bq[x];
                    }
            } else {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int y = y0 + 8 * nt + 2 * g;   // always inside the LUT, see LUT_PAD
                        const f32x4 bq = *reinterpret_cast<const f32x4*>(lb + 4 * y);
#pragma unroll
                        for (int x = 0; x < 4; ++x)
                            st[nt][4 * g + x] = __builtin_fmaf(bq[x], inv_c1, m_neg);
                    }
            }
        }
    };
    auto compute_s = [&](const TileClass& c, int buf, const v8 (&ka)[NT][KS], f32x16 (&st)[NT]) {
        if (c.use_lut) lut_acc(c, st);
        if constexpr (F32) {
            const T* ks = Ks + buf * K_TILE;
            if (!c.use_lut) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) st[nt] = cm;
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const int row = 32 * nt + lr;
#pragma unroll
                for (int s = 0; s < KS; ++s) st[nt] = E::mfma(ks[row * KSTR + 2 * s + hh], qf[s], st[nt]);
            }
        } else {
            if (c.use_lut) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int s = 0; s < KS; ++s) st[nt] = E::mfma(ka[nt][s], qf[s], st[nt]);
            } else {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    st[nt] = E::mfma(ka[nt][0], qf[0], cm);   // cm stays live: untied accumulator input
#pragma unroll
                    for (int s = 1; s < KS; ++s) st[nt] = E::mfma(ka[nt][s], qf[s], st[nt]);
                }
            }
            if constexpr (exact) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) st[nt][r] *= p.c1;
            }
        }
    };

    // mask, row max, lazy raise of the running max; returns true when m_run changed
    // mask of a tile that needs one (the first part of the softmax head)
    auto head_mask = [&](const TileClass& c, f32x16 (&st)[NT]) {
        if (c.need_mask) {   // keys past the end of the segment, or outside the window
            const int s_end = (c.sg ? seg_end[1] : seg_end[0]);
            const bool win = (c.sg ? seg_win[1] : seg_win[0]) != 0 && !win_lut;
            const int qpos = lane_qpos(c.sg);
            // this lane's row sees the keys [lo, hi): one subtraction and one unsigned compare per element
            const int seg_lo = (c.sg == 0 && (LOCAL || TG)) ? key_lo : 0;   // first key of the sequence
            const int lo = win ? max(seg_lo, qpos - p.block_len + 1) : seg_lo;
            const int hi = win ? min(s_end, qpos + p.block_len) : s_end;
            const unsigned span = (unsigned)max(hi - lo, 0);
            const int jl = c.j0 + 4 * hh - lo;
            // block pattern on a padded sequence: a range of the own block's keys that the rows do not see
            int hole_lo = 0, hole_span = 0;
            if (MODE == kBlockBits && c.sg == 1) block_hole(hole_lo, hole_span);
            const unsigned hspan = (unsigned)hole_span;
            const int jh = c.j0 + 4 * hh - hole_lo;
            // masks of any shape: this lane's keys of the tile's validity bits, bit `off` below
            unsigned long long vm = ~0ull;
            if (BITS && kbits != nullptr) vm = tile_valid(c.sg, c.j0) >> (4 * hh);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int off = 32 * nt + 8 * (r >> 2) + (r & 3);
                    bool keep = (unsigned)(jl + off) < span;
                    if (MODE == kBlockBits) keep = keep && !((unsigned)(jh + off) < hspan);
                    if (BITS) keep = keep && ((vm >> off) & 1ull) != 0;
                    st[nt][r] = keep ? st[nt][r] : -INFINITY;
                }
        }
    };
    // the two parts of the head after the mask: the maximum of this lane's half of the row's keys (the other half
    // sits in lane ^ 32 and is only consulted in the rare block: "some lane of the wavefront must raise" is the
    // same question for halves and for rows) ...
    auto head_max = [&](const f32x16 (&st)[NT]) {
        // st already holds (score - m_run)
        float pm[4];   // four independent partial maxima: short dependency chains
#pragma unroll
        for (int c = 0; c < 4; ++c) pm[c] = st[0][4 * c];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int x = 0; x < 4; ++x) pm[c] = max_ieee(pm[c], st[nt][4 * c + x]);
        return max_ieee(max_ieee(pm[0], pm[1]), max_ieee(pm[2], pm[3]));
    };
    // ... and the lazy raise of the running max, when some lane asks for it; returns true when m_run changed.  (The
    // last step of a run of fast steps forms a product past the last tile: it calls this with trigger == false,
    // which leaves the running state alone.)
    auto head_trigger = [&](float mh) {   // (no short-circuit: both tests are one compare, a branch around one costs more)
        const bool hot = mh > raise_limit<T>();
        const bool first = (!started) & (mh > -INFINITY);
        return __any(hot | first) != 0;
    };
    auto head_raise = [&](f32x16 (&st)[NT], float mh, bool trigger) {
        if (trigger) {
            asm volatile("");   // keep this rare block a real branch
            const float mx = xhalf_max(mh);
            // a row's first finite scores: the running max stays at 0 when they are moderate (probabilities
            // between 2^-100 and 2^24 are safe in bf16 / fp32 and fp16's limit is lower still), else it goes to them
            // (sparse patterns only, where most tiles take their bias from the LUT; dense rows go to their first
            // maximum: there the zero start costs long sequences 1 %)
            const bool fresh = !started && mx > -INFINITY;
            const bool raise = (mx > raise_limit<T>()) || (fresh && (DENSE || mx < start_floor<T>()));
            const float delta = raise ? mx : 0.f;
            const float scale = started ? __builtin_amdgcn_exp2f(-delta) : 0.f;
            m_run += delta;
            started = started || fresh;
            m_zero = m_zero && !__any(raise);
            l_run *= scale;
            l_alt *= scale;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int r = 0; r < 16; ++r) st[nt][r] -= delta;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) ot[dt][r] *= scale;
            return true;
        }
        return false;
    };
    auto softmax_head = [&](const TileClass& c, f32x16 (&st)[NT]) {
        head_mask(c, st);
        const float mh = head_max(st);
        return head_raise(st, mh, head_trigger(mh));
    };

    // P = exp2(S^T);  O^T += V^T P^T
    // per-lane part of the transposing V reads (LDS-DMA path): within a group of 16 lanes, lane
    // r = 4j + a supplies the address of V[key j][4a .. 4a+3] and receives, for head dim (lane % 16),
    // the four keys j = 0..3 -- one 16 x 4 fragment of V^T per read, two reads per MFMA operand.
    int vtr_off[DT];   // element offsets per 32-dim block (before the per-block constants)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) vtr_off[dt] = 0;
    if constexpr (DMA) {
        const int g = lane >> 4, r = lane & 15, jj = r >> 2, aa = r & 3;
        const int row = 4 * (g >> 1) + jj;                      // + 32 nt + 16 u (+ 8 for the second read)
        const int x = 2 * (g & 1) + (aa >> 1);
        const int fb = G::vrow_swz(row) >> 2;                   // which 64-byte part of the row holds block 0
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) vtr_off[dt] = row * D + ((4 * (dt ^ fb) + x) * 8) + (aa & 1) * 4;
    }
    auto compute_pv = [&](int buf, f32x16 (&st)[NT]) {
        const T* vs = Vs + buf * V_TILE;
        if constexpr (DMA && D == 64) {
            // Four groups of 16 keys.  The V^T fragments of group g + 1 are requested before the exponentials of
            // group g, into a second set of registers, so that no product waits for the LDS; the scheduling fences
            // keep the requests where they are (left alone, the compiler puts each one directly before its
            // product when registers are scarce, and every product then waits a full LDS round trip).
            typedef short s16x4 __attribute__((ext_vector_type(4)));
            typedef short s16x8 __attribute__((ext_vector_type(8)));
            auto vread = [&](int g, int dt) {
                const T* a0 = vs + vtr_off[dt] + 16 * g * D;
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0));
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0 + 8 * D));
                return __builtin_bit_cast(v8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
            };
            v8 vf[2][DT];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) vf[0][dt] = vread(0, dt);
#pragma unroll
            for (int g = 0; g < 2 * NT; ++g) {
                const int nt = g >> 1, u = g & 1;
                if (g + 1 < 2 * NT) {
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) vf[(g + 1) & 1][dt] = vread(g + 1, dt);
                }
                __builtin_amdgcn_sched_barrier(0x40F);   // ALU and matrix instructions may cross, LDS reads may not
                f32x8 pv;
#pragma unroll
                for (int x = 0; x < 8; ++x) pv[x] = __builtin_amdgcn_exp2f(st[nt][8 * u + x]);
                const v8 pb = __builtin_convertvector(pv, v8);
                if (u == 0) l_run = E::sum8(pb, l_run); else l_alt = E::sum8(pb, l_alt);
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) ot[dt] = E::mfma(vf[g & 1][dt], pb, ot[dt]);
                __builtin_amdgcn_sched_barrier(0x40F);
            }
        } else if constexpr (DMA) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    f32x8 pv;
#pragma unroll
                    for (int x = 0; x < 8; ++x) pv[x] = __builtin_amdgcn_exp2f(st[nt][8 * u + x]);
                    const v8 pb = __builtin_convertvector(pv, v8);
                    if (u == 0) l_run = E::sum8(pb, l_run); else l_alt = E::sum8(pb, l_alt);
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        typedef short s16x4 __attribute__((ext_vector_type(4)));
                        typedef short s16x8 __attribute__((ext_vector_type(8)));
                        const T* a0 = vs + vtr_off[dt] + (32 * nt + 16 * u) * D;
                        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0));
                        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0 + 8 * D));
                        const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                        ot[dt] = E::mfma(__builtin_bit_cast(v8, both), pb, ot[dt]);
                    }
                }
        } else if constexpr (F32) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float e = __builtin_amdgcn_exp2f(st[nt][r]);
                    l_run += e;
                    // MFMA k-slot = lane half: half 0 feeds key 8g+t, half 1 key 8g+4+t
                    const int key = 32 * nt + 8 * (r >> 2) + 4 * hh + (r & 3);
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
                        ot[dt] = E::mfma(vs[key * VROWS + 32 * dt + lr], e, ot[dt]);
                }
        } else {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    f32x8 pv;
#pragma unroll
                    for (int x = 0; x < 8; ++x) pv[x] = __builtin_amdgcn_exp2f(st[nt][8 * u + x]);
                    const v8 pb = __builtin_convertvector(pv, v8);
                    if (u == 0) l_run = E::sum8(pb, l_run); else l_alt = E::sum8(pb, l_alt);
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        const int d = 32 * dt + lr;
                        const v8 a = *reinterpret_cast<const v8*>(vs + d * BN + (((4 * nt + 2 * u + hh) ^ G::vswz(d)) * 8));
                        ot[dt] = E::mfma(a, pb, ot[dt]);
                    }
                }
        }
    };

    auto refill_cm = [&](int side) {
        asm volatile("");
        if (side != 0) side_cur = side;
        cb_cur = side_cur == 1 ? c_neg : (side_cur == 2 ? c_pos : 0.f);
#pragma unroll
        for (int r = 0; r < 16; ++r) cm[r] = (cb_cur - m_run) * inv_c1;
    };

    // ---------------------------------------------------------------- software pipeline
    // Step t:   S MFMAs of tile t+1 with the exponentials of tile t  ->  PV MFMAs of tile t with the softmax head
    // (row maxima, row sums) of tile t+1.
    // A wavefront issues in order and the matrix pipe takes one 32x32x16 product per 32 cycles, so a burst of
    // products stalls its wavefront while the vector ALUs idle, and a stretch of vector work leaves the matrix pipe
    // idle: each half of the step pairs matrix work with vector work that does not depend on it, interleaved
    // instruction by instruction (the fast steps fix that order with scheduling groups).  K tiles are staged two
    // steps ahead and V tiles one step ahead, each in two LDS buffers, with one barrier per step.
    //
    // LDS-DMA path: K(t+4) and V(t+3) are requested in step t into four-stage rings; every step
    // issues the same number of loads per wavefront (2 * SPW; tiles past the end fetch zeros), so
    // "at most two steps' worth outstanding" before the barrier means the tiles of the next step
    // have landed.
    f32x16 sta[NT], stb[NT];
    fill_classes();
    TileClass tc = classify(0);
    // q tiles whose tiles all have the same classes: away from the ends of the sequence (local pattern); whole
    // blocks other than the first, one q tile each, of a sequence without padding (block pattern)
    auto is_interior = [&]() {
        if (BITS && kbits != nullptr) return false;   // (every q tile looks its keys' validity up)
        if (LOCAL) return seg_start[0] >= key_lo && i0 + BM - 1 + p.block_len <= Nseq && i0 + BM <= Mseq;
        if (BLOCK) return !gsplit && tpb == 1 && blk >= 1 && (blk + 1) * p.block_len <= min(Nseq, n_valid) && i0 + BM <= Mseq;
        return false;
    };
    const bool first_interior = is_interior();
    if constexpr (QDMA) {
        // K0 and V0 landed before the barrier that published the LUT
    } else {
        if constexpr (DMA) {
            __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): the tiles requested at the top have landed
        } else if (ntiles > 0) {
            load_tile_k(0); load_tile_v(0);
            store_tile_k(0); store_tile_v(0);
            if (ntiles > 1) { load_tile_k(1); store_tile_k(1); }
        }
        __syncthreads();
    }
    if (tc.side != 0) refill_cm(tc.side);
    T5A_PHASE_VARS;
    bool head_refill = false;   // the head of the current tile moved the running max: cm is stale
    if (ntiles > 0 && !tc.skip) {
        v8 ka0[NT][KS];
        read_k(0, ka0);
        compute_s(tc, 0, ka0, sta);
        head_refill = softmax_head(tc, sta);
    }
    if constexpr (QDMA) wait_vmcnt<3 * G::SPW>();   // K1 has landed; V1 K2 V2 may still be in flight
    __syncthreads();   // the first step overwrites the K buffer this product was read from
    if constexpr (QDMA) {   // K3, into the stage that held the Q rows of two wavefronts
        if constexpr (CURSOR) dma_next(false); else dma_tile(3, false);
    }

    // End of a step: everything but the last two steps' requests has landed.  RUNS: the first two steps of a q tile
    // may also leave the row stores of the q tile before it in flight (2 * DT store instructions per wavefront, issued
    // after the requests that these steps wait for and before their own: requests and stores complete in issue order).
    int relaxed = 0;
    auto step_wait = [&]() {
        if constexpr (RUNS) {
            if (relaxed > 0) { --relaxed; wait_vmcnt<4 * G::SPW + 2 * DT>(); return; }
        }
        wait_vmcnt<4 * G::SPW>();   // everything but the last two steps' requests
    };
    auto step = [&](int t, f32x16 (&st)[NT], f32x16 (&st_next)[NT]) {
        const int kbuf_next = DMA ? (tbase + t + 1) % NSK : (t + 1) & 1;
        const int vbuf = DMA ? (tbase + t) % NSV : t & 1;
        if constexpr (CURSOR) {
            dma_next(false);
            dma_next(true);
        } else if constexpr (DMA) {
            dma_tile(t + 4, false);
            dma_tile(t + 3, true);
        } else {
            if (t + 2 < ntiles) load_tile_k(t + 2);
            if (t + 1 < ntiles) load_tile_v(t + 1);
        }
        const TileClass nx = classify(t + 1);
        v8 ka[NT][KS];
        if (!nx.skip) read_k(kbuf_next, ka);
        if constexpr (!win_lut) {   // (with the window in the LUT no tile has a constant accumulator input)
            if (head_refill || (nx.side != 0 && nx.side != side_cur)) refill_cm(nx.side);
        }
        head_refill = false;
        if (!nx.skip) compute_s(nx, kbuf_next, ka, st_next);
        if (!tc.skip) compute_pv(vbuf, st);
        if (!nx.skip) head_refill = softmax_head(nx, st_next);
        tc = nx;
        if constexpr (DMA) {
            step_wait();
            barrier_lds_only();
        } else {
            if (t + 2 < ntiles) store_tile_k(t & 1);
            if (t + 1 < ntiles) store_tile_v((t + 1) & 1);
            __syncthreads();
        }
    };
    // Both halves of a fast step at head_dim 64 as one instruction stream: sixteen groups, each one matrix product
    // with the vector work that runs beside it, kept in this order by scheduling fences (what the compiler does with
    // the same statements unfenced: all exponentials first, all maxima last, and the matrix pipe idle meanwhile).
    // The first two S products (k-step 0 of both key blocks) are issued by the caller, which knows their accumulator
    // input.
    auto fused_halves = [&](bool live, int vstage, const v8 (&ka)[NT][KS], f32x16 (&st)[NT], f32x16 (&st_next)[NT]) {
        if constexpr (DMA && D == 64) {
            static_assert(NT == 2 && KS == 4 && DT == 2, "four groups of 16 keys, two products each");
            typedef short s16x4 __attribute__((ext_vector_type(4)));
            typedef short s16x8 __attribute__((ext_vector_type(8)));
            const T* vs = Vs + vstage * V_TILE;
            v4 ph[8];        // P, four keys per entry
            v8 vf[4][DT];    // V^T fragments
            auto vread = [&](int g, int dt) {
                const T* a0 = vs + vtr_off[dt] + 16 * g * D;
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0));
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0 + 8 * D));
                vf[g][dt] = __builtin_bit_cast(v8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
            };
            __builtin_amdgcn_sched_barrier(0);
            // first half: exponentials of tile t beside the S products of tile t+1; the V^T fragments of the first
            // 32 keys go into the registers of K fragments that are done with
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                f32x4 pv;
#pragma unroll
                for (int x = 0; x < 4; ++x) pv[x] = __builtin_amdgcn_exp2f(st[i >> 2][4 * (i & 3) + x]);
                ph[i] = __builtin_convertvector(pv, v4);
                if (i >= 2) st_next[i & 1] = E::mfma(ka[i & 1][i >> 1], qf[i >> 1], st_next[i & 1]);
                if (i >= 4) vread((i - 4) >> 1, (i - 4) & 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (exact) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) st_next[nt][r] *= p.c1;
            }
            // second half: PV products of tile t beside its row sums and the row maxima of tile t+1
            float pm[4];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int g = i >> 1, dt = i & 1;
                const v8 pb = __builtin_shufflevector(ph[2 * g], ph[2 * g + 1], 0, 1, 2, 3, 4, 5, 6, 7);
                ot[dt] = E::mfma(vf[g][dt], pb, ot[dt]);
                if (i < 4) vread(2 + (i >> 1), i & 1);
                if ((g & 1) == 0) l_run = E::sum4(ph[i], l_run); else l_alt = E::sum4(ph[i], l_alt);
                // maxima: chain c takes the slots 4c .. 4c+3 of both key blocks, two of them per group
                {
                    const int nt = i >> 2, c = i & 3;
                    const float a = max_ieee(st_next[nt][4 * c], st_next[nt][4 * c + 1]);
                    const float b2 = max_ieee(st_next[nt][4 * c + 2], st_next[nt][4 * c + 3]);
                    pm[c] = nt == 0 ? max_ieee(a, b2) : max_ieee(pm[c], max_ieee(a, b2));
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            const float mh = max_ieee(max_ieee(pm[0], pm[1]), max_ieee(pm[2], pm[3]));
            head_refill = head_raise(st_next, mh, live & head_trigger(mh));
        }
    };
    // Dense and packed modes at head_dim 64: the fast step without row maxima.
    //
    // The vector port, not the matrix pipe, bounds the step (per tile and wavefront: 32 exponentials at half rate,
    // 16 conversions, 16 row-sum instructions and the issue slots of 16 matrix products), so the 19 instructions of
    // the row maximum are worth removing, and the exponentials are worth spreading evenly over all sixteen products
    // instead of sitting beside eight of them:
    //  * No maximum.  The running max may lag behind by 2^24 anyway (raise_limit), and fp32 holds 2^127: whether it
    //    must be raised follows from the tile's row SUM, which the step forms anyway -- a lane's sum of 32
    //    probabilities above 2^24 (2^14 for fp16) means one of them is above 2^19, and only then the exact maximum is
    //    looked up (rare block below), the running max raised and the tile's exponentials formed again from its
    //    scores, which are still in registers.  The test comes BEFORE the tile's PV products, so an overflowing
    //    exponential (inf) never reaches the output accumulators, whatever the inputs.  No probability above the
    //    limit reaches the matrix core: without the trigger every one of them is at most the lane's sum.
    //  * A tile's exponentials in two halves: those of its first 32 keys beside the PV products of the tile before
    //    it (second half of the previous step, as soon as its scores exist), those of its last 32 keys beside the
    //    S products of the tile after it (first half of its own step).  Every product then has two exponentials,
    //    one conversion and one sum instruction beside it: 25 vector cycles against the product's 32.
    // Rows: every row that will ever see a key has seen one in tile 0 (the prologue's head is the exact one), so the
    // fast steps never start a row; a row without keys has scores of -inf, sums of 0 and never triggers.
    // State between the steps: pe = the packed probabilities of the early half of the tile whose scores wait in
    // registers, lt0 / lt1 = its partial row sums (kept apart from l_run until the tile has passed its test).
    constexpr bool V2 = DENSE && DMA && D == 64;
    unsigned pe[8];
    float lt0 = 0.f, lt1 = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) pe[j] = 0u;
    // two exponentials, packed, and added to a partial sum
    auto exp_pair = [&](float a, float b, float& acc) {
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        using v2 = typename E::v2;
        if constexpr (!F32) {
            const f32x2 e = {__builtin_amdgcn_exp2f(a), __builtin_amdgcn_exp2f(b)};
            const v2 pk = __builtin_convertvector(e, v2);
            acc = E::sum2(pk, acc);
            return __builtin_bit_cast(unsigned, pk);
        } else {
            return 0u;
        }
    };
    // entering a run of fast steps: the early half of the tile in `st` (its head has been done: no test needed)
    auto dense_enter = [&](const f32x16 (&st)[NT]) {
        if constexpr (V2) {
            lt0 = 0.f; lt1 = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) pe[j] = exp_pair(st[0][2 * j], st[0][2 * j + 1], (j & 1) ? lt1 : lt0);
        }
    };
    // (LAST: the step that reaches the item's last tile -- no S products and no early exponentials for a tile behind it)
    auto dense_halves = [&](auto last_c, int vstage, const v8 (&ka)[NT][KS], f32x16 (&st)[NT], f32x16 (&st_next)[NT]) {
        constexpr bool LAST = decltype(last_c)::value;
        if constexpr (V2) {
            static_assert(!V2 || (NT == 2 && KS == 4 && DT == 2), "four groups of 16 keys, two products each");
            typedef short s16x4 __attribute__((ext_vector_type(4)));
            typedef short s16x8 __attribute__((ext_vector_type(8)));
            const T* vs = Vs + vstage * V_TILE;
            unsigned pl[8];     // packed probabilities of the late half of tile t
            v8 vf[4][DT];       // V^T fragments
            auto vread = [&](int g, int dt) {
                const T* a0 = vs + vtr_off[dt] + 16 * g * D;
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0));
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(a0 + 8 * D));
                vf[g][dt] = __builtin_bit_cast(v8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
            };
            __builtin_amdgcn_sched_barrier(0);
            // first half: the late exponentials of tile t beside the S products of tile t+1
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                pl[i] = exp_pair(st[1][2 * i], st[1][2 * i + 1], (i & 1) ? lt1 : lt0);
                if constexpr (!LAST) {
                    if (i >= 2) st_next[i & 1] = E::mfma(ka[i & 1][i >> 1], qf[i >> 1], st_next[i & 1]);
                }
                if (i >= 4) vread((i - 4) >> 1, (i - 4) & 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (exact && !LAST) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) st_next[nt][r] *= p.c1;
            }
            // tile t's test: a lane's sum above the limit
            float lt = lt0 + lt1;
            if (__any(lt > __builtin_amdgcn_exp2f(raise_limit<T>()))) {
                asm volatile("");   // keep this rare block a real branch
                const float mx = xhalf_max(head_max(st));
                // (a triggering lane holds a probability above limit - 5: its row is raised)
                const bool raise = mx > raise_limit<T>() - 6.0f;
                const float delta = raise ? mx : 0.f;
                const float scale = __builtin_amdgcn_exp2f(-delta);
                m_run += delta;
                m_zero = m_zero && !__any(raise);
                l_run *= scale;
                l_alt *= scale;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) { st[nt][r] -= delta; if constexpr (!LAST) st_next[nt][r] -= delta; }
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) ot[dt][r] *= scale;
                lt0 = 0.f; lt1 = 0.f;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    pe[j] = exp_pair(st[0][2 * j], st[0][2 * j + 1], (j & 1) ? lt1 : lt0);
                    pl[j] = exp_pair(st[1][2 * j], st[1][2 * j + 1], (j & 1) ? lt1 : lt0);
                }
                lt = lt0 + lt1;
                head_refill = true;
            }
            l_run += lt;
            lt0 = 0.f; lt1 = 0.f;
            __builtin_amdgcn_sched_barrier(0);
            // second half: PV products of tile t beside the early exponentials of tile t+1
            unsigned pn[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int g = i >> 1, dt = i & 1;
                const u32x4 pw = g < 2 ? u32x4{pe[4 * g], pe[4 * g + 1], pe[4 * g + 2], pe[4 * g + 3]}
                                       : u32x4{pl[4 * g - 8], pl[4 * g - 7], pl[4 * g - 6], pl[4 * g - 5]};
                ot[dt] = E::mfma(vf[g][dt], __builtin_bit_cast(v8, pw), ot[dt]);
                if (i < 4) vread(2 + (i >> 1), i & 1);
                if constexpr (!LAST) pn[i] = exp_pair(st_next[0][2 * i], st_next[0][2 * i + 1], (i & 1) ? lt1 : lt0);
                else pn[i] = 0u;
                __builtin_amdgcn_sched_barrier(0);
            }
            // (pinned here: the compiler otherwise sinks the last step's exponentials of an unrolled group of four
            // to the loop's back edge, away from the products they are meant to run beside)
#pragma unroll
            for (int j = 0; j < 8; ++j) { pe[j] = pn[j]; asm volatile("" : "+v"(pe[j])); }
            asm volatile("" : "+v"(lt0), "+v"(lt1));
        }
    };
    // Fast step (LDS-DMA path): tiles t and t+1 are neither skipped nor masked, so the step is the
    // general one minus those cases.  ST is the step index modulo 4, which fixes every LDS stage at
    // compile time.
    int fc_until = 0, fc_side = 0;   // dense fast steps: class of the next tile, valid for tiles below fc_until
    bool fc_lut = false;
    auto fast_step_impl = [&](int t, auto st_c, auto last_c, f32x16 (&st)[NT], f32x16 (&st_next)[NT]) {
        constexpr int ST = decltype(st_c)::value;
        constexpr bool LAST = decltype(last_c)::value;   // nothing follows tile t: no product for a tile t + 1
        if constexpr (DENSE) cursor_dma(ST, (ST + 3) & 3);
        else if constexpr (CURSOR) { dma_next(false, ST); dma_next(true, (ST + 3) & 3); }
        else { dma_tile(t + 4, false, ST); dma_tile(t + 3, true, (ST + 3) & 3); }
        v8 ka[NT][KS];
        if constexpr (LAST) {
            static_assert(!LAST || V2, "only the dense steps without row maxima have this form");
            head_refill = false;
            dense_halves(last_c, ST, ka, st, st_next);
            tc.skip = true;
            T5A_PHASE(0);
            step_wait();
            barrier_lds_only();
            T5A_PHASE(1);
            return;
        }
        read_k((ST + 1) & 3, ka);
        TileClass nx;
        if constexpr (win_lut) {   // one segment, every tile takes its accumulator input from the LUT: nothing to look up
            nx.sg = 0; nx.j0 = i0 - p.block_len + 1 + (t + 1) * BN; nx.side = 0;
            nx.skip = t + 1 >= ntiles; nx.use_lut = true; nx.need_mask = false;
        } else if constexpr (DENSE) {
            // the class only changes at a few tile indices: look it up there, carry it along otherwise
            if (t + 1 >= fc_until) {
                const TileClass c = classify(t + 1);
                fc_lut = c.use_lut; fc_side = c.side;
                fc_until = t + 1 < d_tl ? d_tl : (t + 1 < d_tr ? d_tr : 0x7fffffff);
            }
            nx.sg = 0; nx.j0 = (t + 1) * BN; nx.side = fc_side;
            nx.skip = t + 1 >= ntiles; nx.use_lut = fc_lut; nx.need_mask = false;
            if (head_refill || (fc_side != 0 && fc_side != side_cur)) refill_cm(fc_side);
        } else {
            nx = classify(t + 1);
            if (head_refill || (nx.side != 0 && nx.side != side_cur)) refill_cm(nx.side);
        }
        head_refill = false;
        const bool live = !nx.skip;   // false in the last step of a run that ends with the last tile
        if constexpr (D == 64) {
            if (nx.use_lut) {
                lut_acc(nx, st_next);
                st_next[0] = E::mfma(ka[0][0], qf[0], st_next[0]);
                st_next[1] = E::mfma(ka[1][0], qf[0], st_next[1]);
            } else {
                st_next[0] = E::mfma(ka[0][0], qf[0], cm);   // cm stays live: untied accumulator input
                st_next[1] = E::mfma(ka[1][0], qf[0], cm);
            }
            if constexpr (V2) dense_halves(last_c, ST, ka, st, st_next);
            else fused_halves(live, ST, ka, st, st_next);
        } else {
            __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): one wait for all K fragments instead of one per MFMA
            compute_s(nx, (ST + 1) & 3, ka, st_next);
            compute_pv(ST, st);
            const float mh = head_max(st_next);
            head_refill = head_raise(st_next, mh, live & head_trigger(mh));
        }
        tc = nx;
        T5A_PHASE(0);
        step_wait();
        barrier_lds_only();
        T5A_PHASE(1);
    };
    auto fast_step = [&](int t, auto st_c, f32x16 (&st)[NT], f32x16 (&st_next)[NT]) {
        fast_step_impl(t, st_c, std::false_type{}, st, st_next);
    };
    // number of consecutive tiles from t on that are neither skipped nor masked
    auto plain_run = [&](int t) {
        if (DENSE) return max(0, min(min(d_ts, d_tm), ntiles) - t);
        if (cls_bits) {
            const unsigned long long bad = (cls_skip | cls_mask) >> t;
            return min(bad != 0 ? (int)__builtin_ctzll(bad) : 64, ntiles - t);
        }
        // window tiles: a wavefront's plain ones (every key inside the window of every row) start within an interval
        // of 2 * window - 94 keys; four fast steps take five plain tiles in a row, so narrow windows have none
        if (TG && t < seg_nt[0] && 2 * p.block_len - 94 < 5 * BN) return 0;
        if (TG && t >= seg_nt[0]) {
            // side tiles: none is skipped and only a last, partial one needs a mask -- no need to classify sixteen
            // tiles one by one (some fifty scalar instructions each) to find that out
            return max(0, min(ntiles, seg_nt[0] + seg_end[1] / BN) - t);
        }
        int n = 0;
        for (; t + n < ntiles; ++n) {
            const TileClass c = classify(t + n);
            if (c.skip || c.need_mask) break;
        }
        return n;
    };

    // rows of the current q tile: normalise, convert, store (and the log-sum-exp when asked for)
    auto store_rows = [&](const int irow, const int row_end_) {   // (a run stores a q tile's rows after it has moved on)
        const bool row_ok = irow < row_end_;
        const float l_tot = xhalf_sum(l_run + l_alt);
        const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
        if ((MODE == kDense && p.nsplit > 1) || gsplit) {
            // partial result of a key split: normalised row in fp32, weight 1 (0: no visible key) and log-sum-exp
            if (row_ok) {
                const int64_t prow = (((int64_t)b * p.H + h) * p.nsplit + split) * (gsplit ? Mseq : p.M) + irow;
                float* orow = p.part_o + prow * D;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int d0 = 32 * dt + 8 * g + 4 * hh;
                        if (d0 < D) {
                            f32x4 x;
#pragma unroll
                            for (int tt = 0; tt < 4; ++tt) x[tt] = ot[dt][4 * g + tt] * inv;
                            *reinterpret_cast<f32x4*>(orow + d0) = x;
                        }
                    }
                if (hh == 0) {
                    p.part_l[prow] = l_tot > 0.f ? 1.f : 0.f;
                    p.part_m[prow] = l_tot > 0.f ? (m_run + __builtin_log2f(l_tot)) * 0.6931471805599453f : -INFINITY;
                }
            }
        } else {
            const bool stored = row_ok && irow >= row_lo;
            T* orow = op + (int64_t)irow * p.o_sr;
            if constexpr (F32) {
                if (stored) {
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            const int d0 = 32 * dt + 8 * g + 4 * hh;
                            if (d0 < D) {
                                f32x4 x;
#pragma unroll
                                for (int tt = 0; tt < 4; ++tt) x[tt] = ot[dt][4 * g + tt] * inv;
                                *reinterpret_cast<f32x4*>(orow + d0) = x;
                            }
                        }
                }
            } else {
                // A lane holds four elements of every eight of its row, the lane 32 further on the other four.  The
                // two exchange halves, so that each stores 16 contiguous bytes per instruction: half as many store
                // instructions (2 600 -> 1 500 cycles for the rows of a q tile).  Going on to 64 contiguous bytes
                // per row (a second exchange between lanes 16 apart) changed nothing.
                typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
                typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int k = 0; k < 2; ++k) {
                        if (32 * dt + 16 * k < D) {
                            f32x4 xa, xb;
#pragma unroll
                            for (int tt = 0; tt < 4; ++tt) {
                                xa[tt] = ot[dt][8 * k + tt] * inv;
                                xb[tt] = ot[dt][8 * k + 4 + tt] * inv;
                            }
                            const u32x2 a = __builtin_bit_cast(u32x2, __builtin_convertvector(xa, v4));
                            const u32x2 b2 = __builtin_bit_cast(u32x2, __builtin_convertvector(xb, v4));
                            // (lanes 32..63 of the first operand trade places with lanes 0..31 of the second)
                            const auto s0 = __builtin_amdgcn_permlane32_swap(a[0], b2[0], false, false);
                            const auto s1 = __builtin_amdgcn_permlane32_swap(a[1], b2[1], false, false);
                            const u32x4 piece = {s0[0], s1[0], s0[1], s1[1]};   // elements 32 dt + 16 k + 8 hh .. + 7
                            if (stored) *reinterpret_cast<u32x4*>(orow + 32 * dt + 16 * k + 8 * hh) = piece;
                        }
                    }
            }
            if (stored && p.lse != nullptr && hh == 0) {
                const float ln2 = 0.6931471805599453f;
                p.lse[lse_off + (int64_t)irow * p.lse_sr] = l_tot > 0.f ? (m_run + __builtin_log2f(l_tot)) * ln2 : -INFINITY;
            }
        }
    };

    T5A_STAMP(3);
    bool interior = first_interior;   // the current q tile's classes hold for any q tile away from the ends of the sequence
    if constexpr (RUNS) prefetch_q(qt + 1);
    for (;;) {
        int t = 0;
        while (t < ntiles) {
            if (DMA && ((tbase + t) & 3) == 0 && (t & 1) == 0) {   // (even t: tile t's scores are in sta)
                // steps t .. t+3 are fast when tiles t .. t+4 are plain: run >= 5.  When the run reaches the
                // last tile, the final fast step forms an S product for a tile that does not exist (its K
                // stage holds zeros or a tile of the next q tile) and nobody consumes it, so the run may end
                // exactly there.
                const int run = plain_run(t);
                const bool ends = t + run >= ntiles;                   // the plain tiles reach the item's last tile
                const int fast = ends ? run : run - 1;                 // steps from here on that can be fast ones
                int quads = fast >> 2;
                // (dense kinds) a run that ends with the item's last tile on a group of four: that group is a copy of
                // its own behind the loop, whose last step leaves the product for a tile behind it out
                // (not with exact scores: that instantiation has no registers left for the copy)
                const bool peel = V2 && !exact && ends && quads > 0 && (fast & 3) == 0;
                if (peel) --quads;
                // dense kinds: two more fast steps behind the groups of four (ring stages 0 and 1), so that the tail of
                // a short or causal item takes fewer general steps
                const bool pair = V2 && fast >= 2 && (fast & 3) >= 2;
                const bool ran_fast = quads > 0 || pair || peel;
                if (ran_fast) {
                    tc = classify(t);
                    if constexpr (DENSE) { cursor_seek(t + 4, t + 3); fc_until = 0; }
                }
                if (ran_fast) T5A_PHASE_START();
                if (V2 && ran_fast) dense_enter(sta);
                while (quads > 0) {
                    fast_step(t, std::integral_constant<int, 0>{}, sta, stb);
                    fast_step(t + 1, std::integral_constant<int, 1>{}, stb, sta);
                    fast_step(t + 2, std::integral_constant<int, 2>{}, sta, stb);
                    fast_step(t + 3, std::integral_constant<int, 3>{}, stb, sta);
                    --quads; t += 4;
                }
                if constexpr (V2 && !exact) {
                    if (peel) {
                        fast_step(t, std::integral_constant<int, 0>{}, sta, stb);
                        fast_step(t + 1, std::integral_constant<int, 1>{}, stb, sta);
                        fast_step(t + 2, std::integral_constant<int, 2>{}, sta, stb);
                        fast_step_impl(t + 3, std::integral_constant<int, 3>{}, std::true_type{}, stb, sta);
                        t += 4;
                    }
                }
                if (pair) {
                    fast_step(t, std::integral_constant<int, 0>{}, sta, stb);
                    fast_step(t + 1, std::integral_constant<int, 1>{}, stb, sta);
                    t += 2;
                }
                // (the dense fast steps leave the tile that follows them without its head: the general step wants
                // it done; its early exponentials are simply formed again there)
                if (V2 && ran_fast && !tc.skip) head_refill = softmax_head(tc, sta) || head_refill;
                if (t >= ntiles) break;
            }
            step(t, sta, stb);
            if (t + 1 < ntiles) step(t + 1, stb, sta);
            t += 2;
        }
        T5A_STAMP(trace_slot); ++trace_slot;
        T5A_PHASE_STORE();
        if constexpr (!RUNS) {
            store_rows(irow, row_end);
            break;
        } else {
            // ------------------------------------------------------------ next q tile of the run
            // Its first tiles are in the rings already or on their way (the steps above requested them), the LUT
            // stays, its Q rows were requested a q tile ago.  What is left of a work item's set-up: the geometry
            // and the first score product.
            if (qt + 1 >= qt_last) { store_rows(irow, row_end); break; }
            // The Q rows come through ordinary loads, a q tile ahead.  The compiler copies the freshly requested
            // registers into the ones the loop carries at the loop's back edge, behind a wait for "nothing outstanding":
            // a full round trip to memory (2 300 cycles) when the request is the last thing the switch does.  So the
            // switch reads the rows it has, requests the next ones at once, and does everything else -- stores,
            // geometry, first product -- while they are on their way.
#pragma unroll
            for (int s = 0; s < KS; ++s) qf[s] = qn[s];
            if (!exact) {
#pragma unroll
                for (int s = 0; s < KS; ++s)
#pragma unroll
                    for (int e = 0; e < 8; ++e) qf[s][e] = (T)((float)qf[s][e] * p.c1);
            }
            __builtin_amdgcn_sched_barrier(0);
            prefetch_q(qt + 2);
            __builtin_amdgcn_sched_barrier(0);
            // (a wavefront none of whose rows is stored issues no store at all)
            relaxed = __builtin_amdgcn_ballot_w64(row_ok && irow >= row_lo) != 0 ? 2 : 0;
            store_rows(irow, row_end);
            ++qt;
            tbase += ntiles;
            set_qtile(qt);
            iw0 = i0 + wave * 32; iw1 = iw0 + 31; irow = iw0 + lr; row_ok = irow < row_end;
            set_positions();
            // away from the ends of the sequence every q tile of the local pattern has the same classes
            const bool was_interior = interior;
            interior = is_interior();
            if (!(interior && was_interior)) fill_classes();
            tc = classify(0);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) ot[dt][r] = 0.f;
            m_run = 0.f; l_run = 0.f; l_alt = 0.f; started = false; m_zero = true;
            side_cur = 0; cb_cur = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) cm[r] = 0.f;
            if (tc.side != 0) refill_cm(tc.side);
            head_refill = false;
            if (!tc.skip) {
                v8 ka0[NT][KS];
                read_k(tbase % NSK, ka0);
                compute_s(tc, tbase % NSK, ka0, sta);
                head_refill = softmax_head(tc, sta);
            }
            barrier_lds_only();   // the first step's request overwrites the K stage this product was read from
            T5A_STAMP(trace_slot); ++trace_slot;
        }
    }
    if constexpr (!RUNS) {
        break;
    } else {
        run_left -= qt_count;
        run_next += qt_count;
        if (run_left <= 0) break;
        // the run goes on in the next (batch, head): nothing of this one may still be on its way into the rings
        // (the last steps requested tiles past the end: zeros), and every wavefront must be done with the LUT
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
        __syncthreads();
    }
    }
}

// ------------------------------------------------------------------------ launch
template <typename T, int D, int MODE, bool CAUSAL, bool EXACT>
static hipError_t launch_exact(const FwdParams& p, hipStream_t stream) {
    int sat = p.table != nullptr ? p.bs.sat : 0;
    if (MODE == kLocal) sat = std::max(sat, p.block_len);   // window folded into the LUT
    // the LUT image rounded up to 1 KB (its LDS-DMA requests are that long) and 256 bytes per wavefront
    // for the table column
    const size_t lut_bytes = (((size_t)16 * lut_quads(sat, CAUSAL) * sizeof(float) + 1023) & ~(size_t)1023) + 1024;
    const size_t smem = Geometry<T, D>::kTileBytes + lut_bytes;
    auto kern = fwd_kernel<T, D, MODE, CAUSAL, EXACT>;
    // per instantiation and device: largest dynamic LDS size already allowed (the attribute belongs to the
    // function as loaded on one device)
    constexpr int kMaxDevices = 64;
    static std::atomic<size_t> granted[kMaxDevices] = {};
    int dev = 0;
    if (smem > 48 * 1024) {
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return e;
        const bool known = dev >= 0 && dev < kMaxDevices;
        if (!known || smem > granted[dev].load(std::memory_order_relaxed)) {
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
            if (e != hipSuccess) return e;
            if (known) granted[dev].store(smem, std::memory_order_relaxed);
        }
    }
    unsigned grid = (unsigned)(((p.total_items + 7) / 8) * 8);
    if ((MODE == kBlock || MODE == kBlockBits) && p.block_items > 0)
        grid = (unsigned)(((p.total_items - p.block_items + 7) / 8) * 8 + ((p.block_items + 7) / 8) * 8);
    if (MODE == kPacked && p.plan != nullptr) grid = 8u * (unsigned)p.plan_slots;
    if (CAUSAL && MODE == kDense && p.xcd_lo[8] > 0) {
        unsigned most = 0;
        for (int x = 0; x < 8; ++x)
            if (p.xcd_lo[x + 1] > p.xcd_lo[x])
                most = std::max(most, (unsigned)((p.xcd_lo[x + 1] - 1) / p.tiles_per_seq - p.xcd_lo[x] / p.tiles_per_seq + 1));
        grid = 8u * most * (unsigned)p.tiles_per_seq;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(NTHREADS), smem, stream, p);
    return hipGetLastError();
}

template <typename T, int D, int MODE, bool CAUSAL>
static hipError_t launch_one(const FwdParams& p, hipStream_t stream) {
    if constexpr (sizeof(T) == 2) {
        if (p.exact_scale != 0) return launch_exact<T, D, MODE, CAUSAL, true>(p, stream);
    }
    return launch_exact<T, D, MODE, CAUSAL, false>(p, stream);
}

template <typename T, int D>
static hipError_t launch_mode(const FwdParams& p, int mode, bool causal, hipStream_t s) {
    switch (mode) {
        case kDense: return causal ? launch_one<T, D, kDense, true>(p, s) : launch_one<T, D, kDense, false>(p, s);
        case kPacked: return causal ? launch_one<T, D, kPacked, true>(p, s) : launch_one<T, D, kPacked, false>(p, s);
        case kLocal: return launch_one<T, D, kLocal, false>(p, s);
        case kLocalWide: return launch_one<T, D, kLocalWide, false>(p, s);
        case kBlock: return launch_one<T, D, kBlock, false>(p, s);
        case kBlockBits: return launch_one<T, D, kBlockBits, false>(p, s);
        case kTGlobal: return launch_one<T, D, kTGlobal, false>(p, s);
        case kTGlobalBits: return launch_one<T, D, kTGlobalBits, false>(p, s);
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

#if defined(T5A_TRACE) && T5A_UNIT_DTYPE == 0
// measurement builds only: copies the stamps (kTraceItems x kTraceSlots 64-bit shader-clock values) to the host
extern "C" int t5a_trace_read(unsigned long long* out, int clear) {
    hipError_t e = hipMemcpyFromSymbol(out, HIP_SYMBOL(t5a::t5a_trace_buf), sizeof(unsigned long long) * t5a::kTraceItems * t5a::kTraceSlots);
    if (e == hipSuccess && clear) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(t5a::t5a_trace_buf));
        if (e == hipSuccess) e = hipMemset(ptr, 0, sizeof(unsigned long long) * t5a::kTraceItems * t5a::kTraceSlots);
    }
    return (int)e;
}
#endif
