// Internal declarations shared by the host API and the HIP kernels of libt5attn.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/t5attn.h"

namespace t5a {

constexpr int kMaxThresholds = 128;   // supports num_buckets up to 256
constexpr int kMaxSaturation = 1024;  // largest distance at which buckets still change

// Integer description of the T5 bucket function, derived on the host from the
// per-distance table so that device code never evaluates a logarithm.
// For distance d >= max_exact the bucket is max_exact + #{t : thr[t] <= d}.
struct BucketSpec {
    int bidirectional;
    int nb;         // buckets per direction (num_buckets/2 if bidirectional)
    int max_exact;  // nb / 2
    int n_thr;
    int sat;        // every |rel| >= sat maps to the last bucket of its side
    int thr[kMaxThresholds];
};

// kPacked: dense semantics per sequence of a packed batch (cu_seqlens); a separate instantiation, so that
// the unpacked kernel carries none of its work-item search
// kLocal: sliding window of at most kMaxLutWindow, folded into the distance LUT; kLocalWide: wider windows, masked
// per element at their edges, and masks of any shape; kTGlobalBits, kBlockBits: the transient-global and block
// patterns with masks of any shape
enum Mode { kDense = 0, kLocal = 1, kBlock = 2, kTGlobal = 3, kPacked = 4, kLocalWide = 5, kTGlobalBits = 6, kBlockBits = 7 };
// widest sliding window that is folded into the distance LUT (the LUT then spans 2 * (window + 96) distances;
// 256 keeps it below 12 KB of LDS, so that two workgroups still share a compute unit)
constexpr int kMaxLutWindow = 256;
constexpr int kMaxRunLen = 16;     // most q tiles of one (batch, head) that a sparse work item takes
constexpr int kKeyBitsFront = 8;   // zero words in front of a sequence's validity bits (tiles start up to 255 keys early)

struct FwdParams {
    const void* q; const void* k; const void* v; void* o; float* lse;
    const void* side_k; const void* side_v;
    int64_t q_sb, q_sh, q_sr;
    int64_t k_sb, k_sh, k_sr;
    int64_t v_sb, v_sh, v_sr;
    int64_t o_sb, o_sh, o_sr;
    int64_t sk_sb, sk_sh, sk_sr;
    int64_t sv_sb, sv_sh, sv_sr;
    int64_t lse_sb, lse_sh, lse_sr;
    const int32_t* cu_q; const int32_t* cu_k;   // non-null: packed variable-length batch
    const int32_t* len_q; const int32_t* len_k; // optional lengths (rows between cu[b]+len[b] and cu[b+1] are padding)
    const int32_t* start_k;                     // sparse patterns, optional: first token of each sequence (left padding)
    // local and block patterns, optional: token validity as a bit set, (B, key_bits_stride) words; token j is bit
    // (j & 31) of word kKeyBitsFront + (j >> 5); zero words in front and behind
    const uint32_t* key_bits; int64_t key_bits_stride;
    const int32_t* side_counts;                 // transient-global pattern with key_bits: side tokens per sequence
    // packed batch with a launch plan (plan.hip): workgroup 8 k + x runs the item in plan[x][k]
    const int32_t* plan; const int32_t* plan_counts; int plan_slots;
    int B, H, M, N;
    int tiles_per_seq;   // q tiles per (batch, head) when not packed
    // sparse patterns with 16-bit inputs at head_dim 64 / 128: a work item is a run of run_len consecutive q tiles
    // of one (batch, head) (the last run of a pair may be shorter); total_items = runs_per_seq * H * B
    int run_len, runs_per_seq;
    int total_items;     // number of (q tile, head, batch) work items (upper bound when packed)
    // causal, unpacked, no key split (xcd_lo[8] > 0): items shrink with the tile index, so the list (pair-major,
    // longest tile first inside a (batch, head) pair) is cut into 8 slices of equal WORK, xcd_lo[x] .. xcd_lo[x+1]
    // for XCD x, and an XCD visits its slice level by level: the longest tiles of all its pairs first, so that
    // the kernel's tail is made of short items
    int xcd_lo[9];
    float c1;            // sm_scale * log2(e)
    int exact_scale;     // 16-bit inputs: apply c1 to the fp32 product instead of to Q (see attn_fwd.hip)
    const void* table; int table_dtype; int64_t t_sbucket, t_shead;
    const float* lut_global;   // optional: the distance LUTs of all heads, (H, 4, qlen) floats (lut.hip)
    int lut_window;            // 0: plain images; w: images with the window |rel| < w folded in (local pattern)
    int block_len, aux, n_side;
    int align_end;       // 1: query i sits at key position i + N - M (KV-cache alignment); 0: at i
    // key split (dense, unpacked, align_end == 0): split s of nsplit covers keys [s*split_rows, (s+1)*split_rows)
    // and writes its normalised partial rows, a 1/0 weight and its log-sum-exp to the workspace arrays
    int nsplit, split_rows;
    // block pattern with key splits of its global rows in the same launch: the first block_items work items are the
    // block items, then one item per (batch, head, split); the splits' rows are the first min(aux, M) rows
    int block_items;
    float* part_o; float* part_l; float* part_m;   // (B,H,nsplit,M,D), (B,H,nsplit,M), (B,H,nsplit,M)
    BucketSpec bs;
};

// host side (api.cpp)
int fail(int code, const char* fmt, ...);
int make_bucket_spec(bool bidirectional, int num_buckets, int max_distance, BucketSpec* out);

// distance LUTs of all heads in a caller-provided buffer (lut.hip)
int64_t bias_lut_bytes(int H, const BucketSpec& bs, bool causal, int window = 0);
hipError_t launch_bias_lut(const FwdParams& p, bool causal, float* out, hipStream_t stream, int window = 0);

// launchers (attn_fwd.hip, splitk.hip)
hipError_t launch_fwd_bf16(const FwdParams& p, int D, int mode, bool causal, hipStream_t stream);
hipError_t launch_fwd_f16(const FwdParams& p, int D, int mode, bool causal, hipStream_t stream);
hipError_t launch_fwd_f32(const FwdParams& p, int D, int mode, bool causal, hipStream_t stream);

struct SplitKParams {
    const void* q; const void* k; const void* v; void* o;
    const float* bias;
    float* part_o; float* part_l; float* part_m;
    int64_t q_sb, q_sh, q_sr, k_sb, k_sh, k_sr, v_sb, v_sh, v_sr, o_sb, o_sh, o_sr;
    int64_t b_sb, b_sh, b_sr, b_sc;
    int B, H, M, N, S;
    float sm_scale;
    const int* key_lens; const int* key_starts;   // optional: batch element b only has the keys [start, start + len)
};
hipError_t launch_splitk(const SplitKParams& p, int dtype, int D, hipStream_t stream);
// only the merge over splits (part_o, part_l, part_m -> o)
hipError_t launch_splitk_merge(const SplitKParams& p, int dtype, int D, hipStream_t stream);

// Launch plan of a packed batch: 8 lists (one per XCD) of `slots` entries of 8 ints
// {sequence, head, q tile, len_q, len_k, first q row, first k row, 0}, of which the first counts[x] are in use.
constexpr int kPlanMaxSeqs = 1024;
struct PlanParams {
    const int32_t* cu_q; const int32_t* cu_k; const int32_t* len_q; const int32_t* len_k;
    int B, H, causal;
    int bn_shift;    // log2(keys per tile) of the attention kernel that will run the plan
    int key_shift;   // cost >> key_shift < 512 for every item
    int slots;       // entries per XCD
    int staged;      // 1: build the lists in LDS first (plan_can_stage() said they fit)
    int32_t* counts; // [8]
    int32_t* plan;   // [8][slots][8]
    int32_t* spill;  // scratch: four ints per item
};
bool plan_can_stage(int slots, int H, int max_seqlen_q);
hipError_t launch_varlen_plan(const PlanParams& p, hipStream_t stream);

// Backward of the dense forward (attn_bwd.hip)
struct BwdParams {
    const void* q; const void* k; const void* v; const void* o; const void* dout;
    const float* lse;                 // (B,H,M) natural log-sum-exp of the forward
    void* dq; void* dk; void* dv;
    float* dtable;                    // (n_buckets, H) fp32, or null
    float* delta; float* lse2;        // workspace, (B,H,M) each
    int64_t q_sb, q_sh, q_sr, k_sb, k_sh, k_sr, v_sb, v_sh, v_sr, o_sb, o_sh, o_sr, do_sb, do_sh, do_sr;
    int64_t dq_sb, dq_sh, dq_sr, dk_sb, dk_sh, dk_sr, dv_sb, dv_sh, dv_sr;
    int B, H, M, N;                   // packed: M, N are the longest sequence's lengths
    // packed batch (optional): (B+1) offsets and optional lengths, as in the forward; tensors are (total, H, D),
    // the statistics (total_q, H)
    const int32_t* cu_q; const int32_t* cu_k; const int32_t* len_q; const int32_t* len_k; int total_q;
    float c1;                         // base-2 score factor: sm_scale * log2(e), or 1 for pre-scaled query rows
    int fp32_math;                    // nonzero: fp32 matrix cores also for 16-bit inputs at head_dim 64
    int n_buckets;
    const void* table; int table_dtype; int64_t t_sbucket, t_shead;
    BucketSpec bs;
};
hipError_t launch_bwd_dense(const BwdParams& p, int dtype, int D, bool causal, hipStream_t stream);

struct RmsParams {
    const void* x; const void* weight; void* y;
    const void* residual; void* sum_out;                  // optional: normalise x + residual, write the sum (input type)
    const int* lens;                                      // optional (group > 1): valid rows per batch element
    const int* starts;                                    // optional, with lens: first valid row per batch element
    const uint32_t* key_bits; int64_t key_bits_stride;    // optional (group > 1): token validity bit sets ...
    const int* group_counts;                              // ... and the groups per batch element
    int64_t residual_row_stride;
    int64_t x_batch_stride, x_row_stride, y_row_stride;   // elements
    int64_t out_rows;        // batches * out_per_batch
    int out_per_batch;       // rows_per_batch / group (group == 1: rows_per_batch)
    int rows_per_batch, group, dim;
    float eps;
};
hipError_t launch_rmsnorm(const RmsParams& p, int x_dtype, int w_dtype, hipStream_t stream);

}  // namespace t5a
