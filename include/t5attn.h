/*
 * t5attn.h -- C ABI of the MI355X (gfx950) T5 attention forward library.
 *
 * One shared library, libt5attn.so, replaces the Triton kernels behind the
 * reference's attention hot path.  The reference has no FFI: its boundary is
 * a set of Python functions that launch Triton kernels; each entry point below
 * names the reference interface it stands in for (paths relative to the
 * reference checkout).
 *
 * Conventions
 *  - All tensor pointers are DEVICE pointers owned by the caller.  The library
 *    never allocates, frees or retains device memory, and never synchronises
 *    the host: every launch goes to the hipStream_t passed in (0 = null stream).
 *  - Strides are in ELEMENTS.  The innermost (head_dim) stride must be 1, all
 *    other strides multiples of 8 elements and base pointers 16-byte aligned.
 *  - head_dim D is one of 16, 32, 64, 128 (reference: src/turbot5/ops/
 *    fused_bias_attention.py:827-828).
 *  - Every function returns T5A_OK (0) or a negative t5a_status; the message
 *    of the last failure on the calling thread is t5a_last_error().
 *  - Scores are q.k * sm_scale + bias; the T5 modules pass sm_scale = 1.0.
 *  - Score precision (bf16 and fp16 inputs; the exact_scores field of the dense, varlen and sparse
 *    arguments takes one of the T5A_SCORES_* values below; fp32 inputs are always exact).
 *    T5A_SCORES_DEFAULT (0): the query rows are multiplied by sm_scale * log2(e) and rounded back to the
 *    input type before the matrix product, a relative error of 2^-9 (bf16) on every term of a score.
 *    With unscaled T5 scores of deviation 8 (18) the output error against fp32 math on the same inputs is
 *    about 4.5e-2 (1.1e-1) at worst, 3.6 times below that of the reference's 'basic' path run in bf16
 *    (src/turbot5/ops/naive_attention.py:4-23 rounds the scores themselves to bf16).
 *    T5A_SCORES_EXACT (1): the query rows enter the product as they are and the factor is applied to the
 *    fp32 result, as the reference's fused kernel does (src/turbot5/ops/fused_bias_attention.py:323-337);
 *    the error stays near 1e-2 (the rounding of the output) at any score magnitude; one more vector
 *    multiply per score.
 *    T5A_SCORES_PRESCALED (2): q already holds the query rows times sm_scale * log2(e) -- the caller folded
 *    the factor into the projection that produced q, in fp32, so that q was rounded to its type once.  The
 *    kernel applies no factor (sm_scale is not read); accuracy of T5A_SCORES_EXACT at the speed of
 *    T5A_SCORES_DEFAULT.  This is what the attention modules of this package do.
 *  - The relative-position bias is never materialised: kernels derive
 *    bucket(key_pos - query_pos) from integer positions and read the
 *    (num_buckets, H) table.  Bucket boundaries are computed on the host with
 *    the reference's fp32 formula (src/turbot5/model/attentions.py:78-124).
 */
#ifndef T5ATTN_H
#define T5ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* t5a_stream_t; /* hipStream_t */

typedef enum t5a_status {
    T5A_OK = 0,
    T5A_ERR_NULL = -1,      /* required pointer is NULL */
    T5A_ERR_DTYPE = -2,     /* unsupported element type */
    T5A_ERR_HEAD_DIM = -3,  /* D not in {16,32,64,128} */
    T5A_ERR_SHAPE = -4,     /* negative or inconsistent sizes */
    T5A_ERR_STRIDE = -5,    /* stride not a multiple of 8 elements / pointer not 16-byte aligned */
    T5A_ERR_BUCKETS = -6,   /* num_buckets / max_distance outside the supported range */
    T5A_ERR_PATTERN = -7,   /* unknown sparse pattern or bad pattern parameters */
    T5A_ERR_WORKSPACE = -8, /* workspace missing or too small */
    T5A_ERR_LAUNCH = -9     /* HIP reported an error at launch */
} t5a_status;

typedef enum t5a_dtype { T5A_BF16 = 0, T5A_F32 = 1, T5A_F16 = 2 } t5a_dtype;

typedef enum t5a_pattern {
    T5A_PATTERN_LOCAL = 1,   /* sliding window, |j-i| < block_len */
    T5A_PATTERN_BLOCK = 2,   /* own block + first n_global tokens; the first n_global queries see everything */
    T5A_PATTERN_TGLOBAL = 3  /* sliding window + side tokens (one per aux block of tokens) */
} t5a_pattern;

/*
 * The (num_buckets, H) relative-attention table (nn.Embedding weight).  table == NULL: no bias.
 * lut (optional): t5a_bias_lut_bytes() bytes of 16-byte aligned device memory.  Every work item of the
 * attention kernels starts by expanding its head's table column into a bias-per-distance LUT; with this
 * buffer the LUTs of all heads are built once (on the call's stream, by the first call: lut_ready == 0) and
 * later calls fetch them (lut_ready != 0: the buffer holds the LUTs of the same table values, bucket
 * parameters, H and causal flag).  Results are identical with and without it; it shortens the set-up of a
 * work item (4 % of the run time at B16 H12 L1024 D64).  Rebuild after the table changes.
 */
typedef struct t5a_bias {
    const void* table;
    int32_t table_dtype;          /* T5A_F32, T5A_BF16 or T5A_F16 */
    int32_t num_buckets;
    int32_t max_distance;
    int32_t lut_ready;
    int64_t stride_bucket;        /* elements between buckets (torch stride(0)) */
    int64_t stride_head;          /* elements between heads   (torch stride(1)) */
    void* lut; int64_t lut_bytes;
    /* 0: lut holds the plain images (t5a_bias_lut_bytes).  w > 0: it holds the images with the sliding window
     * |rel| < w folded in (t5a_bias_lut_bytes_windowed), which only t5a_fwd_sparse(T5A_PATTERN_LOCAL) with
     * block_len == w fetches; every other call rejects such a buffer.  A plain buffer handed to the local pattern is
     * ignored (its work items fill their LUTs themselves, 8 % of its run time at L=16384). */
    int32_t lut_window;
    int32_t reserved;
} t5a_bias;
/* 0 when the kernels cannot use a LUT buffer for these parameters (very large max_distance); causal selects
 * the unidirectional buckets, as in t5a_fwd_dense. */
int64_t t5a_bias_lut_bytes(int32_t H, int32_t num_buckets, int32_t max_distance, int32_t causal);
/* Size of a buffer for the images with the window |rel| < window folded in (bidirectional buckets; see
 * t5a_bias.lut_window); 0 when the local pattern cannot use one for this window.  No counterpart in the reference,
 * whose local attention materialises bias and mask per call (src/turbot5/model/attentions.py:598-618). */
int64_t t5a_bias_lut_bytes_windowed(int32_t H, int32_t num_buckets, int32_t max_distance, int32_t window);

/* Layout of the argument structs and set of entry points; a binding compares it with t5a_version() before
 * it passes a struct (a stale library would read pointers from the wrong offsets). */
#define T5A_ABI_VERSION 116
int t5a_version(void);
const char* t5a_last_error(void);

/*
 * Host-only, integer: bucket index for every relative position in
 * [-max_distance, +max_distance] (out[rel + max_distance]); positions beyond
 * that range share the bucket of the nearest end.  Replaces
 * T5Attention._relative_position_bucket (src/turbot5/model/attentions.py:78-124).
 */
int t5a_bucket_lut(int bidirectional, int num_buckets, int max_distance, int32_t* out /* 2*max_distance+1 */);

/*
 * Dense fused-bias flash attention forward.
 * Replaces flash_attention_with_fusing_bias / flash_attn_v2_fwd_bias
 * (src/turbot5/ops/fused_bias_attention.py:876-890, :23-59).
 * q,o: (B,H,M,D); k,v: (B,H,N,D); strides = {batch, head, row}.
 * Queries are aligned to the end of the keys: rel = j - (i + N - M); with
 * causal != 0 key j is visible iff j <= i + N - M and buckets are
 * unidirectional, else bidirectional.  lse (optional) is (B,H,M) contiguous
 * fp32, natural log of the softmax normaliser (fused_bias_attention.py:358).
 */
enum { T5A_SCORES_DEFAULT = 0, T5A_SCORES_EXACT = 1, T5A_SCORES_PRESCALED = 2 };

typedef struct t5a_dense_args {
    const void* q; const void* k; const void* v; void* o; float* lse;
    int64_t q_strides[3]; int64_t k_strides[3]; int64_t v_strides[3]; int64_t o_strides[3];
    int32_t dtype; int32_t B; int32_t H; int32_t M; int32_t N; int32_t D;
    int32_t causal; float sm_scale;
    int32_t exact_scores; int32_t reserved;   /* exact_scores: see "Score precision" above */
    t5a_bias bias;
} t5a_dense_args;
int t5a_fwd_dense(const t5a_dense_args* args, t5a_stream_t stream);

/*
 * Backward of t5a_fwd_dense: dq, dk, dv and the gradient of the (num_buckets, H) bias table.
 * Replaces flash_attn_v2_bwd_bias behind FlashAttentionBias.backward
 * (src/turbot5/ops/fused_bias_attention.py:851-873; kernels :397-820, the table gradient's atomics :617-619).
 * q, k, v, causal, sm_scale, exact_scores and bias as in the forward call; o and lse are what it returned
 * (lse is required); dout is the gradient of o.  dq (B,H,M,D), dk and dv (B,H,N,D) in the tensors' type, any
 * strides {batch, head, row}; dtable (required when bias.table is set): (num_buckets, H) contiguous fp32, overwritten.
 * head_dim 16, 32 or 64; 16-bit tensors also 128.  The table gradient is summed with floating-point atomics: its last bits depend on the
 * order of the workgroups.
 * Arithmetic of the backward.  fp32 tensors, head_dim 16 and 32, and any call with fp32_math != 0: every product on
 * the fp32 matrix cores, inputs widened on their way in (head_dim up to 64).  16-bit tensors at head_dim 64 and 128
 * with fp32_math == 0: the
 * 16-bit matrix cores -- the score and dP products take the inputs as they are, and the probabilities and dS are
 * rounded to the tensors' type before the products that form dq, dk and dv, as the reference rounds them
 * (fused_bias_attention.py:575-590); sums, the softmax statistics and the table gradient stay in fp32.  About
 * five times faster; gradients differ from the fp32 path by the rounding of their own type.
 * workspace: t5a_bwd_workspace_bytes(B, H, M) bytes of 16-byte aligned device memory.
 */
typedef struct t5a_dense_bwd_args {
    const void* q; const void* k; const void* v; const void* o; const void* dout; const float* lse;
    void* dq; void* dk; void* dv; float* dtable;
    void* workspace; int64_t workspace_bytes;
    int64_t q_strides[3]; int64_t k_strides[3]; int64_t v_strides[3]; int64_t o_strides[3]; int64_t dout_strides[3];
    int64_t dq_strides[3]; int64_t dk_strides[3]; int64_t dv_strides[3];
    int32_t dtype; int32_t B; int32_t H; int32_t M; int32_t N; int32_t D;
    int32_t causal; float sm_scale;
    int32_t exact_scores; int32_t fp32_math;   /* fp32_math: see "Arithmetic of the backward" above */
    t5a_bias bias;
} t5a_dense_bwd_args;
int64_t t5a_bwd_workspace_bytes(int32_t B, int32_t H, int32_t M);
int t5a_bwd_dense(const t5a_dense_bwd_args* args, t5a_stream_t stream);

/*
 * Packed variable-length forward.
 * Replaces flash_attention_with_fusing_bias_varlen / flash_attn_v2_fwd_bias
 * (src/turbot5/ops/varlen_fused_bias_attn.py:870-889, :37-80); the q-tile work
 * list of get_mid (:23-35) is derived on the device from cu_seqlens, so there
 * is no host synchronisation.
 * q,o: (total_q,H,D); k,v: (total_k,H,D); strides = {row, head}.
 * cu_seqlens_q/k: DEVICE int32 arrays of B+1 ascending offsets.  Positions are
 * in-sequence; per sequence the semantics equal t5a_fwd_dense.
 * seq_lens_q/k (optional): DEVICE int32 arrays of B lengths.  When given, sequence b is
 * rows [cu[b], cu[b] + lens[b]) and the rows up to cu[b+1] are padding that is neither read
 * nor written: a right-padded (B,L,H,D) batch runs in place with cu = {0, L, 2L, ...} and
 * lens = mask.sum(-1), without the gathers and the scatter of the reference's unpad / pad
 * (src/turbot5/model/padding.py:113-150, :30-44).
 * lse (optional) is (total_q,H) contiguous fp32.
 * workspace (optional): t5a_varlen_workspace_bytes(B, H, total_q) bytes of 16-byte aligned device
 * memory (the function returns 0 when no plan can be made: B > 1024; a workspace is then
 * ignored).  With it a one-workgroup kernel first builds a launch plan from
 * cu_seqlens -- per-XCD item lists of equal WORK, longest item first -- on the same stream, still
 * without host synchronisation; without it workgroups find their item by walking cu_seqlens and
 * XCDs get equal item COUNTS, which leaves them unevenly loaded when lengths differ.  Results are
 * identical either way.  Building the plan takes about 15 us on top of the launch: it pays from a
 * few thousand q tiles x heads on, earlier when several calls share it (workspace_ready).  The
 * workspace may be reused or freed once later work on the stream
 * cannot overlap this call (stream order).
 * workspace_ready != 0: the workspace still holds the plan that an earlier call built from the same
 * cu_seqlens, seq_lens, B, H, D, dtype, causal and max_seqlen values (for instance the previous
 * layer of the same batch): the build is skipped.
 */
typedef struct t5a_varlen_args {
    const void* q; const void* k; const void* v; void* o; float* lse;
    int64_t q_strides[2]; int64_t k_strides[2]; int64_t v_strides[2]; int64_t o_strides[2];
    const int32_t* cu_seqlens_q; const int32_t* cu_seqlens_k;
    const int32_t* seq_lens_q; const int32_t* seq_lens_k;
    void* workspace; int64_t workspace_bytes;
    int32_t dtype; int32_t B; int32_t H; int32_t D;
    int32_t total_q; int32_t total_k; int32_t max_seqlen_q; int32_t max_seqlen_k;
    int32_t causal; float sm_scale;
    int32_t workspace_ready; int32_t exact_scores;
    t5a_bias bias;
} t5a_varlen_args;
int64_t t5a_varlen_workspace_bytes(int32_t B, int32_t H, int32_t total_q);
int t5a_fwd_varlen(const t5a_varlen_args* args, t5a_stream_t stream);

/*
 * Backward of t5a_fwd_varlen: dq (total_q,H,D), dk and dv (total_k,H,D), strides {row, head}, and the table
 * gradient as in t5a_bwd_dense.  Replaces the backward of the reference's packed autograd function
 * (src/turbot5/ops/varlen_fused_bias_attn.py:407-800, :839-868).  cu_seqlens, seq_lens, causal, sm_scale,
 * exact_scores and bias as in the forward call; o and lse (total_q, H) are what it returned.  Rows between
 * cu[b] + seq_lens[b] and cu[b+1] (padding) are not written.  max_seqlen_q / max_seqlen_k size the launch grid:
 * a longer sequence would lose rows.  workspace: t5a_bwd_varlen_workspace_bytes(total_q, H) bytes.
 */
typedef struct t5a_varlen_bwd_args {
    const void* q; const void* k; const void* v; const void* o; const void* dout; const float* lse;
    void* dq; void* dk; void* dv; float* dtable;
    void* workspace; int64_t workspace_bytes;
    int64_t q_strides[2]; int64_t k_strides[2]; int64_t v_strides[2]; int64_t o_strides[2]; int64_t dout_strides[2];
    int64_t dq_strides[2]; int64_t dk_strides[2]; int64_t dv_strides[2];
    const int32_t* cu_seqlens_q; const int32_t* cu_seqlens_k;
    const int32_t* seq_lens_q; const int32_t* seq_lens_k;
    int32_t dtype; int32_t B; int32_t H; int32_t D;
    int32_t total_q; int32_t total_k; int32_t max_seqlen_q; int32_t max_seqlen_k;
    int32_t causal; float sm_scale;
    int32_t exact_scores; int32_t fp32_math;   /* as in t5a_dense_bwd_args */
    t5a_bias bias;
} t5a_varlen_bwd_args;
int64_t t5a_bwd_varlen_workspace_bytes(int32_t total_q, int32_t H);
int t5a_bwd_varlen(const t5a_varlen_bwd_args* args, t5a_stream_t stream);

/*
 * Sparse encoder self-attention as tile skipping (no bias/mask tensor, no
 * replicated K/V).  Replaces the blocked torch code + flash_attention_with_bias
 * (src/turbot5/ops/flash_attention.py:870-884) in T5LocalAttention.forward
 * (src/turbot5/model/attentions.py:583-638), T5BlockAttention.forward (:788-853)
 * and T5TransientGlobalAttention.forward (:977-1052), all-ones attention mask.
 * q,k,v,o: (B,H,L,D); strides = {batch, head, row}.
 *   LOCAL   block_len = window; keys |j-i| < block_len, bias bucket(j-i).
 *   BLOCK   block_len, aux = number of global tokens G (G <= block_len).
 *           Rows < G: all keys.  Other rows: the G global tokens with
 *           rel = g-(G+i%block_len) and the own block with rel = j-i; in block 0
 *           only the first block_len-G own-block tokens are visible and keys of
 *           a ragged last block past L count as zero vectors (both as the
 *           reference computes them, attentions.py:722-732, :807-814).
 *   TGLOBAL block_len = window, aux = tokens per side token; side_k/side_v:
 *           (B,H,n_side,D) projected block aggregates, bias bucket(g - min(i/aux, n_side-1)).
 * seq_lens (optional): (B) int32 on the device, the number of valid tokens of each sequence; seq_starts
 * (optional, LOCAL and TGLOBAL, with seq_lens): (B) int32, the row of its first token (a batch padded on the
 * left; NULL = 0).  The tokens of sequence b are the rows [start, start + len); a token's position stays its
 * row index, as in the reference.  Rows of padding tokens are still written and mean nothing.
 *   LOCAL, TGLOBAL: keys outside the sequence's rows are not attended (the key half of the reference's local
 *           mask, src/turbot5/model/utils.py:174-188).  TGLOBAL: the sequence has one side token per
 *           aux-block END among its rows, (start + len) / aux - start / aux of them, a token's side token
 *           being min(row / aux, count - 1) (utils.py:191-237 for one run of tokens); side_k/side_v rows
 *           past them are not read.
 *   BLOCK   (right padding only) the reference's additive mask as it lays it out
 *           (src/turbot5/model/attentions.py:722-732): in block b, list column c < block_len of
 *           [G global tokens | own block] is masked iff token b * block_len + c is padding, the last G
 *           columns never (always in block 0); the first G rows attend every key, padding included
 *           (:788-800).
 * key_bits (optional; instead of seq_lens / seq_starts): validity of every token as a bit set,
 * for attention masks of any shape (holes, padding on either side).  (B, key_bits_stride) uint32 words on the
 * device; token j of sequence b is bit (j & 31) of word 8 + (j >> 5) -- eight zero words in front, and zero words
 * behind the last token up to at least t5a_sparse_key_bits_words(L, block_len, aux) words in all.
 *   LOCAL   keys whose bit is 0 are not attended (the key half of the reference's local mask,
 *           src/turbot5/model/utils.py:174-188).
 *   BLOCK   the reference's additive mask as it lays it out (attentions.py:722-732), for any mask: list column
 *           c < block_len of [G global tokens | own block] is masked iff token b * block_len + c has bit 0, the
 *           last G columns never (always in block 0); the first G rows attend every key.
 *   TGLOBAL window keys whose bit is 0 are not attended.  side_counts[b] = number of aux-block END positions
 *           (rows p with p % aux == aux - 1) of sequence b whose bit is 1: it has that many side tokens, a
 *           token's side token being min(row / aux, count - 1) (the reference's block ids for any mask,
 *           src/turbot5/model/utils.py:191-237).
 * workspace (optional, BLOCK only): t5a_sparse_workspace_bytes() bytes of device memory.  With it
 * the G global rows, which attend all L keys, are computed as key splits spread over the whole
 * device and merged; without it they run as one workgroup per (batch, head).  Results agree to
 * rounding of the merge.
 */
typedef struct t5a_sparse_args {
    const void* q; const void* k; const void* v; void* o;
    const void* side_k; const void* side_v;
    void* workspace; int64_t workspace_bytes;
    int64_t q_strides[3]; int64_t k_strides[3]; int64_t v_strides[3]; int64_t o_strides[3];
    int64_t side_k_strides[3]; int64_t side_v_strides[3];
    int32_t dtype; int32_t B; int32_t H; int32_t L; int32_t D;
    int32_t pattern; int32_t block_len; int32_t aux; int32_t n_side;
    float sm_scale; int32_t exact_scores;
    t5a_bias bias;
    const int32_t* seq_lens;
    const int32_t* seq_starts;
    const uint32_t* key_bits;
    int64_t key_bits_stride;      /* words per sequence */
    const int32_t* side_counts;   /* TGLOBAL with key_bits: (B) int32, side tokens of each sequence */
    /* LOCAL (windows up to 256) and BLOCK with 16-bit inputs at head_dim 64 / 128: a work item takes run_len
     * consecutive q tiles of one (batch, head).  0: the library chooses from the shape and the device's size;
     * 1..16: this many (tests pin every path with it; results do not depend on it). */
    int32_t run_len; int32_t reserved;
} t5a_sparse_args;
/* words per sequence that key_bits needs (front padding, ceil(L / 32), back padding) */
int64_t t5a_sparse_key_bits_words(int32_t L, int32_t block_len, int32_t aux);
int64_t t5a_sparse_workspace_bytes(int32_t pattern, int32_t B, int32_t H, int32_t L, int32_t D, int32_t block_len, int32_t aux);
int t5a_fwd_sparse(const t5a_sparse_args* args, t5a_stream_t stream);
/*
 * Host-only: the launch plan t5a_fwd_sparse would choose for a shape, without touching the device when
 * compute_units > 0 (0: ask the current device).  No counterpart in the reference (its sparse modules are torch
 * code with one fixed blocking, src/turbot5/model/attentions.py:583-638, :788-853).  with_workspace: the call
 * would pass a workspace of t5a_sparse_workspace_bytes().  run_len as in t5a_sparse_args.
 * out[0] = q tiles per run, out[1] = work items of the launch, out[2] = how many of them are runs when the
 * global rows of the block pattern travel in the same launch as key splits (else 0), out[3] = key splits per
 * (batch, head), out[4] = keys per split, out[5] = q tiles per (batch, head).  Fails (T5A_ERR_LAUNCH) if the plan
 * would not cover every q tile and every key exactly once.
 */
int t5a_sparse_launch_plan(int32_t pattern, int32_t dtype, int32_t B, int32_t H, int32_t L, int32_t D, int32_t block_len,
                           int32_t aux, int32_t with_workspace, int32_t compute_units, int32_t run_len, int32_t* out /* 6 */);

/*
 * Flash-decoding split-K forward for few query rows over a long memory.
 * Replaces flash_attn_v2_fwd (src/turbot5/ops/flash_decoding.py:6-55): the
 * per-split kernel (:57-178) and the merge the reference does in torch (:47-55).
 * q,o: (B,H,M,D), M <= 16; k,v: (B,H,N,D); strides = {batch, head, row}.
 * attn_bias (optional): additive fp32 bias, strides {batch, head, row, col},
 * use 0 to broadcast.  Split s covers keys [s*(N/S), (s+1)*(N/S)), the last
 * split also the remainder.  workspace holds, contiguous fp32, in this order:
 * part_o (B,H,S,M,D) normalised partial outputs, part_l (B,H,S,M) partial
 * sums of exp, part_m (B,H,S,M) partial maxima (scaled scores, natural units).
 */
typedef struct t5a_splitk_args {
    const void* q; const void* k; const void* v; void* o;
    const float* attn_bias;
    void* workspace; int64_t workspace_bytes;
    int64_t q_strides[3]; int64_t k_strides[3]; int64_t v_strides[3]; int64_t o_strides[3];
    int64_t bias_strides[4];
    int32_t dtype; int32_t B; int32_t H; int32_t M; int32_t N; int32_t D;
    int32_t num_splits; float sm_scale;
    /* optional, (B) int32 on the device: batch element b only has the keys [key_starts[b],
     * key_starts[b] + key_lens[b]) of its N rows (a padded encoder memory; key_starts NULL = 0).  The
     * reference masks such keys with an additive bias in T5Attention (src/turbot5/model/attentions.py:235-236);
     * its split-K kernel has no counterpart. */
    const int32_t* key_lens; const int32_t* key_starts;
} t5a_splitk_args;
int64_t t5a_splitk_workspace_bytes(int32_t B, int32_t H, int32_t M, int32_t D, int32_t num_splits);
int t5a_fwd_splitk(const t5a_splitk_args* args, t5a_stream_t stream);

/*
 * t5a_fwd_splitk for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, kernels and
 * results as t5a_fwd_splitk, except that args->workspace and args->workspace_bytes are ignored: the partial
 * results go to a static device array of T5A_STATIC_SCRATCH_BYTES that is part of the library (each GPU the
 * library runs on holds its copy until the process ends).  The call allocates and frees nothing.
 * Limit: t5a_splitk_workspace_bytes(B, H, M, D, num_splits) <= T5A_STATIC_SCRATCH_BYTES, else
 * T5A_ERR_WORKSPACE (batch 64, 12 heads, one query row, head_dim 64, 16 splits need 3.1 MiB).
 * The first call on a device looks the array's address up (hipGetSymbolAddress); make that call outside a
 * graph capture.  All calls on one GPU share the array: calls that may overlap in time (different streams,
 * different threads) race on it; calls ordered on one stream do not.
 */
#define T5A_STATIC_SCRATCH_BYTES (8 * 1024 * 1024)
int t5a_fwd_splitk_static(const t5a_splitk_args* args, t5a_stream_t stream);

/*
 * T5 RMS norm (no mean subtraction, no bias) and, with group > 1, the side-token producer of the
 * transient-global pattern: output row r of a sequence is the norm of the SUM of input rows
 * [r*group, (r+1)*group), the rows left over at the end of the sequence joining its last group.
 * Replaces T5LayerNorm (src/turbot5/model/modules.py:24-67; Triton variant src/turbot5/ops/
 * rms_norm.py:5-48) and, for group > 1, _create_global_aggregates + global_input_layer_norm
 * (src/turbot5/model/utils.py:249-258, :206-212; src/turbot5/model/attentions.py:959-966), all-ones mask.
 * x: (batches, rows_per_batch, dim) with strides {batch, row} in elements, dim contiguous and a
 * multiple of 8; weight: (dim); y: (batches, rows_per_batch / group, dim) contiguous, in the
 * weight's type when that is 16 bit, else fp32 (torch type promotion of the reference code).
 * Arithmetic as the reference's eager path: fp32 variance and scaling, the scaled value rounded to
 * a 16-bit weight's type before the product; block sums are rounded to the input type first.
 * seq_lens / seq_starts (optional, not together with residual): (batches) int32 on the device, the rows
 * [start, start + len) of each batch element are its tokens (seq_starts NULL = 0): it has one group per group END
 * among them, (start + len) / group - start / group, group g taking its tokens of rows [g * group,
 * (g + 1) * group) and the last group every token from there on; groups without a token and output rows past
 * the groups are zero.
 * residual (optional, group == 1 only): rows of x's type and shape with row stride
 * residual_row_stride; the kernel normalises x + residual (rounded to x's type, as torch's add leaves
 * it) and also writes that sum to sum_out (x's type, rows contiguous like y, 16-byte aligned; must
 * not overlap x or residual).  This is the residual add of one T5 sub-layer followed by the norm of
 * the next (src/turbot5/model/modeling.py:159-161, :113-114) in one pass over the rows.
 */
typedef struct t5a_rmsnorm_args {
    const void* x; const void* weight; void* y;
    int64_t x_strides[2];
    int64_t batches; int32_t rows_per_batch; int32_t dim; int32_t group;
    int32_t x_dtype; int32_t weight_dtype; float eps;
    int32_t reserved;
    const void* residual; void* sum_out; int64_t residual_row_stride;
    const int32_t* seq_lens;
    const int32_t* seq_starts;   /* optional, with seq_lens: first valid row of each batch element (NULL = 0) */
    /* optional (group > 1, instead of seq_lens): token validity bit sets laid out as for the sparse patterns; any
     * stride that covers the rows will do: the buffer made for the attention call serves; and the number of groups of each batch element (the END positions of groups
     * whose bit is 1): group g sums the valid rows of [g * group, (g + 1) * group), the last group every valid
     * row from its start on; rows past the groups are zero. */
    const uint32_t* key_bits; int64_t key_bits_stride; const int32_t* group_counts;
} t5a_rmsnorm_args;
int t5a_rmsnorm(const t5a_rmsnorm_args* args, t5a_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* T5ATTN_H */
