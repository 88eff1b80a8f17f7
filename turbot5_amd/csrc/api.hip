// extern "C" entry points of libt5attn.so: argument validation, bucket
// boundaries on the host, parameter packing, launch.  See include/t5attn.h.
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <map>
#include <mutex>
#include <tuple>

#include "t5a_internal.h"

namespace t5a {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

// Bucket of one relative position with the arithmetic of the reference
// (src/turbot5/model/attentions.py:97-124): fp32 division, fp32 log, fp32
// division by the double constant rounded to fp32, fp32 multiply, truncation.
static int bucket_scalar(int rel, bool bidirectional, int num_buckets, int max_distance) {
    int nb = num_buckets, out = 0, d;
    if (bidirectional) {
        nb /= 2;
        if (rel > 0) out += nb;
        d = rel < 0 ? -rel : rel;
    } else {
        d = rel < 0 ? -rel : 0;
    }
    const int max_exact = nb / 2;
    if (d < max_exact) return out + d;
    const float x = logf((float)d / (float)max_exact);
    const float den = (float)log((double)max_distance / (double)max_exact);
    const float y = x / den * (float)(nb - max_exact);
    long big = (long)max_exact + (long)y;
    if (big > nb - 1) big = nb - 1;
    return out + (int)big;
}

static int check_bucket_params(bool bidirectional, int num_buckets, int max_distance) {
    const int nb = bidirectional ? num_buckets / 2 : num_buckets;
    const int max_exact = nb / 2;
    if (num_buckets <= 0 || max_exact < 1 || nb > 2 * kMaxThresholds)
        return fail(T5A_ERR_BUCKETS, "num_buckets=%d unsupported (need %d..%d)", num_buckets,
                    bidirectional ? 4 : 2, bidirectional ? 4 * kMaxThresholds : 2 * kMaxThresholds);
    if (max_distance <= max_exact)
        return fail(T5A_ERR_BUCKETS, "max_distance=%d must exceed num_buckets/%d=%d", max_distance,
                    bidirectional ? 4 : 2, max_exact);
    return T5A_OK;
}

int make_bucket_spec(bool bidirectional, int num_buckets, int max_distance, BucketSpec* out) {
    static std::mutex mu;
    static std::map<std::tuple<int, int, int>, BucketSpec> cache;
    const auto key = std::make_tuple((int)bidirectional, num_buckets, max_distance);
    {
        std::lock_guard<std::mutex> g(mu);
        auto it = cache.find(key);
        if (it != cache.end()) { *out = it->second; return T5A_OK; }
    }
    int rc = check_bucket_params(bidirectional, num_buckets, max_distance);
    if (rc != T5A_OK) return rc;
    BucketSpec s;
    memset(&s, 0, sizeof(s));
    s.bidirectional = bidirectional ? 1 : 0;
    s.nb = bidirectional ? num_buckets / 2 : num_buckets;
    s.max_exact = s.nb / 2;
    s.n_thr = s.nb - 1 - s.max_exact;
    // walk the distances once; the device code counts thresholds, which is exact
    // only for a non-decreasing sequence of buckets
    int prev = s.max_exact, filled = 0;
    for (int d = s.max_exact; d <= max_distance; ++d) {
        const int bk = bucket_scalar(-d, bidirectional, num_buckets, max_distance);
        if (bk < prev) return fail(T5A_ERR_BUCKETS, "bucket sequence not monotone at distance %d", d);
        while (filled < bk - s.max_exact && filled < s.n_thr) s.thr[filled++] = d;
        prev = bk;
    }
    if (prev != s.nb - 1 || filled != s.n_thr)
        return fail(T5A_ERR_BUCKETS, "buckets do not saturate at max_distance=%d", max_distance);
    s.sat = s.n_thr > 0 ? s.thr[s.n_thr - 1] : s.max_exact;
    for (int t = s.n_thr; t < kMaxThresholds; ++t) s.thr[t] = 0x7fffffff;   // unused slots never count
    if (s.sat > kMaxSaturation)
        return fail(T5A_ERR_BUCKETS, "bucket saturation distance %d exceeds %d", s.sat, kMaxSaturation);
    {
        std::lock_guard<std::mutex> g(mu);
        cache[key] = s;
    }
    *out = s;
    return T5A_OK;
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// unit: strides must be multiples of this many elements (16 bytes worth, or 1 for scalar stores)
static int check_tensor(const char* name, const void* ptr, const int64_t* strides, int n, int unit) {
    if (ptr == nullptr) return fail(T5A_ERR_NULL, "%s is NULL", name);
    if (unit > 1 && !aligned16(ptr)) return fail(T5A_ERR_STRIDE, "%s is not 16-byte aligned", name);
    for (int i = 0; i < n; ++i)
        if (strides[i] % unit != 0)
            return fail(T5A_ERR_STRIDE, "%s stride[%d]=%lld is not a multiple of %d elements", name, i, (long long)strides[i], unit);
    return T5A_OK;
}

// The kernels address the key/value rows of one (batch, head) slice with 32-bit byte offsets and
// prefetch a few tiles past the last row (those read as zeros): the slice must stay below 2 GiB.
static int check_rows(const char* name, int64_t rows, int64_t row_stride, int dtype) {
    const int64_t es = dtype == T5A_F32 ? 4 : 2;
    if (row_stride < 0) return fail(T5A_ERR_STRIDE, "%s row stride %lld is negative", name, (long long)row_stride);
    if ((rows + 1024) * row_stride * es > 0x7fffffffLL)
        return fail(T5A_ERR_SHAPE, "%s: %lld rows of stride %lld elements exceed 2 GiB per (batch, head) slice", name,
                    (long long)rows, (long long)row_stride);
    return T5A_OK;
}

static int check_common(int dtype, int D) {
    if (dtype != T5A_BF16 && dtype != T5A_F16 && dtype != T5A_F32) return fail(T5A_ERR_DTYPE, "unsupported dtype %d", dtype);
    if (D != 16 && D != 32 && D != 64 && D != 128) return fail(T5A_ERR_HEAD_DIM, "head_dim %d not in {16,32,64,128}", D);
    return T5A_OK;
}

static int fill_bias(const t5a_bias& b, bool bidirectional, FwdParams* p) {
    p->table = b.table;
    p->table_dtype = b.table_dtype;
    p->t_sbucket = b.stride_bucket;
    p->t_shead = b.stride_head;
    memset(&p->bs, 0, sizeof(p->bs));
    if (b.table == nullptr) return T5A_OK;
    if (b.table_dtype != T5A_F32 && b.table_dtype != T5A_BF16 && b.table_dtype != T5A_F16)
        return fail(T5A_ERR_DTYPE, "unsupported bias table dtype %d", b.table_dtype);
    return make_bucket_spec(bidirectional, b.num_buckets, b.max_distance, &p->bs);
}

// Optional buffer with the distance LUTs of all heads: checked, built on the first use, handed to the kernel.
// window: 0, or the sliding window of the local pattern when it is folded into the LUT
static int prepare_lut(const t5a_bias& b, bool causal, hipStream_t stream, FwdParams* p, int window = 0) {
    if (b.table == nullptr || b.lut == nullptr) return T5A_OK;
    if (b.lut_window < 0) return fail(T5A_ERR_SHAPE, "bias.lut_window %d", b.lut_window);
    if (b.lut_window != window) {
        if (b.lut_window == 0) return T5A_OK;   // plain images, windowed ones wanted: the kernel fills its LUTs itself
        return fail(T5A_ERR_PATTERN, "bias.lut holds the images for the window %d: only the local pattern with that block_len reads them",
                    b.lut_window);
    }
    const int64_t need = bias_lut_bytes(p->H, p->bs, causal, window);
    if (need == 0) return T5A_OK;   // not usable for these parameters: the kernel builds its LUTs itself
    if (b.lut_bytes < need)
        return fail(T5A_ERR_WORKSPACE, "bias.lut too small: %lld bytes, t5a_bias_lut_bytes() asks for %lld",
                    (long long)b.lut_bytes, (long long)need);
    if ((reinterpret_cast<uintptr_t>(b.lut) & 15) != 0) return fail(T5A_ERR_STRIDE, "bias.lut must be 16-byte aligned");
    if (b.lut_ready == 0) {
        hipError_t e = launch_bias_lut(*p, causal, static_cast<float*>(b.lut), stream, window);
        if (e != hipSuccess) return fail(T5A_ERR_LAUNCH, "bias LUT build: %s", hipGetErrorString(e));
    }
    p->lut_global = static_cast<const float*>(b.lut);
    p->lut_window = window;
    return T5A_OK;
}

static int finish(hipError_t e, const char* what) {
    if (e != hipSuccess) return fail(T5A_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return T5A_OK;
}

static const float kLog2e = 1.4426950408889634f;

// How sm_scale * log2(e) reaches the scores (the exact_scores field of the argument structs).
//   T5A_SCORES_DEFAULT   16-bit inputs: Q is multiplied by the factor in the kernel and rounded back to its type
//   T5A_SCORES_EXACT     the factor is applied to the fp32 product (fused_bias_attention.py:323-337 does this)
//   T5A_SCORES_PRESCALED the caller's Q already carries sm_scale * log2(e) (folded into the projection that made
//                        it, so that Q was rounded to its type once): the kernel multiplies by exactly 1
static int score_mode(int mode, float sm_scale, FwdParams* p) {
    if (mode != T5A_SCORES_DEFAULT && mode != T5A_SCORES_EXACT && mode != T5A_SCORES_PRESCALED)
        return fail(T5A_ERR_SHAPE, "exact_scores=%d is none of T5A_SCORES_DEFAULT, _EXACT, _PRESCALED", mode);
    p->c1 = mode == T5A_SCORES_PRESCALED ? 1.0f : sm_scale * kLog2e;
    p->exact_scale = mode == T5A_SCORES_EXACT;
    return T5A_OK;
}

static hipError_t launch_fwd(const FwdParams& p, int dtype, int D, int mode, bool causal, hipStream_t stream) {
    if (p.total_items <= 0) return hipSuccess;
    if (dtype == T5A_BF16) return launch_fwd_bf16(p, D, mode, causal, stream);
    if (dtype == T5A_F16) return launch_fwd_f16(p, D, mode, causal, stream);
    if (dtype == T5A_F32) return launch_fwd_f32(p, D, mode, causal, stream);
    return hipErrorInvalidValue;
}

}  // namespace t5a

using namespace t5a;

extern "C" {

int t5a_version(void) { return T5A_ABI_VERSION; }

const char* t5a_last_error(void) { return g_err; }

int64_t t5a_bias_lut_bytes(int32_t H, int32_t num_buckets, int32_t max_distance, int32_t causal) {
    BucketSpec bs;
    if (H <= 0 || make_bucket_spec(causal == 0, num_buckets, max_distance, &bs) != T5A_OK) return 0;
    return bias_lut_bytes(H, bs, causal != 0);
}

int64_t t5a_bias_lut_bytes_windowed(int32_t H, int32_t num_buckets, int32_t max_distance, int32_t window) {
    BucketSpec bs;
    if (H <= 0 || window <= 0 || window > kMaxLutWindow || make_bucket_spec(true, num_buckets, max_distance, &bs) != T5A_OK) return 0;
    return bias_lut_bytes(H, bs, false, window);
}

int t5a_bucket_lut(int bidirectional, int num_buckets, int max_distance, int32_t* out) {
    if (out == nullptr) return fail(T5A_ERR_NULL, "out is NULL");
    int rc = check_bucket_params(bidirectional != 0, num_buckets, max_distance);
    if (rc != T5A_OK) return rc;
    for (int rel = -max_distance; rel <= max_distance; ++rel)
        out[rel + max_distance] = bucket_scalar(rel, bidirectional != 0, num_buckets, max_distance);
    return T5A_OK;
}

// Causal dense launch: cut the item list (pair-major, longest tile first inside a pair) into 8 slices of
// equal work, one per XCD.  The cost of an item is its number of key tiles plus a constant for its
// set-up and write-back (about five tile steps, from per-item timestamps).
static void causal_slices(FwdParams* p, int dtype, int D) {
    const int tps = p->tiles_per_seq;
    const int bn = (dtype != T5A_F32 && D == 128) ? 32 : 64;   // keys per tile, as the kernel chooses them
    const int64_t shift = (int64_t)p->N - p->M;                 // query i sits at key position i + N - M
    auto cost = [&](int level) {                                // level 0 is the last (longest) q tile
        const int64_t qt = tps - 1 - level;
        const int64_t keys = std::min<int64_t>(p->N, std::max<int64_t>(0, (qt + 1) * 128 + shift));
        return (keys + bn - 1) / bn + 5;
    };
    int64_t per_pair = 0;
    for (int l = 0; l < tps; ++l) per_pair += cost(l);
    const int64_t pairs = (int64_t)p->H * p->B;
    const int64_t total = per_pair * pairs;
    p->xcd_lo[0] = 0;
    for (int x = 1; x < 8; ++x) {
        const int64_t target = total * x / 8;
        const int64_t g = target / per_pair;
        int64_t rem = target - g * per_pair;
        int l = 0;
        while (l < tps && rem >= cost(l)) { rem -= cost(l); ++l; }
        if (l < tps && 2 * rem > cost(l)) ++l;                  // nearer boundary
        p->xcd_lo[x] = (int)std::min<int64_t>(g * tps + l, (int64_t)p->total_items);
    }
    p->xcd_lo[8] = p->total_items;
}

int t5a_fwd_dense(const t5a_dense_args* a, t5a_stream_t stream) {
    if (a == nullptr) return fail(T5A_ERR_NULL, "args is NULL");
    int rc = check_common(a->dtype, a->D);
    if (rc) return rc;
    const int unit = a->dtype == T5A_F32 ? 4 : 8;
    if (a->B < 0 || a->H <= 0 || a->M < 0 || a->N < 0) return fail(T5A_ERR_SHAPE, "bad sizes B=%d H=%d M=%d N=%d", a->B, a->H, a->M, a->N);
    if (a->B == 0 || a->M == 0) return T5A_OK;
    if ((rc = check_tensor("q", a->q, a->q_strides, 3, unit))) return rc;
    if ((rc = check_tensor("o", a->o, a->o_strides, 3, unit))) return rc;
    if (a->N > 0) {
        if ((rc = check_tensor("k", a->k, a->k_strides, 3, unit))) return rc;
        if ((rc = check_tensor("v", a->v, a->v_strides, 3, unit))) return rc;
        if ((rc = check_rows("k", a->N, a->k_strides[2], a->dtype))) return rc;
        if ((rc = check_rows("v", a->N, a->v_strides[2], a->dtype))) return rc;
    }
    if ((rc = check_rows("q", a->M, a->q_strides[2], a->dtype))) return rc;
    FwdParams p;
    memset(&p, 0, sizeof(p));
    p.q = a->q; p.k = a->k; p.v = a->v; p.o = a->o; p.lse = a->lse;
    p.q_sb = a->q_strides[0]; p.q_sh = a->q_strides[1]; p.q_sr = a->q_strides[2];
    p.k_sb = a->k_strides[0]; p.k_sh = a->k_strides[1]; p.k_sr = a->k_strides[2];
    p.v_sb = a->v_strides[0]; p.v_sh = a->v_strides[1]; p.v_sr = a->v_strides[2];
    p.o_sb = a->o_strides[0]; p.o_sh = a->o_strides[1]; p.o_sr = a->o_strides[2];
    p.lse_sb = (int64_t)a->H * a->M; p.lse_sh = a->M; p.lse_sr = 1;
    p.B = a->B; p.H = a->H; p.M = a->M; p.N = a->N;
    p.align_end = 1;
    p.tiles_per_seq = (a->M + 127) / 128;
    const int64_t items = (int64_t)p.tiles_per_seq * a->H * a->B;
    if (items > 0x7fffff00LL) return fail(T5A_ERR_SHAPE, "too many work items (%lld)", (long long)items);
    p.total_items = (int)items;
    if (a->causal != 0 && p.tiles_per_seq > 1) causal_slices(&p, a->dtype, a->D);
    if ((rc = score_mode(a->exact_scores, a->sm_scale, &p))) return rc;
    if ((rc = fill_bias(a->bias, a->causal == 0, &p))) return rc;
    if ((rc = prepare_lut(a->bias, a->causal != 0, (hipStream_t)stream, &p))) return rc;
    return finish(launch_fwd(p, a->dtype, a->D, kDense, a->causal != 0, (hipStream_t)stream), "t5a_fwd_dense");
}

int64_t t5a_bwd_workspace_bytes(int32_t B, int32_t H, int32_t M) {
    if (B < 0 || H < 0 || M < 0) return -1;
    return 2 * (int64_t)B * H * M * (int64_t)sizeof(float);
}

int t5a_bwd_dense(const t5a_dense_bwd_args* a, t5a_stream_t stream) {
    if (a == nullptr) return fail(T5A_ERR_NULL, "args is NULL");
    int rc = check_common(a->dtype, a->D);
    if (rc) return rc;
    if (a->D == 128 && (a->dtype == T5A_F32 || a->fp32_math != 0))
        return fail(T5A_ERR_HEAD_DIM, "backward at head_dim 128: 16-bit tensors on the 16-bit matrix cores only (the fp32 kernels hold a row's head_dim in registers: 16, 32 or 64)");
    const int unit = a->dtype == T5A_F32 ? 4 : 8;
    if (a->B < 0 || a->H <= 0 || a->M < 0 || a->N < 0) return fail(T5A_ERR_SHAPE, "bad sizes B=%d H=%d M=%d N=%d", a->B, a->H, a->M, a->N);
    if (a->B == 0) return T5A_OK;
    struct { const char* name; const void* ptr; const int64_t* st; int rows; } ts[] = {
        {"q", a->q, a->q_strides, a->M}, {"o", a->o, a->o_strides, a->M}, {"dout", a->dout, a->dout_strides, a->M},
        {"dq", a->dq, a->dq_strides, a->M}, {"k", a->k, a->k_strides, a->N}, {"v", a->v, a->v_strides, a->N},
        {"dk", a->dk, a->dk_strides, a->N}, {"dv", a->dv, a->dv_strides, a->N}};
    for (auto& t : ts) {
        if (t.rows == 0) continue;
        if ((rc = check_tensor(t.name, t.ptr, t.st, 3, unit))) return rc;
    }
    if (a->M > 0 && a->lse == nullptr) return fail(T5A_ERR_NULL, "lse is NULL");
    // (the kernels address the rows of a (batch, head) slice with 32-bit byte offsets)
    for (auto& t : ts)
        if (t.rows > 0 && (rc = check_rows(t.name, t.rows, t.st[2], a->dtype))) return rc;
    const int64_t need = t5a_bwd_workspace_bytes(a->B, a->H, a->M);
    if (a->M > 0 && (a->workspace == nullptr || a->workspace_bytes < need))
        return fail(T5A_ERR_WORKSPACE, "t5a_bwd_dense: workspace of %lld bytes needed, %lld given", (long long)need, (long long)a->workspace_bytes);
    if (a->M > 0 && !aligned16(a->workspace)) return fail(T5A_ERR_STRIDE, "workspace is not 16-byte aligned");
    if ((int64_t)a->B > 65535 || (int64_t)a->H > 65535) return fail(T5A_ERR_SHAPE, "B or H too large for the launch grid");
    BwdParams p;
    memset(&p, 0, sizeof(p));
    p.q = a->q; p.k = a->k; p.v = a->v; p.o = a->o; p.dout = a->dout; p.lse = a->lse;
    p.dq = a->dq; p.dk = a->dk; p.dv = a->dv;
    p.q_sb = a->q_strides[0]; p.q_sh = a->q_strides[1]; p.q_sr = a->q_strides[2];
    p.k_sb = a->k_strides[0]; p.k_sh = a->k_strides[1]; p.k_sr = a->k_strides[2];
    p.v_sb = a->v_strides[0]; p.v_sh = a->v_strides[1]; p.v_sr = a->v_strides[2];
    p.o_sb = a->o_strides[0]; p.o_sh = a->o_strides[1]; p.o_sr = a->o_strides[2];
    p.do_sb = a->dout_strides[0]; p.do_sh = a->dout_strides[1]; p.do_sr = a->dout_strides[2];
    p.dq_sb = a->dq_strides[0]; p.dq_sh = a->dq_strides[1]; p.dq_sr = a->dq_strides[2];
    p.dk_sb = a->dk_strides[0]; p.dk_sh = a->dk_strides[1]; p.dk_sr = a->dk_strides[2];
    p.dv_sb = a->dv_strides[0]; p.dv_sh = a->dv_strides[1]; p.dv_sr = a->dv_strides[2];
    p.B = a->B; p.H = a->H; p.M = a->M; p.N = a->N;
    FwdParams f;
    memset(&f, 0, sizeof(f));
    if ((rc = score_mode(a->exact_scores, a->sm_scale, &f))) return rc;
    p.c1 = f.c1;
    if ((rc = fill_bias(a->bias, a->causal == 0, &f))) return rc;
    p.table = f.table; p.table_dtype = f.table_dtype; p.t_sbucket = f.t_sbucket; p.t_shead = f.t_shead; p.bs = f.bs;
    p.n_buckets = a->bias.table != nullptr ? a->bias.num_buckets : 0;
    if (a->bias.table != nullptr && a->dtable == nullptr) return fail(T5A_ERR_NULL, "dtable is NULL (the forward had a bias table)");
    if (p.n_buckets > 4 * kMaxThresholds) return fail(T5A_ERR_BUCKETS, "num_buckets=%d too large for the backward", p.n_buckets);
    p.dtable = a->bias.table != nullptr ? a->dtable : nullptr;
    if (a->M == 0) {
        // no query rows: dk and dv are zero, and so is the table gradient
        hipError_t e = hipSuccess;
        if (a->N > 0) {
            const size_t es = a->dtype == T5A_F32 ? 4 : 2;
            for (void* out : {a->dk, a->dv}) {
                const int64_t* st = out == a->dk ? a->dk_strides : a->dv_strides;
                if (st[2] != a->D || st[1] != (int64_t)a->N * a->D || st[0] != (int64_t)a->H * a->N * a->D)
                    return fail(T5A_ERR_STRIDE, "M == 0: dk and dv must be contiguous");
                if (e == hipSuccess) e = hipMemsetAsync(out, 0, (size_t)a->B * a->H * a->N * a->D * es, (hipStream_t)stream);
            }
        }
        if (e == hipSuccess && p.dtable != nullptr)
            e = hipMemsetAsync(p.dtable, 0, (size_t)p.n_buckets * a->H * sizeof(float), (hipStream_t)stream);
        return finish(e, "t5a_bwd_dense (no query rows)");
    }
    p.fp32_math = a->fp32_math;
    p.delta = reinterpret_cast<float*>(a->workspace);
    p.lse2 = p.delta + (int64_t)a->B * a->H * a->M;
    return finish(launch_bwd_dense(p, a->dtype, a->D, a->causal != 0, (hipStream_t)stream), "t5a_bwd_dense");
}

int64_t t5a_bwd_varlen_workspace_bytes(int32_t total_q, int32_t H) {
    if (total_q < 0 || H < 0) return -1;
    return 2 * (int64_t)total_q * H * (int64_t)sizeof(float);
}

int t5a_bwd_varlen(const t5a_varlen_bwd_args* a, t5a_stream_t stream) {
    if (a == nullptr) return fail(T5A_ERR_NULL, "args is NULL");
    int rc = check_common(a->dtype, a->D);
    if (rc) return rc;
    if (a->D == 128 && (a->dtype == T5A_F32 || a->fp32_math != 0))
        return fail(T5A_ERR_HEAD_DIM, "backward at head_dim 128: 16-bit tensors on the 16-bit matrix cores only (the fp32 kernels hold a row's head_dim in registers: 16, 32 or 64)");
    const int unit = a->dtype == T5A_F32 ? 4 : 8;
    if (a->B < 0 || a->H <= 0 || a->total_q < 0 || a->total_k < 0 || a->max_seqlen_q < 0 || a->max_seqlen_k < 0)
        return fail(T5A_ERR_SHAPE, "bad sizes B=%d H=%d total_q=%d total_k=%d", a->B, a->H, a->total_q, a->total_k);
    if (a->B == 0 || (a->total_q == 0 && a->total_k == 0)) return T5A_OK;
    if (a->cu_seqlens_q == nullptr || a->cu_seqlens_k == nullptr) return fail(T5A_ERR_NULL, "cu_seqlens is NULL");
    if (a->total_q == 0 || a->total_k == 0)
        return fail(T5A_ERR_SHAPE, "t5a_bwd_varlen needs query rows and keys (total_q=%d total_k=%d)", a->total_q, a->total_k);
    struct { const char* name; const void* ptr; const int64_t* st; } ts[] = {
        {"q", a->q, a->q_strides}, {"o", a->o, a->o_strides}, {"dout", a->dout, a->dout_strides}, {"dq", a->dq, a->dq_strides},
        {"k", a->k, a->k_strides}, {"v", a->v, a->v_strides}, {"dk", a->dk, a->dk_strides}, {"dv", a->dv, a->dv_strides}};
    for (auto& t : ts) {
        if ((rc = check_tensor(t.name, t.ptr, t.st, 2, unit))) return rc;
        // (a sequence's rows are addressed with 32-bit byte offsets from its first row)
        if ((rc = check_rows(t.name, a->max_seqlen_q > a->max_seqlen_k ? a->max_seqlen_q : a->max_seqlen_k, t.st[0], a->dtype))) return rc;
    }
    if (a->lse == nullptr) return fail(T5A_ERR_NULL, "lse is NULL");
    const int64_t need = t5a_bwd_varlen_workspace_bytes(a->total_q, a->H);
    if (a->workspace == nullptr || a->workspace_bytes < need)
        return fail(T5A_ERR_WORKSPACE, "t5a_bwd_varlen: workspace of %lld bytes needed, %lld given", (long long)need, (long long)a->workspace_bytes);
    if (!aligned16(a->workspace)) return fail(T5A_ERR_STRIDE, "workspace is not 16-byte aligned");
    if ((int64_t)a->B > 65535 || (int64_t)a->H > 65535) return fail(T5A_ERR_SHAPE, "B or H too large for the launch grid");
    BwdParams p;
    memset(&p, 0, sizeof(p));
    p.q = a->q; p.k = a->k; p.v = a->v; p.o = a->o; p.dout = a->dout; p.lse = a->lse;
    p.dq = a->dq; p.dk = a->dk; p.dv = a->dv;
    p.q_sr = a->q_strides[0]; p.q_sh = a->q_strides[1];
    p.k_sr = a->k_strides[0]; p.k_sh = a->k_strides[1];
    p.v_sr = a->v_strides[0]; p.v_sh = a->v_strides[1];
    p.o_sr = a->o_strides[0]; p.o_sh = a->o_strides[1];
    p.do_sr = a->dout_strides[0]; p.do_sh = a->dout_strides[1];
    p.dq_sr = a->dq_strides[0]; p.dq_sh = a->dq_strides[1];
    p.dk_sr = a->dk_strides[0]; p.dk_sh = a->dk_strides[1];
    p.dv_sr = a->dv_strides[0]; p.dv_sh = a->dv_strides[1];
    p.B = a->B; p.H = a->H; p.M = a->max_seqlen_q; p.N = a->max_seqlen_k;
    p.cu_q = a->cu_seqlens_q; p.cu_k = a->cu_seqlens_k; p.len_q = a->seq_lens_q; p.len_k = a->seq_lens_k;
    p.total_q = a->total_q;
    FwdParams f;
    memset(&f, 0, sizeof(f));
    if ((rc = score_mode(a->exact_scores, a->sm_scale, &f))) return rc;
    p.c1 = f.c1;
    if ((rc = fill_bias(a->bias, a->causal == 0, &f))) return rc;
    p.table = f.table; p.table_dtype = f.table_dtype; p.t_sbucket = f.t_sbucket; p.t_shead = f.t_shead; p.bs = f.bs;
    p.n_buckets = a->bias.table != nullptr ? a->bias.num_buckets : 0;
    if (a->bias.table != nullptr && a->dtable == nullptr) return fail(T5A_ERR_NULL, "dtable is NULL (the forward had a bias table)");
    if (p.n_buckets > 4 * kMaxThresholds) return fail(T5A_ERR_BUCKETS, "num_buckets=%d too large for the backward", p.n_buckets);
    p.dtable = a->bias.table != nullptr ? a->dtable : nullptr;
    if (p.M == 0 || p.N == 0) return fail(T5A_ERR_SHAPE, "max_seqlen_q and max_seqlen_k must be positive");
    p.fp32_math = a->fp32_math;
    p.delta = reinterpret_cast<float*>(a->workspace);
    p.lse2 = p.delta + (int64_t)a->total_q * a->H;
    return finish(launch_bwd_dense(p, a->dtype, a->D, a->causal != 0, (hipStream_t)stream), "t5a_bwd_varlen");
}

// Entries per XCD of a packed batch's launch plan: twice the mean, so that slices of equal work but
// unequal item counts fit (a slice that still outgrows it spills into the others' free slots).
static int plan_slots(int64_t items_bound) { return (int)(2 * ((items_bound + 7) / 8)); }

int64_t t5a_varlen_workspace_bytes(int32_t B, int32_t H, int32_t total_q) {
    if (B <= 0 || H <= 0 || total_q <= 0 || B > kPlanMaxSeqs) return 0;
    const int64_t items = ((int64_t)total_q / 128 + B) * H;
    if (items > 0x03ffff00LL) return 0;
    return 64 + (int64_t)8 * plan_slots(items) * 32 + items * 16;   // counts, the lists, room for spilled items
}

int t5a_fwd_varlen(const t5a_varlen_args* a, t5a_stream_t stream) {
    if (a == nullptr) return fail(T5A_ERR_NULL, "args is NULL");
    int rc = check_common(a->dtype, a->D);
    if (rc) return rc;
    const int unit = a->dtype == T5A_F32 ? 4 : 8;
    if (a->B < 0 || a->H <= 0 || a->total_q < 0 || a->total_k < 0)
        return fail(T5A_ERR_SHAPE, "bad sizes B=%d H=%d total_q=%d total_k=%d", a->B, a->H, a->total_q, a->total_k);
    if (a->B == 0 || a->total_q == 0) return T5A_OK;
    if (a->cu_seqlens_q == nullptr || a->cu_seqlens_k == nullptr) return fail(T5A_ERR_NULL, "cu_seqlens is NULL");
    if ((rc = check_tensor("q", a->q, a->q_strides, 2, unit))) return rc;
    if ((rc = check_tensor("o", a->o, a->o_strides, 2, unit))) return rc;
    if (a->total_k > 0) {
        if ((rc = check_tensor("k", a->k, a->k_strides, 2, unit))) return rc;
        if ((rc = check_tensor("v", a->v, a->v_strides, 2, unit))) return rc;
        if ((rc = check_rows("k", a->max_seqlen_k, a->k_strides[0], a->dtype))) return rc;
        if ((rc = check_rows("v", a->max_seqlen_k, a->v_strides[0], a->dtype))) return rc;
    }
    if ((rc = check_rows("q", a->max_seqlen_q, a->q_strides[0], a->dtype))) return rc;
    FwdParams p;
    memset(&p, 0, sizeof(p));
    p.q = a->q; p.k = a->k; p.v = a->v; p.o = a->o; p.lse = a->lse;
    p.q_sr = a->q_strides[0]; p.q_sh = a->q_strides[1];
    p.k_sr = a->k_strides[0]; p.k_sh = a->k_strides[1];
    p.v_sr = a->v_strides[0]; p.v_sh = a->v_strides[1];
    p.o_sr = a->o_strides[0]; p.o_sh = a->o_strides[1];
    p.lse_sr = a->H; p.lse_sh = 1;
    p.cu_q = a->cu_seqlens_q; p.cu_k = a->cu_seqlens_k;
    p.len_q = a->seq_lens_q; p.len_k = a->seq_lens_k;
    p.B = a->B; p.H = a->H; p.M = a->max_seqlen_q; p.N = a->max_seqlen_k;
    // sum_b ceil(len_b / 128) <= total_q / 128 + B: launch that many, the surplus exits
    const int64_t items = ((int64_t)a->total_q / 128 + a->B) * a->H;
    if (items > 0x7fffff00LL) return fail(T5A_ERR_SHAPE, "too many work items (%lld)", (long long)items);
    p.total_items = (int)items;
    p.tiles_per_seq = 1;
    p.align_end = 1;
    if ((rc = score_mode(a->exact_scores, a->sm_scale, &p))) return rc;
    if ((rc = fill_bias(a->bias, a->causal == 0, &p))) return rc;
    if ((rc = prepare_lut(a->bias, a->causal != 0, (hipStream_t)stream, &p))) return rc;
    const int64_t need = t5a_varlen_workspace_bytes(a->B, a->H, a->total_q);
    if (a->workspace != nullptr && need > 0) {
        // launch plan: per-XCD item lists of equal work, longest first, built on the device
        if (a->workspace_bytes < need)
            return fail(T5A_ERR_WORKSPACE, "workspace too small: %lld bytes, t5a_varlen_workspace_bytes() asks for %lld",
                        (long long)a->workspace_bytes, (long long)need);
        if ((reinterpret_cast<uintptr_t>(a->workspace) & 15) != 0)
            return fail(T5A_ERR_STRIDE, "workspace must be 16-byte aligned");
        PlanParams pl;
        memset(&pl, 0, sizeof(pl));
        pl.cu_q = a->cu_seqlens_q; pl.cu_k = a->cu_seqlens_k; pl.len_q = a->seq_lens_q; pl.len_k = a->seq_lens_k;
        pl.B = a->B; pl.H = a->H; pl.causal = a->causal != 0;
        pl.bn_shift = (a->dtype != T5A_F32 && a->D == 128) ? 5 : 6;
        const int max_cost = (a->max_seqlen_k >> pl.bn_shift) + 8;
        while ((max_cost >> pl.key_shift) >= 512) ++pl.key_shift;
        pl.slots = plan_slots(items);
        pl.staged = plan_can_stage(pl.slots, a->H, a->max_seqlen_q) ? 1 : 0;
        pl.counts = static_cast<int32_t*>(a->workspace);
        pl.plan = pl.counts + 16;
        pl.spill = pl.plan + (size_t)8 * pl.slots * 8;
        if (a->workspace_ready == 0) {
            hipError_t e = launch_varlen_plan(pl, (hipStream_t)stream);
            if (e != hipSuccess) return finish(e, "t5a_fwd_varlen (plan)");
        }
        p.plan = pl.plan;
        p.plan_counts = pl.counts;
        p.plan_slots = pl.slots;
    }
    return finish(launch_fwd(p, a->dtype, a->D, kPacked, a->causal != 0, (hipStream_t)stream), "t5a_fwd_varlen");
}

// Compute units of the current device (cached per device index).
static int device_compute_units() {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static int cus[kMaxDevices] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
    std::lock_guard<std::mutex> g(mu);
    if (cus[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cus[dev] = n;
    }
    return cus[dev];
}

// Sparse patterns: how many consecutive q tiles of one (batch, head) a workgroup takes.  A q tile of a sparse
// pattern is only a few steps long, about as long as the set-up of a work item, which a run pays once; longer runs
// mean fewer workgroups.  Two workgroups fit a compute unit: count the rounds the device needs for the runs and
// charge every round its q tiles plus one set-up.
static void choose_runs(FwdParams* p, int mode, int dtype, int D, int cus, int forced_run_len, int64_t other_items = 0) {
    p->run_len = 1;
    p->runs_per_seq = p->tiles_per_seq;
    const int64_t entries = (int64_t)p->tiles_per_seq * p->H * p->B;   // the (batch, head, q tile) list
    // the geometries staged by LDS-DMA
    const bool runs_ok = (mode == kLocal || mode == kBlock) && dtype != T5A_F32 && (D == 64 || D == 128);
    if (runs_ok) {
        // as many workgroups as the device holds at once (two per compute unit), each with its share of the list;
        // other_items: workgroups of the same launch that are not runs (the block pattern's key splits)
        int64_t slots = 2 * (int64_t)cus - other_items;
        if (slots < 64) slots = 64;
        int64_t rl = (entries + slots - 1) / slots;
        if (rl > kMaxRunLen) rl = kMaxRunLen;
        if (rl < 1) rl = 1;
        p->run_len = (int)rl;
        if (forced_run_len >= 1) p->run_len = forced_run_len;   // the caller's choice (validated: 1 .. kMaxRunLen)
    }
    p->total_items = (int)((entries + p->run_len - 1) / p->run_len);
}

// Key splits for the global rows of the block pattern: enough (batch, head, split) items to fill the
// device about twice, at least four key tiles of 64 per split.
static void global_row_splits(int B, int H, int L, int* nsplit, int* split_rows) {
    const int tiles = (L + 63) / 64;
    const int64_t bh = (int64_t)B * H;
    int64_t want = bh > 0 ? (512 + bh - 1) / bh : 1;
    if (want > tiles / 4) want = tiles / 4;
    if (want < 1) want = 1;
    const int per = (int)((tiles + want - 1) / want);   // tiles per split
    *split_rows = per * 64;
    *nsplit = (tiles + per - 1) / per;
}

// Block pattern with the global rows' key splits in the same launch: run length of the block items and number of
// key splits, chosen together so that runs and splits fill one round of workgroups and end at about the same time.
// Costs in thousands of cycles, measured on an MI355X: a run pays one set-up (15) and per q tile three steps and
// the switch to the next q tile (15.6); a split pays one set-up (16) and 2.0 per key tile.  Never more splits than
// global_row_splits() gives: the workspace size is computed from that.
static void block_fold_plan(FwdParams* p, int dtype, int D, int B, int H, int L, int cus, int forced_run_len,
                            int* nsplit, int* split_rows) {
    global_row_splits(B, H, L, nsplit, split_rows);
    const int most_splits = *nsplit;   // what the workspace was sized for
    const int64_t bh = (int64_t)B * H;
    const int64_t entries = (int64_t)p->tiles_per_seq * bh;
    const int64_t slots = 2 * (int64_t)cus;
    const bool runs_ok = dtype != T5A_F32 && (D == 64 || D == 128);
    if (!runs_ok || forced_run_len >= 1 || entries + (int64_t)*nsplit * bh <= slots) {
        choose_runs(p, kBlock, dtype, D, cus, forced_run_len, (int64_t)*nsplit * bh);
        return;
    }
    const int tiles = (L + 63) / 64;
    double best = 0.0;
    int best_r = 0, best_s = 0;
    for (int r = 1; r <= kMaxRunLen; ++r) {
        const int64_t n_runs = (entries + r - 1) / r;
        const int64_t free_slots = slots - n_runs;
        if (free_slots < bh) continue;
        int64_t per_bh = free_slots / bh;   // >= 1: one split is a whole pass over the keys, still an item of its own
        if (per_bh > most_splits) per_bh = most_splits;
        const int s_tiles = (int)((tiles + per_bh - 1) / per_bh);
        const double run_cost = 15.0 + 15.6 * r, split_cost = 16.0 + 2.0 * s_tiles;
        const double cost = run_cost > split_cost ? run_cost : split_cost;
        if (best_r == 0 || cost < best) { best = cost; best_r = r; best_s = s_tiles; }
    }
    if (best_r == 0) {   // more work than one round holds at any run length
        choose_runs(p, kBlock, dtype, D, cus, forced_run_len, (int64_t)*nsplit * bh);
        return;
    }
    p->run_len = best_r;
    p->runs_per_seq = p->tiles_per_seq;
    p->total_items = (int)((entries + best_r - 1) / best_r);
    *split_rows = best_s * 64;
    *nsplit = (tiles + best_s - 1) / best_s;
}

// What a folded block launch must satisfy before it may start (every item index the kernel decodes stays inside
// the lists): the runs cover the (batch, head, q tile) list, the splits cover the keys, and there are no more
// splits than the workspace holds.
static int check_fold_plan(const FwdParams& p, int B, int H, int L, int nsplit, int split_rows) {
    int most, rows_unused;
    global_row_splits(B, H, L, &most, &rows_unused);
    const int64_t entries = (int64_t)p.tiles_per_seq * H * B;
    if (p.run_len < 1 || p.run_len > kMaxRunLen || (int64_t)p.total_items * p.run_len < entries ||
        (int64_t)(p.total_items - 1) * p.run_len >= entries)
        return fail(T5A_ERR_LAUNCH, "block launch plan: %d runs of %d q tiles do not cover %lld entries", p.total_items,
                    p.run_len, (long long)entries);
    if (nsplit < 1 || nsplit > most || split_rows < 64 || split_rows % 64 != 0 || (int64_t)nsplit * split_rows < L ||
        (int64_t)(nsplit - 1) * split_rows >= L)
        return fail(T5A_ERR_LAUNCH, "block launch plan: %d key splits of %d rows do not cover %d keys (at most %d splits)",
                    nsplit, split_rows, L, most);
    return T5A_OK;
}

int64_t t5a_sparse_key_bits_words(int32_t L, int32_t block_len, int32_t aux) {
    if (L < 0 || block_len <= 0 || aux < 0) return -1;
    // tiles reach up to block_len + 128 keys past the last token, the block pattern looks block_len + aux further
    return kKeyBitsFront + ((int64_t)L + 2 * (int64_t)block_len + aux + 256 + 31) / 32 + 4;
}

int64_t t5a_sparse_workspace_bytes(int32_t pattern, int32_t B, int32_t H, int32_t L, int32_t D, int32_t block_len, int32_t aux) {
    if (B < 0 || H < 0 || L < 0 || D < 0 || block_len <= 0 || aux < 0) return -1;
    if (pattern != T5A_PATTERN_BLOCK || aux == 0 || L < block_len) return 0;
    int nsplit, split_rows;
    global_row_splits(B, H, L, &nsplit, &split_rows);
    if (nsplit < 2) return 0;
    const int64_t G = aux < L ? aux : L;
    return (int64_t)B * H * nsplit * G * ((int64_t)D + 2) * (int64_t)sizeof(float);
}

int t5a_sparse_launch_plan(int32_t pattern, int32_t dtype, int32_t B, int32_t H, int32_t L, int32_t D, int32_t block_len,
                           int32_t aux, int32_t with_workspace, int32_t compute_units, int32_t run_len, int32_t* out) {
    if (out == nullptr) return fail(T5A_ERR_NULL, "out is NULL");
    int rc = check_common(dtype, D);
    if (rc) return rc;
    if (B <= 0 || H <= 0 || L <= 0 || block_len <= 0 || aux < 0 || run_len < 0 || run_len > kMaxRunLen)
        return fail(T5A_ERR_SHAPE, "bad sizes B=%d H=%d L=%d block_len=%d aux=%d run_len=%d", B, H, L, block_len, aux, run_len);
    const int cus = compute_units > 0 ? compute_units : device_compute_units();
    FwdParams p;
    memset(&p, 0, sizeof(p));
    p.B = B; p.H = H; p.M = L; p.N = L;
    int nsplit = 0, split_rows = 0, block_items = 0;
    if (pattern == T5A_PATTERN_BLOCK && L >= block_len) {
        p.tiles_per_seq = ((L + block_len - 1) / block_len) * ((block_len + 127) / 128);
        const int G = aux < L ? aux : L;
        const bool fold = aux > 0 && with_workspace != 0 && G <= 128 &&
                          t5a_sparse_workspace_bytes(pattern, B, H, L, D, block_len, aux) > 0;
        if (fold) {
            block_fold_plan(&p, dtype, D, B, H, L, cus, run_len, &nsplit, &split_rows);
            if ((rc = check_fold_plan(p, B, H, L, nsplit, split_rows))) return rc;
            block_items = p.total_items;
            p.total_items += nsplit * H * B;
        } else {
            choose_runs(&p, kBlock, dtype, D, cus, run_len);
        }
    } else if (pattern == T5A_PATTERN_LOCAL || pattern == T5A_PATTERN_TGLOBAL || pattern == T5A_PATTERN_BLOCK) {
        // (a block pattern over less than one block runs as full attention)
        p.tiles_per_seq = (L + 127) / 128;
        const int mode = pattern == T5A_PATTERN_BLOCK ? kDense : pattern == T5A_PATTERN_TGLOBAL ? kTGlobal
                         : (block_len <= kMaxLutWindow ? kLocal : kLocalWide);
        choose_runs(&p, mode, dtype, D, cus, run_len);
    } else {
        return fail(T5A_ERR_PATTERN, "unknown pattern %d", pattern);
    }
    out[0] = p.run_len; out[1] = p.total_items; out[2] = block_items; out[3] = nsplit; out[4] = split_rows;
    out[5] = p.tiles_per_seq;
    return T5A_OK;
}

int t5a_fwd_sparse(const t5a_sparse_args* a, t5a_stream_t stream) {
    if (a == nullptr) return fail(T5A_ERR_NULL, "args is NULL");
    int rc = check_common(a->dtype, a->D);
    if (rc) return rc;
    const int unit = a->dtype == T5A_F32 ? 4 : 8;
    if (a->B < 0 || a->H <= 0 || a->L < 0) return fail(T5A_ERR_SHAPE, "bad sizes B=%d H=%d L=%d", a->B, a->H, a->L);
    if (a->pattern != T5A_PATTERN_LOCAL && a->pattern != T5A_PATTERN_BLOCK && a->pattern != T5A_PATTERN_TGLOBAL)
        return fail(T5A_ERR_PATTERN, "unknown pattern %d", a->pattern);
    if (a->block_len <= 0) return fail(T5A_ERR_PATTERN, "block_len=%d must be positive", a->block_len);
    if (a->pattern == T5A_PATTERN_BLOCK && (a->aux < 0 || a->aux > a->block_len))
        return fail(T5A_ERR_PATTERN, "block pattern needs 0 <= n_global (%d) <= block_len (%d)", a->aux, a->block_len);
    if (a->pattern == T5A_PATTERN_TGLOBAL && (a->aux <= 0 || a->n_side < 0))
        return fail(T5A_ERR_PATTERN, "transient-global needs aux > 0 and n_side >= 0 (aux=%d n_side=%d)", a->aux, a->n_side);
    if (a->run_len < 0 || a->run_len > kMaxRunLen)
        return fail(T5A_ERR_SHAPE, "run_len=%d: 0 (the library chooses) or 1..%d", a->run_len, kMaxRunLen);
    if (a->B == 0 || a->L == 0) return T5A_OK;
    const int cus = device_compute_units();
    if ((rc = check_tensor("q", a->q, a->q_strides, 3, unit))) return rc;
    if ((rc = check_tensor("k", a->k, a->k_strides, 3, unit))) return rc;
    if ((rc = check_tensor("v", a->v, a->v_strides, 3, unit))) return rc;
    if ((rc = check_tensor("o", a->o, a->o_strides, 3, unit))) return rc;
    if ((rc = check_rows("q", a->L, a->q_strides[2], a->dtype))) return rc;
    if ((rc = check_rows("k", a->L, a->k_strides[2], a->dtype))) return rc;
    if ((rc = check_rows("v", a->L, a->v_strides[2], a->dtype))) return rc;
    if (a->pattern == T5A_PATTERN_TGLOBAL && a->n_side > 0) {
        if ((rc = check_tensor("side_k", a->side_k, a->side_k_strides, 3, unit))) return rc;
        if ((rc = check_tensor("side_v", a->side_v, a->side_v_strides, 3, unit))) return rc;
        if ((rc = check_rows("side_k", a->n_side, a->side_k_strides[2], a->dtype))) return rc;
        if ((rc = check_rows("side_v", a->n_side, a->side_v_strides[2], a->dtype))) return rc;
    }
    FwdParams p;
    memset(&p, 0, sizeof(p));
    p.q = a->q; p.k = a->k; p.v = a->v; p.o = a->o;
    p.side_k = a->side_k; p.side_v = a->side_v;
    p.q_sb = a->q_strides[0]; p.q_sh = a->q_strides[1]; p.q_sr = a->q_strides[2];
    p.k_sb = a->k_strides[0]; p.k_sh = a->k_strides[1]; p.k_sr = a->k_strides[2];
    p.v_sb = a->v_strides[0]; p.v_sh = a->v_strides[1]; p.v_sr = a->v_strides[2];
    p.o_sb = a->o_strides[0]; p.o_sh = a->o_strides[1]; p.o_sr = a->o_strides[2];
    p.sk_sb = a->side_k_strides[0]; p.sk_sh = a->side_k_strides[1]; p.sk_sr = a->side_k_strides[2];
    p.sv_sb = a->side_v_strides[0]; p.sv_sh = a->side_v_strides[1]; p.sv_sr = a->side_v_strides[2];
    p.B = a->B; p.H = a->H; p.M = a->L; p.N = a->L;
    if (a->seq_starts != nullptr && (a->seq_lens == nullptr || a->pattern == T5A_PATTERN_BLOCK))
        return fail(T5A_ERR_PATTERN, "seq_starts needs seq_lens and the local or transient-global pattern");
    p.len_k = a->seq_lens;
    p.start_k = a->seq_starts;
    if (a->key_bits != nullptr) {
        if (a->pattern == T5A_PATTERN_TGLOBAL && a->side_counts == nullptr)
            return fail(T5A_ERR_NULL, "transient-global pattern: key_bits needs side_counts");
        if (a->seq_lens != nullptr) return fail(T5A_ERR_PATTERN, "key_bits and seq_lens are alternatives");
        const int64_t need = t5a_sparse_key_bits_words(a->L, a->block_len, a->aux);
        if (a->key_bits_stride < need)
            return fail(T5A_ERR_SHAPE, "key_bits_stride %lld, t5a_sparse_key_bits_words() asks for %lld",
                        (long long)a->key_bits_stride, (long long)need);
        if ((reinterpret_cast<uintptr_t>(a->key_bits) & 3) != 0) return fail(T5A_ERR_STRIDE, "key_bits must be 4-byte aligned");
        if (a->pattern == T5A_PATTERN_BLOCK && a->L < a->block_len)
            return fail(T5A_ERR_PATTERN, "block pattern: key_bits with a sequence shorter than one block is not supported");
        p.key_bits = a->key_bits;
        p.key_bits_stride = a->key_bits_stride;
        if (a->pattern == T5A_PATTERN_TGLOBAL) p.side_counts = a->side_counts;
    }
    p.block_len = a->block_len; p.aux = a->aux; p.n_side = a->n_side;
    if ((rc = score_mode(a->exact_scores, a->sm_scale, &p))) return rc;
    if ((rc = fill_bias(a->bias, true, &p))) return rc;
    hipStream_t s = (hipStream_t)stream;
    const bool window_in_lut = a->pattern == T5A_PATTERN_LOCAL && a->block_len <= kMaxLutWindow && a->key_bits == nullptr;
    if ((rc = prepare_lut(a->bias, false, s, &p, window_in_lut ? a->block_len : 0))) return rc;

    if (a->pattern == T5A_PATTERN_BLOCK) {
        if (a->L < a->block_len) {
            // shorter than one block: the reference degenerates to full attention (attentions.py:752, :691)
            p.tiles_per_seq = (a->L + 127) / 128;
            p.total_items = p.tiles_per_seq * a->H * a->B;
            if (a->seq_lens != nullptr)
                return fail(T5A_ERR_PATTERN, "block pattern: seq_lens with a sequence shorter than one block is not supported");
            return finish(launch_fwd(p, a->dtype, a->D, kDense, false, s), "t5a_fwd_sparse(block, short)");
        }
        // rows >= G attend [global tokens | own block]; the G global queries attend every key with absolute positions
        // (rel = j - i, no end alignment)
        const int nblk = (a->L + a->block_len - 1) / a->block_len;
        p.tiles_per_seq = nblk * ((a->block_len + 127) / 128);
        const int G = a->aux < a->L ? a->aux : a->L;
        const int64_t need = t5a_sparse_workspace_bytes(a->pattern, a->B, a->H, a->L, a->D, a->block_len, a->aux);
        const bool fold = a->aux > 0 && a->workspace != nullptr && need > 0 && G <= 128;
        int fold_splits = 0, fold_rows = 0;
        if (fold) block_fold_plan(&p, a->dtype, a->D, a->B, a->H, a->L, cus, a->run_len, &fold_splits, &fold_rows);
        else choose_runs(&p, kBlock, a->dtype, a->D, cus, a->run_len);
        if (fold) {
            if ((rc = check_fold_plan(p, a->B, a->H, a->L, fold_splits, fold_rows))) return rc;
            // one launch: the block items, then the global rows as key splits spread over the whole device; one merge
            if (a->workspace_bytes < need)
                return fail(T5A_ERR_WORKSPACE, "workspace of %lld bytes, %lld needed", (long long)a->workspace_bytes, (long long)need);
            if (!aligned16(a->workspace)) return fail(T5A_ERR_STRIDE, "workspace is not 16-byte aligned");
            p.nsplit = fold_splits; p.split_rows = fold_rows;   // (never more splits than the workspace size assumes)
            const int64_t rows = (int64_t)a->B * a->H * p.nsplit * G;
            p.part_o = reinterpret_cast<float*>(a->workspace);
            p.part_l = p.part_o + rows * a->D;
            p.part_m = p.part_l + rows;
            p.block_items = p.total_items;
            const int64_t items = (int64_t)p.block_items + (int64_t)p.nsplit * a->H * a->B;
            if (items > 0x7fffff00LL) return fail(T5A_ERR_SHAPE, "too many work items (%lld)", (long long)items);
            p.total_items = (int)items;
            rc = finish(launch_fwd(p, a->dtype, a->D, (a->key_bits != nullptr || a->seq_lens != nullptr) ? kBlockBits : kBlock, false, s), "t5a_fwd_sparse(block + global rows as key splits)");
            if (rc) return rc;
            SplitKParams m;
            memset(&m, 0, sizeof(m));
            m.o = a->o; m.part_o = p.part_o; m.part_l = p.part_l; m.part_m = p.part_m;
            m.o_sb = p.o_sb; m.o_sh = p.o_sh; m.o_sr = p.o_sr;
            m.B = a->B; m.H = a->H; m.M = G; m.S = p.nsplit;
            return finish(launch_splitk_merge(m, a->dtype, a->D, s), "t5a_fwd_sparse(block, merge)");
        }
        rc = finish(launch_fwd(p, a->dtype, a->D, (a->key_bits != nullptr || a->seq_lens != nullptr) ? kBlockBits : kBlock, false, s), "t5a_fwd_sparse(block)");
        if (rc || a->aux == 0) return rc;
        // the G global queries as a pass of their own: M is clipped to G rows of the same tensors
        FwdParams g = p;
        g.run_len = 1;
        g.len_k = nullptr;
        g.key_bits = nullptr;
        g.M = G;
        g.N = a->L;
        g.tiles_per_seq = (g.M + 127) / 128;
        g.total_items = g.tiles_per_seq * a->H * a->B;
        g.align_end = 0;
        if (a->workspace != nullptr && need > 0) {
            // (more than 128 global rows) key splits over the whole device in a second launch, then one merge
            if (a->workspace_bytes < need)
                return fail(T5A_ERR_WORKSPACE, "workspace of %lld bytes, %lld needed", (long long)a->workspace_bytes, (long long)need);
            if (!aligned16(a->workspace)) return fail(T5A_ERR_STRIDE, "workspace is not 16-byte aligned");
            global_row_splits(a->B, a->H, a->L, &g.nsplit, &g.split_rows);
            const int64_t rows = (int64_t)a->B * a->H * g.nsplit * g.M;
            g.part_o = reinterpret_cast<float*>(a->workspace);
            g.part_l = g.part_o + rows * a->D;
            g.part_m = g.part_l + rows;
            const int64_t items = (int64_t)g.tiles_per_seq * g.nsplit * a->H * a->B;
            if (items > 0x7fffff00LL) return fail(T5A_ERR_SHAPE, "too many work items (%lld)", (long long)items);
            g.total_items = (int)items;
            rc = finish(launch_fwd(g, a->dtype, a->D, kDense, false, s), "t5a_fwd_sparse(block, global rows, key splits)");
            if (rc) return rc;
            SplitKParams m;
            memset(&m, 0, sizeof(m));
            m.o = a->o; m.part_o = g.part_o; m.part_l = g.part_l; m.part_m = g.part_m;
            m.o_sb = p.o_sb; m.o_sh = p.o_sh; m.o_sr = p.o_sr;
            m.B = a->B; m.H = a->H; m.M = g.M; m.S = g.nsplit;
            return finish(launch_splitk_merge(m, a->dtype, a->D, s), "t5a_fwd_sparse(block, merge)");
        }
        return finish(launch_fwd(g, a->dtype, a->D, kDense, false, s), "t5a_fwd_sparse(block, global rows)");
    }
    p.tiles_per_seq = (a->L + 127) / 128;
    // (validity bit sets go with the instantiation that masks per element)
    const int mode = a->pattern == T5A_PATTERN_TGLOBAL ? (a->key_bits != nullptr ? kTGlobalBits : kTGlobal)
                     : (a->block_len <= kMaxLutWindow && a->key_bits == nullptr ? kLocal : kLocalWide);
    choose_runs(&p, mode, a->dtype, a->D, cus, a->run_len);
    return finish(launch_fwd(p, a->dtype, a->D, mode, false, s), "t5a_fwd_sparse");
}

int64_t t5a_splitk_workspace_bytes(int32_t B, int32_t H, int32_t M, int32_t D, int32_t num_splits) {
    if (B < 0 || H < 0 || M < 0 || D < 0 || num_splits < 0) return -1;
    return (int64_t)B * H * num_splits * M * ((int64_t)D + 2) * (int64_t)sizeof(float);
}

// Shared by t5a_fwd_splitk (caller's workspace) and t5a_fwd_splitk_static (the library's static scratch array).
static int splitk_run(const t5a_splitk_args* a, void* workspace, int64_t workspace_bytes, t5a_stream_t stream,
                      const char* what) {
    int rc = check_common(a->dtype, a->D);
    if (rc) return rc;
    if (a->B < 0 || a->H <= 0 || a->M < 0 || a->N < 0) return fail(T5A_ERR_SHAPE, "bad sizes B=%d H=%d M=%d N=%d", a->B, a->H, a->M, a->N);
    if (a->num_splits < 1 || a->num_splits > 65535) return fail(T5A_ERR_SHAPE, "num_splits=%d out of range", a->num_splits);
    if (a->H > 65535 || (int64_t)a->B * ((a->M + 3) / 4 + 1) > 65535) return fail(T5A_ERR_SHAPE, "B*M or H too large for the launch grid");
    if (a->B == 0 || a->M == 0) return T5A_OK;
    const int unit = a->dtype == T5A_F32 ? 4 : 8;
    if ((rc = check_tensor("q", a->q, a->q_strides, 3, unit))) return rc;
    if ((rc = check_tensor("o", a->o, a->o_strides, 3, 1))) return rc;
    if (a->N > 0) {
        if ((rc = check_tensor("k", a->k, a->k_strides, 3, unit))) return rc;
        if ((rc = check_tensor("v", a->v, a->v_strides, 3, unit))) return rc;
    }
    const int64_t need = t5a_splitk_workspace_bytes(a->B, a->H, a->M, a->D, a->num_splits);
    if (workspace == nullptr || workspace_bytes < need)
        return fail(T5A_ERR_WORKSPACE, "%s: workspace of %lld bytes needed, %lld given", what, (long long)need, (long long)workspace_bytes);
    if (!aligned16(workspace)) return fail(T5A_ERR_STRIDE, "workspace is not 16-byte aligned");
    SplitKParams p;
    memset(&p, 0, sizeof(p));
    p.q = a->q; p.k = a->k; p.v = a->v; p.o = a->o; p.bias = a->attn_bias;
    if (a->key_starts != nullptr && a->key_lens == nullptr) return fail(T5A_ERR_NULL, "key_starts given without key_lens");
    p.key_lens = a->key_lens; p.key_starts = a->key_starts;
    const int64_t rows = (int64_t)a->B * a->H * a->num_splits * a->M;
    p.part_o = reinterpret_cast<float*>(workspace);
    p.part_l = p.part_o + rows * a->D;
    p.part_m = p.part_l + rows;
    p.q_sb = a->q_strides[0]; p.q_sh = a->q_strides[1]; p.q_sr = a->q_strides[2];
    p.k_sb = a->k_strides[0]; p.k_sh = a->k_strides[1]; p.k_sr = a->k_strides[2];
    p.v_sb = a->v_strides[0]; p.v_sh = a->v_strides[1]; p.v_sr = a->v_strides[2];
    p.o_sb = a->o_strides[0]; p.o_sh = a->o_strides[1]; p.o_sr = a->o_strides[2];
    p.b_sb = a->bias_strides[0]; p.b_sh = a->bias_strides[1]; p.b_sr = a->bias_strides[2]; p.b_sc = a->bias_strides[3];
    p.B = a->B; p.H = a->H; p.M = a->M; p.N = a->N; p.S = a->num_splits;
    p.sm_scale = a->sm_scale;
    return finish(launch_splitk(p, a->dtype, a->D, (hipStream_t)stream), what);
}

int t5a_fwd_splitk(const t5a_splitk_args* a, t5a_stream_t stream) {
    if (a == nullptr) return fail(T5A_ERR_NULL, "args is NULL");
    return splitk_run(a, a->workspace, a->workspace_bytes, stream, "t5a_fwd_splitk");
}

// ---------------------------------------------------------------------------------------------------
// Split-K forward for callers that cannot allocate: the partial results live in a device array that is
// part of the library's image (every device the library runs on holds its own copy until the process ends).
// In host code the array's name is only a handle for hipGetSymbolAddress, never a device address: the
// address is looked up once per device, with that device current, and kept; kernels and every other use get
// that pointer.
static __device__ __align__(256) unsigned char scratch[T5A_STATIC_SCRATCH_BYTES];

static int static_scratch(void** out) {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static void* ptrs[kMaxDevices] = {};
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(T5A_ERR_LAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(T5A_ERR_LAUNCH, "device index %d out of range", dev);
    std::lock_guard<std::mutex> g(mu);
    if (ptrs[dev] == nullptr) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr)
            return fail(T5A_ERR_LAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
        ptrs[dev] = ptr;
    }
    *out = ptrs[dev];
    return T5A_OK;
}

int t5a_fwd_splitk_static(const t5a_splitk_args* a, t5a_stream_t stream) {
    if (a == nullptr) return fail(T5A_ERR_NULL, "args is NULL");
    const int64_t need = t5a_splitk_workspace_bytes(a->B, a->H, a->M, a->D, a->num_splits);
    if (need > (int64_t)T5A_STATIC_SCRATCH_BYTES)
        return fail(T5A_ERR_WORKSPACE, "t5a_fwd_splitk_static: B=%d H=%d M=%d D=%d num_splits=%d need %lld bytes of partial "
                    "results, the static scratch array holds %lld; use fewer splits or t5a_fwd_splitk with a workspace",
                    a->B, a->H, a->M, a->D, a->num_splits, (long long)need, (long long)T5A_STATIC_SCRATCH_BYTES);
    void* ptr = nullptr;
    int rc = static_scratch(&ptr);
    if (rc) return rc;
    // nothing has to be cleared: the split kernel writes every partial row that the merge of the same call reads
    return splitk_run(a, ptr, (int64_t)T5A_STATIC_SCRATCH_BYTES, stream, "t5a_fwd_splitk_static");
}

int t5a_rmsnorm(const t5a_rmsnorm_args* a, t5a_stream_t stream) {
    if (a == nullptr) return fail(T5A_ERR_NULL, "args is NULL");
    for (int dt : {a->x_dtype, a->weight_dtype})
        if (dt != T5A_BF16 && dt != T5A_F16 && dt != T5A_F32) return fail(T5A_ERR_DTYPE, "unsupported dtype %d", dt);
    if (a->batches < 0 || a->rows_per_batch < 0 || a->dim <= 0 || a->group < 1)
        return fail(T5A_ERR_SHAPE, "bad sizes batches=%lld rows=%d dim=%d group=%d", (long long)a->batches, a->rows_per_batch, a->dim, a->group);
    if (a->dim % 8 != 0) return fail(T5A_ERR_SHAPE, "dim=%d must be a multiple of 8", a->dim);
    const int out_per_batch = a->rows_per_batch / a->group;
    if (a->batches == 0 || out_per_batch == 0) return T5A_OK;
    if (a->x == nullptr || a->weight == nullptr || a->y == nullptr) return fail(T5A_ERR_NULL, "x, weight or y is NULL");
    if (!aligned16(a->x) || (reinterpret_cast<uintptr_t>(a->y) & 31u) != 0) return fail(T5A_ERR_STRIDE, "x must be 16-byte and y 32-byte aligned");
    const int xunit = a->x_dtype == T5A_F32 ? 4 : 8;
    if (a->x_strides[0] % xunit != 0 || a->x_strides[1] % xunit != 0)
        return fail(T5A_ERR_STRIDE, "x strides must be multiples of %d elements", xunit);
    if (a->residual != nullptr) {
        if (a->group != 1) return fail(T5A_ERR_SHAPE, "a residual needs group == 1 (got %d)", a->group);
        if (a->sum_out == nullptr) return fail(T5A_ERR_NULL, "residual given but sum_out is NULL");
        if (!aligned16(a->residual) || !aligned16(a->sum_out) || a->residual_row_stride % xunit != 0 || a->residual_row_stride < 0)
            return fail(T5A_ERR_STRIDE, "residual and sum_out must be 16-byte aligned, the residual row stride a multiple of %d elements", xunit);
        if (a->sum_out == a->x || a->sum_out == a->residual) return fail(T5A_ERR_STRIDE, "sum_out must not overlap x or residual");
    }
    RmsParams p;
    memset(&p, 0, sizeof(p));
    p.x = a->x; p.weight = a->weight; p.y = a->y;
    p.residual = a->residual; p.sum_out = a->residual ? a->sum_out : nullptr; p.residual_row_stride = a->residual_row_stride;
    if (a->seq_lens != nullptr) {
        if (a->residual != nullptr) return fail(T5A_ERR_SHAPE, "seq_lens and residual cannot be combined");
        p.lens = a->seq_lens;
        p.starts = a->seq_starts;
    } else if (a->seq_starts != nullptr) {
        return fail(T5A_ERR_SHAPE, "seq_starts needs seq_lens");
    }
    if (a->key_bits != nullptr) {
        if (a->group <= 1 || a->seq_lens != nullptr || a->residual != nullptr)
            return fail(T5A_ERR_SHAPE, "key_bits is for group > 1, without seq_lens or residual");
        if (a->group_counts == nullptr) return fail(T5A_ERR_NULL, "key_bits needs group_counts");
        const int64_t need = kKeyBitsFront + ((int64_t)a->rows_per_batch + 31) / 32;   // (only the rows' own bits are read)
        if (a->key_bits_stride < need)
            return fail(T5A_ERR_SHAPE, "key_bits_stride %lld, the rows need %lld words", (long long)a->key_bits_stride, (long long)need);
        if ((reinterpret_cast<uintptr_t>(a->key_bits) & 3) != 0) return fail(T5A_ERR_STRIDE, "key_bits must be 4-byte aligned");
        p.key_bits = a->key_bits; p.key_bits_stride = a->key_bits_stride; p.group_counts = a->group_counts;
    }
    p.x_batch_stride = a->x_strides[0]; p.x_row_stride = a->x_strides[1]; p.y_row_stride = a->dim;
    p.out_per_batch = out_per_batch;
    p.out_rows = a->batches * out_per_batch;
    p.rows_per_batch = a->rows_per_batch; p.group = a->group; p.dim = a->dim;
    p.eps = a->eps;
    if ((p.out_rows + 3) / 4 > 0x7fffffffLL) return fail(T5A_ERR_SHAPE, "too many rows (%lld)", (long long)p.out_rows);
    return finish(launch_rmsnorm(p, a->x_dtype, a->weight_dtype, (hipStream_t)stream), "t5a_rmsnorm");
}

}  // extern "C"
