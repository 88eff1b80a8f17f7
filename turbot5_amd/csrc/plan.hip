// Launch plan of a packed (variable-length) batch, built on the device from cu_seqlens.
//
// The attention kernel's workgroup ids go round-robin over the 8 XCDs, so workgroup (8 k + x) is the
// k-th one XCD x starts.  Sequences of different lengths make items of different cost; a plain cut of
// the item list into 8 equal COUNTS leaves the XCDs with unequal work (27 % over the mean for 32
// lengths drawn from 128..4096) and starts long items late.  The plan gives every XCD a slice of equal
// WORK of the (sequence, head, tile) list -- contiguous, so that the q tiles of one (sequence, head)
// mostly share an L2 -- ordered longest item first, and the kernel reads its item from plan[x][k]
// instead of walking cu_seqlens.
//
// One workgroup builds it:
//   1. per sequence: tile count, work; prefix sums over the sequences;
//   2. eight threads turn the work targets x * total / 8 into slice boundaries, as item indices;
//   3. a counting sort by (XCD, cost) in LDS.  The unit of work is a (sequence, tile) pair: its items,
//      one per head, have the same cost and sit nt apart in the (head-major) list, so the heads that
//      fall into an XCD's slice are a range found by division, and a pair costs one counter update
//      per XCD it touches;
//   4. the pairs place their items, a run of consecutive slots per (pair, XCD) -- into an LDS image of
//      the lists (one packed word per slot) when that fits, from which all threads then write the
//      entries with neighbouring lanes on neighbouring addresses.  Entries written straight from the
//      pairs are 32-byte pieces scattered over the lists, one memory request each, and that request
//      stream was most of the kernel's time.
// Cost of an item = its key tiles plus a constant for set-up and write-back.  The lists are data
// dependent but their size is not: `slots` entries per XCD are reserved (twice the mean); a slice that
// outgrows its slots spills into the free slots of the others.  counts[x] tells the attention kernel
// how many entries of list x are in use.
#include <hip/hip_runtime.h>

#include <atomic>

#include "t5a_internal.h"

namespace t5a {

namespace {

constexpr int PLAN_THREADS = 1024;
constexpr int BINS = 512;        // cost classes of the counting sort
constexpr int ITEM_COST0 = 5;    // set-up + write-back of an item, in tile steps

// key tiles of q tile qt (queries sit at the END of the keys when causal: position i + lenk - lenq)
__device__ __forceinline__ int item_cost(const PlanParams& p, int lenq, int lenk, int qt) {
    int keys = lenk;
    if (p.causal) keys = min(lenk, max(0, (qt + 1) * 128 + lenk - lenq));
    return ((keys + (1 << p.bn_shift) - 1) >> p.bn_shift) + ITEM_COST0;
}

template <typename V>
__device__ __forceinline__ V wave_incl_scan(V v, int lane) {
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const V u = __shfl_up(v, d, 64);
        if (lane >= d) v += u;
    }
    return v;
}

__device__ __forceinline__ int ceil_div_clamped(int a, int b, int hi) {   // clamp(ceil(a / b), 0, hi), b > 0
    if (a <= 0) return 0;
    return min(hi, (a + b - 1) / b);
}

__global__ __launch_bounds__(PLAN_THREADS) void varlen_plan_kernel(const PlanParams p) {
    __shared__ int s_nt[kPlanMaxSeqs], s_lenq[kPlanMaxSeqs], s_lenk[kPlanMaxSeqs], s_qs[kPlanMaxSeqs], s_ks[kPlanMaxSeqs];
    __shared__ float s_group[kPlanMaxSeqs];        // work of one (sequence, head) group
    __shared__ int s_tiles[kPlanMaxSeqs + 1];      // exclusive prefix of nt; the item prefix is H times it
    __shared__ float s_work[kPlanMaxSeqs + 1];     // exclusive prefix of the sequences' work
    __shared__ int s_hist[8][BINS];
    __shared__ int s_lo[9];                        // XCD x owns the items [s_lo[x], s_lo[x + 1]) of the list
    __shared__ int s_nx[8], s_free[9], s_nover;
    extern __shared__ int s_stage[];               // [8][slots] packed items (p.staged), else unused
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    // ---- 1. per-sequence figures
    int wide = 0;   // a tile index that the packed LDS image cannot hold
    for (int b = tid; b < p.B; b += PLAN_THREADS) {
        const int qs = p.cu_q[b], ks = p.cu_k[b];
        const int lenq = max(0, p.len_q != nullptr ? p.len_q[b] : p.cu_q[b + 1] - qs);
        const int lenk = max(0, p.len_k != nullptr ? p.len_k[b] : p.cu_k[b + 1] - ks);
        const int nt = (lenq + 127) >> 7;
        wide |= nt > (1 << 14);
        s_nt[b] = nt; s_lenq[b] = lenq; s_lenk[b] = lenk; s_qs[b] = qs; s_ks[b] = ks;
        float g = 0.f;
        if (p.causal) { for (int qt = 0; qt < nt; ++qt) g += (float)item_cost(p, lenq, lenk, qt); }
        else g = (float)nt * (float)item_cost(p, lenq, lenk, 0);
        s_group[b] = g;
    }
    for (int i = tid; i < 8 * BINS; i += PLAN_THREADS) (&s_hist[0][0])[i] = 0;
    if (tid == 0) s_nover = 0;
    const bool staged = p.staged != 0 && __syncthreads_or(wide) == 0;
    // prefix sums over the sequences: wavefront 0, a contiguous chunk per lane
    if (wave == 0) {
        const int per = (p.B + 63) / 64;
        const int b0 = min(lane * per, p.B), b1 = min(b0 + per, p.B);
        int nu = 0; float wk = 0.f;
        for (int b = b0; b < b1; ++b) { nu += s_nt[b]; wk += s_group[b] * p.H; }
        int eu = wave_incl_scan(nu, lane) - nu;
        float ew = wave_incl_scan(wk, lane) - wk;
        for (int b = b0; b < b1; ++b) {
            s_tiles[b] = eu; s_work[b] = ew;
            eu += s_nt[b]; ew += s_group[b] * p.H;
        }
        if (lane == 63) { s_tiles[p.B] = eu; s_work[p.B] = ew; }   // lane 63 owns the last chunk (or an empty one after it)
    }
    __syncthreads();
    const int n_pairs = s_tiles[p.B];
    const int n_items = n_pairs * p.H;

    // ---- 2. slice boundaries: the item at which the work in front reaches x * total / 8.  Any
    // non-decreasing boundaries give a valid plan; float rounding only moves them by an item or two.
    if (tid <= 8) {
        int at = tid == 8 ? n_items : 0;
        if (tid > 0 && tid < 8 && n_items > 0) {
            const float target = s_work[p.B] * (float)tid * 0.125f;
            int lo = 0, hi = p.B;            // last b with s_work[b] <= target
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (s_work[mid] <= target) lo = mid; else hi = mid;
            }
            const int b = lo, nt = s_nt[b];
            at = s_tiles[b] * p.H;
            if (nt > 0 && s_group[b] > 0.f) {
                float rem = target - s_work[b];
                const int h = min(p.H - 1, (int)(rem / s_group[b]));
                rem -= (float)h * s_group[b];
                // tiles of group h in front of the boundary, in the group's order
                float fr;
                if (p.causal) {
                    // cost of rank r is about a (nt - r) + c: solve a/2 r^2 - (a nt + a/2 + c) r + rem = 0
                    const float a = 128.0f / (float)(1 << p.bn_shift);
                    const float c = (float)(s_lenk[b] - s_lenq[b]) / (float)(1 << p.bn_shift) + ITEM_COST0;
                    const float bq = a * (float)nt + 0.5f * a + c;
                    fr = (bq - sqrtf(fmaxf(bq * bq - 2.0f * a * rem, 0.f))) / a;
                } else {
                    fr = rem / (float)item_cost(p, s_lenq[b], s_lenk[b], 0);
                }
                const int r = min(nt, max(0, (int)(fr + 0.5f)));
                at += h * nt + r;
            }
        }
        s_lo[tid] = at;
    }
    __syncthreads();
    if (tid == 0) {   // non-decreasing, whatever the rounding did
        for (int x = 1; x < 8; ++x) s_lo[x] = min(n_items, max(s_lo[x], s_lo[x - 1]));
    }
    __syncthreads();

    // Walks the (sequence, tile) pairs.  The item of head h sits at list index first + h * nt with
    // first = H * s_tiles[b] + r, so the heads inside XCD x's slice are
    // [ceil((lo[x] - first) / nt), ceil((lo[x + 1] - first) / nt)).  f(b, qt, x, bin, h0, h1) is called
    // for every non-empty range.
    auto for_pairs = [&](auto&& f) {
        for (int pr = tid; pr < n_pairs; pr += PLAN_THREADS) {
            int lo = 0, hi = p.B;            // last b with s_tiles[b] <= pr
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (s_tiles[mid] <= pr) lo = mid; else hi = mid;
            }
            const int b = lo, nt = s_nt[b], r = pr - s_tiles[b];
            const int qt = p.causal ? nt - 1 - r : r;     // longest tile first inside a causal group
            const int key = min(BINS - 1, item_cost(p, s_lenq[b], s_lenk[b], qt) >> p.key_shift);
            const int first = s_tiles[b] * p.H + r;
            int h0 = ceil_div_clamped(s_lo[0] - first, nt, p.H);
            for (int x = 0; x < 8 && h0 < p.H; ++x) {
                const int h1 = ceil_div_clamped(s_lo[x + 1] - first, nt, p.H);
                if (h1 > h0) f(b, qt, x, x * BINS + key, h0, h1);
                h0 = h1;
            }
        }
    };

    // ---- 3. histogram of (XCD, cost class), then per XCD the offsets in DESCENDING cost order
    for_pairs([&](int, int, int, int bin, int h0, int h1) { atomicAdd(&(&s_hist[0][0])[bin], h1 - h0); });
    __syncthreads();
    if (wave < 8) {   // wavefront x handles XCD x, 8 classes per lane
        constexpr int PER = BINS / 64;
        int sum = 0;
#pragma unroll
        for (int c = 0; c < PER; ++c) sum += s_hist[wave][BINS - 1 - (lane * PER + c)];
        int off = wave_incl_scan(sum, lane) - sum;
#pragma unroll
        for (int c = 0; c < PER; ++c) {
            const int k = BINS - 1 - (lane * PER + c);
            const int n = s_hist[wave][k];
            s_hist[wave][k] = off;
            off += n;
        }
        if (lane == 63) s_nx[wave] = off;
    }
    __syncthreads();
    if (tid == 0) {
        int f = 0;
        for (int x = 0; x < 8; ++x) { s_free[x] = f; f += max(0, p.slots - s_nx[x]); }
        s_free[8] = f;
    }

    // ---- 4. entries
    auto write_entry = [&](int x, int k, int b, int h, int qt) {
        int4* e = reinterpret_cast<int4*>(p.plan) + ((x * p.slots + k) << 1);
        e[0] = int4{b, h, qt, s_lenq[b]};
        e[1] = int4{s_lenk[b], s_qs[b], s_ks[b], 0};
    };
    // packed item of the LDS image: sequence (10 bits), head (8), tile (14); the host stages only when they fit
    auto pack = [](int b, int h, int qt) { return b | (h << 10) | (qt << 18); };
    for_pairs([&](int b, int qt, int x, int bin, int h0, int h1) {
        const int k0 = atomicAdd(&(&s_hist[0][0])[bin], h1 - h0);
        for (int h = h0; h < h1; ++h) {
            const int k = k0 + (h - h0);
            if (k >= p.slots) reinterpret_cast<int4*>(p.spill)[atomicAdd(&s_nover, 1)] = int4{b, h, qt, 0};
            else if (staged) s_stage[x * p.slots + k] = pack(b, h, qt);
            else write_entry(x, k, b, h, qt);
        }
    });
    __threadfence_block();
    __syncthreads();
    const int n_over = s_nover;
    if (staged) {
        // spilled items join the image, then lane pairs write the two halves of consecutive entries
        for (int j = tid; j < n_over; j += PLAN_THREADS) {
            int x = 0;
            while (x < 7 && s_free[x + 1] <= j) ++x;
            const int4 it = reinterpret_cast<const int4*>(p.spill)[j];
            s_stage[x * p.slots + s_nx[x] + (j - s_free[x])] = pack(it.x, it.y, it.z);
        }
        __syncthreads();
        {   // two wavefronts per XCD list, so that all lists are written at the same time
            const int x = wave >> 1;
            const int room = max(0, p.slots - s_nx[x]);
            const int used = min(s_nx[x], p.slots) + min(room, max(0, n_over - s_free[x]));
            int4* list = reinterpret_cast<int4*>(p.plan) + ((x * p.slots) << 1);
#pragma unroll 4
            for (int i = (wave & 1) * 64 + lane; i < 2 * used; i += 128) {
                const int w = s_stage[x * p.slots + (i >> 1)];
                const int b = w & 1023;
                list[i] = (i & 1) ? int4{s_lenk[b], s_qs[b], s_ks[b], 0}
                                  : int4{b, (w >> 10) & 255, (int)((unsigned)w >> 18), s_lenq[b]};
            }
        }
    } else {
        // spilled items go to the free slots, XCD by XCD
        for (int j = tid; j < n_over; j += PLAN_THREADS) {
            int x = 0;
            while (x < 7 && s_free[x + 1] <= j) ++x;
            const int4 it = reinterpret_cast<const int4*>(p.spill)[j];
            write_entry(x, s_nx[x] + (j - s_free[x]), it.x, it.y, it.z);
        }
    }
    if (tid < 8) {
        const int room = max(0, p.slots - s_nx[tid]);
        p.counts[tid] = min(s_nx[tid], p.slots) + min(room, max(0, n_over - s_free[tid]));
    }
}

}  // namespace

// LDS image of the lists: 4 bytes per slot next to the 48 KB of fixed arrays, within the 160 KB of a CU
bool plan_can_stage(int slots, int H, int max_seqlen_q) {
    return (int64_t)8 * slots * 4 <= 100 * 1024 && H <= 256 && (max_seqlen_q + 127) / 128 <= (1 << 14);
}

hipError_t launch_varlen_plan(const PlanParams& p, hipStream_t stream) {
    const size_t dyn = p.staged ? (size_t)8 * p.slots * sizeof(int) : 0;
    // per device: largest dynamic LDS size already allowed (the attribute belongs to the function as loaded on one device)
    constexpr int kMaxDevices = 64;
    static std::atomic<size_t> granted[kMaxDevices] = {};
    if (dyn > 0) {   // static + dynamic LDS beyond 64 KB must be allowed first
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return e;
        const bool known = dev >= 0 && dev < kMaxDevices;
        if (!known || dyn > granted[dev].load(std::memory_order_relaxed)) {
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(varlen_plan_kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn);
            if (e != hipSuccess) return e;
            if (known) granted[dev].store(dyn, std::memory_order_relaxed);
        }
    }
    hipLaunchKernelGGL(varlen_plan_kernel, dim3(1), dim3(PLAN_THREADS), dyn, stream, p);
    return hipGetLastError();
}

}  // namespace t5a
