// Issue costs of the instructions that make up the attention kernel's tile loop, measured on the device this runs
// on: cycles per instruction and wavefront with one and with two workgroups of 256 threads per compute unit (one and
// two wavefronts per SIMD), and LDS read throughput per compute unit.  A measurement tool, not part of the library:
//
//     python -m turbot5_amd.build --measure      # writes turbot5_amd/csrc/measure/issue_costs
//     turbot5_amd/csrc/measure/issue_costs
//
// Every kernel runs a bounded loop of unrolled blocks of 16 instructions from inline assembly (scalar clobbers are
// declared, the loop counter is the compiler's own).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <vector>

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

#define MFMA(acc) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb, acc, 0, 0, 0)

enum Kind {
    kExp, kAdd, kMax3, kCvt, kDot2, kMov, kSalu, kMfma4Acc, kMfma2Chains, kMfmaExpCvt, kMfma7Max3, kMfma5Max3,
    kMfma4Max3Salu, kMax3Salu, kMfmaRaw, kDotChains, kKinds
};

template <int KIND>
__global__ __launch_bounds__(256) void issue_kernel(float* out, unsigned long long* cyc, int iters) {
    float a[16];
    for (int i = 0; i < 16; ++i) a[i] = threadIdx.x * 0.001f + i;
    f32x16 acc0 = {0}, acc1 = {0}, acc2 = {0}, acc3 = {0};
    bf16x8 fa, fb;
    for (int i = 0; i < 8; ++i) { fa[i] = (__bf16)(float)(threadIdx.x + i); fb[i] = (__bf16)(float)i; }
    const unsigned xa = threadIdx.x, ones = 0x3f803f80u;
    __syncthreads();
    const unsigned long long t0 = __builtin_readcyclecounter();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {   // 16 blocks of 16 instructions
            if (KIND == kExp) {
#pragma unroll
                for (int i = 0; i < 16; ++i) asm volatile("v_exp_f32 %0, %0" : "+v"(a[i]));
            } else if (KIND == kAdd) {
#pragma unroll
                for (int i = 0; i < 16; ++i) asm volatile("v_add_f32 %0, %0, %0" : "+v"(a[i]));
            } else if (KIND == kMax3) {
#pragma unroll
                for (int i = 0; i < 16; ++i) asm volatile("v_maximum3_f32 %0, %0, %0, %0" : "+v"(a[i]));
            } else if (KIND == kCvt) {
#pragma unroll
                for (int i = 0; i < 16; ++i) asm volatile("v_cvt_pk_bf16_f32 %0, %0, %0" : "+v"(a[i]));
            } else if (KIND == kDot2) {
#pragma unroll
                for (int i = 0; i < 16; ++i) asm volatile("v_dot2c_f32_bf16 %0, %1, %2" : "+v"(a[i]) : "v"(ones), "v"(xa));
            } else if (KIND == kMov) {
#pragma unroll
                for (int i = 0; i < 16; ++i) asm volatile("v_mov_b32 %0, %1" : "=v"(a[i]) : "v"(xa));
            } else if (KIND == kSalu) {   // dependent scalar instructions
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    asm volatile("s_add_u32 s20, s20, s21\n s_xor_b32 s22, s22, s20\n s_and_b32 s23, s22, s20\n s_add_u32 s21, s23, s21"
                                 ::: "s20", "s21", "s22", "s23", "scc");
            } else if (KIND == kMfma4Acc) {
#pragma unroll
                for (int i = 0; i < 4; ++i) { MFMA(acc0); MFMA(acc1); MFMA(acc2); MFMA(acc3); }
            } else if (KIND == kMfma2Chains) {   // the kernel's pattern: two accumulators in turn
#pragma unroll
                for (int i = 0; i < 8; ++i) { MFMA(acc0); MFMA(acc1); }
            } else if (KIND == kMfmaExpCvt) {    // first half of a step: 1 MFMA, 4 exp, 2 cvt (+ 1 mov to make 8)
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    if (i == 0) MFMA(acc0); else MFMA(acc1);
#pragma unroll
                    for (int j = 0; j < 4; ++j) asm volatile("v_exp_f32 %0, %0" : "+v"(a[6 * i + j]));
                    asm volatile("v_cvt_pk_bf16_f32 %0, %0, %0" : "+v"(a[6 * i + 4]));
                    asm volatile("v_cvt_pk_bf16_f32 %0, %0, %0" : "+v"(a[6 * i + 5]));
                    asm volatile("v_mov_b32 %0, %0" : "+v"(a[12 + i]));
                }
            } else if (KIND == kMfma7Max3) {
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    if (i == 0) MFMA(acc0); else MFMA(acc1);
#pragma unroll
                    for (int j = 0; j < 7; ++j) asm volatile("v_maximum3_f32 %0, %0, %0, %0" : "+v"(a[7 * i + j]));
                }
            } else if (KIND == kMfma5Max3) {     // (two s_nop to make 8)
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    if (i == 0) MFMA(acc0); else MFMA(acc1);
#pragma unroll
                    for (int j = 0; j < 5; ++j) asm volatile("v_maximum3_f32 %0, %0, %0, %0" : "+v"(a[7 * i + j]));
                    asm volatile("s_nop 0\n s_nop 0");
                }
            } else if (KIND == kMfma4Max3Salu) { // 1 MFMA, 4 max3, 3 scalar
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    if (i == 0) MFMA(acc0); else MFMA(acc1);
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        asm volatile("v_maximum3_f32 %0, %0, %0, %0" : "+v"(a[7 * i + j]));
                        if (j < 3) asm volatile("s_add_u32 s20, s20, s21" ::: "s20", "scc");
                    }
                }
            } else if (KIND == kMax3Salu) {      // 4 max3, 12 scalar
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    asm volatile("v_maximum3_f32 %0, %0, %0, %0" : "+v"(a[j]));
                    asm volatile("s_add_u32 s20, s20, s21\n s_xor_b32 s22, s22, s20\n s_and_b32 s23, s22, s20" ::: "s20", "s22", "s23", "scc");
                }
            } else if (KIND == kMfmaRaw) {       // a vector instruction that reads the MFMA's result, 4 x (1 + 3)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    MFMA(acc0);
                    const float t = acc0[0];
                    asm volatile("v_add_f32 %0, %0, %1" : "+v"(a[i]) : "v"(t));
                    asm volatile("v_add_f32 %0, %0, %0" : "+v"(a[4 + i]));
                    asm volatile("v_add_f32 %0, %0, %0" : "+v"(a[8 + i]));
                }
            } else if (KIND == kDotChains) {     // the row sums: two dependent chains
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    asm volatile("v_dot2c_f32_bf16 %0, %1, %2" : "+v"(a[0]) : "v"(ones), "v"(xa));
                    asm volatile("v_dot2c_f32_bf16 %0, %1, %2" : "+v"(a[1]) : "v"(ones), "v"(xa));
                }
            }
        }
    }
    const unsigned long long t1 = __builtin_readcyclecounter();
    float s = 0;
    for (int i = 0; i < 16; ++i) s += a[i] + acc0[i] + acc1[i] + acc2[i] + acc3[i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
    if (threadIdx.x == 0) cyc[blockIdx.x] = t1 - t0;
}

#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); exit(1); } } while (0)

static int g_cus = 0;

template <int KIND>
static void run_issue(const char* name) {
    printf("%-44s", name);
    for (int wg = 1; wg <= 2; ++wg) {
        const int iters = 200, blocks = g_cus * wg;
        float* out; unsigned long long* cyc;
        CHECK(hipMalloc(&out, (size_t)blocks * 256 * 4)); CHECK(hipMalloc(&cyc, (size_t)blocks * 8));
        for (int w = 0; w < 3; ++w) issue_kernel<KIND><<<blocks, 256>>>(out, cyc, iters);
        CHECK(hipDeviceSynchronize());
        std::vector<unsigned long long> h(blocks);
        CHECK(hipMemcpy(h.data(), cyc, (size_t)blocks * 8, hipMemcpyDeviceToHost));
        std::sort(h.begin(), h.end());
        printf("  %7.2f", (double)h[blocks / 2] / ((double)iters * 256));
        CHECK(hipFree(out)); CHECK(hipFree(cyc));
    }
    printf("\n");
}

// LDS reads: 0 linear ds_read_b128, 1 ds_read_b64_tr_b16, 2 ds_read_b64
template <int KIND>
__global__ __launch_bounds__(256) void lds_kernel(float* out, unsigned long long* cyc, int iters) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    for (int i = threadIdx.x; i < 16384; i += 256) reinterpret_cast<float*>(smem)[i] = (float)i;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;
    const unsigned a16 = base + wave * 4096 + lane * 16, a8 = base + wave * 4096 + lane * 8;
    f32x4 acc = {0, 0, 0, 0};
    const unsigned long long t0 = __builtin_readcyclecounter();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            if (KIND == 0) {
                f32x4 v;
                asm volatile("ds_read_b128 %0, %1\n s_waitcnt lgkmcnt(8)" : "=v"(v) : "v"(a16));
                acc += v;
            } else {
                f32x2 v;
                if (KIND == 1) asm volatile("ds_read_b64_tr_b16 %0, %1\n s_waitcnt lgkmcnt(8)" : "=v"(v) : "v"(a8));
                else asm volatile("ds_read_b64 %0, %1\n s_waitcnt lgkmcnt(8)" : "=v"(v) : "v"(a8));
                acc[0] += v[0]; acc[1] += v[1];
            }
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)");
    const unsigned long long t1 = __builtin_readcyclecounter();
    out[blockIdx.x * 256 + threadIdx.x] = acc[0] + acc[1] + acc[2] + acc[3];
    if (threadIdx.x == 0) cyc[blockIdx.x] = t1 - t0;
}

template <int KIND>
static void run_lds(const char* name, int bytes_per_lane) {
    CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(lds_kernel<KIND>), hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
    printf("%-44s", name);
    for (int wg = 1; wg <= 2; ++wg) {
        const int iters = 2000, blocks = g_cus * wg;
        float* out; unsigned long long* cyc;
        CHECK(hipMalloc(&out, (size_t)blocks * 256 * 4)); CHECK(hipMalloc(&cyc, (size_t)blocks * 8));
        for (int w = 0; w < 3; ++w) lds_kernel<KIND><<<blocks, 256, 65536>>>(out, cyc, iters);
        CHECK(hipDeviceSynchronize());
        std::vector<unsigned long long> h(blocks);
        CHECK(hipMemcpy(h.data(), cyc, (size_t)blocks * 8, hipMemcpyDeviceToHost));
        std::sort(h.begin(), h.end());
        const double cycles = (double)h[blocks / 2], instr = (double)iters * 16 * 4 * wg;   // wavefront instructions per CU
        printf("  %7.2f (%5.1f B/clk)", cycles / instr, instr * 64 * bytes_per_lane / cycles);
        CHECK(hipFree(out)); CHECK(hipFree(cyc));
    }
    printf("\n");
}

int main() {
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    g_cus = prop.multiProcessorCount;
    printf("%s, %d compute units\n", prop.gcnArchName, g_cus);
    printf("shader-clock cycles per instruction and wavefront; columns: one / two workgroups of 256 threads per CU\n\n");
    run_issue<kExp>("v_exp_f32");
    run_issue<kAdd>("v_add_f32");
    run_issue<kMax3>("v_maximum3_f32");
    run_issue<kCvt>("v_cvt_pk_bf16_f32");
    run_issue<kDot2>("v_dot2c_f32_bf16");
    run_issue<kDotChains>("v_dot2c_f32_bf16, two dependent chains");
    run_issue<kMov>("v_mov_b32");
    run_issue<kSalu>("scalar ALU (dependent)");
    run_issue<kMfma4Acc>("v_mfma_f32_32x32x16_bf16, 4 accumulators");
    run_issue<kMfma2Chains>("v_mfma_f32_32x32x16_bf16, 2 accumulators");
    run_issue<kMfmaExpCvt>("1 mfma + 4 exp + 2 cvt + 1 mov (per instr.)");
    run_issue<kMfma7Max3>("1 mfma + 7 max3 (per instr.)");
    run_issue<kMfma5Max3>("1 mfma + 5 max3 + 2 s_nop (per instr.)");
    run_issue<kMfma4Max3Salu>("1 mfma + 4 max3 + 3 scalar (per instr.)");
    run_issue<kMax3Salu>("4 max3 + 12 scalar (per instr.)");
    run_issue<kMfmaRaw>("1 mfma + 1 add reading it + 2 add (per instr.)");
    printf("\nLDS reads, conflict-free addresses: cycles per wavefront instruction and CU (bytes per clock and CU)\n\n");
    run_lds<0>("ds_read_b128", 16);
    run_lds<1>("ds_read_b64_tr_b16", 8);
    run_lds<2>("ds_read_b64", 8);
    return 0;
}
