// Measures the fp32 vector issue rate of the GPU with the instruction mixes of the adder kernels.
//
// A CDNA SIMD starts at most one vector instruction per wave every four cycles, but it can start
// two in the same four cycles when they come from two different waves.  The ceiling of a
// VALU-bound kernel is therefore 2 x CUs x 64 lanes x clock lane-instructions per second, and it
// is only reachable with at least two waves per SIMD that are both ready to issue.  This program
// prints what a pure instruction stream reaches with one, two and four waves per SIMD:
//   fwd   pair    v_sub d, s_w, v_x ; v_sub acc, acc, |d|                   (forward)
//   gradx pair    v_fma d, s_w, 0.5, v_c clamp ; v_fmac acc, d, g          (input gradient)
//   sgpr  only    v_sub acc, s_w, acc    (every instruction reads a scalar register: one per slot)
//   vgpr  pair    the gradx pair with the weight in a vector register (no scalar operand at all)
// Output: one line per case, "<name> <waves per SIMD> <lane-instructions per second>".
//
// A second table is about the fp64 matrix instruction of the weight-gradient kernel,
// v_mfma_f64_16x16x4_f64 (2048 flop): a bare stream of nine independent accumulators, the same
// with one v_cvt_f64_f32 + one fp32 add per MFMA, and with four fp32 FMAs per MFMA.  If vector
// instructions ran beside the matrix pipe the last two would cost nothing.
// Output: "<name> <waves per SIMD> <fp64 flop per second> <cycles per MFMA per SIMD at the reported clock>".
#include <hip/hip_runtime.h>
#include <cstdio>

#define CHECK(e)                                                                          \
    do {                                                                                  \
        hipError_t err_ = (e);                                                            \
        if (err_ != hipSuccess) {                                                         \
            std::fprintf(stderr, "%s: %s\n", #e, hipGetErrorString(err_));                \
            return 1;                                                                     \
        }                                                                                 \
    } while (0)

constexpr int kChains = 16, kRepeat = 8;

template <int MODE>
__global__ __launch_bounds__(1024) void issue_kernel(float *out, int iters, float w) {
    float acc[kChains], tmp[kChains];
    const float x = threadIdx.x * 0.5f, g = threadIdx.x * 0.25f, wv = w + threadIdx.x * 0.125f;
#pragma unroll
    for (int i = 0; i < kChains; ++i) { acc[i] = threadIdx.x * 0.001f + i; tmp[i] = 0.f; }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < kRepeat; ++r)
#pragma unroll
            for (int i = 0; i < kChains; ++i) {
                if (MODE == 0)
                    asm volatile("v_sub_f32_e32 %1, %2, %3\n v_sub_f32_e64 %0, %0, |%1|"
                                 : "+v"(acc[i]), "+v"(tmp[i]) : "s"(w), "v"(x));
                else if (MODE == 1)
                    asm volatile("v_fma_f32 %1, %2, 0.5, %3 clamp\n v_fmac_f32_e32 %0, %1, %4"
                                 : "+v"(acc[i]), "+v"(tmp[i]) : "s"(w), "v"(x), "v"(g));
                else if (MODE == 3)
                    asm volatile("v_fma_f32 %1, %2, 0.5, %3 clamp\n v_fmac_f32_e32 %0, %1, %4"
                                 : "+v"(acc[i]), "+v"(tmp[i]) : "v"(wv), "v"(x), "v"(g));
                else
                    asm volatile("v_sub_f32_e32 %0, %1, %0\n v_sub_f32_e32 %0, %1, %0" : "+v"(acc[i]) : "s"(w));
            }
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < kChains; ++i) s += acc[i] + tmp[i];
    if (s == 12345.678f) out[0] = s;   // keeps the arithmetic alive; never true in practice
}

typedef double double4v __attribute__((ext_vector_type(4)));
constexpr int kAccs = 9;

// MODE 0: MFMAs only; 1: + v_cvt_f64_f32 and v_add_f32 per MFMA; 2: + four dependent v_fma_f32 per MFMA
template <int MODE>
__global__ __launch_bounds__(512) void mfma64_kernel(float *out, const float *in, int iters) {
    double4v acc[kAccs];
    float f[kAccs];
    const double a = in[threadIdx.x & 63], b = in[64 + (threadIdx.x & 63)];
    const float g = in[threadIdx.x & 31];
#pragma unroll
    for (int i = 0; i < kAccs; ++i) { acc[i] = double4v{0.0, 0.0, 0.0, 0.0}; f[i] = in[i + (threadIdx.x & 15)]; }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < kAccs; ++i) {
            double bb = b;
            if (MODE == 1) { bb = (double)f[i]; f[i] += 1.0f; }
            if (MODE == 2) {
#pragma unroll
                for (int r = 0; r < 4; ++r) f[i] = fmaf(f[i], g, 1.0f);
            }
            acc[i] = __builtin_amdgcn_mfma_f64_16x16x4f64(a, bb, acc[i], 0, 0, 0);
        }
    }
    double s = 0.0;
#pragma unroll
    for (int i = 0; i < kAccs; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3] + f[i];
    if (s == 12345.678) out[0] = (float)s;
}

template <int MODE>
static int run_mfma64(const char *name, float *out, const float *in, int cus, int clock_khz) {
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    for (int waves : {1, 2, 4}) {       // per SIMD: one workgroup of 4 or 8 waves per CU, or two of 8
        const int wg = waves == 1 ? 256 : 512, groups = cus * (waves == 4 ? 2 : 1), iters = 2000;
        hipLaunchKernelGGL(mfma64_kernel<MODE>, dim3(groups), dim3(wg), 0, 0, out, in, 10);
        CHECK(hipDeviceSynchronize());
        CHECK(hipEventRecord(e0));
        hipLaunchKernelGGL(mfma64_kernel<MODE>, dim3(groups), dim3(wg), 0, 0, out, in, iters);
        CHECK(hipEventRecord(e1));
        CHECK(hipEventSynchronize(e1));
        float ms = 0.f;
        CHECK(hipEventElapsedTime(&ms, e0, e1));
        const double mfmas = (double)groups * (wg / 64) * iters * kAccs;
        std::printf("%s %d %.4e %.1f\n", name, waves, mfmas * 2048 / (ms * 1e-3),
                    ms * 1e-3 * clock_khz * 1e3 / (mfmas / (4.0 * cus)));
    }
    return 0;
}

template <int MODE>
static int run(const char *name, int per_group, float *out, int cus) {
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    for (int wg : {256, 512, 1024}) {   // one workgroup per CU: 1, 2, 4 waves per SIMD
        const int iters = 2000;
        hipLaunchKernelGGL(issue_kernel<MODE>, dim3(cus), dim3(wg), 0, 0, out, 10, 1.0001f);
        CHECK(hipDeviceSynchronize());
        CHECK(hipEventRecord(e0));
        hipLaunchKernelGGL(issue_kernel<MODE>, dim3(cus), dim3(wg), 0, 0, out, iters, 1.0001f);
        CHECK(hipEventRecord(e1));
        CHECK(hipEventSynchronize(e1));
        float ms = 0.f;
        CHECK(hipEventElapsedTime(&ms, e0, e1));
        const double inst = (double)cus * wg * iters * kRepeat * kChains * per_group;
        std::printf("%s %d %.4e\n", name, wg / 256, inst / (ms * 1e-3));
    }
    return 0;
}

int main() {
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;
    float *out = nullptr;
    CHECK(hipMalloc(&out, 4096));
    std::printf("device %s cus %d clock_mhz %d\n", prop.name, cus, prop.clockRate / 1000);
    if (run<0>("fwd_pair", 2, out, cus)) return 1;
    if (run<1>("gradx_pair", 2, out, cus)) return 1;
    if (run<2>("sgpr_only", 2, out, cus)) return 1;
    if (run<3>("vgpr_pair", 2, out, cus)) return 1;
    float *in = nullptr;
    CHECK(hipMalloc(&in, 4096));
    CHECK(hipMemset(in, 0, 4096));
    if (run_mfma64<0>("mfma64", out, in, cus, prop.clockRate)) return 1;
    if (run_mfma64<1>("mfma64_cvt_add", out, in, cus, prop.clockRate)) return 1;
    if (run_mfma64<2>("mfma64_fma4", out, in, cus, prop.clockRate)) return 1;
    CHECK(hipFree(in));
    CHECK(hipFree(out));
    return 0;
}
