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
// Output: one line per case, "<name> <waves per SIMD> <lane-instructions per second>".
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
    const float x = threadIdx.x * 0.5f, g = threadIdx.x * 0.25f;
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
                else
                    asm volatile("v_sub_f32_e32 %0, %1, %0\n v_sub_f32_e32 %0, %1, %0" : "+v"(acc[i]) : "s"(w));
            }
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < kChains; ++i) s += acc[i] + tmp[i];
    if (s == 12345.678f) out[0] = s;   // keeps the arithmetic alive; never true in practice
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
    CHECK(hipFree(out));
    return 0;
}
