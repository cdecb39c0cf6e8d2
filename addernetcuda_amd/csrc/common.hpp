// Shared device/host helpers for the gfx950 AdderNet kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/addernet_hip.h"

namespace adder {

// Wave-uniform read-only data (weights) is fetched through the scalar cache:
// a load from the constant address space with a uniform address becomes
// s_load_dword*, and the value is then used directly as the SGPR operand of the
// vector subtract, so weights cost neither VGPRs nor LDS bandwidth.
typedef const __attribute__((address_space(4))) float *uniform_f32_ptr;

__device__ __forceinline__ uniform_f32_ptr as_uniform(const float *p) {
    return (uniform_f32_ptr)p;
}

// Touch `rows` runs of `len` floats, `pitch` floats apart, with one vector load per 128-byte line, so that
// the scalar weight loads of a kernel's main loop -- which run only one unit ahead and would otherwise wait
// for HBM on every new line, all workgroups at the same place -- find their lines in L2.
__device__ __forceinline__ void l2_warm(const float *p, int rows, int pitch, int len) {
    const int lines = (len + 31) / 32;
    for (int i = threadIdx.x; i < rows * lines; i += blockDim.x) {
        const int r = i / lines, l = i - r * lines;
        const float v = p[(size_t)r * pitch + min(l * 32, len - 1)];
        asm volatile("" ::"v"(v));
    }
}

// Storage types of activations: float, or bfloat16 (the upper half of a float, round to nearest even on the way
// out) for the optional reduced-storage mode; arithmetic is fp32 (fp64 for the weight gradient) either way.
typedef uint16_t bf16_t;
__device__ __forceinline__ float bf16_to_f32(bf16_t h) { return __uint_as_float((uint32_t)h << 16); }
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    u += 0x7fffu + ((u >> 16) & 1u);   // round to nearest, ties to even (NaN payloads are not preserved)
    return (bf16_t)(u >> 16);
}
__device__ __forceinline__ float ldf(const float *p) { return *p; }
__device__ __forceinline__ float ldf(const bf16_t *p) { return bf16_to_f32(*p); }
__device__ __forceinline__ void stf(float *p, float v) { *p = v; }
__device__ __forceinline__ void stf(bf16_t *p, float v) { *p = f32_to_bf16(v); }
// four / two consecutive elements at an address aligned to their total size
__device__ __forceinline__ float4 ldf4(const float *p) { return *reinterpret_cast<const float4 *>(p); }
__device__ __forceinline__ float4 ldf4(const bf16_t *p) {
    const uint2 u = *reinterpret_cast<const uint2 *>(p);
    return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                       __uint_as_float(u.y & 0xffff0000u));
}
__device__ __forceinline__ void stf4(float *p, float4 v) { *reinterpret_cast<float4 *>(p) = v; }
__device__ __forceinline__ void stf4(bf16_t *p, float4 v) {
    uint2 u;
    u.x = (uint32_t)f32_to_bf16(v.x) | ((uint32_t)f32_to_bf16(v.y) << 16);
    u.y = (uint32_t)f32_to_bf16(v.z) | ((uint32_t)f32_to_bf16(v.w) << 16);
    *reinterpret_cast<uint2 *>(p) = u;
}
__device__ __forceinline__ float2 ldf2(const float *p) { return *reinterpret_cast<const float2 *>(p); }
__device__ __forceinline__ float2 ldf2(const bf16_t *p) {
    const uint32_t u = *reinterpret_cast<const uint32_t *>(p);
    return make_float2(__uint_as_float(u << 16), __uint_as_float(u & 0xffff0000u));
}
__device__ __forceinline__ void stf2(float *p, float2 v) { *reinterpret_cast<float2 *>(p) = v; }
__device__ __forceinline__ void stf2(bf16_t *p, float2 v) {
    *reinterpret_cast<uint32_t *>(p) = (uint32_t)f32_to_bf16(v.x) | ((uint32_t)f32_to_bf16(v.y) << 16);
}

// Clamp to [0, 1]: the compiler folds it into the clamp output modifier of the instruction that
// produces v, so it costs no instruction of its own.
__device__ __forceinline__ float sat01(float v) { return __builtin_amdgcn_fmed3f(v, 0.f, 1.f); }

// hardtanh of adder.cu:17 (x<-1 -> -1, x<=1 -> x, else 1) is one v_med3_f32.
__device__ __forceinline__ float hardtanh(float v) {
    return __builtin_amdgcn_fmed3f(v, -1.0f, 1.0f);
}

// Kernels with more than 48 KB of dynamic LDS need hipFuncAttributeMaxDynamicSharedMemorySize, once per device
// (the attribute belongs to the device's copy of the function).  One flag word per kernel instantiation.
int record_hip_error(hipError_t e);
template <auto Kernel>
inline int allow_dynamic_lds(int bytes) {
    static unsigned long long done = 0;   // bit d: set on device d (benign race: setting it twice is harmless)
    if (bytes <= 48 * 1024) return 0;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return record_hip_error(e);
    if (dev >= 0 && dev < 64 && ((done >> dev) & 1ull)) return 0;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(Kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return record_hip_error(e);
    if (dev >= 0 && dev < 64) done |= 1ull << dev;
    return 0;
}

__host__ __device__ constexpr int ceil_div(int a, int b) { return (a + b - 1) / b; }
__host__ __device__ constexpr long ceil_div_l(long a, long b) { return (a + b - 1) / b; }
__host__ __device__ constexpr int round_up(int a, int b) { return ceil_div(a, b) * b; }

// Read `CNT` consecutive floats from LDS, `ALIGN` (1, 2 or 4 floats) being the
// alignment the caller guarantees for `p`; widest ds_read that alignment allows.
template <int CNT, int ALIGN>
__device__ __forceinline__ void lds_read_strip(const float *p, float (&dst)[CNT]) {
    int e = 0;
    if constexpr (ALIGN >= 4) {
#pragma unroll
        for (; e + 4 <= CNT; e += 4) {
            const float4 v = *reinterpret_cast<const float4 *>(p + e);
            dst[e] = v.x; dst[e + 1] = v.y; dst[e + 2] = v.z; dst[e + 3] = v.w;
        }
    }
    if constexpr (ALIGN >= 2) {
#pragma unroll
        for (; e + 2 <= CNT; e += 2) {
            const float2 v = *reinterpret_cast<const float2 *>(p + e);
            dst[e] = v.x; dst[e + 1] = v.y;
        }
    }
#pragma unroll
    for (; e < CNT; ++e) dst[e] = p[e];
}

// The same for `CNT` consecutive floats in global memory at an address aligned to `ALIGN` floats.
template <int CNT, int ALIGN>
__device__ __forceinline__ void global_read_strip(const float *__restrict__ p, float (&dst)[CNT]) {
    lds_read_strip<CNT, ALIGN>(p, dst);
}

// Sum over the 64 lanes of a wave; every lane receives the total.
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// Sum over the 64 lanes without LDS traffic: four DPP steps inside each row of 16 lanes, then the four row
// sums are read back as scalars.  The result is wave-uniform.
__device__ __forceinline__ float wave_sum_dpp(float v) {
    int t;
    t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true);    // quad_perm [1,0,3,2]
    v += __int_as_float(t);
    t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true);    // quad_perm [2,3,0,1]
    v += __int_as_float(t);
    t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true);   // row_half_mirror
    v += __int_as_float(t);
    t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true);   // row_mirror
    v += __int_as_float(t);
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return (r0 + r1) + (r2 + r3);
}

// The same sum for a caller that needs it in one lane only: the row sums travel on with two row broadcasts
// (lane 15 of each row into the next row, lane 31 into the upper half) instead of through scalar registers.
// The result is valid in lanes 48..63.
__device__ __forceinline__ float wave_sum_top_row(float v) {
    int t;
    t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true);    // quad_perm [1,0,3,2]
    v += __int_as_float(t);
    t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true);    // quad_perm [2,3,0,1]
    v += __int_as_float(t);
    t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true);   // row_half_mirror
    v += __int_as_float(t);
    t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true);   // row_mirror
    v += __int_as_float(t);
    t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x142, 0xA, 0xF, false);  // row_bcast:15 into rows 1, 3
    v += __int_as_float(t);
    t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x143, 0xC, 0xF, false);  // row_bcast:31 into rows 2, 3
    v += __int_as_float(t);
    return v;
}

// K sums over the 64 lanes at once (K = 4, 8 or 16) for a caller that needs each of them in one lane only: a
// reduce-scatter.  In each of the first log2(K) steps a lane keeps half of its values, hands the other half to its
// partner and adds what the partner hands over, so that the values halve while the lanes per sum double (partners: lane
// ^ 1, lane ^ 2, then the lanes 4 and 8 further round the row of 16, which pairs the quads just as well); what is left
// of the four in-row steps are plain sums, and the four rows are added lane by lane through the LDS crossbar (two
// ds_bpermute; the row broadcasts of DPP hand on lane 15 only).  K + K/2 + ... additions instead of 6 K.
// Returns, in every lane, the sum of v[j] over the wave with j = wave_sum_scatter_index<K>(lane); v is used up.
template <int CTRL>
__device__ __forceinline__ float dpp_row_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int K>
__device__ __forceinline__ int wave_sum_scatter_index(int lane) {
    constexpr int BITS = K == 16 ? 4 : (K == 8 ? 3 : 2);
    return (int)(__brev((unsigned)lane) >> (32 - BITS));   // step s splits on bit s of the lane and on bit BITS-1-s of j
}
template <int K, int S, int CTRL>
__device__ __forceinline__ void wave_sum_scatter_step(float (&v)[K], int lane) {
    constexpr int n = (K >> S) > 1 ? (K >> S) : 1;   // values still held before this step
    if constexpr (n > 1) {
        constexpr int h = n / 2;
        const bool up = (lane >> S) & 1;
#pragma unroll
        for (int i = 0; i < h; ++i) {
            const float keep = up ? v[i + h] : v[i], send = up ? v[i] : v[i + h];
            v[i] = keep + dpp_row_move<CTRL>(send);
        }
    } else {
        v[0] += dpp_row_move<CTRL>(v[0]);
    }
}
template <int K>
__device__ __forceinline__ float wave_sum_scatter(float (&v)[K], int lane) {
    static_assert(K == 4 || K == 8 || K == 16, "4, 8 or 16 sums");
    wave_sum_scatter_step<K, 0, 0xB1>(v, lane);    // quad_perm [1,0,3,2]
    wave_sum_scatter_step<K, 1, 0x4E>(v, lane);    // quad_perm [2,3,0,1]
    wave_sum_scatter_step<K, 2, 0x124>(v, lane);   // row_ror:4
    wave_sum_scatter_step<K, 3, 0x128>(v, lane);   // row_ror:8
    float r = v[0];
    r += __shfl_xor(r, 16, 64);
    r += __shfl_xor(r, 32, 64);
    return r;
}

struct ConvDims {
    int N, Ci, H, W, Co, kh, kw, stride, pad, Ho, Wo;
    __host__ __device__ int K() const { return Ci * kh * kw; }
};

// ---- host-side launch plumbing -------------------------------------------------
int record_hip_error(hipError_t e);  // stores the message, returns ADDER_ERR_HIP
int check_launch();                  // hipGetLastError -> status

// Launchers implemented in the kernel translation units.
int launch_fwd(const float *x, const float *w, float *y, double *stats, const ConvDims &d, hipStream_t s);
int fwd_stats_slots(const ConvDims &d);
bool fwd_pair_supported(const ConvDims &d);
int launch_fwd_pair(const float *x, const float *w, const float *w_side, float *y, float *y_side, double *stats,
                    double *stats_side, const ConvDims &d, hipStream_t s);
int launch_mulconv_fwd(const float *x, const float *w, float *y, double *stats, const ConvDims &d, hipStream_t s);   // 0: no statistics epilogue for these dimensions
int launch_grad_x(const float *gy, const float *x, const float *w, float *gx, const ConvDims &d,
                  hipStream_t s, const float *gadd = nullptr);
size_t grad_w_workspace_bytes(const ConvDims &d);
// The sums of the backward of the BatchNorm behind a layer, as the consumer's input-gradient kernel left them
// ((C, slots, 2) floats -- a wave's fp32 totals: sum dz, sum dz * xhat), with what turns them into the four coefficients per channel.
// A weight-gradient kernel that is given these instead of ready coefficients adds the slots itself (every
// workgroup its own channels, all in the same order) and writes dgamma / dbeta on the way.  part == null: not used.
struct BnSums {
    const float *part;
    int slots;
    double count;            // N * Ho * Wo: values per channel of the BatchNorm
    const float *gamma, *mean, *rstd;
    float *dgamma, *dbeta;
};
static constexpr BnSums kNoBnSums{nullptr, 0, 0.0, nullptr, nullptr, nullptr, nullptr, nullptr};
int launch_grad_w(const float *gy, const float *x, const float *w, float *gw, float eta,
                  void *ws, size_t ws_bytes, const ConvDims &d, hipStream_t s, const float *bn_y = nullptr,
                  const float *bn_coef = nullptr, float *gy_out = nullptr, const BnSums &sums = kNoBnSums);
// the BatchNorm backward passes of a layer's neighbours inside the layer's backward kernels (adder_bn_links)
int grad_x_bn_slots(const ConvDims &d);
int launch_grad_x_bn(const float *gy, const float *x, const float *w, float *gx, const ConvDims &d, hipStream_t s,
                     const float *gadd, const adder_bn_links &bn);
bool grad_w_bn_supported(const ConvDims &d, const void *gy, const void *x, const void *bn_y, const void *bn_coef);
int launch_bn_bwd_coef(const float *part, int slots, const float *gamma, const float *mean, const float *rstd,
                       double count, float *coef, float *dgamma, float *dbeta, int C, hipStream_t s);

// matrix-core weight gradient of the 3x3 / pad-1 layers (grad_w_mfma.hip); variant 0 = not applicable
struct GradWMfmaPlan { int variant, slots, gy, gz, tilesH, tilesW, ntiles; };
GradWMfmaPlan plan_grad_w_mfma(const ConvDims &d);
int launch_grad_w_mfma(const float *gy, const float *x, double *part, double *sgpart, const ConvDims &d,
                       const GradWMfmaPlan &p, hipStream_t s);
int launch_grad_w_mfma_bn(const float *gy, const float *x, double *part, double *sgpart, const ConvDims &d,
                          const GradWMfmaPlan &p, const float *bn_y, const float *bn_coef, float *gy_out, hipStream_t s,
                          const BnSums &sums = kNoBnSums);

// 1x1 / pad 0 / stride 1-2 kernels (conv1x1.hip)
bool conv1x1_supported(const ConvDims &d, const void *a, const void *b);
int fwd_1x1_stats_slots(const ConvDims &d);
int launch_fwd_1x1(const float *x, const float *w, float *y, double *stats, const ConvDims &d, hipStream_t s);
int launch_grad_x_1x1(const float *gy, const float *x, const float *w, float *gx, const ConvDims &d,
                      hipStream_t s);
int grad_w_1x1_slots(const ConvDims &d);
int launch_grad_w_1x1(const float *gy, const float *x, float *part, float *sgpart, int slots,
                      const ConvDims &d, hipStream_t s);

// fused BatchNorm + residual + ReLU (bn_act.hip)
size_t bn_workspace_bytes(int N, int C, int HW);
size_t bn_mask_words(int N, int C, int HW);
int launch_bn_act_fwd(const float *x, const float *res, const float *gamma, const float *beta, float *y,
                      unsigned *mask, float *mean, float *rstd, float *running_mean, float *running_var,
                      long long *num_batches, float momentum, float eps, int relu, int N, int C, int HW, void *ws,
                      const double *stats, int stats_slots, hipStream_t s);
int launch_bn_act_bwd(const float *dy, const float *y, const unsigned *mask, const float *x, const float *gamma,
                      const float *mean, const float *rstd, float *dx, float *dres, float *dgamma, float *dbeta,
                      int relu, int N, int C, int HW, void *ws, hipStream_t s);

// average pool over the whole map -> matrix product -> BatchNorm of the ResNet classifier head (head.hip)
bool head_supported(int N, int C, int HW, int J);
int launch_head_fwd(const float *x, const float *w, const float *gamma, const float *beta, float *pooled, float *z,
                    float *y, float *mean, float *rstd, float *running_mean, float *running_var, long long *num_batches,
                    float momentum, float eps, int N, int C, int HW, int J, hipStream_t s);
int launch_head_bwd(const float *dy, const float *z, const float *pooled, const float *w, const float *gamma,
                    const float *mean, const float *rstd, float *dz, float *dx, float *dw, float *dgamma, float *dbeta,
                    int N, int C, int HW, int J, hipStream_t s);

int launch_ce_fwd(const float *y, const long long *target, float *loss, float *lse, int N, int J, hipStream_t s);
int launch_ce_bwd(const float *y, const long long *target, const float *lse, const float *grad_loss, float *gy, int N,
                  int J, hipStream_t s);

size_t norm_scale_workspace_bytes(long n);
int launch_norm_scale(float *g, long n, float eta, float eps, void *ws, hipStream_t s);
static constexpr int kNormBatchMax = ADDER_NORM_BATCH_MAX;
static constexpr int kSgdBatchMax = ADDER_SGD_BATCH_MAX;
int launch_sgd_momentum(int count, float *const *p, const float *const *g, float *const *buf, const long *n,
                        const float *lr_ptr, float lr, float momentum, float weight_decay, hipStream_t s);
static constexpr int kGwFinishMax = ADDER_GRAD_W_FINISH_MAX;
int launch_grad_w_staged(const float *gy, const float *x, const float *w, float *gw, float eta, void *ws,
                         size_t ws_bytes, const ConvDims &d, adder_grad_w_stage *stage, hipStream_t s,
                         const float *bn_y = nullptr, const float *bn_coef = nullptr, float *gy_out = nullptr,
                         const BnSums &sums = kNoBnSums);
size_t grad_w_finish_workspace_bytes(int count, const adder_grad_w_stage *st);
int launch_grad_w_finish(int count, const adder_grad_w_stage *st, void *ws, hipStream_t s);
size_t norm_scale_batched_workspace_bytes(int count);
int launch_norm_scale_batched(int count, float *const *g, const long *n, const float *eta, float eps, void *ws,
                              hipStream_t s);

int launch_grad_w_slab_finalize(const double *part, const double *sgpart, const float *w, float *gw, int slots, int Co,
                                int K, bool accumulate, hipStream_t s);
// bfloat16 storage of x / y / gy / gx (weights and weight gradients stay fp32): the tiled 3x3 / pad-1 kernels and
// the generic ones
int launch_fwd_bf16(const bf16_t *x, const float *w, bf16_t *y, const ConvDims &d, hipStream_t s);
int launch_grad_x_bf16(const bf16_t *gy, const bf16_t *x, const float *w, bf16_t *gx, const ConvDims &d, hipStream_t s);
int launch_grad_w_bf16(const bf16_t *gy, const bf16_t *x, const float *w, float *gw, float eta, void *ws, size_t ws_bytes,
                       const ConvDims &d, hipStream_t s);
int launch_grad_w_mfma_bf16(const bf16_t *gy, const bf16_t *x, double *part, double *sgpart, const ConvDims &d,
                            const GradWMfmaPlan &p, hipStream_t s);
int launch_col_fwd(const float *X, const float *W, float *out, int K, long NL, int Co, hipStream_t s);
size_t col_grad_w_workspace_bytes(int K, long NL, int Co);
int launch_col_grad_w(const float *gy, const float *X, const float *W, float *gW, int K, long NL,
                      int Co, void *ws, hipStream_t s);
int launch_col_grad_x(const float *gy, const float *X, const float *W, float *gX, int K, long NL,
                      int Co, hipStream_t s);
int launch_col_bwd_small(const float *gy, const float *X, const float *W, float *gW, float *gX, int K, long NL, int Co,
                         hipStream_t s);
int launch_col_bwd_fused(const float *gy, const float *X, const float *W, float *gW, float *gX, int K, long NL, int Co,
                         void *ws, hipStream_t s);

}  // namespace adder
