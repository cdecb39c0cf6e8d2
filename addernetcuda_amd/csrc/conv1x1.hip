// 1x1 AdderNet convolution, pad 0, stride S = 1 or 2 (the ResNet downsample
// path, resnet20.py:66-70): the same three operations as the 3x3 kernels with
// K = Ci, so there is no halo and no LDS tile -- every lane reads its own
// float4 of the source row and keeps a TM x TN register tile; weights are
// wave-uniform SGPR operands.
//   forward  y[n,co,ho,wo]  = -sum_ci |w[co,ci] - x[n,ci,ho*S,wo*S]|
//   grad_x   gx[n,ci,hi,wi] =  sum_co hardtanh(w[co,ci] - x) * gy[n,co,hi/S,wi/S]  on the sampled
//                              grid, exactly 0 on the positions stride 2 skips
//   grad_w   gw[co,ci]      =  sum x*gy - w * sum gy   (partials folded per wave, summed in fp64)
// Replaces adder.cu:19-70 / 194-272 for these shapes together with the
// unfold/fold copies of adder.py:32-33,38-39.
#include "common.hpp"

namespace adder {

// A lane owns 4/S adjacent outputs of one output row: one float4 of the source row.
template <int S>
struct Lane1x1 {
    static constexpr int TN = 4 / S;
    int n, ho, wo0;   // first output of the lane
    bool ok;
    __device__ __forceinline__ Lane1x1(int g, int groups, int gpr, int Ho) {
        ok = g < groups;
        if (!ok) g = groups - 1;
        const int q = g % gpr;
        ho = (g / gpr) % Ho;
        n = g / (gpr * Ho);
        wo0 = q * TN;
    }
};

// Four consecutive floats of a row.  VEC: one aligned float4.  Otherwise (stride 1 on planes whose size is
// not a multiple of 4, walked as one long row) element by element, `valid` of them inside the row.
template <bool VEC>
__device__ __forceinline__ float4 ld4(const float *p, int valid) {
    if constexpr (VEC) return *reinterpret_cast<const float4 *>(p);
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (valid > 0) v.x = p[0];
    if (valid > 1) v.y = p[1];
    if (valid > 2) v.z = p[2];
    if (valid > 3) v.w = p[3];
    return v;
}
template <bool VEC>
__device__ __forceinline__ void st4(float *p, const float4 v, int valid) {
    if constexpr (VEC) {
        *reinterpret_cast<float4 *>(p) = v;
    } else {
        if (valid > 0) p[0] = v.x;
        if (valid > 1) p[1] = v.y;
        if (valid > 2) p[2] = v.z;
        if (valid > 3) p[3] = v.w;
    }
}

template <bool VEC>
__device__ __forceinline__ float2 ld2(const float *p, int valid) {
    if constexpr (VEC) return *reinterpret_cast<const float2 *>(p);
    float2 v = make_float2(0.f, 0.f);
    if (valid > 0) v.x = p[0];
    if (valid > 1) v.y = p[1];
    return v;
}
template <bool VEC>
__device__ __forceinline__ void st2(float *p, const float2 v, int valid) {
    if constexpr (VEC) {
        *reinterpret_cast<float2 *>(p) = v;
    } else {
        if (valid > 0) p[0] = v.x;
        if (valid > 1) p[1] = v.y;
    }
}

template <int S, int TM, bool VEC = true>
__global__ __launch_bounds__(256) void fwd_1x1_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                      float *__restrict__ y, double *__restrict__ stats, int N, int Ci,
                                                      int H, int W, int Co, int Ho, int Wo, int gpr, int groups) {
    constexpr int TN = 4 / S;
    const Lane1x1<S> L(blockIdx.x * 256 + threadIdx.x, groups, gpr, Ho);
    const int co0 = blockIdx.y * TM;
    uniform_f32_ptr wc = as_uniform(w);
    int wrow[TM];
#pragma unroll
    for (int m = 0; m < TM; ++m) wrow[m] = min(co0 + m, Co - 1) * Ci;
    float acc[TM][TN], tot[TM][TN];   // two-level sum: acc holds at most 64 channels
#pragma unroll
    for (int m = 0; m < TM; ++m)
#pragma unroll
        for (int t = 0; t < TN; ++t) acc[m][t] = tot[m][t] = 0.f;

    l2_warm(w + (size_t)co0 * Ci, 1, 0, min(TM, Co - co0) * Ci);   // the scalar weight loads below run one step ahead

    const size_t plane = (size_t)H * W;
    const float *xp = x + (size_t)L.n * Ci * plane + (size_t)(L.ho * S) * W + L.wo0 * S;
    const int valid = L.ok ? W - L.wo0 * S : 0;   // only read when !VEC
    int ci = 0;
    for (; ci + 4 <= Ci; ci += 4) {
        if ((ci & 63) == 0) {
#pragma unroll
            for (int m = 0; m < TM; ++m)
#pragma unroll
                for (int t = 0; t < TN; ++t) { tot[m][t] += acc[m][t]; acc[m][t] = 0.f; }
        }
        float4 xv[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) xv[e] = ld4<VEC>(xp + (size_t)(ci + e) * plane, valid);
#pragma unroll
        for (int m = 0; m < TM; ++m)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float wv = wc[wrow[m] + ci + e];
                const float xs[4] = {xv[e].x, xv[e].y, xv[e].z, xv[e].w};
#pragma unroll
                for (int t = 0; t < TN; ++t) acc[m][t] -= fabsf(wv - xs[t * S]);
            }
    }
    for (; ci < Ci; ++ci) {
        const float4 v = ld4<VEC>(xp + (size_t)ci * plane, valid);
        const float xs[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int m = 0; m < TM; ++m) {
            const float wv = wc[wrow[m] + ci];
#pragma unroll
            for (int t = 0; t < TN; ++t) acc[m][t] -= fabsf(wv - xs[t * S]);
        }
    }
#pragma unroll
    for (int m = 0; m < TM; ++m)
#pragma unroll
        for (int t = 0; t < TN; ++t) tot[m][t] += acc[m][t];
    if (stats) {
        // BatchNorm statistics of the output on the way out, as in the tiled forward kernels: per wave and output
        // channel the sums of y and y*y over the wave's valid outputs (deviations from a pivot in fp32, moved
        // back to the origin in fp64), slot = wave of this launch
        const int lane = threadIdx.x & 63;
        const int slots = gridDim.x * 4, slot = blockIdx.x * 4 + (threadIdx.x >> 6);
        const int nvalid = L.ok ? min(TN, Wo - L.wo0) : 0;
        const double count = (double)wave_sum_dpp((float)nvalid);
#pragma unroll
        for (int m = 0; m < TM; ++m) {
            const float pivot = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(tot[m][0])));
            float s1 = 0.f, s2 = 0.f;
#pragma unroll
            for (int t = 0; t < TN; ++t)
                if (t < nvalid) {
                    const float dv = tot[m][t] - pivot;
                    s1 += dv;
                    s2 = fmaf(dv, dv, s2);
                }
            const double d1 = (double)wave_sum_dpp(s1), d2 = (double)wave_sum_dpp(s2), c = (double)pivot;
            if (lane == 0 && co0 + m < Co) {
                stats[((size_t)(co0 + m) * slots + slot) * 2] = d1 + count * c;
                stats[((size_t)(co0 + m) * slots + slot) * 2 + 1] = d2 + 2.0 * c * d1 + count * c * c;
            }
        }
    }
    if (L.ok) {
#pragma unroll
        for (int m = 0; m < TM; ++m) {
            if (co0 + m >= Co) continue;
            float *dst = y + (((size_t)L.n * Co + co0 + m) * Ho + L.ho) * Wo + L.wo0;
            if constexpr (TN == 4)
                st4<VEC>(dst, make_float4(tot[m][0], tot[m][1], tot[m][2], tot[m][3]), valid);
            else
                st2<VEC>(dst, make_float2(tot[m][0], tot[m][1]), L.ok ? Wo - L.wo0 : 0);
        }
    }
}

template <int S, int TM, bool VEC = true>
__global__ __launch_bounds__(256) void grad_x_1x1_kernel(const float *__restrict__ gy,
                                                         const float *__restrict__ x,
                                                         const float *__restrict__ w, float *__restrict__ gx,
                                                         int N, int Ci, int H, int W, int Co, int Ho, int Wo,
                                                         int gpr, int groups) {
    constexpr int TN = 4 / S;
    const Lane1x1<S> L(blockIdx.x * 256 + threadIdx.x, groups, gpr, Ho);
    const int ci0 = blockIdx.y * TM;
    uniform_f32_ptr wc = as_uniform(w);
    const size_t plane = (size_t)H * W;
    const size_t xoff = (size_t)L.n * Ci * plane + (size_t)(L.ho * S) * W + L.wo0 * S;
    const int valid = L.ok ? W - L.wo0 * S : 0;   // only read when !VEC
    // clamp(w - x, -1, 1) = 2 * sat(0.5 w + cr) - 1 with cr = 0.5 - 0.5 x and sat the [0, 1] clamp modifier of
    // v_fma_f32: two instructions per term; sg collects the gy sum that the "- 1" multiplies
    float cr[TM][TN], acc[TM][TN], tot[TM][TN];   // two-level sum: acc holds at most 64 output channels
    float sg[TN], sgt[TN];
#pragma unroll
    for (int t = 0; t < TN; ++t) sg[t] = sgt[t] = 0.f;
#pragma unroll
    for (int m = 0; m < TM; ++m) {
        const float4 v = ld4<VEC>(x + xoff + (size_t)min(ci0 + m, Ci - 1) * plane, valid);
        const float xs[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int t = 0; t < TN; ++t) { cr[m][t] = fmaf(-0.5f, xs[t * S], 0.5f); acc[m][t] = tot[m][t] = 0.f; }
    }
    l2_warm(w + min(ci0, Ci - 1), Co, Ci, min(TM, Ci - ci0));   // one run of TM weights per output channel
    const size_t gplane = (size_t)Ho * Wo;
    const float *gp = gy + (size_t)L.n * Co * gplane + (size_t)L.ho * Wo + L.wo0;
    // eight output channels per round: their gy loads are issued together (little arithmetic per load, so
    // the loop is bound by how many loads are in flight); channels past Co load nothing and count as gy = 0
    constexpr int UN = 8;
    for (int co0 = 0; co0 < Co; co0 += UN) {
        float g[UN][TN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const bool live = co0 + u < Co;
            const float *src = gp + (size_t)min(co0 + u, Co - 1) * gplane;
            if constexpr (TN == 4) {
                const float4 v = ld4<VEC>(src, live ? valid : 0);
                g[u][0] = v.x; g[u][1] = v.y; g[u][2] = v.z; g[u][3] = v.w;
            } else {
                const float2 v = ld2<VEC>(src, live && L.ok ? Wo - L.wo0 : 0);
                g[u][0] = v.x; g[u][1] = v.y;
            }
            if (VEC && !live) {
#pragma unroll
                for (int t = 0; t < TN; ++t) g[u][t] = 0.f;
            }
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int co = min(co0 + u, Co - 1);
#pragma unroll
            for (int m = 0; m < TM; ++m) {
                const float wv = wc[co * Ci + min(ci0 + m, Ci - 1)];
#pragma unroll
                for (int t = 0; t < TN; ++t) acc[m][t] = fmaf(sat01(fmaf(wv, 0.5f, cr[m][t])), g[u][t], acc[m][t]);
            }
#pragma unroll
            for (int t = 0; t < TN; ++t) sg[t] += g[u][t];
        }
        if ((co0 & 63) == 64 - UN || co0 + UN >= Co) {
#pragma unroll
            for (int m = 0; m < TM; ++m)
#pragma unroll
                for (int t = 0; t < TN; ++t) { tot[m][t] += acc[m][t]; acc[m][t] = 0.f; }
#pragma unroll
            for (int t = 0; t < TN; ++t) { sgt[t] += sg[t]; sg[t] = 0.f; }
        }
    }
#pragma unroll
    for (int m = 0; m < TM; ++m)
#pragma unroll
        for (int t = 0; t < TN; ++t) tot[m][t] = fmaf(2.f, tot[m][t], -sgt[t]);
    if (L.ok) {
        const bool row2 = S == 2 && L.ho * 2 + 1 < H;  // the odd row below: never sampled by stride 2
#pragma unroll
        for (int m = 0; m < TM; ++m) {
            if (ci0 + m >= Ci) continue;
            float *dst = gx + xoff + (size_t)(ci0 + m) * plane;
            if constexpr (S == 1) {
                st4<VEC>(dst, make_float4(tot[m][0], tot[m][1], tot[m][2], tot[m][3]), valid);
            } else {
                st4<VEC>(dst, make_float4(tot[m][0], 0.f, tot[m][1], 0.f), valid);
                if (row2) st4<VEC>(dst + W, make_float4(0.f, 0.f, 0.f, 0.f), valid);
            }
        }
    }
}

// grad_w: a wave owns TM output channels x TC input channels; its lanes walk over position
// groups, then the 64 lanes are folded through LDS (16 sums per round).
template <int S, int TM, int TC, bool VEC = true>
__global__ __launch_bounds__(256) void grad_w_1x1_kernel(const float *__restrict__ gy,
                                                         const float *__restrict__ x, float *__restrict__ part,
                                                         float *__restrict__ sgpart, int N, int Ci, int H,
                                                         int W, int Co, int Ho, int Wo, int gpr, int groups) {
    constexpr int TN = 4 / S, A = TM * TC;
    const int co0 = blockIdx.y * TM, ci0 = blockIdx.z * TC;
    const size_t plane = (size_t)H * W, gplane = (size_t)Ho * Wo;
    float acc[TM][TC], sg[TM];
#pragma unroll
    for (int m = 0; m < TM; ++m) {
        sg[m] = 0.f;
#pragma unroll
        for (int c = 0; c < TC; ++c) acc[m][c] = 0.f;
    }
    for (int g0 = blockIdx.x * 256 + threadIdx.x; g0 < groups; g0 += gridDim.x * 256) {
        const Lane1x1<S> L(g0, groups, gpr, Ho);
        const float *xp = x + (size_t)L.n * Ci * plane + (size_t)(L.ho * S) * W + L.wo0 * S;
        const float *gp = gy + (size_t)L.n * Co * gplane + (size_t)L.ho * Wo + L.wo0;
        const int valid = W - L.wo0 * S;   // only read when !VEC
        float xs[TC][TN], gs[TM][TN];
#pragma unroll
        for (int c = 0; c < TC; ++c) {
            const float4 v = ld4<VEC>(xp + (size_t)min(ci0 + c, Ci - 1) * plane, valid);
            const float t4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int t = 0; t < TN; ++t) xs[c][t] = t4[t * S];
        }
#pragma unroll
        for (int m = 0; m < TM; ++m) {
            const float *p = gp + (size_t)min(co0 + m, Co - 1) * gplane;
            if constexpr (TN == 4) {
                const float4 v = ld4<VEC>(p, valid);
                gs[m][0] = v.x; gs[m][1] = v.y; gs[m][2] = v.z; gs[m][3] = v.w;
            } else {
                const float2 v = ld2<VEC>(p, Wo - L.wo0);
                gs[m][0] = v.x; gs[m][1] = v.y;
            }
        }
#pragma unroll
        for (int m = 0; m < TM; ++m) {
#pragma unroll
            for (int t = 0; t < TN; ++t) {
                sg[m] += gs[m][t];
#pragma unroll
                for (int c = 0; c < TC; ++c) acc[m][c] = fmaf(gs[m][t], xs[c][t], acc[m][c]);
            }
        }
    }
    // fold lanes, then the 4 waves of the workgroup
    __shared__ float red[4][64 * 17];
    __shared__ float wsum[4][A + TM];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    constexpr int TOT = A + TM;
    float all[TOT];
#pragma unroll
    for (int a = 0; a < A; ++a) all[a] = acc[a / TC][a % TC];
#pragma unroll
    for (int m = 0; m < TM; ++m) all[A + m] = sg[m];
    constexpr int ROUNDS = ceil_div(TOT, 16);
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
#pragma unroll
        for (int e = 0; e < 16; ++e) red[wave][lane * 17 + e] = (r * 16 + e < TOT) ? all[(r * 16 + e) % TOT] : 0.f;
        __syncthreads();
        const int e = lane & 15, rg = lane >> 4;
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < 16; ++k) s += red[wave][(rg * 16 + k) * 17 + e];
        s += __shfl_xor(s, 16, 64);
        s += __shfl_xor(s, 32, 64);
        if (rg == 0 && r * 16 + e < TOT) wsum[wave][r * 16 + e] = s;
        __syncthreads();
    }
    if (threadIdx.x < TOT) {
        const int a = threadIdx.x;
        const float s = (wsum[0][a] + wsum[1][a]) + (wsum[2][a] + wsum[3][a]);
        if (a < A) {
            const int co = co0 + a / TC, ci = ci0 + a % TC;
            if (co < Co && ci < Ci) part[(size_t)blockIdx.x * Co * Ci + (size_t)co * Ci + ci] = s;
        } else if (blockIdx.z == 0) {
            const int co = co0 + a - A;
            if (co < Co) sgpart[(size_t)blockIdx.x * Co + co] = s;
        }
    }
}

// ---- host side ------------------------------------------------------------------
// Stride 1: positions are independent, so every (H, W) plane is walked as one row of H*W elements; planes
// whose size is not a multiple of 4 (7x7) or whose base is not 16-byte aligned take the element-wise loads.
// Stride 2: one float4 of the source row per lane (two of its elements are sampled) and a float2 of the
// output row; rows that are not whole aligned groups (W % 4, Wo % 2, base pointers) are read element-wise.
bool conv1x1_supported(const ConvDims &d, const void *, const void *) {
    return d.kh == 1 && d.kw == 1 && d.pad == 0 && (d.stride == 1 || d.stride == 2);
}

// dimensions the kernels are launched with
static ConvDims lane_dims(const ConvDims &d) {
    ConvDims f = d;
    if (d.stride == 1) { f.H = 1; f.W = d.H * d.W; f.Ho = 1; f.Wo = d.H * d.W; }
    return f;
}

static bool vec_ok(const ConvDims &f, const void *a, const void *b, const void *c) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c);
    if (f.stride == 2) return f.W % 4 == 0 && f.Wo % 2 == 0 && (bits & 15) == 0;
    return f.W % 4 == 0 && (bits & 15) == 0;
}

static void lane_space(const ConvDims &f, int &gpr, int &groups) {
    gpr = ceil_div(f.Wo, 4 / f.stride);
    groups = f.N * f.Ho * gpr;
}

// partial-sum slots per channel of the statistics epilogue (one per wave of the launch)
int fwd_1x1_stats_slots(const ConvDims &d) {
    const ConvDims f = lane_dims(d);
    int gpr, groups;
    lane_space(f, gpr, groups);
    return ceil_div(groups, 256) * 4;
}

// stats (nullable): per-channel partial sums of y and y*y, fwd_1x1_stats_slots(d) slots per channel
int launch_fwd_1x1(const float *x, const float *w, float *y, double *stats, const ConvDims &d, hipStream_t s) {
    constexpr int TM = 8;
    const ConvDims f = lane_dims(d);
    int gpr, groups;
    lane_space(f, gpr, groups);
    const dim3 grid(ceil_div(groups, 256), ceil_div(f.Co, TM));
    if (f.stride == 2 && vec_ok(f, x, y, nullptr))
        hipLaunchKernelGGL((fwd_1x1_kernel<2, TM, true>), grid, dim3(256), 0, s, x, w, y, stats, f.N, f.Ci, f.H, f.W, f.Co,
                           f.Ho, f.Wo, gpr, groups);
    else if (f.stride == 2)
        hipLaunchKernelGGL((fwd_1x1_kernel<2, TM, false>), grid, dim3(256), 0, s, x, w, y, stats, f.N, f.Ci, f.H, f.W, f.Co,
                           f.Ho, f.Wo, gpr, groups);
    else if (vec_ok(f, x, y, nullptr))
        hipLaunchKernelGGL((fwd_1x1_kernel<1, TM, true>), grid, dim3(256), 0, s, x, w, y, stats, f.N, f.Ci, f.H, f.W, f.Co,
                           f.Ho, f.Wo, gpr, groups);
    else
        hipLaunchKernelGGL((fwd_1x1_kernel<1, TM, false>), grid, dim3(256), 0, s, x, w, y, stats, f.N, f.Ci, f.H, f.W, f.Co,
                           f.Ho, f.Wo, gpr, groups);
    return check_launch();
}

int launch_grad_x_1x1(const float *gy, const float *x, const float *w, float *gx, const ConvDims &d,
                      hipStream_t s) {
    constexpr int TM = 4;   // latency-bound at ResNet sizes: more workgroups beat more reuse per lane
    const ConvDims f = lane_dims(d);
    int gpr, groups;
    lane_space(f, gpr, groups);
    const dim3 grid(ceil_div(groups, 256), ceil_div(f.Ci, TM));
    if (f.stride == 2 && vec_ok(f, gy, x, gx))
        hipLaunchKernelGGL((grad_x_1x1_kernel<2, TM, true>), grid, dim3(256), 0, s, gy, x, w, gx, f.N, f.Ci, f.H, f.W,
                           f.Co, f.Ho, f.Wo, gpr, groups);
    else if (f.stride == 2)
        hipLaunchKernelGGL((grad_x_1x1_kernel<2, TM, false>), grid, dim3(256), 0, s, gy, x, w, gx, f.N, f.Ci, f.H,
                           f.W, f.Co, f.Ho, f.Wo, gpr, groups);
    else if (vec_ok(f, gy, x, gx))
        hipLaunchKernelGGL((grad_x_1x1_kernel<1, TM, true>), grid, dim3(256), 0, s, gy, x, w, gx, f.N, f.Ci, f.H, f.W,
                           f.Co, f.Ho, f.Wo, gpr, groups);
    else
        hipLaunchKernelGGL((grad_x_1x1_kernel<1, TM, false>), grid, dim3(256), 0, s, gy, x, w, gx, f.N, f.Ci, f.H,
                           f.W, f.Co, f.Ho, f.Wo, gpr, groups);
    return check_launch();
}

static constexpr int kGw1x1TM = 8, kGw1x1TC = 8;

int grad_w_1x1_slots(const ConvDims &d) {
    const ConvDims f = lane_dims(d);
    int gpr, groups;
    lane_space(f, gpr, groups);
    const int blocks_yz = ceil_div(f.Co, kGw1x1TM) * ceil_div(f.Ci, kGw1x1TC);
    int want = ceil_div(1024, blocks_yz);                 // ~4 workgroups per CU
    const int cap = ceil_div(groups, 256 * 4);            // at least 4 position groups per lane
    if (want > cap) want = cap;
    return want < 1 ? 1 : want;
}

int launch_grad_w_1x1(const float *gy, const float *x, float *part, float *sgpart, int slots,
                      const ConvDims &d, hipStream_t s) {
    const ConvDims f = lane_dims(d);
    int gpr, groups;
    lane_space(f, gpr, groups);
    const dim3 grid(slots, ceil_div(f.Co, kGw1x1TM), ceil_div(f.Ci, kGw1x1TC));
    if (f.stride == 2 && vec_ok(f, gy, x, nullptr))
        hipLaunchKernelGGL((grad_w_1x1_kernel<2, kGw1x1TM, kGw1x1TC, true>), grid, dim3(256), 0, s, gy, x, part,
                           sgpart, f.N, f.Ci, f.H, f.W, f.Co, f.Ho, f.Wo, gpr, groups);
    else if (f.stride == 2)
        hipLaunchKernelGGL((grad_w_1x1_kernel<2, kGw1x1TM, kGw1x1TC, false>), grid, dim3(256), 0, s, gy, x, part,
                           sgpart, f.N, f.Ci, f.H, f.W, f.Co, f.Ho, f.Wo, gpr, groups);
    else if (vec_ok(f, gy, x, nullptr))
        hipLaunchKernelGGL((grad_w_1x1_kernel<1, kGw1x1TM, kGw1x1TC, true>), grid, dim3(256), 0, s, gy, x, part,
                           sgpart, f.N, f.Ci, f.H, f.W, f.Co, f.Ho, f.Wo, gpr, groups);
    else
        hipLaunchKernelGGL((grad_w_1x1_kernel<1, kGw1x1TM, kGw1x1TC, false>), grid, dim3(256), 0, s, gy, x, part,
                           sgpart, f.N, f.Ci, f.H, f.W, f.Co, f.Ho, f.Wo, gpr, groups);
    return check_launch();
}

}  // namespace adder
