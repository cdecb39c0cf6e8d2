// The classifier head behind the last adder block of the ResNets (the reference's resnet20.py:55-57, 89-93):
//   AvgPool2d over the whole map -> 1x1 convolution without bias (a matrix product on a 1x1 map) -> BatchNorm2d
// in training mode, as two launches forward and two launches backward.  The vendor path spends 4 + 4 launches of
// 5-10 us each on tensors of N x 10 and N x 64 values; nothing here is bound by anything but launch latency, so
// the kernels are written for few launches and short dependent chains, and every sum has a fixed order.
//
//   forward 1 (one workgroup per image):  pooled[n, c] = mean over the plane,  z[n, j] = sum_c w[j, c] * pooled[n, c]
//   forward 2 (one workgroup):            per class j the batch statistics of z, y = gamma * (z - mean) * rstd + beta,
//                                         running statistics
//   backward 1 (one workgroup):           dgamma, dbeta, dz = gamma * rstd * (dy - mean(dy) - zhat * mean(dy * zhat)),
//                                         dw[j, c] = sum_n dz[n, j] * pooled[n, c]
//   backward 2 (one workgroup per image): dpooled[c] = sum_j dz[n, j] * w[j, c],  dx[n, c, :, :] = dpooled[c] / HW
#include "common.hpp"

namespace adder {

static constexpr int kHeadThreads = 256;
static constexpr int kHeadMaxClasses = 32;    // two per wave of the one-workgroup kernels
static constexpr int kHeadMaxChannels = 256;  // channels divide the 256-thread workgroups of the per-image kernels

// G lanes (a power of two <= 64, aligned) share a plane: their sum in the first of them
template <int G>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
    for (int off = G / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// HW4 = float4 groups per plane, a power of two <= 64 (template), so that the lanes of a plane sit side by side
template <int HW4>
__global__ __launch_bounds__(kHeadThreads) void head_pool_fc_kernel(const float *__restrict__ x,
                                                                    const float *__restrict__ w,
                                                                    float *__restrict__ pooled,
                                                                    float *__restrict__ z, int C, int J) {
    __shared__ float pl[kHeadMaxChannels];
    const int n = blockIdx.x;
    const float4 *src = reinterpret_cast<const float4 *>(x) + (size_t)n * C * HW4;
    const int total = C * HW4;
    const float inv = 1.f / (float)(HW4 * 4);
    for (int i0 = 0; i0 < total; i0 += kHeadThreads) {   // (C * HW4 is a multiple of HW4, so whole planes per pass)
        const int i = i0 + threadIdx.x;
        float s = 0.f;
        if (i < total) {
            const float4 v = src[i];
            s = (v.x + v.y) + (v.z + v.w);
        }
        s = group_sum<HW4>(s);
        if (i < total && (i & (HW4 - 1)) == 0) pl[i / HW4] = s * inv;
    }
    __syncthreads();
    for (int c = threadIdx.x; c < C; c += kHeadThreads) pooled[(size_t)n * C + c] = pl[c];
    // one wave per class: 64 lanes over the channels
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int j = wave; j < J; j += kHeadThreads / 64) {
        float s = 0.f;
        for (int c = lane; c < C; c += 64) s = fmaf(w[(size_t)j * C + c], pl[c], s);
        s = wave_sum(s);
        if (lane == 0) z[(size_t)n * J + j] = s;
    }
}

// The two one-workgroup kernels below work on (N, J) matrices with 1024 threads: on its own a workgroup pays a full
// memory round trip for every load it waits for, so all global loads of a phase are issued together (clamped
// indices instead of branches, a handful per thread), and everything after them works from LDS.
// Sums over the batch: the matrix goes to LDS transposed (row stride NS = N | 1: conflict-free) and wave w adds the
// classes w, w + 16, ... (64 lanes over the images, fp64).  The loops over a wave's classes run to a compile-time
// bound (PER = classes rounded up to 16 or 32, over the 16 waves) so that they unroll without a branch per class.
static constexpr int kHeadWide = 1024, kHeadWaves = kHeadWide / 64, kHeadBatch = 4;
static constexpr int kHeadDw = 512;   // threads of the weight-gradient phase (their partial sums must fit the LDS)

// sa[j] = sum_n at[j][n], sb[j] = sum_n bt[j][n], or of the squares of at (SQ; bt unused)
template <int PER, bool SQ>
__device__ __forceinline__ void head_class_sums(const float *at, const float *bt, int N, int NS, int J, double *sa,
                                                double *sb) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    double a[PER], b[PER];
#pragma unroll
    for (int k = 0; k < PER; ++k) a[k] = b[k] = 0.0;
    for (int n = lane; n < N; n += 64)
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            const int j = min(wave + kHeadWaves * k, J - 1);   // (classes past J repeat the last one; not stored)
            const double av = (double)at[j * NS + n];
            a[k] += av;
            b[k] += SQ ? av * av : (double)bt[j * NS + n];
        }
#pragma unroll
    for (int k = 0; k < PER; ++k) {
        a[k] = wave_sum(a[k]);
        b[k] = wave_sum(b[k]);
    }
    if (lane == 0) {
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            const int j = wave + kHeadWaves * k;
            if (j < J) { sa[j] = a[k]; sb[j] = b[k]; }
        }
    }
}

// LDS (dynamic): z transposed, J * NS floats
template <int PER>
__global__ __launch_bounds__(kHeadWide) void head_bn_fwd_kernel(const float *__restrict__ z,
                                                                const float *__restrict__ gamma,
                                                                const float *__restrict__ beta, float *__restrict__ y,
                                                                float *__restrict__ mean, float *__restrict__ rstd,
                                                                float *__restrict__ running_mean,
                                                                float *__restrict__ running_var,
                                                                long long *__restrict__ num_batches, float momentum,
                                                                float eps, int N, int J) {
    extern __shared__ __align__(16) float lds[];
    __shared__ double s1[kHeadMaxClasses], s2[kHeadMaxClasses];
    __shared__ float mu_s[kHeadMaxClasses], rs_s[kHeadMaxClasses], g_s[kHeadMaxClasses], b_s[kHeadMaxClasses];
    const int NS = N | 1, NJ = N * J;
    float *zt = lds;
    // the per-class operands of the last phases, asked for now
    const int jc = min((int)threadIdx.x, J - 1);
    const float g_own = gamma[jc], b_own = beta[jc];
    const float rm_own = running_mean ? running_mean[jc] : 0.f, rv_own = running_var ? running_var[jc] : 0.f;
    for (int i0 = threadIdx.x; i0 < NJ; i0 += kHeadWide * kHeadBatch) {
        float v[kHeadBatch];
#pragma unroll
        for (int u = 0; u < kHeadBatch; ++u) v[u] = z[min(i0 + u * kHeadWide, NJ - 1)];
#pragma unroll
        for (int u = 0; u < kHeadBatch; ++u) {
            const int i = i0 + u * kHeadWide;
            if (i < NJ) {
                const int n = i / J, j = i - n * J;
                zt[j * NS + n] = v[u];
            }
        }
    }
    __syncthreads();
    head_class_sums<PER, true>(zt, zt, N, NS, J, s1, s2);
    __syncthreads();
    if (threadIdx.x < J) {
        const int j = threadIdx.x;
        const double mu = s1[j] / N;
        double var = s2[j] / N - mu * mu;
        if (var < 0.0) var = 0.0;
        const float rs = (float)(1.0 / sqrt(var + (double)eps));
        mu_s[j] = (float)mu;
        rs_s[j] = rs;
        g_s[j] = g_own;
        b_s[j] = b_own;
        mean[j] = (float)mu;
        rstd[j] = rs;
        if (running_mean) {
            const double unbiased = N > 1 ? var * N / (N - 1.0) : var;
            running_mean[j] = (float)((1.0 - momentum) * (double)rm_own + momentum * mu);
            running_var[j] = (float)((1.0 - momentum) * (double)rv_own + momentum * unbiased);
        }
        if (j == 0 && num_batches) *num_batches += 1;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < NJ; i += kHeadWide) {
        const int n = i / J, j = i - n * J;
        y[i] = fmaf((zt[j * NS + n] - mu_s[j]) * rs_s[j], g_s[j], b_s[j]);
    }
}

static size_t head_fwd_lds_bytes(int N, int J) { return sizeof(float) * (size_t)J * (N | 1); }

// JP = 16 * PER: the classes rounded up to 16 or 32.
// LDS (dynamic): pooled (N, C) | dz with zero-padded rows (N, JP) | dy, dy * zhat and zhat transposed (3, J, NS), which
// the partial sums of dw (512 / C slices, JP, C) take over once they are used up
template <int PER>
__global__ __launch_bounds__(kHeadWide) void head_bn_bwd_kernel(const float *__restrict__ dy,
                                                                const float *__restrict__ z,
                                                                const float *__restrict__ pooled,
                                                                const float *__restrict__ gamma,
                                                                const float *__restrict__ mean,
                                                                const float *__restrict__ rstd, float *__restrict__ dz,
                                                                float *__restrict__ dw, float *__restrict__ dgamma,
                                                                float *__restrict__ dbeta, int N, int C, int J) {
    extern __shared__ __align__(16) float lds[];
    __shared__ double s1[kHeadMaxClasses], s2[kHeadMaxClasses];
    __shared__ float gr_s[kHeadMaxClasses], m1_s[kHeadMaxClasses], m2_s[kHeadMaxClasses];   // gamma * rstd, the two means
    const int NS = N | 1, NJ = N * J;
    constexpr int JP = 16 * PER;
    float *pl = lds, *dzl = pl + N * C, *gt = dzl + N * JP, *ht = gt + (size_t)J * NS, *zt = ht + (size_t)J * NS,
          *part = gt;
    if (threadIdx.x < J) gr_s[threadIdx.x] = gamma[threadIdx.x] * rstd[threadIdx.x];
    // dy and zhat (transposed) and pooled (N * C is a multiple of four) into LDS
    const int total = N * C / 4;
    for (int i0 = threadIdx.x; i0 < max(NJ, total); i0 += kHeadWide * kHeadBatch) {
        float g[kHeadBatch], zv[kHeadBatch], mu[kHeadBatch], rs[kHeadBatch];
        float4 pv[kHeadBatch];
#pragma unroll
        for (int u = 0; u < kHeadBatch; ++u) {
            const int i = min(i0 + u * kHeadWide, NJ - 1), j = i % J;
            g[u] = dy[i];
            zv[u] = z[i];
            mu[u] = mean[j];
            rs[u] = rstd[j];
            pv[u] = reinterpret_cast<const float4 *>(pooled)[min(i0 + u * kHeadWide, total - 1)];
        }
#pragma unroll
        for (int u = 0; u < kHeadBatch; ++u) {
            const int i = i0 + u * kHeadWide;
            if (i < NJ) {
                const int n = i / J, j = i - n * J;
                const float zh = (zv[u] - mu[u]) * rs[u];
                gt[j * NS + n] = g[u];
                ht[j * NS + n] = g[u] * zh;
                zt[j * NS + n] = zh;
            }
            if (i < total) reinterpret_cast<float4 *>(pl)[i] = pv[u];
        }
    }
    __syncthreads();
    head_class_sums<PER, false>(gt, ht, N, NS, J, s1, s2);
    __syncthreads();
    if (threadIdx.x < J) {   // (once per class: a double-precision division per element costs microseconds here)
        dbeta[threadIdx.x] = (float)s1[threadIdx.x];
        dgamma[threadIdx.x] = (float)s2[threadIdx.x];
        m1_s[threadIdx.x] = (float)(s1[threadIdx.x] / N);
        m2_s[threadIdx.x] = (float)(s2[threadIdx.x] / N);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < N * JP; i += kHeadWide) {
        const int n = i / JP, j = i % JP;
        float v = 0.f;
        if (j < J) {
            v = gr_s[j] * (gt[j * NS + n] - m1_s[j] - zt[j * NS + n] * m2_s[j]);
            dz[n * J + j] = v;
        }
        dzl[i] = v;   // (classes past J: zeros, so the unrolled products below add nothing)
    }
    __syncthreads();
    // dw[j, c] = sum_n dz[n, j] * pooled[n, c], by the first 512 threads: thread (slice, c) adds the images slice,
    // slice + S, ... (S = 512 / C) for all classes at once -- one read of pooled and JP / 4 reads of a dz row per JP
    // products (a read per product keeps the one CU's LDS busy for microseconds) -- and the slices are added in order
    const int S = kHeadDw / C;
    if (threadIdx.x < kHeadDw) {
        const int c = threadIdx.x % C, sl = threadIdx.x / C;
        float acc[JP];
#pragma unroll
        for (int j = 0; j < JP; ++j) acc[j] = 0.f;
#pragma unroll 2
        for (int n = sl; n < N; n += S) {
            const float p = pl[n * C + c];
            float d[JP];
            lds_read_strip<JP, 4>(dzl + n * JP, d);
#pragma unroll
            for (int j = 0; j < JP; ++j) acc[j] = fmaf(d[j], p, acc[j]);
        }
#pragma unroll
        for (int j = 0; j < JP; ++j) part[(sl * JP + j) * C + c] = acc[j];
    }
    __syncthreads();
    for (int i = threadIdx.x; i < J * C; i += kHeadWide) {
        const int j = i / C, cc = i - j * C;
        float t = 0.f;
        for (int k = 0; k < S; ++k) t += part[(k * JP + j) * C + cc];
        dw[i] = t;
    }
}

static size_t head_bwd_lds_bytes(int N, int C, int J) {
    const size_t JP = J <= kHeadWaves ? 16 : 32;
    const size_t sums = 3 * (size_t)J * (N | 1), part = (size_t)kHeadDw * JP;
    return sizeof(float) * ((size_t)N * C + (size_t)N * JP + (sums > part ? sums : part));
}

template <int HW4>
__global__ __launch_bounds__(kHeadThreads) void head_expand_kernel(const float *__restrict__ dz,
                                                                   const float *__restrict__ w,
                                                                   float *__restrict__ dx, int C, int J) {
    __shared__ float dp[kHeadMaxChannels];
    const int n = blockIdx.x;
    const float inv = 1.f / (float)(HW4 * 4);
    for (int c = threadIdx.x; c < C; c += kHeadThreads) {
        float s = 0.f;
        for (int j = 0; j < J; ++j) s = fmaf(dz[(size_t)n * J + j], w[(size_t)j * C + c], s);
        dp[c] = s * inv;
    }
    __syncthreads();
    float4 *dst = reinterpret_cast<float4 *>(dx) + (size_t)n * C * HW4;
    const int total = C * HW4;
    for (int i = threadIdx.x; i < total; i += kHeadThreads) {
        const float v = dp[i / HW4];
        dst[i] = make_float4(v, v, v, v);
    }
}

// a power-of-two plane of 4 .. 256 positions, channels that divide the workgroup, and a batch whose pooled matrix
// fits the backward kernel's LDS
bool head_supported(int N, int C, int HW, int J) {
    const int hw4 = HW / 4;
    return N >= 2 && HW % 4 == 0 && hw4 >= 1 && hw4 <= 64 && (hw4 & (hw4 - 1)) == 0 && C >= 1 &&
           C <= kHeadThreads && kHeadThreads % C == 0 && ((long)N * C) % 4 == 0 && J >= 1 && J <= kHeadMaxClasses &&
           head_bwd_lds_bytes(N, C, J) <= 144 * 1024 && head_fwd_lds_bytes(N, J) <= 144 * 1024;
}

template <int HW4>
static void launch_pool_fc(const float *x, const float *w, float *pooled, float *z, int N, int C, int J, hipStream_t s) {
    hipLaunchKernelGGL(head_pool_fc_kernel<HW4>, dim3(N), dim3(kHeadThreads), 0, s, x, w, pooled, z, C, J);
}

template <int HW4>
static void launch_expand(const float *dz, const float *w, float *dx, int N, int C, int J, hipStream_t s) {
    hipLaunchKernelGGL(head_expand_kernel<HW4>, dim3(N), dim3(kHeadThreads), 0, s, dz, w, dx, C, J);
}

// ---- the loss of the training script (main.py:66,90: torch.nn.CrossEntropyLoss, mean over the batch) ----------
// On N x classes logits the framework runs log_softmax and nll_loss forward and backward plus two fills: six launches
// of 4-8 us.  One workgroup each way here: a thread per image keeps the image's logits in registers.
static constexpr int kCeThreads = 1024, kCeMaxClasses = 32;

// loss = mean_n (lse_n - y[n, t_n]), lse_n = log sum_j exp(y[n, j]); lse (N) is kept for the backward.
__global__ __launch_bounds__(kCeThreads) void ce_fwd_kernel(const float *__restrict__ y,
                                                            const long long *__restrict__ target,
                                                            float *__restrict__ loss, float *__restrict__ lse, int N,
                                                            int J) {
    __shared__ float wsum[kCeThreads / 64];
    float mine = 0.f;
    for (int n = threadIdx.x; n < N; n += kCeThreads) {
        float v[kCeMaxClasses];
#pragma unroll
        for (int j = 0; j < kCeMaxClasses; ++j) v[j] = y[(size_t)n * J + min(j, J - 1)];   // (all loads in flight)
        const int t = (int)min(max(target[n], 0LL), (long long)J - 1);
        float m = v[0];
#pragma unroll
        for (int j = 1; j < kCeMaxClasses; ++j) m = fmaxf(m, v[j]);
        float sum = 0.f, yt = v[0];
#pragma unroll
        for (int j = 0; j < kCeMaxClasses; ++j) {
            sum += j < J ? expf(v[j] - m) : 0.f;
            yt = j == t ? v[j] : yt;
        }
        const float l = m + logf(sum);
        lse[n] = l;
        mine += l - yt;
    }
    mine = wave_sum(mine);   // (64 lanes in a fixed butterfly, then the waves in order: the same bits every run)
    if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = mine;
    __syncthreads();
    if (threadIdx.x == 0) {
        float total = 0.f;
        for (int w = 0; w < kCeThreads / 64; ++w) total += wsum[w];
        loss[0] = total / (float)N;
    }
}

// grad_logits[n, j] = (exp(y[n, j] - lse_n) - [j == t_n]) * grad_loss / N
__global__ __launch_bounds__(kCeThreads) void ce_bwd_kernel(const float *__restrict__ y,
                                                            const long long *__restrict__ target,
                                                            const float *__restrict__ lse,
                                                            const float *__restrict__ grad_loss,
                                                            float *__restrict__ gy, int N, int J) {
    const float scale = grad_loss[0] / (float)N;
    const int i = blockIdx.x * kCeThreads + threadIdx.x;
    if (i < N * J) {
        const int n = i / J, j = i - n * J;
        const float p = expf(y[i] - lse[n]);
        gy[i] = (p - (target[n] == (long long)j ? 1.f : 0.f)) * scale;
    }
}

int launch_ce_fwd(const float *y, const long long *target, float *loss, float *lse, int N, int J, hipStream_t s) {
    if (J > kCeMaxClasses) return ADDER_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(ce_fwd_kernel, dim3(1), dim3(kCeThreads), 0, s, y, target, loss, lse, N, J);
    return check_launch();
}

int launch_ce_bwd(const float *y, const long long *target, const float *lse, const float *grad_loss, float *gy, int N,
                  int J, hipStream_t s) {
    if (J > kCeMaxClasses) return ADDER_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(ce_bwd_kernel, dim3(ceil_div(N * J, kCeThreads)), dim3(kCeThreads), 0, s, y, target, lse, grad_loss,
                       gy, N, J);
    return check_launch();
}

#define ADDER_HEAD_DISPATCH(fn, ...)                       \
    switch (HW / 4) {                                      \
        case 1: fn<1>(__VA_ARGS__); break;                 \
        case 2: fn<2>(__VA_ARGS__); break;                 \
        case 4: fn<4>(__VA_ARGS__); break;                 \
        case 8: fn<8>(__VA_ARGS__); break;                 \
        case 16: fn<16>(__VA_ARGS__); break;               \
        case 32: fn<32>(__VA_ARGS__); break;               \
        default: fn<64>(__VA_ARGS__); break;               \
    }

int launch_head_fwd(const float *x, const float *w, const float *gamma, const float *beta, float *pooled, float *z,
                    float *y, float *mean, float *rstd, float *running_mean, float *running_var, long long *num_batches,
                    float momentum, float eps, int N, int C, int HW, int J, hipStream_t s) {
    if (!head_supported(N, C, HW, J)) return ADDER_ERR_UNSUPPORTED;
    ADDER_HEAD_DISPATCH(launch_pool_fc, x, w, pooled, z, N, C, J, s)
    const size_t lds = head_fwd_lds_bytes(N, J);
    if (J <= kHeadWaves) {
        if (int rc = allow_dynamic_lds<&head_bn_fwd_kernel<1>>((int)lds)) return rc;
        hipLaunchKernelGGL(head_bn_fwd_kernel<1>, dim3(1), dim3(kHeadWide), lds, s, z, gamma, beta, y, mean, rstd,
                           running_mean, running_var, num_batches, momentum, eps, N, J);
    } else {
        if (int rc = allow_dynamic_lds<&head_bn_fwd_kernel<2>>((int)lds)) return rc;
        hipLaunchKernelGGL(head_bn_fwd_kernel<2>, dim3(1), dim3(kHeadWide), lds, s, z, gamma, beta, y, mean, rstd,
                           running_mean, running_var, num_batches, momentum, eps, N, J);
    }
    return check_launch();
}

int launch_head_bwd(const float *dy, const float *z, const float *pooled, const float *w, const float *gamma,
                    const float *mean, const float *rstd, float *dz, float *dx, float *dw, float *dgamma, float *dbeta,
                    int N, int C, int HW, int J, hipStream_t s) {
    if (!head_supported(N, C, HW, J)) return ADDER_ERR_UNSUPPORTED;
    const size_t lds = head_bwd_lds_bytes(N, C, J);
    if (J <= kHeadWaves) {
        if (int rc = allow_dynamic_lds<&head_bn_bwd_kernel<1>>((int)lds)) return rc;
        hipLaunchKernelGGL(head_bn_bwd_kernel<1>, dim3(1), dim3(kHeadWide), lds, s, dy, z, pooled, gamma, mean, rstd, dz,
                           dw, dgamma, dbeta, N, C, J);
    } else {
        if (int rc = allow_dynamic_lds<&head_bn_bwd_kernel<2>>((int)lds)) return rc;
        hipLaunchKernelGGL(head_bn_bwd_kernel<2>, dim3(1), dim3(kHeadWide), lds, s, dy, z, pooled, gamma, mean, rstd, dz,
                           dw, dgamma, dbeta, N, C, J);
    }
    if (dx) ADDER_HEAD_DISPATCH(launch_expand, dz, w, dx, N, C, J, s)
    return check_launch();
}

}  // namespace adder
