// Training-mode BatchNorm2d fused with the residual add and ReLU that follow every adder layer
// (resnet20.py:28-39: out = relu(bn(conv(x)) [+ residual])).  After the adder kernels these
// element-wise neighbours dominate a training step; they are HBM-bound, so the point of the fusion
// is to touch each activation as few times as possible:
//   forward   pass 1  per-channel sum / sum of squares (fp64 partials)    reads x
//             pass 2  y = relu(gamma * (x - mean) * rstd + beta + res)    reads x (+ res), writes y
//   backward  pass 1  per-channel sum(dz), sum(dz * xhat), dz = dy * [y > 0]      reads dy, y, x
//             pass 2  dx = gamma * rstd * (dz - mean(dz) - xhat * mean(dz * xhat)),
//                     dres = dz                                           reads dy, y, x, writes dx (+ dres)
// The backward needs y only for its sign, so the forward can leave a bit per element instead (relu_mask,
// planes of a multiple of 32 elements): word k holds the elements 32k .. 32k+31 of the tensor, which
// takes a quarter of the backward's read traffic away.
// Statistics follow torch.nn.BatchNorm2d: biased variance for normalisation, unbiased for running_var.
#include "common.hpp"

namespace adder {

static constexpr int kBnThreads = 256;

// V consecutive floats (V = 4 when HW is a multiple of 4, else 1)
template <int V> struct Pack { float v[V]; };
template <int V> __device__ __forceinline__ Pack<V> ld(const float *p, size_t i) {
    Pack<V> r;
    if constexpr (V == 4) {
        const float4 t = reinterpret_cast<const float4 *>(p)[i];
        r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w;
    } else {
        r.v[0] = p[i];
    }
    return r;
}
template <int V> __device__ __forceinline__ void st(float *p, size_t i, const Pack<V> &r) {
    if constexpr (V == 4) reinterpret_cast<float4 *>(p)[i] = make_float4(r.v[0], r.v[1], r.v[2], r.v[3]);
    else p[i] = r.v[0];
}

// Per-channel partial sums.  grid = (S, C); block (s, c) walks over the float4 groups
// i = s*256 + tid, s*256 + tid + S*256, ... of channel c (i = n * HW/4 + q).
// the four mask bits of float4 group `off` (V == 4 only)
__device__ __forceinline__ unsigned mask_nibble(const unsigned *__restrict__ mask, size_t off) {
    return mask[off >> 3] >> (4 * (unsigned)(off & 7));
}

template <bool BWD, int V>
__global__ __launch_bounds__(kBnThreads) void bn_partial_kernel(const float *__restrict__ x,
                                                                const float *__restrict__ dy,
                                                                const float *__restrict__ y,
                                                                const unsigned *__restrict__ mask,
                                                                const float *__restrict__ mean,
                                                                const float *__restrict__ rstd, int relu,
                                                                int N, int C, int HW4 /* HW / V */,
                                                                double *__restrict__ part) {
    const int c = blockIdx.y, S = gridDim.x;
    const int total = N * HW4;
    float mu = 0.f, rs = 0.f;
    if (BWD) { mu = mean[c]; rs = rstd[c]; }
    double a = 0.0, b = 0.0;
    for (int i0 = blockIdx.x * kBnThreads; i0 < total; i0 += S * kBnThreads) {
        const int i = i0 + threadIdx.x;
        float s1 = 0.f, s2 = 0.f;
        if (i < total) {
            const int n = i / HW4, q = i - n * HW4;
            const size_t off = ((size_t)n * C + c) * HW4 + q;
            const Pack<V> xv = ld<V>(x, off);
            if (!BWD) {
                // squares and sums in fp64: x * x is exact there, so E[x^2] - E[x]^2 keeps its digits when
                // |mean| >> std (a rounded fp32 square of x = -100 is already off by 5e-4)
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    const double xd = (double)xv.v[e];
                    a += xd;
                    b = fma(xd, xd, b);
                }
            } else {
                Pack<V> g = ld<V>(dy, off);
                if (relu && mask) {
                    const unsigned bits = mask_nibble(mask, off);
#pragma unroll
                    for (int e = 0; e < V; ++e) g.v[e] = (bits >> e) & 1u ? g.v[e] : 0.f;
                } else if (relu) {
                    const Pack<V> yv = ld<V>(y, off);
#pragma unroll
                    for (int e = 0; e < V; ++e) g.v[e] = yv.v[e] > 0.f ? g.v[e] : 0.f;
                }
#pragma unroll
                for (int e = 0; e < V; ++e) { s1 += g.v[e]; s2 = fmaf(g.v[e], (xv.v[e] - mu) * rs, s2); }
            }
        }
        a += (double)s1;   // backward: at most four elements per fp32 partial, everything above in fp64
        b += (double)s2;
    }
    __shared__ double ra[kBnThreads / 64], rb[kBnThreads / 64];
    a = wave_sum(a);
    b = wave_sum(b);
    if ((threadIdx.x & 63) == 0) { ra[threadIdx.x >> 6] = a; rb[threadIdx.x >> 6] = b; }
    __syncthreads();
    if (threadIdx.x == 0) {
        part[((size_t)c * S + blockIdx.x) * 2 + 0] = (ra[0] + ra[1]) + (ra[2] + ra[3]);
        part[((size_t)c * S + blockIdx.x) * 2 + 1] = (rb[0] + rb[1]) + (rb[2] + rb[3]);
    }
}

// Every workgroup of the second pass adds the S partials of its channel itself (same order in every
// workgroup, so all of them see the same statistics) instead of waiting for a finalize launch.
template <class T>
__device__ __forceinline__ void bn_reduce_partials(const T *__restrict__ part, int c, int S, double &s1,
                                                   double &s2) {
    double a = 0.0, b = 0.0;
    for (int s = threadIdx.x; s < S; s += kBnThreads) {
        a += (double)part[((size_t)c * S + s) * 2];
        b += (double)part[((size_t)c * S + s) * 2 + 1];
    }
    __shared__ double ra[kBnThreads / 64], rb[kBnThreads / 64];
    a = wave_sum(a);
    b = wave_sum(b);
    if ((threadIdx.x & 63) == 0) { ra[threadIdx.x >> 6] = a; rb[threadIdx.x >> 6] = b; }
    __syncthreads();
    s1 = (ra[0] + ra[1]) + (ra[2] + ra[3]);
    s2 = (rb[0] + rb[1]) + (rb[2] + rb[3]);
}

// Forward pass 2.  grid = (A, C); block (a, c) finishes the statistics of channel c and normalises the
// float4 groups a*256 + tid, a*256 + tid + A*256, ... of that channel.  Block (0, c) also stores
// mean / rstd for the backward pass and updates the running statistics; block (0, 0) advances
// num_batches_tracked (nullable), saving PyTorch a launch of its own.
template <int V>
__global__ __launch_bounds__(kBnThreads) void bn_apply_kernel(const float *__restrict__ x,
                                                              const float *__restrict__ res,
                                                              const double *__restrict__ part, int S, double count,
                                                              float eps, float momentum,
                                                              const float *__restrict__ gamma,
                                                              const float *__restrict__ beta, float *__restrict__ y,
                                                              unsigned *__restrict__ mask,
                                                              float *__restrict__ mean, float *__restrict__ rstd,
                                                              float *__restrict__ running_mean,
                                                              float *__restrict__ running_var,
                                                              long long *__restrict__ num_batches, int relu, int N,
                                                              int C, int HW4) {
    const int c = blockIdx.y;
    // The loads of the first PRE rounds are issued before the partial sums are added: they do not depend on the
    // statistics, and a workgroup that first waits for its 16 KB of partial sums and only then asks for its data
    // spends 1-2 us of a 5-11 us kernel with nothing in flight.
    constexpr int PRE = 4;
    const int total = N * HW4, i0 = blockIdx.x * kBnThreads + threadIdx.x, stride = gridDim.x * kBnThreads;
    Pack<V> pv[PRE], pr[PRE];
    size_t poff[PRE];
#pragma unroll
    for (int k = 0; k < PRE; ++k) {
        const int i = min(i0 + k * stride, total - 1), n = i / HW4, q = i - n * HW4;
        poff[k] = ((size_t)n * C + c) * HW4 + q;
        pv[k] = ld<V>(x, poff[k]);
#pragma unroll
        for (int e = 0; e < V; ++e) pr[k].v[e] = 0.f;
    }
    if (res) {
#pragma unroll
        for (int k = 0; k < PRE; ++k) pr[k] = ld<V>(res, poff[k]);
    }
    double s1, s2;
    bn_reduce_partials(part, c, S, s1, s2);
    const double mud = s1 / count;
    double var = s2 / count - mud * mud;
    if (var < 0.0) var = 0.0;
    const float mu = (float)mud, rs = (float)(1.0 / sqrt(var + (double)eps));
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        mean[c] = mu;
        rstd[c] = rs;
        if (running_mean) {
            const double unbiased = count > 1.0 ? var * count / (count - 1.0) : var;
            running_mean[c] = (float)((1.0 - momentum) * (double)running_mean[c] + momentum * mud);
            running_var[c] = (float)((1.0 - momentum) * (double)running_var[c] + momentum * unbiased);
        }
        if (c == 0 && num_batches) *num_batches += 1;
    }
    const float sc = gamma[c] * rs, sh = beta[c];
    auto emit = [&](const size_t off, const Pack<V> &v, const Pack<V> &r) {
        Pack<V> o;
#pragma unroll
        for (int e = 0; e < V; ++e) o.v[e] = fmaf(v.v[e] - mu, sc, sh);   // subtract first: |x| >> |x - mean| here
        if (res) {
#pragma unroll
            for (int e = 0; e < V; ++e) o.v[e] += r.v[e];
        }
        if (relu) {
            unsigned bits = 0;
#pragma unroll
            for (int e = 0; e < V; ++e) {
                if (o.v[e] > 0.f) bits |= 1u << e;
                o.v[e] = fmaxf(o.v[e], 0.f);
            }
            if (V == 4 && mask) {
                // planes are whole multiples of 8 float4 groups, so the eight lanes of an aligned group hold
                // the eight consecutive groups of one mask word and are all inside a round together
                unsigned w = bits << (4 * (unsigned)(off & 7));
                w |= __shfl_xor(w, 1, 64);
                w |= __shfl_xor(w, 2, 64);
                w |= __shfl_xor(w, 4, 64);
                if ((off & 7) == 0) mask[off >> 3] = w;
            }
        }
        st<V>(y, off, o);
    };
#pragma unroll
    for (int k = 0; k < PRE; ++k)
        if (i0 + k * stride < total) emit(poff[k], pv[k], pr[k]);
    for (int i = i0 + PRE * stride; i < total; i += stride) {
        const int n = i / HW4, q = i - n * HW4;
        const size_t off = ((size_t)n * C + c) * HW4 + q;
        const Pack<V> v = ld<V>(x, off);
        Pack<V> r = pr[0];   // (any value: not used without a residual)
        if (res) r = ld<V>(res, off);
        emit(off, v, r);
    }
}

// Backward pass 2, same grid.  Block (0, c) stores dgamma / dbeta.
template <int V>
__global__ __launch_bounds__(kBnThreads) void bn_bwd_apply_kernel(const float *__restrict__ dy,
                                                                  const float *__restrict__ y,
                                                                  const unsigned *__restrict__ mask,
                                                                  const float *__restrict__ x,
                                                                  const double *__restrict__ part, int S, double count,
                                                                  const float *__restrict__ mean,
                                                                  const float *__restrict__ rstd,
                                                                  const float *__restrict__ gamma,
                                                                  float *__restrict__ dx, float *__restrict__ dres,
                                                                  float *__restrict__ dgamma, float *__restrict__ dbeta,
                                                                  int relu, int N, int C, int HW4) {
    const int c = blockIdx.y;
    double s1, s2;
    bn_reduce_partials(part, c, S, s1, s2);
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        dbeta[c] = (float)s1;
        dgamma[c] = (float)s2;
    }
    const float m1 = (float)(s1 / count), m2 = (float)(s2 / count);   // mean(dz), mean(dz * xhat)
    const float mu = mean[c], rs = rstd[c], k = gamma[c] * rs;
    const int total = N * HW4;
    for (int i = blockIdx.x * kBnThreads + threadIdx.x; i < total; i += gridDim.x * kBnThreads) {
        const int n = i / HW4, q = i - n * HW4;
        const size_t off = ((size_t)n * C + c) * HW4 + q;
        Pack<V> g = ld<V>(dy, off);
        if (relu && mask) {
            const unsigned bits = mask_nibble(mask, off);
#pragma unroll
            for (int e = 0; e < V; ++e) g.v[e] = (bits >> e) & 1u ? g.v[e] : 0.f;
        } else if (relu) {
            const Pack<V> yv = ld<V>(y, off);
#pragma unroll
            for (int e = 0; e < V; ++e) g.v[e] = yv.v[e] > 0.f ? g.v[e] : 0.f;
        }
        if (dres) st<V>(dres, off, g);
        const Pack<V> v = ld<V>(x, off);
        Pack<V> o;
#pragma unroll
        for (int e = 0; e < V; ++e) o.v[e] = k * (g.v[e] - m1 - (v.v[e] - mu) * rs * m2);
        st<V>(dx, off, o);
    }
}

// The whole BatchNorm backward that is left when the neighbouring adder layers do the two passes inside their own
// kernels: one workgroup per channel adds the partial sums of dz and dz * xhat that the consumer's input-gradient
// kernel left (fixed order: the result does not depend on which workgroup finished first) and writes dbeta, dgamma
// and the four numbers per channel from which the producer's backward kernels form their output gradient,
//   dx = k * dz + c2 * (x - mean) - km1,   k = gamma * rstd, c2 = -k * rstd * mean(dz * xhat), km1 = k * mean(dz).
__global__ __launch_bounds__(kBnThreads) void bn_bwd_coef_kernel(const float *__restrict__ part, int S, double count,
                                                                 const float *__restrict__ gamma,
                                                                 const float *__restrict__ mean,
                                                                 const float *__restrict__ rstd,
                                                                 float *__restrict__ coef, float *__restrict__ dgamma,
                                                                 float *__restrict__ dbeta) {
    const int c = blockIdx.x;
    double s1, s2;
    bn_reduce_partials(part, c, S, s1, s2);
    if (threadIdx.x == 0) {
        dbeta[c] = (float)s1;
        dgamma[c] = (float)s2;
        const float m1 = (float)(s1 / count), m2 = (float)(s2 / count);
        const float rs = rstd[c], k = gamma[c] * rs;
        reinterpret_cast<float4 *>(coef)[c] = make_float4(k, -k * rs * m2, mean[c], k * m1);
    }
}

int launch_bn_bwd_coef(const float *part, int slots, const float *gamma, const float *mean, const float *rstd,
                       double count, float *coef, float *dgamma, float *dbeta, int C, hipStream_t s) {
    hipLaunchKernelGGL(bn_bwd_coef_kernel, dim3(C), dim3(kBnThreads), 0, s, part, slots, count, gamma, mean, rstd, coef,
                       dgamma, dbeta);
    return check_launch();
}

static int bn_splits(int N, int C, int HW4) {
    const long per_channel = (long)N * HW4;
    long s = 2048 / C;                                   // ~2048 workgroups over the chip
    const long cap = ceil_div_l(per_channel, 4L * kBnThreads);  // at least ~4 float4 per thread
    if (s > cap) s = cap;
    return (int)(s < 1 ? 1 : s);
}

static bool bn_vec4(int HW, const void *a, const void *b, const void *c, const void *d, const void *e) {
    const uintptr_t m = reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c) |
                        reinterpret_cast<uintptr_t>(d) | reinterpret_cast<uintptr_t>(e);
    return HW % 4 == 0 && (m & 15) == 0;
}

// words of the ReLU sign mask, or 0 where the shape has none (planes must be whole mask words)
size_t bn_mask_words(int N, int C, int HW) { return HW % 32 == 0 ? (size_t)N * C * HW / 32 : 0; }

size_t bn_workspace_bytes(int N, int C, int HW) {
    // sized for the scalar layout (the larger of the two) so the choice can depend on pointer alignment
    return ((size_t)C * bn_splits(N, C, HW) * 2 * sizeof(double) + 255) & ~(size_t)255;
}

// second-pass workgroups per channel: ~1024 over the chip (four per CU; every one of them first adds the
// channel's partial sums), at least one float4 group per thread
static int apply_splits(int N, int C, int HW4) {
    const long per_channel = (long)N * HW4;
    long a = ceil_div_l(1024, C);
    const long cap = ceil_div_l(per_channel, kBnThreads);
    if (a > cap) a = cap;
    return (int)(a < 1 ? 1 : a);
}

template <int V>
static int bn_fwd_v(const float *x, const float *res, const float *gamma, const float *beta, float *y, unsigned *mask,
                    float *mean, float *rstd, float *running_mean, float *running_var, long long *num_batches, float momentum,
                    float eps, int relu, int N, int C, int HW, void *ws, const double *stats, int stats_slots,
                    hipStream_t s) {
    const int HWV = HW / V;
    int S = stats_slots;
    const double *part = stats;
    if (!stats) {   // statistics pass of our own; otherwise the producer of x already wrote the partial sums
        S = bn_splits(N, C, HWV);
        double *own = reinterpret_cast<double *>(ws);
        hipLaunchKernelGGL((bn_partial_kernel<false, V>), dim3(S, C), dim3(kBnThreads), 0, s, x, nullptr, nullptr,
                           nullptr, nullptr, nullptr, 0, N, C, HWV, own);
        part = own;
    }
    hipLaunchKernelGGL(bn_apply_kernel<V>, dim3(apply_splits(N, C, HWV), C), dim3(kBnThreads), 0, s, x, res, part, S,
                       (double)N * HW, eps, momentum, gamma, beta, y, V == 4 ? mask : nullptr, mean, rstd, running_mean,
                       running_var, num_batches, relu, N, C, HWV);
    return check_launch();
}

// mask (nullable): bn_mask_words(N, C, HW) > 0 words that receive the sign bits of y; needs 16-byte aligned x, y, res
int launch_bn_act_fwd(const float *x, const float *res, const float *gamma, const float *beta, float *y,
                      unsigned *mask, float *mean, float *rstd, float *running_mean, float *running_var,
                      long long *num_batches, float momentum, float eps, int relu, int N, int C, int HW, void *ws,
                      const double *stats, int stats_slots, hipStream_t s) {
    if (bn_vec4(HW, x, res, y, nullptr, nullptr))
        return bn_fwd_v<4>(x, res, gamma, beta, y, mask, mean, rstd, running_mean, running_var, num_batches, momentum,
                           eps, relu, N, C, HW, ws, stats, stats_slots, s);
    if (mask) return ADDER_ERR_UNSUPPORTED;
    return bn_fwd_v<1>(x, res, gamma, beta, y, nullptr, mean, rstd, running_mean, running_var, num_batches, momentum,
                       eps, relu, N, C, HW, ws, stats, stats_slots, s);
}

template <int V>
static int bn_bwd_v(const float *dy, const float *y, const unsigned *mask, const float *x, const float *gamma, const float *mean,
                    const float *rstd, float *dx, float *dres, float *dgamma, float *dbeta, int relu, int N, int C,
                    int HW, void *ws, hipStream_t s) {
    const int HWV = HW / V, S = bn_splits(N, C, HWV);
    double *part = reinterpret_cast<double *>(ws);
    hipLaunchKernelGGL((bn_partial_kernel<true, V>), dim3(S, C), dim3(kBnThreads), 0, s, x, dy, y, mask, mean, rstd, relu,
                       N, C, HWV, part);
    hipLaunchKernelGGL(bn_bwd_apply_kernel<V>, dim3(apply_splits(N, C, HWV), C), dim3(kBnThreads), 0, s, dy, y, mask, x,
                       part, S, (double)N * HW, mean, rstd, gamma, dx, dres, dgamma, dbeta, relu, N, C, HWV);
    return check_launch();
}

// mask (nullable): the sign bits the forward left; replaces y
int launch_bn_act_bwd(const float *dy, const float *y, const unsigned *mask, const float *x, const float *gamma,
                      const float *mean, const float *rstd, float *dx, float *dres, float *dgamma, float *dbeta,
                      int relu, int N, int C, int HW, void *ws, hipStream_t s) {
    if (bn_vec4(HW, dy, y, x, dx, dres))
        return bn_bwd_v<4>(dy, y, mask, x, gamma, mean, rstd, dx, dres, dgamma, dbeta, relu, N, C, HW, ws, s);
    if (mask) return ADDER_ERR_UNSUPPORTED;
    return bn_bwd_v<1>(dy, y, nullptr, x, gamma, mean, rstd, dx, dres, dgamma, dbeta, relu, N, C, HW, ws, s);
}

}  // namespace adder
