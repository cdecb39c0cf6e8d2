// Weight gradient of the AdderNet convolution, NCHW, deterministic (no atomics):
//   gw[co,ci,i,j] = sum_{n,ho,wo} (xpad[n,ci,ho*s+i-p,wo*s+j-p] - w[co,ci,i,j]) * gy[n,co,ho,wo]
// followed (eta > 0) by the adaptive learning-rate scaling of adder.py:78,
//   gw <- gw / max(||gw||_2, 1e-12) * sqrt(numel) * eta.
// Replaces the grad_w half of adder_cuda/adder.cu:194-272 (CONV_BACKWARD),
// adder.cu:72-131 (CONV_WEIGHT) and the five elementwise kernels PyTorch
// launches for adder.py:78.
//
// The 3x3 and 1x1 kernels use  sum (x - w) g = sum x g - w * sum g : the first term is a
// plain (co) x (ci,i,j) matrix product over positions, the second needs only sum_g per
// output channel.  They write per-workgroup partial slabs (3x3: grad_w_mfma.hip, 1x1:
// conv1x1.hip); the finalize kernel in this file adds the slabs in fp64 and applies -w*sum_g.
#include "common.hpp"

namespace adder {

static constexpr int kNormBlocksMax = 16384;  // sum-of-squares partials kept at the head of the workspace

// ---------------------------------------------------------------------------
// Generic kernel: one workgroup per (co, ci) [KH x KW taps in registers] or,
// for KH = 0, one workgroup per (co, ci, i, j).  Direct (x - w) * g form.
// ---------------------------------------------------------------------------
template <int KH, int KW, class ST = float>
__global__ __launch_bounds__(256) void grad_w_generic_kernel(const ST *__restrict__ gy,
                                                             const ST *__restrict__ x,
                                                             const float *__restrict__ w,
                                                             float *__restrict__ gw, ConvDims d) {
    constexpr int T = KH > 0 ? KH * KW : 1;
    const int KK = d.kh * d.kw;
    int b = blockIdx.x;
    int tap0 = 0;
    if (KH == 0) { tap0 = b % KK; b /= KK; }
    const int ci = b % d.Ci, co = b / d.Ci;
    const float *wp = w + ((size_t)co * d.Ci + ci) * KK;
    float wv[T];
    int ti[T], tj[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        wv[t] = wp[tap0 + t];
        ti[t] = (tap0 + t) / d.kw;
        tj[t] = (tap0 + t) % d.kw;
    }
    float acc[T];
#pragma unroll
    for (int t = 0; t < T; ++t) acc[t] = 0.f;
    double dacc[T];
#pragma unroll
    for (int t = 0; t < T; ++t) dacc[t] = 0.0;

    const int L = d.Ho * d.Wo;
    const int total = d.N * L;
    int it = 0;
    for (int pos = threadIdx.x; pos < total; pos += 256) {
        const int l = pos % L, n = pos / L;
        const int ho = l / d.Wo, wo = l % d.Wo;
        const float g = ldf(gy + ((size_t)n * d.Co + co) * L + l);
        const ST *xp = x + ((size_t)n * d.Ci + ci) * d.H * d.W;
#pragma unroll
        for (int t = 0; t < T; ++t) {
            const int hi = ho * d.stride + ti[t] - d.pad, wi = wo * d.stride + tj[t] - d.pad;
            const bool v = hi >= 0 && hi < d.H && wi >= 0 && wi < d.W;
            const float xv = v ? ldf(xp + (size_t)hi * d.W + wi) : 0.f;
            acc[t] = fmaf(xv - wv[t], g, acc[t]);
        }
        if (++it == 64) {  // keep fp32 runs short; carry the rest in fp64
#pragma unroll
            for (int t = 0; t < T; ++t) { dacc[t] += acc[t]; acc[t] = 0.f; }
            it = 0;
        }
    }
    __shared__ double red[4][T];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
    for (int t = 0; t < T; ++t) {
        const double s = wave_sum(dacc[t] + (double)acc[t]);
        if (lane == 0) red[wave][t] = s;
    }
    __syncthreads();
    if (threadIdx.x < T) {
        const int t = threadIdx.x;
        gw[((size_t)co * d.Ci + ci) * KK + tap0 + t] = (float)(red[0][t] + red[1][t] + red[2][t] + red[3][t]);
    }
}

// ---------------------------------------------------------------------------
// Finalize: gw = sum_slots part - w * sum_slots sgpart, plus the per-block sums of
// squares the scaling kernel needs.  A workgroup finishes kFinOut outputs: thread
// (sl, o) adds slots sl, sl+kFinLanes, ... of output o in fp64, so the dependent
// chain is slots/kFinLanes long.
// ---------------------------------------------------------------------------
static constexpr int kFinOut = 16, kFinLanes = 16;   // a wave reads four full 64-byte runs per slot row
static constexpr int kFinThreads = kFinOut * kFinLanes;
// The batched finalize picks the block shape per layer: layers with few slabs give a workgroup more outputs (32 x 8
// or 64 x 4 threads), so that every thread still has a few loads in flight and a layer with 16 slabs does not need
// four times the workgroups of one with 256.
__host__ __device__ inline int fin_out_for(int slots) { return slots >= 128 ? 16 : (slots >= 32 ? 32 : 64); }
// ACC: the result is added to gw (the column-matrix entry points accumulate, as the reference's atomicAdd does).
// fo: outputs per workgroup (16, 32 or 64); kFinThreads / fo threads share the slots of an output.
template <typename PT, bool ACC = false>
__device__ __forceinline__ void grad_w_finalize_block(const PT *__restrict__ part, const PT *__restrict__ sgpart,
                                                      const float *__restrict__ w, float *__restrict__ gw,
                                                      double *__restrict__ ss, int slots, int Co, int K, int block,
                                                      const int fo = kFinOut) {
    const int kFinOut = fo, kFinLanes = kFinThreads / fo;   // (the names of the fixed shape, for this workgroup's)
    const int o = threadIdx.x % kFinOut, sl = threadIdx.x / kFinOut;
    const int total = Co * K;
    const int idx = block * kFinOut + o;
    const int idc = idx < total ? idx : total - 1;
    const int co = idc / K;
    // four slots per round, so that eight loads are in flight per thread (the loop is latency-bound)
    double a4[4] = {0.0, 0.0, 0.0, 0.0}, s4[4] = {0.0, 0.0, 0.0, 0.0};
    int p = sl;
    for (; p + 3 * kFinLanes < slots; p += 4 * kFinLanes) {
        PT va[4], vs[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            va[u] = part[(size_t)(p + u * kFinLanes) * total + idc];
            vs[u] = sgpart[(size_t)(p + u * kFinLanes) * Co + co];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) { a4[u] += (double)va[u]; s4[u] += (double)vs[u]; }
    }
    for (; p < slots; p += kFinLanes) {
        a4[0] += (double)part[(size_t)p * total + idc];
        s4[0] += (double)sgpart[(size_t)p * Co + co];
    }
    const double a = (a4[0] + a4[1]) + (a4[2] + a4[3]), sgs = (s4[0] + s4[1]) + (s4[2] + s4[3]);
    __shared__ double ra[kFinThreads + 16], rs[kFinThreads + 16];   // [lane][output], rows one element apart in banks
    ra[sl * (kFinOut + 1) + o] = a;
    rs[sl * (kFinOut + 1) + o] = sgs;
    __syncthreads();
    if (threadIdx.x < kFinOut) {
        double ta = 0.0, ts = 0.0;
        for (int k = 0; k < kFinLanes; ++k) { ta += ra[k * (kFinOut + 1) + o]; ts += rs[k * (kFinOut + 1) + o]; }
        double v = 0.0;
        if (idx < total) {
            float r = (float)(w ? ta - (double)w[idx] * ts : ta);   // no weights: the plain sum of x * gy
            if constexpr (ACC) r += gw[idx];
            gw[idx] = r;
            v = (double)r * (double)r;
        }
        for (int off = kFinOut / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
        if (threadIdx.x == 0 && ss) ss[block] = v;
    }
}

template <typename PT, bool ACC = false>
__global__ __launch_bounds__(kFinOut * kFinLanes) void grad_w_finalize_kernel(const PT *__restrict__ part,
                                                                              const PT *__restrict__ sgpart,
                                                                              const float *__restrict__ w,
                                                                              float *__restrict__ gw,
                                                                              double *__restrict__ ss, int slots,
                                                                              int Co, int K) {
    grad_w_finalize_block<PT, ACC>(part, sgpart, w, gw, ss, slots, Co, K, blockIdx.x, fin_out_for(slots));
}

// gw (+)= sum of `slots` fp64 slabs - w * sum of the gy partials: the finalize on its own, for the column-matrix path
int launch_grad_w_slab_finalize(const double *part, const double *sgpart, const float *w, float *gw, int slots, int Co,
                                int K, bool accumulate, hipStream_t s) {
    const int nb = (int)ceil_div_l((long)Co * K, fin_out_for(slots));
    if (accumulate)
        hipLaunchKernelGGL((grad_w_finalize_kernel<double, true>), dim3(nb), dim3(kFinOut * kFinLanes), 0, s, part, sgpart,
                           w, gw, nullptr, slots, Co, K);
    else
        hipLaunchKernelGGL((grad_w_finalize_kernel<double, false>), dim3(nb), dim3(kFinOut * kFinLanes), 0, s, part, sgpart,
                           w, gw, nullptr, slots, Co, K);
    return check_launch();
}

// The finalize of up to kGwFinishMax layers in one launch and their scaling in a second: for callers that
// leave the partial slabs of every layer in its workspace during the backward pass and finish all weight
// gradients together at its end.  The finalize grid is the concatenation of the layers' own grids
// (first[t] = first workgroup of layer t); the scaling grid is (P, layers).
struct GwStageBatch {
    adder_grad_w_stage it[kGwFinishMax];
    int first[kGwFinishMax + 1];
    int count;
};

__global__ __launch_bounds__(kFinOut * kFinLanes) void batch_finalize_kernel(const GwStageBatch b,
                                                                             double *__restrict__ ss) {
    int t = 0;
    while (t + 1 < b.count && (int)blockIdx.x >= b.first[t + 1]) ++t;   // wave-uniform, at most 31 steps
    const adder_grad_w_stage &it = b.it[t];
    const int block = blockIdx.x - b.first[t];
    double *mine = ss + b.first[t];
    const int fo = fin_out_for(it.slots);
    if (it.fp64)
        grad_w_finalize_block<double>(static_cast<const double *>(it.part), static_cast<const double *>(it.sgpart), it.w,
                                      it.gw, mine, it.slots, it.Co, it.K, block, fo);
    else
        grad_w_finalize_block<float>(static_cast<const float *>(it.part), static_cast<const float *>(it.sgpart), it.w,
                                     it.gw, mine, it.slots, it.Co, it.K, block, fo);
}

__global__ __launch_bounds__(256) void batch_finish_scale_kernel(const GwStageBatch b, const double *__restrict__ ss,
                                                                 float eps) {
    const int t = blockIdx.y;
    const adder_grad_w_stage &it = b.it[t];
    if (!(it.eta > 0.f)) return;   // left raw
    const long n = (long)it.Co * it.K;
    __shared__ double red[4];
    double v = 0.0;
    for (int i = b.first[t] + threadIdx.x; i < b.first[t + 1]; i += 256) v += ss[i];
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    const double total = (red[0] + red[1]) + (red[2] + red[3]);
    float nrm = (float)sqrt(total);   // same fp32 steps as norm_scale_kernel
    nrm = fmaxf(nrm, eps);
    const float rt = sqrtf((float)n);
    float *g = it.gw;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256)
        g[i] = g[i] / nrm * rt * it.eta;
}

// ---------------------------------------------------------------------------
// Adaptive scaling (adder.py:78): g <- g / max(||g||_2, eps) * sqrt(n) * eta.
// Two launches: per-block sums of squares (fp64), then every block re-adds the
// partials in the same order and scales its slice.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void sumsq_kernel(const float *__restrict__ g, long n,
                                                    double *__restrict__ ss) {
    double v = 0.0;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
        const double t = g[i];
        v += t * t;
    }
    __shared__ double red[4];
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    if (threadIdx.x == 0) ss[blockIdx.x] = (red[0] + red[1]) + (red[2] + red[3]);
}

__global__ __launch_bounds__(256) void norm_scale_kernel(float *__restrict__ g, long n,
                                                         const double *__restrict__ ss, int nss, float eta,
                                                         float eps) {
    __shared__ double red[4];
    double v = 0.0;
    for (int i = threadIdx.x; i < nss; i += 256) v += ss[i];
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    const double total = (red[0] + red[1]) + (red[2] + red[3]);
    // fp32 steps in the order adder.py:78 applies them: / norm, * sqrt(n), * eta
    float nrm = (float)sqrt(total);
    nrm = fmaxf(nrm, eps);
    const float rt = sqrtf((float)n);
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256)
        g[i] = g[i] / nrm * rt * eta;
}

size_t norm_scale_workspace_bytes(long) { return sizeof(double) * kNormBlocksMax; }

// ---------------------------------------------------------------------------
// The same scaling for up to kNormBatchMax tensors at once (every adder layer of a network after its
// backward pass): two launches in all instead of one or two per layer.  grid = (P, count); block (p, t)
// handles a slice of tensor t.  The tensor table travels by value in the kernel arguments.
// ---------------------------------------------------------------------------
struct NormBatch {
    float *g[kNormBatchMax];
    long n[kNormBatchMax];
    float eta[kNormBatchMax];
};

__global__ __launch_bounds__(256) void batch_sumsq_kernel(const NormBatch b, double *__restrict__ ss) {
    const int t = blockIdx.y;
    const float *g = b.g[t];
    const long n = b.n[t];
    double v = 0.0;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
        const double e = g[i];
        v += e * e;
    }
    __shared__ double red[4];
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    if (threadIdx.x == 0) ss[(size_t)t * gridDim.x + blockIdx.x] = (red[0] + red[1]) + (red[2] + red[3]);
}

__global__ __launch_bounds__(256) void batch_norm_scale_kernel(const NormBatch b, const double *__restrict__ ss,
                                                               float eps) {
    const int t = blockIdx.y, P = gridDim.x;
    __shared__ double red[4];
    double v = 0.0;
    for (int i = threadIdx.x; i < P; i += 256) v += ss[(size_t)t * P + i];
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    const double total = (red[0] + red[1]) + (red[2] + red[3]);
    float *g = b.g[t];
    const long n = b.n[t];
    const float eta = b.eta[t];
    float nrm = (float)sqrt(total);   // same fp32 steps as norm_scale_kernel
    nrm = fmaxf(nrm, eps);
    const float rt = sqrtf((float)n);
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256)
        g[i] = g[i] / nrm * rt * eta;
}

static int batch_blocks(int count, const long *n) {
    long most = 1;
    for (int t = 0; t < count; ++t) most = n[t] > most ? n[t] : most;
    const long p = ceil_div_l(most, 2048);   // ~8 elements per thread for the largest tensor
    return (int)(p < 1 ? 1 : (p > 256 ? 256 : p));
}

size_t norm_scale_batched_workspace_bytes(int count) { return sizeof(double) * 256 * (size_t)count; }

int launch_norm_scale_batched(int count, float *const *g, const long *n, const float *eta, float eps, void *ws,
                              hipStream_t s) {
    NormBatch b{};
    for (int t = 0; t < count; ++t) { b.g[t] = g[t]; b.n[t] = n[t]; b.eta[t] = eta[t]; }
    const int P = batch_blocks(count, n);
    double *ss = reinterpret_cast<double *>(ws);
    hipLaunchKernelGGL(batch_sumsq_kernel, dim3(P, count), dim3(256), 0, s, b, ss);
    hipLaunchKernelGGL(batch_norm_scale_kernel, dim3(P, count), dim3(256), 0, s, b, ss, eps);
    return check_launch();
}

static int norm_blocks(long n) {
    long b = ceil_div_l(n, 1024);
    return (int)(b < 1 ? 1 : (b > kNormBlocksMax ? kNormBlocksMax : b));
}

int launch_norm_scale(float *g, long n, float eta, float eps, void *ws, hipStream_t s) {
    double *ss = reinterpret_cast<double *>(ws);
    const int nb = norm_blocks(n);
    hipLaunchKernelGGL(sumsq_kernel, dim3(nb), dim3(256), 0, s, g, n, ss);
    hipLaunchKernelGGL(norm_scale_kernel, dim3(nb), dim3(256), 0, s, g, n, ss, nb, eta, eps);
    return check_launch();
}

// ---- dispatch -----------------------------------------------------------------
struct GradWPlan {
    int variant;  // 0 generic, 1 1x1 kernel (fp32 partial slabs), 2 3x3 matrix-core kernel (fp64 partial slabs)
    GradWMfmaPlan mfma;
    int slots;
};

static GradWPlan plan_grad_w(const ConvDims &d) {
    GradWPlan p{};
    const long partial_cap = 1L << 28;  // partial slab elements
    p.mfma = plan_grad_w_mfma(d);
    if (p.mfma.variant) {
        p.variant = 2;
        p.slots = p.mfma.slots;
    } else if (conv1x1_supported(d, nullptr, nullptr)) {
        p.variant = 1;
        p.slots = grad_w_1x1_slots(d);
    }
    if (p.variant && (long)p.slots * d.Co * d.K() > partial_cap) p.variant = 0;
    return p;
}

// whether launch_grad_w / launch_grad_w_staged take the BatchNorm link for this layer and these tensors
bool grad_w_bn_supported(const ConvDims &d, const void *gy, const void *x, const void *bn_y, const void *bn_coef) {
    const GradWPlan p = plan_grad_w(d);
    const uintptr_t align = reinterpret_cast<uintptr_t>(gy) | reinterpret_cast<uintptr_t>(x) |
                            reinterpret_cast<uintptr_t>(bn_y) | reinterpret_cast<uintptr_t>(bn_coef);
    const int v = p.mfma.variant;
    const bool k3 = ((v >= 1 && v <= 5) || v == 14) && d.W % 4 == 0 && d.Wo % 4 == 0;
    const bool k1 = (v == 6 || v == 7 || v == 10 || v == 12) && d.stride == 1 && (d.H * d.W) % 4 == 0;
    return p.variant == 2 && (k3 || k1) && (align & 15) == 0;
}

size_t grad_w_workspace_bytes(const ConvDims &d) {
    const GradWPlan p = plan_grad_w(d);
    size_t bytes = sizeof(double) * kNormBlocksMax;
    if (p.variant)
        bytes += (p.variant == 2 ? sizeof(double) : sizeof(float)) * (size_t)p.slots * ((size_t)d.Co * d.K() + d.Co);
    return (bytes + 255) & ~(size_t)255;
}

// bn_y with either bn_coef or sums.part: gy is the gradient dz of the output of the BatchNorm behind the layer and
// the kernel forms the layer's own output gradient from it, leaving it in gy_out (nullable) on the way (matrix-core
// kernels only: ADDER_ERR_UNSUPPORTED, nothing launched, elsewhere)
int launch_grad_w(const float *gy, const float *x, const float *w, float *gw, float eta, void *ws,
                  size_t ws_bytes, const ConvDims &d, hipStream_t s, const float *bn_y, const float *bn_coef,
                  float *gy_out, const BnSums &sums) {
    if (ws_bytes < grad_w_workspace_bytes(d)) return ADDER_ERR_WORKSPACE;
    GradWPlan p = plan_grad_w(d);
    if (bn_y && !grad_w_bn_supported(d, gy, x, bn_y, bn_coef ? (const void *)bn_coef : (const void *)sums.part))
        return ADDER_ERR_UNSUPPORTED;
    // float4 loads need 16-byte aligned bases; tensors whose rows are read element by element do not
    // (1x1 layers on the matrix cores walk whole planes as rows: their row length is H*W)
    const bool rows_1x1 = p.variant == 2 && d.kh == 1;
    const bool need_x16 = p.variant == 2 && !(rows_1x1 && d.stride > 1) &&   // (a strided 1x1 layer samples x element-wise)
                          (rows_1x1 ? d.H * d.W : d.W) % 4 == 0;
    const bool need_g16 = p.variant == 2 && (rows_1x1 ? d.Ho * d.Wo : d.Wo) % 4 == 0;
    if (p.variant && ((need_x16 && (reinterpret_cast<uintptr_t>(x) & 15)) ||
                      (need_g16 && (reinterpret_cast<uintptr_t>(gy) & 15))))
        p.variant = 0;
    double *ss = reinterpret_cast<double *>(ws);
    const int K = d.K();
    const long n = (long)d.Co * K;
    if (p.variant) {
        const int nb = (int)ceil_div_l(n, fin_out_for(p.slots));
        const bool fused_norm = eta > 0.f && nb <= kNormBlocksMax;
        int rc;
        if (p.variant == 2) {
            double *part = reinterpret_cast<double *>(ss + kNormBlocksMax);
            double *sgpart = part + (size_t)p.slots * d.Co * K;
            rc = bn_y ? launch_grad_w_mfma_bn(gy, x, part, sgpart, d, p.mfma, bn_y, bn_coef, gy_out, s, sums)
                      : launch_grad_w_mfma(gy, x, part, sgpart, d, p.mfma, s);
            if (rc) return rc;
            hipLaunchKernelGGL(grad_w_finalize_kernel<double>, dim3(nb), dim3(kFinOut * kFinLanes), 0, s, part,
                               sgpart, w, gw, fused_norm ? ss : nullptr, p.slots, d.Co, K);
        } else {
            float *part = reinterpret_cast<float *>(ss + kNormBlocksMax);
            float *sgpart = part + (size_t)p.slots * d.Co * K;
            rc = launch_grad_w_1x1(gy, x, part, sgpart, p.slots, d, s);
            if (rc) return rc;
            hipLaunchKernelGGL(grad_w_finalize_kernel<float>, dim3(nb), dim3(kFinOut * kFinLanes), 0, s, part,
                               sgpart, w, gw, fused_norm ? ss : nullptr, p.slots, d.Co, K);
        }
        if (fused_norm)
            hipLaunchKernelGGL(norm_scale_kernel, dim3(norm_blocks(n)), dim3(256), 0, s, gw, n, ss, nb, eta,
                               1e-12f);
        rc = check_launch();
        if (rc || fused_norm || !(eta > 0.f)) return rc;
        return launch_norm_scale(gw, n, eta, 1e-12f, ws, s);
    }
    const int KK = d.kh * d.kw;
    const long wgs = (long)d.Co * d.Ci;
    if (d.kh == 3 && d.kw == 3)
        hipLaunchKernelGGL((grad_w_generic_kernel<3, 3>), dim3((unsigned)wgs), dim3(256), 0, s, gy, x, w, gw, d);
    else if (d.kh == 1 && d.kw == 1)
        hipLaunchKernelGGL((grad_w_generic_kernel<1, 1>), dim3((unsigned)wgs), dim3(256), 0, s, gy, x, w, gw, d);
    else
        hipLaunchKernelGGL((grad_w_generic_kernel<0, 0>), dim3((unsigned)(wgs * KK)), dim3(256), 0, s, gy, x, w,
                           gw, d);
    int rc = check_launch();
    if (rc) return rc;
    if (eta > 0.f) return launch_norm_scale(gw, n, eta, 1e-12f, ws, s);
    return ADDER_OK;
}

// bfloat16 storage of gy and x (gw and w stay fp32): the matrix-core kernel for 3x3 / pad-1 layers, the generic
// kernel for everything else; the same finalize and scaling as the fp32 path
int launch_grad_w_bf16(const bf16_t *gy, const bf16_t *x, const float *w, float *gw, float eta, void *ws,
                       size_t ws_bytes, const ConvDims &d, hipStream_t s) {
    if (ws_bytes < grad_w_workspace_bytes(d)) return ADDER_ERR_WORKSPACE;
    GradWPlan p = plan_grad_w(d);
    const bool tiled = p.variant == 2 && d.kh == 3 && (d.W % 4 != 0 || (reinterpret_cast<uintptr_t>(x) & 7) == 0) &&
                       (d.Wo % 4 != 0 || (reinterpret_cast<uintptr_t>(gy) & 7) == 0);
    double *ss = reinterpret_cast<double *>(ws);
    const int K = d.K();
    const long n = (long)d.Co * K;
    if (tiled) {
        double *part = reinterpret_cast<double *>(ss + kNormBlocksMax);
        double *sgpart = part + (size_t)p.slots * d.Co * K;
        if (int rc = launch_grad_w_mfma_bf16(gy, x, part, sgpart, d, p.mfma, s)) return rc;
        const int nb = (int)ceil_div_l(n, fin_out_for(p.slots));
        hipLaunchKernelGGL(grad_w_finalize_kernel<double>, dim3(nb), dim3(kFinOut * kFinLanes), 0, s, part, sgpart, w, gw,
                           nullptr, p.slots, d.Co, K);
    } else {
        const int KK = d.kh * d.kw;
        const long wgs = (long)d.Co * d.Ci;
        if (d.kh == 3 && d.kw == 3)
            hipLaunchKernelGGL((grad_w_generic_kernel<3, 3, bf16_t>), dim3((unsigned)wgs), dim3(256), 0, s, gy, x, w, gw, d);
        else if (d.kh == 1 && d.kw == 1)
            hipLaunchKernelGGL((grad_w_generic_kernel<1, 1, bf16_t>), dim3((unsigned)wgs), dim3(256), 0, s, gy, x, w, gw, d);
        else
            hipLaunchKernelGGL((grad_w_generic_kernel<0, 0, bf16_t>), dim3((unsigned)(wgs * KK)), dim3(256), 0, s, gy, x, w,
                               gw, d);
    }
    if (int rc = check_launch()) return rc;
    if (eta > 0.f) return launch_norm_scale(gw, n, eta, 1e-12f, ws, s);
    return ADDER_OK;
}

// ---- staged weight gradient: partial slabs now, finalize + scaling for many layers later --------------
int launch_grad_w_staged(const float *gy, const float *x, const float *w, float *gw, float eta, void *ws,
                         size_t ws_bytes, const ConvDims &d, adder_grad_w_stage *stage, hipStream_t s,
                         const float *bn_y, const float *bn_coef, float *gy_out, const BnSums &sums) {
    if (ws_bytes < grad_w_workspace_bytes(d)) return ADDER_ERR_WORKSPACE;
    GradWPlan p = plan_grad_w(d);
    if (bn_y && !grad_w_bn_supported(d, gy, x, bn_y, bn_coef ? (const void *)bn_coef : (const void *)sums.part))
        return ADDER_ERR_UNSUPPORTED;
    const bool rows_1x1 = p.variant == 2 && d.kh == 1;
    const bool need_x16 = p.variant == 2 && !(rows_1x1 && d.stride > 1) && (rows_1x1 ? d.H * d.W : d.W) % 4 == 0;
    const bool need_g16 = p.variant == 2 && (rows_1x1 ? d.Ho * d.Wo : d.Wo) % 4 == 0;
    if (!p.variant || (need_x16 && (reinterpret_cast<uintptr_t>(x) & 15)) ||
        (need_g16 && (reinterpret_cast<uintptr_t>(gy) & 15)))
        return ADDER_ERR_UNSUPPORTED;   // no slab-based kernel for this layer: nothing to stage
    double *ss = reinterpret_cast<double *>(ws);
    const int K = d.K();
    int rc;
    if (p.variant == 2) {
        double *part = reinterpret_cast<double *>(ss + kNormBlocksMax);
        double *sgpart = part + (size_t)p.slots * d.Co * K;
        rc = bn_y ? launch_grad_w_mfma_bn(gy, x, part, sgpart, d, p.mfma, bn_y, bn_coef, gy_out, s, sums)
                  : launch_grad_w_mfma(gy, x, part, sgpart, d, p.mfma, s);
        stage->part = part;
        stage->sgpart = sgpart;
    } else {
        float *part = reinterpret_cast<float *>(ss + kNormBlocksMax);
        float *sgpart = part + (size_t)p.slots * d.Co * K;
        rc = launch_grad_w_1x1(gy, x, part, sgpart, p.slots, d, s);
        stage->part = part;
        stage->sgpart = sgpart;
    }
    stage->w = w;
    stage->gw = gw;
    stage->slots = p.slots;
    stage->Co = d.Co;
    stage->K = K;
    stage->fp64 = p.variant == 2;
    stage->eta = eta;
    return rc;
}

static long finish_blocks(int count, const adder_grad_w_stage *st) {
    long total = 0;
    for (int t = 0; t < count; ++t) total += ceil_div(st[t].Co * st[t].K, fin_out_for(st[t].slots));
    return total;
}

size_t grad_w_finish_workspace_bytes(int count, const adder_grad_w_stage *st) {
    return ((size_t)finish_blocks(count, st) * sizeof(double) + 255) & ~(size_t)255;
}

int launch_grad_w_finish(int count, const adder_grad_w_stage *st, void *ws, hipStream_t s) {
    GwStageBatch b{};
    long most_n = 1;
    b.count = count;
    for (int t = 0; t < count; ++t) {
        b.it[t] = st[t];
        b.first[t + 1] = b.first[t] + ceil_div(st[t].Co * st[t].K, fin_out_for(st[t].slots));
        const long n = (long)st[t].Co * st[t].K;
        most_n = n > most_n ? n : most_n;
    }
    if (finish_blocks(count, st) > 0x7fffffffL) return ADDER_ERR_TOO_LARGE;
    double *ss = reinterpret_cast<double *>(ws);
    hipLaunchKernelGGL(batch_finalize_kernel, dim3((unsigned)b.first[count]), dim3(kFinOut * kFinLanes), 0, s, b, ss);
    long P = ceil_div_l(most_n, 2048);
    P = P < 1 ? 1 : (P > 256 ? 256 : P);
    hipLaunchKernelGGL(batch_finish_scale_kernel, dim3((unsigned)P, count), dim3(256), 0, s, b, ss, 1e-12f);
    return check_launch();
}

}  // namespace adder
