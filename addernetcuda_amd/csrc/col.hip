// Column-matrix entry points with the reference extension's exact contract:
//   X (K, NL), W (Co, K), out / gy (Co, NL), gW (Co, K), gX (K, NL); column
//   index nl = l*N + n as adder.py:33 lays it out (the kernels never look
//   inside nl, so any column order works).
// Replaces adder_cuda/adder.cu:19-70 (CONV), 72-131 (CONV_WEIGHT), 133-192
// (CONV_INPUT) and 194-272 (CONV_BACKWARD) for callers that already hold an
// unfolded X_col.  Gradients ACCUMULATE into their outputs, as the reference's
// atomicAdd kernels do into caller-zeroed buffers; the sums themselves are
// deterministic (fixed order, no atomics).
#include "common.hpp"

namespace adder {

// out[co, nl] = -sum_k |W[co,k] - X[k,nl]| : lane = column, TM rows of W per lane.
template <int TM>
__global__ __launch_bounds__(256) void col_fwd_kernel(const float *__restrict__ X,
                                                      const float *__restrict__ Wm,
                                                      float *__restrict__ out, int K, long NL, int Co) {
    long nl = (long)blockIdx.x * 256 + threadIdx.x;
    const bool active = nl < NL;
    if (!active) nl = NL - 1;
    const int co0 = blockIdx.y * TM;
    uniform_f32_ptr wc = as_uniform(Wm);
    int wrow[TM];
#pragma unroll
    for (int m = 0; m < TM; ++m) wrow[m] = min(co0 + m, Co - 1) * K;
    float acc[TM], tot[TM];   // two-level sum: acc holds at most 64 rows of X
#pragma unroll
    for (int m = 0; m < TM; ++m) acc[m] = tot[m] = 0.f;
    const float *xp = X + nl;
    int k = 0;
    for (; k + 4 <= K; k += 4) {
        if ((k & 63) == 0) {
#pragma unroll
            for (int m = 0; m < TM; ++m) { tot[m] += acc[m]; acc[m] = 0.f; }
        }
        float xv[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) xv[e] = xp[(size_t)(k + e) * NL];
#pragma unroll
        for (int m = 0; m < TM; ++m)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[m] -= fabsf(wc[wrow[m] + k + e] - xv[e]);
    }
    for (; k < K; ++k) {
        const float xv = xp[(size_t)k * NL];
#pragma unroll
        for (int m = 0; m < TM; ++m) acc[m] -= fabsf(wc[wrow[m] + k] - xv);
    }
    if (active) {
#pragma unroll
        for (int m = 0; m < TM; ++m)
            if (co0 + m < Co) out[(size_t)(co0 + m) * NL + nl] = tot[m] + acc[m];
    }
}

// gX[k, nl] += sum_co hardtanh(W[co,k] - X[k,nl]) * gy[co,nl] : lane = column, TK rows of X per lane.
template <int TK>
__global__ __launch_bounds__(256) void col_grad_x_kernel(const float *__restrict__ gy,
                                                         const float *__restrict__ X,
                                                         const float *__restrict__ Wm,
                                                         float *__restrict__ gX, int K, long NL, int Co) {
    long nl = (long)blockIdx.x * 256 + threadIdx.x;
    const bool active = nl < NL;
    if (!active) nl = NL - 1;
    const int k0 = blockIdx.y * TK;
    uniform_f32_ptr wc = as_uniform(Wm);
    float xv[TK], acc[TK], tot[TK];   // two-level sum: acc holds at most 64 rows of W
    int kk[TK];
#pragma unroll
    for (int t = 0; t < TK; ++t) {
        kk[t] = min(k0 + t, K - 1);
        xv[t] = X[(size_t)kk[t] * NL + nl];
        acc[t] = tot[t] = 0.f;
    }
    for (int co = 0; co < Co; ++co) {
        const float g = gy[(size_t)co * NL + nl];
#pragma unroll
        for (int t = 0; t < TK; ++t) acc[t] = fmaf(hardtanh(wc[co * K + kk[t]] - xv[t]), g, acc[t]);
        if ((co & 63) == 63) {
#pragma unroll
            for (int t = 0; t < TK; ++t) { tot[t] += acc[t]; acc[t] = 0.f; }
        }
    }
    if (active) {
#pragma unroll
        for (int t = 0; t < TK; ++t)
            if (k0 + t < K) gX[(size_t)(k0 + t) * NL + nl] += tot[t] + acc[t];
    }
}

// gW[co, k] += sum_nl (X[k,nl] - W[co,k]) * gy[co,nl] : one workgroup per TM x TK block of gW.
template <int TM, int TK>
__global__ __launch_bounds__(256) void col_grad_w_kernel(const float *__restrict__ gy,
                                                         const float *__restrict__ X,
                                                         const float *__restrict__ Wm,
                                                         float *__restrict__ gW, int K, long NL, int Co) {
    const int k0 = blockIdx.x * TK, co0 = blockIdx.y * TM;
    int kk[TK], cc[TM];
#pragma unroll
    for (int t = 0; t < TK; ++t) kk[t] = min(k0 + t, K - 1);
#pragma unroll
    for (int m = 0; m < TM; ++m) cc[m] = min(co0 + m, Co - 1);
    float wv[TM][TK], acc[TM][TK];
    double dacc[TM][TK];
#pragma unroll
    for (int m = 0; m < TM; ++m)
#pragma unroll
        for (int t = 0; t < TK; ++t) {
            wv[m][t] = Wm[(size_t)cc[m] * K + kk[t]];
            acc[m][t] = 0.f;
            dacc[m][t] = 0.0;
        }
    int it = 0;
    for (long nl = threadIdx.x; nl < NL; nl += 256) {
        float xv[TK], g[TM];
#pragma unroll
        for (int t = 0; t < TK; ++t) xv[t] = X[(size_t)kk[t] * NL + nl];
#pragma unroll
        for (int m = 0; m < TM; ++m) g[m] = gy[(size_t)cc[m] * NL + nl];
#pragma unroll
        for (int m = 0; m < TM; ++m)
#pragma unroll
            for (int t = 0; t < TK; ++t) acc[m][t] = fmaf(xv[t] - wv[m][t], g[m], acc[m][t]);
        if (++it == 64) {
#pragma unroll
            for (int m = 0; m < TM; ++m)
#pragma unroll
                for (int t = 0; t < TK; ++t) { dacc[m][t] += acc[m][t]; acc[m][t] = 0.f; }
            it = 0;
        }
    }
    __shared__ double red[4][TM * TK];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
    for (int m = 0; m < TM; ++m)
#pragma unroll
        for (int t = 0; t < TK; ++t) {
            const double s = wave_sum(dacc[m][t] + (double)acc[m][t]);
            if (lane == 0) red[wave][m * TK + t] = s;
        }
    __syncthreads();
    if (threadIdx.x < TM * TK) {
        const int m = threadIdx.x / TK, t = threadIdx.x % TK;
        if (co0 + m < Co && k0 + t < K) {
            const int e = threadIdx.x;
            gW[(size_t)(co0 + m) * K + k0 + t] += (float)((red[0][e] + red[1][e]) + (red[2][e] + red[3][e]));
        }
    }
}

int launch_col_fwd(const float *X, const float *Wm, float *out, int K, long NL, int Co, hipStream_t s) {
    constexpr int TM = 16;
    hipLaunchKernelGGL(col_fwd_kernel<TM>, dim3((unsigned)ceil_div_l(NL, 256), ceil_div(Co, TM)), dim3(256), 0, s,
                       X, Wm, out, K, NL, Co);
    return check_launch();
}

size_t col_grad_w_workspace_bytes(int, long, int) { return 0; }

int launch_col_grad_w(const float *gy, const float *X, const float *Wm, float *gW, int K, long NL, int Co,
                      void *, hipStream_t s) {
    constexpr int TM = 4, TK = 4;
    hipLaunchKernelGGL((col_grad_w_kernel<TM, TK>), dim3(ceil_div(K, TK), ceil_div(Co, TM)), dim3(256), 0, s, gy, X,
                       Wm, gW, K, NL, Co);
    return check_launch();
}

int launch_col_grad_x(const float *gy, const float *X, const float *Wm, float *gX, int K, long NL, int Co,
                      hipStream_t s) {
    constexpr int TK = 8;
    hipLaunchKernelGGL(col_grad_x_kernel<TK>, dim3((unsigned)ceil_div_l(NL, 256), ceil_div(K, TK)), dim3(256), 0, s,
                       gy, X, Wm, gX, K, NL, Co);
    return check_launch();
}

}  // namespace adder
