/*
 * Plain-C restatement of the AdderNet convolution, indexing NCHW directly.
 *
 * TEST INFRASTRUCTURE ONLY: the shipped library never links or loads this.
 *
 * It deliberately shares no structure with the PyTorch restatement in
 * adder_oracle.py (no unfold, no column matrix): every output is a literal
 * loop nest over (n, co, ho, wo, ci, i, j), accumulated in double.  Agreement
 * between the two pins the im2col layout conventions of the reference
 * (adder.py:22-41: K-order (ci, i, j), zero padding taps that DO contribute
 * |w - 0|, floor output size) independently of F.unfold.
 *
 * Arithmetic followed:
 *   forward   out = -sum |w - x|                      adder_cuda/adder.cu:57-58, test_cuda.py:21
 *   grad_W    sum (x - w) * g                         adder_cuda/adder.cu:247,   test_cuda.py:39-40
 *   grad_X    sum hardtanh(w - x) * g, padding taps dropped   adder.cu:17,246, test_cuda.py:58-59
 *   eta scale g / max(||g||, 1e-12) * sqrt(numel) * eta        adder.py:78
 *
 * Inputs are float (what the kernels see); results are double so they can act
 * as ground truth for both fp32 implementations.
 */
#include <math.h>
#include <stddef.h>
#include <string.h>

static int out_dim(int h, int k, int p, int s) { return (h - k + 2 * p) / s + 1; }

static double hardtanh(double v) { return v < -1.0 ? -1.0 : (v <= 1.0 ? v : 1.0); }

int oracle_out_dim(int h, int k, int p, int s) { return out_dim(h, k, p, s); }

void oracle_conv2d_fwd(const float *x, const float *w, double *y,
                       int N, int Ci, int H, int W, int Co, int kh, int kw, int s, int p)
{
    const int Ho = out_dim(H, kh, p, s), Wo = out_dim(W, kw, p, s);
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; ++n)
        for (int co = 0; co < Co; ++co)
            for (int ho = 0; ho < Ho; ++ho)
                for (int wo = 0; wo < Wo; ++wo) {
                    double acc = 0.0;
                    for (int ci = 0; ci < Ci; ++ci)
                        for (int i = 0; i < kh; ++i)
                            for (int j = 0; j < kw; ++j) {
                                const int hi = ho * s + i - p, wi = wo * s + j - p;
                                const double xv = (hi >= 0 && hi < H && wi >= 0 && wi < W)
                                    ? (double)x[(((size_t)n * Ci + ci) * H + hi) * W + wi] : 0.0;
                                const double wv = w[(((size_t)co * Ci + ci) * kh + i) * kw + j];
                                acc -= fabs(wv - xv);
                            }
                    y[(((size_t)n * Co + co) * Ho + ho) * Wo + wo] = acc;
                }
}

void oracle_conv2d_grad_w(const float *gy, const float *x, const float *w, double *gw,
                          int N, int Ci, int H, int W, int Co, int kh, int kw, int s, int p)
{
    const int Ho = out_dim(H, kh, p, s), Wo = out_dim(W, kw, p, s);
#pragma omp parallel for collapse(2) schedule(static)
    for (int co = 0; co < Co; ++co)
        for (int ci = 0; ci < Ci; ++ci)
            for (int i = 0; i < kh; ++i)
                for (int j = 0; j < kw; ++j) {
                    const double wv = w[(((size_t)co * Ci + ci) * kh + i) * kw + j];
                    double acc = 0.0;
                    for (int n = 0; n < N; ++n)
                        for (int ho = 0; ho < Ho; ++ho)
                            for (int wo = 0; wo < Wo; ++wo) {
                                const int hi = ho * s + i - p, wi = wo * s + j - p;
                                const double xv = (hi >= 0 && hi < H && wi >= 0 && wi < W)
                                    ? (double)x[(((size_t)n * Ci + ci) * H + hi) * W + wi] : 0.0;
                                acc += (xv - wv) * (double)gy[(((size_t)n * Co + co) * Ho + ho) * Wo + wo];
                            }
                    gw[(((size_t)co * Ci + ci) * kh + i) * kw + j] = acc;
                }
}

void oracle_conv2d_grad_x(const float *gy, const float *x, const float *w, double *gx,
                          int N, int Ci, int H, int W, int Co, int kh, int kw, int s, int p)
{
    const int Ho = out_dim(H, kh, p, s), Wo = out_dim(W, kw, p, s);
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; ++n)
        for (int ci = 0; ci < Ci; ++ci) {
            double *plane = gx + ((size_t)n * Ci + ci) * H * W;
            memset(plane, 0, sizeof(double) * (size_t)H * W);
            for (int co = 0; co < Co; ++co)
                for (int ho = 0; ho < Ho; ++ho)
                    for (int wo = 0; wo < Wo; ++wo) {
                        const double g = gy[(((size_t)n * Co + co) * Ho + ho) * Wo + wo];
                        for (int i = 0; i < kh; ++i)
                            for (int j = 0; j < kw; ++j) {
                                const int hi = ho * s + i - p, wi = wo * s + j - p;
                                if (hi < 0 || hi >= H || wi < 0 || wi >= W) continue; /* fold drops padding */
                                const double xv = x[(((size_t)n * Ci + ci) * H + hi) * W + wi];
                                const double wv = w[(((size_t)co * Ci + ci) * kh + i) * kw + j];
                                plane[(size_t)hi * W + wi] += hardtanh(wv - xv) * g;
                            }
                    }
        }
}

void oracle_eta_scale(const double *g, double *out, size_t n, double eta)
{
    double ss = 0.0;
    for (size_t i = 0; i < n; ++i) ss += g[i] * g[i];
    double nrm = sqrt(ss);
    if (nrm < 1e-12) nrm = 1e-12;
    const double f = sqrt((double)n) * eta / nrm;
    for (size_t i = 0; i < n; ++i) out[i] = g[i] * f;
}

/* Column-matrix entry points: X (K, NL), W (Co, K), g/out (Co, NL). */
void oracle_col_fwd(const float *X, const float *W, double *out, int K, long NL, int Co)
{
#pragma omp parallel for schedule(static)
    for (int co = 0; co < Co; ++co)
        for (long nl = 0; nl < NL; ++nl) {
            double acc = 0.0;
            for (int k = 0; k < K; ++k) acc -= fabs((double)W[(size_t)co * K + k] - (double)X[(size_t)k * NL + nl]);
            out[(size_t)co * NL + nl] = acc;
        }
}

void oracle_col_grad_w(const float *g, const float *X, const float *W, double *gw, int K, long NL, int Co)
{
#pragma omp parallel for collapse(2) schedule(static)
    for (int co = 0; co < Co; ++co)
        for (int k = 0; k < K; ++k) {
            double acc = 0.0;
            const double wv = W[(size_t)co * K + k];
            for (long nl = 0; nl < NL; ++nl)
                acc += ((double)X[(size_t)k * NL + nl] - wv) * (double)g[(size_t)co * NL + nl];
            gw[(size_t)co * K + k] = acc;
        }
}

void oracle_col_grad_x(const float *g, const float *X, const float *W, double *gx, int K, long NL, int Co)
{
#pragma omp parallel for schedule(static)
    for (int k = 0; k < K; ++k)
        for (long nl = 0; nl < NL; ++nl) {
            double acc = 0.0;
            const double xv = X[(size_t)k * NL + nl];
            for (int co = 0; co < Co; ++co)
                acc += hardtanh((double)W[(size_t)co * K + k] - xv) * (double)g[(size_t)co * NL + nl];
            gx[(size_t)k * NL + nl] = acc;
        }
}
