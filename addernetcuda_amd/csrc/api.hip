// C ABI of libaddernet_hip.so: argument validation and dispatch.  Every check
// that can fail does so before the first HIP call, so the error paths can be
// exercised on a machine without a GPU.
#include "common.hpp"

#include <atomic>
#include <cstdlib>
#include <string>

namespace adder {

static thread_local std::string g_last_hip_error;

int record_hip_error(hipError_t e) {
    g_last_hip_error = hipGetErrorString(e);
    return ADDER_ERR_HIP;
}

int check_launch() {
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? ADDER_OK : record_hip_error(e);
}

static const long kMaxElems = 0x7fffffffL;

// Scratch of the allocation-free backward (adder_conv2d_bwd_noalloc_f32): part of the device image, one copy per
// GPU.  In host code `scratch` is only a handle for hipGetSymbolAddress -- never a device address; the address
// each device gives its copy is looked up once per device and kept in g_scratch.
static __device__ __align__(256) unsigned char scratch[ADDER_NOALLOC_SCRATCH_BYTES];
static constexpr int kMaxDevices = 64;
static std::atomic<void *> g_scratch[kMaxDevices];

// Device address of the current device's copy of `scratch`.
static int scratch_of_current_device(void **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return record_hip_error(e);
    if (dev < 0 || dev >= kMaxDevices) return ADDER_ERR_UNSUPPORTED;
    void *p = g_scratch[dev].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));   // the address on the device that is current now
        if (e != hipSuccess) return record_hip_error(e);
        if (!p) return ADDER_ERR_HIP;
        g_scratch[dev].store(p, std::memory_order_release);   // two threads racing here store the same address
    }
    *out = p;
    return ADDER_OK;
}

static int make_dims(int N, int Ci, int H, int W, int Co, int kh, int kw, int stride, int pad, ConvDims &d) {
    if (N <= 0 || Ci <= 0 || H <= 0 || W <= 0 || Co <= 0 || kh <= 0 || kw <= 0 || stride <= 0 || pad < 0)
        return ADDER_ERR_BAD_SHAPE;
    if (H + 2 * pad < kh || W + 2 * pad < kw) return ADDER_ERR_BAD_SHAPE;
    d = ConvDims{N, Ci, H, W, Co, kh, kw, stride, pad, (H - kh + 2 * pad) / stride + 1,
                 (W - kw + 2 * pad) / stride + 1};
    const long nx = (long)N * Ci * H * W, ny = (long)N * Co * d.Ho * d.Wo, nw = (long)Co * Ci * kh * kw;
    if (nx > kMaxElems || ny > kMaxElems || nw > kMaxElems) return ADDER_ERR_TOO_LARGE;
    return ADDER_OK;
}

static bool overlaps(const void *a, size_t na, const void *b, size_t nb) {
    if (!a || !b) return false;
    const uintptr_t pa = reinterpret_cast<uintptr_t>(a), pb = reinterpret_cast<uintptr_t>(b);
    return pa < pb + nb && pb < pa + na;
}

struct Span { const void *p; size_t bytes; };

// no output may overlap an input or another output
template <int NO, int NI>
static bool any_alias(const Span (&outs)[NO], const Span (&ins)[NI]) {
    for (int o = 0; o < NO; ++o) {
        for (int i = 0; i < NI; ++i)
            if (overlaps(outs[o].p, outs[o].bytes, ins[i].p, ins[i].bytes)) return true;
        for (int q = o + 1; q < NO; ++q)
            if (overlaps(outs[o].p, outs[o].bytes, outs[q].p, outs[q].bytes)) return true;
    }
    return false;
}

// The out_* half of adder_bn_links: out_x with exactly one of out_coef and out_part (+ what belongs to it).
static int bn_out_half(const adder_bn_links &bn, const ConvDims &d, BnSums &sums) {
    sums = kNoBnSums;
    if (!bn.out_x) return (bn.out_coef || bn.out_part || bn.out_gy) ? ADDER_ERR_NULL_POINTER : ADDER_OK;
    if ((bn.out_coef == nullptr) == (bn.out_part == nullptr)) return ADDER_ERR_NULL_POINTER;
    if (bn.out_part) {
        if (!bn.out_gamma || !bn.out_mean || !bn.out_rstd || !bn.out_dgamma || !bn.out_dbeta)
            return ADDER_ERR_NULL_POINTER;
        if (bn.out_slots < 1) return ADDER_ERR_BAD_SHAPE;
        sums = BnSums{bn.out_part, bn.out_slots, (double)d.N * d.Ho * d.Wo, bn.out_gamma, bn.out_mean, bn.out_rstd,
                      bn.out_dgamma, bn.out_dbeta};
    }
    return ADDER_OK;
}

}  // namespace adder

using namespace adder;

extern "C" {

const char *adder_strerror(int status) {
    switch (status) {
        case ADDER_OK: return "ok";
        case ADDER_ERR_NULL_POINTER: return "a required pointer is NULL";
        case ADDER_ERR_BAD_SHAPE: return "non-positive or inconsistent dimension";
        case ADDER_ERR_TOO_LARGE: return "tensor exceeds 2^31-1 elements";
        case ADDER_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
        case ADDER_ERR_HIP: return "HIP runtime error";
        case ADDER_ERR_ALIAS: return "an output overlaps an input";
        case ADDER_ERR_UNSUPPORTED: return "this variant of the call does not exist for these dimensions or alignments";
        default: return "unknown status";
    }
}

const char *adder_last_hip_error(void) { return g_last_hip_error.c_str(); }

int adder_abi_version(void) { return 6; }

int adder_out_dim(int h, int k, int pad, int stride) {
    if (h <= 0 || k <= 0 || pad < 0 || stride <= 0 || h + 2 * pad < k) return 0;
    return (h - k + 2 * pad) / stride + 1;
}

int adder_conv2d_fwd_f32(const float *x, const float *w, float *y, int N, int Ci, int H, int W, int Co,
                         int kh, int kw, int stride, int pad, void *stream) {
    if (!x || !w || !y) return ADDER_ERR_NULL_POINTER;
    ConvDims d;
    if (int rc = make_dims(N, Ci, H, W, Co, kh, kw, stride, pad, d)) return rc;
    const size_t nx = sizeof(float) * (size_t)N * Ci * H * W, nw = sizeof(float) * (size_t)Co * d.K(),
                 ny = sizeof(float) * (size_t)N * Co * d.Ho * d.Wo;
    if (overlaps(y, ny, x, nx) || overlaps(y, ny, w, nw)) return ADDER_ERR_ALIAS;
    return launch_fwd(x, w, y, nullptr, d, static_cast<hipStream_t>(stream));
}

int adder_conv2d_fwd_stats_slots(int N, int Ci, int H, int W, int Co, int kh, int kw, int stride, int pad,
                                 int *slots) {
    if (!slots) return ADDER_ERR_NULL_POINTER;
    ConvDims d;
    if (int rc = make_dims(N, Ci, H, W, Co, kh, kw, stride, pad, d)) return rc;
    *slots = fwd_stats_slots(d);
    return ADDER_OK;
}

int adder_conv2d_fwd_stats_f32(const float *x, const float *w, float *y, double *stats, int stats_slots, int N,
                               int Ci, int H, int W, int Co, int kh, int kw, int stride, int pad, void *stream) {
    if (!x || !w || !y || !stats) return ADDER_ERR_NULL_POINTER;
    ConvDims d;
    if (int rc = make_dims(N, Ci, H, W, Co, kh, kw, stride, pad, d)) return rc;
    const int slots = fwd_stats_slots(d);
    if (slots == 0) return ADDER_ERR_UNSUPPORTED;
    if (stats_slots != slots) return ADDER_ERR_BAD_SHAPE;
    const size_t nx = sizeof(float) * (size_t)N * Ci * H * W, nw = sizeof(float) * (size_t)Co * d.K(),
                 ny = sizeof(float) * (size_t)N * Co * d.Ho * d.Wo, ns = sizeof(double) * 2 * (size_t)Co * slots;
    if (overlaps(y, ny, x, nx) || overlaps(y, ny, w, nw) || overlaps(stats, ns, x, nx) || overlaps(stats, ns, w, nw) ||
        overlaps(stats, ns, y, ny))
        return ADDER_ERR_ALIAS;
    return launch_fwd(x, w, y, stats, d, static_cast<hipStream_t>(stream));
}

int adder_conv2d_fwd_pair_stats_f32(const float *x, const float *w, const float *w_side, float *y, float *y_side,
                                    double *stats, double *stats_side, int stats_slots, int N, int Ci, int H, int W,
                                    int Co, int kh, int kw, int stride, int pad, void *stream) {
    if (!x || !w || !w_side || !y || !y_side || !stats || !stats_side) return ADDER_ERR_NULL_POINTER;
    ConvDims d;
    if (int rc = make_dims(N, Ci, H, W, Co, kh, kw, stride, pad, d)) return rc;
    if (!fwd_pair_supported(d)) return ADDER_ERR_UNSUPPORTED;
    const uintptr_t align = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y) |
                            reinterpret_cast<uintptr_t>(y_side);
    if (align & 15) return ADDER_ERR_UNSUPPORTED;
    const int slots = fwd_stats_slots(d);
    if (slots == 0) return ADDER_ERR_UNSUPPORTED;
    if (stats_slots != slots) return ADDER_ERR_BAD_SHAPE;
    const size_t nx = sizeof(float) * (size_t)N * Ci * H * W, nw = sizeof(float) * (size_t)Co * d.K(),
                 nws = sizeof(float) * (size_t)Co * Ci, ny = sizeof(float) * (size_t)N * Co * d.Ho * d.Wo,
                 ns = sizeof(double) * 2 * (size_t)Co * slots;
    const void *ins[3] = {x, w, w_side};
    const size_t in_bytes[3] = {nx, nw, nws};
    void *outs[4] = {y, y_side, stats, stats_side};
    const size_t out_bytes[4] = {ny, ny, ns, ns};
    for (int o = 0; o < 4; ++o) {
        for (int i = 0; i < 3; ++i)
            if (overlaps(outs[o], out_bytes[o], ins[i], in_bytes[i])) return ADDER_ERR_ALIAS;
        for (int o2 = o + 1; o2 < 4; ++o2)
            if (overlaps(outs[o], out_bytes[o], outs[o2], out_bytes[o2])) return ADDER_ERR_ALIAS;
    }
    return launch_fwd_pair(x, w, w_side, y, y_side, stats, stats_side, d, static_cast<hipStream_t>(stream));
}

int adder_plain_conv2d_fwd_f32(const float *x, const float *w, float *y, double *stats, int stats_slots, int N,
                               int Ci, int H, int W, int Co, int kh, int kw, int stride, int pad, void *stream) {
    if (!x || !w || !y) return ADDER_ERR_NULL_POINTER;
    ConvDims d;
    if (int rc = make_dims(N, Ci, H, W, Co, kh, kw, stride, pad, d)) return rc;
    const size_t nx = sizeof(float) * (size_t)N * Ci * H * W, nw = sizeof(float) * (size_t)Co * d.K(),
                 ny = sizeof(float) * (size_t)N * Co * d.Ho * d.Wo;
    if (overlaps(y, ny, x, nx) || overlaps(y, ny, w, nw)) return ADDER_ERR_ALIAS;
    if (stats) {
        const int slots = fwd_stats_slots(d);
        if (slots == 0) return ADDER_ERR_UNSUPPORTED;
        if (stats_slots != slots) return ADDER_ERR_BAD_SHAPE;
        const size_t ns = sizeof(double) * 2 * (size_t)Co * slots;
        if (overlaps(stats, ns, x, nx) || overlaps(stats, ns, w, nw) || overlaps(stats, ns, y, ny))
            return ADDER_ERR_ALIAS;
    }
    return launch_mulconv_fwd(x, w, y, stats, d, static_cast<hipStream_t>(stream));
}

int adder_conv2d_bwd_workspace_bytes(int N, int Ci, int H, int W, int Co, int kh, int kw, int stride,
                                     int pad, size_t *bytes) {
    if (!bytes) return ADDER_ERR_NULL_POINTER;
    ConvDims d;
    if (int rc = make_dims(N, Ci, H, W, Co, kh, kw, stride, pad, d)) return rc;
    *bytes = grad_w_workspace_bytes(d);
    return ADDER_OK;
}

static int conv2d_bwd(const float *gy, const float *x, const float *w, const float *gx_add, float *gx, float *gw,
                      float eta, void *ws, size_t ws_bytes, int N, int Ci, int H, int W, int Co, int kh, int kw,
                      int stride, int pad, void *stream);

int adder_conv2d_bwd_f32(const float *gy, const float *x, const float *w, float *gx, float *gw, float eta,
                         void *ws, size_t ws_bytes, int N, int Ci, int H, int W, int Co, int kh, int kw,
                         int stride, int pad, void *stream) {
    return conv2d_bwd(gy, x, w, nullptr, gx, gw, eta, ws, ws_bytes, N, Ci, H, W, Co, kh, kw, stride, pad, stream);
}

int adder_conv2d_bwd_add_f32(const float *gy, const float *x, const float *w, const float *gx_add, float *gx,
                             float *gw, float eta, void *ws, size_t ws_bytes, int N, int Ci, int H, int W, int Co,
                             int kh, int kw, int stride, int pad, void *stream) {
    if (!gx_add || !gx) return ADDER_ERR_NULL_POINTER;
    return conv2d_bwd(gy, x, w, gx_add, gx, gw, eta, ws, ws_bytes, N, Ci, H, W, Co, kh, kw, stride, pad, stream);
}

static int conv2d_bwd(const float *gy, const float *x, const float *w, const float *gx_add, float *gx, float *gw,
                      float eta, void *ws, size_t ws_bytes, int N, int Ci, int H, int W, int Co, int kh, int kw,
                      int stride, int pad, void *stream) {
    if (!gy || !x || !w) return ADDER_ERR_NULL_POINTER;
    if (!gx && !gw) return ADDER_ERR_NULL_POINTER;
    if (!(eta >= 0.f)) return ADDER_ERR_BAD_SHAPE;
    ConvDims d;
    if (int rc = make_dims(N, Ci, H, W, Co, kh, kw, stride, pad, d)) return rc;
    const size_t nx = sizeof(float) * (size_t)N * Ci * H * W, nw = sizeof(float) * (size_t)Co * d.K(),
                 ny = sizeof(float) * (size_t)N * Co * d.Ho * d.Wo;
    if (overlaps(gx, nx, x, nx) || overlaps(gx, nx, w, nw) || overlaps(gx, nx, gy, ny) ||
        overlaps(gw, nw, x, nx) || overlaps(gw, nw, w, nw) || overlaps(gw, nw, gy, ny) ||
        overlaps(gw, nw, gx, nx) || overlaps(gx, nx, gx_add, nx) || overlaps(gw, nw, gx_add, nx))
        return ADDER_ERR_ALIAS;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (gw) {
        const size_t need = grad_w_workspace_bytes(d);
        if (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255)) return ADDER_ERR_WORKSPACE;
        if (overlaps(ws, need, x, nx) || overlaps(ws, need, w, nw) || overlaps(ws, need, gy, ny) ||
            overlaps(ws, need, gx, nx) || overlaps(ws, need, gw, nw) || overlaps(ws, need, gx_add, nx))
            return ADDER_ERR_ALIAS;
    }
    if (gx)
        if (int rc = launch_grad_x(gy, x, w, gx, d, s, gx_add)) return rc;
    if (gw)
        if (int rc = launch_grad_w(gy, x, w, gw, eta, ws, ws_bytes, d, s)) return rc;
    return ADDER_OK;
}

int adder_conv2d_fwd_bf16(const adder_bf16 *x, const float *w, adder_bf16 *y, int N, int Ci, int H, int W, int Co,
                          int kh, int kw, int stride, int pad, void *stream) {
    if (!x || !w || !y) return ADDER_ERR_NULL_POINTER;
    ConvDims d;
    if (int rc = make_dims(N, Ci, H, W, Co, kh, kw, stride, pad, d)) return rc;
    const size_t nx = sizeof(adder_bf16) * (size_t)N * Ci * H * W, nw = sizeof(float) * (size_t)Co * d.K(),
                 ny = sizeof(adder_bf16) * (size_t)N * Co * d.Ho * d.Wo;
    if (overlaps(y, ny, x, nx) || overlaps(y, ny, w, nw)) return ADDER_ERR_ALIAS;
    return launch_fwd_bf16(x, w, y, d, static_cast<hipStream_t>(stream));
}

int adder_conv2d_bwd_bf16(const adder_bf16 *gy, const adder_bf16 *x, const float *w, adder_bf16 *gx, float *gw,
                          float eta, void *ws, size_t ws_bytes, int N, int Ci, int H, int W, int Co, int kh, int kw,
                          int stride, int pad, void *stream) {
    if (!gy || !x || !w) return ADDER_ERR_NULL_POINTER;
    if (!gx && !gw) return ADDER_ERR_NULL_POINTER;
    if (!(eta >= 0.f)) return ADDER_ERR_BAD_SHAPE;
    ConvDims d;
    if (int rc = make_dims(N, Ci, H, W, Co, kh, kw, stride, pad, d)) return rc;
    const size_t nx = sizeof(adder_bf16) * (size_t)N * Ci * H * W, nw = sizeof(float) * (size_t)Co * d.K(),
                 ny = sizeof(adder_bf16) * (size_t)N * Co * d.Ho * d.Wo;
    if (overlaps(gx, nx, x, nx) || overlaps(gx, nx, w, nw) || overlaps(gx, nx, gy, ny) || overlaps(gw, nw, x, nx) ||
        overlaps(gw, nw, w, nw) || overlaps(gw, nw, gy, ny) || overlaps(gw, nw, gx, nx))
        return ADDER_ERR_ALIAS;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (gw) {
        const size_t need = grad_w_workspace_bytes(d);
        if (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255)) return ADDER_ERR_WORKSPACE;
        if (overlaps(ws, need, x, nx) || overlaps(ws, need, w, nw) || overlaps(ws, need, gy, ny) ||
            overlaps(ws, need, gx, nx) || overlaps(ws, need, gw, nw))
            return ADDER_ERR_ALIAS;
    }
    if (gx)
        if (int rc = launch_grad_x_bf16(gy, x, w, gx, d, s)) return rc;
    if (gw)
        if (int rc = launch_grad_w_bf16(gy, x, w, gw, eta, ws, ws_bytes, d, s)) return rc;
    return ADDER_OK;
}

int adder_conv2d_bwd_noalloc_f32(const float *gy, const float *x, const float *w, float *gx, float *gw, float eta,
                                 int N, int Ci, int H, int W, int Co, int kh, int kw, int stride, int pad,
                                 void *stream) {
    if (!gy || !x || !w) return ADDER_ERR_NULL_POINTER;
    if (!gx && !gw) return ADDER_ERR_NULL_POINTER;
    ConvDims d;
    if (int rc = make_dims(N, Ci, H, W, Co, kh, kw, stride, pad, d)) return rc;
    void *ws = nullptr;
    size_t need = 0;
    if (gw) {   // only the weight gradient uses scratch
        need = grad_w_workspace_bytes(d);
        if (need > ADDER_NOALLOC_SCRATCH_BYTES) return ADDER_ERR_WORKSPACE;   // before any HIP call
        if (int rc = scratch_of_current_device(&ws)) return rc;
    }
    // every kernel writes the part of the scratch it later reads (slabs, norm partials): nothing to clear
    return conv2d_bwd(gy, x, w, nullptr, gx, gw, eta, ws, need, N, Ci, H, W, Co, kh, kw, stride, pad, stream);
}

static int check_col(int K, long NL, int Co) {
    if (K <= 0 || NL <= 0 || Co <= 0) return ADDER_ERR_BAD_SHAPE;
    if ((long)K * NL > kMaxElems || (long)Co * NL > kMaxElems || (long)Co * K > kMaxElems)
        return ADDER_ERR_TOO_LARGE;
    return ADDER_OK;
}

int adder_col_fwd_f32(const float *Xcol, const float *Wcol, float *out, int K, long NL, int Co, void *stream) {
    if (!Xcol || !Wcol || !out) return ADDER_ERR_NULL_POINTER;
    if (int rc = check_col(K, NL, Co)) return rc;
    const size_t nx = sizeof(float) * (size_t)K * NL, nw = sizeof(float) * (size_t)Co * K,
                 ny = sizeof(float) * (size_t)Co * NL;
    if (overlaps(out, ny, Xcol, nx) || overlaps(out, ny, Wcol, nw)) return ADDER_ERR_ALIAS;
    return launch_col_fwd(Xcol, Wcol, out, K, NL, Co, static_cast<hipStream_t>(stream));
}

int adder_col_bwd_workspace_bytes(int K, long NL, int Co, size_t *bytes) {
    if (!bytes) return ADDER_ERR_NULL_POINTER;
    if (int rc = check_col(K, NL, Co)) return rc;
    *bytes = col_grad_w_workspace_bytes(K, NL, Co);
    return ADDER_OK;
}

// the slab workspace of the column-matrix weight gradient (none for matrices the slab kernel does not serve)
static int check_col_ws(const void *ws, size_t ws_bytes, int K, long NL, int Co) {
    const size_t need = col_grad_w_workspace_bytes(K, NL, Co);
    if (need == 0) return ADDER_OK;
    if (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255)) return ADDER_ERR_WORKSPACE;
    return ADDER_OK;
}

static int col_alias(const float *gy, const float *X, const float *Wm, const float *gW, const float *gX, int K,
                     long NL, int Co) {
    const size_t nx = sizeof(float) * (size_t)K * NL, nw = sizeof(float) * (size_t)Co * K,
                 ny = sizeof(float) * (size_t)Co * NL;
    if (overlaps(gW, nw, X, nx) || overlaps(gW, nw, Wm, nw) || overlaps(gW, nw, gy, ny) ||
        overlaps(gX, nx, X, nx) || overlaps(gX, nx, Wm, nw) || overlaps(gX, nx, gy, ny) ||
        overlaps(gX, nx, gW, nw))
        return ADDER_ERR_ALIAS;
    return ADDER_OK;
}

int adder_col_gradw_f32(const float *gy, const float *Xcol, const float *Wcol, float *gW, int K, long NL,
                        int Co, void *ws, size_t ws_bytes, void *stream) {
    if (!gy || !Xcol || !Wcol || !gW) return ADDER_ERR_NULL_POINTER;
    if (int rc = check_col(K, NL, Co)) return rc;
    if (int rc = col_alias(gy, Xcol, Wcol, gW, nullptr, K, NL, Co)) return rc;
    if (int rc = check_col_ws(ws, ws_bytes, K, NL, Co)) return rc;
    return launch_col_grad_w(gy, Xcol, Wcol, gW, K, NL, Co, ws, static_cast<hipStream_t>(stream));
}

int adder_col_gradx_f32(const float *gy, const float *Xcol, const float *Wcol, float *gX, int K, long NL,
                        int Co, void *stream) {
    if (!gy || !Xcol || !Wcol || !gX) return ADDER_ERR_NULL_POINTER;
    if (int rc = check_col(K, NL, Co)) return rc;
    if (int rc = col_alias(gy, Xcol, Wcol, nullptr, gX, K, NL, Co)) return rc;
    return launch_col_grad_x(gy, Xcol, Wcol, gX, K, NL, Co, static_cast<hipStream_t>(stream));
}

int adder_col_bwd_f32(const float *gy, const float *Xcol, const float *Wcol, float *gW, float *gX, int K,
                      long NL, int Co, void *ws, size_t ws_bytes, void *stream) {
    if (!gy || !Xcol || !Wcol || !gW || !gX) return ADDER_ERR_NULL_POINTER;
    if (int rc = check_col(K, NL, Co)) return rc;
    if (int rc = col_alias(gy, Xcol, Wcol, gW, gX, K, NL, Co)) return rc;
    if (int rc = check_col_ws(ws, ws_bytes, K, NL, Co)) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int small = launch_col_bwd_small(gy, Xcol, Wcol, gW, gX, K, NL, Co, s);   // few columns: one launch
    if (small != ADDER_ERR_UNSUPPORTED) return small;
    const int fused = launch_col_bwd_fused(gy, Xcol, Wcol, gW, gX, K, NL, Co, ws, s);   // one pass over Xcol where it applies
    if (fused != ADDER_ERR_UNSUPPORTED) return fused;
    if (int rc = launch_col_grad_x(gy, Xcol, Wcol, gX, K, NL, Co, s)) return rc;
    return launch_col_grad_w(gy, Xcol, Wcol, gW, K, NL, Co, ws, s);
}

int adder_norm_scale_workspace_bytes(long n, size_t *bytes) {
    if (!bytes) return ADDER_ERR_NULL_POINTER;
    if (n <= 0) return ADDER_ERR_BAD_SHAPE;
    *bytes = norm_scale_workspace_bytes(n);
    return ADDER_OK;
}

int adder_grad_norm_scale_f32(float *g, long n, float eta, float eps, void *ws, size_t ws_bytes, void *stream) {
    if (!g) return ADDER_ERR_NULL_POINTER;
    if (n <= 0 || !(eta >= 0.f) || !(eps > 0.f)) return ADDER_ERR_BAD_SHAPE;
    if (!ws || ws_bytes < norm_scale_workspace_bytes(n) || (reinterpret_cast<uintptr_t>(ws) & 255))
        return ADDER_ERR_WORKSPACE;
    return launch_norm_scale(g, n, eta, eps, ws, static_cast<hipStream_t>(stream));
}

int adder_conv2d_grad_w_staged_f32(const float *gy, const float *x, const float *w, float *gw, float eta, void *ws,
                                   size_t ws_bytes, int N, int Ci, int H, int W, int Co, int kh, int kw, int stride,
                                   int pad, adder_grad_w_stage *stage, void *stream) {
    return adder_conv2d_grad_w_staged_bn_f32(gy, x, w, gw, eta, ws, ws_bytes, N, Ci, H, W, Co, kh, kw, stride, pad,
                                             nullptr, stage, stream);
}

int adder_conv2d_grad_w_staged_bn_f32(const float *gy, const float *x, const float *w, float *gw, float eta, void *ws,
                                      size_t ws_bytes, int N, int Ci, int H, int W, int Co, int kh, int kw, int stride,
                                      int pad, const adder_bn_links *links, adder_grad_w_stage *stage, void *stream) {
    if (!gy || !x || !gw || !stage) return ADDER_ERR_NULL_POINTER;
    if (!(eta >= 0.f)) return ADDER_ERR_BAD_SHAPE;
    ConvDims d;
    if (int rc = make_dims(N, Ci, H, W, Co, kh, kw, stride, pad, d)) return rc;
    const adder_bn_links bn = links ? *links : adder_bn_links{};
    BnSums sums;
    if (int rc = bn_out_half(bn, d, sums)) return rc;
    const size_t nx = sizeof(float) * (size_t)N * Ci * H * W, nw = sizeof(float) * (size_t)Co * d.K(),
                 ny = sizeof(float) * (size_t)N * Co * d.Ho * d.Wo, nco = sizeof(float) * (size_t)Co;
    const size_t need = grad_w_workspace_bytes(d);
    if (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255)) return ADDER_ERR_WORKSPACE;
    const Span outs[] = {{ws, need}, {gw, nw}, {bn.out_gy, ny}, {bn.out_dgamma, nco}, {bn.out_dbeta, nco}};
    const Span ins[] = {{x, nx}, {w, nw}, {gy, ny}, {bn.out_x, ny}, {bn.out_coef, 4 * nco},
                        {bn.out_part, sizeof(float) * 2 * (size_t)Co * (size_t)(bn.out_slots > 0 ? bn.out_slots : 0)},
                        {bn.out_gamma, nco}, {bn.out_mean, nco}, {bn.out_rstd, nco}};
    if (any_alias(outs, ins)) return ADDER_ERR_ALIAS;
    return launch_grad_w_staged(gy, x, w, gw, eta, ws, ws_bytes, d, stage, static_cast<hipStream_t>(stream), bn.out_x,
                                bn.out_coef, bn.out_gy, sums);
}

int adder_conv2d_bwd_bn_slots(int N, int Ci, int H, int W, int Co, int kh, int kw, int stride, int pad, int *slots) {
    if (!slots) return ADDER_ERR_NULL_POINTER;
    ConvDims d;
    if (int rc = make_dims(N, Ci, H, W, Co, kh, kw, stride, pad, d)) return rc;
    // both halves of the links or neither: the layer needs the fused input-gradient and weight-gradient kernels
    *slots = grad_w_bn_supported(d, nullptr, nullptr, nullptr, nullptr) ? grad_x_bn_slots(d) : 0;
    return ADDER_OK;
}

int adder_conv2d_bwd_bn_f32(const float *gy, const float *x, const float *w, const float *gx_add, float *gx, float *gw,
                            float eta, void *ws, size_t ws_bytes, int N, int Ci, int H, int W, int Co, int kh, int kw,
                            int stride, int pad, const adder_bn_links *links, void *stream) {
    if (!gy || !x || !w || !links) return ADDER_ERR_NULL_POINTER;
    if (!gx && !gw) return ADDER_ERR_NULL_POINTER;
    if (!(eta >= 0.f)) return ADDER_ERR_BAD_SHAPE;
    const adder_bn_links bn = *links;
    ConvDims d;
    if (int rc = make_dims(N, Ci, H, W, Co, kh, kw, stride, pad, d)) return rc;
    BnSums sums;
    if (int rc = bn_out_half(bn, d, sums)) return rc;
    if (bn.out_x && gx && !bn.out_gy) return ADDER_ERR_NULL_POINTER;   // grad_X reads the gradient grad_W leaves there
    if (bn.in_part && (!bn.in_x || !bn.in_mean || !bn.in_rstd || !gx)) return ADDER_ERR_NULL_POINTER;
    if ((bn.in_gamma == nullptr) != (bn.in_beta == nullptr)) return ADDER_ERR_NULL_POINTER;
    if ((bn.side_gy == nullptr) != (bn.side_w == nullptr)) return ADDER_ERR_NULL_POINTER;
    if (bn.side_gy && (!bn.in_part || kh != 3 || kw != 3 || stride != 2 || pad != 1 || (H & 1) || (W & 1)))
        return ADDER_ERR_UNSUPPORTED;
    const int slots = grad_w_bn_supported(d, nullptr, nullptr, nullptr, nullptr) ? grad_x_bn_slots(d) : 0;
    if (slots == 0 || (bn.out_x && !gw)) return ADDER_ERR_UNSUPPORTED;   // (the grad_W kernel is the one that forms gy)
    if (bn.in_part && bn.in_slots != slots) return ADDER_ERR_BAD_SHAPE;
    const size_t nx = sizeof(float) * (size_t)N * Ci * H * W, nw = sizeof(float) * (size_t)Co * d.K(),
                 ny = sizeof(float) * (size_t)N * Co * d.Ho * d.Wo, np = sizeof(float) * 2 * (size_t)Ci * slots,
                 nci = sizeof(float) * (size_t)Ci, nco = sizeof(float) * (size_t)Co;
    const size_t need = gw ? grad_w_workspace_bytes(d) : 0;
    if (gw && (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255))) return ADDER_ERR_WORKSPACE;
    const Span outs[] = {{gx, nx}, {gw, nw}, {bn.in_part, np}, {bn.out_gy, ny}, {gw ? ws : nullptr, need},
                         {bn.out_dgamma, nco}, {bn.out_dbeta, nco}};
    const Span ins[] = {{gy, ny}, {x, nx}, {w, nw}, {gx_add, nx}, {bn.out_x, ny}, {bn.out_coef, 4 * nco},
                        {bn.out_part, sizeof(float) * 2 * (size_t)Co * (size_t)(bn.out_slots > 0 ? bn.out_slots : 0)},
                        {bn.out_gamma, nco}, {bn.out_mean, nco}, {bn.out_rstd, nco},
                        {bn.in_x, nx}, {bn.in_mean, nci}, {bn.in_rstd, nci}, {bn.in_gamma, nci}, {bn.in_beta, nci},
                        {bn.side_gy, ny}, {bn.side_w, sizeof(float) * (size_t)Co * Ci}};
    if (any_alias(outs, ins)) return ADDER_ERR_ALIAS;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (bn.out_x && !grad_w_bn_supported(d, gy, x, bn.out_x, bn.out_coef ? (const void *)bn.out_coef : (const void *)bn.out_part))
        return ADDER_ERR_UNSUPPORTED;
    if ((reinterpret_cast<uintptr_t>(bn.out_gy) | reinterpret_cast<uintptr_t>(gx) | reinterpret_cast<uintptr_t>(gx_add) |
         reinterpret_cast<uintptr_t>(gy) | reinterpret_cast<uintptr_t>(bn.in_x)) & 15)
        return ADDER_ERR_UNSUPPORTED;   // before the first launch: the grad_X kernel would refuse these
    // grad_W first: with the out_* half it is the kernel that turns dz into the gradient of y, which grad_X reads
    if (gw)
        if (int rc = launch_grad_w(gy, x, w, gw, eta, ws, ws_bytes, d, s, bn.out_x, bn.out_coef, bn.out_gy, sums))
            return rc;
    if (gx)
        if (int rc = launch_grad_x_bn(bn.out_x ? bn.out_gy : gy, x, w, gx, d, s, gx_add, bn)) return rc;
    return ADDER_OK;
}

int adder_bn_bwd_coef_f32(const float *part, int slots, const float *gamma, const float *save_mean,
                          const float *save_rstd, double count, float *coef, float *dgamma, float *dbeta, int C,
                          void *stream) {
    if (!part || !gamma || !save_mean || !save_rstd || !coef || !dgamma || !dbeta) return ADDER_ERR_NULL_POINTER;
    if (slots <= 0 || C <= 0 || !(count >= 1.0)) return ADDER_ERR_BAD_SHAPE;
    if (reinterpret_cast<uintptr_t>(coef) & 15) return ADDER_ERR_UNSUPPORTED;
    return launch_bn_bwd_coef(part, slots, gamma, save_mean, save_rstd, count, coef, dgamma, dbeta, C,
                              static_cast<hipStream_t>(stream));
}

static int check_stages(int count, const adder_grad_w_stage *st) {
    if (!st) return ADDER_ERR_NULL_POINTER;
    if (count <= 0 || count > ADDER_GRAD_W_FINISH_MAX) return ADDER_ERR_BAD_SHAPE;
    for (int t = 0; t < count; ++t) {
        if (!st[t].part || !st[t].sgpart || !st[t].gw) return ADDER_ERR_NULL_POINTER;
        if (st[t].slots <= 0 || st[t].Co <= 0 || st[t].K <= 0 || !(st[t].eta >= 0.f)) return ADDER_ERR_BAD_SHAPE;
        if ((long)st[t].Co * st[t].K > kMaxElems) return ADDER_ERR_TOO_LARGE;
    }
    return ADDER_OK;
}

int adder_grad_w_finish_workspace_bytes(int count, const adder_grad_w_stage *stages, size_t *bytes) {
    if (!bytes) return ADDER_ERR_NULL_POINTER;
    if (int rc = check_stages(count, stages)) return rc;
    *bytes = grad_w_finish_workspace_bytes(count, stages);
    return ADDER_OK;
}

int adder_grad_w_finish_f32(int count, const adder_grad_w_stage *stages, void *ws, size_t ws_bytes, void *stream) {
    if (int rc = check_stages(count, stages)) return rc;
    if (!ws || ws_bytes < grad_w_finish_workspace_bytes(count, stages) || (reinterpret_cast<uintptr_t>(ws) & 255))
        return ADDER_ERR_WORKSPACE;
    return launch_grad_w_finish(count, stages, ws, static_cast<hipStream_t>(stream));
}

int adder_norm_scale_batched_workspace_bytes(int count, size_t *bytes) {
    if (!bytes) return ADDER_ERR_NULL_POINTER;
    if (count <= 0 || count > ADDER_NORM_BATCH_MAX) return ADDER_ERR_BAD_SHAPE;
    *bytes = norm_scale_batched_workspace_bytes(count);
    return ADDER_OK;
}

int adder_grad_norm_scale_batched_f32(int count, float *const *g, const long *n, const float *eta, float eps,
                                      void *ws, size_t ws_bytes, void *stream) {
    if (!g || !n || !eta) return ADDER_ERR_NULL_POINTER;
    if (count <= 0 || count > ADDER_NORM_BATCH_MAX || !(eps > 0.f)) return ADDER_ERR_BAD_SHAPE;
    for (int t = 0; t < count; ++t) {
        if (!g[t]) return ADDER_ERR_NULL_POINTER;
        if (n[t] <= 0 || !(eta[t] > 0.f)) return ADDER_ERR_BAD_SHAPE;
        if (n[t] > kMaxElems) return ADDER_ERR_TOO_LARGE;
    }
    if (!ws || ws_bytes < norm_scale_batched_workspace_bytes(count) || (reinterpret_cast<uintptr_t>(ws) & 255))
        return ADDER_ERR_WORKSPACE;
    return launch_norm_scale_batched(count, g, n, eta, eps, ws, static_cast<hipStream_t>(stream));
}

static int check_bn(int N, int C, int HW) {
    if (N <= 0 || C <= 0 || HW <= 0) return ADDER_ERR_BAD_SHAPE;
    if ((long)N * C * HW > kMaxElems) return ADDER_ERR_TOO_LARGE;
    return ADDER_OK;
}

int adder_bn_act_workspace_bytes(int N, int C, int HW, size_t *bytes) {
    if (!bytes) return ADDER_ERR_NULL_POINTER;
    if (int rc = check_bn(N, C, HW)) return rc;
    *bytes = bn_workspace_bytes(N, C, HW);
    return ADDER_OK;
}

int adder_bn_act_mask_words(int N, int C, int HW, size_t *words) {
    if (!words) return ADDER_ERR_NULL_POINTER;
    if (int rc = check_bn(N, C, HW)) return rc;
    *words = bn_mask_words(N, C, HW);
    return ADDER_OK;
}

// a sign mask needs ReLU, a shape that has one, and float4-aligned tensors
static int check_mask(const void *mask, int relu, int N, int C, int HW) {
    if (!mask) return ADDER_OK;
    if (!relu || bn_mask_words(N, C, HW) == 0) return ADDER_ERR_UNSUPPORTED;
    return ADDER_OK;
}

int adder_bn_act_fwd_f32(const float *x, const float *residual, const float *gamma, const float *beta, float *y,
                         unsigned int *relu_mask, float *save_mean, float *save_rstd, float *running_mean,
                         float *running_var, long long *num_batches_tracked, float momentum, float eps, int relu,
                         int N, int C, int HW, void *ws, size_t ws_bytes, void *stream) {
    if (!x || !gamma || !beta || !y || !save_mean || !save_rstd) return ADDER_ERR_NULL_POINTER;
    if ((running_mean == nullptr) != (running_var == nullptr)) return ADDER_ERR_NULL_POINTER;
    if (int rc = check_bn(N, C, HW)) return rc;
    if (int rc = check_mask(relu_mask, relu, N, C, HW)) return rc;
    if (!(eps > 0.f) || !(momentum >= 0.f && momentum <= 1.f)) return ADDER_ERR_BAD_SHAPE;
    if (!ws || ws_bytes < bn_workspace_bytes(N, C, HW) || (reinterpret_cast<uintptr_t>(ws) & 255))
        return ADDER_ERR_WORKSPACE;
    return launch_bn_act_fwd(x, residual, gamma, beta, y, relu_mask, save_mean, save_rstd, running_mean, running_var,
                             num_batches_tracked, momentum, eps, relu != 0, N, C, HW, ws, nullptr, 0,
                             static_cast<hipStream_t>(stream));
}

int adder_bn_act_fwd_stats_f32(const float *x, const float *residual, const float *gamma, const float *beta, float *y,
                               unsigned int *relu_mask, float *save_mean, float *save_rstd, float *running_mean,
                               float *running_var, long long *num_batches_tracked, float momentum, float eps, int relu,
                               int N, int C, int HW, const double *stats, int stats_slots, void *stream) {
    if (!x || !gamma || !beta || !y || !save_mean || !save_rstd || !stats) return ADDER_ERR_NULL_POINTER;
    if ((running_mean == nullptr) != (running_var == nullptr)) return ADDER_ERR_NULL_POINTER;
    if (int rc = check_bn(N, C, HW)) return rc;
    if (int rc = check_mask(relu_mask, relu, N, C, HW)) return rc;
    if (stats_slots <= 0) return ADDER_ERR_BAD_SHAPE;
    if (!(eps > 0.f) || !(momentum >= 0.f && momentum <= 1.f)) return ADDER_ERR_BAD_SHAPE;
    return launch_bn_act_fwd(x, residual, gamma, beta, y, relu_mask, save_mean, save_rstd, running_mean, running_var,
                             num_batches_tracked, momentum, eps, relu != 0, N, C, HW, nullptr, stats, stats_slots,
                             static_cast<hipStream_t>(stream));
}

int adder_bn_act_bwd_f32(const float *dy, const float *y, const unsigned int *relu_mask, const float *x,
                         const float *gamma, const float *save_mean, const float *save_rstd, float *dx,
                         float *dresidual, float *dgamma, float *dbeta, int relu, int N, int C, int HW, void *ws,
                         size_t ws_bytes, void *stream) {
    if (!dy || !x || !gamma || !save_mean || !save_rstd || !dx || !dgamma || !dbeta) return ADDER_ERR_NULL_POINTER;
    if (relu && !y && !relu_mask) return ADDER_ERR_NULL_POINTER;
    if (int rc = check_bn(N, C, HW)) return rc;
    if (int rc = check_mask(relu_mask, relu, N, C, HW)) return rc;
    if (!ws || ws_bytes < bn_workspace_bytes(N, C, HW) || (reinterpret_cast<uintptr_t>(ws) & 255))
        return ADDER_ERR_WORKSPACE;
    return launch_bn_act_bwd(dy, y, relu_mask, x, gamma, save_mean, save_rstd, dx, dresidual, dgamma, dbeta, relu != 0,
                             N, C, HW, ws, static_cast<hipStream_t>(stream));
}

int adder_sgd_momentum_step_f32(int count, float *const *params, const float *const *grads, float *const *momentum_bufs,
                                const long *n, const float *lr_device, float lr, float momentum, float weight_decay,
                                void *stream) {
    if (!params || !grads || !momentum_bufs || !n) return ADDER_ERR_NULL_POINTER;
    if (count <= 0 || count > ADDER_SGD_BATCH_MAX) return ADDER_ERR_BAD_SHAPE;
    if (!(momentum >= 0.f) || !(weight_decay >= 0.f) || !(lr_device || lr >= 0.f)) return ADDER_ERR_BAD_SHAPE;
    long blocks = 0;
    for (int t = 0; t < count; ++t) {
        if (!params[t] || !grads[t] || !momentum_bufs[t]) return ADDER_ERR_NULL_POINTER;
        if (n[t] <= 0) return ADDER_ERR_BAD_SHAPE;
        if (n[t] > kMaxElems) return ADDER_ERR_TOO_LARGE;
        blocks += (n[t] + 1023) / 1024;
    }
    if (blocks > kMaxElems) return ADDER_ERR_TOO_LARGE;
    for (int t = 0; t < count; ++t) {
        const size_t bytes = sizeof(float) * (size_t)n[t];
        if (overlaps(params[t], bytes, grads[t], bytes) || overlaps(params[t], bytes, momentum_bufs[t], bytes) ||
            overlaps(momentum_bufs[t], bytes, grads[t], bytes))
            return ADDER_ERR_ALIAS;
        for (int u = t + 1; u < count; ++u) {
            const size_t other = sizeof(float) * (size_t)n[u];
            if (overlaps(params[t], bytes, params[u], other) || overlaps(momentum_bufs[t], bytes, momentum_bufs[u], other) ||
                overlaps(params[t], bytes, momentum_bufs[u], other) || overlaps(momentum_bufs[t], bytes, params[u], other))
                return ADDER_ERR_ALIAS;
        }
    }
    return launch_sgd_momentum(count, params, grads, momentum_bufs, n, lr_device, lr, momentum, weight_decay,
                               static_cast<hipStream_t>(stream));
}

int adder_cross_entropy_fwd_f32(const float *logits, const long long *target, float *loss, float *lse, int N,
                                int classes, void *stream) {
    if (!logits || !target || !loss || !lse) return ADDER_ERR_NULL_POINTER;
    if (N <= 0 || classes <= 0) return ADDER_ERR_BAD_SHAPE;
    if ((long)N * classes > kMaxElems) return ADDER_ERR_TOO_LARGE;
    const size_t nz = sizeof(float) * (size_t)N * classes, nn = sizeof(float) * (size_t)N;
    const Span outs[] = {{loss, sizeof(float)}, {lse, nn}};
    const Span ins[] = {{logits, nz}, {target, sizeof(long long) * (size_t)N}};
    if (any_alias(outs, ins)) return ADDER_ERR_ALIAS;
    return launch_ce_fwd(logits, target, loss, lse, N, classes, static_cast<hipStream_t>(stream));
}

int adder_cross_entropy_bwd_f32(const float *logits, const long long *target, const float *lse, const float *grad_loss,
                                float *grad_logits, int N, int classes, void *stream) {
    if (!logits || !target || !lse || !grad_loss || !grad_logits) return ADDER_ERR_NULL_POINTER;
    if (N <= 0 || classes <= 0) return ADDER_ERR_BAD_SHAPE;
    if ((long)N * classes > kMaxElems) return ADDER_ERR_TOO_LARGE;
    const size_t nz = sizeof(float) * (size_t)N * classes, nn = sizeof(float) * (size_t)N;
    const Span outs[] = {{grad_logits, nz}};
    const Span ins[] = {{logits, nz}, {target, sizeof(long long) * (size_t)N}, {lse, nn}, {grad_loss, sizeof(float)}};
    if (any_alias(outs, ins)) return ADDER_ERR_ALIAS;
    return launch_ce_bwd(logits, target, lse, grad_loss, grad_logits, N, classes, static_cast<hipStream_t>(stream));
}

int adder_head_supported(int N, int C, int HW, int classes) {
    return (N > 0 && C > 0 && HW > 0 && classes > 0 && head_supported(N, C, HW, classes)) ? 1 : 0;
}

int adder_head_fwd_f32(const float *x, const float *w, const float *gamma, const float *beta, float *pooled, float *z,
                       float *y, float *save_mean, float *save_rstd, float *running_mean, float *running_var,
                       long long *num_batches_tracked, float momentum, float eps, int N, int C, int HW, int classes,
                       void *stream) {
    if (!x || !w || !gamma || !beta || !pooled || !z || !y || !save_mean || !save_rstd) return ADDER_ERR_NULL_POINTER;
    if ((running_mean == nullptr) != (running_var == nullptr)) return ADDER_ERR_NULL_POINTER;
    if (N <= 0 || C <= 0 || HW <= 0 || classes <= 0 || !(eps >= 0.f)) return ADDER_ERR_BAD_SHAPE;
    if ((long)N * C * HW > kMaxElems) return ADDER_ERR_TOO_LARGE;
    if (!head_supported(N, C, HW, classes)) return ADDER_ERR_UNSUPPORTED;
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(pooled)) & 15) return ADDER_ERR_UNSUPPORTED;
    const size_t nx = sizeof(float) * (size_t)N * C * HW, nw = sizeof(float) * (size_t)classes * C,
                 np = sizeof(float) * (size_t)N * C, nz = sizeof(float) * (size_t)N * classes,
                 nj = sizeof(float) * (size_t)classes;
    const Span outs[] = {{pooled, np}, {z, nz}, {y, nz}, {save_mean, nj}, {save_rstd, nj}, {running_mean, nj},
                         {running_var, nj}, {num_batches_tracked, sizeof(long long)}};
    const Span ins[] = {{x, nx}, {w, nw}, {gamma, nj}, {beta, nj}};
    if (any_alias(outs, ins)) return ADDER_ERR_ALIAS;
    return launch_head_fwd(x, w, gamma, beta, pooled, z, y, save_mean, save_rstd, running_mean, running_var,
                           num_batches_tracked, momentum, eps, N, C, HW, classes, static_cast<hipStream_t>(stream));
}

int adder_head_bwd_f32(const float *dy, const float *z, const float *pooled, const float *w, const float *gamma,
                       const float *save_mean, const float *save_rstd, float *dz, float *dx, float *dw, float *dgamma,
                       float *dbeta, int N, int C, int HW, int classes, void *stream) {
    if (!dy || !z || !pooled || !w || !gamma || !save_mean || !save_rstd || !dz || !dw || !dgamma || !dbeta)
        return ADDER_ERR_NULL_POINTER;
    if (N <= 0 || C <= 0 || HW <= 0 || classes <= 0) return ADDER_ERR_BAD_SHAPE;
    if ((long)N * C * HW > kMaxElems) return ADDER_ERR_TOO_LARGE;
    if (!head_supported(N, C, HW, classes)) return ADDER_ERR_UNSUPPORTED;
    if ((reinterpret_cast<uintptr_t>(dx) | reinterpret_cast<uintptr_t>(pooled)) & 15) return ADDER_ERR_UNSUPPORTED;
    const size_t nx = sizeof(float) * (size_t)N * C * HW, nw = sizeof(float) * (size_t)classes * C,
                 np = sizeof(float) * (size_t)N * C, nz = sizeof(float) * (size_t)N * classes,
                 nj = sizeof(float) * (size_t)classes;
    const Span outs[] = {{dz, nz}, {dx, nx}, {dw, nw}, {dgamma, nj}, {dbeta, nj}};
    const Span ins[] = {{dy, nz}, {z, nz}, {pooled, np}, {w, nw}, {gamma, nj}, {save_mean, nj}, {save_rstd, nj}};
    if (any_alias(outs, ins)) return ADDER_ERR_ALIAS;
    return launch_head_bwd(dy, z, pooled, w, gamma, save_mean, save_rstd, dz, dx, dw, dgamma, dbeta, N, C, HW, classes,
                           static_cast<hipStream_t>(stream));
}

}  // extern "C"
