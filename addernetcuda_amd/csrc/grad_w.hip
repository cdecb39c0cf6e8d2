// Weight gradient of the AdderNet convolution, NCHW, deterministic (no atomics):
//   gw[co,ci,i,j] = sum_{n,ho,wo} (xpad[n,ci,ho*s+i-p,wo*s+j-p] - w[co,ci,i,j]) * gy[n,co,ho,wo]
// followed (eta > 0) by the adaptive learning-rate scaling of adder.py:78,
//   gw <- gw / max(||gw||_2, 1e-12) * sqrt(numel) * eta.
// Replaces the grad_w half of adder_cuda/adder.cu:194-272 (CONV_BACKWARD),
// adder.cu:72-131 (CONV_WEIGHT) and the five elementwise kernels PyTorch
// launches for adder.py:78.
//
// The tiled kernel uses  sum (x - w) g = sum x g - w * sum g : the first term is
// one v_fma_f32 per (co,k,position) term, the second needs only sum_g per
// output channel, which the gy tile loader collects on its way to LDS.
#include "common.hpp"
#include "tile3x3.hpp"

namespace adder {

static constexpr int kNormBlocksMax = 4096;  // sum-of-squares partials kept at the head of the workspace

// ---------------------------------------------------------------------------
// Generic kernel: one workgroup per (co, ci) [KH x KW taps in registers] or,
// for KH = 0, one workgroup per (co, ci, i, j).  Direct (x - w) * g form.
// ---------------------------------------------------------------------------
template <int KH, int KW>
__global__ __launch_bounds__(256) void grad_w_generic_kernel(const float *__restrict__ gy,
                                                             const float *__restrict__ x,
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
        const float g = gy[((size_t)n * d.Co + co) * L + l];
        const float *xp = x + ((size_t)n * d.Ci + ci) * d.H * d.W;
#pragma unroll
        for (int t = 0; t < T; ++t) {
            const int hi = ho * d.stride + ti[t] - d.pad, wi = wo * d.stride + tj[t] - d.pad;
            const bool v = hi >= 0 && hi < d.H && wi >= 0 && wi < d.W;
            const float xv = v ? xp[(size_t)hi * d.W + wi] : 0.f;
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
// Tiled kernel for 3x3, pad 1, stride S = 1 or 2.
//
// Lanes own output positions (strip of TN in one row).  A wave owns a fixed
// block of TM output channels x CQ input channels and keeps the TM*CQ*9
// partial sums of its own positions in registers while the workgroup walks
// over tiles (images / row bands); NCOB x NCIB waves share each staged tile.
// LDS per buffer: haloed x tile [img][CIB][TH+2][PITCH] and the gy tile
// [img][COB][TH][TW].  At the end every wave folds its 64 lanes through an
// LDS transpose and writes one partial (Co*K floats per grid.x slot) to the
// workspace; grad_w_finalize_kernel sums the slots in fp64.
// ---------------------------------------------------------------------------
template <int TN_, int SPR_, int TH_, int NIMG_, int TM_, int CQ_, int NCOB_, int NCIB_, int S_ = 1>
struct GradWCfg {
    static constexpr int TN = TN_, SPR = SPR_, TH = TH_, NIMG = NIMG_, TM = TM_, CQ = CQ_, NCOB = NCOB_,
                         NCIB = NCIB_, S = S_;
    static constexpr int COB = TM * NCOB, CIB = CQ * NCIB, NW = NCOB * NCIB;
    using XT = Tile3x3Cfg<TN, SPR, TH, NIMG, TM, NW, CIB, CQ, S>;  // haloed x tile, staged by all NW waves
    static constexpr int TW = XT::TW;
    static constexpr int NTHREADS = XT::NTHREADS;
    static constexpr int GPLANE = TH * TW;
    static constexpr int GBUF = NIMG * COB * GPLANE;
    static constexpr int GUNITS = GBUF / 4;
    static constexpr int GITER = ceil_div(GUNITS, NTHREADS);
    static constexpr int BUF = XT::BUF + GBUF;  // floats per (x, gy) buffer pair
    static constexpr int A = TM * CQ * 9;       // partial sums per lane
    static constexpr int RED_PITCH = 17;
    static constexpr int RED_FLOATS = NW * 64 * RED_PITCH;
    static constexpr int LDS_FLOATS = (2 * BUF > RED_FLOATS + GUNITS) ? 2 * BUF : RED_FLOATS + GUNITS;
    static constexpr int LDS_BYTES = LDS_FLOATS * 4;
    static_assert(XT::LANES == 64, "one position wave per channel block");
    static_assert(NTHREADS <= 1024, "workgroup too large");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
};

template <class G>
struct GyStage {
    float4 v[G::GITER];
};

template <class G>
__device__ __forceinline__ void gy_fetch(GyStage<G> &st, const float *__restrict__ gy, int co0, int Co,
                                         int n0, int N, int h0, int w0, int Ho, int Wo) {
#pragma unroll
    for (int it = 0; it < G::GITER; ++it) {
        const int u = threadIdx.x + it * G::NTHREADS;
        const int q = u % (G::TW / 4);
        const int r = (u / (G::TW / 4)) % G::TH;
        const int c = (u / (G::TW / 4) / G::TH) % G::COB;
        const int img = u / (G::TW / 4) / G::TH / G::COB;
        const int n = n0 + img, co = co0 + c, ho = h0 + r, wo = w0 + 4 * q;
        const bool ok = (G::GUNITS % G::NTHREADS == 0 || u < G::GUNITS) && n < N && co < Co && ho < Ho && wo < Wo;
        float4 val = make_float4(0.f, 0.f, 0.f, 0.f);
        if (ok) val = *reinterpret_cast<const float4 *>(gy + (((n * Co + co) * Ho + ho) * Wo + wo));
        st.v[it] = val;
    }
}

template <class G>
__device__ __forceinline__ void gy_commit(const GyStage<G> &st, float *buf, float (&sg)[G::GITER]) {
#pragma unroll
    for (int it = 0; it < G::GITER; ++it) {
        const int u = threadIdx.x + it * G::NTHREADS;
        if (G::GUNITS % G::NTHREADS == 0 || u < G::GUNITS) {
            *reinterpret_cast<float4 *>(buf + 4 * u) = st.v[it];
            sg[it] += (st.v[it].x + st.v[it].y) + (st.v[it].z + st.v[it].w);
        }
    }
}

template <class G>
__global__ __launch_bounds__(G::NTHREADS) void grad_w_3x3_kernel(const float *__restrict__ gy,
                                                                   const float *__restrict__ x,
                                                                   float *__restrict__ part,
                                                                   float *__restrict__ sgpart, int N, int Ci,
                                                                   int H, int W, int Co, int Ho, int Wo,
                                                                   int tilesH, int tilesW, int ntiles) {
    using XT = typename G::XT;
    constexpr int TN = G::TN, TM = G::TM, CQ = G::CQ, S = G::S, STRIP = XT::STRIP;
    extern __shared__ __align__(16) float smem[];

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int cob = wave % G::NCOB, cib = wave / G::NCOB;
    const int strip = lane % G::SPR;
    const int row = (lane / G::SPR) % G::TH;
    const int img = lane / (G::SPR * G::TH);
    const int co_blk = blockIdx.y * G::COB, ci_blk = blockIdx.z * G::CIB;

    float acc[TM][CQ][9];
#pragma unroll
    for (int m = 0; m < TM; ++m)
#pragma unroll
        for (int q = 0; q < CQ; ++q)
#pragma unroll
            for (int e = 0; e < 9; ++e) acc[m][q][e] = 0.f;
    float sg[G::GITER];
#pragma unroll
    for (int it = 0; it < G::GITER; ++it) sg[it] = 0.f;

    const int x_off = (img * G::CIB + cib * CQ) * XT::PLANE + row * S * XT::PITCH + strip * TN * S;
    const int g_off = XT::BUF + (img * G::COB + cob * TM) * G::GPLANE + row * G::TW + strip * TN;

    TileStage<typename XT::Patch> xs;
    GyStage<G> gs;
    int tile = blockIdx.x;
    int n0 = 0, h0 = 0, w0 = 0;
    auto decode = [&](int t) {
        const int tw = t % tilesW; t /= tilesW;
        const int th = t % tilesH; t /= tilesH;
        n0 = t * G::NIMG; h0 = th * G::TH; w0 = tw * G::TW;
    };
    if (tile < ntiles) {
        decode(tile);
        tile_fetch<typename XT::Patch>(xs, x, ci_blk, Ci, n0, N, h0 * S - 1, w0 * S, H, W);
        gy_fetch<G>(gs, gy, co_blk, Co, n0, N, h0, w0, Ho, Wo);
        tile_commit<typename XT::Patch>(xs, smem);
        gy_commit<G>(gs, smem + XT::BUF, sg);
    }
    __syncthreads();

    int cur = 0;
    for (; tile < ntiles; tile += gridDim.x) {
        const int next = tile + gridDim.x;
        if (next < ntiles) {
            decode(next);
            tile_fetch<typename XT::Patch>(xs, x, ci_blk, Ci, n0, N, h0 * S - 1, w0 * S, H, W);
            gy_fetch<G>(gs, gy, co_blk, Co, n0, N, h0, w0, Ho, Wo);
        }
        const float *base = smem + cur * G::BUF;
        float xr[CQ][3][STRIP];
#pragma unroll
        for (int q = 0; q < CQ; ++q)
#pragma unroll
            for (int i = 0; i < 3; ++i)
                lds_read_strip<STRIP, XT::STRIP_ALIGN>(base + x_off + q * XT::PLANE + i * XT::PITCH, xr[q][i]);
#pragma unroll
        for (int m = 0; m < TM; ++m) {
            float gr[TN];
            lds_read_strip<TN, (TN % 4 == 0 ? 4 : (TN % 2 == 0 ? 2 : 1))>(base + g_off + m * G::GPLANE, gr);
#pragma unroll
            for (int q = 0; q < CQ; ++q)
#pragma unroll
                for (int i = 0; i < 3; ++i)
#pragma unroll
                    for (int j = 0; j < 3; ++j)
#pragma unroll
                        for (int t = 0; t < TN; ++t)
                            acc[m][q][i * 3 + j] = fmaf(gr[t], xr[q][i][t * S + j], acc[m][q][i * 3 + j]);
        }
        if (next < ntiles) {
            tile_commit<typename XT::Patch>(xs, smem + (cur ^ 1) * G::BUF);
            gy_commit<G>(gs, smem + (cur ^ 1) * G::BUF + XT::BUF, sg);
        }
        __syncthreads();
        cur ^= 1;
    }

    // ---- fold the 64 lanes of each wave: 16 partial sums per round through LDS ----
    float *red = smem + wave * 64 * G::RED_PITCH;
    float *flat = &acc[0][0][0];
    const int K = Ci * 9;
    float *dst = part + (size_t)blockIdx.x * Co * K;
    constexpr int ROUNDS = ceil_div(G::A, 16);
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
#pragma unroll
        for (int e = 0; e < 16; ++e) red[lane * G::RED_PITCH + e] = (r * 16 + e < G::A) ? flat[r * 16 + e] : 0.f;
        __syncthreads();
        const int e = lane & 15, rg = lane >> 4;
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < 16; ++k) s += red[(rg * 16 + k) * G::RED_PITCH + e];
        s += __shfl_xor(s, 16, 64);
        s += __shfl_xor(s, 32, 64);
        __syncthreads();
        const int a = r * 16 + e;
        if (rg == 0 && a < G::A) {
            const int m = a / (CQ * 9), q = (a / 9) % CQ, tap = a % 9;
            const int co = co_blk + cob * TM + m, ci = ci_blk + cib * CQ + q;
            if (co < Co && ci < Ci) dst[((size_t)co * Ci + ci) * 9 + tap] = s;
        }
    }

    // ---- sum of gy per output channel (only the first input-channel block reports it) ----
    if (blockIdx.z == 0) {
        __syncthreads();
        float *sgl = smem + G::RED_FLOATS;
#pragma unroll
        for (int it = 0; it < G::GITER; ++it) {
            const int u = threadIdx.x + it * G::NTHREADS;
            if (G::GUNITS % G::NTHREADS == 0 || u < G::GUNITS) sgl[u] = sg[it];
        }
        __syncthreads();
        constexpr int UPC = G::GPLANE / 4;  // units per (img, co)
        if (threadIdx.x < G::COB) {
            const int c = threadIdx.x;
            double s = 0.0;
            for (int im = 0; im < G::NIMG; ++im)
                for (int k = 0; k < UPC; ++k) s += (double)sgl[(im * G::COB + c) * UPC + k];
            if (co_blk + c < Co) sgpart[(size_t)blockIdx.x * Co + co_blk + c] = (float)s;
        }
    }
}

// gw = sum_slots part - w * sum_slots sgpart ; per-block sum of squares for the norm when ss != NULL.
// A workgroup finishes 16 outputs: thread (sl, o) adds slots sl, sl+16, ... of output o in fp64, so the
// dependent chain is slots/16 long and every 16-lane group reads 64 contiguous bytes.
static constexpr int kFinOut = 16;
__global__ __launch_bounds__(256) void grad_w_finalize_kernel(const float *__restrict__ part,
                                                              const float *__restrict__ sgpart,
                                                              const float *__restrict__ w,
                                                              float *__restrict__ gw, double *__restrict__ ss,
                                                              int slots, int Co, int K) {
    const int o = threadIdx.x & 15, sl = threadIdx.x >> 4;
    const int total = Co * K;
    const int idx = blockIdx.x * kFinOut + o;
    const int idc = idx < total ? idx : total - 1;
    const int co = idc / K;
    double a = 0.0, sgs = 0.0;
    for (int p = sl; p < slots; p += 16) {
        a += (double)part[(size_t)p * total + idc];
        sgs += (double)sgpart[(size_t)p * Co + co];
    }
    __shared__ double ra[16][kFinOut + 1], rs[16][kFinOut + 1];
    ra[sl][o] = a;
    rs[sl][o] = sgs;
    __syncthreads();
    if (threadIdx.x < kFinOut) {
        double ta = 0.0, ts = 0.0;
#pragma unroll
        for (int k = 0; k < 16; ++k) { ta += ra[k][o]; ts += rs[k][o]; }
        double v = 0.0;
        if (idx < total) {
            const float r = (float)(ta - (double)w[idx] * ts);
            gw[idx] = r;
            v = (double)r * (double)r;
        }
        // lanes 0..15 of wave 0 hold the squares
#pragma unroll
        for (int off = 8; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
        if (threadIdx.x == 0 && ss) ss[blockIdx.x] = v;
    }
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
// Channel blocking of a workgroup: TM x CQ (co, ci) pairs per wave, NCOB x NCIB waves.
struct GwChan0 { static constexpr int TM = 8, CQ = 2, NCOB = 2, NCIB = 4; };   // 144 sums per lane, 8 waves
struct GwChan1 { static constexpr int TM = 8, CQ = 1, NCOB = 2, NCIB = 4; };   // 72 sums per lane, 8 waves
struct GwChan2 { static constexpr int TM = 4, CQ = 2, NCOB = 4, NCIB = 2; };   // 72 sums per lane, 8 waves
struct GwChan3 { static constexpr int TM = 8, CQ = 1, NCOB = 2, NCIB = 8; };   // 72 sums per lane, 16 waves
struct GwChan4 { static constexpr int TM = 4, CQ = 2, NCOB = 4, NCIB = 4; };   // 72 sums per lane, 16 waves
//                                     TN SPR TH NIMG
template <class Ch> using GwW32   = GradWCfg<4, 8, 8, 1, Ch::TM, Ch::CQ, Ch::NCOB, Ch::NCIB, 1>;
template <class Ch> using GwW16   = GradWCfg<4, 4, 16, 1, Ch::TM, Ch::CQ, Ch::NCOB, Ch::NCIB, 1>;
template <class Ch> using GwW8    = GradWCfg<4, 2, 8, 4, Ch::TM, Ch::CQ, Ch::NCOB, Ch::NCIB, 1>;
template <class Ch> using GwW16S2 = GradWCfg<4, 4, 16, 1, Ch::TM, Ch::CQ, Ch::NCOB, Ch::NCIB, 2>;
template <class Ch> using GwW8S2  = GradWCfg<4, 2, 8, 4, Ch::TM, Ch::CQ, Ch::NCOB, Ch::NCIB, 2>;

struct GradWPlan {
    int variant;  // 0 generic, 1 W32, 2 W16, 3 W8, 4 W16S2, 5 W8S2, 6 1x1
    int chan;     // channel blocking (GwChan<chan>) of the tiled variants
    int slots, gy, gz, tilesH, tilesW, ntiles;
};

template <class G>
static void plan_tiled(const ConvDims &d, GradWPlan &p) {
    p.tilesH = ceil_div(d.Ho, G::TH);
    p.tilesW = ceil_div(d.Wo, G::TW);
    p.ntiles = ceil_div(d.N, G::NIMG) * p.tilesH * p.tilesW;
    p.gy = ceil_div(d.Co, G::COB);
    p.gz = ceil_div(d.Ci, G::CIB);
    // enough workgroups to fill the chip, but at least ~4 tiles each so the fold is amortised
    static const int wgs = tune_knob("GW_WGS", 256);
    int want = ceil_div(wgs, p.gy * p.gz);
    int cap = p.ntiles / 4 > 0 ? p.ntiles / 4 : 1;
    p.slots = want < cap ? want : cap;
    if (p.slots > p.ntiles) p.slots = p.ntiles;
}

template <class Ch>
static void plan_shape(const ConvDims &d, GradWPlan &p) {
    switch (p.variant) {
        case 1: plan_tiled<GwW32<Ch>>(d, p); break;
        case 2: plan_tiled<GwW16<Ch>>(d, p); break;
        case 3: plan_tiled<GwW8<Ch>>(d, p); break;
        case 4: plan_tiled<GwW16S2<Ch>>(d, p); break;
        case 5: plan_tiled<GwW8S2<Ch>>(d, p); break;
    }
}

static GradWPlan plan_grad_w(const ConvDims &d) {
    GradWPlan p{};
    const bool k3p1 = d.kh == 3 && d.kw == 3 && d.pad == 1 && d.W % 4 == 0 && d.Wo % 4 == 0;
    const long partial_cap = 1L << 28;  // keep the partial buffer below 1 GiB
    if (k3p1 && d.stride == 1) p.variant = d.Wo > 16 ? 1 : (d.Wo > 8 ? 2 : 3);
    else if (k3p1 && d.stride == 2) p.variant = d.Wo > 8 ? 4 : 5;
    if (p.variant) {
        static const int chan_s1 = tune_knob("GW_CHAN", 0), chan_s2 = tune_knob("GW_CHAN_S2", 1);
        p.chan = d.stride == 1 ? chan_s1 : chan_s2;
        if (d.stride == 2 && (p.chan == 0)) p.chan = 1;   // 144 sums + stride-2 strips do not fit the register file
        switch (p.chan) {
            case 0: plan_shape<GwChan0>(d, p); break;
            case 1: plan_shape<GwChan1>(d, p); break;
            case 2: plan_shape<GwChan2>(d, p); break;
            case 3: plan_shape<GwChan3>(d, p); break;
            default: p.chan = 4; plan_shape<GwChan4>(d, p); break;
        }
    }
    if (!p.variant && conv1x1_supported(d, nullptr, nullptr)) {
        p.variant = 6;
        p.slots = grad_w_1x1_slots(d);
    }
    if (p.variant && (long)p.slots * d.Co * d.K() > partial_cap) p.variant = 0;
    return p;
}

size_t grad_w_workspace_bytes(const ConvDims &d) {
    const GradWPlan p = plan_grad_w(d);
    size_t bytes = sizeof(double) * kNormBlocksMax;
    if (p.variant) bytes += sizeof(float) * (size_t)p.slots * ((size_t)d.Co * d.K() + d.Co);
    return (bytes + 255) & ~(size_t)255;
}

template <class G>
static int launch_tiled(const float *gy, const float *x, float *part, float *sgpart, const ConvDims &d,
                        const GradWPlan &p, hipStream_t s) {
    static bool attr_set = false;
    if (!attr_set && G::LDS_BYTES > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&grad_w_3x3_kernel<G>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, G::LDS_BYTES);
        if (e != hipSuccess) return record_hip_error(e);
        attr_set = true;
    }
    hipLaunchKernelGGL(grad_w_3x3_kernel<G>, dim3(p.slots, p.gy, p.gz), dim3(G::NTHREADS), G::LDS_BYTES, s, gy,
                       x, part, sgpart, d.N, d.Ci, d.H, d.W, d.Co, d.Ho, d.Wo, p.tilesH, p.tilesW, p.ntiles);
    return check_launch();
}

template <class Ch>
static int launch_shape(const float *gy, const float *x, float *part, float *sgpart, const ConvDims &d,
                        const GradWPlan &p, hipStream_t s) {
    switch (p.variant) {
        case 1: return launch_tiled<GwW32<Ch>>(gy, x, part, sgpart, d, p, s);
        case 2: return launch_tiled<GwW16<Ch>>(gy, x, part, sgpart, d, p, s);
        case 3: return launch_tiled<GwW8<Ch>>(gy, x, part, sgpart, d, p, s);
        case 4: if constexpr (Ch::TM * Ch::CQ <= 8) return launch_tiled<GwW16S2<Ch>>(gy, x, part, sgpart, d, p, s);
        default: if constexpr (Ch::TM * Ch::CQ <= 8) return launch_tiled<GwW8S2<Ch>>(gy, x, part, sgpart, d, p, s);
    }
    return ADDER_ERR_BAD_SHAPE;
}

int launch_grad_w(const float *gy, const float *x, const float *w, float *gw, float eta, void *ws,
                  size_t ws_bytes, const ConvDims &d, hipStream_t s) {
    if (ws_bytes < grad_w_workspace_bytes(d)) return ADDER_ERR_WORKSPACE;
    GradWPlan p = plan_grad_w(d);
    if (p.variant && ((reinterpret_cast<uintptr_t>(gy) | reinterpret_cast<uintptr_t>(x)) & 15)) p.variant = 0;
    double *ss = reinterpret_cast<double *>(ws);
    const int K = d.K();
    const long n = (long)d.Co * K;
    if (p.variant) {
        float *part = reinterpret_cast<float *>(ss + kNormBlocksMax);
        float *sgpart = part + (size_t)p.slots * d.Co * K;
        int rc;
        if (p.variant == 6) {
            rc = launch_grad_w_1x1(gy, x, part, sgpart, p.slots, d, s);
        } else {
            switch (p.chan) {
                case 0: rc = launch_shape<GwChan0>(gy, x, part, sgpart, d, p, s); break;
                case 1: rc = launch_shape<GwChan1>(gy, x, part, sgpart, d, p, s); break;
                case 2: rc = launch_shape<GwChan2>(gy, x, part, sgpart, d, p, s); break;
                case 3: rc = launch_shape<GwChan3>(gy, x, part, sgpart, d, p, s); break;
                default: rc = launch_shape<GwChan4>(gy, x, part, sgpart, d, p, s); break;
            }
        }
        if (rc) return rc;
        const int nb = (int)ceil_div_l(n, kFinOut);
        const bool fused_norm = eta > 0.f && nb <= kNormBlocksMax;
        hipLaunchKernelGGL(grad_w_finalize_kernel, dim3(nb), dim3(256), 0, s, part, sgpart, w, gw,
                           fused_norm ? ss : nullptr, p.slots, d.Co, K);
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

}  // namespace adder
