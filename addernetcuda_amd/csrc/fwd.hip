// Forward AdderNet convolution, NCHW in -> NCHW out, implicit im2col.
//   y[n,co,ho,wo] = - sum_{ci,i,j} | w[co,ci,i,j] - xpad[n,ci,ho*s+i-p,wo*s+j-p] |
// Replaces adder_cuda/adder.cu:19-70 (CONV) together with the unfold + permute
// copies of adder.py:32-33,38-39 that feed it.
//
// The inner operation is two fp32 VALU instructions per (co,k,position) term
// -- v_sub_f32 d, s_w, v_x ; v_sub_f32 acc, acc, |d| -- and cannot use FMA or
// MFMA, so the kernels are built to keep everything else off the vector ALU:
//   * lanes own output positions, weights are wave-uniform and arrive through
//     the scalar cache as SGPR operands (no VGPRs, no LDS bandwidth);
//   * the haloed input tile of a workgroup is staged once in LDS with the
//     padding zeros materialised, and each lane reads its (TN+2)-wide strips
//     with ds_read_b128/b64 at immediate offsets;
//   * each lane keeps TM x TN accumulators so one strip read feeds 9*TM*TN terms.
#include "common.hpp"
#include "tile3x3.hpp"

namespace adder {

// ---------------------------------------------------------------------------
// Generic kernel: any kernel size / stride / padding / channel count.
// One output position per lane, TM output channels per lane, input read
// straight from global memory with bounds checks.
// ---------------------------------------------------------------------------
template <int TM, class T = float>
__global__ __launch_bounds__(256) void fwd_generic_kernel(const T *__restrict__ x,
                                                          const float *__restrict__ w,
                                                          T *__restrict__ y, ConvDims d) {
    const int total = d.N * d.Ho * d.Wo;
    int pos = blockIdx.x * 256 + threadIdx.x;
    const bool active = pos < total;
    if (!active) pos = total - 1;
    const int wo = pos % d.Wo;
    const int ho = (pos / d.Wo) % d.Ho;
    const int n = pos / (d.Wo * d.Ho);
    const int co0 = blockIdx.y * TM;
    const int K = d.K();
    uniform_f32_ptr wc = as_uniform(w);

    float acc[TM], tot[TM];   // acc: at most 16 channels' taps, tot: the rest (keeps fp32 error small for large K)
#pragma unroll
    for (int m = 0; m < TM; ++m) acc[m] = tot[m] = 0.f;

    int wrow[TM];
#pragma unroll
    for (int m = 0; m < TM; ++m) wrow[m] = min(co0 + m, d.Co - 1) * K;

    const T *xn = x + (size_t)n * d.Ci * d.H * d.W;
    for (int ci = 0; ci < d.Ci; ++ci) {
        for (int i = 0; i < d.kh; ++i) {
            const int hi = ho * d.stride + i - d.pad;
            const bool hv = hi >= 0 && hi < d.H;
            for (int j = 0; j < d.kw; ++j) {
                const int wi = wo * d.stride + j - d.pad;
                const bool v = hv && wi >= 0 && wi < d.W;
                const float xv = v ? ldf(xn + ((size_t)ci * d.H + hi) * d.W + wi) : 0.f;
                const int k = (ci * d.kh + i) * d.kw + j;
#pragma unroll
                for (int m = 0; m < TM; ++m) acc[m] -= fabsf(wc[wrow[m] + k] - xv);
            }
        }
        if ((ci & 15) == 15 || ci + 1 == d.Ci) {
#pragma unroll
            for (int m = 0; m < TM; ++m) { tot[m] += acc[m]; acc[m] = 0.f; }
        }
    }
    if (active) {
#pragma unroll
        for (int m = 0; m < TM; ++m)
            if (co0 + m < d.Co) stf(y + (((size_t)n * d.Co + co0 + m) * d.Ho + ho) * d.Wo + wo, tot[m]);
    }
}

// ---------------------------------------------------------------------------
// Tiled kernel for 3x3, pad 1, stride S = 1 or 2.
//
// A workgroup owns NIMG images x a TH x TW patch of output positions and
// TM*COW output channels.  TW = TN*SPR: each lane owns a strip of TN adjacent
// outputs in one row, SPR strips side by side.  The 64*POSW position lanes are
// replicated COW times, each replica ("co-wave group") taking its own TM
// output channels and sharing the LDS tile.
//
// LDS tile: [img][cc][TH+2][PITCH] floats, double buffered over chunks of CC
// input channels.  Column 0 of a row is input column w0*S-1, so a lane's strip
// starts at column strip*TN*S, which is 16-byte aligned when TN*S is a multiple of 4.
// ---------------------------------------------------------------------------
// MUL: the same kernel as an ordinary convolution, y = sum w * x (one v_fmac per term), for the regular
// stem layer that precedes the adder layers of a network.
// T: storage type of x and y (float, or bf16_t for the reduced-storage mode); the arithmetic is fp32 either way.
// PAIR (3x3 taps at stride 2 only): the strided 1x1 layer that reads the same x beside this layer (the downsample
// branch of a residual block, resnet20.py:66-70) is computed along with it -- its one tap is the centre tap of the
// 3x3 window, so the x values are in registers already: weights w_side (Co, Ci), output y_side and statistics
// stats_side shaped like y and stats.
template <class C, bool VEC = true, bool SUB = false, bool MUL = false, class T = float, bool PAIR = false>
__global__ __launch_bounds__(C::NTHREADS) void fwd_3x3_kernel(const T *__restrict__ x,
                                                                const float *__restrict__ w,
                                                                T *__restrict__ y,
                                                                double *__restrict__ stats, int N, int Ci,
                                                                int H, int W, int Co, int Ho, int Wo,
                                                                int tilesH, int tilesW, const Subsample sub,
                                                                const float *__restrict__ w_side = nullptr,
                                                                T *__restrict__ y_side = nullptr,
                                                                double *__restrict__ stats_side = nullptr) {
    static_assert(!PAIR || (C::S == 2 && C::KS == 3 && !MUL && !SUB), "the side layer is a strided 1x1 beside a strided 3x3");
    constexpr int TN = C::TN, TM = C::TM, CQ = C::CQ, S = C::S, STRIP = C::STRIP, KS = C::KS, KK = C::KK;
    extern __shared__ __align__(16) float smem[];

    int b = blockIdx.x;
    const int tw = b % tilesW; b /= tilesW;
    const int th = b % tilesH; b /= tilesH;
    const int n0 = b * C::NIMG;
    const int h0 = th * C::TH, w0 = tw * C::TW;

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int pw = wave % C::POSW, cw = wave / C::POSW;
    int p = pw * 64 + lane;
    const bool lane_ok = p < C::LANES;
    if (!lane_ok) p = C::LANES - 1;
    const int strip = p % C::SPR;
    const int row = (p / C::SPR) % C::TH;
    const int img = p / (C::SPR * C::TH);
    const int co_base = (blockIdx.y * C::COW + cw) * TM;
    const int K = Ci * KK;
    uniform_f32_ptr wc = as_uniform(w);

    // wave-uniform weight row offsets (clamped so tail channels read valid memory)
    int wrow[TM];
#pragma unroll
    for (int m = 0; m < TM; ++m)
        wrow[m] = __builtin_amdgcn_readfirstlane(min(co_base + m, Co - 1) * K);
    uniform_f32_ptr wsc = as_uniform(w_side);
    int wsrow[PAIR ? TM : 1];
    float tots[PAIR ? TM : 1][TN];   // PAIR: the side layer's sums (Ci terms each: one level)
    if constexpr (PAIR) {
#pragma unroll
        for (int m = 0; m < TM; ++m) {
            wsrow[m] = __builtin_amdgcn_readfirstlane(min(co_base + m, Co - 1) * Ci);
#pragma unroll
            for (int t = 0; t < TN; ++t) tots[m][t] = 0.f;
        }
    }

    // two-level sum: `acc` collects one channel chunk (<= 9*CC terms), `tot` the chunks, so the
    // rounding error grows with the square roots of the two lengths instead of with K
    float acc[TM][TN], tot[TM][TN];
#pragma unroll
    for (int m = 0; m < TM; ++m)
#pragma unroll
        for (int t = 0; t < TN; ++t) acc[m][t] = tot[m][t] = 0.f;

    const int lane_off = img * C::CC * C::PLANE + row * S * C::PITCH + strip * TN * S;
    const int nchunks = ceil_div(Ci, C::CC);

    TileStage<typename C::Patch> st;
    tile_fetch<typename C::Patch, VEC, SUB, T>(st, x, 0, Ci, n0, N, h0 * S - C::PAD, w0 * S, H, W, sub);
    {   // this workgroup's output channels: one contiguous run of weights
        const int co_blk = blockIdx.y * C::COW * TM;
        l2_warm(w + (size_t)co_blk * K, 1, 0, min(C::COW * TM, Co - co_blk) * K);
    }
    tile_commit<typename C::Patch>(st, smem);
    __syncthreads();

    for (int c = 0; c < nchunks; ++c) {
        const int ci0 = c * C::CC;
        if (c + 1 < nchunks) tile_fetch<typename C::Patch, VEC, SUB, T>(st, x, ci0 + C::CC, Ci, n0, N, h0 * S - C::PAD, w0 * S, H, W, sub);

        const float *lbase = smem + (c & 1) * C::BUF + lane_off;
        const int ccnt = min(C::CC, Ci - ci0);
        // Software pipeline over the input channels of the chunk: the strips of channel
        // group cc+CQ and the weights of the next output channel are requested right after
        // the first subtract of the current one, i.e. after the wait for the current
        // operands and with the rest of the arithmetic still ahead to hide the latency.
        float xr[2][CQ][KS][STRIP];
        float wv[2][CQ * KK];
        float wsv[2][CQ];   // PAIR: the side layer's weights, buffered like wv
#pragma unroll
        for (int q = 0; q < CQ; ++q)
#pragma unroll
            for (int i = 0; i < KS; ++i)
                lds_read_strip<STRIP, C::STRIP_ALIGN>(lbase + q * C::PLANE + i * C::PITCH, xr[0][q][i]);
#pragma unroll
        for (int e = 0; e < CQ * KK; ++e) wv[0][e] = wc[wrow[0] + ci0 * KK + e];
        if constexpr (PAIR) {
#pragma unroll
            for (int q = 0; q < CQ; ++q) wsv[0][q] = wsc[wsrow[0] + ci0 + q];
        }

        auto half = [&](const int cc, const int cur) {
            // cur = 0/1: which xr buffer holds channel group cc
            const int kofs = (ci0 + cc) * KK;
            const bool more = cc + CQ < ccnt;
            const int knext = more ? kofs + CQ * KK : kofs;  // clamped: stays inside the weight row
#pragma unroll
            for (int m = 0; m < TM; ++m) {
#pragma unroll
                for (int idx = 0; idx < CQ * KK * TN; ++idx) {
                    const int t = idx % TN, j = (idx / TN) % KS, i = (idx / TN / KS) % KS, q = idx / TN / KK;
                    if constexpr (MUL)
                        acc[m][t] = fmaf(wv[m & 1][q * KK + i * KS + j], xr[cur][q][i][t * S + j], acc[m][t]);
                    else
                        acc[m][t] -= fabsf(wv[m & 1][q * KK + i * KS + j] - xr[cur][q][i][t * S + j]);
                    if (idx == 0) {
                        __builtin_amdgcn_sched_barrier(0);
                        if (m + 1 < TM) {
#pragma unroll
                            for (int e = 0; e < CQ * KK; ++e) wv[(m + 1) & 1][e] = wc[wrow[m + 1] + kofs + e];
                            if constexpr (PAIR) {
#pragma unroll
                                for (int q2 = 0; q2 < CQ; ++q2) wsv[(m + 1) & 1][q2] = wsc[wsrow[m + 1] + ci0 + cc + q2];
                            }
                        } else {
#pragma unroll
                            for (int e = 0; e < CQ * KK; ++e) wv[(m + 1) & 1][e] = wc[wrow[0] + knext + e];
                            if constexpr (PAIR) {
#pragma unroll
                                for (int q2 = 0; q2 < CQ; ++q2)
                                    wsv[(m + 1) & 1][q2] = wsc[wsrow[0] + ci0 + (more ? cc + CQ : cc) + q2];
                            }
                        }
                        if (m == 0 && more) {
#pragma unroll
                            for (int q2 = 0; q2 < CQ; ++q2)
#pragma unroll
                                for (int i2 = 0; i2 < KS; ++i2)
                                    lds_read_strip<STRIP, C::STRIP_ALIGN>(
                                        lbase + (cc + CQ + q2) * C::PLANE + i2 * C::PITCH, xr[cur ^ 1][q2][i2]);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                if constexpr (PAIR) {   // the centre tap (1, 1) is the strided 1x1 layer's only tap
#pragma unroll
                    for (int q = 0; q < CQ; ++q)
#pragma unroll
                        for (int t = 0; t < TN; ++t) tots[m][t] -= fabsf(wsv[m & 1][q] - xr[cur][q][1][t * S + 1]);
                }
            }
        };
        static_assert(TM % 2 == 0, "weight double buffer assumes an even number of channels per lane");
#pragma unroll 1
        for (int cc = 0; cc < ccnt; cc += 2 * CQ) {
            half(cc, 0);
            if (cc + CQ < ccnt) half(cc + CQ, 1);
        }

#pragma unroll
        for (int m = 0; m < TM; ++m)
#pragma unroll
            for (int t = 0; t < TN; ++t) { tot[m][t] += acc[m][t]; acc[m][t] = 0.f; }

        if (c + 1 < nchunks) tile_commit<typename C::Patch>(st, smem + ((c + 1) & 1) * C::BUF);
        __syncthreads();
    }

    const int n = n0 + img, ho = h0 + row, wo = w0 + strip * TN;
    auto finish = [&](float (&tot)[TM][TN], T *__restrict__ y, double *__restrict__ stats) {
    if (stats) {
        // BatchNorm statistics of the layer's output on the way out: per wave and output channel the sums of
        // y and y*y over the wave's valid positions, in the partial-sum layout of the BatchNorm kernels
        // (slot = position wave of this launch, stats[(co * slots + slot) * 2 + {0, 1}]).
        // The lanes sum deviations from a pivot (lane 0's first value) in fp32 and lane 0 moves the sums back
        // to the origin in fp64, so the cancellation in E[y*y] - E[y]^2 happens in double precision.
        const bool row_ok = lane_ok && n < N && ho < Ho;
        const int slots = gridDim.x * C::POSW, slot = blockIdx.x * C::POSW + pw;
        float cnt = 0.f;
#pragma unroll
        for (int t = 0; t < TN; ++t) cnt += (row_ok && wo + t < Wo) ? 1.f : 0.f;
        const double count = (double)wave_sum_dpp(cnt);
        if constexpr (TM == 2 || TM == 4 || TM == 8) {
            // all 2 TM sums of the wave in one reduce-scatter: lane l < 2 TM ends with sum number j(l) (channel j / 2,
            // first or second moment j % 2), fetches the other moment of its channel from the lane that holds it,
            // and moves its own one back to the origin
            float sums[2 * TM], pivot[TM];
#pragma unroll
            for (int m = 0; m < TM; ++m) {
                pivot[m] = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(tot[m][0])));
                float s1 = 0.f, s2 = 0.f;
#pragma unroll
                for (int t = 0; t < TN; ++t)
                    if (row_ok && wo + t < Wo) {
                        const float dv = tot[m][t] - pivot[m];
                        s1 += dv;
                        s2 = fmaf(dv, dv, s2);
                    }
                sums[2 * m] = s1;
                sums[2 * m + 1] = s2;
            }
            const float mine = wave_sum_scatter<2 * TM>(sums, lane);
            constexpr int TOP = TM;   // lane bit that j % 2 comes from: j is the bit reversal of the lane
            const float other = __shfl_xor(mine, TOP, 64);
            const int j = wave_sum_scatter_index<2 * TM>(lane), m = j >> 1;
            float piv = pivot[0];
#pragma unroll
            for (int k = 1; k < TM; ++k) piv = m == k ? pivot[k] : piv;
            const double c = (double)piv;
            const int co = co_base + m;
            if (lane < 2 * TM && co < Co) {
                // j % 2 == 0: sum of y = d1 + n c;  else: sum of y*y = d2 + 2 c d1 + n c*c
                const double v = (j & 1) ? (double)mine + 2.0 * c * (double)other + count * c * c : (double)mine + count * c;
                stats[((size_t)co * slots + slot) * 2 + (j & 1)] = v;
            }
        } else {
#pragma unroll
            for (int m = 0; m < TM; ++m) {
                const float pivot = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(tot[m][0])));
                float s1 = 0.f, s2 = 0.f;
#pragma unroll
                for (int t = 0; t < TN; ++t)
                    if (row_ok && wo + t < Wo) {
                        const float dv = tot[m][t] - pivot;
                        s1 += dv;
                        s2 = fmaf(dv, dv, s2);
                    }
                const double d1 = (double)wave_sum_dpp(s1), d2 = (double)wave_sum_dpp(s2), c = (double)pivot;
                const int co = co_base + m;
                if (lane == 0 && co < Co) {
                    stats[((size_t)co * slots + slot) * 2] = d1 + count * c;
                    stats[((size_t)co * slots + slot) * 2 + 1] = d2 + 2.0 * c * d1 + count * c * c;
                }
            }
        }
    }
    if (lane_ok && n < N && ho < Ho) {
        const bool vec = TN % 4 == 0 && (Wo & 3) == 0 && wo + TN <= Wo;
#pragma unroll
        for (int m = 0; m < TM; ++m) {
            const int co = co_base + m;
            if (co < Co) {
                T *dst = y + (((size_t)n * Co + co) * Ho + ho) * Wo + wo;
                if (vec) {
#pragma unroll
                    for (int t = 0; t + 3 < TN; t += 4)
                        stf4(dst + t, make_float4(tot[m][t], tot[m][t + 1], tot[m][t + 2], tot[m][t + 3]));
                } else {
#pragma unroll
                    for (int t = 0; t < TN; ++t)
                        if (wo + t < Wo) stf(dst + t, tot[m][t]);
                }
            }
        }
    }
    };
    finish(tot, y, stats);
    if constexpr (PAIR) finish(tots, y_side, stats_side);
}

template <class C, bool VEC, bool SUB = false, bool MUL = false, class T = float>
static int launch_fwd_3x3_v(const T *x, const float *w, T *y, double *stats, const ConvDims &d,
                            hipStream_t s, const Subsample sub = Subsample{1, 0, 0, 0}) {
    const int tilesH = ceil_div(d.Ho, C::TH), tilesW = ceil_div(d.Wo, C::TW);
    const long gx = (long)ceil_div(d.N, C::NIMG) * tilesH * tilesW;
    const int gy = ceil_div(d.Co, C::TM * C::COW);
    if (gx > 0x7fffffffL) return ADDER_ERR_TOO_LARGE;
    if (int rc = allow_dynamic_lds<&fwd_3x3_kernel<C, VEC, SUB, MUL, T>>(C::LDS_BYTES)) return rc;
    hipLaunchKernelGGL((fwd_3x3_kernel<C, VEC, SUB, MUL, T>), dim3((unsigned)gx, gy), dim3(C::NTHREADS), C::LDS_BYTES, s, x, w, y,
                       stats, d.N, d.Ci, d.H, d.W, d.Co, d.Ho, d.Wo, tilesH, tilesW, sub);
    return check_launch();
}

template <class C, class T = float>
static int launch_fwd_3x3(const T *x, const float *w, T *y, double *stats, const ConvDims &d,
                          hipStream_t s) {
    // element-wise tile loads when the rows of the staged tensor are not whole groups of four
    if (d.W % 4 == 0) return launch_fwd_3x3_v<C, true, false, false, T>(x, w, y, stats, d, s);
    return launch_fwd_3x3_v<C, false, false, false, T>(x, w, y, stats, d, s);
}

// the same tile shapes as an ordinary convolution (3x3 / stride 1 / pad 1 only)
template <class C>
static int launch_mulconv_3x3(const float *x, const float *w, float *y, double *stats, const ConvDims &d,
                              hipStream_t s) {
    if (d.W % 4 == 0) return launch_fwd_3x3_v<C, true, false, true>(x, w, y, stats, d, s);
    return launch_fwd_3x3_v<C, false, false, true>(x, w, y, stats, d, s);
}

// partial-sum slots per channel the statistics epilogue of this tile shape writes
template <class C>
static int stats_slots_3x3(const ConvDims &d) {
    const long gx = (long)ceil_div(d.N, C::NIMG) * ceil_div(d.Ho, C::TH) * ceil_div(d.Wo, C::TW);
    return (int)(gx * C::POSW);
}

// Tile shapes per output width, picked by timing sweeps on MI355X.  What they have in common: a ResNet-20
// layer at batch 256 launches 2048-4096 waves in 256-512 workgroups of eight waves; a lane keeps only
// 2-4 output channels x 4 positions (few registers, short dependent chains); one pipeline unit is one
// output channel x one input channel (CQ = 1: 9 weights, 18*TN vector instructions), which keeps the two
// weight buffers far from the 102-SGPR limit (spilled SGPRs come back as v_readlane inside the hot loop)
// and works for odd channel counts too.
//                           TN SPR TH NIMG TM COW CC CQ S
using FwdW32   = Tile3x3Cfg<4, 8, 16, 1, 4, 4, 8, 1, 1>;    // outputs 32 wide: half an image x 16 channels
using FwdW16   = Tile3x3Cfg<4, 4, 16, 1, 4, 8, 16, 1, 1>;   // outputs 16 wide: one image x 32 channels
using FwdW8    = Tile3x3Cfg<4, 2, 8, 4, 2, 8, 16, 1, 1>;    // outputs 8 wide: four images x 16 channels
using FwdW16S2 = Tile3x3Cfg<2, 8, 16, 1, 4, 8, 8, 1, 2>;    // stride 2, outputs 16 wide: one image x 32 channels
using FwdW8S2  = Tile3x3Cfg<2, 4, 8, 2, 4, 8, 16, 1, 2>;    // stride 2, outputs 8 wide: two images x 32 channels
// ... with chunks of 8 input channels: two workgroups fit a CU's LDS instead of one, which pays from 128
// input channels on (512 -> 512 @14x14, batch 64: 740 -> 530 us; at 32 channels the extra barriers cost 2 %)
using FwdW8S2L = Tile3x3Cfg<2, 4, 8, 2, 4, 8, 8, 1, 2>;
// 1x1, stride 1: every (H, W) plane is one row of H*W positions; a unit is one output channel x 8 input
// channels (8 weights, 64 vector instructions), eight output-channel waves share the staged x tile.
using Fwd1x1   = Tile3x3Cfg<4, 64, 1, 1, 4, 8, 16, 8, 1, 1>;   // 256 positions of one image x 32 channels
using Fwd1x1s  = Tile3x3Cfg<4, 16, 1, 4, 4, 8, 16, 8, 1, 1>;   // planes of <= 64 positions: four images
// 1x1 with a stride: the tile loader gathers the sampled x element by element, which costs several times what the
// aligned float4 loads of a stride-1 plane cost, so a workgroup takes 64 output channels per staged tile instead of
// 32 (eight per lane, chunks of eight input channels to stay within 128 registers); ResNet-50's three downsample
// layers at batch 64: 538 -> 319, 621 -> 376, 591 -> 374 us.  (On stride-1 planes this shape is slower.)
using Fwd1x1sub = Tile3x3Cfg<4, 16, 1, 4, 8, 8, 8, 8, 1, 1>;   // 64 sampled positions of four images x 64 channels
// the same two with units of four input channels, for channel counts that are multiples of 4 but not of 8
// (DenseNet's multiples of 12)
using Fwd1x1q  = Tile3x3Cfg<4, 64, 1, 1, 4, 8, 16, 4, 1, 1>;
using Fwd1x1sq = Tile3x3Cfg<4, 16, 1, 4, 4, 8, 16, 4, 1, 1>;

// ... the same register tile in workgroups of four waves that cover fewer rows, for maps whose height is not a
// multiple of 16: 56 rows are 7 x 8, 28 rows 7 x 4 (ResNet-50 at batch 64: 64 -> 64 @56x56 340 -> 294 us,
// 128 -> 128 @28x28 330 -> 298 us); on 32 rows they are no faster than FwdW32
using FwdW32H8 = Tile3x3Cfg<4, 8, 8, 1, 4, 4, 8, 1, 1>;    // 8 rows of one image x 16 channels
using FwdW32H4 = Tile3x3Cfg<4, 8, 4, 2, 4, 4, 8, 1, 1>;    // 4 rows of two images x 16 channels
// rows per tile (16, 8 or 4) that pad a map of H rows least; the larger tile on a tie
static int rows_per_tile_w32(int H) {
    const int p16 = round_up(H, 16), p8 = round_up(H, 8), p4 = round_up(H, 4);
    return p16 <= p8 && p16 <= p4 ? 16 : (p8 <= p4 ? 8 : 4);
}

// which tiled kernel serves these dimensions (0 = none): 1..3 3x3 stride 1 by output width, 4..5 3x3 stride 2,
// 6..7 1x1 stride 1 by plane size, 8..9 1x1 with a stride (the sampled positions walked like a stride-1 plane),
// 10..13 = 6..9 with units of four input channels
static int fwd_tiled_variant(const ConvDims &d) {
    // (below 64 input channels the plain 1x1 kernel of conv1x1.hip is as fast or faster)
    if (d.kh == 1 && d.kw == 1 && d.pad == 0 && d.Ci % Fwd1x1q::CQ == 0 && d.Ci >= 64) {
        const int quad = d.Ci % Fwd1x1::CQ ? 4 : 0;
        // 256 positions of one image per workgroup, or 64 positions of four: whichever pads the plane less
        // (28x28 = 784 positions fill 64-wide tiles to 94 %, 256-wide ones to 77 %: 216 -> 169 us for 128 -> 512)
        const int plane = d.Ho * d.Wo;
        const bool wide = ceil_div(plane, Fwd1x1::TW) * Fwd1x1::TW <= ceil_div(plane, Fwd1x1s::TW) * Fwd1x1s::TW;
        if (d.stride == 1) return (wide ? 6 : 7) + quad;
        return (wide ? 8 : 9) + quad;
    }
    if (d.kh != 3 || d.kw != 3 || d.pad != 1) return 0;
    if (d.stride == 1) return d.Wo > 16 ? 1 : (d.Wo > 8 ? 2 : 3);
    if (d.stride == 2) return d.Wo > 8 ? 4 : 5;
    return 0;
}

// a 1x1 layer seen as N x Ci "images" of one row of Ho*Wo positions (the whole plane when the stride is 1)
static ConvDims as_one_row(const ConvDims &d) {
    ConvDims f = d;
    f.H = f.Ho = 1;
    f.W = f.Wo = d.Ho * d.Wo;
    f.stride = 1;
    return f;
}
static Subsample sampling_of(const ConvDims &d) { return Subsample{d.stride, d.Wo, d.W, d.H * d.W}; }

// A strided 3x3 / pad 1 layer and the strided 1x1 / pad 0 layer beside it (same x, same Co, Ho, Wo) in one launch;
// d describes the 3x3 layer.  Both outputs with their statistics (fwd_stats_slots(d) slots each).  Rows of whole
// float4 groups only; ADDER_ERR_UNSUPPORTED otherwise.
template <class C>
static int launch_fwd_pair_3x3(const float *x, const float *w, const float *w_side, float *y, float *y_side,
                               double *stats, double *stats_side, const ConvDims &d, hipStream_t s) {
    const int tilesH = ceil_div(d.Ho, C::TH), tilesW = ceil_div(d.Wo, C::TW);
    const long gx = (long)ceil_div(d.N, C::NIMG) * tilesH * tilesW;
    const int gy = ceil_div(d.Co, C::TM * C::COW);
    if (gx > 0x7fffffffL) return ADDER_ERR_TOO_LARGE;
    if (int rc = allow_dynamic_lds<&fwd_3x3_kernel<C, true, false, false, float, true>>(C::LDS_BYTES)) return rc;
    hipLaunchKernelGGL((fwd_3x3_kernel<C, true, false, false, float, true>), dim3((unsigned)gx, gy), dim3(C::NTHREADS),
                       C::LDS_BYTES, s, x, w, y, stats, d.N, d.Ci, d.H, d.W, d.Co, d.Ho, d.Wo, tilesH, tilesW,
                       Subsample{1, 0, 0, 0}, w_side, y_side, stats_side);
    return check_launch();
}

bool fwd_pair_supported(const ConvDims &d) {
    return d.kh == 3 && d.kw == 3 && d.pad == 1 && d.stride == 2 && d.W % 4 == 0 && d.H % 2 == 0 && d.W % 2 == 0;
}

int launch_fwd_pair(const float *x, const float *w, const float *w_side, float *y, float *y_side, double *stats,
                    double *stats_side, const ConvDims &d, hipStream_t s) {
    if (!fwd_pair_supported(d)) return ADDER_ERR_UNSUPPORTED;
    if (d.Wo > 8) return launch_fwd_pair_3x3<FwdW16S2>(x, w, w_side, y, y_side, stats, stats_side, d, s);
    return d.Ci >= 128 ? launch_fwd_pair_3x3<FwdW8S2L>(x, w, w_side, y, y_side, stats, stats_side, d, s)
                       : launch_fwd_pair_3x3<FwdW8S2>(x, w, w_side, y, y_side, stats, stats_side, d, s);
}

int fwd_stats_slots(const ConvDims &d) {
    switch (fwd_tiled_variant(d)) {
        case 1: switch (rows_per_tile_w32(d.Ho)) {
            case 16: return stats_slots_3x3<FwdW32>(d);
            case 8: return stats_slots_3x3<FwdW32H8>(d);
            default: return stats_slots_3x3<FwdW32H4>(d);
        }
        case 2: return stats_slots_3x3<FwdW16>(d);
        case 3: return stats_slots_3x3<FwdW8>(d);
        case 4: return stats_slots_3x3<FwdW16S2>(d);
        case 5: return stats_slots_3x3<FwdW8S2>(d);
        case 6: return stats_slots_3x3<Fwd1x1>(as_one_row(d));
        case 7: return stats_slots_3x3<Fwd1x1s>(as_one_row(d));
        case 8: case 9: return stats_slots_3x3<Fwd1x1sub>(as_one_row(d));
        case 10: return stats_slots_3x3<Fwd1x1q>(as_one_row(d));
        case 11: return stats_slots_3x3<Fwd1x1sq>(as_one_row(d));
        case 12: return stats_slots_3x3<Fwd1x1q>(as_one_row(d));
        case 13: return stats_slots_3x3<Fwd1x1sq>(as_one_row(d));
        default: return conv1x1_supported(d, nullptr, nullptr) ? fwd_1x1_stats_slots(d) : 0;
    }
}

// stats (nullable): per-channel partial sums of y and y*y, fwd_stats_slots(d) > 0 slots per channel
int launch_fwd(const float *x, const float *w, float *y, double *stats, const ConvDims &d, hipStream_t s) {
    // rows that are whole float4 groups are moved as float4 and need 16-byte aligned bases
    const bool k3p1 = d.kh == 3 && d.kw == 3 && d.pad == 1 &&
                      (d.W % 4 != 0 || (reinterpret_cast<uintptr_t>(x) & 15) == 0) &&
                      (d.Wo % 4 != 0 || (reinterpret_cast<uintptr_t>(y) & 15) == 0);
    const int variant = fwd_tiled_variant(d);
    const bool strided = variant == 8 || variant == 9 || variant == 12 || variant == 13;
    if (strided) {   // x is read element by element; y is a dense row per plane
        const ConvDims f = as_one_row(d);
        if (f.Wo % 4 != 0 || (reinterpret_cast<uintptr_t>(y) & 15) == 0) switch (variant) {
            case 8: case 9: return launch_fwd_3x3_v<Fwd1x1sub, false, true>(x, w, y, stats, f, s, sampling_of(d));
            case 12: return launch_fwd_3x3_v<Fwd1x1q, false, true>(x, w, y, stats, f, s, sampling_of(d));
            default: return launch_fwd_3x3_v<Fwd1x1sq, false, true>(x, w, y, stats, f, s, sampling_of(d));
        }
    } else if (variant >= 6) {
        const ConvDims f = as_one_row(d);
        if (f.W % 4 != 0 || ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0) switch (variant) {
            case 6: return launch_fwd_3x3<Fwd1x1>(x, w, y, stats, f, s);
            case 7: return launch_fwd_3x3<Fwd1x1s>(x, w, y, stats, f, s);
            case 10: return launch_fwd_3x3<Fwd1x1q>(x, w, y, stats, f, s);
            default: return launch_fwd_3x3<Fwd1x1sq>(x, w, y, stats, f, s);
        }
    }
    if (k3p1) {
        switch (variant) {
            case 1: switch (rows_per_tile_w32(d.Ho)) {
                case 16: return launch_fwd_3x3<FwdW32>(x, w, y, stats, d, s);
                case 8: return launch_fwd_3x3<FwdW32H8>(x, w, y, stats, d, s);
                default: return launch_fwd_3x3<FwdW32H4>(x, w, y, stats, d, s);
            }
            case 2: return launch_fwd_3x3<FwdW16>(x, w, y, stats, d, s);
            case 3: return launch_fwd_3x3<FwdW8>(x, w, y, stats, d, s);
            case 4: return launch_fwd_3x3<FwdW16S2>(x, w, y, stats, d, s);
            case 5: return d.Ci >= 128 ? launch_fwd_3x3<FwdW8S2L>(x, w, y, stats, d, s)
                                       : launch_fwd_3x3<FwdW8S2>(x, w, y, stats, d, s);
            default: break;
        }
    }
    if (conv1x1_supported(d, x, y)) {
        // (a tiled variant that was turned down for its alignment counted its statistics slots differently)
        if (stats && variant != 0) return ADDER_ERR_UNSUPPORTED;
        return launch_fwd_1x1(x, w, y, stats, d, s);
    }
    if (stats) return ADDER_ERR_UNSUPPORTED;   // the generic kernel has no statistics epilogue
    constexpr int TM = 8;
    const long total = (long)d.N * d.Ho * d.Wo;
    hipLaunchKernelGGL(fwd_generic_kernel<TM>, dim3((unsigned)ceil_div_l(total, 256), ceil_div(d.Co, TM)),
                       dim3(256), 0, s, x, w, y, d);
    return check_launch();
}

// bfloat16 storage: the tiled 3x3 / pad-1 kernels (stride 1 or 2), the generic kernel for everything else
int launch_fwd_bf16(const bf16_t *x, const float *w, bf16_t *y, const ConvDims &d, hipStream_t s) {
    const bool k3p1 = d.kh == 3 && d.kw == 3 && d.pad == 1 &&
                      (d.W % 4 != 0 || (reinterpret_cast<uintptr_t>(x) & 7) == 0) &&
                      (d.Wo % 4 != 0 || (reinterpret_cast<uintptr_t>(y) & 7) == 0);
    if (k3p1) {
        const int variant = d.stride == 1 ? (d.Wo > 16 ? 1 : (d.Wo > 8 ? 2 : 3)) : (d.stride == 2 ? (d.Wo > 8 ? 4 : 5) : 0);
        switch (variant) {
            case 1: return launch_fwd_3x3<FwdW32, bf16_t>(x, w, y, nullptr, d, s);
            case 2: return launch_fwd_3x3<FwdW16, bf16_t>(x, w, y, nullptr, d, s);
            case 3: return launch_fwd_3x3<FwdW8, bf16_t>(x, w, y, nullptr, d, s);
            case 4: return launch_fwd_3x3<FwdW16S2, bf16_t>(x, w, y, nullptr, d, s);
            case 5: return d.Ci >= 128 ? launch_fwd_3x3<FwdW8S2L, bf16_t>(x, w, y, nullptr, d, s)
                                       : launch_fwd_3x3<FwdW8S2, bf16_t>(x, w, y, nullptr, d, s);
            default: break;
        }
    }
    constexpr int TM = 8;
    const long total = (long)d.N * d.Ho * d.Wo;
    hipLaunchKernelGGL((fwd_generic_kernel<TM, bf16_t>), dim3((unsigned)ceil_div_l(total, 256), ceil_div(d.Co, TM)),
                       dim3(256), 0, s, x, w, y, d);
    return check_launch();
}

// An ordinary convolution y = sum w * x through the tiled forward kernels: 3x3 / stride 1 / pad 1 only
// (ADDER_ERR_UNSUPPORTED elsewhere).  stats as in launch_fwd; the slot count is fwd_stats_slots(d).
int launch_mulconv_fwd(const float *x, const float *w, float *y, double *stats, const ConvDims &d, hipStream_t s) {
    const bool ok = d.kh == 3 && d.kw == 3 && d.pad == 1 && d.stride == 1 &&
                    (d.W % 4 != 0 || ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0);
    if (!ok) return ADDER_ERR_UNSUPPORTED;
    switch (fwd_tiled_variant(d)) {
        case 1: switch (rows_per_tile_w32(d.Ho)) {   // (the statistics slots are counted per tile shape)
            case 16: return launch_mulconv_3x3<FwdW32>(x, w, y, stats, d, s);
            case 8: return launch_mulconv_3x3<FwdW32H8>(x, w, y, stats, d, s);
            default: return launch_mulconv_3x3<FwdW32H4>(x, w, y, stats, d, s);
        }
        case 2: return launch_mulconv_3x3<FwdW16>(x, w, y, stats, d, s);
        case 3: return launch_mulconv_3x3<FwdW8>(x, w, y, stats, d, s);
        default: return ADDER_ERR_UNSUPPORTED;
    }
}

}  // namespace adder
