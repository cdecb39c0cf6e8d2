// Input gradient of the AdderNet convolution, NCHW, gather form (no atomics):
//   gx[n,ci,hi,wi] = sum_{co,i,j} hardtanh(w[co,ci,i,j] - x[n,ci,hi,wi]) * gy[n,co,ho,wo]
//   with ho = (hi + p - i)/s, wo = (wi + p - j)/s when those divide exactly and
//   fall inside the output; taps that land in the padding are dropped.
// Replaces the grad_i half of adder_cuda/adder.cu:194-272 (CONV_BACKWARD),
// adder.cu:133-192 (CONV_INPUT), and the permute + F.fold (col2im) autograd
// runs after them for adder.py:32-33.  hardtanh is adder.cu:17.
//
// The generic kernel spends three fp32 VALU instructions per term: v_sub (SGPR
// weight - own x), v_med3 (clamp), v_fma (times gy).  The tiled kernels spend two:
//   hardtanh(w - x) = 2 * sat(0.5 * w + (0.5 - 0.5 * x)) - 1,   sat = clamp to [0, 1],
// and sat is the clamp output modifier of v_fma_f32, so with cr = 0.5 - 0.5 x kept per
// own position the term is  v_fma_f32 d, s_w, 0.5, v_cr clamp ; v_fmac_f32 acc, d, g  and
//   gx = 2 * sum d * g - sum g,
// where the second sum (over the output channels and the taps a position met) does not
// depend on the input channel: it is a box sum of the channel-summed gy tile, which the
// workgroup collects once per chunk in LDS.  d lies in [0, 1], so the sums keep the
// magnitude they have in the three-instruction form; 0.5 * w + cr is exact wherever
// w - x is (small integers, the golden fixtures), and the rounding of cr is at most
// one ulp of (|x| + 1) / 2 -- for terms that do not saturate, |x| <= |w| + 1.
// Lanes own input positions, so cr and the accumulators stay in registers for the whole
// kernel, weights are SGPR operands, and the haloed gy tile is staged in LDS with zeros
// outside the output so invalid taps vanish without predication.
#include "common.hpp"
#include "tile3x3.hpp"

namespace adder {

// Partial-sum slots a workgroup of the BatchNorm-linked kernels leaves per channel: one per position wave -- except
// that two position waves add theirs through LDS first (the consumer of the sums, the weight-gradient kernel of the
// layer in front, reads all slots of its channels in every one of its workgroups: half the slots, half that prologue).
template <class C>
constexpr int bn_slots_per_wg() { return C::POSW == 2 ? 1 : C::POSW; }

// ---------------------------------------------------------------------------
// Generic kernel: any kernel size / stride / padding.
// ---------------------------------------------------------------------------
template <int TM, class T = float>
__global__ __launch_bounds__(256) void grad_x_generic_kernel(const T *__restrict__ gy,
                                                             const T *__restrict__ x,
                                                             const float *__restrict__ w,
                                                             T *__restrict__ gx, ConvDims d) {
    const int total = d.N * d.H * d.W;
    int pos = blockIdx.x * 256 + threadIdx.x;
    const bool active = pos < total;
    if (!active) pos = total - 1;
    const int wi = pos % d.W;
    const int hi = (pos / d.W) % d.H;
    const int n = pos / (d.W * d.H);
    const int ci0 = blockIdx.y * TM;
    const int KK = d.kh * d.kw;
    const int K = d.Ci * KK;
    uniform_f32_ptr wc = as_uniform(w);

    float xr[TM], acc[TM], tot[TM];   // two-level sum: acc holds at most 16 output channels' taps
    int wofs[TM];
#pragma unroll
    for (int m = 0; m < TM; ++m) {
        const int ci = min(ci0 + m, d.Ci - 1);
        xr[m] = ldf(x + (((size_t)n * d.Ci + ci) * d.H + hi) * d.W + wi);
        acc[m] = tot[m] = 0.f;
        wofs[m] = ci * KK;
    }
    const T *gn = gy + (size_t)n * d.Co * d.Ho * d.Wo;
    for (int co = 0; co < d.Co; ++co) {
        for (int i = 0; i < d.kh; ++i) {
            const int th = hi + d.pad - i;
            const int ho = th / d.stride;
            const bool hv = th >= 0 && ho * d.stride == th && ho < d.Ho;
            for (int j = 0; j < d.kw; ++j) {
                const int tw = wi + d.pad - j;
                const int wo = tw / d.stride;
                const bool v = hv && tw >= 0 && wo * d.stride == tw && wo < d.Wo;
                const float g = v ? ldf(gn + ((size_t)co * d.Ho + ho) * d.Wo + wo) : 0.f;
                const int kofs = co * K + i * d.kw + j;
#pragma unroll
                for (int m = 0; m < TM; ++m)
                    acc[m] = fmaf(hardtanh(wc[kofs + wofs[m]] - xr[m]), g, acc[m]);
            }
        }
        if ((co & 15) == 15 || co + 1 == d.Co) {
#pragma unroll
            for (int m = 0; m < TM; ++m) { tot[m] += acc[m]; acc[m] = 0.f; }
        }
    }
    if (active) {
#pragma unroll
        for (int m = 0; m < TM; ++m)
            if (ci0 + m < d.Ci) stf(gx + (((size_t)n * d.Ci + ci0 + m) * d.H + hi) * d.W + wi, tot[m]);
    }
}

// ---------------------------------------------------------------------------
// Tiled kernel for 3x3, stride 1, pad 1.  Same tile geometry as the forward
// kernel with the roles swapped: the LDS tile holds gy (chunks of CC output
// channels, reduction axis), a lane owns TN input positions x TM input
// channels, COW wave groups take different input channels.
//   gx[hi,wi] += hardtanh(w[co,ci,i,j] - x[hi,wi]) * gy[hi+1-i, wi+1-j]
// In tile coordinates (row 0 = h0-1, column 0 = w0-1) that is row+2-i, t+2-j.
// ---------------------------------------------------------------------------
// SUB (single tap only): x and gx are sampled tensors (see Subsample); the kernel walks the sampled
// positions as one row per plane, reads x there, and stores each result together with the zeros of the
// s x s block of input positions around it that the layer never read.
// T: storage type of gy, x, gx and gadd (float, or bf16_t for the reduced-storage mode).
// FUSE: the statistics pass of the backward of the BatchNorm in front of the layer is done here (the in_* fields
// of adder_bn_links): the result is masked with x > 0 (bn.in_relu) and its per-channel sums are left in
// bn.in_part, (Ci, gridDim.x * bn_slots_per_wg, 2) floats.  Float storage, rows of whole float4 groups, no sampling.
template <class C, bool VEC = true, bool SAT = true, bool SUB = false, class T = float, bool FUSE = false>
__global__ __launch_bounds__(C::NTHREADS, 4) void grad_x_3x3s1_kernel(const T *__restrict__ gy,
                                                                   const T *__restrict__ x,
                                                                   const float *__restrict__ w,
                                                                   T *__restrict__ gx, int N, int Ci,
                                                                   int H, int W, int Co, int tilesH,
                                                                   int tilesW, const Subsample sub,
                                                                   const T *__restrict__ gadd,
                                                                   const adder_bn_links bn) {
    static_assert(!SUB || C::KS == 1, "sampling is for single-tap layers");
    static_assert(!FUSE || (VEC && !SUB && sizeof(T) == 4 && C::TM * C::TN <= 32),
                  "the BatchNorm link belongs to the float kernels that read whole rows");
    constexpr int TN = C::TN, TM = C::TM, CQ = C::CQ, KS = C::KS, KK = C::KK;
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
    // The last channel group is shifted down to end at Ci (Ci >= TM is a launch precondition) so
    // that the TM channels of a wave are always valid and their weights contiguous; channels
    // below ci_first belong to the previous group and are not stored.
    const int ci_first = (blockIdx.y * C::COW + cw) * TM;
    const int ci_base = __builtin_amdgcn_readfirstlane(min(ci_first, Ci - TM));
    const int K = Ci * KK;
    uniform_f32_ptr wc = as_uniform(w) + ci_base * KK;

    const int n = n0 + img, hi = h0 + row, wi0 = w0 + strip * TN;
    const bool pos_ok = lane_ok && n < N && hi < H;
    const int nc = min(n, N - 1), hc = min(hi, H - 1);

    // cr = 0.5 - 0.5 x of the own positions (x itself in the three-instruction form, SAT = false) and the
    // accumulators live in registers for the whole kernel (two-level sum: acc collects one chunk of
    // output channels, tot the chunks)
    float cr[TM][TN], acc[TM][TN], tot[TM][TN];
    int xoff[TN];   // offset of the own positions in their plane
#pragma unroll
    for (int t = 0; t < TN; ++t) {
        const int pos = min(wi0 + t, W - 1);
        if constexpr (SUB) {
            const int ho = pos / sub.wv;
            xoff[t] = ho * sub.s * sub.pitch + (pos - ho * sub.wv) * sub.s;
        } else {
            xoff[t] = hc * W + pos;
        }
    }
    const int xplane = SUB ? sub.plane : H * W;
    unsigned xpos = 0;   // FUSE: bit m * TN + t = (x > 0) of the own positions
#pragma unroll
    for (int m = 0; m < TM; ++m) {
        const int ci = ci_base + m;
        const T *src = x + ((size_t)nc * Ci + ci) * xplane;
#pragma unroll
        for (int t = 0; t < TN; ++t) {
            const float xv = ldf(src + xoff[t]);
            cr[m][t] = SAT ? fmaf(-0.5f, xv, 0.5f) : xv;
            acc[m][t] = tot[m][t] = 0.f;
            if constexpr (FUSE) xpos |= (xv > 0.f ? 1u : 0u) << (m * TN + t);
        }
    }
    // (pinned here: left alone, the compiler moves the comparisons down to where the bits are used and keeps all
    // the x values in registers through the main loop for that)
    if constexpr (FUSE) asm volatile("" : "+v"(xpos));
    // per tile position, the sum of gy over all output channels: every thread owns GITER elements of the
    // plane and adds them up in double in registers (one conversion and one add per chunk -- the sum is taken
    // off a sum of the same size at the end, so its rounding counts), the plane itself is written once
    constexpr int GN = C::NIMG * C::PLANE, GITER = ceil_div(GN, C::NTHREADS);
    float *gplane = smem + 2 * C::BUF;
    double gsum[GITER];
#pragma unroll
    for (int it = 0; it < GITER; ++it) gsum[it] = 0.0;

    const int lane_off = img * C::CC * C::PLANE + row * C::PITCH + strip * TN;
    const int nchunks = ceil_div(Co, C::CC);

    TileStage<typename C::Patch> st;
    tile_fetch<typename C::Patch, VEC, false, T>(st, gy, 0, Co, n0, N, h0 - C::PAD, w0, H, W);
    {   // this workgroup's input channels: one run of weights per output channel
        const int ci_blk = min((int)blockIdx.y * C::COW * TM, Ci - TM);
        l2_warm(w + ci_blk * KK, Co, K, min(C::COW * TM, Ci - ci_blk) * KK);
    }
    tile_commit<typename C::Patch>(st, smem);
    __syncthreads();

    for (int c = 0; c < nchunks; ++c) {
        const int co0 = c * C::CC;
        if (c + 1 < nchunks) tile_fetch<typename C::Patch, VEC, false, T>(st, gy, co0 + C::CC, Co, n0, N, h0 - C::PAD, w0, H, W);

        const float *lbase = smem + (c & 1) * C::BUF + lane_off;
        const int ccnt = min(C::CC, Co - co0);
        if constexpr (KS == 1 && CQ > 1) {
            // Single tap: a unit of one output channel would be TM * TN terms, too few instructions to hide the wait
            // for its operands behind -- a unit is CQ output channels here (CQ * TM weights, CQ gy strips).
            constexpr int CU = CQ;
            static_assert(C::CC % CU == 0, "a chunk holds whole units (planes past Co are staged as zeros)");
            float gr[2][CU][TN];
            float wv[2][CU * TM];
#pragma unroll
            for (int u = 0; u < CU; ++u) {
                lds_read_strip<TN, C::STRIP_ALIGN>(lbase + u * C::PLANE, gr[0][u]);
                const int wrow = min(co0 + u, Co - 1) * K;   // rows past Co meet gy = 0: any finite weight will do
#pragma unroll
                for (int e = 0; e < TM; ++e) wv[0][u * TM + e] = wc[wrow + e];
            }
            auto unit = [&](const int cc, const int cur) {
                const bool more = cc + CU < ccnt;
                const int cnext = more ? cc + CU : cc;
#pragma unroll
                for (int idx = 0; idx < CU * TM * TN; ++idx) {
                    const int t = idx % TN, mm = (idx / TN) % TM, u = idx / (TN * TM);
                    const float wgt = wv[cur][u * TM + mm];
                    const float d = SAT ? sat01(fmaf(wgt, 0.5f, cr[mm][t])) : hardtanh(wgt - cr[mm][t]);
                    acc[mm][t] = fmaf(d, gr[cur][u][t], acc[mm][t]);
                    if (idx == 0) {
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int u2 = 0; u2 < CU; ++u2) {
                            const int wrow = min(co0 + cnext + u2, Co - 1) * K;
#pragma unroll
                            for (int e = 0; e < TM; ++e) wv[cur ^ 1][u2 * TM + e] = wc[wrow + e];
                        }
                        if (more) {
#pragma unroll
                            for (int u2 = 0; u2 < CU; ++u2)
                                lds_read_strip<TN, C::STRIP_ALIGN>(lbase + (cc + CU + u2) * C::PLANE, gr[cur ^ 1][u2]);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            };
#pragma unroll 1
            for (int cc = 0; cc < ccnt; cc += 2 * CU) {
                unit(cc, 0);
                if (cc + CU < ccnt) unit(cc + CU, 1);
            }
        } else {
            // Software pipeline over the output channels of the chunk, in units of HM input channels
            // (9*HM contiguous weights): right after the first instruction of a unit, i.e. after the
            // wait for its operands, the weights of the next unit and (once per output channel) the
            // gy strips of the next channel are requested.
            static_assert(CQ == 1, "this pipeline takes one output channel per step");
            // input channels per unit: keeps ~100 vector instructions per unit and both weight
            // buffers (2 * 9 * HM SGPRs) well inside the scalar register file
            constexpr int HM = KS == 1 ? TM : (TN >= 4 ? 1 : 2), NU = TM / HM, HW = HM * KK;
            static_assert(TM % HM == 0 && (NU % 2 == 0 || NU == 1), "one unit or an even number of units per output channel");
            float gr[2][KS][TN + KS - 1];
            float wv[2][HW];
#pragma unroll
            for (int i = 0; i < KS; ++i) lds_read_strip<TN + KS - 1, C::STRIP_ALIGN>(lbase + i * C::PITCH, gr[0][i]);
#pragma unroll
            for (int e = 0; e < HW; ++e) wv[0][e] = wc[co0 * K + e];

            auto one_channel = [&](const int cc, const int cur) {
                const int kofs = (co0 + cc) * K;
                const bool more = cc + 1 < ccnt;
                const int knext = more ? kofs + K : kofs;
#pragma unroll
                for (int h = 0; h < NU; ++h) {
                    // weight buffer of this unit: the buffers alternate from unit to unit, also across channels
                    const int wb = (cur * (NU & 1) + h) & 1;
#pragma unroll
                    for (int idx = 0; idx < HM * KK * TN; ++idx) {
                        const int t = idx % TN, j = (idx / TN) % KS, i = (idx / TN / KS) % KS, mm = idx / TN / KK;
                        const int m = h * HM + mm;
                        const float wgt = wv[wb][mm * KK + i * KS + j];
                        const float d = SAT ? sat01(fmaf(wgt, 0.5f, cr[m][t])) : hardtanh(wgt - cr[m][t]);
                        acc[m][t] = fmaf(d, gr[cur][KS - 1 - i][t + KS - 1 - j], acc[m][t]);
                        if (idx == 0) {
                            __builtin_amdgcn_sched_barrier(0);
                            if (h + 1 < NU) {
#pragma unroll
                                for (int e = 0; e < HW; ++e) wv[wb ^ 1][e] = wc[kofs + (h + 1) * HW + e];
                            } else {
#pragma unroll
                                for (int e = 0; e < HW; ++e) wv[wb ^ 1][e] = wc[knext + e];
                            }
                            if (h == 0 && more) {
#pragma unroll
                                for (int i2 = 0; i2 < KS; ++i2)
                                    lds_read_strip<TN + KS - 1, C::STRIP_ALIGN>(lbase + (cc + 1) * C::PLANE + i2 * C::PITCH,
                                                                           gr[cur ^ 1][i2]);
                            }
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                }
            };
#pragma unroll 1
            for (int cc = 0; cc < ccnt; cc += 2) {
                one_channel(cc, 0);
                if (cc + 1 < ccnt) one_channel(cc + 1, 1);
                // the two-instruction form folds its first-level sums every eight output channels (72 terms): with
                // 144-term first levels its worst element sat at 0.71 of the parity tolerance for 1152 terms per
                // output, with 72-term ones at 0.51
                if (SAT && KS == 3 && ((cc + 2) & 7) == 0 && cc + 2 < ccnt) {
#pragma unroll
                    for (int m = 0; m < TM; ++m)
#pragma unroll
                        for (int t = 0; t < TN; ++t) { tot[m][t] += acc[m][t]; acc[m][t] = 0.f; }
                }
            }

        }
        // a single tap makes a chunk only CC terms long: fold every fourth chunk, so that the two levels of
        // the sum stay comparable in length (2048 output channels: 64 x 32 instead of 16 x 128)
        constexpr int FOLD = KS == 1 ? 4 : 1;
        if (FOLD == 1 || (c & (FOLD - 1)) == FOLD - 1 || c + 1 == nchunks) {
#pragma unroll
            for (int m = 0; m < TM; ++m)
#pragma unroll
                for (int t = 0; t < TN; ++t) { tot[m][t] += acc[m][t]; acc[m][t] = 0.f; }
        }

        // channel sum of this chunk (planes past Co were staged as zeros)
        if constexpr (SAT) {
#pragma unroll
            for (int it = 0; it < GITER; ++it) {
                const int e = threadIdx.x + it * C::NTHREADS;
                if (GN % C::NTHREADS == 0 || e < GN) {
                    const float *src = smem + (c & 1) * C::BUF + (e / C::PLANE) * C::CC * C::PLANE + e % C::PLANE;
                    float sum = 0.f;
#pragma unroll
                    for (int cc = 0; cc < C::CC; ++cc) sum += src[cc * C::PLANE];
                    gsum[it] += (double)sum;
                }
            }
        }

        if (c + 1 < nchunks) tile_commit<typename C::Patch>(st, smem + ((c + 1) & 1) * C::BUF);
        __syncthreads();
    }

    // FUSE: what the epilogue needs from memory is asked for now, behind the last barrier of the main loop, so that
    // it arrives while the correction below is worked out (the main loop's registers are free from here on).
    // The strips' offset is formed from values the compiler cannot connect with the loads of x at the top -- it would
    // keep their sixteen 64-bit addresses in registers through the whole main loop.  Rows are whole strips here; a
    // strip beyond the row (a tile wider than the tensor) reads the row's last one.  Every lane loads, from inside
    // the tensor; invalid lanes are dropped when the sums are taken.
    // With bn.in_gamma / in_beta (a BatchNorm whose output went through nothing but the ReLU, x = relu(gamma * xhat +
    // beta)) the BatchNorm's input is not read at all: where the ReLU passed, xhat = (x - beta) / gamma comes from the
    // x this lane holds, and where it did not, dz is zero.  Channels whose |gamma| is too small for that division
    // (below max(1, |beta|) / 64) read the input after all, in the epilogue.
    // The per-channel constants come through the scalar cache (nothing writes them while the kernel runs), also
    // asked for here: as vector loads in the epilogue they would share the counter of the stores there, and every
    // channel's loads would wait for the previous channel's sums to reach memory.
    float bx[FUSE ? TM : 1][TN], ga[FUSE ? TM : 1][TN];
    float bn_mu[FUSE ? TM : 1], bn_rs[FUSE ? TM : 1], bn_g[FUSE ? TM : 1], bn_be[FUSE ? TM : 1];
    int pofs = 0;
    if constexpr (FUSE) {
        static_assert(!FUSE || TN == 2 || TN == 4, "the strips are read as one float2 / float4");
        pofs = (nc * Ci + ci_base) * (H * W) + hc * W + min(wi0, W - TN);
        asm volatile("" : "+v"(pofs));
#pragma unroll
        for (int m = 0; m < TM; ++m) {
            bn_mu[m] = as_uniform(bn.in_mean)[ci_base + m];
            bn_rs[m] = as_uniform(bn.in_rstd)[ci_base + m];
            bn_g[m] = bn.in_gamma ? as_uniform(bn.in_gamma)[ci_base + m] : 0.f;
            bn_be[m] = bn.in_gamma ? as_uniform(bn.in_beta)[ci_base + m] : 0.f;
            if (!bn.in_gamma) {
                global_read_strip<TN, TN>(bn.in_x + pofs + m * (H * W), bx[m]);
            } else {
                // (x, as this lane holds it, in the place of the BatchNorm's input: no registers of its own)
#pragma unroll
                for (int t = 0; t < TN; ++t) bx[m][t] = cr[m][t];
            }
            if (gadd) global_read_strip<TN, TN>(reinterpret_cast<const float *>(gadd) + pofs + m * (H * W), ga[m]);
        }
    }

    // sum over (co, taps) of the gy values a position met = box sum of the channel-sum plane
    if constexpr (SAT) {
#pragma unroll
        for (int it = 0; it < GITER; ++it) {
            const int e = threadIdx.x + it * C::NTHREADS;
            if (GN % C::NTHREADS == 0 || e < GN) gplane[e] = (float)gsum[it];
        }
        __syncthreads();
        float gs[KS][TN + KS - 1];
#pragma unroll
        for (int i = 0; i < KS; ++i)
            lds_read_strip<TN + KS - 1, C::STRIP_ALIGN>(gplane + img * C::PLANE + row * C::PITCH + strip * TN + i * C::PITCH,
                                                        gs[i]);
#pragma unroll
        for (int t = 0; t < TN; ++t) {
            float sg = 0.f;
#pragma unroll
            for (int i = 0; i < KS; ++i)
#pragma unroll
                for (int j = 0; j < KS; ++j) sg += gs[i][t + j];
#pragma unroll
            for (int m = 0; m < TM; ++m) tot[m][t] = fmaf(2.f, tot[m][t], -sg);
        }
    }

    if constexpr (FUSE) {
        // x = relu(bn(in_x) [+ residual]): what leaves here is the gradient of the BatchNorm's output before the
        // ReLU, dz = (gx + gadd) * [x > 0], and per channel and position wave the sums of dz and dz * xhat in the
        // partial-sum layout of the BatchNorm kernels (a wave's 64 * TN terms in fp32, the rest in fp64).
        // With one round of workgroups on the chip nothing overlaps this epilogue, so it is kept short: one mask bit
        // per position decides what counts (inside the tensor, an own channel, the ReLU passed); per term one
        // select, one add, one subtract and one multiply-add; the scale of xhat is applied to the wave's sum.
        constexpr bool MERGE = C::POSW == 2;   // see bn_slots_per_wg
        const int slots = gridDim.x * bn_slots_per_wg<C>(), slot = MERGE ? (int)blockIdx.x : (int)blockIdx.x * C::POSW + pw;
        __shared__ float pw_sums[MERGE ? C::COW * 2 * TM : 1];
        unsigned keep = 0;
#pragma unroll
        for (int t = 0; t < TN; ++t) keep |= (pos_ok && wi0 + t < W ? 1u : 0u) << t;
        {
            unsigned all = 0;
#pragma unroll
            for (int m = 0; m < TM; ++m) all |= (ci_base + m >= ci_first ? keep : 0u) << (m * TN);
            keep = bn.in_relu ? all & xpos : all;
        }
        if (gadd) {
#pragma unroll
            for (int m = 0; m < TM; ++m)
#pragma unroll
                for (int t = 0; t < TN; ++t) tot[m][t] += ga[m][t];
        }
        float sums[2 * TM];   // per channel: dz, dz * xhat
#pragma unroll
        for (int m = 0; m < TM; ++m) {
            // |gamma| large enough that the rounding of x - beta stays ~1e-5 of xhat
            const bool from_x = bn.in_gamma && fabsf(bn_g[m]) >= 0x1p-6f * fmaxf(1.f, fabsf(bn_be[m]));
            if (bn.in_gamma && !from_x) global_read_strip<TN, TN>(bn.in_x + pofs + m * (H * W), bx[m]);
            // xhat = (bx - off) * scale, with bx = cr where xhat comes from x (x = 1 - 2 cr in the two-instruction
            // form: xhat = (cr - (1 - beta) / 2) * (-2 / gamma))
            const float off = from_x ? (SAT ? 0.5f - 0.5f * bn_be[m] : bn_be[m]) : bn_mu[m];
            const float scale = from_x ? (SAT ? -2.f : 1.f) * __builtin_amdgcn_rcpf(bn_g[m]) : bn_rs[m];
            float a1 = 0.f, a2 = 0.f;
#pragma unroll
            for (int t = 0; t < TN; ++t) {
                // (what is zeroed for being outside the tensor or another group's channel is not stored below)
                const int bit = __builtin_amdgcn_sbfe((int)keep, m * TN + t, 1);   // 0 or all ones
                const float v = __int_as_float(__float_as_int(tot[m][t]) & bit);
                tot[m][t] = v;
                a1 += v;
                a2 = fmaf(v, bx[m][t] - off, a2);
            }
            sums[2 * m] = a1;
            sums[2 * m + 1] = a2 * scale;
        }
        // all 2 TM wave sums at once; lane l ends with the one numbered wave_sum_scatter_index(l)
        const float total = wave_sum_scatter<2 * TM>(sums, lane);
        // Only stores from here on, and nothing that would have to be waited for between them: loads and stores
        // share one counter, in order, so a wait for any later load is a wait for every store before it -- a round
        // trip to memory per channel.
        if (!MERGE && lane < 2 * TM) {
            const int j = wave_sum_scatter_index<2 * TM>(lane), ci = ci_base + (j >> 1);
            if (ci >= ci_first) bn.in_part[((size_t)ci * slots + slot) * 2 + (j & 1)] = total;
        }
        if (MERGE && pw == 1 && lane < 2 * TM) pw_sums[cw * 2 * TM + lane] = total;
        if (pos_ok && wi0 < W) {
#pragma unroll
            for (int m = 0; m < TM; ++m) {
                if (ci_base + m < ci_first) continue;
                float *dst = reinterpret_cast<float *>(gx) + pofs + m * (H * W);
                if constexpr (TN == 4) stf4(dst, make_float4(tot[m][0], tot[m][1], tot[m][2], tot[m][3]));
                else stf2(dst, make_float2(tot[m][0], tot[m][1]));
            }
        }
        if constexpr (MERGE) {   // the second position wave's sums, added behind the stores of dz
            __syncthreads();
            if (pw == 0 && lane < 2 * TM) {
                const int j = wave_sum_scatter_index<2 * TM>(lane), ci = ci_base + (j >> 1);
                if (ci >= ci_first)
                    bn.in_part[((size_t)ci * slots + slot) * 2 + (j & 1)] = total + pw_sums[cw * 2 * TM + lane];
            }
        }
        return;
    }

    // A second gradient of the same tensor (a residual shortcut) is added on the way out -- all of it is read before
    // the first store: loads and stores share one counter, in order, so a wait for a load behind a store is a wait
    // for the store's round trip to memory as well.
    if (gadd && pos_ok) {
#pragma unroll
        for (int m = 0; m < TM; ++m) {
            const T *src = gadd + (((size_t)n * Ci + ci_base + m) * H + hi) * W + wi0;
            if (TN % 4 == 0 && (W & 3) == 0 && wi0 + TN <= W) {
#pragma unroll
                for (int t = 0; t < TN; t += 4) {
                    const float4 a = ldf4(src + t);
                    tot[m][t] += a.x; tot[m][t + 1] += a.y; tot[m][t + 2] += a.z; tot[m][t + 3] += a.w;
                }
            } else {
#pragma unroll
                for (int t = 0; t < TN; ++t)
                    if (wi0 + t < W) tot[m][t] += ldf(src + t);
            }
        }
    }
    if (pos_ok) {
#pragma unroll
        for (int m = 0; m < TM; ++m) {
            const int ci = ci_base + m;
            if (ci >= ci_first) {
                if constexpr (SUB) {
                    T *plane = gx + ((size_t)n * Ci + ci) * sub.plane;
                    const int rows = sub.plane / sub.pitch;
#pragma unroll
                    for (int t = 0; t < TN; ++t) {
                        if (wi0 + t >= W) continue;
                        const int r0 = xoff[t] / sub.pitch, c0 = xoff[t] - r0 * sub.pitch;
                        for (int a = 0; a < sub.s && r0 + a < rows; ++a)
                            for (int b = 0; b < sub.s && c0 + b < sub.pitch; ++b)
                                stf(plane + xoff[t] + a * sub.pitch + b, (a | b) ? 0.f : tot[m][t]);
                    }
                    continue;
                }
                const size_t o = (((size_t)n * Ci + ci) * H + hi) * W + wi0;
                T *dst = gx + o;
                if (TN % 4 == 0 && (W & 3) == 0 && wi0 + TN <= W) {
#pragma unroll
                    for (int t = 0; t < TN; t += 4)
                        stf4(dst + t, make_float4(tot[m][t], tot[m][t + 1], tot[m][t + 2], tot[m][t + 3]));
                } else {
#pragma unroll
                    for (int t = 0; t < TN; ++t)
                        if (wi0 + t < W) stf(dst + t, tot[m][t]);
                }
            }
        }
    }
}

// The two-instruction form doubles a sum of products whose factors lie in [0, 1] and takes a second
// sum off it, which about doubles the rounding error of the three-instruction form.  Measured against fp64
// as the worst element's share of the parity tolerance |err| <= 1e-4 + 1e-5 |gx| over 8 seeds x {Kaiming,
// N(0,1)} weights x input scale {1, 5}, first-level sums of at most 72 terms: 0.26 at 576 terms per output,
// 0.51 at 1152, 0.62 at 2304 (256 output channels x 9 taps; 0.96 with 144-term first levels: too close), where
// the three-instruction form sits at 0.45, and at 0.54 for 4608.  Layers with more than 1152 terms per output
// therefore keep the three-instruction form.  Single-tap layers stop at 1024: their chunks are CC terms long, not 9 * CC, so the second level of the
// sum is long and carries the full magnitude (0.46 at 1024 with the first level folded every fourth chunk).
static constexpr int kSatMaxTerms = 1152, kSatMaxTerms1x1 = 1024;

static const adder_bn_links kNoLinks{};

template <class C, bool VEC, bool SAT, bool SUB = false, class T = float, bool FUSE = false>
static int launch_grad_x_3x3s1_v(const T *gy, const T *x, const float *w, T *gx,
                               const ConvDims &d, hipStream_t s, const Subsample sub = Subsample{1, 0, 0, 0},
                               const T *gadd = nullptr, const adder_bn_links &bn = kNoLinks) {
    const int tilesH = ceil_div(d.H, C::TH), tilesW = ceil_div(d.W, C::TW);
    const long gxd = (long)ceil_div(d.N, C::NIMG) * tilesH * tilesW;
    const int gyd = ceil_div(d.Ci, C::TM * C::COW);
    if (gxd > 0x7fffffffL) return ADDER_ERR_TOO_LARGE;
    if (FUSE && (!bn.in_part || bn.in_slots != gxd * bn_slots_per_wg<C>())) return ADDER_ERR_BAD_SHAPE;
    constexpr int LDS_BYTES = C::LDS_BYTES + C::NIMG * C::PLANE * 4;   // two gy chunk buffers + the channel-sum plane
    if (int rc = allow_dynamic_lds<&grad_x_3x3s1_kernel<C, VEC, SAT, SUB, T, FUSE>>(LDS_BYTES)) return rc;
    hipLaunchKernelGGL((grad_x_3x3s1_kernel<C, VEC, SAT, SUB, T, FUSE>), dim3((unsigned)gxd, gyd), dim3(C::NTHREADS),
                       LDS_BYTES, s, gy, x, w, gx, d.N, d.Ci, d.H, d.W, d.Co, tilesH, tilesW, sub, gadd, bn);
    return check_launch();
}

// the same with the in_* half of adder_bn_links (float tensors with rows of whole float4 groups)
template <class C>
static int launch_grad_x_3x3s1_bn(const float *gy, const float *x, const float *w, float *gx, const ConvDims &d,
                                  hipStream_t s, const float *gadd, const adder_bn_links &bn) {
    if (d.Co * C::KK > (C::KS == 1 ? kSatMaxTerms1x1 : kSatMaxTerms))
        return launch_grad_x_3x3s1_v<C, true, false, false, float, true>(gy, x, w, gx, d, s, Subsample{1, 0, 0, 0}, gadd, bn);
    return launch_grad_x_3x3s1_v<C, true, true, false, float, true>(gy, x, w, gx, d, s, Subsample{1, 0, 0, 0}, gadd, bn);
}

// picks the element-wise tile loads (rows of the staged tensor that are not whole float4 groups) and the
// three-instruction form (more terms per output than kSatMaxTerms)
template <class C, bool SUB = false, class T = float>
static int launch_grad_x_3x3s1(const T *gy, const T *x, const float *w, T *gx,
                               const ConvDims &d, hipStream_t s, const T *gadd = nullptr,
                               const Subsample sub = Subsample{1, 0, 0, 0}) {
    const bool vec = d.W % 4 == 0;
    if (d.Co * C::KK > (C::KS == 1 ? kSatMaxTerms1x1 : kSatMaxTerms))
        return vec ? launch_grad_x_3x3s1_v<C, true, false, SUB, T>(gy, x, w, gx, d, s, sub, gadd)
                   : launch_grad_x_3x3s1_v<C, false, false, SUB, T>(gy, x, w, gx, d, s, sub, gadd);
    return vec ? launch_grad_x_3x3s1_v<C, true, true, SUB, T>(gy, x, w, gx, d, s, sub, gadd)
               : launch_grad_x_3x3s1_v<C, false, true, SUB, T>(gy, x, w, gx, d, s, sub, gadd);
}

// ---------------------------------------------------------------------------
// Tiled kernel for 3x3, stride 2, pad 1.
//
// With stride 2 only taps of matching parity reach an input position:
//   even row 2a   : i = 1 -> ho = a            odd row 2a+1 : i = 0 -> ho = a+1, i = 2 -> ho = a
// and likewise for columns, so a 2 x 2 block of input positions sees the 9
// taps exactly once between its four members.  A lane owns 2 rows x TNW
// columns (TNW even) x TM input channels; the gy patch it needs is rows
// a, a+1 and columns b .. b+TNW/2 of the output (halo on the bottom / right
// only, zero beyond the output).
// ---------------------------------------------------------------------------
template <int TNW_, int BPR_, int TH_, int NIMG_, int TM_, int CIW_, int CC_>
struct GradX3x3S2Cfg {
    static constexpr int TNW = TNW_, BPR = BPR_, TH = TH_, NIMG = NIMG_, TM = TM_, CIW = CIW_, CC = CC_;
    static constexpr int TW = TNW * BPR;
    static constexpr int LANES = NIMG * (TH / 2) * BPR;
    static constexpr int POSW = ceil_div(LANES, 64);
    static constexpr int NTHREADS = 64 * POSW * CIW;
    using Patch = PatchCfg<NIMG, CC, TH / 2 + 1, TW / 2, 0, 1, NTHREADS>;
    static constexpr int PITCH = Patch::PITCH, PLANE = Patch::PLANE, BUF = Patch::BUF;
    static constexpr int LDS_BYTES = 2 * BUF * 4;
    static constexpr int GSTRIP = TNW / 2 + 1;
    static_assert(TNW % 2 == 0 && TH % 2 == 0, "lanes own 2 x 2 parity blocks");
};

// FUSE, bn: as in the stride-1 kernel.
// PAIR (with FUSE): the input gradient of the strided 1x1 layer that reads the same x beside this layer (the
// downsample branch of a residual block) is added in here: bn.side_gy is that layer's output gradient (shaped like
// gy), bn.side_w its weights (Co, Ci).  Its one tap is the centre tap of the 3x3 window, so its gradient lands on
// the even positions -- element (0, 0) of every lane's 2 x 2 block -- and takes the gy value of the block's own
// output position.  side_gy is staged in LDS chunk by chunk beside gy (a load from memory per lane and output
// channel, asked for one channel ahead, has a few hundred cycles to arrive and needs a microsecond: +10 us).
template <class C, bool VEC = true, bool SAT = true, class T = float, bool FUSE = false, bool PAIR = false>
__global__ __launch_bounds__(C::NTHREADS) void grad_x_3x3s2_kernel(const T *__restrict__ gy,
                                                                   const T *__restrict__ x,
                                                                   const float *__restrict__ w,
                                                                   T *__restrict__ gx, int N, int Ci,
                                                                   int H, int W, int Co, int Ho, int Wo,
                                                                   int tilesH, int tilesW,
                                                                   const T *__restrict__ gadd,
                                                                   const adder_bn_links bn) {
    constexpr int TNW = C::TNW, TM = C::TM, GSTRIP = C::GSTRIP;
    static_assert(!FUSE || (VEC && sizeof(T) == 4 && TM * 2 * TNW <= 32), "the BatchNorm link belongs to the float kernels");
    static_assert(!PAIR || (FUSE && TNW == 2), "the side layer rides on the linked kernel; one 2 x 2 block per lane");
    extern __shared__ __align__(16) float smem[];

    int b = blockIdx.x;
    const int tw = b % tilesW; b /= tilesW;
    const int th = b % tilesH; b /= tilesH;
    const int n0 = b * C::NIMG;
    const int h0 = th * C::TH, w0 = tw * C::TW;  // both even

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int pw = wave % C::POSW, cw = wave / C::POSW;
    int p = pw * 64 + lane;
    const bool lane_ok = p < C::LANES;
    if (!lane_ok) p = C::LANES - 1;
    const int bcol = p % C::BPR;
    const int brow = (p / C::BPR) % (C::TH / 2);
    const int img = p / (C::BPR * (C::TH / 2));
    // as in the stride-1 kernel: the last channel group is shifted down so all TM channels are valid
    const int ci_first = (blockIdx.y * C::CIW + cw) * TM;
    const int ci_base = __builtin_amdgcn_readfirstlane(min(ci_first, Ci - TM));
    const int K = Ci * 9;
    uniform_f32_ptr wc = as_uniform(w) + ci_base * 9;

    const int n = n0 + img, hi0 = h0 + 2 * brow, wi0 = w0 + bcol * TNW;
    const int nc = min(n, N - 1);

    float cr[TM][2][TNW], acc[TM][2][TNW], tot[TM][2][TNW];   // cr = 0.5 - 0.5 x, as in the stride-1 kernel
    unsigned xpos = 0;   // FUSE: bit (m * 2 + rp) * TNW + t = (x > 0) of the own positions
#pragma unroll
    for (int m = 0; m < TM; ++m) {
        const int ci = ci_base + m;
#pragma unroll
        for (int rp = 0; rp < 2; ++rp) {
            const T *src = x + (((size_t)nc * Ci + ci) * H + min(hi0 + rp, H - 1)) * W;
#pragma unroll
            for (int t = 0; t < TNW; ++t) {
                const float xv = ldf(src + min(wi0 + t, W - 1));
                cr[m][rp][t] = SAT ? fmaf(-0.5f, xv, 0.5f) : xv;
                acc[m][rp][t] = tot[m][rp][t] = 0.f;
                if constexpr (FUSE) xpos |= (xv > 0.f ? 1u : 0u) << ((m * 2 + rp) * TNW + t);
            }
        }
    }
    if constexpr (FUSE) asm volatile("" : "+v"(xpos));   // pinned here, as in the stride-1 kernel
    constexpr int GN = C::NIMG * C::PLANE, GITER = ceil_div(GN, C::NTHREADS);
    float *gplane = smem + 2 * C::BUF;   // per tile position, the sum of gy over all output channels
    double gsum[GITER];                  // ... collected in double in registers, as in the stride-1 kernel
#pragma unroll
    for (int it = 0; it < GITER; ++it) gsum[it] = 0.0;

    const int lane_off = img * C::CC * C::PLANE + brow * C::PITCH + bcol * (TNW / 2);
    const int nchunks = ceil_div(Co, C::CC);
    const int hb = h0 / 2, wb = w0 / 2;
    // PAIR: the side layer's gy chunks, staged like gy behind the channel-sum plane (the lane needs the value at its
    // own output position: no halo involved), its weights for the lane's TM channels, and the sum of its gy for the
    // correction at the end
    uniform_f32_ptr wsc = as_uniform(bn.side_w) + ci_base;
    float *side_lds = gplane + GN;
    float gd_next = 0.f, gd_sum = 0.f;

    TileStage<typename C::Patch> st, st_side;
    tile_fetch<typename C::Patch, VEC, false, T>(st, gy, 0, Co, n0, N, hb, wb, Ho, Wo);
    if constexpr (PAIR) tile_fetch<typename C::Patch, VEC, false, T>(st_side, bn.side_gy, 0, Co, n0, N, hb, wb, Ho, Wo);
    {   // this workgroup's input channels: one run of weights per output channel
        const int ci_blk = min((int)blockIdx.y * C::CIW * TM, Ci - TM);
        l2_warm(w + ci_blk * 9, Co, K, min(C::CIW * TM, Ci - ci_blk) * 9);
    }
    tile_commit<typename C::Patch>(st, smem);
    if constexpr (PAIR) tile_commit<typename C::Patch>(st_side, side_lds);
    __syncthreads();

    for (int c = 0; c < nchunks; ++c) {
        const int co0 = c * C::CC;
        if (c + 1 < nchunks) {
            tile_fetch<typename C::Patch, VEC, false, T>(st, gy, co0 + C::CC, Co, n0, N, hb, wb, Ho, Wo);
            if constexpr (PAIR)
                tile_fetch<typename C::Patch, VEC, false, T>(st_side, bn.side_gy, co0 + C::CC, Co, n0, N, hb, wb, Ho, Wo);
        }

        const float *lbase = smem + (c & 1) * C::BUF + lane_off;
        const float *sbase = side_lds + (c & 1) * C::BUF + lane_off;   // (PAIR)
        const int ccnt = min(C::CC, Co - co0);
        // same software pipeline as the stride-1 kernel: units of HM input channels, next unit's
        // weights and next channel's gy strips requested right after a unit's first instruction
        constexpr int HM = 2, NU = TM / HM, HW = HM * 9, TERMS = 9 * (TNW / 2);
        static_assert(TM % HM == 0 && NU % 2 == 0, "even number of units per output channel");
        // (row parity, tap row i, gy row) and (col parity, tap col j, gy col offset)
        constexpr int RP[3] = {0, 1, 1}, RI[3] = {1, 0, 2}, RG[3] = {0, 1, 0};
        float gr[2][2][GSTRIP];
        float wv[2][HW];
        float wsv[2][PAIR ? TM : 1];   // PAIR: the side layer's weights of this and the next output channel
#pragma unroll
        for (int r = 0; r < 2; ++r) lds_read_strip<GSTRIP, 1>(lbase + r * C::PITCH, gr[0][r]);
#pragma unroll
        for (int e = 0; e < HW; ++e) wv[0][e] = wc[co0 * K + e];
        if constexpr (PAIR) {
#pragma unroll
            for (int m = 0; m < TM; ++m) wsv[0][m] = wsc[co0 * Ci + m];
            gd_next = sbase[0];
        }

        auto one_channel = [&](const int cc, const int cur) {
            const int kofs = (co0 + cc) * K;
            const bool more = cc + 1 < ccnt;
            const int knext = more ? kofs + K : kofs;
            float gd = 0.f;
            if constexpr (PAIR) gd = gd_next;
#pragma unroll
            for (int h = 0; h < NU; ++h) {
#pragma unroll
                for (int idx = 0; idx < HM * TERMS; ++idx) {
                    const int cp = idx % (TNW / 2), bb = (idx / (TNW / 2)) % 3, a = (idx / (TNW / 2) / 3) % 3,
                              mm = idx / TERMS;
                    const int m = h * HM + mm, t = 2 * cp + RP[bb];
                    const float wgt = wv[h & 1][mm * 9 + RI[a] * 3 + RI[bb]];
                    const float d = SAT ? sat01(fmaf(wgt, 0.5f, cr[m][RP[a]][t])) : hardtanh(wgt - cr[m][RP[a]][t]);
                    acc[m][RP[a]][t] = fmaf(d, gr[cur][RG[a]][cp + RG[bb]], acc[m][RP[a]][t]);
                    if (idx == 0) {
                        __builtin_amdgcn_sched_barrier(0);
                        if (h + 1 < NU) {
#pragma unroll
                            for (int e = 0; e < HW; ++e) wv[(h + 1) & 1][e] = wc[kofs + (h + 1) * HW + e];
                        } else {
#pragma unroll
                            for (int e = 0; e < HW; ++e) wv[0][e] = wc[knext + e];
                        }
                        if (h == 0 && more) {
#pragma unroll
                            for (int r = 0; r < 2; ++r)
                                lds_read_strip<GSTRIP, 1>(lbase + (cc + 1) * C::PLANE + r * C::PITCH, gr[cur ^ 1][r]);
                        }
                        if constexpr (PAIR) {
                            if (h == 0) {   // the next output channel's side operands (the last one asks for itself again)
                                const int cn = min(co0 + cc + 1, Co - 1);
                                gd_next = sbase[(more ? cc + 1 : cc) * C::PLANE];
#pragma unroll
                                for (int m2 = 0; m2 < TM; ++m2) wsv[cur ^ 1][m2] = wsc[cn * Ci + m2];
                            }
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
            if constexpr (PAIR) {
#pragma unroll
                for (int m = 0; m < TM; ++m) {
                    const float wgt = wsv[cur][m];
                    const float d = SAT ? sat01(fmaf(wgt, 0.5f, cr[m][0][0])) : hardtanh(wgt - cr[m][0][0]);
                    acc[m][0][0] = fmaf(d, gd, acc[m][0][0]);
                }
                gd_sum += gd;
            }
        };
#pragma unroll 1
        for (int cc = 0; cc < ccnt; cc += 2) {
            one_channel(cc, 0);
            if (cc + 1 < ccnt) one_channel(cc + 1, 1);
        }

#pragma unroll
        for (int m = 0; m < TM; ++m)
#pragma unroll
            for (int rp = 0; rp < 2; ++rp)
#pragma unroll
                for (int t = 0; t < TNW; ++t) { tot[m][rp][t] += acc[m][rp][t]; acc[m][rp][t] = 0.f; }

        // channel sum of this chunk (planes past Co were staged as zeros)
        if constexpr (SAT) {
#pragma unroll
            for (int it = 0; it < GITER; ++it) {
                const int e = threadIdx.x + it * C::NTHREADS;
                if (GN % C::NTHREADS == 0 || e < GN) {
                    const float *src = smem + (c & 1) * C::BUF + (e / C::PLANE) * C::CC * C::PLANE + e % C::PLANE;
                    float sum = 0.f;
#pragma unroll
                    for (int cc = 0; cc < C::CC; ++cc) sum += src[cc * C::PLANE];
                    gsum[it] += (double)sum;
                }
            }
        }

        if (c + 1 < nchunks) {
            tile_commit<typename C::Patch>(st, smem + ((c + 1) & 1) * C::BUF);
            if constexpr (PAIR) tile_commit<typename C::Patch>(st_side, side_lds + ((c + 1) & 1) * C::BUF);
        }
        __syncthreads();
    }

    // FUSE: the epilogue's loads, issued here as in the stride-1 kernel
    float bx[FUSE ? TM : 1][2][TNW], ga[FUSE ? TM : 1][2][TNW];
    int pofs[2] = {0, 0};
    if constexpr (FUSE) {
        static_assert(!FUSE || TNW == 2, "the strips are read as one float2");
#pragma unroll
        for (int rp = 0; rp < 2; ++rp) {
            pofs[rp] = ((nc * Ci + ci_base) * H + min(hi0 + rp, H - 1)) * W + min(wi0, W - TNW);
            asm volatile("" : "+v"(pofs[rp]));
#pragma unroll
            for (int m = 0; m < TM; ++m) {
                global_read_strip<TNW, TNW>(bn.in_x + pofs[rp] + m * (H * W), bx[m][rp]);
                if (gadd)
                    global_read_strip<TNW, TNW>(reinterpret_cast<const float *>(gadd) + pofs[rp] + m * (H * W), ga[m][rp]);
            }
        }
    }

    // clamp = 2 * sat - 1: take off the sum of the gy values each position met (same taps as above)
    if constexpr (SAT) {
#pragma unroll
        for (int it = 0; it < GITER; ++it) {
            const int e = threadIdx.x + it * C::NTHREADS;
            if (GN % C::NTHREADS == 0 || e < GN) gplane[e] = (float)gsum[it];
        }
        __syncthreads();
        constexpr int RP[3] = {0, 1, 1}, RG[3] = {0, 1, 0};
        float gs[2][GSTRIP], sg[2][TNW];
#pragma unroll
        for (int r = 0; r < 2; ++r)
            lds_read_strip<GSTRIP, 1>(gplane + img * C::PLANE + (brow + r) * C::PITCH + bcol * (TNW / 2), gs[r]);
#pragma unroll
        for (int rp = 0; rp < 2; ++rp)
#pragma unroll
            for (int t = 0; t < TNW; ++t) sg[rp][t] = 0.f;
#pragma unroll
        for (int a = 0; a < 3; ++a)
#pragma unroll
            for (int bb = 0; bb < 3; ++bb)
#pragma unroll
                for (int cp = 0; cp < TNW / 2; ++cp) sg[RP[a]][2 * cp + RP[bb]] += gs[RG[a]][cp + RG[bb]];
#pragma unroll
        for (int m = 0; m < TM; ++m)
#pragma unroll
            for (int rp = 0; rp < 2; ++rp)
#pragma unroll
                for (int t = 0; t < TNW; ++t) tot[m][rp][t] = fmaf(2.f, tot[m][rp][t], -sg[rp][t]);
        if constexpr (PAIR) {   // the side layer's terms met the even position only
#pragma unroll
            for (int m = 0; m < TM; ++m) tot[m][0][0] -= gd_sum;
        }
    }

    if constexpr (FUSE) {
        // dz = (gx + gadd) * [x > 0] and its per-channel sums, as in the stride-1 kernel (one mask bit per position,
        // every load before the first store)
        constexpr bool MERGE = C::POSW == 2;   // see bn_slots_per_wg
        const int slots = gridDim.x * bn_slots_per_wg<C>(), slot = MERGE ? (int)blockIdx.x : (int)blockIdx.x * C::POSW + pw;
        __shared__ float pw_sums[MERGE ? C::CIW * 2 * TM : 1];
        unsigned keep = 0;
#pragma unroll
        for (int rp = 0; rp < 2; ++rp)
#pragma unroll
            for (int t = 0; t < TNW; ++t)
                keep |= (lane_ok && n < N && hi0 + rp < H && wi0 + t < W ? 1u : 0u) << (rp * TNW + t);
        {
            unsigned all = 0;
#pragma unroll
            for (int m = 0; m < TM; ++m) all |= (ci_base + m >= ci_first ? keep : 0u) << (m * 2 * TNW);
            keep = bn.in_relu ? all & xpos : all;
        }
        float sums[2 * TM];   // per channel: dz, dz * xhat
#pragma unroll
        for (int m = 0; m < TM; ++m) {
            const float mu = as_uniform(bn.in_mean)[ci_base + m], rs = as_uniform(bn.in_rstd)[ci_base + m];
            float a1 = 0.f, a2 = 0.f;
#pragma unroll
            for (int rp = 0; rp < 2; ++rp) {
#pragma unroll
                for (int t = 0; t < TNW; ++t) {
                    const int bit = __builtin_amdgcn_sbfe((int)keep, (m * 2 + rp) * TNW + t, 1);   // 0 or all ones
                    const float g = gadd ? tot[m][rp][t] + ga[m][rp][t] : tot[m][rp][t];
                    const float v = __int_as_float(__float_as_int(g) & bit);
                    tot[m][rp][t] = v;
                    a1 += v;
                    a2 = fmaf(v, bx[m][rp][t] - mu, a2);
                }
            }
            sums[2 * m] = a1;
            sums[2 * m + 1] = a2 * rs;
        }
        const float total = wave_sum_scatter<2 * TM>(sums, lane);
        if (!MERGE && lane < 2 * TM) {
            const int j = wave_sum_scatter_index<2 * TM>(lane), ci = ci_base + (j >> 1);
            if (ci >= ci_first) bn.in_part[((size_t)ci * slots + slot) * 2 + (j & 1)] = total;
        }
        if (MERGE && pw == 1 && lane < 2 * TM) pw_sums[cw * 2 * TM + lane] = total;
        if (lane_ok && n < N && wi0 < W) {
#pragma unroll
            for (int m = 0; m < TM; ++m) {
                if (ci_base + m < ci_first) continue;
#pragma unroll
                for (int rp = 0; rp < 2; ++rp)
                    if (hi0 + rp < H)
                        stf2(reinterpret_cast<float *>(gx) + pofs[rp] + m * (H * W), make_float2(tot[m][rp][0], tot[m][rp][1]));
            }
        }
        if constexpr (MERGE) {   // the second position wave's sums, added behind the stores of dz
            __syncthreads();
            if (pw == 0 && lane < 2 * TM) {
                const int j = wave_sum_scatter_index<2 * TM>(lane), ci = ci_base + (j >> 1);
                if (ci >= ci_first)
                    bn.in_part[((size_t)ci * slots + slot) * 2 + (j & 1)] = total + pw_sums[cw * 2 * TM + lane];
            }
        }
        return;
    }

    // (a second gradient of the same tensor is read before the first store, as in the stride-1 kernel)
    if (gadd && lane_ok && n < N) {
#pragma unroll
        for (int m = 0; m < TM; ++m)
#pragma unroll
            for (int rp = 0; rp < 2; ++rp) {
                if (hi0 + rp >= H) continue;
                const T *src = gadd + (((size_t)n * Ci + ci_base + m) * H + hi0 + rp) * W + wi0;
                if ((W & 1) == 0 && wi0 + TNW <= W) {
#pragma unroll
                    for (int t = 0; t < TNW; t += 2) {
                        const float2 a = ldf2(src + t);
                        tot[m][rp][t] += a.x; tot[m][rp][t + 1] += a.y;
                    }
                } else {
#pragma unroll
                    for (int t = 0; t < TNW; ++t)
                        if (wi0 + t < W) tot[m][rp][t] += ldf(src + t);
                }
            }
    }
    if (lane_ok && n < N) {
#pragma unroll
        for (int m = 0; m < TM; ++m) {
            const int ci = ci_base + m;
            if (ci < ci_first) continue;
#pragma unroll
            for (int rp = 0; rp < 2; ++rp) {
                const int hi = hi0 + rp;
                if (hi >= H) continue;
                const size_t o = (((size_t)n * Ci + ci) * H + hi) * W + wi0;
                T *dst = gx + o;
                if ((W & 1) == 0 && wi0 + TNW <= W) {
#pragma unroll
                    for (int t = 0; t < TNW; t += 2) stf2(dst + t, make_float2(tot[m][rp][t], tot[m][rp][t + 1]));
                } else {
#pragma unroll
                    for (int t = 0; t < TNW; ++t)
                        if (wi0 + t < W) stf(dst + t, tot[m][rp][t]);
                }
            }
        }
    }
}

template <class C, bool VEC, bool SAT, class T = float, bool FUSE = false, bool PAIR = false>
static int launch_grad_x_3x3s2_v(const T *gy, const T *x, const float *w, T *gx,
                               const ConvDims &d, hipStream_t s, const T *gadd, const adder_bn_links &bn = kNoLinks) {
    const int tilesH = ceil_div(d.H, C::TH), tilesW = ceil_div(d.W, C::TW);
    const long gxd = (long)ceil_div(d.N, C::NIMG) * tilesH * tilesW;
    const int gyd = ceil_div(d.Ci, C::TM * C::CIW);
    if (gxd > 0x7fffffffL) return ADDER_ERR_TOO_LARGE;
    if (FUSE && (!bn.in_part || bn.in_slots != gxd * bn_slots_per_wg<C>())) return ADDER_ERR_BAD_SHAPE;
    // two gy chunk buffers + the channel-sum plane (+ two chunk buffers of the side layer's gy)
    constexpr int LDS_BYTES = C::LDS_BYTES + C::NIMG * C::PLANE * 4 + (PAIR ? C::LDS_BYTES : 0);
    static_assert(LDS_BYTES <= 48 * 1024, "raise the dynamic LDS limit for this tile");
    hipLaunchKernelGGL((grad_x_3x3s2_kernel<C, VEC, SAT, T, FUSE, PAIR>), dim3((unsigned)gxd, gyd), dim3(C::NTHREADS),
                       LDS_BYTES, s, gy, x, w, gx, d.N, d.Ci, d.H, d.W, d.Co, d.Ho, d.Wo, tilesH, tilesW, gadd, bn);
    return check_launch();
}

template <class C>
static int launch_grad_x_3x3s2_bn(const float *gy, const float *x, const float *w, float *gx, const ConvDims &d,
                                  hipStream_t s, const float *gadd, const adder_bn_links &bn) {
    if (bn.side_gy) {   // (H, W even: the two layers' outputs have one size)
        if (d.Co * 4 > kSatMaxTerms)
            return launch_grad_x_3x3s2_v<C, true, false, float, true, true>(gy, x, w, gx, d, s, gadd, bn);
        return launch_grad_x_3x3s2_v<C, true, true, float, true, true>(gy, x, w, gx, d, s, gadd, bn);
    }
    if (d.Co * 4 > kSatMaxTerms) return launch_grad_x_3x3s2_v<C, true, false, float, true>(gy, x, w, gx, d, s, gadd, bn);
    return launch_grad_x_3x3s2_v<C, true, true, float, true>(gy, x, w, gx, d, s, gadd, bn);
}

template <class C, class T = float>
static int launch_grad_x_3x3s2(const T *gy, const T *x, const float *w, T *gx,
                               const ConvDims &d, hipStream_t s, const T *gadd) {
    // element-wise tile loads when the rows of the staged tensor are not whole groups of four
    const bool vec = d.Wo % 4 == 0;
    if (d.Co * 4 > kSatMaxTerms)   // an input position meets at most four of the nine taps per output channel
        return vec ? launch_grad_x_3x3s2_v<C, true, false, T>(gy, x, w, gx, d, s, gadd)
                   : launch_grad_x_3x3s2_v<C, false, false, T>(gy, x, w, gx, d, s, gadd);
    return vec ? launch_grad_x_3x3s2_v<C, true, true, T>(gy, x, w, gx, d, s, gadd)
               : launch_grad_x_3x3s2_v<C, false, true, T>(gy, x, w, gx, d, s, gadd);
}

//                              TNW BPR TH NIMG TM CIW CC
using GxS2W32 = GradX3x3S2Cfg<2, 16, 16, 1, 4, 4, 16>;   // inputs 32 wide: half an image x 16 channels, 8 waves
using GxS2W16 = GradX3x3S2Cfg<2, 8, 16, 1, 4, 8, 16>;    // inputs 16 wide: one image x 32 channels, 8 waves

// Stride-1 tile shapes, picked by timing sweeps on MI355X: eight waves per workgroup, four input channels
// x 2-4 positions per lane (few registers; more channels per lane were 20 % slower on every map size).
//                        TN SPR TH NIMG TM COW CC CQ
using GxW32 = Tile3x3Cfg<4, 8, 16, 1, 4, 4, 8, 1>;    // inputs 32 wide: half an image x 16 channels
using GxW16 = Tile3x3Cfg<4, 4, 16, 1, 4, 8, 16, 1>;   // inputs 16 wide: one image x 32 channels
using GxW8  = Tile3x3Cfg<2, 4, 8, 2, 4, 8, 16, 1>;    // inputs 8 wide: two images x 32 channels
// 1x1, stride 1: (H, W) planes walked as one row; a unit is one output channel x the lane's 8 input channels
using Gx1x1  = Tile3x3Cfg<2, 64, 1, 1, 8, 8, 16, 2, 1, 1>;    // 128 positions of one image x 64 channels
using Gx1x1s = Tile3x3Cfg<4, 16, 1, 4, 8, 8, 16, 1, 1, 1>;    // planes of <= 64 positions: four images
using Gx1x1t = Tile3x3Cfg<2, 32, 1, 2, 4, 8, 16, 8, 1, 1>;    // ... two images x 32 channels, where Gx1x1s would leave CUs idle

// Planes of <= 64 positions with few images x few channel blocks: the smaller workgroup tile, so that every CU
// gets work (512 -> 2048 @7x7 at batch 64: 760 us with the larger tile, 305 with this one; from about two
// workgroups per CU on the larger tile is as fast or faster).
static bool small_plane_tile(const ConvDims &f) {
    return (long)ceil_div(f.N, Gx1x1s::NIMG) * ceil_div(f.Ci, Gx1x1s::TM * Gx1x1s::COW) <= 256;
}
// ... in workgroups of four waves that cover fewer rows, for maps whose height is not a multiple of 16 (56 = 7 x 8,
// 28 = 7 x 4: ResNet-50 at batch 64, 64 -> 64 @56x56 366 -> 321 us, 128 -> 128 @28x28 345 -> 332 us)
using GxW32H8 = Tile3x3Cfg<4, 8, 8, 1, 4, 4, 8, 1>;    // 8 rows of one image x 16 channels
using GxW32H4 = Tile3x3Cfg<4, 8, 4, 2, 4, 4, 8, 1>;    // 4 rows of two images x 16 channels
// rows per tile (16, 8 or 4) that pad a map of H rows least; the larger tile on a tie
static int rows_per_tile_w32(int H) {
    const int p16 = round_up(H, 16), p8 = round_up(H, 8), p4 = round_up(H, 4);
    return p16 <= p8 && p16 <= p4 ? 16 : (p8 <= p4 ? 8 : 4);
}
static_assert(GxW32::TM == GxW16::TM && GxW16::TM == GxW8::TM && GxS2W32::TM == GxS2W16::TM,
              "the launcher checks Ci against one TM per stride");

// gadd (nullable): a tensor shaped like gx that is added to the result (tiled 3x3 / pad 1 kernels and the tiled
// 1x1 stride-1 kernels only; ADDER_ERR_UNSUPPORTED elsewhere)
int launch_grad_x(const float *gy, const float *x, const float *w, float *gx, const ConvDims &d,
                  hipStream_t s, const float *gadd) {
    const bool k3s1p1 = d.kh == 3 && d.kw == 3 && d.stride == 1 && d.pad == 1;
    if (k3s1p1 && d.Ci >= GxW32::TM &&
        (d.W % 4 != 0 || ((reinterpret_cast<uintptr_t>(gy) | reinterpret_cast<uintptr_t>(gx) |
                           reinterpret_cast<uintptr_t>(gadd)) & 15) == 0)) {
        if (d.W > 16) switch (rows_per_tile_w32(d.H)) {
            case 16: return launch_grad_x_3x3s1<GxW32>(gy, x, w, gx, d, s, gadd);
            case 8: return launch_grad_x_3x3s1<GxW32H8>(gy, x, w, gx, d, s, gadd);
            default: return launch_grad_x_3x3s1<GxW32H4>(gy, x, w, gx, d, s, gadd);
        }
        if (d.W > 8) return launch_grad_x_3x3s1<GxW16>(gy, x, w, gx, d, s, gadd);
        return launch_grad_x_3x3s1<GxW8>(gy, x, w, gx, d, s, gadd);
    }
    if (d.kh == 3 && d.kw == 3 && d.stride == 2 && d.pad == 1 && d.W % 2 == 0 && d.Ci >= GxS2W32::TM &&
        (d.Wo % 4 != 0 || (reinterpret_cast<uintptr_t>(gy) & 15) == 0) &&
        ((reinterpret_cast<uintptr_t>(gx) | reinterpret_cast<uintptr_t>(gadd)) & 7) == 0) {
        if (d.W > 16) return launch_grad_x_3x3s2<GxS2W32>(gy, x, w, gx, d, s, gadd);
        return launch_grad_x_3x3s2<GxS2W16>(gy, x, w, gx, d, s, gadd);
    }
    // (from 48 output channels on the tiled kernel is ahead of the plain one: DenseNet's 48-channel bottlenecks)
    if (d.kh == 1 && d.kw == 1 && d.pad == 0 && d.stride == 1 && d.Ci >= 64 && d.Co >= 48) {
        ConvDims f = d;   // every (H, W) plane as one row of H*W positions
        f.H = f.Ho = 1;
        f.W = f.Wo = d.H * d.W;
        if (f.W % 4 != 0 || ((reinterpret_cast<uintptr_t>(gy) | reinterpret_cast<uintptr_t>(gx) |
                              reinterpret_cast<uintptr_t>(gadd)) & 15) == 0) {
            if (f.W > 64) return launch_grad_x_3x3s1<Gx1x1>(gy, x, w, gx, f, s, gadd);
            return small_plane_tile(f) ? launch_grad_x_3x3s1<Gx1x1t>(gy, x, w, gx, f, s, gadd)
                                       : launch_grad_x_3x3s1<Gx1x1s>(gy, x, w, gx, f, s, gadd);
        }
    }
    if (gadd) return ADDER_ERR_UNSUPPORTED;
    if (d.kh == 1 && d.kw == 1 && d.pad == 0 && d.stride > 1 && d.Ci >= 64 && d.Co >= 64) {
        ConvDims f = d;   // the sampled positions of every plane as one row; x and gx are read / written in place
        f.H = f.Ho = 1;
        f.W = f.Wo = d.Ho * d.Wo;
        f.stride = 1;
        const Subsample sub{d.stride, d.Wo, d.W, d.H * d.W};
        if (f.W % 4 != 0 || (reinterpret_cast<uintptr_t>(gy) & 15) == 0) {
            if (f.W > 64) return launch_grad_x_3x3s1<Gx1x1, true>(gy, x, w, gx, f, s, (const float *)nullptr, sub);
            return small_plane_tile(f) ? launch_grad_x_3x3s1<Gx1x1t, true>(gy, x, w, gx, f, s, (const float *)nullptr, sub)
                                       : launch_grad_x_3x3s1<Gx1x1s, true>(gy, x, w, gx, f, s, (const float *)nullptr, sub);
        }
    }
    if (conv1x1_supported(d, gy, gx))
        return launch_grad_x_1x1(gy, x, w, gx, d, s);
    constexpr int TM = 8;
    const long total = (long)d.N * d.H * d.W;
    hipLaunchKernelGGL(grad_x_generic_kernel<TM>, dim3((unsigned)ceil_div_l(total, 256), ceil_div(d.Ci, TM)),
                       dim3(256), 0, s, gy, x, w, gx, d);
    return check_launch();
}

// a 1x1 stride-1 layer seen as images of one row of H * W positions
static ConvDims one_row(const ConvDims &d) {
    ConvDims f = d;
    f.H = f.Ho = 1;
    f.W = f.Wo = d.H * d.W;
    return f;
}

// Which tiled kernel carries the BatchNorm link for this layer: 1 GxW32, 2 GxW16, 3 GxW8 (3x3 stride 1), 4 GxS2W32,
// 5 GxS2W16 (3x3 stride 2), 6 Gx1x1, 7 Gx1x1t, 8 Gx1x1s (1x1 stride 1 from 64 input / 48 output channels); 0: none
// (other kernel sizes, rows or planes that are not whole float4 groups, too few channels).
static int grad_x_bn_variant(const ConvDims &d) {
    if (d.kh == 1 && d.kw == 1 && d.pad == 0 && d.stride == 1 && d.Ci >= 64 && d.Co >= 48 && (d.H * d.W) % 4 == 0) {
        const ConvDims f = one_row(d);
        return f.W > 64 ? 6 : (small_plane_tile(f) ? 7 : 8);
    }
    if (d.kh != 3 || d.kw != 3 || d.pad != 1 || d.Ci < GxW32::TM) return 0;
    if (d.stride == 1 && d.W % 4 == 0) return d.W > 16 ? 1 : (d.W > 8 ? 2 : 3);
    if (d.stride == 2 && d.W % 4 == 0 && d.Wo % 4 == 0) return d.W > 16 ? 4 : 5;
    return 0;
}

template <class C>
static int bn_slots_of(const ConvDims &d) {
    return ceil_div(d.N, C::NIMG) * ceil_div(d.H, C::TH) * ceil_div(d.W, C::TW) * bn_slots_per_wg<C>();
}

// partial-sum slots per input channel that launch_grad_x_bn writes into bn.in_part; 0: no such kernel for the layer
int grad_x_bn_slots(const ConvDims &d) {
    switch (grad_x_bn_variant(d)) {
        case 1: switch (rows_per_tile_w32(d.H)) {
            case 16: return bn_slots_of<GxW32>(d);
            case 8: return bn_slots_of<GxW32H8>(d);
            default: return bn_slots_of<GxW32H4>(d);
        }
        case 2: return bn_slots_of<GxW16>(d);
        case 3: return bn_slots_of<GxW8>(d);
        case 4: return bn_slots_of<GxS2W32>(d);
        case 5: return bn_slots_of<GxS2W16>(d);
        case 6: return bn_slots_of<Gx1x1>(one_row(d));
        case 7: return bn_slots_of<Gx1x1t>(one_row(d));
        case 8: return bn_slots_of<Gx1x1s>(one_row(d));
        default: return 0;
    }
}

// launch_grad_x with the statistics pass of the BatchNorm in front of the layer folded in (the in_* fields of
// adder_bn_links); ADDER_ERR_UNSUPPORTED where the layer has no such kernel or a tensor is not 16-byte aligned
int launch_grad_x_bn(const float *gy, const float *x, const float *w, float *gx, const ConvDims &d, hipStream_t s,
                     const float *gadd, const adder_bn_links &bn) {
    const uintptr_t align = reinterpret_cast<uintptr_t>(gy) | reinterpret_cast<uintptr_t>(gx) |
                            reinterpret_cast<uintptr_t>(gadd) | reinterpret_cast<uintptr_t>(bn.in_x) |
                            reinterpret_cast<uintptr_t>(bn.in_part);
    if (align & 15) return ADDER_ERR_UNSUPPORTED;
    if (!bn.in_part) return launch_grad_x(gy, x, w, gx, d, s, gadd);   // nothing to leave for a BatchNorm in front
    switch (grad_x_bn_variant(d)) {
        case 1: switch (rows_per_tile_w32(d.H)) {
            case 16: return launch_grad_x_3x3s1_bn<GxW32>(gy, x, w, gx, d, s, gadd, bn);
            case 8: return launch_grad_x_3x3s1_bn<GxW32H8>(gy, x, w, gx, d, s, gadd, bn);
            default: return launch_grad_x_3x3s1_bn<GxW32H4>(gy, x, w, gx, d, s, gadd, bn);
        }
        case 2: return launch_grad_x_3x3s1_bn<GxW16>(gy, x, w, gx, d, s, gadd, bn);
        case 3: return launch_grad_x_3x3s1_bn<GxW8>(gy, x, w, gx, d, s, gadd, bn);
        case 4: return launch_grad_x_3x3s2_bn<GxS2W32>(gy, x, w, gx, d, s, gadd, bn);
        case 5: return launch_grad_x_3x3s2_bn<GxS2W16>(gy, x, w, gx, d, s, gadd, bn);
        case 6: return launch_grad_x_3x3s1_bn<Gx1x1>(gy, x, w, gx, one_row(d), s, gadd, bn);
        case 7: return launch_grad_x_3x3s1_bn<Gx1x1t>(gy, x, w, gx, one_row(d), s, gadd, bn);
        case 8: return launch_grad_x_3x3s1_bn<Gx1x1s>(gy, x, w, gx, one_row(d), s, gadd, bn);
        default: return ADDER_ERR_UNSUPPORTED;
    }
}

// bfloat16 storage: the tiled 3x3 / pad-1 kernels (stride 1 or 2), the generic kernel for everything else
int launch_grad_x_bf16(const bf16_t *gy, const bf16_t *x, const float *w, bf16_t *gx, const ConvDims &d,
                       hipStream_t s) {
    const bf16_t *none = nullptr;
    if (d.kh == 3 && d.kw == 3 && d.stride == 1 && d.pad == 1 && d.Ci >= GxW32::TM &&
        (d.W % 4 != 0 || ((reinterpret_cast<uintptr_t>(gy) | reinterpret_cast<uintptr_t>(gx)) & 7) == 0)) {
        if (d.W > 16) return launch_grad_x_3x3s1<GxW32, false, bf16_t>(gy, x, w, gx, d, s, none);
        if (d.W > 8) return launch_grad_x_3x3s1<GxW16, false, bf16_t>(gy, x, w, gx, d, s, none);
        return launch_grad_x_3x3s1<GxW8, false, bf16_t>(gy, x, w, gx, d, s, none);
    }
    if (d.kh == 3 && d.kw == 3 && d.stride == 2 && d.pad == 1 && d.W % 2 == 0 && d.Ci >= GxS2W32::TM &&
        (d.Wo % 4 != 0 || (reinterpret_cast<uintptr_t>(gy) & 7) == 0) && (reinterpret_cast<uintptr_t>(gx) & 3) == 0) {
        if (d.W > 16) return launch_grad_x_3x3s2<GxS2W32, bf16_t>(gy, x, w, gx, d, s, none);
        return launch_grad_x_3x3s2<GxS2W16, bf16_t>(gy, x, w, gx, d, s, none);
    }
    constexpr int TM = 8;
    const long total = (long)d.N * d.H * d.W;
    hipLaunchKernelGGL((grad_x_generic_kernel<TM, bf16_t>), dim3((unsigned)ceil_div_l(total, 256), ceil_div(d.Ci, TM)),
                       dim3(256), 0, s, gy, x, w, gx, d);
    return check_launch();
}

}  // namespace adder
