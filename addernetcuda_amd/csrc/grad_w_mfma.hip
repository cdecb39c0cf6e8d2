// Weight gradient of the AdderNet convolution (3x3 / pad 1, or 1x1 / stride 1) on the matrix cores, in full precision.
//
//   gw[co,k] = sum_pos xcol[k,pos] * gy[co,pos]  -  w[co,k] * sum_pos gy[co,pos]      (k = (ci, i, j))
//
// Unlike the forward and the input gradient (|a-b| and clamp are not multiply-accumulates), the
// first term of the weight gradient IS a GEMM, G (Co x P) times Xcol^T (P x K), reduced over the
// positions P = N*Ho*Wo (262 144 for the first ResNet-20 stage at batch 256).  Summing that many
// O(1) products in fp32 leaves ~1e-4 absolute error whatever the order (an fp32 torch evaluation
// of the reference formula is off by 1e-3), which is the size of the parity bar itself; AdderNet
// also singles this gradient out as the full-precision one.  So the products and sums are done in
// fp64 by v_mfma_f64_16x16x4_f64: fp64 MFMA runs at the rate of v_fma_f32, leaves the VALU free and
// does the position reduction inside the instruction (no cross-lane fold).
// Mapping: M = output channels (16 per tile), N = k columns (16 per tile), MFMA-K = 4 adjacent
// output positions of one row.
//   A fragment  lane l: gy[co0 + l%16][pos0 + l/16]           from the gy tile in LDS (fp32 -> fp64)
//   B fragment  lane l: x[ci(k), ho*S + i(k), (wo0 + l/16)*S + j(k)],  k = k0 + l%16, from the
//               haloed x tile in LDS: the im2col happens in the ds_read addresses.
//   C/D         lane l, reg r: gw[co0 + 4*r + l/16][k0 + l%16]
// A wave keeps MT x NT accumulator tiles (8 VGPRs each) in registers for the whole kernel and walks
// over its share of the positions of every staged tile; PW waves split the positions, MW x NW waves
// the (co, k) block of the workgroup; the waves are folded in fp64 through LDS at the end.
// sum_pos gy is collected on the A fragments.  Partials: one fp64 (Co, K) slab per grid.x slot.
#include "common.hpp"
#include "tile3x3.hpp"

namespace adder {

typedef double double4v __attribute__((ext_vector_type(4)));

template <int S_, int TH_, int TW_, int NIMG_, int MT_, int NT_, int MW_, int NW_, int PW_, int KS_ = 3>
struct GwMfmaCfg {
    static constexpr int S = S_, TH = TH_, TW = TW_, NIMG = NIMG_, MT = MT_, NT = NT_, MW = MW_, NW = NW_, PW = PW_;
    static constexpr int KS = KS_, KK = KS_ * KS_, PAD = KS_ / 2;   // 3x3 taps with pad 1, or a single tap
    static constexpr int COB = 16 * MT * MW;          // output channels per workgroup
    static constexpr int KB = 16 * NT * NW;           // k columns per workgroup
    static constexpr int CIB = ceil_div(KB, KK);      // input channels per workgroup (staged)
    // false: the k block ends inside an input channel -- usable only where one block holds all of K (a layer with
    // very few input channels; the columns past K read a channel that does not exist, i.e. staged zeros)
    static constexpr bool WHOLE = KB % KK == 0;
    static constexpr int NWAVES = MW * NW * PW;
    static constexpr int NTHREADS = 64 * NWAVES;
    // LPAD puts the interior columns on a 16-byte boundary (3 + one halo column, or no halo at all)
    using XP = PatchCfg<NIMG, CIB, (TH - 1) * S + KS, TW * S, PAD, (S == 1) ? PAD : 0, NTHREADS, PAD ? 3 : 0>;
    static constexpr int GPLANE = TH * TW + 4;        // +4: channel planes start 4 banks apart
    static constexpr int GBUF = NIMG * COB * GPLANE;
    static constexpr int GUNITS = NIMG * COB * TH * TW / 4;
    static constexpr int GITER = ceil_div(GUNITS, NTHREADS);
    static constexpr int BUF = XP::BUF + GBUF;        // floats per (x, gy) buffer pair
    static constexpr int STEPS = NIMG * TH * TW / 4;  // MFMA steps (4 positions each) per tile
    static constexpr int WSTEPS = STEPS / PW;         // ... per wave
    static constexpr int REGS = MT * NT * 4;          // accumulator values (fp64) per lane
    static constexpr int RED = 2 * (NWAVES / 2) * (REGS + MT) * 64;  // fp64 fold area, in floats
    static constexpr int LDS_FLOATS = (2 * BUF > RED) ? 2 * BUF : RED;
    static constexpr int LDS_BYTES = LDS_FLOATS * 4;
    static_assert(TW % 4 == 0 && STEPS % PW == 0, "positions must split evenly over the position waves");
    static_assert((PW & (PW - 1)) == 0, "the fold is a binary tree over the position waves");
    static_assert(NTHREADS <= 1024 && LDS_BYTES <= 160 * 1024, "workgroup limits");
    static_assert(XP::BUF % 4 == 0 && GPLANE % 4 == 0, "float4 alignment of the gy tile");
};

template <class G>
struct GyStageM { float4 v[G::GITER]; };

template <class G, bool VEC, class T = float>
__device__ __forceinline__ void gy_fetch_m(GyStageM<G> &st, const T *__restrict__ gy, int co0, int Co, int n0,
                                           int N, int h0, int w0, int Ho, int Wo) {
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
        if (ok) {
            const T *row = gy + (((n * Co + co) * Ho + ho) * Wo + wo);
            if constexpr (VEC) {
                val = ldf4(row);
            } else {   // rows are not whole aligned groups of four (Wo % 4 != 0)
                val.x = ldf(row);
                if (wo + 1 < Wo) val.y = ldf(row + 1);
                if (wo + 2 < Wo) val.z = ldf(row + 2);
                if (wo + 3 < Wo) val.w = ldf(row + 3);
            }
        }
        st.v[it] = val;
    }
}

template <class G>
__device__ __forceinline__ void gy_commit_m(const GyStageM<G> &st, float *buf) {
#pragma unroll
    for (int it = 0; it < G::GITER; ++it) {
        const int u = threadIdx.x + it * G::NTHREADS;
        if (G::GUNITS % G::NTHREADS == 0 || u < G::GUNITS) {
            const int q = u % (G::TW / 4);
            const int r = (u / (G::TW / 4)) % G::TH;
            const int pc = u / (G::TW / 4) / G::TH;   // = img*COB + c
            *reinterpret_cast<float4 *>(buf + pc * G::GPLANE + r * G::TW + 4 * q) = st.v[it];
        }
    }
}

// The gy tile of a layer that is followed by a BatchNorm, formed from the gradient dz of that BatchNorm's output
// (already masked by the ReLU behind it), the layer's own output y and four numbers per channel,
//   gy = k * dz + (c2 * (y - mu) - km1),      coef[channel] = {k, c2, mu, km1}
// (k = gamma * rstd, c2 = -k * rstd * mean(dz * xhat), km1 = k * mean(dz)): the second pass of the BatchNorm
// backward, done on the way into LDS.  gy_out (nullable): the same values go to this tensor, shaped like gy, for
// the input-gradient kernel that runs next.  coef: the workgroup's COB channels, in LDS.
template <class G>
__device__ __forceinline__ void gy_commit_m_bn(const GyStageM<G> &sg, const GyStageM<G> &sy, float *buf,
                                               const float4 *coef, float *__restrict__ gy_out, int co0, int Co, int n0,
                                               int N, int h0, int w0, int Ho, int Wo) {
#pragma unroll
    for (int it = 0; it < G::GITER; ++it) {
        const int u = threadIdx.x + it * G::NTHREADS;
        if (G::GUNITS % G::NTHREADS == 0 || u < G::GUNITS) {
            const int q = u % (G::TW / 4);
            const int r = (u / (G::TW / 4)) % G::TH;
            const int pc = u / (G::TW / 4) / G::TH;   // = img*COB + c
            const int c = pc % G::COB, img = pc / G::COB;
            const bool ok = n0 + img < N && co0 + c < Co && h0 + r < Ho && w0 + 4 * q < Wo;   // rows are whole groups of four
            const float4 cf = coef[c];
            const float4 g = sg.v[it], y = sy.v[it];
            float4 v;
            v.x = ok ? fmaf(cf.x, g.x, fmaf(cf.y, y.x - cf.z, -cf.w)) : 0.f;
            v.y = ok ? fmaf(cf.x, g.y, fmaf(cf.y, y.y - cf.z, -cf.w)) : 0.f;
            v.z = ok ? fmaf(cf.x, g.z, fmaf(cf.y, y.z - cf.z, -cf.w)) : 0.f;
            v.w = ok ? fmaf(cf.x, g.w, fmaf(cf.y, y.w - cf.z, -cf.w)) : 0.f;
            *reinterpret_cast<float4 *>(buf + pc * G::GPLANE + r * G::TW + 4 * q) = v;
            if (gy_out && ok)
                *reinterpret_cast<float4 *>(gy_out + ((((n0 + img) * Co + co0 + c) * Ho + h0 + r) * Wo + w0 + 4 * q)) = v;
        }
    }
}

// The four coefficients of gy_commit_m_bn for the workgroup's COB channels, from the sums the consumer's
// input-gradient kernel left (BnSums): 32 lanes add the slots of one channel, always in the same order, so every
// workgroup that needs a channel arrives at the same bits.  `write`: also store dgamma / dbeta of these channels
// (one workgroup per channel block does).  Stands in for a launch of its own between the two kernels.
template <class G>
__device__ __forceinline__ void bn_coef_from_sums(const BnSums &b, int co0, int Co, float4 *coef, bool write) {
    constexpr int GROUPS = G::NTHREADS / 32;
    constexpr int CHUNK = 16;
    const int sub = threadIdx.x & 31, grp = threadIdx.x >> 5;
    for (int cb = 0; cb < G::COB; cb += GROUPS) {
        const int c = cb + grp;
        if (G::COB % GROUPS == 0 || c < G::COB) {
            const int co = min(co0 + c, Co - 1);
            const float rs = b.rstd[co], gm = b.gamma[co], mu = b.mean[co];
            const float2 *p = reinterpret_cast<const float2 *>(b.part) + (size_t)co * b.slots;
            double s1 = 0.0, s2 = 0.0;
            for (int s0 = sub; s0 < b.slots; s0 += 32 * CHUNK) {   // CHUNK loads in flight, then added in slot order
                float2 v[CHUNK];
#pragma unroll
                for (int j = 0; j < CHUNK; ++j) v[j] = p[min(s0 + 32 * j, b.slots - 1)];   // (unconditional: no waits between them)
#pragma unroll
                for (int j = 0; j < CHUNK; ++j) {
                    const bool in = s0 + 32 * j < b.slots;
                    s1 += in ? (double)v[j].x : 0.0;
                    s2 += in ? (double)v[j].y : 0.0;
                }
            }
#pragma unroll
            for (int m = 16; m >= 1; m >>= 1) {   // (stays inside the 32-lane half)
                s1 += __shfl_xor(s1, m, 64);
                s2 += __shfl_xor(s2, m, 64);
            }
            if (sub == 0) {
                const float m1 = (float)(s1 / b.count), m2 = (float)(s2 / b.count);
                const float k = gm * rs;
                coef[c] = make_float4(k, -k * rs * m2, mu, k * m1);
                if (write && co0 + c < Co) {
                    b.dbeta[co] = (float)s1;
                    b.dgamma[co] = (float)s2;
                }
            }
        }
    }
}

// SUB (single tap only): x is a sampled tensor (see Subsample), read element by element at the sampled
// positions; gy is dense.  VEC then only says how gy is read.
// T: storage type of gy and x (float, or bf16_t for the reduced-storage mode); staged as fp32, multiplied in fp64.
// FUSE: gy holds dz and the gy tiles are formed from (dz, bn_y, bn_coef) on the way into LDS (gy_commit_m_bn), and
// written to gy_out (nullable) by the workgroups of the first k block; float storage, rows of whole float4 groups.
template <class G, bool VEC = true, bool SUB = false, class T = float, bool FUSE = false>
__global__ __launch_bounds__(G::NTHREADS) void grad_w_mfma_kernel(const T *__restrict__ gy,
                                                                  const T *__restrict__ x,
                                                                  double *__restrict__ part,
                                                                  double *__restrict__ sgpart, int N, int Ci, int H,
                                                                  int W, int Co, int Ho, int Wo, int tilesH,
                                                                  int tilesW, int ntiles, const Subsample sub,
                                                                  const float *__restrict__ bn_y,
                                                                  const float *__restrict__ bn_coef,
                                                                  float *__restrict__ gy_out, const BnSums sums) {
    static_assert(!FUSE || (VEC && !SUB && sizeof(T) == 4), "the BatchNorm link belongs to the float kernels");
    using XP = typename G::XP;
    constexpr int S = G::S, MT = G::MT, NT = G::NT;
    extern __shared__ __align__(16) float smem[];

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int pw = wave % G::PW, mw = (wave / G::PW) % G::MW, nw = wave / (G::PW * G::MW);
    const int co_blk = blockIdx.y * G::COB, k_blk = blockIdx.z * G::KB, ci_blk = blockIdx.z * G::CIB;
    const int l16 = lane & 15, lk = lane >> 4;

    // per-lane LDS offsets of the fragments at position (img 0, row 0, column group 0)
    int a_base[MT], b_base[NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) a_base[mt] = XP::BUF + ((mw * MT + mt) * 16 + l16) * G::GPLANE + lk;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int j = (nw * NT + nt) * 16 + l16;        // k column within the workgroup's block
        const int ci = j / G::KK, tap = j - ci * G::KK, ti = tap / G::KS, tj = tap - ti * G::KS;
        b_base[nt] = ci * XP::PLANE + ti * XP::PITCH + XP::ICOL0 - G::PAD + tj + lk * S;
    }

    double4v acc[MT][NT];
    double sgt[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        sgt[mt] = 0.0;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = double4v{0.0, 0.0, 0.0, 0.0};
    }

    TileStage<XP> xs;
    GyStageM<G> gs, ys;   // (ys: FUSE only)
    const float4 *coef = reinterpret_cast<const float4 *>(smem + G::LDS_FLOATS);
    float *const gy_dst = blockIdx.z == 0 ? gy_out : nullptr;   // every gy tile is staged once per k block
    int tile = blockIdx.x;
    int n0 = 0, h0 = 0, w0 = 0;
    auto decode = [&](int t) {
        const int tw = t % tilesW; t /= tilesW;
        const int th = t % tilesH; t /= tilesH;
        n0 = t * G::NIMG; h0 = th * G::TH; w0 = tw * G::TW;
    };
    if (tile < ntiles) {
        decode(tile);
        tile_fetch<XP, VEC && !SUB, SUB, T>(xs, x, ci_blk, Ci, n0, N, h0 * S - G::PAD, w0 * S, H, W, sub);
        gy_fetch_m<G, VEC, T>(gs, gy, co_blk, Co, n0, N, h0, w0, Ho, Wo);
        if constexpr (FUSE) gy_fetch_m<G, true, float>(ys, bn_y, co_blk, Co, n0, N, h0, w0, Ho, Wo);
    }
    if constexpr (FUSE) {   // the block's coefficients, while the first tile's loads are under way
        float4 *cdst = reinterpret_cast<float4 *>(smem + G::LDS_FLOATS);
        if (sums.part) {
            bn_coef_from_sums<G>(sums, co_blk, Co, cdst, blockIdx.x == 0 && blockIdx.z == 0);
        } else {
            for (int e = threadIdx.x; e < G::COB; e += G::NTHREADS)
                cdst[e] = reinterpret_cast<const float4 *>(bn_coef)[min(co_blk + e, Co - 1)];
        }
        __syncthreads();
    }
    if (tile < ntiles) {
        tile_commit<XP>(xs, smem);
        if constexpr (FUSE) gy_commit_m_bn<G>(gs, ys, smem + XP::BUF, coef, gy_dst, co_blk, Co, n0, N, h0, w0, Ho, Wo);
        else gy_commit_m<G>(gs, smem + XP::BUF);
    }
    __syncthreads();

    int cur = 0;
    for (; tile < ntiles; tile += gridDim.x) {
        const int next = tile + gridDim.x;
        if (next < ntiles) {   // next tile's global loads fly during this tile's arithmetic
            decode(next);
            tile_fetch<XP, VEC && !SUB, SUB, T>(xs, x, ci_blk, Ci, n0, N, h0 * S - G::PAD, w0 * S, H, W, sub);
            gy_fetch_m<G, VEC, T>(gs, gy, co_blk, Co, n0, N, h0, w0, Ho, Wo);
            if constexpr (FUSE) gy_fetch_m<G, true, float>(ys, bn_y, co_blk, Co, n0, N, h0, w0, Ho, Wo);
        }
        const float *base = smem + cur * G::BUF;
        auto steps = [&](const int first, const int last) {
#pragma unroll 8
            for (int ws = first; ws < last; ++ws) {
                const int st = pw + ws * G::PW;                 // wave-uniform step: (img, row, column group)
                const int c4 = st % (G::TW / 4);
                const int r = (st / (G::TW / 4)) % G::TH;
                const int img = st / (G::TW / 4) / G::TH;
                const int a_off = img * G::COB * G::GPLANE + r * G::TW + 4 * c4;
                const int b_off = img * G::CIB * XP::PLANE + r * S * XP::PITCH + 4 * c4 * S;
                double a[MT], b[NT];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) a[mt] = (double)base[a_base[mt] + a_off];
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) b[nt] = (double)base[b_base[nt] + b_off];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    sgt[mt] += a[mt];
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt)
                        acc[mt][nt] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[mt], b[nt], acc[mt][nt], 0, 0, 0);
                }
            }
        };
        // the next tile is written to the other LDS buffer half-way through, so that the ds_writes
        // issue while this tile's queued MFMAs keep the matrix pipe busy
        steps(0, G::WSTEPS / 2);
        if (next < ntiles) {
            tile_commit<XP>(xs, smem + (cur ^ 1) * G::BUF);
            if constexpr (FUSE)
                gy_commit_m_bn<G>(gs, ys, smem + (cur ^ 1) * G::BUF + XP::BUF, coef, gy_dst, co_blk, Co, n0, N, h0, w0, Ho,
                                  Wo);
            else
                gy_commit_m<G>(gs, smem + (cur ^ 1) * G::BUF + XP::BUF);
        }
        steps(G::WSTEPS / 2, G::WSTEPS);
        __syncthreads();
        cur ^= 1;
    }

    // ---- fold the PW position waves of each (mw, nw) block into its pw = 0 wave: binary tree, fp64, via LDS ----
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {           // the four position lanes that share an output channel
        sgt[mt] += __shfl_xor(sgt[mt], 16, 64);
        sgt[mt] += __shfl_xor(sgt[mt], 32, 64);
    }
    double *red = reinterpret_cast<double *>(smem);
    constexpr int SLOT = (G::REGS + MT) * 64;   // doubles per sending wave
    const int blk = nw * G::MW + mw;
    for (int half = G::PW / 2; half >= 1; half >>= 1) {
        double *mine = red + (size_t)(blk * (G::PW / 2) + (pw % half)) * SLOT;
        if (pw >= half && pw < 2 * half) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                mine[(G::REGS + mt) * 64 + lane] = sgt[mt];
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int e = 0; e < 4; ++e) mine[((mt * NT + nt) * 4 + e) * 64 + lane] = acc[mt][nt][e];
            }
        }
        __syncthreads();
        if (pw < half) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                sgt[mt] += mine[(G::REGS + mt) * 64 + lane];
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[mt][nt][e] += mine[((mt * NT + nt) * 4 + e) * 64 + lane];
            }
        }
        __syncthreads();
    }
    if (pw != 0) return;

    const int K = Ci * G::KK;
    double *dst = part + (size_t)blockIdx.x * Co * K;   // fp64 slabs: partials of opposite sign cancel across slots
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int kcol = k_blk + (nw * NT + nt) * 16 + l16;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int co = co_blk + (mw * MT + mt) * 16 + 4 * e + lk;
                if (co < Co && kcol < K) dst[(size_t)co * K + kcol] = acc[mt][nt][e];
            }
        }
    if (nw == 0 && blockIdx.z == 0 && lane < 16) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int co = co_blk + (mw * MT + mt) * 16 + lane;
            if (co < Co) sgpart[(size_t)blockIdx.x * Co + co] = sgt[mt];
        }
    }
}

// ---- host side ------------------------------------------------------------------
// One blocking for every layer: a workgroup of twelve waves owns 16 output channels x 16 input channels (nine
// 16x16 fp64 accumulator tiles: three k waves with three tiles each, times four position waves) and 256 positions
// per staged tile.  Small (co, k) blocks keep the partial slabs at Co*K values per position split whatever the layer.
// (Eight position waves with all nine tiles each were 1.5-3 us per launch slower: a three-round fold of 72
// registers per lane through LDS at the end, against two rounds of 24.)
//                            S  TH  TW NIMG MT NT MW NW PW
using GmW32   = GwMfmaCfg<1, 8, 32, 1, 1, 3, 1, 3, 4>;   // outputs 32 wide: 8 rows of one image
using GmW16   = GwMfmaCfg<1, 16, 16, 1, 1, 3, 1, 3, 4>;  // outputs 16 wide: one image
using GmW8    = GwMfmaCfg<1, 8, 8, 4, 1, 3, 1, 3, 4>;    // outputs 8 wide:  four images
using GmW16S2 = GwMfmaCfg<2, 8, 16, 1, 1, 3, 1, 3, 4>;   // stride 2, outputs 16 wide: half an image
using GmW8S2  = GwMfmaCfg<2, 8, 8, 2, 1, 3, 1, 3, 4>;    // stride 2, outputs 8 wide: two images
// At most three input channels (the 3 -> 16 stem that precedes the adder layers: K = 27): two accumulator tiles cover
// all of K, eight position waves.  Through the 144-column block above, four fifths of the matrix instructions of
// such a layer multiply staged zeros: 28 us for 0.23 GFLOP.
using GmW32K32 = GwMfmaCfg<1, 8, 32, 1, 1, 2, 1, 1, 8>;
// 1x1, stride 1: a plain (Co x positions) x (positions x Ci) product; (H, W) planes walked as one row.
// 64 output channels x 64 input channels per workgroup (two k waves with eight accumulator tiles each, times four
// position waves), 128 positions per staged tile; every wave does eight steps of 8 MFMAs on 4 + 2 LDS reads per tile.
using Gm1x1   = GwMfmaCfg<1, 1, 128, 1, 4, 2, 1, 2, 4, 1>;
using Gm1x1s  = GwMfmaCfg<1, 1, 64, 2, 4, 2, 1, 2, 4, 1>;    // planes of <= 64 positions: two images
// From 128 channels on either side: 128 x 128 channels per workgroup (2 x 2 waves of 64 x 64 and two position
// waves), 64 positions per staged tile.  The 64 x 64 blocking reads every x tile Co / 64 times and every gy tile
// Ci / 64 times, which is what bounds it on the wide layers; this one halves that (5-15 % less time).
using Gm1x1b  = GwMfmaCfg<1, 1, 64, 1, 4, 4, 2, 2, 2, 1>;
// the same block with 52 positions per tile (2 x 4 waves of 64 x 32, no position split): 14x14 and 7x7 planes
// (196 = 3 x 52 + 40 and 49 positions) fill tiles of 52 to 94 %, tiles of 64 to 77 %
using Gm1x1c  = GwMfmaCfg<1, 1, 52, 1, 4, 2, 2, 4, 1, 1>;

template <class G>
static void plan_one(const ConvDims &d, GradWMfmaPlan &p) {
    p.tilesH = ceil_div(d.Ho, G::TH);
    p.tilesW = ceil_div(d.Wo, G::TW);
    p.ntiles = ceil_div(d.N, G::NIMG) * p.tilesH * p.tilesW;
    p.gy = ceil_div(d.Co, G::COB);
    p.gz = ceil_div(d.Ci * G::KK, G::KB);
    // one workgroup per CU (a workgroup's two staged tiles fill half of a CU's LDS and more)
    int want = ceil_div(256, p.gy * p.gz);
    p.slots = want < p.ntiles ? want : p.ntiles;
    if (p.slots < 1) p.slots = 1;
}

// a 1x1 layer seen as images of one row of Ho*Wo positions (the whole plane when the stride is 1)
static ConvDims mfma_one_row(const ConvDims &d) {
    ConvDims f = d;
    f.H = f.Ho = 1;
    f.W = f.Wo = d.Ho * d.Wo;
    f.stride = 1;
    return f;
}

GradWMfmaPlan plan_grad_w_mfma(const ConvDims &d) {
    GradWMfmaPlan p{};
    if (d.kh == 1 && d.kw == 1 && d.pad == 0 && d.Ci >= 64 && d.Co >= 64) {
        const ConvDims f = mfma_one_row(d);
        if (d.Ci >= 128 && d.Co >= 128) {
            const bool narrow = ceil_div(f.W, Gm1x1c::TW) * Gm1x1c::TW < ceil_div(f.W, Gm1x1b::TW) * Gm1x1b::TW;
            p.variant = (narrow ? 12 : 10) + (d.stride > 1 ? 1 : 0);   // 11, 13: x sampled at every stride-th row and column
            if (narrow) plan_one<Gm1x1c>(f, p);
            else plan_one<Gm1x1b>(f, p);
            return p;
        }
        p.variant = (f.W > 64 ? 6 : 7) + (d.stride > 1 ? 2 : 0);   // 8, 9: x sampled likewise
        if (f.W > 64) plan_one<Gm1x1>(f, p);
        else plan_one<Gm1x1s>(f, p);
        return p;
    }
    const bool ok = d.kh == 3 && d.kw == 3 && d.pad == 1;
    if (!ok) return p;
    if (d.stride == 1) p.variant = d.Wo > 16 ? (d.Ci * 9 <= GmW32K32::KB ? 14 : 1) : (d.Wo > 8 ? 2 : 3);
    else if (d.stride == 2) p.variant = d.Wo > 8 ? 4 : 5;
    switch (p.variant) {
        case 14: plan_one<GmW32K32>(d, p); break;
        case 1: plan_one<GmW32>(d, p); break;
        case 2: plan_one<GmW16>(d, p); break;
        case 3: plan_one<GmW8>(d, p); break;
        case 4: plan_one<GmW16S2>(d, p); break;
        case 5: plan_one<GmW8S2>(d, p); break;
        default: break;
    }
    return p;
}

template <class G, bool VEC, bool SUB = false, class T = float, bool FUSE = false>
static int launch_one_v(const T *gy, const T *x, double *part, double *sgpart, const ConvDims &d,
                      const GradWMfmaPlan &p, hipStream_t s, const Subsample sub = Subsample{1, 0, 0, 0},
                      const float *bn_y = nullptr, const float *bn_coef = nullptr, float *gy_out = nullptr,
                      const BnSums &sums = kNoBnSums) {
    constexpr int LDS_BYTES = G::LDS_BYTES + (FUSE ? G::COB * 16 : 0);   // + the BatchNorm coefficients of the block
    if (int rc = allow_dynamic_lds<&grad_w_mfma_kernel<G, VEC, SUB, T, FUSE>>(LDS_BYTES)) return rc;
    hipLaunchKernelGGL((grad_w_mfma_kernel<G, VEC, SUB, T, FUSE>), dim3(p.slots, p.gy, p.gz), dim3(G::NTHREADS), LDS_BYTES, s,
                       gy, x, part, sgpart, d.N, d.Ci, d.H, d.W, d.Co, d.Ho, d.Wo, p.tilesH, p.tilesW, p.ntiles, sub, bn_y,
                       bn_coef, gy_out, sums);
    return check_launch();
}

template <class G, class T = float>
static int launch_one(const T *gy, const T *x, double *part, double *sgpart, const ConvDims &d,
                      const GradWMfmaPlan &p, hipStream_t s) {
    // element-wise tile loads unless the rows of both x and gy are whole groups of four
    if (d.W % 4 == 0 && d.Wo % 4 == 0) return launch_one_v<G, true, false, T>(gy, x, part, sgpart, d, p, s);
    return launch_one_v<G, false, false, T>(gy, x, part, sgpart, d, p, s);
}

// bfloat16 storage of gy and x: the 3x3 / pad-1 variants (1..5 of the plan)
int launch_grad_w_mfma_bf16(const bf16_t *gy, const bf16_t *x, double *part, double *sgpart, const ConvDims &d,
                            const GradWMfmaPlan &p, hipStream_t s) {
    switch (p.variant) {
        case 1: return launch_one<GmW32, bf16_t>(gy, x, part, sgpart, d, p, s);
        case 2: return launch_one<GmW16, bf16_t>(gy, x, part, sgpart, d, p, s);
        case 3: return launch_one<GmW8, bf16_t>(gy, x, part, sgpart, d, p, s);
        case 4: return launch_one<GmW16S2, bf16_t>(gy, x, part, sgpart, d, p, s);
        case 5: return launch_one<GmW8S2, bf16_t>(gy, x, part, sgpart, d, p, s);
        case 14: return launch_one<GmW32K32, bf16_t>(gy, x, part, sgpart, d, p, s);
        default: return ADDER_ERR_UNSUPPORTED;
    }
}

// The 3x3 / pad-1 and the stride-1 1x1 variants with gy formed from (dz = gy, bn_y, bn_coef) while it is staged and
// left in gy_out (nullable) on the way (see gy_commit_m_bn); ADDER_ERR_UNSUPPORTED for other variants and for rows
// (planes, for 1x1 layers) that are not whole float4 groups.
int launch_grad_w_mfma_bn(const float *gy, const float *x, double *part, double *sgpart, const ConvDims &d,
                          const GradWMfmaPlan &p, const float *bn_y, const float *bn_coef, float *gy_out, hipStream_t s,
                          const BnSums &sums) {
    const Subsample none{1, 0, 0, 0};
    if (((p.variant >= 1 && p.variant <= 5) || p.variant == 14) && (d.W % 4 != 0 || d.Wo % 4 != 0))
        return ADDER_ERR_UNSUPPORTED;
    switch (p.variant) {
        case 14: return launch_one_v<GmW32K32, true, false, float, true>(gy, x, part, sgpart, d, p, s, none, bn_y, bn_coef,
                                                                            gy_out, sums);
        case 1: return launch_one_v<GmW32, true, false, float, true>(gy, x, part, sgpart, d, p, s, none, bn_y, bn_coef, gy_out, sums);
        case 2: return launch_one_v<GmW16, true, false, float, true>(gy, x, part, sgpart, d, p, s, none, bn_y, bn_coef, gy_out, sums);
        case 3: return launch_one_v<GmW8, true, false, float, true>(gy, x, part, sgpart, d, p, s, none, bn_y, bn_coef, gy_out, sums);
        case 4: return launch_one_v<GmW16S2, true, false, float, true>(gy, x, part, sgpart, d, p, s, none, bn_y, bn_coef, gy_out, sums);
        case 5: return launch_one_v<GmW8S2, true, false, float, true>(gy, x, part, sgpart, d, p, s, none, bn_y, bn_coef, gy_out, sums);
        default: break;
    }
    // 1x1 stride-1 layers: whole planes as rows
    const ConvDims f = mfma_one_row(d);
    if (d.stride != 1 || f.W % 4 != 0) return ADDER_ERR_UNSUPPORTED;
    switch (p.variant) {
        case 6: return launch_one_v<Gm1x1, true, false, float, true>(gy, x, part, sgpart, f, p, s, none, bn_y, bn_coef, gy_out, sums);
        case 7: return launch_one_v<Gm1x1s, true, false, float, true>(gy, x, part, sgpart, f, p, s, none, bn_y, bn_coef, gy_out, sums);
        case 10: return launch_one_v<Gm1x1b, true, false, float, true>(gy, x, part, sgpart, f, p, s, none, bn_y, bn_coef, gy_out, sums);
        case 12: return launch_one_v<Gm1x1c, true, false, float, true>(gy, x, part, sgpart, f, p, s, none, bn_y, bn_coef, gy_out, sums);
        default: return ADDER_ERR_UNSUPPORTED;
    }
}

int launch_grad_w_mfma(const float *gy, const float *x, double *part, double *sgpart, const ConvDims &d,
                       const GradWMfmaPlan &p, hipStream_t s) {
    switch (p.variant) {
        case 1: return launch_one<GmW32>(gy, x, part, sgpart, d, p, s);
        case 2: return launch_one<GmW16>(gy, x, part, sgpart, d, p, s);
        case 3: return launch_one<GmW8>(gy, x, part, sgpart, d, p, s);
        case 4: return launch_one<GmW16S2>(gy, x, part, sgpart, d, p, s);
        case 5: return launch_one<GmW8S2>(gy, x, part, sgpart, d, p, s);
        case 14: return launch_one<GmW32K32>(gy, x, part, sgpart, d, p, s);
        case 6: return launch_one<Gm1x1>(gy, x, part, sgpart, mfma_one_row(d), p, s);
        case 7: return launch_one<Gm1x1s>(gy, x, part, sgpart, mfma_one_row(d), p, s);
        case 10: return launch_one<Gm1x1b>(gy, x, part, sgpart, mfma_one_row(d), p, s);
        case 11: {
            const ConvDims f = mfma_one_row(d);
            const Subsample sub{d.stride, d.Wo, d.W, d.H * d.W};
            return f.Wo % 4 == 0 ? launch_one_v<Gm1x1b, true, true>(gy, x, part, sgpart, f, p, s, sub)
                                 : launch_one_v<Gm1x1b, false, true>(gy, x, part, sgpart, f, p, s, sub);
        }
        case 12: return launch_one<Gm1x1c>(gy, x, part, sgpart, mfma_one_row(d), p, s);
        case 13: {
            const ConvDims f = mfma_one_row(d);
            const Subsample sub{d.stride, d.Wo, d.W, d.H * d.W};
            return f.Wo % 4 == 0 ? launch_one_v<Gm1x1c, true, true>(gy, x, part, sgpart, f, p, s, sub)
                                 : launch_one_v<Gm1x1c, false, true>(gy, x, part, sgpart, f, p, s, sub);
        }
        case 8:
        case 9: {
            const ConvDims f = mfma_one_row(d);
            const Subsample sub{d.stride, d.Wo, d.W, d.H * d.W};
            const bool vec = f.Wo % 4 == 0;
            if (p.variant == 8)
                return vec ? launch_one_v<Gm1x1, true, true>(gy, x, part, sgpart, f, p, s, sub)
                           : launch_one_v<Gm1x1, false, true>(gy, x, part, sgpart, f, p, s, sub);
            return vec ? launch_one_v<Gm1x1s, true, true>(gy, x, part, sgpart, f, p, s, sub)
                       : launch_one_v<Gm1x1s, false, true>(gy, x, part, sgpart, f, p, s, sub);
        }
        default: return ADDER_ERR_BAD_SHAPE;
    }
}

}  // namespace adder
