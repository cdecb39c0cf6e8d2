// Tile geometry and global->LDS staging shared by the tiled 3x3 / pad-1 kernels
// (stride 1 or 2).  A workgroup covers NIMG images x TH x TW positions of the
// "lane space" (output positions for the forward and weight-gradient kernels,
// input positions for the stride-1 input gradient) and stages, per channel, the
// haloed patch of the source tensor those positions touch:
//   rows  h0*S-1 .. h0*S-1 + (TH-1)*S+2,   columns  w0*S-1 .. w0*S-1 + (TW-1)*S+2,
// zero-filled outside the tensor.  (For the forward the zeros are the padding
// taps, x = 0; for the input gradient they are output positions that do not
// exist and must contribute nothing.)
#pragma once
#include "common.hpp"

namespace adder {

// A rectangular patch of an NCHW tensor staged per channel into LDS as
// [img][cc][ROWS][PITCH]: ICOLS float4-aligned interior columns starting at LDS
// column LPAD + LHALO, plus an optional single halo column on either side.  LPAD = 3 puts the
// interior on a 16-byte boundary (one ds_write_b128 per staged float4) for kernels whose reads
// do not care about alignment; LPAD = 0 keeps a lane's strips aligned instead.
template <int NIMG_, int CC_, int ROWS_, int ICOLS_, int LHALO_, int RHALO_, int NTHREADS_, int LPAD_ = 0>
struct PatchCfg {
    static constexpr int NIMG = NIMG_, CC = CC_, ROWS = ROWS_, ICOLS = ICOLS_, LHALO = LHALO_, RHALO = RHALO_,
                         NTHREADS = NTHREADS_, LPAD = LPAD_;
    static constexpr int ICOL0 = LPAD + LHALO;          // LDS column of the first interior element
    static constexpr int PITCH = round_up(ICOL0 + ICOLS + RHALO, 4);
    static constexpr int PLANE = ROWS * PITCH;
    static constexpr int BUF = NIMG * CC * PLANE;  // floats per buffer
    static constexpr int NUV = NIMG * CC * ROWS * (ICOLS / 4);
    static constexpr int VITER = ceil_div(NUV, NTHREADS);
    static constexpr int NSIDES = LHALO + RHALO;
    static constexpr int SIDE_DIV = NSIDES ? NSIDES : 1;   // divisor of the halo loops (which are empty without a halo)
    static constexpr int NUH = NIMG * CC * ROWS * NSIDES;
    static constexpr int HITER = NSIDES ? ceil_div(NUH, NTHREADS) : 0;
    static_assert(ICOLS % 4 == 0, "interior must cover whole float4 groups of the source");
    static_assert(LHALO == 0 || LHALO == 1, "at most one halo column per side");
    static_assert(RHALO == 0 || RHALO == 1, "at most one halo column per side");
};

// A tensor that is read at every s-th row and column only (a strided single-tap layer): the kernels walk
// the sampled positions of a plane, `wv` per row, as one long row; `pitch` and `plane` are the row length
// and the plane size of the tensor as it lies in memory.
struct Subsample {
    int s, wv, pitch, plane;
};

template <class P>
struct TileStage {
    float4 v[P::VITER];
    float h[P::HITER > 0 ? P::HITER : 1];
};

// Issue the global loads of one channel chunk into registers.  src is
// (nimg_total, nchan, H, W); (hb, wb) is the source position of the first
// interior element of the patch.  Everything outside the tensor reads as zero.  VEC = false is for
// tensors whose rows are not float4-aligned (W % 4 != 0): element-wise loads.  Index arithmetic is
// 32-bit: the C ABI refuses tensors of 2^31 elements or more.
// SUB: src is sampled as described by `sub`; (H, W) = (1, sampled positions per plane).
// T: the storage type of src (float or bf16_t); the staged values are floats either way.
template <class P, bool VEC = true, bool SUB = false, class T = float>
__device__ __forceinline__ void tile_fetch(TileStage<P> &st, const T *__restrict__ src,
                                           int chan0, int nchan, int n0, int nimg_total, int hb,
                                           int wb, int H, int W, const Subsample sub = Subsample{1, 0, 0, 0}) {
    static_assert(!(SUB && VEC), "sampled tensors are read element by element");
    static_assert(!SUB || (P::ROWS == 1 && P::NSIDES == 0), "sampling is for single-tap tiles walked as one row");
    const int tid = threadIdx.x;
#pragma unroll
    for (int it = 0; it < P::VITER; ++it) {
        const int u = tid + it * P::NTHREADS;
        const int q = u % (P::ICOLS / 4);
        const int r = (u / (P::ICOLS / 4)) % P::ROWS;
        const int cc = (u / (P::ICOLS / 4) / P::ROWS) % P::CC;
        const int img = u / (P::ICOLS / 4) / P::ROWS / P::CC;
        const int n = n0 + img, ch = chan0 + cc, hi = hb + r, wi = wb + 4 * q;
        const bool ok = (P::NUV % P::NTHREADS == 0 || u < P::NUV) && n < nimg_total && ch < nchan &&
                        hi >= 0 && hi < H && wi < W;
        float4 val = make_float4(0.f, 0.f, 0.f, 0.f);
        if (ok) {
            if constexpr (SUB) {
                const T *base = src + (size_t)(n * nchan + ch) * sub.plane;
                int ho = wi / sub.wv, wo = wi - ho * sub.wv;
                float e[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    e[k] = wi + k < W ? ldf(base + ho * sub.s * sub.pitch + wo * sub.s) : 0.f;
                    if (++wo == sub.wv) { wo = 0; ++ho; }
                }
                st.v[it] = make_float4(e[0], e[1], e[2], e[3]);
                continue;
            }
            const T *row = src + (((n * nchan + ch) * H + hi) * W + wi);
            if constexpr (VEC) {
                val = ldf4(row);
            } else {   // rows are not whole aligned groups of four (W % 4 != 0): four guarded element loads
                val.x = ldf(row);
                if (wi + 1 < W) val.y = ldf(row + 1);
                if (wi + 2 < W) val.z = ldf(row + 2);
                if (wi + 3 < W) val.w = ldf(row + 3);
            }
        }
        st.v[it] = val;
    }
#pragma unroll
    for (int it = 0; it < P::HITER; ++it) {
        const int u = tid + it * P::NTHREADS;
        const int side = P::LHALO ? u % P::SIDE_DIV : 1;  // 0 = left, 1 = right
        const int rest = u / P::SIDE_DIV;
        const int r = rest % P::ROWS;
        const int cc = rest / P::ROWS % P::CC;
        const int img = rest / P::ROWS / P::CC;
        const int n = n0 + img, ch = chan0 + cc, hi = hb + r, wi = side ? wb + P::ICOLS : wb - 1;
        const bool ok = (P::NUH % P::NTHREADS == 0 || u < P::NUH) && n < nimg_total && ch < nchan &&
                        hi >= 0 && hi < H && wi >= 0 && wi < W;
        st.h[it] = ok ? ldf(src + (((n * nchan + ch) * H + hi) * W + wi)) : 0.f;
    }
}

// Write the staged chunk into one LDS buffer.
template <class P>
__device__ __forceinline__ void tile_commit(const TileStage<P> &st, float *buf) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int it = 0; it < P::VITER; ++it) {
        const int u = tid + it * P::NTHREADS;
        if (P::NUV % P::NTHREADS == 0 || u < P::NUV) {
            const int q = u % (P::ICOLS / 4);
            const int rest = u / (P::ICOLS / 4);  // = (img*CC + cc)*ROWS + r
            float *dst = buf + rest * P::PITCH + P::ICOL0 + 4 * q;
            if (P::ICOL0 % 4 == 0) {
                *reinterpret_cast<float4 *>(dst) = st.v[it];
            } else {
                dst[0] = st.v[it].x; dst[1] = st.v[it].y; dst[2] = st.v[it].z; dst[3] = st.v[it].w;
            }
        }
    }
#pragma unroll
    for (int it = 0; it < P::HITER; ++it) {
        const int u = tid + it * P::NTHREADS;
        if (P::NUH % P::NTHREADS == 0 || u < P::NUH) {
            const int side = P::LHALO ? u % P::SIDE_DIV : 1;
            const int rest = u / P::SIDE_DIV;
            buf[rest * P::PITCH + (side ? P::ICOL0 + P::ICOLS : P::LPAD)] = st.h[it];
        }
    }
}

// Geometry of the tiled kernels (see the header comment).  KS = 3: 3x3 taps, pad 1.  KS = 1: a single tap,
// pad 0 -- no halo; the forward uses it for 1x1 layers, whose (H, W) planes it walks as one long row.
template <int TN_, int SPR_, int TH_, int NIMG_, int TM_, int COW_, int CC_, int CQ_, int S_ = 1, int KS_ = 3>
struct Tile3x3Cfg {
    static constexpr int TN = TN_, SPR = SPR_, TH = TH_, NIMG = NIMG_, TM = TM_, COW = COW_,
                         CC = CC_, CQ = CQ_, S = S_, KS = KS_, KK = KS_ * KS_, PAD = KS_ / 2;
    static constexpr int TW = TN * SPR;
    static constexpr int LANES = NIMG * TH * SPR;
    static constexpr int POSW = ceil_div(LANES, 64);
    static constexpr int NTHREADS = 64 * POSW * COW;
    // stride 2 never reads past the interior on the right; a single tap has no halo at all
    using Patch = PatchCfg<NIMG, CC, (TH - 1) * S + KS, TW * S, PAD, (S == 1) ? PAD : 0, NTHREADS>;
    static constexpr int PITCH = Patch::PITCH, PLANE = Patch::PLANE, BUF = Patch::BUF;
    static constexpr int LDS_BYTES = 2 * BUF * 4;
    static constexpr int STRIP = (TN - 1) * S + KS;  // floats a lane reads per tile row
    static constexpr int STRIP_ALIGN = ((TN * S) % 4 == 0) ? 4 : ((TN * S) % 2 == 0 ? 2 : 1);
    static_assert(S == 1 || S == 2, "stride 1 or 2");
    static_assert(KS == 1 || KS == 3, "one tap or 3x3 taps");
    static_assert(CC % CQ == 0, "CC must be a multiple of CQ");
};

}  // namespace adder
