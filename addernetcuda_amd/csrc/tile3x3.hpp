// Tile geometry and global->LDS staging shared by the 3x3 / stride-1 / pad-1
// forward and input-gradient kernels.  Both stage a haloed (TH+2) x (TW+2)
// patch of some NCHW tensor per channel, zero-filled outside the image (the
// forward's padding taps are x = 0; the input gradient's out-of-range output
// positions contribute nothing).
#pragma once
#include "common.hpp"

namespace adder {

template <int TN_, int SPR_, int TH_, int NIMG_, int TM_, int COW_, int CC_, int CQ_>
struct Tile3x3Cfg {
    static constexpr int TN = TN_, SPR = SPR_, TH = TH_, NIMG = NIMG_, TM = TM_, COW = COW_,
                         CC = CC_, CQ = CQ_;
    static constexpr int TW = TN * SPR;
    static constexpr int LANES = NIMG * TH * SPR;
    static constexpr int POSW = ceil_div(LANES, 64);
    static constexpr int NTHREADS = 64 * POSW * COW;
    static constexpr int PITCH = round_up(TW + 2, 4);
    static constexpr int ROWS = TH + 2;
    static constexpr int PLANE = ROWS * PITCH;
    static constexpr int BUF = NIMG * CC * PLANE;  // floats per buffer
    static constexpr int LDS_BYTES = 2 * BUF * 4;
    static constexpr int STRIP_ALIGN = (TN % 4 == 0) ? 4 : (TN % 2 == 0 ? 2 : 1);
    // global -> LDS staging: interior as float4 units, halo columns as scalars
    static constexpr int NUV = NIMG * CC * ROWS * (TW / 4);
    static constexpr int VITER = ceil_div(NUV, NTHREADS);
    static constexpr int NUH = NIMG * CC * ROWS * 2;
    static constexpr int HITER = ceil_div(NUH, NTHREADS);
    static_assert(TW % 4 == 0, "tile width must be a multiple of 4");
    static_assert(CC % CQ == 0, "CC must be a multiple of CQ");
};

template <class C>
struct TileStage {
    float4 v[C::VITER];
    float h[C::HITER];
};

// Issue the global loads of one channel chunk into registers.
template <class C>
__device__ __forceinline__ void tile_fetch(TileStage<C> &st, const float *__restrict__ src,
                                           int chan0, int nchan, int n0, int nimg_total, int h0,
                                           int w0, int H, int W) {
    // src is (nimg_total, nchan, H, W); the tile covers rows h0-1.., cols w0-1..
    const int tid = threadIdx.x;
#pragma unroll
    for (int it = 0; it < C::VITER; ++it) {
        const int u = tid + it * C::NTHREADS;
        const int q = u % (C::TW / 4);
        const int r = (u / (C::TW / 4)) % C::ROWS;
        const int cc = (u / (C::TW / 4) / C::ROWS) % C::CC;
        const int img = u / (C::TW / 4) / C::ROWS / C::CC;
        const int n = n0 + img, ch = chan0 + cc, hi = h0 - 1 + r, wi = w0 + 4 * q;
        const bool ok = (C::NUV % C::NTHREADS == 0 || u < C::NUV) && n < nimg_total && ch < nchan &&
                        hi >= 0 && hi < H && wi < W;
        float4 val = make_float4(0.f, 0.f, 0.f, 0.f);
        if (ok) val = *reinterpret_cast<const float4 *>(src + (((size_t)n * nchan + ch) * H + hi) * W + wi);
        st.v[it] = val;
    }
#pragma unroll
    for (int it = 0; it < C::HITER; ++it) {
        const int u = tid + it * C::NTHREADS;
        const int side = u & 1;
        const int r = (u >> 1) % C::ROWS;
        const int cc = (u >> 1) / C::ROWS % C::CC;
        const int img = (u >> 1) / C::ROWS / C::CC;
        const int n = n0 + img, ch = chan0 + cc, hi = h0 - 1 + r, wi = side ? w0 + C::TW : w0 - 1;
        const bool ok = (C::NUH % C::NTHREADS == 0 || u < C::NUH) && n < nimg_total && ch < nchan &&
                        hi >= 0 && hi < H && wi >= 0 && wi < W;
        st.h[it] = ok ? src[(((size_t)n * nchan + ch) * H + hi) * W + wi] : 0.f;
    }
}

// Write the staged chunk into one LDS buffer.
template <class C>
__device__ __forceinline__ void tile_commit(const TileStage<C> &st, float *buf) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int it = 0; it < C::VITER; ++it) {
        const int u = tid + it * C::NTHREADS;
        if (C::NUV % C::NTHREADS == 0 || u < C::NUV) {
            const int q = u % (C::TW / 4);
            const int rest = u / (C::TW / 4);  // = (img*CC + cc)*ROWS + r
            float *dst = buf + rest * C::PITCH + 1 + 4 * q;
            dst[0] = st.v[it].x; dst[1] = st.v[it].y; dst[2] = st.v[it].z; dst[3] = st.v[it].w;
        }
    }
#pragma unroll
    for (int it = 0; it < C::HITER; ++it) {
        const int u = tid + it * C::NTHREADS;
        if (C::NUH % C::NTHREADS == 0 || u < C::NUH) {
            const int side = u & 1;
            const int rest = u >> 1;
            buf[rest * C::PITCH + (side ? C::TW + 1 : 0)] = st.h[it];
        }
    }
}

}  // namespace adder
