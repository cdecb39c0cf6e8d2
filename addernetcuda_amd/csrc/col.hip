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

typedef double double4v __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------------------
// out[co, nl] = -sum_k |W[co,k] - X[k,nl]|
// A lane owns COLS adjacent columns and TM rows of W; the rows of X are streamed PF at a time, the next batch
// in flight while the current one is in the arithmetic, so that a wave always has PF row loads outstanding.
// X is read once per block of TM output channels.
// VEC: columns are moved COLS at a time (NL % COLS == 0 and aligned bases), else element by element.
// ---------------------------------------------------------------------------
template <int COLS>
struct ColVec { float v[COLS]; };

template <int COLS, bool VEC>
__device__ __forceinline__ ColVec<COLS> col_load(const float *__restrict__ row, long c0, long NL) {
    ColVec<COLS> r;
    if constexpr (VEC && COLS == 2) {
        const float2 t = *reinterpret_cast<const float2 *>(row + c0);
        r.v[0] = t.x; r.v[1] = t.y;
    } else if constexpr (VEC && COLS == 4) {
        const float4 t = *reinterpret_cast<const float4 *>(row + c0);
        r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w;
    } else {
#pragma unroll
        for (int e = 0; e < COLS; ++e) r.v[e] = row[c0 + e < NL ? c0 + e : NL - 1];
    }
    return r;
}

// The weights live in LDS, not in scalar registers: the block's TM rows of W sit transposed ([k][TM], blocks of
// KB rows of X at a time) and every lane reads the same four at a time (broadcast ds_read_b128).  LDS reads return
// in order, so the waits for them are counted ones and several rows' weights stay in flight; scalar loads return
// out of order and every wait for them is a wait for all of them (measured on K = 144, NL = 262 144, 16 rows of W:
// 50 us with scalar weights in any blocking, 39 us like this).
// KW = 4 (matrices with few columns): the four waves of a workgroup share their 64 * COLS columns and split the
// rows of every block of X between them, so that the chain of dependent row batches is a quarter as long; their
// partial sums are added through LDS at the end.
template <int TM, int COLS, bool VEC, int PF, int KW>
__global__ __launch_bounds__(256) void col_fwd_lds_kernel(const float *__restrict__ X,
                                                          const float *__restrict__ Wm,
                                                          float *__restrict__ out, int K, long NL, int Co, int KB) {
    static_assert(KW == 1 || KW == 4, "all waves on their own columns, or all four on the same");
    extern __shared__ __align__(16) float wt[];   // [KB][TM]
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    long c0 = (KW == 1 ? (long)blockIdx.x * 256 + threadIdx.x : (long)blockIdx.x * 64 + lane) * COLS;
    const bool active = c0 < NL;
    if (!active) c0 = VEC ? NL - COLS : NL - 1;
    const int co0 = blockIdx.y * TM;
    float acc[TM][COLS], tot[TM][COLS];
#pragma unroll
    for (int m = 0; m < TM; ++m)
#pragma unroll
        for (int e = 0; e < COLS; ++e) acc[m][e] = tot[m][e] = 0.f;

    auto one_row = [&](const int kk, const ColVec<COLS> xv) {
#pragma unroll
        for (int q = 0; q < TM / 4; ++q) {
            const float4 w4 = *reinterpret_cast<const float4 *>(wt + kk * TM + 4 * q);
            const float wv[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int e = 0; e < COLS; ++e) acc[4 * q + j][e] -= fabsf(wv[j] - xv.v[e]);
        }
    };

    for (int k0 = 0; k0 < K; k0 += KB) {
        const int kcnt = min(KB, K - k0);
        if (k0) __syncthreads();
        for (int i = threadIdx.x; i < kcnt * TM; i += 256) {
            const int m = i / kcnt, kk = i - m * kcnt;   // consecutive threads read consecutive k of one row of W
            wt[kk * TM + m] = Wm[(size_t)min(co0 + m, Co - 1) * K + k0 + kk];
        }
        // this wave's rows of the block
        const int share = KW == 1 ? kcnt : ceil_div(kcnt, KW);
        const int kb = KW == 1 ? 0 : min(wave * share, kcnt), ke = KW == 1 ? kcnt : min(kb + share, kcnt);
        ColVec<COLS> nxt[PF];
        const int kfull = kb + (ke - kb) / PF * PF;
        if (kfull > kb) {
#pragma unroll
            for (int r = 0; r < PF; ++r) nxt[r] = col_load<COLS, VEC>(X + (size_t)(k0 + kb + r) * NL, c0, NL);
        }
        __syncthreads();
        for (int kk = kb; kk < kfull; kk += PF) {
            ColVec<COLS> cur[PF];
#pragma unroll
            for (int r = 0; r < PF; ++r) cur[r] = nxt[r];
            if (kk + PF < kfull) {
#pragma unroll
                for (int r = 0; r < PF; ++r) nxt[r] = col_load<COLS, VEC>(X + (size_t)(k0 + kk + PF + r) * NL, c0, NL);
            }
#pragma unroll
            for (int r = 0; r < PF; ++r) one_row(kk + r, cur[r]);
            if ((((kk - kb) / PF) & (64 / PF - 1)) == 64 / PF - 1) {   // two-level sum: acc holds at most 64 rows of X
#pragma unroll
                for (int m = 0; m < TM; ++m)
#pragma unroll
                    for (int e = 0; e < COLS; ++e) { tot[m][e] += acc[m][e]; acc[m][e] = 0.f; }
            }
        }
        for (int kk = kfull; kk < ke; ++kk) one_row(kk, col_load<COLS, VEC>(X + (size_t)(k0 + kk) * NL, c0, NL));
    }
#pragma unroll
    for (int m = 0; m < TM; ++m)
#pragma unroll
        for (int e = 0; e < COLS; ++e) tot[m][e] += acc[m][e];
    if constexpr (KW > 1) {
        __shared__ float red[(KW - 1) * TM * COLS * 64];
        if (wave > 0) {
#pragma unroll
            for (int m = 0; m < TM; ++m)
#pragma unroll
                for (int e = 0; e < COLS; ++e) red[(((wave - 1) * TM + m) * COLS + e) * 64 + lane] = tot[m][e];
        }
        __syncthreads();
        if (wave > 0) return;
        for (int wv = 0; wv < KW - 1; ++wv)
#pragma unroll
            for (int m = 0; m < TM; ++m)
#pragma unroll
                for (int e = 0; e < COLS; ++e) tot[m][e] += red[((wv * TM + m) * COLS + e) * 64 + lane];
    }
    if (active) {
#pragma unroll
        for (int m = 0; m < TM; ++m)
            if (co0 + m < Co) {
                float *dst = out + (size_t)(co0 + m) * NL + c0;
                if constexpr (VEC && COLS == 2) {
                    *reinterpret_cast<float2 *>(dst) = make_float2(tot[m][0], tot[m][1]);
                } else {
#pragma unroll
                    for (int e = 0; e < COLS; ++e)
                        if (c0 + e < NL) dst[e] = tot[m][e];
                }
            }
    }
}

// ---------------------------------------------------------------------------
// gX[k, nl] += sum_co hardtanh(W[co,k] - X[k,nl]) * gy[co,nl], layers with at most COB output channels:
// a lane owns COLS adjacent columns and keeps their gy values (COB x COLS) in registers for the whole
// kernel, the rows of X stream past once (PF rows in flight) and every row's result is finished on the
// spot, so X, gy and gX cross HBM once each.  The weights of the block's rows sit transposed in LDS
// ([k][co]); every lane reads the same four at a time (a broadcast ds_read_b128).
// Two vector instructions per term, as in the fused NCHW kernels:
//   hardtanh(w - x) = 2 * sat(0.5 * w + (0.5 - 0.5 * x)) - 1   ->   gX = 2 * sum_co sat(..) * g - sum_co g.
// blockIdx.y selects a block of KB rows.
// ---------------------------------------------------------------------------
template <int COB, int COLS, bool VEC>
__global__ __launch_bounds__(256) void col_grad_x_reg_kernel(const float *__restrict__ gy,
                                                             const float *__restrict__ X,
                                                             const float *__restrict__ Wm,
                                                             float *__restrict__ gX, int K, long NL, int Co,
                                                             int KB) {
    constexpr int PF = 4;
    extern __shared__ __align__(16) float wt[];   // [KB][COB]
    const int k0 = blockIdx.y * KB, kcnt = min(KB, K - k0);
    for (int i = threadIdx.x; i < kcnt * COB; i += 256) {
        const int co = i / kcnt, kk = i - co * kcnt;       // consecutive threads read consecutive k of one row of W
        wt[kk * COB + co] = co < Co ? Wm[(size_t)co * K + k0 + kk] : 0.f;
    }
    long c0 = ((long)blockIdx.x * 256 + threadIdx.x) * COLS;
    const bool active = c0 < NL;
    if (!active) c0 = VEC ? NL - COLS : NL - 1;
    float g[COB][COLS], s2[COLS];
#pragma unroll
    for (int e = 0; e < COLS; ++e) s2[e] = 0.f;
#pragma unroll
    for (int co = 0; co < COB; ++co) {
        if (co < Co) {
            const ColVec<COLS> t = col_load<COLS, VEC>(gy + (size_t)co * NL, c0, NL);
#pragma unroll
            for (int e = 0; e < COLS; ++e) { g[co][e] = t.v[e]; s2[e] += t.v[e]; }
        } else {
#pragma unroll
            for (int e = 0; e < COLS; ++e) g[co][e] = 0.f;   // with w = 0 in LDS: sat(..) * 0
        }
    }
    __syncthreads();

    auto one_row = [&](const int kk, const ColVec<COLS> xv, const ColVec<COLS> old) {
        float c[COLS], acc[COLS];
#pragma unroll
        for (int e = 0; e < COLS; ++e) { c[e] = fmaf(-0.5f, xv.v[e], 0.5f); acc[e] = 0.f; }
#pragma unroll
        for (int q = 0; q < COB / 4; ++q) {
            const float4 w4 = *reinterpret_cast<const float4 *>(wt + kk * COB + 4 * q);
            const float wv[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int e = 0; e < COLS; ++e)
                    acc[e] = fmaf(sat01(fmaf(wv[j], 0.5f, c[e])), g[4 * q + j][e], acc[e]);
        }
        if (active) {
            float *dst = gX + (size_t)(k0 + kk) * NL + c0;
            if constexpr (VEC && COLS == 2) {
                *reinterpret_cast<float2 *>(dst) =
                    make_float2(old.v[0] + fmaf(2.f, acc[0], -s2[0]), old.v[1] + fmaf(2.f, acc[1], -s2[1]));
            } else {
#pragma unroll
                for (int e = 0; e < COLS; ++e)
                    if (c0 + e < NL) dst[e] = old.v[e] + fmaf(2.f, acc[e], -s2[e]);
            }
        }
    };

    ColVec<COLS> nx[PF], no[PF];
    const int kfull = kcnt / PF * PF;
    if (kfull > 0) {
#pragma unroll
        for (int r = 0; r < PF; ++r) {
            nx[r] = col_load<COLS, VEC>(X + (size_t)(k0 + r) * NL, c0, NL);
            no[r] = col_load<COLS, VEC>(gX + (size_t)(k0 + r) * NL, c0, NL);
        }
    }
    for (int kk = 0; kk < kfull; kk += PF) {
        ColVec<COLS> cx[PF], co_[PF];
#pragma unroll
        for (int r = 0; r < PF; ++r) { cx[r] = nx[r]; co_[r] = no[r]; }
        if (kk + PF < kfull) {
#pragma unroll
            for (int r = 0; r < PF; ++r) {
                nx[r] = col_load<COLS, VEC>(X + (size_t)(k0 + kk + PF + r) * NL, c0, NL);
                no[r] = col_load<COLS, VEC>(gX + (size_t)(k0 + kk + PF + r) * NL, c0, NL);
            }
        }
#pragma unroll
        for (int r = 0; r < PF; ++r) one_row(kk + r, cx[r], co_[r]);
    }
    for (int kk = kfull; kk < kcnt; ++kk)
        one_row(kk, col_load<COLS, VEC>(X + (size_t)(k0 + kk) * NL, c0, NL),
                col_load<COLS, VEC>(gX + (size_t)(k0 + kk) * NL, c0, NL));
}

// ---------------------------------------------------------------------------
// ADDER_BACKWARD in one pass over X for layers with at most 16 output channels: the kernel above with the
// weight gradient folded in, so that X (the largest tensor by far: K rows against the Co rows of gy) crosses
// HBM once for both gradients.
//   gX: as above, lane = 2 adjacent columns, gy of those columns in registers, two instructions per term.
//   gW: per wave and batch of 16 rows of X, the 16 x 16 block  sum_cols gy[co, col] * X[k, col]  over the wave's
//       128 columns on v_mfma_f64_16x16x4_f64 (32 steps of 4 columns).  The MFMA wants lane l to hold row l % 16
//       at column 4 * step + l / 16, the streaming layout has lane l hold all rows at columns 2l, 2l + 1: gy is
//       transposed through LDS once per kernel (its fragments then stay in registers as doubles), every batch of
//       X once per batch.  The four waves' blocks are added through LDS and go to this workgroup's fp64 slab
//       (one slab per 512 columns); grad_w.hip's slab finalize adds the slabs and applies - W * sum gy.
// blockIdx.y selects a block of KB rows (KB a multiple of 16).
// ---------------------------------------------------------------------------
static constexpr int kFusedPitch = 132;   // floats per staged row of 128 columns (+4: the 16 rows land in different banks)

__global__ __launch_bounds__(256) void col_bwd_fused_kernel(const float *__restrict__ gy, const float *__restrict__ X,
                                                            const float *__restrict__ Wm, float *__restrict__ gX,
                                                            double *__restrict__ part, double *__restrict__ sgpart,
                                                            int K, long NL, int Co, int KB) {
    constexpr int COB = 16, PF = 8;
    extern __shared__ __align__(16) float smem[];
    float *wt = smem;                                          // [KB][16] transposed weights of this row block
    float *stage = smem + KB * COB;                            // [4 waves][16][kFusedPitch]: gy once, then batches of X
    double *cred = reinterpret_cast<double *>(stage + 4 * 16 * kFusedPitch);   // [4 waves][256] blocks to fold
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, l16 = lane & 15, lk = lane >> 4;
    const int k0 = blockIdx.y * KB, kcnt = min(KB, K - k0);
    for (int i = threadIdx.x; i < kcnt * COB; i += 256) {
        const int co = i / kcnt, kk = i - co * kcnt;
        wt[kk * COB + co] = co < Co ? Wm[(size_t)co * K + k0 + kk] : 0.f;
    }
    long c0 = ((long)blockIdx.x * 256 + threadIdx.x) * 2;
    const bool active = c0 < NL;
    if (!active) c0 = NL - 2;
    float g[COB][2], s2[2] = {0.f, 0.f};
    float *mine = stage + wave * 16 * kFusedPitch;
#pragma unroll
    for (int co = 0; co < COB; ++co) {
        float2 t = make_float2(0.f, 0.f);
        if (co < Co && active) t = *reinterpret_cast<const float2 *>(gy + (size_t)co * NL + c0);   // idle lanes: gy = 0
        g[co][0] = t.x; g[co][1] = t.y;
        s2[0] += t.x; s2[1] += t.y;
        *reinterpret_cast<float2 *>(mine + co * kFusedPitch + 2 * lane) = t;
    }
    __syncthreads();
    double ga[32], sgt = 0.0;   // the wave's gy as MFMA A fragments: row l16, column 4 * step + lk
#pragma unroll
    for (int st = 0; st < 32; ++st) {
        ga[st] = (double)mine[l16 * kFusedPitch + 4 * st + lk];
        sgt += ga[st];
    }
    sgt += __shfl_xor(sgt, 16, 64);
    sgt += __shfl_xor(sgt, 32, 64);
    __syncthreads();   // the staging area now takes batches of X

    auto one_row = [&](const int kk, const float2 xv, const float2 old) {
        const float c0v = fmaf(-0.5f, xv.x, 0.5f), c1v = fmaf(-0.5f, xv.y, 0.5f);
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int q = 0; q < COB / 4; ++q) {
            const float4 w4 = *reinterpret_cast<const float4 *>(wt + kk * COB + 4 * q);
            const float wv[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                a0 = fmaf(sat01(fmaf(wv[j], 0.5f, c0v)), g[4 * q + j][0], a0);
                a1 = fmaf(sat01(fmaf(wv[j], 0.5f, c1v)), g[4 * q + j][1], a1);
            }
        }
        if (active)
            *reinterpret_cast<float2 *>(gX + (size_t)(k0 + kk) * NL + c0) =
                make_float2(old.x + fmaf(2.f, a0, -s2[0]), old.y + fmaf(2.f, a1, -s2[1]));
        // for the weight gradient; idle lanes (columns past NL, re-pointed at the last two) stage zeros, so that a
        // non-finite X there cannot reach the products of every row through 0 * Inf
        *reinterpret_cast<float2 *>(mine + (kk & 15) * kFusedPitch + 2 * lane) = active ? xv : make_float2(0.f, 0.f);
    };
    auto ld2 = [&](const float *base, int kk) {
        return *reinterpret_cast<const float2 *>(base + (size_t)(k0 + min(kk, kcnt - 1)) * NL + c0);
    };

    float2 nx[PF], no[PF];
#pragma unroll
    for (int r = 0; r < PF; ++r) { nx[r] = ld2(X, r); no[r] = ld2(gX, r); }
    const int nbatches = ceil_div(kcnt, 16);
    for (int b = 0; b < nbatches; ++b) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            float2 cx[PF], co_[PF];
#pragma unroll
            for (int r = 0; r < PF; ++r) { cx[r] = nx[r]; co_[r] = no[r]; }
            const int kb = b * 16 + h * PF;
#pragma unroll
            for (int r = 0; r < PF; ++r) { nx[r] = ld2(X, kb + PF + r); no[r] = ld2(gX, kb + PF + r); }
#pragma unroll
            for (int r = 0; r < PF; ++r) {
                if (kb + r < kcnt) one_row(kb + r, cx[r], co_[r]);
                else *reinterpret_cast<float2 *>(mine + ((kb + r) & 15) * kFusedPitch + 2 * lane) = make_float2(0.f, 0.f);
            }
        }
        __syncthreads();
        double4v acc = double4v{0.0, 0.0, 0.0, 0.0};
#pragma unroll
        for (int st = 0; st < 32; ++st) {
            const double xb = (double)mine[l16 * kFusedPitch + 4 * st + lk];
            acc = __builtin_amdgcn_mfma_f64_16x16x4f64(ga[st], xb, acc, 0, 0, 0);
        }
        // C layout: lane l, register e -> gy row 4 e + l / 16, X row l % 16
#pragma unroll
        for (int e = 0; e < 4; ++e) cred[wave * 256 + (4 * e + lk) * 16 + l16] = acc[e];
        __syncthreads();
        {
            const int co = threadIdx.x >> 4, kk = b * 16 + (threadIdx.x & 15);
            const double v = (cred[threadIdx.x] + cred[256 + threadIdx.x]) + (cred[512 + threadIdx.x] + cred[768 + threadIdx.x]);
            if (co < Co && kk < kcnt) part[(size_t)blockIdx.x * Co * K + (size_t)co * K + k0 + kk] = v;
        }
        // (the next batch's writes to the staging area and to cred come after the next barrier pair's first half:
        // every wave passes the barrier above only after all reads of this batch's staging data)
    }
    if (blockIdx.y == 0) {
        __syncthreads();
        if (lane < 16) cred[wave * 16 + lane] = sgt;
        __syncthreads();
        if (threadIdx.x < 16 && threadIdx.x < Co)
            sgpart[(size_t)blockIdx.x * Co + threadIdx.x] =
                (cred[threadIdx.x] + cred[16 + threadIdx.x]) + (cred[32 + threadIdx.x] + cred[48 + threadIdx.x]);
    }
}

// gX[k, nl] += sum_co hardtanh(W[co,k] - X[k,nl]) * gy[co,nl], any number of output channels: lane = column,
// TK rows of X per lane in registers, gy streamed per output channel.
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

// ---------------------------------------------------------------------------
// gW[co, k] += sum_nl (X[k,nl] - W[co,k]) * gy[co,nl]  =  sum_nl gy * X  -  W * sum_nl gy
// The first term is a (Co x NL) x (NL x K) matrix product whose operands are both contiguous along the
// reduction axis: it runs on v_mfma_f64_16x16x4_f64 straight from global memory.  Lane l of a wave loads
// one float4 of row (l % 16) of each operand tile at columns nl0 + 4 * (l / 16) .. + 3 (64 contiguous bytes
// per row and instruction) and feeds component j of both to MFMA step j, so every column meets its partner.
// A wave owns CT x KT accumulator tiles (16 x 16 fp64 each) and its own share of the 16-column groups, with
// the next group's loads in flight during the 4 * CT * KT MFMAs of the current one; the four waves of a
// workgroup are folded through LDS and leave one fp64 slab (+ sum_nl gy per row) per workgroup, which the
// slab finalize of the NCHW weight gradient adds up (grad_w.hip).  fp64 products and sums: see grad_w_mfma.hip.
// ---------------------------------------------------------------------------
template <int CT, int KT>
__global__ __launch_bounds__(256, 2) void col_grad_w_mfma_kernel(const float *__restrict__ gy,
                                                              const float *__restrict__ X,
                                                              double *__restrict__ part,
                                                              double *__restrict__ sgpart, int K, long NL, int Co) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, l16 = lane & 15, lk = lane >> 4;
    const int co_blk = blockIdx.z * (16 * CT), k_blk = blockIdx.y * (16 * KT);
    const float *arow[CT], *brow[KT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) arow[ct] = gy + (size_t)min(co_blk + ct * 16 + l16, Co - 1) * NL + 4 * lk;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) brow[kt] = X + (size_t)min(k_blk + kt * 16 + l16, K - 1) * NL + 4 * lk;

    double4v acc[CT][KT];
    double sgt[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        sgt[ct] = 0.0;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) acc[ct][kt] = double4v{0.0, 0.0, 0.0, 0.0};
    }
    const long ngroups = NL / 16;                       // whole groups; the launcher hands the tail to a second pass
    const long stride = (long)gridDim.x * 4;
    long grp = (long)blockIdx.x * 4 + wave;
    float4 an[CT], bn[KT];
    if (grp < ngroups) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) an[ct] = *reinterpret_cast<const float4 *>(arow[ct] + grp * 16);
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) bn[kt] = *reinterpret_cast<const float4 *>(brow[kt] + grp * 16);
    }
    for (; grp < ngroups; grp += stride) {
        float4 ac[CT], bc[KT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) ac[ct] = an[ct];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) bc[kt] = bn[kt];
        if (grp + stride < ngroups) {
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) an[ct] = *reinterpret_cast<const float4 *>(arow[ct] + (grp + stride) * 16);
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) bn[kt] = *reinterpret_cast<const float4 *>(brow[kt] + (grp + stride) * 16);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            double a[CT], b[KT];
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                a[ct] = (double)(j == 0 ? ac[ct].x : j == 1 ? ac[ct].y : j == 2 ? ac[ct].z : ac[ct].w);
                sgt[ct] += a[ct];
            }
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
                b[kt] = (double)(j == 0 ? bc[kt].x : j == 1 ? bc[kt].y : j == 2 ? bc[kt].z : bc[kt].w);
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
#pragma unroll
                for (int kt = 0; kt < KT; ++kt)
                    acc[ct][kt] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[ct], b[kt], acc[ct][kt], 0, 0, 0);
        }
    }
    // the columns past the last whole group (NL % 16 of them, NL % 4 == 0): one more step on wave 0 of block 0,
    // lanes whose float4 lies past the end contribute zeros
    if (blockIdx.x == 0 && wave == 0 && ngroups * 16 < NL) {
        const bool in = ngroups * 16 + 4 * lk < NL;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            double a[CT], b[KT];
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                a[ct] = in ? (double)arow[ct][ngroups * 16 + j] : 0.0;
                sgt[ct] += a[ct];
            }
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) b[kt] = in ? (double)brow[kt][ngroups * 16 + j] : 0.0;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
#pragma unroll
                for (int kt = 0; kt < KT; ++kt)
                    acc[ct][kt] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[ct], b[kt], acc[ct][kt], 0, 0, 0);
        }
    }

    // fold the four waves in fp64 through LDS: waves 1..3 park their registers, wave 0 adds them in a fixed order
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {           // the four lanes that hold the same row of gy
        sgt[ct] += __shfl_xor(sgt[ct], 16, 64);
        sgt[ct] += __shfl_xor(sgt[ct], 32, 64);
    }
    constexpr int REGS = CT * KT * 4 + CT;
    __shared__ double red[3 * REGS * 64];
    if (wave > 0) {
        double *mine = red + (size_t)(wave - 1) * REGS * 64;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            mine[(CT * KT * 4 + ct) * 64 + lane] = sgt[ct];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int e = 0; e < 4; ++e) mine[((ct * KT + kt) * 4 + e) * 64 + lane] = acc[ct][kt][e];
        }
    }
    __syncthreads();
    if (wave > 0) return;
    for (int wv = 0; wv < 3; ++wv) {
        const double *theirs = red + (size_t)wv * REGS * 64;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            sgt[ct] += theirs[(CT * KT * 4 + ct) * 64 + lane];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[ct][kt][e] += theirs[((ct * KT + kt) * 4 + e) * 64 + lane];
        }
    }
    double *dst = part + (size_t)blockIdx.x * Co * K;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            const int kcol = k_blk + kt * 16 + l16;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int co = co_blk + ct * 16 + 4 * e + lk;    // C layout: lane l, register e -> row 4 e + l / 16
                if (co < Co && kcol < K) dst[(size_t)co * K + kcol] = acc[ct][kt][e];
            }
        }
    if (blockIdx.y == 0 && lane < 16) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            const int co = co_blk + ct * 16 + lane;
            if (co < Co) sgpart[(size_t)blockIdx.x * Co + co] = sgt[ct];
        }
    }
}

// gW[co, k] += sum_nl (X[k,nl] - W[co,k]) * gy[co,nl], matrices whose rows are not whole float4 groups
// (NL % 4 != 0 or unaligned bases): one workgroup per TM x TK block of gW, element-wise loads.
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
    double wv[TM][TK], dacc[TM][TK];   // products and sums in double: NL can be hundreds of thousands of terms
#pragma unroll
    for (int m = 0; m < TM; ++m)
#pragma unroll
        for (int t = 0; t < TK; ++t) {
            wv[m][t] = (double)Wm[(size_t)cc[m] * K + kk[t]];
            dacc[m][t] = 0.0;
        }
    for (long nl = threadIdx.x; nl < NL; nl += 256) {
        double xv[TK], g[TM];
#pragma unroll
        for (int t = 0; t < TK; ++t) xv[t] = (double)X[(size_t)kk[t] * NL + nl];
#pragma unroll
        for (int m = 0; m < TM; ++m) g[m] = (double)gy[(size_t)cc[m] * NL + nl];
#pragma unroll
        for (int m = 0; m < TM; ++m)
#pragma unroll
            for (int t = 0; t < TK; ++t) dacc[m][t] = fma(xv[t] - wv[m][t], g[m], dacc[m][t]);
    }
    __shared__ double red[4][TM * TK];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
    for (int m = 0; m < TM; ++m)
#pragma unroll
        for (int t = 0; t < TK; ++t) {
            const double s = wave_sum(dacc[m][t]);
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

// ---------------------------------------------------------------------------
// Both gradients of a matrix with few columns in ONE launch and without a workspace (the reference's own
// comparison shape, adder_cuda/test_cuda.py:161-176: Co = 32, K = 288, NL = 1024).  With so few columns the slab
// kernels above are a chain of launches that each last as long as a launch takes; here a workgroup owns KB rows of
// X over ALL columns, so the weight gradient of its rows needs no partner: thread t holds columns t, t + 256, ... of
// its rows in registers, walks the output channels once (gy straight from memory, coalesced; the weight as a scalar),
// finishes its elements of gX on the spot and leaves, per output channel, its share of sum_c X[k,c] gy[co,c] and of
// sum_c gy[co,c] to a wave reduction.  The per-thread shares are at most CPT terms long and the sums over the
// columns at most 2048: fp32 throughout (the slab kernels use fp64 because they sum 262 144).
//   gX[k,c] += sum_co hardtanh(W[co,k] - X[k,c]) gy[co,c]        (test_cuda.py:57-60; adder.cu:17,246)
//   gW[co,k] += sum_c X[k,c] gy[co,c] - W[co,k] sum_c gy[co,c]   (test_cuda.py:35-41; adder.cu:247)
// gW or gX may be null (ADDER_CONV_INPUT / ADDER_CONV_WEIGHT).
// ---------------------------------------------------------------------------
template <int KB, int CPT, int GB>
__global__ __launch_bounds__(256) void col_bwd_small_kernel(const float *__restrict__ gy, const float *__restrict__ X,
                                                            const float *__restrict__ Wm, float *__restrict__ gW,
                                                            float *__restrict__ gX, int K, int NL, int Co) {
    extern __shared__ __align__(16) float smem[];
    float *wl = smem;                      // [Co][KB] weights of this workgroup's rows
    float *red = smem + Co * KB;           // [4 waves][Co][KB + 1] wave sums
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int k0 = blockIdx.x * KB;
    for (int e = threadIdx.x; e < Co * KB; e += 256) {
        const int co = e / KB, kk = e - co * KB;
        wl[e] = Wm[(size_t)co * K + min(k0 + kk, K - 1)];
    }
    float x[KB][CPT], acc[KB][CPT];
#pragma unroll
    for (int kk = 0; kk < KB; ++kk)
#pragma unroll
        for (int j = 0; j < CPT; ++j) {
            const int c = threadIdx.x + j * 256;
            x[kk][j] = (k0 + kk < K && c < NL) ? X[(size_t)(k0 + kk) * NL + c] : 0.f;
            acc[kk][j] = 0.f;
        }
    // gy of the own columns, GB output channels at a time with the next GB in flight: a channel's arithmetic is a
    // few dozen instructions, far shorter than a trip to memory
    float g[2][GB][CPT];
    auto fetch = [&](int co0, float (&dst)[GB][CPT]) {
#pragma unroll
        for (int u = 0; u < GB; ++u)
#pragma unroll
            for (int j = 0; j < CPT; ++j) {
                const int c = threadIdx.x + j * 256;
                dst[u][j] = (co0 + u < Co && c < NL) ? gy[(size_t)(co0 + u) * NL + c] : 0.f;
            }
    };
    fetch(0, g[0]);
    __syncthreads();
    auto batch = [&](int co0, const float (&gb)[GB][CPT]) {
        // (channels past Co were fetched as zeros: their terms vanish and their sums are not stored)
        float sxg[GB * KB], sg[GB];
#pragma unroll
        for (int u = 0; u < GB; ++u) {
            const int co = min(co0 + u, Co - 1);
            sg[u] = 0.f;
#pragma unroll
            for (int j = 0; j < CPT; ++j) sg[u] += gb[u][j];
#pragma unroll
            for (int kk = 0; kk < KB; ++kk) {
                const float w = wl[co * KB + kk];
                float pw = 0.f;
#pragma unroll
                for (int j = 0; j < CPT; ++j) {
                    acc[kk][j] = fmaf(hardtanh(w - x[kk][j]), gb[u][j], acc[kk][j]);
                    pw = fmaf(x[kk][j], gb[u][j], pw);
                }
                sxg[u * KB + kk] = pw;
            }
        }
        if (gW) {
            // all sums of the batch at once: a reduce-scatter over the lanes, lane l ends with sum number index(l)
            const float a = wave_sum_scatter<GB * KB>(sxg, lane);
            const float c = wave_sum_scatter<GB>(sg, lane);
            if (lane < GB * KB) {
                const int e = wave_sum_scatter_index<GB * KB>(lane), u = e / KB, kk = e - u * KB;
                if (co0 + u < Co) red[(wave * Co + co0 + u) * (KB + 1) + kk] = a;
            }
            if (lane < GB) {
                const int u = wave_sum_scatter_index<GB>(lane);
                if (co0 + u < Co) red[(wave * Co + co0 + u) * (KB + 1) + KB] = c;
            }
        }
    };
    for (int co0 = 0; co0 < Co; co0 += 2 * GB) {
        if (co0 + GB < Co) fetch(co0 + GB, g[1]);
        batch(co0, g[0]);
        if (co0 + 2 * GB < Co) fetch(co0 + 2 * GB, g[0]);
        if (co0 + GB < Co) batch(co0 + GB, g[1]);
    }
    if (gX) {
#pragma unroll
        for (int kk = 0; kk < KB; ++kk)
#pragma unroll
            for (int j = 0; j < CPT; ++j) {
                const int c = threadIdx.x + j * 256;
                if (k0 + kk < K && c < NL) gX[(size_t)(k0 + kk) * NL + c] += acc[kk][j];
            }
    }
    if (gW) {
        __syncthreads();
        const int stride = Co * (KB + 1);
        for (int e = threadIdx.x; e < Co * KB; e += 256) {
            const int co = e / KB, kk = e - co * KB;
            if (k0 + kk >= K) continue;
            const float *r = red + co * (KB + 1);
            const float sxg = (r[kk] + r[stride + kk]) + (r[2 * stride + kk] + r[3 * stride + kk]);
            const float sg = (r[KB] + r[stride + KB]) + (r[2 * stride + KB] + r[3 * stride + KB]);
            gW[(size_t)co * K + k0 + kk] += sxg - wl[e] * sg;
        }
    }
}

// matrices the one-launch kernel above serves: few columns, a wave-sum table that fits the LDS
static bool col_bwd_small_applies(int K, long NL, int Co) { return NL <= 2048 && Co <= 512; }

// gW / gX: either may be null
int launch_col_bwd_small(const float *gy, const float *X, const float *Wm, float *gW, float *gX, int K, long NL, int Co,
                         hipStream_t s) {
    if (!col_bwd_small_applies(K, NL, Co)) return ADDER_ERR_UNSUPPORTED;
    const int cpt = (int)ceil_div_l(NL, 256);
#define ADDER_COL_SMALL(KB, CPT, GB)                                                                                 \
    hipLaunchKernelGGL((col_bwd_small_kernel<KB, CPT, GB>), dim3(ceil_div(K, KB)), dim3(256),                            \
                       (Co * KB + 4 * Co * (KB + 1)) * 4, s, gy, X, Wm, gW, gX, K, (int)NL, Co)
    // one row of X per workgroup while that fills the chip, two on taller matrices
    const bool tall = K >= 1024;
    if (cpt <= 1) { if (tall) ADDER_COL_SMALL(2, 1, 8); else ADDER_COL_SMALL(1, 1, 8); }
    else if (cpt <= 2) { if (tall) ADDER_COL_SMALL(2, 2, 8); else ADDER_COL_SMALL(1, 2, 8); }
    else if (cpt <= 4) { if (tall) ADDER_COL_SMALL(2, 4, 8); else ADDER_COL_SMALL(1, 4, 8); }
    else { if (tall) ADDER_COL_SMALL(2, 8, 4); else ADDER_COL_SMALL(1, 8, 4); }
#undef ADDER_COL_SMALL
    return check_launch();
}

static bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
static bool aligned8(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 7) == 0; }

int launch_col_fwd(const float *X, const float *Wm, float *out, int K, long NL, int Co, hipStream_t s) {
    const int KB = K < 512 ? K : 512;   // rows of X per LDS block of weights (32 KB at 16 rows of W)
    if (NL >= 65536 && NL % 2 == 0 && aligned8(X) && aligned8(out)) {
        // many columns: two per lane (twice the arithmetic per row load), 16 rows of W per lane
        hipLaunchKernelGGL((col_fwd_lds_kernel<16, 2, true, 8, 1>), dim3((unsigned)ceil_div_l(NL, 512), ceil_div(Co, 16)),
                           dim3(256), KB * 16 * 4, s, X, Wm, out, K, NL, Co, KB);
    } else if (NL >= 16384) {
        hipLaunchKernelGGL((col_fwd_lds_kernel<16, 1, false, 8, 1>), dim3((unsigned)ceil_div_l(NL, 256), ceil_div(Co, 16)),
                           dim3(256), KB * 16 * 4, s, X, Wm, out, K, NL, Co, KB);
    } else {
        // few columns: the work is a chain of row batches per wave -- 8 rows of W per lane (more workgroups) and the
        // rows of X split over the four waves of a workgroup
        hipLaunchKernelGGL((col_fwd_lds_kernel<8, 1, false, 8, 4>), dim3((unsigned)ceil_div_l(NL, 64), ceil_div(Co, 8)),
                           dim3(256), KB * 8 * 4, s, X, Wm, out, K, NL, Co, KB);
    }
    return check_launch();
}

// ---- weight gradient: slab plan -------------------------------------------------------------------------
struct ColGwPlan { int ct, kt, slots, gy, gz; bool mfma; };

static ColGwPlan plan_col_grad_w(int K, long NL, int Co) {
    ColGwPlan p{};
    p.mfma = NL % 4 == 0 && NL >= 16;
    if (!p.mfma) return p;
    // accumulator tiles per wave: one row of up to five for layers with up to 16 output channels (X is read once,
    // gy once per block of 80 rows of X), else 2 x 4 or 2 x 2 / 3 x 1: enough to amortise the operand loads, few
    // enough for two waves per SIMD (nine tiles were slower: one wave per SIMD, or spills)
    const int ctn = ceil_div(Co, 16), ktn = ceil_div(K, 16);
    if (ctn == 1) { p.ct = 1; p.kt = ktn < 5 ? (ktn < 4 ? (ktn < 2 ? 1 : 2) : 4) : 5; }
    else { p.ct = 2; p.kt = ktn < 2 ? 1 : 2; }
    p.gz = ceil_div(Co, 16 * p.ct);
    p.gy = ceil_div(K, 16 * p.kt);
    // two workgroups per CU (two waves per SIMD: the accumulator tiles are chosen to leave room for that), at least
    // one 16-column group per wave
    long want = ceil_div_l(512, (long)p.gy * p.gz);
    const long most = ceil_div_l(NL / 16, 4);
    if (want > most) want = most;
    p.slots = (int)(want < 1 ? 1 : want);
    return p;
}

// the fused backward serves layers with up to 16 output channels on matrices with many columns (one slab per 512)
static bool col_bwd_fused_applies(int K, long NL, int Co) { return Co <= 16 && NL % 2 == 0 && NL >= 65536 && K >= 16; }
static int col_bwd_fused_slots(long NL) { return (int)ceil_div_l(NL, 512); }

size_t col_grad_w_workspace_bytes(int K, long NL, int Co) {
    if (col_bwd_small_applies(K, NL, Co)) return 0;   // one launch, no slabs
    const ColGwPlan p = plan_col_grad_w(K, NL, Co);
    int slots = p.mfma ? p.slots : 0;
    if (col_bwd_fused_applies(K, NL, Co) && col_bwd_fused_slots(NL) > slots) slots = col_bwd_fused_slots(NL);
    if (!slots) return 0;
    return (sizeof(double) * (size_t)slots * ((size_t)Co * K + Co) + 255) & ~(size_t)255;
}

// Both gradients in one pass over X (col_bwd_fused_kernel); ADDER_ERR_UNSUPPORTED (nothing launched) where it does
// not apply, and the caller runs the two separate kernels.
int launch_col_bwd_fused(const float *gy, const float *X, const float *Wm, float *gW, float *gX, int K, long NL, int Co,
                         void *ws, hipStream_t s) {
    if (!col_bwd_fused_applies(K, NL, Co) || !ws || !aligned8(X) || !aligned8(gy) || !aligned8(gX) ||
        (reinterpret_cast<uintptr_t>(ws) & 255))
        return ADDER_ERR_UNSUPPORTED;
    const int slots = col_bwd_fused_slots(NL);
    int KB = round_up(K, 16);
    if (KB > 256) KB = 256;
    const int lds = KB * 16 * 4 + 4 * 16 * kFusedPitch * 4 + 4 * 256 * 8;
    if (int rc = allow_dynamic_lds<&col_bwd_fused_kernel>(lds)) return rc;
    double *part = reinterpret_cast<double *>(ws);
    double *sgpart = part + (size_t)slots * Co * K;
    hipLaunchKernelGGL(col_bwd_fused_kernel, dim3(slots, ceil_div(K, KB)), dim3(256), lds, s, gy, X, Wm, gX, part, sgpart,
                       K, NL, Co, KB);
    if (int rc = check_launch()) return rc;
    return launch_grad_w_slab_finalize(part, sgpart, Wm, gW, slots, Co, K, /*accumulate=*/true, s);
}

template <int CT, int KT>
static void launch_col_gw(const float *gy, const float *X, double *part, double *sgpart, int K, long NL, int Co,
                          const ColGwPlan &p, hipStream_t s) {
    hipLaunchKernelGGL((col_grad_w_mfma_kernel<CT, KT>), dim3(p.slots, p.gy, p.gz), dim3(256), 0, s, gy, X, part, sgpart,
                       K, NL, Co);
}

int launch_col_grad_w(const float *gy, const float *X, const float *Wm, float *gW, int K, long NL, int Co,
                      void *ws, hipStream_t s) {
    if (col_bwd_small_applies(K, NL, Co)) return launch_col_bwd_small(gy, X, Wm, gW, nullptr, K, NL, Co, s);
    const ColGwPlan p = plan_col_grad_w(K, NL, Co);
    if (p.mfma && ws && aligned16(X) && aligned16(gy) && (reinterpret_cast<uintptr_t>(ws) & 255) == 0) {
        double *part = reinterpret_cast<double *>(ws);
        double *sgpart = part + (size_t)p.slots * Co * K;
        const int tag = p.ct * 16 + p.kt;
        switch (tag) {
            case 1 * 16 + 1: launch_col_gw<1, 1>(gy, X, part, sgpart, K, NL, Co, p, s); break;
            case 1 * 16 + 2: launch_col_gw<1, 2>(gy, X, part, sgpart, K, NL, Co, p, s); break;
            case 1 * 16 + 4: launch_col_gw<1, 4>(gy, X, part, sgpart, K, NL, Co, p, s); break;
            case 1 * 16 + 5: launch_col_gw<1, 5>(gy, X, part, sgpart, K, NL, Co, p, s); break;
            case 2 * 16 + 1: launch_col_gw<2, 1>(gy, X, part, sgpart, K, NL, Co, p, s); break;
            default: launch_col_gw<2, 2>(gy, X, part, sgpart, K, NL, Co, p, s); break;
        }
        if (int rc = check_launch()) return rc;
        return launch_grad_w_slab_finalize(part, sgpart, Wm, gW, p.slots, Co, K, /*accumulate=*/true, s);
    }
    constexpr int TM = 4, TK = 4;
    hipLaunchKernelGGL((col_grad_w_kernel<TM, TK>), dim3(ceil_div(K, TK), ceil_div(Co, TM)), dim3(256), 0, s, gy, X,
                       Wm, gW, K, NL, Co);
    return check_launch();
}

int launch_col_grad_x(const float *gy, const float *X, const float *Wm, float *gX, int K, long NL, int Co,
                      hipStream_t s) {
    if (col_bwd_small_applies(K, NL, Co)) return launch_col_bwd_small(gy, X, Wm, nullptr, gX, K, NL, Co, s);
    if (Co <= 32) {
        // gy in registers, X streamed once; rows in blocks of KB whose weights fit a 32 KB LDS tile
        const int COB = Co <= 16 ? 16 : 32;
        int KB = 32 * 1024 / (4 * COB);
        if (KB > K) KB = K;
        // enough workgroups for the chip when there are few columns: split the rows further
        const long colblocks = ceil_div_l(NL, 256);
        while (KB > 16 && colblocks * ceil_div(K, KB) < 1024) KB = (KB + 1) / 2;
        const int lds = KB * COB * 4;
        const bool vec2 = NL % 2 == 0 && aligned8(X) && aligned8(gy) && aligned8(gX) && NL >= 65536;
        if (COB == 16 && vec2)
            hipLaunchKernelGGL((col_grad_x_reg_kernel<16, 2, true>), dim3((unsigned)ceil_div_l(NL, 512), ceil_div(K, KB)),
                               dim3(256), lds, s, gy, X, Wm, gX, K, NL, Co, KB);
        else if (COB == 16)
            hipLaunchKernelGGL((col_grad_x_reg_kernel<16, 1, false>), dim3((unsigned)colblocks, ceil_div(K, KB)),
                               dim3(256), lds, s, gy, X, Wm, gX, K, NL, Co, KB);
        else
            hipLaunchKernelGGL((col_grad_x_reg_kernel<32, 1, false>), dim3((unsigned)colblocks, ceil_div(K, KB)),
                               dim3(256), lds, s, gy, X, Wm, gX, K, NL, Co, KB);
        return check_launch();
    }
    constexpr int TK = 8;
    hipLaunchKernelGGL(col_grad_x_kernel<TK>, dim3((unsigned)ceil_div_l(NL, 256), ceil_div(K, TK)), dim3(256), 0, s,
                       gy, X, Wm, gX, K, NL, Co);
    return check_launch();
}

}  // namespace adder
