// The parameter update of the training script (main.py:67 of the reference: torch.optim.SGD with momentum and weight
// decay) for all tensors of a parameter group in one launch:
//     g' = g + weight_decay * p,   buf = momentum * buf + g',   p = p - lr * buf.
// A network of adder layers has many small parameters (ResNet-20: 65 tensors, 272 000 values, the largest 36 864);
// the framework's fused update gives every tensor one workgroup that walks it alone, 15 us per launch and two
// launches.  Here a workgroup takes 1024 values of whichever tensor its index falls into; the table of tensors
// travels by value in the kernel arguments.
#include "common.hpp"

namespace adder {

struct SgdBatch {
    float *p[kSgdBatchMax];
    const float *g[kSgdBatchMax];
    float *buf[kSgdBatchMax];
    int n[kSgdBatchMax];
    int first_block[kSgdBatchMax + 1];   // workgroups [first_block[t], first_block[t + 1]) belong to tensor t
};

static constexpr int kSgdChunk = 1024;   // values per workgroup: 256 threads x one float4

template <bool VEC>
__global__ __launch_bounds__(256) void sgd_momentum_kernel(const SgdBatch b, int count, const float *__restrict__ lr_ptr,
                                                           float lr, float momentum, float weight_decay) {
    // the tensor this workgroup belongs to: last t with first_block[t] <= blockIdx.x
    int lo = 0, hi = count - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (b.first_block[mid] <= (int)blockIdx.x) lo = mid; else hi = mid - 1;
    }
    const int t = lo, n = b.n[t];
    float *__restrict__ p = b.p[t];
    const float *__restrict__ g = b.g[t];
    float *__restrict__ buf = b.buf[t];
    const float rate = lr_ptr ? *lr_ptr : lr;
    const int i = ((int)blockIdx.x - b.first_block[t]) * kSgdChunk + threadIdx.x * 4;
    if (VEC && i + 4 <= n) {
        const float4 pv = *reinterpret_cast<const float4 *>(p + i), gv = *reinterpret_cast<const float4 *>(g + i),
                     bv = *reinterpret_cast<const float4 *>(buf + i);
        float4 nb, np;
        nb.x = fmaf(momentum, bv.x, fmaf(weight_decay, pv.x, gv.x));
        nb.y = fmaf(momentum, bv.y, fmaf(weight_decay, pv.y, gv.y));
        nb.z = fmaf(momentum, bv.z, fmaf(weight_decay, pv.z, gv.z));
        nb.w = fmaf(momentum, bv.w, fmaf(weight_decay, pv.w, gv.w));
        np.x = fmaf(-rate, nb.x, pv.x);
        np.y = fmaf(-rate, nb.y, pv.y);
        np.z = fmaf(-rate, nb.z, pv.z);
        np.w = fmaf(-rate, nb.w, pv.w);
        *reinterpret_cast<float4 *>(buf + i) = nb;
        *reinterpret_cast<float4 *>(p + i) = np;
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (i + e < n) {
                const float pv = p[i + e];
                const float nb = fmaf(momentum, buf[i + e], fmaf(weight_decay, pv, g[i + e]));
                buf[i + e] = nb;
                p[i + e] = fmaf(-rate, nb, pv);
            }
    }
}

int launch_sgd_momentum(int count, float *const *p, const float *const *g, float *const *buf, const long *n,
                        const float *lr_ptr, float lr, float momentum, float weight_decay, hipStream_t s) {
    SgdBatch b;
    int blocks = 0;
    bool vec = true;
    for (int t = 0; t < count; ++t) {
        b.p[t] = p[t];
        b.g[t] = g[t];
        b.buf[t] = buf[t];
        b.n[t] = (int)n[t];
        b.first_block[t] = blocks;
        blocks += (int)ceil_div_l(n[t], kSgdChunk);
        vec = vec && ((reinterpret_cast<uintptr_t>(p[t]) | reinterpret_cast<uintptr_t>(g[t]) |
                       reinterpret_cast<uintptr_t>(buf[t])) & 15) == 0;
    }
    b.first_block[count] = blocks;
    if (vec)
        hipLaunchKernelGGL(sgd_momentum_kernel<true>, dim3(blocks), dim3(256), 0, s, b, count, lr_ptr, lr, momentum,
                           weight_decay);
    else
        hipLaunchKernelGGL(sgd_momentum_kernel<false>, dim3(blocks), dim3(256), 0, s, b, count, lr_ptr, lr, momentum,
                           weight_decay);
    return check_launch();
}

}  // namespace adder
