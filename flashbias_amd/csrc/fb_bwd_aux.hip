// delta = rowsum(o * dout), the memory-bound first step of the backward pass.  The scratch
// buffer receives what the two main kernels consume: -delta in its first B*H*Lq floats and
// lse * log2(e) in the next B*H*Lq.
// Replaces _bwd_preprocess_do_o_dot of the reference (flash_bias/flash_bias_triton.py:358-400).
#include "fb_kernels.h"

namespace fb {

template <class T>
__global__ __launch_bounds__(256) void bwd_preprocess_kernel(const BwdArgs a) {
    const int64_t rows = (int64_t)a.B * a.H * a.Lq;
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t nthreads = (int64_t)gridDim.x * blockDim.x;
    const bool vec = a.o.vec_ok && a.dout.vec_ok && a.d % 8 == 0;
    for (int64_t rix = gid; rix < rows; rix += nthreads) {
        const int i = (int)(rix % a.Lq);
        const int bh = (int)(rix / a.Lq);
        const int b = bh / a.H, h = bh % a.H;
        const uint16_t *orow = a.o.ptr + b * a.o.sb + h * a.o.sh + (int64_t)i * a.o.ss;
        const uint16_t *drow = a.dout.ptr + b * a.dout.sb + h * a.dout.sh + (int64_t)i * a.dout.ss;
        float acc = 0.f;
        for (int c0 = 0; c0 < a.d; c0 += 8) {
            u32x4_t x, y;
            if (vec) {
                x = load_chunk<true>(orow, 0, 0, 1, c0, a.d);
                y = load_chunk<true>(drow, 0, 0, 1, c0, a.d);
            } else {
                x = load_chunk<false>(orow, 0, 0, 1, c0, a.d);
                y = load_chunk<false>(drow, 0, 0, 1, c0, a.d);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                acc += T::to_float((uint16_t)(x[e] & 0xffffu)) * T::to_float((uint16_t)(y[e] & 0xffffu));
                acc += T::to_float((uint16_t)(x[e] >> 16)) * T::to_float((uint16_t)(y[e] >> 16));
            }
        }
        a.delta[rix] = -acc;
        a.delta[rows + rix] = a.lse[rix] * kLog2e;
    }
}

hipError_t launch_bwd_preprocess(const BwdArgs &a, bool bf16, hipStream_t stream) {
    const int64_t rows = (int64_t)a.B * a.H * a.Lq;
    int64_t blocks = (rows + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (blocks < 1) blocks = 1;
    if (bf16)
        hipLaunchKernelGGL(bwd_preprocess_kernel<BF16>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
    else
        hipLaunchKernelGGL(bwd_preprocess_kernel<F16>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
    return hipGetLastError();
}

} // namespace fb
