// Small memory-bound helpers of the backward pass (see fb_bwd.hip for the main kernel).
#include "fb_kernels.h"

namespace fb {

// ------------------------------------------------------------------------------ preprocess
template <class T>
__global__ __launch_bounds__(256) void bwd_preprocess_kernel(const BwdArgs a, int64_t ws_floats) {
    const int64_t rows = (int64_t)a.B * a.H * a.Lq;
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t nthreads = (int64_t)gridDim.x * blockDim.x;
    for (int64_t rix = gid; rix < rows; rix += nthreads) {
        const int i = (int)(rix % a.Lq);
        const int bh = (int)(rix / a.Lq);
        const int b = bh / a.H, h = bh % a.H;
        const uint16_t *orow = a.o.ptr + b * a.o.sb + h * a.o.sh + (int64_t)i * a.o.ss;
        const uint16_t *drow = a.dout.ptr + b * a.dout.sb + h * a.dout.sh + (int64_t)i * a.dout.ss;
        float acc = 0.f;
        const bool vec = a.o.vec_ok && a.dout.vec_ok && a.d % 8 == 0;
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
        a.delta[rix] = acc;
    }
    f32x4_t *ws4 = reinterpret_cast<f32x4_t *>(a.dq_acc);
    const f32x4_t z = {0.f, 0.f, 0.f, 0.f};
    for (int64_t i = gid; i < ws_floats / 4; i += nthreads) ws4[i] = z;
}

// -------------------------------------------------------------------------------- finalize
template <class T>
__global__ __launch_bounds__(256) void bwd_finalize_kernel(const BwdArgs a) {
    const int64_t rows = (int64_t)a.B * a.H * a.Lq;
    const int64_t rix = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (rix >= rows) return;
    const int i = (int)(rix % a.Lq);
    const int bh = (int)(rix / a.Lq);
    const int b = bh / a.H, h = bh % a.H;
    const float *src = a.dq_acc + (int64_t)bh * a.dq_rows * a.lq_pad + i;
    uint16_t *dqrow = const_cast<uint16_t *>(a.dq.ptr) + b * a.dq.sb + h * a.dq.sh + (int64_t)i * a.dq.ss;
    for (int ch = 0; ch < a.d; ++ch) dqrow[ch] = T::from_float(src[(int64_t)ch * a.lq_pad] * a.scale);
    if (a.r > 0) {
        uint16_t *dqbrow = const_cast<uint16_t *>(a.dqb.ptr) + b * a.dqb.sb + h * a.dqb.sh + (int64_t)i * a.dqb.ss;
        for (int ch = 0; ch < a.r; ++ch) dqbrow[ch] = T::from_float(src[(int64_t)(a.r_row0 + ch) * a.lq_pad]);
    }
}

// ------------------------------------------------------------------------------- launchers
hipError_t launch_bwd_preprocess(const BwdArgs &a, bool bf16, hipStream_t stream) {
    const int64_t ws_floats = (int64_t)a.B * a.H * a.dq_rows * a.lq_pad;
    const int64_t rows = (int64_t)a.B * a.H * a.Lq;
    int64_t blocks = (rows + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (blocks < 1) blocks = 1;
    if (bf16)
        hipLaunchKernelGGL(bwd_preprocess_kernel<BF16>, dim3((unsigned)blocks), dim3(256), 0, stream, a, ws_floats);
    else
        hipLaunchKernelGGL(bwd_preprocess_kernel<F16>, dim3((unsigned)blocks), dim3(256), 0, stream, a, ws_floats);
    return hipGetLastError();
}

hipError_t launch_bwd_finalize(const BwdArgs &a, bool bf16, hipStream_t stream) {
    const int64_t rows = (int64_t)a.B * a.H * a.Lq;
    const int64_t blocks = (rows + 255) / 256;
    if (bf16)
        hipLaunchKernelGGL(bwd_finalize_kernel<BF16>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
    else
        hipLaunchKernelGGL(bwd_finalize_kernel<F16>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
    return hipGetLastError();
}

} // namespace fb
