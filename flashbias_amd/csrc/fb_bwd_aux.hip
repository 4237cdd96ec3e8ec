// delta = rowsum(o * dout), the memory-bound first step of the backward pass.  The scratch
// buffer receives what the two main kernels consume: -delta in its first B*H*Lq floats,
// lse * log2(e) in the next B*H*Lq, and (where the streamlined dk/dv kernel will run) both again
// as one chunk of 16-bit parts per query (stat_chunk, from stat_offset on).
// Replaces _bwd_preprocess_do_o_dot of the reference (flash_bias/flash_bias_triton.py:358-400).
// Also here: the sum over the batch of a full-shape factor gradient, the memory-bound last step
// of the backward pass for factors that all batch entries share.
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
                acc = __builtin_fmaf(T::to_float((uint16_t)(x[e] & 0xffffu)), T::to_float((uint16_t)(y[e] & 0xffffu)), acc);
                acc = __builtin_fmaf(T::to_float((uint16_t)(x[e] >> 16)), T::to_float((uint16_t)(y[e] >> 16)), acc);
            }
        }
        const float l2 = a.lse[rix] * kLog2e;
        a.delta[rix] = -acc;
        a.delta[rows + rix] = l2;
        if (a.stat_chunks) reinterpret_cast<u32x4_t *>(a.delta + stat_offset(rows))[rix] = stat_chunk<T>(-acc, l2);
    }
}

// Coalesced variant for 16-byte aligned tensors whose rows are 1, 2, 4, 8 or 16 chunks of 8
// channels: one thread per chunk (consecutive threads read consecutive 16 bytes of a row), the
// CH partial sums of a row are added across neighbouring lanes.
// IDX: uint32_t when rows * CH fits (the index arithmetic is a good part of this kernel's work
// and 64-bit divisions are several times as long), else int64_t.
template <class T, int CH, class IDX>
__global__ __launch_bounds__(256) void bwd_preprocess_chunks_kernel(const BwdArgs a) {
    const int64_t rows = (int64_t)a.B * a.H * a.Lq;
    const IDX gid = (IDX)blockIdx.x * blockDim.x + threadIdx.x;
    const IDX nthreads = (IDX)gridDim.x * blockDim.x;
    const IDX total = (IDX)(rows * CH);
    for (IDX cix = gid; cix < total; cix += nthreads) { // rows * CH is a multiple of CH: whole rows per pass
        const int c = (int)(cix % CH);
        const IDX r = cix / CH; // rows in memory order (b, i, h): neighbouring heads are adjacent
        const IDX ri = r / (IDX)a.H;
        const int h = (int)(r - ri * (IDX)a.H);
        const int b = (int)(ri / (IDX)a.Lq);
        const int i = (int)(ri - (IDX)b * (IDX)a.Lq);
        const uint16_t *orow = a.o.ptr + b * a.o.sb + h * a.o.sh + (int64_t)i * a.o.ss;
        const uint16_t *drow = a.dout.ptr + b * a.dout.sb + h * a.dout.sh + (int64_t)i * a.dout.ss;
        float acc = 0.f;
        if (c * 8 < a.d) {
            const u32x4_t x = *reinterpret_cast<const u32x4_t *>(orow + c * 8);
            const u32x4_t y = *reinterpret_cast<const u32x4_t *>(drow + c * 8);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                acc = __builtin_fmaf(T::to_float((uint16_t)(x[e] & 0xffffu)), T::to_float((uint16_t)(y[e] & 0xffffu)), acc);
                acc = __builtin_fmaf(T::to_float((uint16_t)(x[e] >> 16)), T::to_float((uint16_t)(y[e] >> 16)), acc);
            }
        }
#pragma unroll
        for (int m = 1; m < CH; m <<= 1) acc += __shfl_xor(acc, m, 64);
        if (c == 0) {
            const int64_t rix = ((int64_t)b * a.H + h) * a.Lq + i;
            const float l2 = a.lse[rix] * kLog2e;
            a.delta[rix] = -acc;
            a.delta[rows + rix] = l2;
            if (a.stat_chunks) reinterpret_cast<u32x4_t *>(a.delta + stat_offset(rows))[rix] = stat_chunk<T>(-acc, l2);
        }
    }
}

template <class T>
static void launch_preprocess_t(const BwdArgs &a, hipStream_t stream) {
    const int64_t rows = (int64_t)a.B * a.H * a.Lq;
    const bool vec = a.o.vec_ok && a.dout.vec_ok && a.d % 8 == 0;
    const int chunks = (a.d + 7) / 8;
    int ch = 1;
    while (ch < chunks) ch <<= 1;
    if (vec && ch <= 16) {
        int64_t blocks = (rows * ch + 255) / 256;
        if (blocks > 262144) blocks = 262144; // grid-stride beyond that; 256 * blocks stays a multiple of ch
        const dim3 grid((unsigned)blocks), block(256);
        // (the grid-stride step must not overflow either: 2^30 leaves room for it)
        const bool small = rows * ch < ((int64_t)1 << 30);
#define FB_PRE(CHN)                                                                                          \
    if (small)                                                                                               \
        hipLaunchKernelGGL((bwd_preprocess_chunks_kernel<T, CHN, uint32_t>), grid, block, 0, stream, a);     \
    else                                                                                                     \
        hipLaunchKernelGGL((bwd_preprocess_chunks_kernel<T, CHN, int64_t>), grid, block, 0, stream, a);
        switch (ch) {
        case 1: FB_PRE(1) break;
        case 2: FB_PRE(2) break;
        case 4: FB_PRE(4) break;
        case 8: FB_PRE(8) break;
        default: FB_PRE(16) break;
        }
#undef FB_PRE
        return;
    }
    int64_t blocks = (rows + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(bwd_preprocess_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
}

// out[j] = sum over b of full[b * sb + j], j < n (a multiple of 8), fp32 accumulation in a fixed
// order: every thread adds the rows b = lane, lane + 32, ... of its 8 columns, then the 32 partial
// sums of a column are added in lane order.  One workgroup owns 64 consecutive columns (128 bytes
// of every row: whole cache lines) and streams down all rows, 32 rows per pass.
template <class T, bool OUT_F32>
__global__ __launch_bounds__(256) void sum_over_batch_kernel(const uint16_t *full, void *out, int64_t B, int64_t n, int64_t sb) {
    __shared__ float part[32][65]; // (65: the column sums below walk down a column of this array)
    const int cg = threadIdx.x & 7, rl = threadIdx.x >> 3;
    const int64_t col = (int64_t)blockIdx.x * 64 + cg * 8;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (col < n) {
        const uint16_t *p = full + col;
#pragma unroll 4
        for (int64_t b = rl; b < B; b += 32) {
            const u32x4_t x = *reinterpret_cast<const u32x4_t *>(p + b * sb);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                acc[2 * e] += T::to_float((uint16_t)(x[e] & 0xffffu));
                acc[2 * e + 1] += T::to_float((uint16_t)(x[e] >> 16));
            }
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) part[rl][cg * 8 + e] = acc[e];
    __syncthreads();
    if (threadIdx.x < 64) {
        const int64_t j = (int64_t)blockIdx.x * 64 + threadIdx.x;
        float s = 0.f;
#pragma unroll
        for (int r = 0; r < 32; ++r) s += part[r][threadIdx.x];
        if (j < n) {
            if (OUT_F32)
                static_cast<float *>(out)[j] = s;
            else
                static_cast<uint16_t *>(out)[j] = T::from_float(s);
        }
    }
}

hipError_t launch_sum_over_batch(const void *full, void *out, bool bf16, bool out_f32, int64_t B, int64_t n, int64_t sb,
                                 hipStream_t stream) {
    (void)hipGetLastError();
    const dim3 grid((unsigned)((n + 63) / 64)), block(256);
    const uint16_t *in = static_cast<const uint16_t *>(full);
    if (bf16) {
        if (out_f32) hipLaunchKernelGGL((sum_over_batch_kernel<BF16, true>), grid, block, 0, stream, in, out, B, n, sb);
        else hipLaunchKernelGGL((sum_over_batch_kernel<BF16, false>), grid, block, 0, stream, in, out, B, n, sb);
    } else {
        if (out_f32) hipLaunchKernelGGL((sum_over_batch_kernel<F16, true>), grid, block, 0, stream, in, out, B, n, sb);
        else hipLaunchKernelGGL((sum_over_batch_kernel<F16, false>), grid, block, 0, stream, in, out, B, n, sb);
    }
    return hipGetLastError();
}

// out[row][c] = c < min(r_in, r_out) ? in[row][c] : 0 for contiguous rows of 16-bit elements: one thread per row.
__global__ __launch_bounds__(256) void resize_rank_kernel(const uint16_t *in, uint16_t *out, int64_t rows, int r_in, int r_out) {
    const int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (row >= rows) return;
    const uint16_t *src = in + row * r_in;
    uint16_t *dst = out + row * r_out;
    const int keep = r_in < r_out ? r_in : r_out;
    if (r_out % 8 == 0 && keep <= 8 && reinterpret_cast<uintptr_t>(out) % 16 == 0) {
        // the usual case (a rank below 8 padded to 8 or 16): the row leaves as 16-byte stores
        uint16_t x[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) x[c] = c < keep ? src[c] : (uint16_t)0;
        u32x4_t first;
#pragma unroll
        for (int e = 0; e < 4; ++e) first[e] = (uint32_t)x[2 * e] | ((uint32_t)x[2 * e + 1] << 16);
        *reinterpret_cast<u32x4_t *>(dst) = first;
        for (int c = 8; c < r_out; c += 8) *reinterpret_cast<u32x4_t *>(dst + c) = u32x4_t{0u, 0u, 0u, 0u};
        return;
    }
    for (int c = 0; c < r_out; ++c) dst[c] = c < keep ? src[c] : (uint16_t)0;
}

hipError_t launch_resize_rank(const void *in, void *out, int64_t rows, int r_in, int r_out, hipStream_t stream) {
    (void)hipGetLastError();
    hipLaunchKernelGGL(resize_rank_kernel, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, stream,
                       static_cast<const uint16_t *>(in), static_cast<uint16_t *>(out), rows, r_in, r_out);
    return hipGetLastError();
}

hipError_t launch_bwd_preprocess(const BwdArgs &a, bool bf16, hipStream_t stream) {
    (void)hipGetLastError(); // (an earlier, unrelated error of the process is not this launch's)
    if (bf16)
        launch_preprocess_t<BF16>(a, stream);
    else
        launch_preprocess_t<F16>(a, stream);
    return hipGetLastError();
}

} // namespace fb
