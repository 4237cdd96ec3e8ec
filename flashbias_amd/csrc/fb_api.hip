// C ABI of the library (declared in include/flashbias.h): translation of fb_params into kernel
// argument blocks and dispatch to the instantiation that covers (dtype, head dim, rank).  The
// argument checks themselves (fb_check) are plain C++ in fb_checks.cpp.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "flashbias.h"
#include "fb_checks.h"
#include "fb_kernels.h"

namespace fb {
#define FB_DECL(sfx)                                                          \
    hipError_t launch_fwd_##sfx(const FwdArgs &a, hipStream_t stream);        \
    hipError_t launch_bwd_dkv_##sfx(const BwdArgs &a, hipStream_t stream);    \
    hipError_t launch_bwd_dq_##sfx(const BwdArgs &a, hipStream_t stream);
FB_DECL(bf16_1) FB_DECL(bf16_2) FB_DECL(bf16_4) FB_DECL(bf16_8)
FB_DECL(f16_1) FB_DECL(f16_2) FB_DECL(f16_4) FB_DECL(f16_8)
#undef FB_DECL
hipError_t launch_bwd_both_bf16_2(const BwdArgs &a, hipStream_t stream);
hipError_t launch_bwd_both_f16_2(const BwdArgs &a, hipStream_t stream);
hipError_t launch_bwd_both_general_bf16_2(const BwdArgs &a, hipStream_t stream);
hipError_t launch_bwd_both_general_f16_2(const BwdArgs &a, hipStream_t stream);
hipError_t launch_bwd_win_bf16_2(const BwdArgs &a, hipStream_t stream);
hipError_t launch_bwd_win_f16_2(const BwdArgs &a, hipStream_t stream);

hipError_t launch_fwd(const FwdArgs &a, bool bf16, hipStream_t stream) {
    switch (nkd_of(a.d)) {
    case 1: return bf16 ? launch_fwd_bf16_1(a, stream) : launch_fwd_f16_1(a, stream);
    case 2: return bf16 ? launch_fwd_bf16_2(a, stream) : launch_fwd_f16_2(a, stream);
    case 4: return bf16 ? launch_fwd_bf16_4(a, stream) : launch_fwd_f16_4(a, stream);
    default: return bf16 ? launch_fwd_bf16_8(a, stream) : launch_fwd_f16_8(a, stream);
    }
}

hipError_t launch_bwd_dkv(const BwdArgs &a, bool bf16, hipStream_t stream) {
    switch (nkd_of(a.d)) {
    case 1: return bf16 ? launch_bwd_dkv_bf16_1(a, stream) : launch_bwd_dkv_f16_1(a, stream);
    case 2: return bf16 ? launch_bwd_dkv_bf16_2(a, stream) : launch_bwd_dkv_f16_2(a, stream);
    case 4: return bf16 ? launch_bwd_dkv_bf16_4(a, stream) : launch_bwd_dkv_f16_4(a, stream);
    default: return bf16 ? launch_bwd_dkv_bf16_8(a, stream) : launch_bwd_dkv_f16_8(a, stream);
    }
}

hipError_t launch_bwd_dq(const BwdArgs &a, bool bf16, hipStream_t stream) {
    switch (nkd_of(a.d)) {
    case 1: return bf16 ? launch_bwd_dq_bf16_1(a, stream) : launch_bwd_dq_f16_1(a, stream);
    case 2: return bf16 ? launch_bwd_dq_bf16_2(a, stream) : launch_bwd_dq_f16_2(a, stream);
    case 4: return bf16 ? launch_bwd_dq_bf16_4(a, stream) : launch_bwd_dq_f16_4(a, stream);
    default: return bf16 ? launch_bwd_dq_bf16_8(a, stream) : launch_bwd_dq_f16_8(a, stream);
    }
}
// dq and dk/dv workgroups of the streamlined kernels in one launch (fb_bwd_both.hip; head dim 32)
hipError_t launch_bwd_both(const BwdArgs &a, bool bf16, hipStream_t stream) {
    return bf16 ? launch_bwd_both_bf16_2(a, stream) : launch_bwd_both_f16_2(a, stream);
}
// the same for the general kernels with factors of rank 8 ... 32
hipError_t launch_bwd_both_general(const BwdArgs &a, bool bf16, hipStream_t stream) {
    return bf16 ? launch_bwd_both_general_bf16_2(a, stream) : launch_bwd_both_general_f16_2(a, stream);
}
// all five gradients of a short sequence in one workgroup (fb_bwd_win.hip; head dim 32)
hipError_t launch_bwd_win(const BwdArgs &a, bool bf16, hipStream_t stream) {
    return bf16 ? launch_bwd_win_bf16_2(a, stream) : launch_bwd_win_f16_2(a, stream);
}
} // namespace fb

// Scratch of fb_bwd_static: device memory that belongs to the library image, so that the entry
// point never calls an allocator.  One copy per GPU that loads the library; it keeps the last
// call's contents (the backward overwrites every element it later reads, nothing has to start
// at zero).  In host code the array's name is only a handle for hipGetSymbolAddress: the kernels
// get the address that call returns.
static __device__ __align__(256) unsigned char scratch[FB_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {nullptr}; // address of `scratch` on each device, looked up once

// Address of this device's copy of the scratch array (looked up on first use with the device
// current), or nullptr with *err set.
void *static_scratch(hipError_t *err) {
    int dev = 0;
    *err = hipGetDevice(&dev);
    if (*err != hipSuccess) return nullptr;
    if (dev < 0 || dev >= kMaxDevices) {
        *err = hipErrorInvalidDevice;
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        *err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (*err != hipSuccess) return nullptr;
        g_scratch_ptr[dev] = ptr;
    }
    return g_scratch_ptr[dev];
}

bool vec_ok(const fb_tensor &t) {
    return (reinterpret_cast<uintptr_t>(t.ptr) % 16 == 0) && t.stride_b % 8 == 0 && t.stride_h % 8 == 0 &&
           t.stride_s % 8 == 0;
}

fb::Tensor dev(const fb_tensor &t) {
    fb::Tensor o;
    o.ptr = static_cast<const uint16_t *>(t.ptr);
    o.sb = t.stride_b;
    o.sh = t.stride_h;
    o.ss = t.stride_s;
    o.vec_ok = vec_ok(t) ? 1 : 0;
    return o;
}

fb::MaskDesc dev_mask(const fb_params *p) {
    fb::MaskDesc m;
    m.ptr = p->mask_type ? p->mask.ptr : nullptr;
    m.sb = p->mask.stride_b;
    m.sh = p->mask.stride_h;
    m.sm = p->mask_type == FB_MASK_MATRIX ? p->mask.stride_s : 0;
    m.type = p->mask_type;
    m.is_f32 = p->mask_dtype == FB_F32;
    const uintptr_t align = m.is_f32 ? 16 : 8; // four consecutive keys
    m.vec_ok = p->mask_type && reinterpret_cast<uintptr_t>(m.ptr) % align == 0 && m.sb % 4 == 0 && m.sh % 4 == 0 &&
               m.sm % 4 == 0;
    return m;
}

fb::FwdArgs fwd_args(const fb_params *p) {
    fb::FwdArgs a;
    std::memset(&a, 0, sizeof(a));
    a.q = dev(p->q);
    a.k = dev(p->k);
    a.v = dev(p->v);
    a.o = dev(p->o);
    if (p->r > 0) {
        a.qb = dev(p->q_bias);
        a.kb = dev(p->k_bias);
    }
    a.mask = dev_mask(p);
    a.lse = p->lse;
    a.B = p->B; a.H = p->H; a.Lq = p->Lq; a.Lk = p->Lk; a.d = p->d; a.r = p->r;
    a.causal = p->causal ? 1 : 0;
    a.scale = p->scale;
    return a;
}

fb::BwdArgs bwd_args(const fb_params *p) {
    fb::BwdArgs a;
    std::memset(&a, 0, sizeof(a));
    a.q = dev(p->q);
    a.k = dev(p->k);
    a.v = dev(p->v);
    a.o = dev(p->o);
    a.dout = dev(p->dout);
    a.dq = dev(p->dq);
    a.dk = dev(p->dk);
    a.dv = dev(p->dv);
    if (p->r > 0) {
        a.qb = dev(p->q_bias);
        a.kb = dev(p->k_bias);
        a.dqb = dev(p->dq_bias);
        a.dkb = dev(p->dk_bias);
    }
    a.mask = dev_mask(p);
    a.lse = p->lse;
    a.delta = p->delta;
    a.B = p->B; a.H = p->H; a.Lq = p->Lq; a.Lk = p->Lk; a.d = p->d; a.r = p->r;
    a.causal = p->causal ? 1 : 0;
    a.scale = p->scale;
    a.group = p->r > 0 && p->bias_grad_group > 1 ? p->bias_grad_group : 1;
    a.stat_chunks = fb::dkv_streamlined(a) ? 1 : 0;
    return a;
}

int launched(hipError_t e, const char *what) {
    if (e == hipSuccess) return FB_OK;
    return fb::api_fail(FB_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
}

} // namespace

extern "C" {

int fb_init(void) {
    fb::api_clear_error();
    hipError_t e = hipSuccess;
    if (!static_scratch(&e)) return launched(e, "fb_init (hipGetSymbolAddress)");
    return FB_OK;
}

int fb_fwd(const fb_params *p, void *stream) {
    const int rc = fb_check(p, 0);
    if (rc) return rc;
    return launched(fb::launch_fwd(fwd_args(p), p->dtype == FB_BF16, static_cast<hipStream_t>(stream)), "fb_fwd");
}

int fb_bwd_preprocess(const fb_params *p, void *stream) {
    const int rc = fb_check(p, 1);
    if (rc) return rc;
    return launched(fb::launch_bwd_preprocess(bwd_args(p), p->dtype == FB_BF16, static_cast<hipStream_t>(stream)),
                    "fb_bwd_preprocess");
}

int fb_bwd_dkv(const fb_params *p, void *stream) {
    const int rc = fb_check(p, 1);
    if (rc) return rc;
    return launched(fb::launch_bwd_dkv(bwd_args(p), p->dtype == FB_BF16, static_cast<hipStream_t>(stream)),
                    "fb_bwd_dkv");
}

int fb_bwd_dq(const fb_params *p, void *stream) {
    const int rc = fb_check(p, 1);
    if (rc) return rc;
    return launched(fb::launch_bwd_dq(bwd_args(p), p->dtype == FB_BF16, static_cast<hipStream_t>(stream)),
                    "fb_bwd_dq");
}

int fb_sum_over_batch(const void *full, void *out, int dtype, int out_dtype, int64_t B, int64_t n, int64_t batch_stride,
                      void *stream) {
    fb::api_clear_error();
    if (!full || !out) return fb::api_fail(FB_ERR_NULL, "fb_sum_over_batch: null pointer");
    if (dtype != FB_F16 && dtype != FB_BF16) return fb::api_fail(FB_ERR_DTYPE, "only fp16 and bf16 are supported");
    if (out_dtype != dtype && out_dtype != FB_F32) return fb::api_fail(FB_ERR_DTYPE, "output must have the input dtype or fp32");
    if (B <= 0 || n <= 0 || (n + 63) / 64 > 0x7fffffff) return fb::api_fail(FB_ERR_SHAPE, "B and n must be positive (n below 2^37)");
    if (n % 8 != 0 || batch_stride % 8 != 0 || batch_stride < n || reinterpret_cast<uintptr_t>(full) % 16 != 0)
        return fb::api_fail(FB_ERR_STRIDE, "fb_sum_over_batch: rows must be 16-byte aligned multiples of 8 elements that do not overlap");
    return launched(fb::launch_sum_over_batch(full, out, dtype == FB_BF16, out_dtype == FB_F32, B, n, batch_stride,
                                              static_cast<hipStream_t>(stream)),
                    "fb_sum_over_batch");
}

int fb_resize_rank(const void *in, void *out, int64_t rows, int r_in, int r_out, void *stream) {
    fb::api_clear_error();
    if (!in || !out) return fb::api_fail(FB_ERR_NULL, "fb_resize_rank: null pointer");
    if (rows <= 0 || r_in <= 0 || r_out <= 0 || r_in > 4096 || r_out > 4096 || (rows + 255) / 256 > 0x7fffffff)
        return fb::api_fail(FB_ERR_SHAPE, "fb_resize_rank: rows and both ranks must be positive (ranks up to 4096, rows below 2^39)");
    return launched(fb::launch_resize_rank(in, out, rows, r_in, r_out, static_cast<hipStream_t>(stream)), "fb_resize_rank");
}

int fb_bwd_static(const fb_params *p, void *stream) {
    // fb_bwd with the scratch buffer taken from the library's own static device array instead of
    // fb_params.delta (which is ignored): no allocation, here or in anything it calls.
    fb::api_clear_error();
    if (!p) return fb::api_fail(FB_ERR_NULL, "params: null pointer");
    if (p->size != sizeof(fb_params)) return fb::api_fail(FB_ERR_ABI, "fb_params.size does not match this library");
    const size_t need = fb_bwd_workspace_bytes(p);
    if (need == 0) return fb::api_fail(FB_ERR_SHAPE, "B, H, Lq, Lk must be positive");
    if (need > (size_t)FB_STATIC_SCRATCH_BYTES)
        return fb::api_fail(FB_ERR_SHAPE, "fb_bwd_static: B * H * Lq exceeds the static scratch buffer (FB_STATIC_SCRATCH_BYTES); use fb_bwd");
    hipError_t e = hipSuccess;
    void *ptr = static_scratch(&e);
    if (!ptr) return launched(e, "fb_bwd_static (hipGetSymbolAddress)");
    fb_params q = *p;
    q.delta = static_cast<float *>(ptr);
    return fb_bwd(&q, stream);
}

int fb_bwd(const fb_params *p, void *stream) {
    // Two launches: the dq kernel computes delta for its own queries on the way (each query belongs
    // to exactly one of its workgroups) and leaves the statistics in the scratch buffer for the
    // dk/dv kernel.  The three phases above stay callable one by one.
    const int rc = fb_check(p, 1);
    if (rc) return rc;
    fb::BwdArgs a = bwd_args(p);
    if (fb::window_backward(a)) // whole sequences of at most 256 positions: one workgroup per (batch, head), one launch
        return launched(fb::launch_bwd_win(a, p->dtype == FB_BF16, static_cast<hipStream_t>(stream)), "fb_bwd (window)");
    const bool general_mix = p->dtype == FB_BF16 ? fb::mixed_general_backward<fb::BF16>(a) : fb::mixed_general_backward<fb::F16>(a);
    if (fb::mixed_backward(a) || general_mix) {
        // small grids of the streamlined kernels: the preprocess step, then one launch that holds the dq and
        // the dk/dv workgroups side by side (same bits as the two launches)
        const int rc1 = launched(fb::launch_bwd_preprocess(a, p->dtype == FB_BF16, static_cast<hipStream_t>(stream)),
                                 "fb_bwd_preprocess");
        if (rc1) return rc1;
        return launched((general_mix ? fb::launch_bwd_both_general : fb::launch_bwd_both)(a, p->dtype == FB_BF16, static_cast<hipStream_t>(stream)),
                        "fb_bwd (dq + dk/dv)");
    }
    a.stats_here = 1;
    const int rc2 = launched(fb::launch_bwd_dq(a, p->dtype == FB_BF16, static_cast<hipStream_t>(stream)), "fb_bwd_dq");
    if (rc2) return rc2;
    a.stats_here = 0;
    return launched(fb::launch_bwd_dkv(a, p->dtype == FB_BF16, static_cast<hipStream_t>(stream)), "fb_bwd_dkv");
}

} // extern "C"
