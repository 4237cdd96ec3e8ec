// Argument checks and size queries of the C ABI (declared in include/flashbias.h): plain C++, no
// HIP call and no GPU involved, so that they can be unit-tested anywhere and built under
// AddressSanitizer / UBSan (`make sanitize`).  The entry points that launch kernels are in fb_api.hip.
#include <cmath>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "fb_checks.h"
#include "flashbias.h"

namespace {

thread_local char g_err[256] = "";

int fail(int code, const char *fmt, const char *what = "") {
    std::snprintf(g_err, sizeof(g_err), fmt, what);
    return code;
}

// input: may broadcast over batch / head (stride 0), never negative strides; a sequence stride
// smaller than a row (other than 0) would make rows overlap, which no caller of the operator means
int check_in(const fb_tensor &t, int channels, int L, const char *name) {
    if (!t.ptr) return fail(FB_ERR_NULL, "%s: null pointer", name);
    if (t.stride_b < 0 || t.stride_h < 0 || t.stride_s < 0) return fail(FB_ERR_STRIDE, "%s: negative stride", name);
    if (L > 1 && t.stride_s != 0 && t.stride_s < channels)
        return fail(FB_ERR_STRIDE, "%s: sequence stride smaller than a row", name);
    return FB_OK;
}

// output: rows must not alias each other
int check_out(const fb_tensor &t, int channels, int B, int H, int L, const char *name) {
    if (!t.ptr) return fail(FB_ERR_NULL, "%s: null pointer", name);
    if (t.stride_b < 0 || t.stride_h < 0 || t.stride_s < 0) return fail(FB_ERR_STRIDE, "%s: negative stride", name);
    if ((L > 1 && t.stride_s < channels) || (B > 1 && t.stride_b == 0) || (H > 1 && t.stride_h == 0))
        return fail(FB_ERR_STRIDE, "%s: output rows alias (zero or too small stride)", name);
    return FB_OK;
}

} // namespace

namespace fb {

int api_fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

void api_clear_error() { g_err[0] = 0; }

} // namespace fb

extern "C" {

int fb_version(void) { return FB_VERSION; }

const char *fb_last_error(void) { return g_err; }

size_t fb_bwd_workspace_bytes(const fb_params *p) {
    if (!p || p->B <= 0 || p->H <= 0 || p->Lq <= 0) return 0;
    return fb::bwd_scratch_bytes((int64_t)p->B * p->H * p->Lq);
}

int fb_suggest_bias_grad_group(const fb_params *p) {
    if (!p || p->r <= 0 || p->B < 32 || p->H <= 0 || p->Lq <= 0 || p->Lk <= 0) return 1;
    if (p->q_bias.stride_b != 0 || p->k_bias.stride_b != 0) return 1;
    // sequences of 1024 and more run kernels that keep one batch entry per workgroup
    if (p->Lq >= 1024 || p->Lk >= 1024) return 1;
    const int64_t lmin = p->Lq < p->Lk ? p->Lq : p->Lk;
    // (measured on 4096 x 16 windows of 256 tokens: backward + reduction 5.34 ms ungrouped, 5.13 / 4.93 / 4.84 /
    // 4.89 / 5.01 ms with groups of 2 / 4 / 8 / 16 / 32; 768 rows x 4 heads of 768 tokens, rank 32: 1.76 ungrouped,
    // 1.68 / 1.64 / 1.66 / 1.79 with 2 / 4 / 8 / 16; 1024 x 8 windows of 256: 0.735, 0.689 / 0.668 / 0.657 / 0.669:
    // the largest group that leaves two 256-row workgroups per workgroup slot of the chip)
    // Whole sequences of at most 256 positions at head dim 32 run one workgroup per (batch, head) pair, which fills a
    // compute unit by itself and pays for every start with an LDS clear and a first window whose loads nothing
    // overlaps (about 4.6 us: 4096 x 16 windows 5.33 ms ungrouped, 4.29 in groups of 8): groups of up to 32 there,
    // as long as four workgroups per compute unit remain.
    const bool window = p->d == 32 && p->r % 8 == 0 && p->r <= 32 && p->Lq <= 256 && p->Lk <= 256 && !p->causal && p->mask_type == 0;
    for (int g = window ? 32 : 8; g > 1; g /= 2)
        if (((int64_t)p->B + g - 1) / g * p->H * ((lmin + 255) / 256) >= 1024) return g;
    return 1;
}

int fb_check(const fb_params *p, int pass) {
    g_err[0] = 0;
    if (!p) return fail(FB_ERR_NULL, "params: null pointer");
    if (p->size != sizeof(fb_params)) return fail(FB_ERR_ABI, "fb_params.size does not match this library");
    if (p->dtype != FB_F16 && p->dtype != FB_BF16) return fail(FB_ERR_DTYPE, "only fp16 and bf16 are supported");
    if (p->B <= 0 || p->H <= 0 || p->Lq <= 0 || p->Lk <= 0) return fail(FB_ERR_SHAPE, "B, H, Lq, Lk must be positive");
    if (p->d <= 0 || p->d > FB_MAX_HEADDIM) return fail(FB_ERR_SHAPE, "head dim must be in 1..128");
    if (p->r < 0 || p->r > FB_MAX_RANK) return fail(FB_ERR_SHAPE, "bias rank must be in 0..128");
    if (!std::isfinite(p->scale) || p->scale == 0.f) return fail(FB_ERR_SCALE, "softmax scale must be finite and non-zero");
    {   // every kernel's grid is B * H * (tiles of at least 32 rows) workgroups in one dimension
        const int64_t lmax = p->Lq > p->Lk ? p->Lq : p->Lk;
        if ((int64_t)p->B * p->H * ((lmax + 31) / 32) > 0x7fffffffLL)
            return fail(FB_ERR_SHAPE, "B * H * ceil(L / 32) exceeds the grid limit of 2^31 - 1 workgroups");
    }
    int rc;
    if ((rc = check_in(p->q, p->d, p->Lq, "q"))) return rc;
    if ((rc = check_in(p->k, p->d, p->Lk, "k"))) return rc;
    if ((rc = check_in(p->v, p->d, p->Lk, "v"))) return rc;
    if (p->r > 0) {
        if ((rc = check_in(p->q_bias, p->r, p->Lq, "q_bias"))) return rc;
        if ((rc = check_in(p->k_bias, p->r, p->Lk, "k_bias"))) return rc;
    }
    if (p->mask_type != FB_MASK_NONE) {
        if (p->mask_type != FB_MASK_VECTOR && p->mask_type != FB_MASK_MATRIX)
            return fail(FB_ERR_MASK, "mask_type must be none, vector or matrix");
        if (p->mask_dtype != p->dtype && p->mask_dtype != FB_F32)
            return fail(FB_ERR_MASK, "mask must have the input dtype or fp32");
        if (!p->mask.ptr) return fail(FB_ERR_NULL, "%s: null pointer", "mask");
        if (p->mask.stride_b < 0 || p->mask.stride_h < 0 || p->mask.stride_s < 0)
            return fail(FB_ERR_STRIDE, "%s: negative stride", "mask");
    }
    if (!p->lse) return fail(FB_ERR_NULL, "%s: null pointer", "lse");
    if (pass == 0) return check_out(p->o, p->d, p->B, p->H, p->Lq, "o");
    if ((rc = check_in(p->o, p->d, p->Lq, "o"))) return rc;
    if ((rc = check_in(p->dout, p->d, p->Lq, "dout"))) return rc;
    if ((rc = check_out(p->dq, p->d, p->B, p->H, p->Lq, "dq"))) return rc;
    if ((rc = check_out(p->dk, p->d, p->B, p->H, p->Lk, "dk"))) return rc;
    if ((rc = check_out(p->dv, p->d, p->B, p->H, p->Lk, "dv"))) return rc;
    if (p->bias_grad_group < 0) return fail(FB_ERR_SHAPE, "bias_grad_group must not be negative");
    if (p->r > 0) {
        // with groups of g batch entries the factor gradients have ceil(B / g) batch rows
        const int g = p->bias_grad_group > 1 ? p->bias_grad_group : 1;
        const int rows = (int)(((int64_t)p->B + g - 1) / g);
        // both pointers null: the caller does not want the factor gradients (constant factors)
        if (p->dq_bias.ptr || p->dk_bias.ptr) {
            if ((rc = check_out(p->dq_bias, p->r, rows, p->H, p->Lq, "dq_bias"))) return rc;
            if ((rc = check_out(p->dk_bias, p->r, rows, p->H, p->Lk, "dk_bias"))) return rc;
        }
    }
    if (!p->delta) return fail(FB_ERR_NULL, "%s: null pointer", "delta");
    if (reinterpret_cast<uintptr_t>(p->delta) % 16 != 0) return fail(FB_ERR_STRIDE, "%s: must be 16-byte aligned", "delta");
    return FB_OK;
}

} // extern "C"
