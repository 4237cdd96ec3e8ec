// One launch for both halves of the backward on small grids: the streamlined dq and dk/dv
// workgroups (fb_bwd_dq_lean.h, fb_bwd_dkv_lean.h) side by side.
//
// Each of the two kernels keeps one (batch, head, 128-row tile) per workgroup, so a problem of
// B H ceil(L / 128) <= 256 tiles (the B2 H4 benchmark family up to L = 4096) gives every SIMD of an
// MI355X a single wave per launch, and a lone wave leaves the matrix and vector pipes idle about
// half of the time.  Neither kernel depends on the other once the per-query statistics exist, so
// after the preprocess step one grid can hold both: workgroups of the two kinds alternate in
// blocks of eight ids (one per XCD, which keeps the XCD-wise numbering each kind uses for L2
// locality), every compute unit gets one of each, and every SIMD two waves with different
// instruction mixes.  Results are those of the separate launches, bit for bit: the bodies are the
// same code, and every output element is still written by exactly one workgroup.
#define FB_BODIES_ONLY
#include "fb_bwd_dq.hip"
#include "fb_bwd_dkv.hip"

namespace fb {

template <class T, int NKR, bool BG>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void bwd_both_lean_kernel(const BwdArgs a) {
    const void *kernargs = (const void *)__builtin_amdgcn_kernarg_segment_ptr();
    const int ndq = a.ntiles_m * a.B * a.H, ndkv = a.ntiles_n * a.B * a.H;
    // both counts are multiples of 8 here (the launcher checks), so whole blocks of eight alternate
    const int paired = min(ndq, ndkv);
    const int id = blockIdx.x;
    bool is_dq;
    int wg;
    if (id < 2 * paired) {
        is_dq = ((id >> 3) & 1) == 0;
        wg = (id >> 4) * 8 + (id & 7);
    } else { // what the longer kind has left
        is_dq = ndq > ndkv;
        wg = id - paired;
    }
    if (is_dq)
        bwd_dq_lean_body<T, DqLeanCfg<T, NKR, BG>>(a, wg, kernargs);
    else
        bwd_dkv_lean_body<T, DkvLeanCfg<T, NKR, BG>>(a, wg, kernargs);
}

template <class T, int NKR, bool BG = true>
static hipError_t launch_both_lean(const BwdArgs &a0, hipStream_t stream) {
    typedef DqLeanCfg<T, NKR, BG> Cq;
    typedef DkvLeanCfg<T, NKR, BG> Ck;
    BwdArgs a = a0;
    a.ntiles_m = (a.Lq + Cq::BM - 1) / Cq::BM;
    a.ntiles_n = (a.Lk + Ck::BN - 1) / Ck::BN;
    constexpr int lds = Cq::LDS_BYTES > Ck::LDS_BYTES ? Cq::LDS_BYTES : Ck::LDS_BYTES;
    auto kern = bwd_both_lean_kernel<T, NKR, BG>;
    static KernelOnce once;
    const hipError_t e = allow_lds(kern, lds, once);
    if (e != hipSuccess) return e;
    const int64_t total = ((int64_t)a.ntiles_m + a.ntiles_n) * a.B * a.H;
    return launch_flat(kern, total, 256, lds, stream, a);
}

// Compiled once per element type for head dim 32 (see Makefile).  When fb_bwd takes this path is decided by
// mixed_backward() in fb_kernels.h.
#define FB_CAT2(a, b) a##b
#define FB_CAT(a, b) FB_CAT2(a, b)
hipError_t FB_CAT(launch_bwd_both_, FB_SUFFIX)(const BwdArgs &a, hipStream_t stream) {
    if (a.r == 0) return launch_both_lean<FB_T, 0>(a, stream);
    return a.dqb.ptr ? launch_both_lean<FB_T, 1>(a, stream) : launch_both_lean<FB_T, 1, false>(a, stream);
}

} // namespace fb
