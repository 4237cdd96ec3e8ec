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
    a.slots = slots_per_cu(kern, 256, lds, total, once);
    return launch_flat(kern, total, 256, lds, stream, a);
}

// The same for the general kernels of head dim 32 with factors of rank 8 ... 32 (aligned, unmasked, 128-row
// workgroups of one block per wave: fb_bwd_dq.hip, fb_bwd_dkv.hip), where the grid is small in another way: under
// a causal mask a launch lasts at least as long as its longest workgroup, which at a few hundred workgroups per
// kind is about twice what the work would need (B1 H50 L=2048: 800 workgroups of 1 to 16 tiles on 768 slots), and
// the two kinds in one launch fill each other's tails.  The ids alternate as above, which keeps each kind's own
// order (longest first within every XCD's share, work_order in fb_order.h).
template <class T, int NKR, bool FOLD, bool BG>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void bwd_both_kernel(const BwdArgs a) {
    typedef DqCfg<T, 2, NKR, true, false, false, FOLD, false, BG> Cq;
    typedef DkvCfg<T, 2, NKR, 1, true, false, 0, FOLD, BG> Ck;
    const int group = a.group > 1 ? a.group : 1;
    const int nbg = (a.B + group - 1) / group;
    const int ndq = a.ntiles_m * nbg * a.H, ndkv = a.ntiles_n * nbg * a.H;
    const int paired = min(ndq, ndkv); // (both counts are multiples of 8: the launcher checks)
    const int id = blockIdx.x;
    if (id < 2 * paired ? ((id >> 3) & 1) == 0 : ndq > ndkv)
        bwd_dq_body<T, Cq>(a, id < 2 * paired ? (id >> 4) * 8 + (id & 7) : id - paired);
    else
        bwd_dkv_body<T, Ck>(a, id < 2 * paired ? (id >> 4) * 8 + (id & 7) : id - paired);
}

template <class T, int NKR, bool FOLD, bool BG>
static hipError_t launch_both_general(const BwdArgs &a0, hipStream_t stream) {
    typedef DqCfg<T, 2, NKR, true, false, false, FOLD, false, BG> Cq;
    typedef DkvCfg<T, 2, NKR, 1, true, false, 0, FOLD, BG> Ck;
    static_assert(Cq::NTHREADS == 256 && Ck::NTHREADS == 256 && Cq::BM == 128 && Ck::BN == 128, "128-row workgroups of four waves");
    BwdArgs a = a0;
    a.ntiles_m = (a.Lq + Cq::BM - 1) / Cq::BM;
    a.ntiles_n = (a.Lk + Ck::BN - 1) / Ck::BN;
    constexpr int lds = Cq::LDS_BYTES > Ck::LDS_BYTES ? Cq::LDS_BYTES : Ck::LDS_BYTES;
    auto kern = bwd_both_kernel<T, NKR, FOLD, BG>;
    static KernelOnce once;
    const hipError_t e = allow_lds(kern, lds, once);
    if (e != hipSuccess) return e;
    const int group = a.group > 1 ? a.group : 1;
    const int64_t total = ((int64_t)a.ntiles_m + a.ntiles_n) * ((a.B + group - 1) / group) * a.H;
    a.slots = slots_per_cu(kern, 256, lds, total, once);
    return launch_flat(kern, total, 256, lds, stream, a);
}

template <class T, int NKR>
static hipError_t launch_both_general_r(const BwdArgs &a, hipStream_t stream) {
    const bool bg = a.dqb.ptr != nullptr;
    if (fold_scale_ok<T>(a.scale, a.r, a.Lk)) // (mixed_general_backward() made sure that both kinds agree on this)
        return bg ? launch_both_general<T, NKR, true, true>(a, stream) : launch_both_general<T, NKR, true, false>(a, stream);
    return bg ? launch_both_general<T, NKR, false, true>(a, stream) : launch_both_general<T, NKR, false, false>(a, stream);
}

// Compiled once per element type for head dim 32 (see Makefile).  When fb_bwd takes these paths is decided by
// mixed_backward() and mixed_general_backward() in fb_kernels.h.
#define FB_CAT2(a, b) a##b
#define FB_CAT(a, b) FB_CAT2(a, b)
hipError_t FB_CAT(launch_bwd_both_, FB_SUFFIX)(const BwdArgs &a, hipStream_t stream) {
    if (a.r == 0) return launch_both_lean<FB_T, 0>(a, stream);
    return a.dqb.ptr ? launch_both_lean<FB_T, 1>(a, stream) : launch_both_lean<FB_T, 1, false>(a, stream);
}
hipError_t FB_CAT(launch_bwd_both_general_, FB_SUFFIX)(const BwdArgs &a, hipStream_t stream) {
    return nkr_of(a.r) == 1 ? launch_both_general_r<FB_T, 1>(a, stream) : launch_both_general_r<FB_T, 2>(a, stream);
}

} // namespace fb
