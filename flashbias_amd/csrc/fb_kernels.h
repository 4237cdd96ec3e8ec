// Host-visible kernel argument blocks and launchers (implemented in fb_fwd.hip / fb_bwd.hip).
#pragma once
#include <atomic>

#include "fb_checks.h"
#include <cmath>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fb_device.h"

namespace fb {

struct FwdArgs {
    Tensor q, k, v, qb, kb, o;
    MaskDesc mask;
    float *lse; // (B, H, Lq)
    int B, H, Lq, Lk, d, r;
    int causal;
    float scale;
    int ntiles_m; // query tiles per (batch, head)
    int slots;    // workgroups of this launch that share a compute unit (priority turn-taking)
};

struct BwdArgs {
    Tensor q, k, v, qb, kb, o, dout;
    Tensor dq, dk, dv, dqb, dkb;
    MaskDesc mask;
    const float *lse; // (B, H, Lq)
    float *delta;     // scratch: -delta (B, H, Lq), lse * log2(e) (B, H, Lq), then one stat_chunk per query at stat_offset()
    int B, H, Lq, Lk, d, r;
    int causal;
    float scale;
    int ntiles_n; // key tiles per (batch, head), dk/dv kernel
    int ntiles_m; // query tiles per (batch, head), dq kernel
    int slots;    // workgroups of this launch that share a compute unit (priority turn-taking)
    int stats_here; // dq kernel: compute -delta and lse * log2(e) itself (and store them) instead of reading them
    int stat_chunks; // writers of the scratch buffer: also store the statistics chunks (dkv_streamlined())
    int group; // > 1: a workgroup serves this many consecutive batch entries and sums their factor gradients (row b / group)
    int walk;  // window backward without such sums: batch entries a workgroup walks (set by its launcher)
};

// Each returns hipSuccess or the launch error.  `bf16` selects the element type.
hipError_t launch_fwd(const FwdArgs &a, bool bf16, hipStream_t stream);
hipError_t launch_bwd_preprocess(const BwdArgs &a, bool bf16, hipStream_t stream);
hipError_t launch_bwd_dkv(const BwdArgs &a, bool bf16, hipStream_t stream);
hipError_t launch_bwd_dq(const BwdArgs &a, bool bf16, hipStream_t stream);
// out[j] = sum_b full[b * sb + j] for j < n; 16-bit elements in, the same type or fp32 out.
hipError_t launch_sum_over_batch(const void *full, void *out, bool bf16, bool out_f32, int64_t B, int64_t n, int64_t sb,
                                 hipStream_t stream);

// out[row][c] = c < min(r_in, r_out) ? in[row][c] : 0: contiguous rows of 16-bit elements.
hipError_t launch_resize_rank(const void *in, void *out, int64_t rows, int r_in, int r_out, hipStream_t stream);

// Compute units of the current device (cached per device; 256 on MI355X).  The launchers pick
// smaller query tiles when the larger ones would leave compute units without a workgroup.
inline int num_cus() {
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev].store(n, std::memory_order_relaxed); // (concurrent first calls store the same value)
    }
    return n;
}

// A grid that leaves the chip under-filled even at the general kernels' occupancy: fewer than two
// 128-row workgroups per compute unit.
inline bool small_grid(int B, int H, int L) { return (int64_t)B * H * ((L + 127) / 128) < 2 * (int64_t)num_cus(); }

// A short sequence whose last 256-row workgroup would be half empty (an odd number of 128-row
// blocks, at most three): 128-row workgroups waste nothing there.
inline bool half_empty_256(int L) { return L <= 384 && ((L + 127) / 128) % 2 == 1; }

// Whether the backward of a call runs the streamlined dk/dv kernel (fb_bwd_dkv_lean.h), which is
// also whether the writers of the scratch buffer (preprocess step, dq kernel) add the statistics
// chunks it reads: aligned tensors, no mask, head dim 32 exactly and rank 8 or none (its copies
// fill whole rows, there is no zero padding of the channels), row pitches that fit its 32-bit
// offsets.  With scale * log2(e) <= 1 the folded k cannot leave the 16-bit range; a folded k_b
// that does sends its workgroup to the general kernel.  And a loop long enough to pay for the
// kernel's six-stage pipeline: on grids that fill the chip the general kernel's three waves per SIMD
// hide a short loop's latencies better (4096 x 16 windows, general against streamlined: 2.61 against
// 3.09 ms at 256 queries, 2.05 against 2.18 at 512, 0.457 against 0.442 at 1024 with B64 H16); on
// small grids the streamlined kernel is ahead at every length measured (B2 H4 from L=1024).
inline bool dkv_streamlined(const BwdArgs &a) {
    const int64_t lim = (int64_t)1 << 24;
    return a.mask.type == 0 && a.d == 32 && (a.r == 8 || a.r == 0) && a.q.vec_ok && a.k.vec_ok && a.v.vec_ok && a.dout.vec_ok &&
           (a.r == 0 || (a.qb.vec_ok && a.kb.vec_ok && a.qb.ss < lim)) && a.q.ss < lim && a.dout.ss < lim &&
           a.scale > 1e-6f && a.scale * 1.4426950408889634f <= 1.f && (a.Lq >= 1024 || small_grid(a.B, a.H, a.Lk)) &&
           a.group <= 1; // (factor gradients summed over groups of batch entries: the general kernels do that)
}

// The same for the streamlined dq kernel (fb_bwd_dq_lean.h), which streams K, K_b and V (general
// against streamlined on grids that fill the chip: 2.10 against 2.86 ms at 4096 x 16 windows of 256
// keys, 1.61 against 1.84 at 512, 0.352 against 0.371 at 1024 with B64 H16, 0.150 against 0.117 at
// 2048 causal).
inline bool dq_streamlined(const BwdArgs &a) {
    const int64_t lim = (int64_t)1 << 24;
    return a.mask.type == 0 && a.d == 32 && (a.r == 8 || a.r == 0) && a.q.vec_ok && a.k.vec_ok && a.v.vec_ok && a.dout.vec_ok &&
           (a.r == 0 || (a.qb.vec_ok && a.kb.vec_ok && a.kb.ss < lim)) && a.k.ss < lim && a.v.ss < lim &&
           (!a.stats_here || a.o.vec_ok) && a.scale > 1e-6f && a.scale * 1.4426950408889634f <= 1.f &&
           (a.Lk >= 2048 || small_grid(a.B, a.H, a.Lq)) && a.group <= 1;
}

// Whether fb_bwd runs the preprocess step and then one launch that mixes the streamlined dq and dk/dv workgroups
// (fb_bwd_both.hip) instead of the dq and dk/dv launches: both streamlined kernels cover the call with the
// statistics read from the scratch buffer, neither kind alone has more than one workgroup per compute unit
// (measured at B2 H4, two launches against the mixed one: 0.035 / 0.021 ms at L=1024, 0.058 / 0.036 at 2048,
// 0.112 / 0.096 at 4096, and 0.330 / 0.340 at 8192, where every SIMD has its two waves anyway), and both
// kinds' workgroup counts split evenly over the eight XCDs (the mixed numbering alternates blocks of eight).
inline bool mixed_backward(const BwdArgs &a0) {
    BwdArgs a = a0;
    a.stats_here = 0;
    if (!(a.d == 32 && dq_streamlined(a) && dkv_streamlined(a))) return false;
    const int64_t ndq = (int64_t)a.B * a.H * ((a.Lq + 127) / 128), ndkv = (int64_t)a.B * a.H * ((a.Lk + 127) / 128);
    return ndq % 8 == 0 && ndkv % 8 == 0 && ndq <= num_cus() && ndkv <= num_cus();
}

// The same question for the general dq and dk/dv kernels of head dim 32 with factors (launch_both_general in
// fb_bwd_both.hip): both kernels would run their aligned, unmasked 128-row instantiations with the same folding of
// the scale, the counts of both kinds split evenly over the eight XCDs, and the grid is small: at most one
// workgroup per compute unit and kind, or, under a causal mask, at most one and a half per workgroup slot (three
// slots per compute unit), where a launch's length is that of its longest workgroup and the two kinds fill each
// other's tails.  Declared after fold_scale_ok below.
template <class T>
inline bool mixed_general_backward(const BwdArgs &a0);

// Whether fb_bwd runs the window kernel (fb_bwd_win.hip: one workgroup per (batch, head) forms the per-query
// statistics and all five gradients, dq summed inside the workgroup) instead of the dq and dk/dv launches: whole
// sequences of at most 256 positions, head dim 32, rank a multiple of 8 up to 32, aligned tensors, no additive or
// causal mask, and at least one workgroup per compute unit (a workgroup fills a compute unit by itself).  Such
// sequences are bound by memory traffic, and the two-kernel backward reads q, k, v, o and dO twice.
inline bool window_backward(const BwdArgs &a) {
    const int64_t lim = (int64_t)1 << 22; // (32-bit byte offsets of 256 tile rows)
    const int group = a.group > 1 ? a.group : 1;
    return a.mask.type == 0 && !a.causal && a.d == 32 && a.r % 8 == 0 && a.r <= 32 && a.Lq <= 256 && a.Lk <= 256 &&
           a.q.vec_ok && a.k.vec_ok && a.v.vec_ok && a.o.vec_ok && a.dout.vec_ok && (a.r == 0 || (a.qb.vec_ok && a.kb.vec_ok)) &&
           a.q.ss < lim && a.k.ss < lim && a.dout.ss < lim && (a.r == 0 || (a.qb.ss < lim && a.kb.ss < lim)) &&
           (int64_t)((a.B + group - 1) / group) * a.H >= num_cus();
}

// What a launcher remembers about one kernel instantiation (one static object per instantiation;
// the only mutable state of the library besides num_cus() and fb_bwd_static's scratch address:
// write-once values, atomics, so concurrent first calls from several threads are fine).
struct KernelOnce {
    std::atomic<int> lds_set{0};   // the dynamic-LDS limit of the kernel has been raised
    std::atomic<int> occupancy{0}; // workgroups per compute unit that registers and LDS admit
};

// Raises the kernel's dynamic LDS limit on its first launch if it needs more than the default 48 KB.
template <class K>
inline hipError_t allow_lds(K kern, size_t lds_bytes, KernelOnce &once) {
    if (lds_bytes <= 48 * 1024 || once.lds_set.load(std::memory_order_acquire)) return hipSuccess;
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                             (int)lds_bytes);
    if (e == hipSuccess) once.lds_set.store(1, std::memory_order_release);
    return e;
}

// One-dimensional launch; the error it returns is this launch's own (an error that some earlier,
// unrelated call of the process left behind is cleared first, not reported as ours).
template <class K, class A>
inline hipError_t launch_flat(K kern, int64_t total, int threads, size_t lds_bytes, hipStream_t stream, const A &args) {
    if (total <= 0 || total > 0x7fffffffLL) return hipErrorInvalidConfiguration; // (fb_check bounds the sizes)
    (void)hipGetLastError();
    hipLaunchKernelGGL(kern, dim3((unsigned)total), dim3(threads), lds_bytes, stream, args);
    return hipGetLastError();
}

// Workgroups of a launch of `total` workgroups that sit on one compute unit at a time: what the
// kernel's registers and LDS admit (queried once per kernel instantiation; *cache holds it), or
// fewer when the grid does not fill the chip that often.
template <class K>
inline int slots_per_cu(K kern, int threads, size_t lds_bytes, int64_t total, KernelOnce &once) {
    int occ = once.occupancy.load(std::memory_order_relaxed);
    if (occ == 0) {
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, kern, threads, lds_bytes) != hipSuccess || occ <= 0) occ = 1;
        once.occupancy.store(occ, std::memory_order_relaxed); // (concurrent first calls store the same value)
    }
    const int64_t cus = num_cus();
    const int64_t share = (total + cus - 1) / cus;
    return (int)(share < occ ? (share < 1 ? 1 : share) : occ);
}

// Padded sizes the dispatchers use: d is covered by 16-wide contraction steps of the
// QK^T product (NKD of them) and the rank by NKR more; both rounded up to the next
// instantiated size (1, 2, 4, 8 steps).
inline int steps_pow2(int n16) { return n16 <= 1 ? 1 : n16 <= 2 ? 2 : n16 <= 4 ? 4 : 8; }
inline int nkd_of(int d) { return steps_pow2((d + 15) / 16); }
inline int nkr_of(int r) { return r == 0 ? 0 : steps_pow2((r + 15) / 16); }

// Whether a kernel may compute scale * (q k^T + (q_b / scale) k_b^T) in one MFMA chain instead of
// scale * q k^T + q_b k_b^T (one FMA per score less) and still match the fp32 scaling of the
// reference: always without factors; with factors only for an element type with the exponent
// range of fp32 (the division cannot overflow) and either a power-of-two scale (the division is
// exact) or r <= 8 (the low-order half of q_b / scale travels in the unused half of the 16-wide
// MFMA step, which leaves a relative error of 2^-16 in the bias product).  `len` is the length
// of the loop a workgroup runs (keys in the forward and dq kernels, queries in dk/dv): dividing
// the resident factor costs about as much as the FMAs of 256 loop positions, so short loops keep
// the FMA.  A scale of exactly 1 (what the reference's Swin and AlphaFold3 blocks pass, having
// scaled q themselves: swin_transformer_v2.py:178-203, primitives.py:636-643) needs no division
// at all: folded for every element type and length, the factors used as they are.
template <class T>
inline bool fold_scale_ok(float scale, int r, int len) {
    if (!(scale > 1e-6f && scale < 1e6f)) return false; // (also false for NaN; keeps 1 / scale and scale * score well inside fp32)
    if (r == 0 || scale == 1.f) return true;
    if (!T::kWideRange || len < 512) return false;
    int e;
    return r <= 8 || std::frexp(scale, &e) == 0.5f;
}

template <class T>
inline bool mixed_general_backward(const BwdArgs &a0) {
    BwdArgs a = a0;
    a.stats_here = 0;
    const int64_t lim = (int64_t)1 << 24;
    if (!(a.d == 32 && a.r >= 8 && a.r <= 32 && a.r % 8 == 0 && a.mask.type == 0) || dq_streamlined(a) || dkv_streamlined(a)) return false;
    if (!(a.q.vec_ok && a.k.vec_ok && a.v.vec_ok && a.dout.vec_ok && a.qb.vec_ok && a.kb.vec_ok && a.q.ss < lim && a.k.ss < lim &&
          a.v.ss < lim && a.dout.ss < lim && a.qb.ss < lim && a.kb.ss < lim))
        return false;
    if (fold_scale_ok<T>(a.scale, a.r, a.Lk) != fold_scale_ok<T>(a.scale, a.r, a.Lq)) return false;
    const int group = a.group > 1 ? a.group : 1;
    const int64_t units = (int64_t)((a.B + group - 1) / group) * a.H;
    const int64_t ndq = units * ((a.Lq + 127) / 128), ndkv = units * ((a.Lk + 127) / 128);
    if (ndq % 8 != 0 || ndkv % 8 != 0) return false;
    const int64_t most = ndq > ndkv ? ndq : ndkv;
    return most <= num_cus() || (a.causal && 2 * most <= 9 * (int64_t)num_cus());
}

} // namespace fb
