// Forward FlashBias attention for gfx950:  o = softmax(scale q k^T + q_b k_b^T + mask) v, lse.
// Replaces _fwd_kernel of the reference (flash_bias/flash_bias_triton.py:62-355).
//
// One workgroup (4 waves) owns BM = 128 * QBLK consecutive queries of one (batch, head); each
// wave owns 32 * QBLK of them.  Keys are streamed in tiles of BN = 64 through double-buffered
// LDS.  Everything is computed transposed so that a lane owns one query:
//
//   S^T (keys x queries) = [K | K_b] [Q | Q_b]^T       A = key tile from LDS, B = query regs
//   O^T (d x queries)   += V^T P^T                     A = V^T tile from LDS, B = P^T regs
//
// In the C layout a lane holds one query column and 16 keys of it, so the row max / sum of
// the online softmax are in-lane reductions plus one exchange with lane ^ 32, the rescale
// factor is a per-lane scalar, and P^T is already in the B-operand layout of the second MFMA
// (no LDS round trip for P).  The contraction runs over the concatenated channels
// [d | r], zero-padded in LDS to 16-wide MFMA steps; the fp32 accumulator is multiplied by
// the softmax scale after the d steps and before the r steps, so the bias product is never
// scaled (flash_bias_triton.py:246-256).
#include "fb_kernels.h"

namespace fb {

// VEC: every streamed tensor is 16-byte aligned (base and strides) and d, r are multiples of 8.
template <class T, int NKD_, int NKR_, int NDV_, int QBLK_, bool VEC_, bool MASK_>
struct FwdCfg {
    static constexpr int NKD = NKD_, NKR = NKR_, NDV = NDV_, QBLK = QBLK_;
    static constexpr bool VEC = VEC_, MASK = MASK_;
    static constexpr int NWAVES = 4, NTHREADS = 64 * NWAVES;
    static constexpr int BM = NWAVES * QBLK * 32;
    static constexpr int KBLK = 2, BN = 32 * KBLK;
    static constexpr int NK = NKD + NKR;
    static constexpr int DKP = 16 * NK + 8; // LDS row of [K | K_b], elements (16 B of padding)
    static constexpr int DV = 32 * NDV;
    static constexpr int BNP = BN + 8; // LDS row of V^T
    static constexpr int SK_ELEMS = BN * DKP, SV_ELEMS = DV * BNP;
    static constexpr int LDS_BYTES = 2 * (SK_ELEMS + SV_ELEMS) * 2;
    // cooperative loader: 8-channel chunks of K and K_b, (4 keys x 8 channels) blocks of V
    static constexpr int CD = 2 * NKD, CR = 2 * NKR;
    static constexpr int K_TASKS = BN * CD, KB_TASKS = BN * CR, V_TASKS = (BN / 4) * (DV / 8);
    static constexpr int K_PT = (K_TASKS + NTHREADS - 1) / NTHREADS;
    static constexpr int KB_PT = (KB_TASKS + NTHREADS - 1) / NTHREADS;
    static constexpr int V_PT = (V_TASKS + NTHREADS - 1) / NTHREADS;
};

template <class C>
struct FwdStage { // one key tile in flight from HBM to LDS
    u32x4_t k[C::K_PT];
    u32x4_t kb[C::KB_PT > 0 ? C::KB_PT : 1];
    u32x4_t v[C::V_PT][4];
};

template <class C>
__device__ __forceinline__ void fwd_load_tile(FwdStage<C> &st, const FwdArgs &a, const uint16_t *kbase,
                                              const uint16_t *kbbase, const uint16_t *vbase, int n0, int tid) {
#pragma unroll
    for (int i = 0; i < C::K_PT; ++i) {
        const int task = tid + i * C::NTHREADS;
        const int row = task / C::CD, ch = task % C::CD;
        if (C::K_TASKS % C::NTHREADS == 0 || task < C::K_TASKS)
            st.k[i] = load_chunk<C::VEC>(kbase, a.k.ss, n0 + row, a.Lk, ch * 8, a.d);
    }
    if constexpr (C::NKR > 0) {
#pragma unroll
        for (int i = 0; i < C::KB_PT; ++i) {
            const int task = tid + i * C::NTHREADS;
            const int row = task / C::CR, ch = task % C::CR;
            if (C::KB_TASKS % C::NTHREADS == 0 || task < C::KB_TASKS)
                st.kb[i] = load_chunk<C::VEC>(kbbase, a.kb.ss, n0 + row, a.Lk, ch * 8, a.r);
        }
    }
#pragma unroll
    for (int i = 0; i < C::V_PT; ++i) {
        const int task = (C::NTHREADS - 1 - tid) + i * C::NTHREADS;
        const int quad = task / (C::DV / 8), ch = task % (C::DV / 8);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (C::V_TASKS % C::NTHREADS == 0 || task < C::V_TASKS)
                st.v[i][j] = load_chunk<C::VEC>(vbase, a.v.ss, n0 + quad * 4 + j, a.Lk, ch * 8, a.d);
        }
    }
}

template <class C>
__device__ __forceinline__ void fwd_store_tile(const FwdStage<C> &st, uint16_t *sK, uint16_t *sVt, int tid) {
#pragma unroll
    for (int i = 0; i < C::K_PT; ++i) {
        const int task = tid + i * C::NTHREADS;
        const int row = task / C::CD, ch = task % C::CD;
        if (task < C::K_TASKS) *reinterpret_cast<u32x4_t *>(sK + row * C::DKP + ch * 8) = st.k[i];
    }
    if constexpr (C::NKR > 0) {
#pragma unroll
        for (int i = 0; i < C::KB_PT; ++i) {
            const int task = tid + i * C::NTHREADS;
            const int row = task / C::CR, ch = task % C::CR;
            if (task < C::KB_TASKS)
                *reinterpret_cast<u32x4_t *>(sK + row * C::DKP + 16 * C::NKD + ch * 8) = st.kb[i];
        }
    }
#pragma unroll
    for (int i = 0; i < C::V_PT; ++i) {
        const int task = (C::NTHREADS - 1 - tid) + i * C::NTHREADS;
        const int quad = task / (C::DV / 8), ch = task % (C::DV / 8);
        if (task < C::V_TASKS) {
            const int col = slot_of(quad * 4); // 4 keys stay adjacent, quads are permuted
#pragma unroll
            for (int e = 0; e < 8; ++e) { // channel ch*8 + e gets the four keys as one 8-byte store
                const int w = e >> 1, sh = (e & 1) * 16;
                u32x2_t pk;
                pk[0] = ((st.v[i][0][w] >> sh) & 0xffffu) | (((st.v[i][1][w] >> sh) & 0xffffu) << 16);
                pk[1] = ((st.v[i][2][w] >> sh) & 0xffffu) | (((st.v[i][3][w] >> sh) & 0xffffu) << 16);
                *reinterpret_cast<u32x2_t *>(sVt + (ch * 8 + e) * C::BNP + col) = pk;
            }
        }
    }
}

// Additive mask value for (query, key); 0 outside the tensor (those scores are -inf anyway).
template <class T>
__device__ __forceinline__ float mask_at(const MaskDesc &m, const uint8_t *base, int query, int key, int Lq, int Lk) {
    if (key >= Lk || query >= Lq) return 0.f;
    const int64_t off = (m.type == 2 ? (int64_t)query * m.sm : 0) + key;
    if (m.is_f32) return reinterpret_cast<const float *>(base)[off];
    return T::to_float(reinterpret_cast<const uint16_t *>(base)[off]);
}

template <class T, class C>
__global__ __launch_bounds__(C::NTHREADS) __attribute__((amdgpu_waves_per_eu(2, 3))) void fwd_kernel(const FwdArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint16_t *sKbuf = reinterpret_cast<uint16_t *>(smem);
    uint16_t *sVbuf = sKbuf + 2 * C::SK_ELEMS;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = lane & 31, g = lane >> 5;

    const int total = a.ntiles_m * a.B * a.H;
    const int work = xcd_remap(blockIdx.x, total);
    const int bh = work / a.ntiles_m;
    int tile_m = work % a.ntiles_m;
    if (a.causal) tile_m = a.ntiles_m - 1 - tile_m; // long rows first
    const int b = bh / a.H, h = bh % a.H;
    const int m0 = tile_m * C::BM;
    const int wq0 = m0 + wave * (32 * C::QBLK); // first query of this wave

    const uint16_t *qbase = a.q.ptr + b * a.q.sb + h * a.q.sh;
    const uint16_t *kbase = a.k.ptr + b * a.k.sb + h * a.k.sh;
    const uint16_t *vbase = a.v.ptr + b * a.v.sb + h * a.v.sh;
    const uint16_t *qbbase = nullptr, *kbbase = nullptr;
    if constexpr (C::NKR > 0) {
        qbbase = a.qb.ptr + b * a.qb.sb + h * a.qb.sh;
        kbbase = a.kb.ptr + b * a.kb.sb + h * a.kb.sh;
    }
    const uint8_t *mbase = nullptr;
    if constexpr (C::MASK)
        mbase = reinterpret_cast<const uint8_t *>(a.mask.ptr) +
                (b * a.mask.sb + h * a.mask.sh) * (a.mask.is_f32 ? 4 : 2);

    // ---- query operand, resident in registers for the whole key loop
    u32x4_t qreg[C::QBLK][C::NK];
#pragma unroll
    for (int qb = 0; qb < C::QBLK; ++qb) {
        const int query = wq0 + qb * 32 + c;
#pragma unroll
        for (int t = 0; t < C::NK; ++t) {
            if (t < C::NKD)
                qreg[qb][t] = load_chunk<C::VEC>(qbase, a.q.ss, query, a.Lq, 16 * t + 8 * g, a.d);
            else if constexpr (C::NKR > 0)
                qreg[qb][t] = load_chunk<C::VEC>(qbbase, a.qb.ss, query, a.Lq, 16 * (t - C::NKD) + 8 * g, a.r);
        }
    }

    f32x16_t acc_o[C::QBLK][C::NDV];
    float m_run[C::QBLK], l_run[C::QBLK]; // running max (natural units), per-lane partial row sum
#pragma unroll
    for (int qb = 0; qb < C::QBLK; ++qb) {
        m_run[qb] = -INFINITY;
        l_run[qb] = 0.f;
#pragma unroll
        for (int n = 0; n < C::NDV; ++n)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc_o[qb][n][v] = 0.f;
    }

    // causal: tiles past the last query of this workgroup are never visible (:202)
    int k_end = a.Lk;
    if (a.causal && m0 + C::BM < k_end) k_end = m0 + C::BM;
    const int ntiles_k = (k_end + C::BN - 1) / C::BN;

    FwdStage<C> st;
    fwd_load_tile<C>(st, a, kbase, kbbase, vbase, 0, tid);
    fwd_store_tile<C>(st, sKbuf, sVbuf, tid);
    __syncthreads();

    for (int it = 0; it < ntiles_k; ++it) {
        const int cur = it & 1;
        const int n0 = it * C::BN;
        const bool more = it + 1 < ntiles_k;
        if (more) fwd_load_tile<C>(st, a, kbase, kbbase, vbase, n0 + C::BN, tid);

        const uint16_t *sK = sKbuf + cur * C::SK_ELEMS;
        const uint16_t *sVt = sVbuf + cur * C::SV_ELEMS;
        const int wq_last = wq0 + 32 * C::QBLK - 1;
        const bool visible = !(a.causal && n0 > wq_last) && wq0 < a.Lq;
        if (visible) {
            // ---- S^T = [K | K_b] [Q | Q_b]^T
            f32x16_t s[C::KBLK][C::QBLK];
#pragma unroll
            for (int kb = 0; kb < C::KBLK; ++kb) {
                u32x4_t ka[C::NK];
#pragma unroll
                for (int t = 0; t < C::NK; ++t)
                    ka[t] = *reinterpret_cast<const u32x4_t *>(sK + (kb * 32 + c) * C::DKP + 16 * t + 8 * g);
#pragma unroll
                for (int qb = 0; qb < C::QBLK; ++qb) {
                    f32x16_t acc;
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc[v] = 0.f;
#pragma unroll
                    for (int t = 0; t < C::NKD; ++t) acc = T::mfma(ka[t], qreg[qb][t], acc);
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc[v] *= a.scale;
#pragma unroll
                    for (int t = C::NKD; t < C::NK; ++t) acc = T::mfma(ka[t], qreg[qb][t], acc);
                    s[kb][qb] = acc;
                }
            }
            // ---- additive mask, then -inf for keys past the end and causal-hidden pairs
            if constexpr (C::MASK) {
#pragma unroll
                for (int kb = 0; kb < C::KBLK; ++kb)
#pragma unroll
                    for (int qb = 0; qb < C::QBLK; ++qb)
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const int key = n0 + kb * 32 + 8 * (v >> 2) + 4 * g + (v & 3);
                            s[kb][qb][v] += mask_at<T>(a.mask, mbase, wq0 + qb * 32 + c, key, a.Lq, a.Lk);
                        }
            }
            const bool ragged = n0 + C::BN > a.Lk;
            const bool diag = a.causal && (n0 + C::BN - 1 > wq0);
            if (ragged || diag) {
#pragma unroll
                for (int kb = 0; kb < C::KBLK; ++kb)
#pragma unroll
                    for (int qb = 0; qb < C::QBLK; ++qb)
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const int key = n0 + kb * 32 + 8 * (v >> 2) + 4 * g + (v & 3);
                            const int query = wq0 + qb * 32 + c;
                            if (key >= a.Lk || (a.causal && key > query)) s[kb][qb][v] = -INFINITY;
                        }
            }
            // ---- online softmax, one query per lane (two lanes share a query)
#pragma unroll
            for (int qb = 0; qb < C::QBLK; ++qb) {
                float mx = m_run[qb];
#pragma unroll
                for (int kb = 0; kb < C::KBLK; ++kb)
#pragma unroll
                    for (int v = 0; v < 16; ++v) mx = fmaxf(mx, s[kb][qb][v]);
                mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
                const float mref = (mx == -INFINITY) ? 0.f : mx; // whole row hidden so far
                const float m2 = mref * kLog2e;
                const float alpha = fast_exp2(m_run[qb] * kLog2e - m2);
                float lsum = 0.f;
#pragma unroll
                for (int kb = 0; kb < C::KBLK; ++kb)
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const float p = fast_exp2(__builtin_fmaf(s[kb][qb][v], kLog2e, -m2));
                        s[kb][qb][v] = p;
                        lsum += p;
                    }
                l_run[qb] = l_run[qb] * alpha + lsum;
                m_run[qb] = mx;
#pragma unroll
                for (int n = 0; n < C::NDV; ++n)
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc_o[qb][n][v] *= alpha;
            }
            // ---- O^T += V^T P^T
#pragma unroll
            for (int kb = 0; kb < C::KBLK; ++kb)
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    u32x4_t pb[C::QBLK];
#pragma unroll
                    for (int qb = 0; qb < C::QBLK; ++qb)
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            pb[qb][e] = T::pack2(s[kb][qb][8 * t + 2 * e], s[kb][qb][8 * t + 2 * e + 1]);
#pragma unroll
                    for (int n = 0; n < C::NDV; ++n) {
                        const u32x4_t va = *reinterpret_cast<const u32x4_t *>(
                            sVt + (32 * n + c) * C::BNP + kb * 32 + 16 * t + 8 * g);
#pragma unroll
                        for (int qb = 0; qb < C::QBLK; ++qb) acc_o[qb][n] = T::mfma(va, pb[qb], acc_o[qb][n]);
                    }
                }
        }
        if (more) fwd_store_tile<C>(st, sKbuf + (cur ^ 1) * C::SK_ELEMS, sVbuf + (cur ^ 1) * C::SV_ELEMS, tid);
        __syncthreads();
    }

    // ---- epilogue: o = acc / l, lse = m + ln(l)
    uint16_t *obase = const_cast<uint16_t *>(a.o.ptr) + b * a.o.sb + h * a.o.sh;
#pragma unroll
    for (int qb = 0; qb < C::QBLK; ++qb) {
        const int query = wq0 + qb * 32 + c;
        const float l = l_run[qb] + __shfl_xor(l_run[qb], 32, 64);
        const float inv = 1.f / l;
        if (query < a.Lq) {
            if (g == 0) a.lse[(int64_t)bh * a.Lq + query] = m_run[qb] + __builtin_amdgcn_logf(l) * kLn2;
            uint16_t *orow = obase + (int64_t)query * a.o.ss;
#pragma unroll
            for (int n = 0; n < C::NDV; ++n)
#pragma unroll
                for (int bq = 0; bq < 4; ++bq) {
                    const int ch = 32 * n + 8 * bq + 4 * g;
                    if (C::VEC && ch + 4 <= a.d) {
                        u32x2_t pk;
                        pk[0] = T::pack2(acc_o[qb][n][4 * bq] * inv, acc_o[qb][n][4 * bq + 1] * inv);
                        pk[1] = T::pack2(acc_o[qb][n][4 * bq + 2] * inv, acc_o[qb][n][4 * bq + 3] * inv);
                        *reinterpret_cast<u32x2_t *>(orow + ch) = pk;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (ch + e < a.d) orow[ch + e] = T::from_float(acc_o[qb][n][4 * bq + e] * inv);
                    }
                }
        }
    }
}

template <class T, int NKD, int NKR, int NDV, bool VEC, bool MASK>
static hipError_t launch_fwd_vec(const FwdArgs &a0, hipStream_t stream) {
    constexpr int QBLK = 1;
    typedef FwdCfg<T, NKD, NKR, NDV, QBLK, VEC, MASK> C;
    FwdArgs a = a0;
    a.ntiles_m = (a.Lq + C::BM - 1) / C::BM;
    auto kern = fwd_kernel<T, C>;
    if (C::LDS_BYTES > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
        if (e != hipSuccess) return e;
    }
    const int total = a.ntiles_m * a.B * a.H;
    hipLaunchKernelGGL(kern, dim3(total), dim3(C::NTHREADS), C::LDS_BYTES, stream, a);
    return hipGetLastError();
}

template <class T, int NKD, int NKR, int NDV>
static hipError_t launch_fwd_cfg(const FwdArgs &a, hipStream_t stream) {
    const bool vec = a.q.vec_ok && a.k.vec_ok && a.v.vec_ok && a.o.vec_ok && a.d % 8 == 0 &&
                     (a.r == 0 || (a.qb.vec_ok && a.kb.vec_ok && a.r % 8 == 0));
    if (a.mask.type)
        return vec ? launch_fwd_vec<T, NKD, NKR, NDV, true, true>(a, stream)
                   : launch_fwd_vec<T, NKD, NKR, NDV, false, true>(a, stream);
    return vec ? launch_fwd_vec<T, NKD, NKR, NDV, true, false>(a, stream)
               : launch_fwd_vec<T, NKD, NKR, NDV, false, false>(a, stream);
}

template <class T, int NKD, int NDV>
static hipError_t launch_fwd_r(const FwdArgs &a, hipStream_t stream) {
    switch (nkr_of(a.r)) {
    case 0: return launch_fwd_cfg<T, NKD, 0, NDV>(a, stream);
    case 1: return launch_fwd_cfg<T, NKD, 1, NDV>(a, stream);
    case 2: return launch_fwd_cfg<T, NKD, 2, NDV>(a, stream);
    case 4: return launch_fwd_cfg<T, NKD, 4, NDV>(a, stream);
    default: return launch_fwd_cfg<T, NKD, 8, NDV>(a, stream);
    }
}

// This file is compiled once per (element type, head-dim bucket); FB_T and FB_NKD / FB_NDV pick
// the instantiation and FB_SUFFIX names the launcher (see Makefile).
#define FB_CAT2(a, b) a##b
#define FB_CAT(a, b) FB_CAT2(a, b)
hipError_t FB_CAT(launch_fwd_, FB_SUFFIX)(const FwdArgs &a, hipStream_t stream) {
    return launch_fwd_r<FB_T, FB_NKD, FB_NDV>(a, stream);
}

} // namespace fb
