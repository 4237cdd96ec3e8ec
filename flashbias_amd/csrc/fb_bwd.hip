// Backward FlashBias attention for gfx950: dq, dk, dv, dq_bias, dk_bias.
// Replaces _bwd_preprocess_do_o_dot, _bwd_kernel and the final dq copies of the reference
// (flash_bias/flash_bias_triton.py:358-400, :450-1097, :1340-1342).
//
// Three launches:
//   preprocess  delta[i] = sum_c o[i,c] dout[i,c]; zero the dq workspace.
//   main        one workgroup (4 waves) owns 128 consecutive keys of one (batch, head), wave w
//               owns keys [32w, 32w+32).  Queries are streamed in steps of 64 (two 32-blocks)
//               through LDS (next step prefetched into registers).  With lane = key, register = query (C layout of
//               S = [Q|Q_b][K|K_b]^T with A from LDS, B from key registers):
//                 P   = exp(S - lse)                      recomputed from the saved lse
//                 dP  = dout V^T - delta                  accumulator starts at -delta
//                 dS  = P * dP
//                 dV^T     += dout^T P                    A = dout^T tile (LDS), B = P regs
//                 [dK|dK_b]^T += [Q|Q_b]^T dS             A = [Q|Q_b]^T tile (LDS), B = dS regs
//               so P and dS feed their MFMAs straight from registers.  dS is also written to
//               LDS as (query, key) bf16/fp16; after a barrier each wave contracts one
//               32-row block of [dQ|dQ_b]^T over all 128 keys of the workgroup
//                 [dQ|dQ_b]^T (channels x queries) = [K|K_b]^T dS^T
//               and adds it with fp32 atomics into a transposed workspace (channel-major, so
//               that the 32 lanes of a row hit 128 consecutive bytes).  Only one partial sum
//               per (128 keys, query) reaches HBM and the N x N matrices never do.
//   finalize    workspace -> dq (times scale), dq_bias in the input dtype.
#include "fb_kernels.h"

namespace fb {

// ------------------------------------------------------------------------------------ main
// VEC: every streamed tensor is 16-byte aligned (base and strides) and d, r are multiples of 8.
template <class T, int NKD_, int NKR_, int NDV_, bool VEC_, bool MASK_>
struct BwdCfg {
    static constexpr int NKD = NKD_, NKR = NKR_, NDV = NDV_;
    static constexpr bool VEC = VEC_, MASK = MASK_;
    static constexpr int NWAVES = 4, NTHREADS = 64 * NWAVES;
    static constexpr int BN = 32 * NWAVES; // keys per workgroup
    static constexpr int QBLK = 2, BMQ = 32 * QBLK; // queries per step
    static constexpr int NK = NKD + NKR;
    static constexpr int MB = (NK + 1) / 2;             // 32-row blocks of [dK|dK_b]^T, [dQ|dQ_b]^T
    static constexpr int NT2 = MB * QBLK;               // dQ^T tiles per step
    // Phase-2 tiles are dealt to the waves in "slots"; each slot pins one 32-row block of
    // [K|K_b]^T in registers.  Few row blocks: slot i of wave w is tile w + 4i (row block
    // tile % MB, query block tile / MB).  Many: slot i is row block w + 4i, both query blocks.
    static constexpr bool BY_MB = MB >= 4;
    static constexpr int KT_SLOTS = BY_MB ? (MB + NWAVES - 1) / NWAVES : (NT2 + NWAVES - 1) / NWAVES;
    static constexpr int DKP = 16 * NK + 8;   // sQ row (elements)
    static constexpr int DOP = 16 * NKD + 8;  // sdO row
    static constexpr int QTP = BMQ + 8;       // sQt / sdOt row (queries, slot-permuted)
    static constexpr int DSP = BN + 8;        // sdS row (keys)
    static constexpr int SQ = BMQ * DKP, SDO = BMQ * DOP, SQT = 32 * MB * QTP, SDOT = 32 * NDV * QTP;
    static constexpr int STAGE_ELEMS = SQ + SDO + SQT + SDOT + 4 * BMQ; // + lse2, delta as fp32
    static constexpr int SDS = BMQ * DSP;
    static constexpr int LDS_BYTES = (STAGE_ELEMS + SDS) * 2;
    // loader tasks: (4 queries x 8 channels) blocks of Q, Q_b and dout
    static constexpr int CQ = 2 * NKD, CR = 2 * NKR, CO = 2 * NKD;
    static constexpr int QUADS = BMQ / 4;
    static constexpr int TASKS = QUADS * (CQ + CR + CO);
    static constexpr int PT = (TASKS + NTHREADS - 1) / NTHREADS;
    // register budget: 2 waves per SIMD (256 registers each) for the small shapes, which keeps
    // the MFMA accumulators in ordinary VGPRs; the big ones need the whole file
    static constexpr int WAVES_EU = (NK <= 4 && NDV <= 2) ? 2 : 1;
};

template <class C>
struct BwdStage {
    u32x4_t x[C::PT][4];
    float lse2, delta;
};

// task -> (kind, quad, chunk): kind 0 = Q, 1 = Q_b, 2 = dout
template <class C>
__device__ __forceinline__ void bwd_task(int task, int &kind, int &quad, int &ch) {
    quad = task % C::QUADS;
    const int cc = task / C::QUADS;
    if (cc < C::CQ) {
        kind = 0;
        ch = cc;
    } else if (cc < C::CQ + C::CR) {
        kind = 1;
        ch = cc - C::CQ;
    } else {
        kind = 2;
        ch = cc - C::CQ - C::CR;
    }
}

template <class C>
__device__ __forceinline__ void bwd_load_step(BwdStage<C> &st, const BwdArgs &a, const uint16_t *qbase,
                                              const uint16_t *qbbase, const uint16_t *dobase, const float *lse,
                                              const float *delta, int m0, int tid) {
#pragma unroll
    for (int i = 0; i < C::PT; ++i) {
        const int task = tid + i * C::NTHREADS;
        int kind, quad, ch;
        bwd_task<C>(task, kind, quad, ch);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int query = m0 + quad * 4 + j;
            // one load per task: pick the tensor by lane (all three share the chunk geometry)
            const uint16_t *base = kind == 0 ? qbase : kind == 1 ? qbbase : dobase;
            const int64_t ld = kind == 0 ? a.q.ss : kind == 1 ? a.qb.ss : a.dout.ss;
            const int ncols = kind == 1 ? a.r : a.d;
            st.x[i][j] = u32x4_t{0u, 0u, 0u, 0u};
            if (task < C::TASKS) st.x[i][j] = load_chunk<C::VEC>(base, ld, query, a.Lq, ch * 8, ncols);
        }
    }
    st.lse2 = INFINITY; // rows past the end: P = exp2(-inf) = 0
    st.delta = 0.f;
    if (tid < C::BMQ && m0 + tid < a.Lq) {
        st.lse2 = lse[m0 + tid] * kLog2e;
        st.delta = delta[m0 + tid];
    }
}

template <class C>
__device__ __forceinline__ void bwd_store_step(const BwdStage<C> &st, uint16_t *stage, int tid) {
    uint16_t *sQ = stage, *sdO = sQ + C::SQ, *sQt = sdO + C::SDO, *sdOt = sQt + C::SQT;
    float *sStat = reinterpret_cast<float *>(sdOt + C::SDOT);
#pragma unroll
    for (int i = 0; i < C::PT; ++i) {
        const int task = tid + i * C::NTHREADS;
        int kind, quad, ch;
        bwd_task<C>(task, kind, quad, ch);
        if (task < C::TASKS) {
            // row-major copy (A operand of S and dP) ...
            uint16_t *rm = kind == 2 ? sdO : sQ;
            const int ld = kind == 2 ? C::DOP : C::DKP;
            const int col0 = (kind == 1 ? 16 * C::NKD : 0) + ch * 8;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                *reinterpret_cast<u32x4_t *>(rm + (quad * 4 + j) * ld + col0) = st.x[i][j];
            // ... and transposed copy (A operand of dV^T and [dK|dK_b]^T), queries slot-permuted
            uint16_t *tr = kind == 2 ? sdOt : sQt;
            const int qcol = slot_of(quad * 4);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int w = e >> 1, sh = (e & 1) * 16;
                u32x2_t pk;
                pk[0] = ((st.x[i][0][w] >> sh) & 0xffffu) | (((st.x[i][1][w] >> sh) & 0xffffu) << 16);
                pk[1] = ((st.x[i][2][w] >> sh) & 0xffffu) | (((st.x[i][3][w] >> sh) & 0xffffu) << 16);
                *reinterpret_cast<u32x2_t *>(tr + (col0 + e) * C::QTP + qcol) = pk;
            }
        }
    }
    if (tid < C::BMQ) {
        sStat[tid] = st.lse2;
        sStat[C::BMQ + tid] = st.delta;
    }
}

template <class T>
__device__ __forceinline__ float mask_at_b(const MaskDesc &m, const uint8_t *base, int query, int key, int Lq,
                                           int Lk) {
    if (key >= Lk || query >= Lq) return 0.f;
    const int64_t off = (m.type == 2 ? (int64_t)query * m.sm : 0) + key;
    if (m.is_f32) return reinterpret_cast<const float *>(base)[off];
    return T::to_float(reinterpret_cast<const uint16_t *>(base)[off]);
}

template <class T, class C>
__global__ __launch_bounds__(C::NTHREADS) __attribute__((amdgpu_waves_per_eu(C::WAVES_EU, C::WAVES_EU))) void bwd_kernel(const BwdArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint16_t *stage0 = reinterpret_cast<uint16_t *>(smem);
    uint16_t *sdS = stage0 + C::STAGE_ELEMS;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = lane & 31, g = lane >> 5;

    const int total = a.ntiles_n * a.B * a.H;
    const int work = xcd_remap(blockIdx.x, total);
    const int bh = work / a.ntiles_n;
    const int tile_n = work % a.ntiles_n; // causal: low key tiles see the most queries, they go first
    const int b = bh / a.H, h = bh % a.H;
    const int n0 = tile_n * C::BN;
    const int wk0 = n0 + wave * 32;
    const int key = wk0 + c; // this lane's key in phase 1

    const uint16_t *qbase = a.q.ptr + b * a.q.sb + h * a.q.sh;
    const uint16_t *kbase = a.k.ptr + b * a.k.sb + h * a.k.sh;
    const uint16_t *vbase = a.v.ptr + b * a.v.sb + h * a.v.sh;
    const uint16_t *dobase = a.dout.ptr + b * a.dout.sb + h * a.dout.sh;
    const uint16_t *qbbase = nullptr, *kbbase = nullptr;
    if constexpr (C::NKR > 0) {
        qbbase = a.qb.ptr + b * a.qb.sb + h * a.qb.sh;
        kbbase = a.kb.ptr + b * a.kb.sb + h * a.kb.sh;
    }
    const float *lse = a.lse + (int64_t)bh * a.Lq;
    const float *delta = a.delta + (int64_t)bh * a.Lq;
    const uint8_t *mbase = nullptr;
    if constexpr (C::MASK)
        mbase = reinterpret_cast<const uint8_t *>(a.mask.ptr) +
                (b * a.mask.sb + h * a.mask.sh) * (a.mask.is_f32 ? 4 : 2);

    // ---- key-side operands, resident in registers
    u32x4_t kreg[C::NK];  // B operand of S: this lane's key, channels 16t + 8g ..
    u32x4_t vreg[C::NKD]; // B operand of dP
#pragma unroll
    for (int t = 0; t < C::NK; ++t) {
        if (t < C::NKD)
            kreg[t] = load_chunk<C::VEC>(kbase, a.k.ss, key, a.Lk, 16 * t + 8 * g, a.d);
        else if constexpr (C::NKR > 0)
            kreg[t] = load_chunk<C::VEC>(kbbase, a.kb.ss, key, a.Lk, 16 * (t - C::NKD) + 8 * g, a.r);
    }
#pragma unroll
    for (int t = 0; t < C::NKD; ++t) {
        vreg[t] = load_chunk<C::VEC>(vbase, a.v.ss, key, a.Lk, 16 * t + 8 * g, a.d);
    }
    // A operand of phase 2: rows = channels of [K|K_b] (32 per block), k-slots = the 128 keys
    // of the workgroup in natural order.
    u32x4_t ktreg[C::KT_SLOTS][8];
#pragma unroll
    for (int sl = 0; sl < C::KT_SLOTS; ++sl) {
        const int mb = C::BY_MB ? wave + C::NWAVES * sl : (wave + C::NWAVES * sl) % C::MB;
        const int ch = 32 * mb + c; // channel in the padded [16*NKD | 16*NKR] numbering
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            uint16_t e[8];
#pragma unroll
            for (int x = 0; x < 8; ++x) {
                const int kk = n0 + 16 * s + 8 * g + x;
                uint16_t val = 0;
                if (kk < a.Lk) {
                    if (ch < 16 * C::NKD) {
                        if (ch < a.d) val = kbase[(int64_t)kk * a.k.ss + ch];
                    } else if constexpr (C::NKR > 0) {
                        if (ch - 16 * C::NKD < a.r) val = kbbase[(int64_t)kk * a.kb.ss + ch - 16 * C::NKD];
                    }
                }
                e[x] = val;
            }
#pragma unroll
            for (int x = 0; x < 4; ++x) ktreg[sl][s][x] = (uint32_t)e[2 * x] | ((uint32_t)e[2 * x + 1] << 16);
        }
    }

    f32x16_t acc_dv[C::NDV], acc_dk[C::MB];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
#pragma unroll
        for (int n = 0; n < C::NDV; ++n) acc_dv[n][v] = 0.f;
#pragma unroll
        for (int n = 0; n < C::MB; ++n) acc_dk[n][v] = 0.f;
    }

    // causal: the first query step that can see this key tile (:498)
    const int step0 = a.causal ? n0 / C::BMQ : 0;
    const int nsteps = (a.Lq + C::BMQ - 1) / C::BMQ;

    // Workgroups of one (batch, head) walk the query steps in rotated order: at any moment
    // they add into different rows of the dq workspace instead of all hitting the same ones.
    const int span = nsteps - step0;
    const int rot = span > 0 ? (int)(((int64_t)tile_n * 7) % span) : 0;
    auto step_of = [&](int it) {
        const int x = it + rot;
        return step0 + (x >= span ? x - span : x);
    };

    BwdStage<C> st;
    if (span > 0) {
        bwd_load_step<C>(st, a, qbase, qbbase, dobase, lse, delta, step_of(0) * C::BMQ, tid);
        bwd_store_step<C>(st, stage0, tid);
    }
    __syncthreads();

    for (int it = 0; it < span; ++it) {
        const int m0 = step_of(it) * C::BMQ;
        const bool more = it + 1 < span;
        if (more) bwd_load_step<C>(st, a, qbase, qbbase, dobase, lse, delta, step_of(it + 1) * C::BMQ, tid);

        const uint16_t *sQ = stage0;
        const uint16_t *sdO = sQ + C::SQ, *sQt = sdO + C::SDO, *sdOt = sQt + C::SQT;
        const float *sStat = reinterpret_cast<const float *>(sdOt + C::SDOT);

        // ------------------------------------------------------------------ phase 1
        const bool visible = !(a.causal && wk0 > m0 + C::BMQ - 1) && wk0 < a.Lk;
#pragma unroll
        for (int qb = 0; qb < C::QBLK; ++qb) {
            u32x4_t pds[2]; // dS, packed, per 16-query step
            if (visible) {
                f32x16_t s, dp;
#pragma unroll
                for (int v = 0; v < 16; ++v) s[v] = 0.f;
#pragma unroll
                for (int t = 0; t < C::NKD; ++t)
                    s = T::mfma(*reinterpret_cast<const u32x4_t *>(sQ + (qb * 32 + c) * C::DKP + 16 * t + 8 * g),
                                kreg[t], s);
#pragma unroll
                for (int v = 0; v < 16; ++v) s[v] *= a.scale;
#pragma unroll
                for (int t = C::NKD; t < C::NK; ++t)
                    s = T::mfma(*reinterpret_cast<const u32x4_t *>(sQ + (qb * 32 + c) * C::DKP + 16 * t + 8 * g),
                                kreg[t], s);
                // per-register query statistics: query = qb*32 + 8*(v/4) + 4g + v%4
                float lse2[16];
#pragma unroll
                for (int bq = 0; bq < 4; ++bq) {
                    const f32x4_t l4 = *reinterpret_cast<const f32x4_t *>(sStat + qb * 32 + 8 * bq + 4 * g);
                    const f32x4_t d4 = *reinterpret_cast<const f32x4_t *>(sStat + C::BMQ + qb * 32 + 8 * bq + 4 * g);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        lse2[4 * bq + e] = l4[e];
                        dp[4 * bq + e] = -d4[e];
                    }
                }
#pragma unroll
                for (int t = 0; t < C::NKD; ++t)
                    dp = T::mfma(*reinterpret_cast<const u32x4_t *>(sdO + (qb * 32 + c) * C::DOP + 16 * t + 8 * g),
                                 vreg[t], dp);
                if constexpr (C::MASK) {
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        s[v] += mask_at_b<T>(a.mask, mbase, m0 + qb * 32 + 8 * (v >> 2) + 4 * g + (v & 3), key, a.Lq,
                                             a.Lk);
                }
                const bool edge = (wk0 + 32 > a.Lk) || (a.causal && wk0 + 31 > m0 + qb * 32);
                if (edge) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int query = m0 + qb * 32 + 8 * (v >> 2) + 4 * g + (v & 3);
                        if (key >= a.Lk || (a.causal && key > query)) s[v] = -INFINITY;
                    }
                }
                u32x4_t pp[2];
#pragma unroll
                for (int v = 0; v < 16; v += 2) {
                    const float p0 = fast_exp2(__builtin_fmaf(s[v], kLog2e, -lse2[v]));
                    const float p1 = fast_exp2(__builtin_fmaf(s[v + 1], kLog2e, -lse2[v + 1]));
                    pp[v >> 3][(v & 7) >> 1] = T::pack2(p0, p1);
                    pds[v >> 3][(v & 7) >> 1] = T::pack2(p0 * dp[v], p1 * dp[v + 1]);
                }
                // dV^T += dout^T P ; [dK|dK_b]^T += [Q|Q_b]^T dS   (contraction over this block's queries)
#pragma unroll
                for (int t = 0; t < 2; ++t) {
#pragma unroll
                    for (int n = 0; n < C::NDV; ++n)
                        acc_dv[n] = T::mfma(*reinterpret_cast<const u32x4_t *>(sdOt + (32 * n + c) * C::QTP + qb * 32 +
                                                                               16 * t + 8 * g),
                                            pp[t], acc_dv[n]);
#pragma unroll
                    for (int n = 0; n < C::MB; ++n)
                        acc_dk[n] = T::mfma(*reinterpret_cast<const u32x4_t *>(sQt + (32 * n + c) * C::QTP + qb * 32 +
                                                                               16 * t + 8 * g),
                                            pds[t], acc_dk[n]);
                }
            } else {
#pragma unroll
                for (int t = 0; t < 2; ++t) pds[t] = u32x4_t{0u, 0u, 0u, 0u};
            }
            // dS (query, key) to LDS for phase 2: register v of step t=v/8 is query 8*(v/4)+4g+v%4
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t w = pds[v >> 3][(v & 7) >> 1];
                const uint16_t val = (uint16_t)((v & 1) ? (w >> 16) : (w & 0xffffu));
                sdS[(qb * 32 + 8 * (v >> 2) + 4 * g + (v & 3)) * C::DSP + wave * 32 + c] = val;
            }
        }
        __syncthreads();

        // ------------------------------------------------------------------ phase 2
        float *dq_bh = a.dq_acc + (int64_t)bh * a.dq_rows * a.lq_pad;
        auto dq_tile = [&](const u32x4_t(&kt)[8], int mb, int qb) {
            f32x16_t acc;
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[v] = 0.f;
#pragma unroll
            for (int s = 0; s < 8; ++s)
                acc = T::mfma(kt[s], *reinterpret_cast<const u32x4_t *>(sdS + (qb * 32 + c) * C::DSP + 16 * s + 8 * g),
                              acc);
            const int query = m0 + qb * 32 + c;
            if (query < a.Lq) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int ch = 32 * mb + 8 * (v >> 2) + 4 * g + (v & 3);
                    int row = -1;
                    if (ch < 16 * C::NKD) {
                        if (ch < a.d) row = ch;
                    } else if (ch - 16 * C::NKD < a.r) {
                        row = a.r_row0 + ch - 16 * C::NKD;
                    }
#ifdef FB_EXPERIMENT_NO_ATOMIC
                    if (row >= 0 && acc[v] == 12345.678f) dq_bh[(int64_t)row * a.lq_pad + query] = acc[v];
#else
                    if (row >= 0) unsafeAtomicAdd(dq_bh + (int64_t)row * a.lq_pad + query, acc[v]);
#endif
                }
            }
        };
#pragma unroll
        for (int sl = 0; sl < C::KT_SLOTS; ++sl) {
            if constexpr (C::BY_MB) {
                const int mb = wave + C::NWAVES * sl;
                if (mb < C::MB) {
#pragma unroll
                    for (int qb = 0; qb < C::QBLK; ++qb) dq_tile(ktreg[sl], mb, qb);
                }
            } else {
                const int t2 = wave + C::NWAVES * sl;
                if (t2 < C::NT2) dq_tile(ktreg[sl], t2 % C::MB, t2 / C::MB);
            }
        }
        // every wave is past the barrier above, so nobody still reads this step's tiles
        if (more) bwd_store_step<C>(st, stage0, tid);
        __syncthreads();
    }

    // ---- epilogue: dv, dk (times scale), dk_bias for this lane's key
    if (key < a.Lk) {
        uint16_t *dvrow = const_cast<uint16_t *>(a.dv.ptr) + b * a.dv.sb + h * a.dv.sh + (int64_t)key * a.dv.ss;
        uint16_t *dkrow = const_cast<uint16_t *>(a.dk.ptr) + b * a.dk.sb + h * a.dk.sh + (int64_t)key * a.dk.ss;
        uint16_t *dkbrow = nullptr;
        if constexpr (C::NKR > 0)
            dkbrow = const_cast<uint16_t *>(a.dkb.ptr) + b * a.dkb.sb + h * a.dkb.sh + (int64_t)key * a.dkb.ss;
#pragma unroll
        for (int n = 0; n < C::NDV; ++n)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int ch = 32 * n + 8 * (v >> 2) + 4 * g + (v & 3);
                if (ch < a.d) dvrow[ch] = T::from_float(acc_dv[n][v]);
            }
#pragma unroll
        for (int n = 0; n < C::MB; ++n)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int ch = 32 * n + 8 * (v >> 2) + 4 * g + (v & 3);
                if (ch < 16 * C::NKD) {
                    if (ch < a.d) dkrow[ch] = T::from_float(acc_dk[n][v] * a.scale);
                } else if constexpr (C::NKR > 0) {
                    if (ch - 16 * C::NKD < a.r) dkbrow[ch - 16 * C::NKD] = T::from_float(acc_dk[n][v]);
                }
            }
    }
}

// ------------------------------------------------------------------------------- launchers
template <class T, int NKD, int NKR, int NDV, bool VEC, bool MASK>
static hipError_t launch_bwd_vec(const BwdArgs &a0, hipStream_t stream) {
    typedef BwdCfg<T, NKD, NKR, NDV, VEC, MASK> C;
    BwdArgs a = a0;
    a.ntiles_n = (a.Lk + C::BN - 1) / C::BN;
    auto kern = bwd_kernel<T, C>;
    if (C::LDS_BYTES > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
        if (e != hipSuccess) return e;
    }
    const int total = a.ntiles_n * a.B * a.H;
    hipLaunchKernelGGL(kern, dim3(total), dim3(C::NTHREADS), C::LDS_BYTES, stream, a);
    return hipGetLastError();
}

template <class T, int NKD, int NKR, int NDV>
static hipError_t launch_bwd_cfg(const BwdArgs &a, hipStream_t stream) {
    const bool vec = a.q.vec_ok && a.k.vec_ok && a.v.vec_ok && a.dout.vec_ok && a.d % 8 == 0 &&
                     (a.r == 0 || (a.qb.vec_ok && a.kb.vec_ok && a.r % 8 == 0));
    if (a.mask.type)
        return vec ? launch_bwd_vec<T, NKD, NKR, NDV, true, true>(a, stream)
                   : launch_bwd_vec<T, NKD, NKR, NDV, false, true>(a, stream);
    return vec ? launch_bwd_vec<T, NKD, NKR, NDV, true, false>(a, stream)
               : launch_bwd_vec<T, NKD, NKR, NDV, false, false>(a, stream);
}

template <class T, int NKD, int NDV>
static hipError_t launch_bwd_r(const BwdArgs &a, hipStream_t stream) {
    switch (nkr_of(a.r)) {
    case 0: return launch_bwd_cfg<T, NKD, 0, NDV>(a, stream);
    case 1: return launch_bwd_cfg<T, NKD, 1, NDV>(a, stream);
    case 2: return launch_bwd_cfg<T, NKD, 2, NDV>(a, stream);
    case 4: return launch_bwd_cfg<T, NKD, 4, NDV>(a, stream);
    default: return launch_bwd_cfg<T, NKD, 8, NDV>(a, stream);
    }
}

// This file is compiled once per (element type, head-dim bucket); FB_T and FB_NKD / FB_NDV pick
// the instantiation and FB_SUFFIX names the launcher (see Makefile).
#define FB_CAT2(a, b) a##b
#define FB_CAT(a, b) FB_CAT2(a, b)
hipError_t FB_CAT(launch_bwd_main_, FB_SUFFIX)(const BwdArgs &a, hipStream_t stream) {
    return launch_bwd_r<FB_T, FB_NKD, FB_NDV>(a, stream);
}

} // namespace fb
