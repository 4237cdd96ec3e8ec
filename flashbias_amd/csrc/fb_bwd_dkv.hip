// Backward FlashBias attention for gfx950, part 1 of 2: dk, dv and dk_bias.
// Together with fb_bwd_dq.hip this replaces _bwd_kernel of the reference
// (flash_bias/flash_bias_triton.py:450-1097); this kernel covers the key-block loop of
// _bwd_kernel_one_col_block (:575-869) except its dq / dq_bias updates.
//
// Key-stationary: one workgroup (4 waves) owns 64 * KBW consecutive keys of one
// (batch, head), wave w owns KBW blocks of 32 of them, whose K, K_b and V stay in registers.
// Queries are streamed in steps of 64 (two 32-blocks) through a ring of three LDS stages that
// global_load_lds fills directly, two steps ahead of the arithmetic (one step of arithmetic is
// shorter than a trip to memory), without passing through registers.  With lane = key, register = query (C layout of S with A = query rows from
// LDS, B = key registers):
//
//   S   = [Q | Q_b] [K | K_b]^T, the q k^T part times scale  (:638-641)
//   P   = exp(S - lse)                                         (:670)
//   dP  = dO V^T - delta      accumulator starts at -delta, read from LDS into place (:705-714);
//                             lse * log2(e) and -delta come from the preprocess step
//   dS  = P * dP
//   dV^T          += dO^T P              A = dO tile read column-wise (LDS),      B = P registers   (:697)
//   [dK | dK_b]^T += [Q | Q_b]^T dS      A = [Q | Q_b] tile read column-wise (LDS), B = dS registers (:717-719)
//
// P and dS feed their MFMAs straight from the accumulator layout (no LDS round trip); every
// A operand read from LDS is used for all KBW key blocks of the wave.  The accumulators are
// summed in a fixed order: dk, dv, dk_bias are bit-reproducible.
#include "fb_kernels.h"

namespace fb {

// PART: 0 = dv, dk and dk_bias in one pass; 1 = dv only; 2 = [dk | dk_bias] only; 3 / 4 = the
// lower / upper half of the 32-row blocks of [dk | dk_bias] only.  Head dims above 64 run as two
// launches (1, 2) while the accumulators of pass 2 fit 256 registers (ranks up to 32, no mask),
// else as three (1, 3, 4), with 32-query steps: each pass keeps its accumulators in registers and
// its LDS stages small enough for two waves per SIMD, which is worth recomputing S.
// FOLD_: the scores are scale * (q k^T + q_b (k_b / scale)^T), no multiply per score for the scale
// (the launcher says when that is exact).
// BG_: also accumulate dk_bias (false: the caller does not want the factor gradients; the accumulator blocks that
// hold nothing but dk_bias are then left out).
template <class T, int NKD_, int NKR_, int NDV_, bool VEC_, bool MASK_, int PART_ = 0, bool FOLD_ = false, bool BG_ = true>
struct DkvCfg {
    static constexpr bool FOLD = FOLD_;
    static_assert(!FOLD_ || (VEC_ && !MASK_), "folded scale: direct loader, no additive mask");
    // folded scale with r <= 8: the Q_b columns 8..15 of a step hold a second copy of q_b, the
    // partner of the low parts of k_b / scale in the key operand
    static __device__ __forceinline__ bool low_parts(const BwdArgs &a) { return FOLD_ && NKR_ == 1 && a.r <= 8 && a.scale != 1.f; }
    static constexpr int NKD = NKD_, NKR = NKR_, NDV = NDV_;
    static constexpr bool VEC = VEC_, MASK = MASK_;
    static constexpr bool DO_DV = PART_ <= 1, DO_DK = PART_ != 1;
    static constexpr int NWAVES = 4, NTHREADS = 64 * NWAVES;
    static constexpr int NK = NKD + NKR;
    static constexpr int MB = (NK + 1) / 2; // 32-row blocks of [dK | dK_b]^T
    // ... of which this instantiation accumulates [MB0, MB1)
    static constexpr int MB0 = PART_ == 4 ? MB / 2 : 0,
                         MB1 = PART_ == 1 ? 0 : PART_ == 3 ? MB / 2 : (BG_ ? MB : (NKD_ + 1) / 2);
    static_assert(BG_ || PART_ == 0, "");
    static constexpr int KBW = 1; // key blocks per wave
    static constexpr int BN = 32 * KBW * NWAVES;              // keys per workgroup
    static constexpr int QBLK = PART_ == 0 ? 2 : 1, BMQ = 32 * QBLK; // queries per step
    // sQ row: [Q | Q_b] of one query, sdO row: dout of one query, both in swizzled 16-byte
    // chunks; each tile is kept once and read row-wise (S, dP) and column-wise (dK, dV)
    static constexpr int ROWCH = 2 * NK <= 8 ? 8 : 2 * NK <= 16 ? 16 : 32;
    static constexpr int ROWCHO = 2 * NKD <= 8 ? 8 : 16;
    static constexpr int SQ = BMQ * ROWCH * 8, SDO = BMQ * ROWCHO * 8;
    // masked, aligned instantiations also stage the step's 64 x 128 tile of a 16-bit matrix mask
    static constexpr bool MTILE = VEC_ && MASK_;
    static constexpr int MROWCH = BN / 8; // chunks per mask-tile row
    static constexpr int SM = MTILE ? BMQ * BN : 0;
    static constexpr int STAGE_ELEMS = SQ + SDO + 4 * BMQ + SM; // + lse * log2(e), -delta as fp32
    // direct loader: three stages, two steps ahead; with a mask tile (or the element-wise loader) two
    // stages, one step ahead
    static constexpr int AHEAD = (VEC_ && !MASK_) ? 2 : 1;
    static constexpr int NSTAGE = AHEAD + 1;
    static constexpr int LDS_BYTES = NSTAGE * STAGE_ELEMS * 2;
    // loader tasks: 8-channel chunks of Q, Q_b and dout, one query row each
    static constexpr int CQ = 2 * NKD, CR = 2 * NKR, CO = 2 * NKD;
    static constexpr int TASKS = BMQ * (CQ + CR + CO);
    static constexpr int PT = (TASKS + NTHREADS - 1) / NTHREADS;
    // one wave per SIMD (512 registers) where two would spill: large head dims in one pass, and
    // masked instantiations beyond the smallest (they also hold a step's mask values)
    static constexpr bool BIG = MASK_ && PART_ == 0 && (NDV_ >= 2 || NKD_ + NKR_ >= 5);
    // (aligned, unmasked, at most four operand steps, head dim <= 32: 164-168 registers, and the third wave is worth
    // more than the few that the allocator would otherwise take beyond 168)
    static constexpr int WAVES_EU = BIG ? 1 : (VEC_ && !MASK_ && PART_ == 0 && NK <= 4 && NDV == 1) ? 3 : ((NK <= 8 && NDV <= 2) || PART_ != 0) ? 2 : 1;
};

template <class C>
struct DkvStage { // register staging of one step: only the element-wise loader uses x
    u32x4_t x[C::VEC ? 1 : C::PT];
    float lse2, negd;
};

// task -> (kind, row, chunk): kind 0 = Q, 1 = Q_b, 2 = dout
template <class C>
__device__ __forceinline__ void dkv_task(int task, int &kind, int &row, int &ch) {
    row = task % C::BMQ;
    const int cc = task / C::BMQ;
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

// lse * log2(e) and -delta of query m0 + tid (as the preprocess step left them), for the first
// BMQ threads; rows past the end get P = exp2(-inf) = 0.
template <class C>
__device__ __forceinline__ void dkv_load_stats(DkvStage<C> &st, const float *lse2, const float *negd, int m0, int Lq,
                                               int tid) {
    if (tid < C::BMQ) {
        const bool ok = m0 + tid < Lq;
        const int q = ok ? m0 + tid : Lq - 1;
        const float l = lse2[q], d = negd[q];
        st.lse2 = ok ? l : INFINITY;
        st.negd = ok ? d : 0.f;
    }
}

template <class C>
__device__ __forceinline__ void dkv_store_stats(const DkvStage<C> &st, uint16_t *stage, int tid) {
    float *sStat = reinterpret_cast<float *>(stage + C::SQ + C::SDO);
    if (tid < C::BMQ) {
        sStat[tid] = st.lse2;
        sStat[C::BMQ + tid] = st.negd;
    }
}

// Element-wise loader (tensors that are not 16-byte aligned, d or r not a multiple of 8):
// clamped loads into registers, written to LDS after the step's arithmetic.
template <class C>
__device__ __forceinline__ void dkv_load_step(DkvStage<C> &st, const BwdArgs &a, const uint16_t *qbase,
                                              const uint16_t *qbbase, const uint16_t *dobase, int m0, int tid) {
#pragma unroll
    for (int i = 0; i < (C::VEC ? 1 : C::PT); ++i) {
        const int task = tid + i * C::NTHREADS;
        int kind, row, ch;
        dkv_task<C>(task, kind, row, ch);
        // one load per task: pick the tensor by lane (all three share the chunk geometry)
        const uint16_t *base = kind == 0 ? qbase : kind == 1 ? qbbase : dobase;
        const int64_t ld = kind == 0 ? a.q.ss : kind == 1 ? a.qb.ss : a.dout.ss;
        const int ncols = kind == 1 ? a.r : a.d;
        st.x[i] = u32x4_t{0u, 0u, 0u, 0u};
        if (C::TASKS % C::NTHREADS == 0 || task < C::TASKS)
            st.x[i] = load_chunk<false>(base, ld, m0 + row, a.Lq, ch * 8, ncols);
    }
}

template <class C>
__device__ __forceinline__ void dkv_store_step(const DkvStage<C> &st, const BwdArgs &a, uint16_t *stage, int tid) {
    uint16_t *sQ = stage, *sdO = sQ + C::SQ;
#pragma unroll
    for (int i = 0; i < (C::VEC ? 1 : C::PT); ++i) {
        const int task = tid + i * C::NTHREADS;
        int kind, row, ch;
        dkv_task<C>(task, kind, row, ch);
        // chunks in the zero padding of the channel dim are never written (LDS cleared once)
        if (task < C::TASKS && ch * 8 < (kind == 1 ? a.r : a.d)) {
            if (kind == 2)
                *reinterpret_cast<u32x4_t *>(sdO + swz_off<C::ROWCHO>(row, ch)) = st.x[i];
            else
                *reinterpret_cast<u32x4_t *>(sQ + swz_off<C::ROWCH>(row, (kind == 1 ? 2 * C::NKD : 0) + ch)) = st.x[i];
        }
    }
}

// Direct loader (16-byte aligned tensors, d and r multiples of 8): the [Q | Q_b] and dout
// tiles of a step plus its statistics rows, copied straight into an LDS stage.
template <class C>
struct DkvDirect {
    TileDma<C::BMQ, C::ROWCH, C::NWAVES, (C::NKR > 0)> q;
    TileDma<C::BMQ, C::ROWCHO, C::NWAVES, false> d;
    TileDma<C::BMQ, C::MROWCH, C::NWAVES, false> m; // mask tile (masked instantiations, 16-bit matrix masks)
    bool mtile;
    static constexpr int N = decltype(q)::NINST + decltype(d)::NINST;
    // waves 0 and 1 also fetch the step's lse * log2(e) and -delta rows (BMQ = 64 floats: one
    // 4-byte copy per lane)
    static constexpr int NS = 1;
    const float *stat; // this wave's statistics row of the (batch, head), or null
    int wave, lane;

    __device__ __forceinline__ void init(const BwdArgs &a, const uint16_t *qbase, const uint16_t *qbbase,
                                         const uint16_t *dobase, const float *lse2, const float *negd, int wave_,
                                         int lane_, int m0) {
        static_assert(C::BMQ <= 64, "one statistics row per copy instruction");
        wave = wave_;
        lane = lane_;
        stat = wave == 0 ? lse2 : wave == 1 ? negd : nullptr;
        q.init(qbase, a.q.ss, a.d, 2 * C::NKD, C::NKR > 0 ? qbbase : nullptr, C::NKR > 0 ? a.qb.ss : 0, a.r, wave, lane, m0,
               C::low_parts(a));
        d.init(dobase, a.dout.ss, a.d, C::ROWCHO, nullptr, 0, 0, wave, lane, m0);
        mtile = false;
    }

    // The workgroup's columns [n0, n0 + BN) of the (batch, head) mask matrix, 16-bit elements.
    __device__ __forceinline__ void init_mask(const BwdArgs &a, const uint8_t *mbase, int n0, int m0) {
        mtile = true;
        const int ncols = a.Lk - n0 < C::BN ? a.Lk - n0 : C::BN;
        m.init(reinterpret_cast<const uint16_t *>(mbase) + n0, a.mask.sm, ncols, C::MROWCH, nullptr, 0, 0, wave, lane, m0);
    }

    __device__ __forceinline__ void issue(const BwdArgs &a, uint16_t *stage, int m0, int Lq) {
        const uint32_t base = lds_addr_of(stage);
        q.issue(base, m0, Lq, a.q.ss, C::NKR > 0 ? a.qb.ss : 0, 2 * C::NKD);
        d.issue(base + 2 * C::SQ, m0, Lq, a.dout.ss, 0, C::ROWCHO);
        if (wave < 2 && lane < C::BMQ)
            lds_dma4(stat + min(m0 + lane, Lq - 1), base + 2 * (C::SQ + C::SDO) + wave * (4 * C::BMQ));
        if constexpr (C::MTILE) {
            if (mtile) m.issue(base + 2 * (C::SQ + C::SDO + 4 * C::BMQ), m0, Lq, a.mask.sm, 0, C::MROWCH);
        }
    }

    // Loads of this wave that may stay in flight when the data of the step before them is needed.
    template <bool KEEP>
    __device__ __forceinline__ void wait_older() const {
        if (!KEEP)
            wait_vmcnt<0>();
        else if (wave < 2)
            wait_vmcnt<N + NS>();
        else
            wait_vmcnt<N>();
    }

    // A last step that runs past the sequence fetched clamped rows: give them P = 0.
    __device__ __forceinline__ void fix_ragged(uint16_t *stage, int m0, int Lq, int tid) const {
        if (m0 + C::BMQ > Lq) {
            float *sStat = reinterpret_cast<float *>(stage + C::SQ + C::SDO);
            if (tid < C::BMQ && m0 + tid >= Lq) {
                sStat[tid] = INFINITY;
                sStat[C::BMQ + tid] = 0.f;
            }
            barrier_lds();
        }
    }
};

// Epilogue stores of the dk/dv kernel: dv and the dk part of the accumulators (BIAS = false, batch
// row `brow`) or their dk_bias part (BIAS = true, batch row `brow` of dk_bias).  Block n of acc_dk
// holds channels [32 n, 32 n + 32) of [dK | dK_b]; dK_b starts at channel 16 NKD (a multiple of 16,
// so a 16-channel half of a block is all dk or all dk_bias).
template <class T, class C, bool BIAS>
__device__ __forceinline__ void dkv_store(const BwdArgs &a, const f32x16_t (&acc_dv)[C::KBW][C::DO_DV ? C::NDV : 1],
                                          const f32x16_t (&acc_dk)[C::KBW][C::DO_DK ? C::MB1 - C::MB0 : 1], int brow, int h,
                                          int wk0, int c, int g) {
    const Tensor &t = BIAS ? a.dkb : a.dk;
    const float mul = BIAS ? 1.f : a.scale;
    const int ncols = BIAS ? a.r : a.d;
    constexpr int CH0 = BIAS ? 16 * C::NKD : 0;          // first channel of this part in [dK | dK_b]
    constexpr int END = BIAS ? 32 * C::MB : 16 * C::NKD; // one past its last channel
#pragma unroll
    for (int kb = 0; kb < C::KBW; ++kb) {
        int key = wk0 + kb * 32 + c;
        asm volatile("" : "+v"(key)); // (keeps the address arithmetic below the query loop: its registers are all taken)
        const bool ok = key < a.Lk;
        const int64_t krow = ok ? key : 0;
        if constexpr (!BIAS && C::DO_DV) {
            uint16_t *dvrow = const_cast<uint16_t *>(a.dv.ptr) + brow * a.dv.sb + h * a.dv.sh + krow * a.dv.ss;
#pragma unroll
            for (int n = 0; n < C::NDV; ++n)
                store_acc_rows<T, C::VEC>(dvrow + 32 * n, ok, a.dv.vec_ok, acc_dv[kb][n], 1.f, a.d - 32 * n, g);
        }
        if constexpr (C::DO_DK) {
            uint16_t *row = const_cast<uint16_t *>(t.ptr) + brow * t.sb + h * t.sh + krow * t.ss;
#pragma unroll
            for (int n = C::MB0; n < C::MB1; ++n) {
                const f32x16_t &blk = acc_dk[kb][n - C::MB0];
                const int lo_ch = 32 * n, hi_ch = 32 * n + 32;
                if (hi_ch <= CH0 || lo_ch >= END) continue; // the block has nothing of this part
                if (lo_ch >= CH0 && hi_ch <= END) {
                    store_acc_rows<T, C::VEC>(row + (lo_ch - CH0), ok, t.vec_ok, blk, mul, ncols - (lo_ch - CH0), g);
                } else { // the block straddles: channels [32 n, 32 n + 16) are dk, the rest dk_bias
                    f32x16_t half;
#pragma unroll
                    for (int v = 0; v < 8; ++v) {
                        half[v] = blk[BIAS ? 8 + v : v];
                        half[8 + v] = 0.f;
                    }
                    const int off = BIAS ? 0 : lo_ch;
                    store_acc_rows<T, C::VEC>(row + off, ok, t.vec_ok, half, mul, min(ncols - off, 16), g);
                }
            }
        }
    }
}

template <class T, class C>
__device__ __forceinline__ void bwd_dkv_body(const BwdArgs &a, int wg) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint16_t *stage0 = reinterpret_cast<uint16_t *>(smem);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 31, g = lane >> 5;

    // One workgroup serves `group` consecutive batch entries of its (head, key tile), one after the
    // other: dk and dv are written per entry, the dk_bias accumulators run on and are written once, as
    // row b / group of the dk_bias tensor (factors shared by the batch: their gradient is the sum).
    const int group = a.group > 1 ? a.group : 1;
    const int nbg = (a.B + group - 1) / group;
    const int total = a.ntiles_n * nbg * a.H;
    int bgh, tile_n; // (causal: the first key tile sees the most queries)
    work_order(wg, a.ntiles_n, total, a.causal, bgh, tile_n);
    const int bg = bgh / a.H, h = bgh % a.H;
    const int n0 = tile_n * C::BN;
    const int wk0 = n0 + wave * (32 * C::KBW); // first key of this wave

    {   // clear the stages once: the zero padding of the channel dimension is never rewritten
        u32x4_t *z = reinterpret_cast<u32x4_t *>(smem);
        for (int i = tid; i < C::LDS_BYTES / 16; i += C::NTHREADS) z[i] = u32x4_t{0u, 0u, 0u, 0u};
    }
    __syncthreads();

    f32x16_t acc_dv[C::KBW][C::DO_DV ? C::NDV : 1], acc_dk[C::KBW][C::DO_DK ? C::MB1 - C::MB0 : 1];
#pragma unroll
    for (int kb = 0; kb < C::KBW; ++kb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
#pragma unroll
            for (int n = 0; n < (C::DO_DV ? C::NDV : 1); ++n) acc_dv[kb][n][v] = 0.f;
#pragma unroll
            for (int n = 0; n < (C::DO_DK ? C::MB1 - C::MB0 : 1); ++n) acc_dk[kb][n][v] = 0.f;
        }

    // the key-side factor operand outlives a batch entry when the batch shares the factor (stride 0)
    u32x4_t kbreg[C::KBW][C::NKR > 0 ? C::NKR : 1];

    for (int bi = 0; bi < group; ++bi) {
    const int b = __builtin_amdgcn_readfirstlane(bg * group + bi); // (wave-uniform, and the compiler should know)
    if (b >= a.B) break;
    // (the lane's coordinates again, opaque to the compiler: what it derives from them is computed per batch
    // entry, as in a workgroup of its own, instead of being kept in registers across this loop)
    int tid_again = threadIdx.x;
    asm volatile("" : "+v"(tid_again));
    const int tid = tid_again, lane = tid & 63, c = lane & 31, g = lane >> 5;
    const int bh = b * a.H + h;

    const uint16_t *qbase = a.q.ptr + b * a.q.sb + h * a.q.sh;
    const uint16_t *kbase = a.k.ptr + b * a.k.sb + h * a.k.sh;
    const uint16_t *vbase = a.v.ptr + b * a.v.sb + h * a.v.sh;
    const uint16_t *dobase = a.dout.ptr + b * a.dout.sb + h * a.dout.sh;
    const uint16_t *qbbase = nullptr, *kbbase = nullptr;
    if constexpr (C::NKR > 0) {
        qbbase = a.qb.ptr + b * a.qb.sb + h * a.qb.sh;
        kbbase = a.kb.ptr + b * a.kb.sb + h * a.kb.sh;
    }
    // the preprocess step left -delta and lse * log2(e) in the scratch buffer
    const float *negd = a.delta + (int64_t)bh * a.Lq;
    const float *lse2 = a.delta + ((int64_t)a.B * a.H + bh) * a.Lq;
    const uint8_t *mbase = nullptr;
    if constexpr (C::MASK)
        mbase = reinterpret_cast<const uint8_t *>(a.mask.ptr) +
                (b * a.mask.sb + h * a.mask.sh) * (a.mask.is_f32 ? 4 : 2);

    const float to_log2 = C::FOLD ? a.scale * kLog2e : kLog2e; // the scores are in units of 1 / scale when folded

    // ---- key-side operands, resident in registers
    u32x4_t kreg[C::KBW][C::NK];  // B operand of S: this lane's key, channels 16t + 8g ..
    u32x4_t vreg[C::KBW][C::DO_DK ? C::NKD : 1]; // B operand of dP
#pragma unroll
    for (int kb = 0; kb < C::KBW; ++kb) {
        const int key = wk0 + kb * 32 + c;
#pragma unroll
        for (int t = 0; t < C::NK; ++t) {
            if (t < C::NKD)
                kreg[kb][t] = load_chunk<C::VEC>(kbase, a.k.ss, key, a.Lk, 16 * t + 8 * g, a.d);
            else if constexpr (C::NKR > 0) {
                u32x4_t &keep = kbreg[kb][t - C::NKD];
                if (bi == 0 || a.kb.sb != 0) {
                    const bool low = C::low_parts(a) && g == 1;
                    keep = load_chunk<C::VEC>(kbbase, a.kb.ss, key, a.Lk, low ? 0 : 16 * (t - C::NKD) + 8 * g, a.r);
                    if (C::FOLD && a.scale != 1.f) keep = fold_scale_chunk<T>(keep, 1.f / a.scale, C::low_parts(a), low);
                }
                kreg[kb][t] = keep;
            }
        }
        if constexpr (C::DO_DK) {
#pragma unroll
            for (int t = 0; t < C::NKD; ++t)
                vreg[kb][t] = load_chunk<C::VEC>(vbase, a.v.ss, key, a.Lk, 16 * t + 8 * g, a.d);
        }
        // (element v of block n is channel 32 n + 8 (v / 4) + 4 g + v % 4: below 16 NKD it belongs to dk)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
#pragma unroll
            for (int n = 0; n < (C::DO_DV ? C::NDV : 0); ++n) acc_dv[kb][n][v] = 0.f;
#pragma unroll
            for (int n = C::MB0; n < C::MB1; ++n)
                if (32 * n + 8 * (v >> 2) < 16 * C::NKD) acc_dk[kb][n - C::MB0][v] = 0.f;
        }
    }

    // causal: the first query step that can see this key tile (:498)
    const int step0 = a.causal ? n0 / C::BMQ : 0;
    const int nsteps = (a.Lq + C::BMQ - 1) / C::BMQ;

    // Step s is computed from stage (s - step0) % NSTAGE.  Direct loader: the tiles of step
    // s + AHEAD are requested at the top of step s; element-wise loader: step s + 1 goes through
    // registers.
    constexpr int AHEAD = C::AHEAD;
    DkvDirect<C> direct;
    DkvStage<C> st;
    if constexpr (C::VEC) {
        direct.init(a, qbase, qbbase, dobase, lse2, negd, wave, lane, step0 * C::BMQ);
        if constexpr (C::MTILE) {
            // a 16-bit matrix mask whose rows allow 16-byte copies goes through the LDS stages
            if (a.mask.type == 2 && a.mask.vec_ok && !a.mask.is_f32 && a.Lk % 8 == 0 && a.mask.sm % 8 == 0 && a.mask.sm < (1 << 24) &&
                reinterpret_cast<uintptr_t>(mbase) % 16 == 0)
                direct.init_mask(a, mbase, n0, step0 * C::BMQ);
        }
#pragma unroll
        for (int k = 0; k < AHEAD; ++k)
            if (step0 + k < nsteps) direct.issue(a, stage0 + k * C::STAGE_ELEMS, (step0 + k) * C::BMQ, a.Lq);
        // the first step's tiles must have landed; the second step's may still be in flight
        if (AHEAD == 2 && step0 + 1 < nsteps)
            direct.template wait_older<true>();
        else
            direct.template wait_older<false>();
    } else if (step0 < nsteps) {
        dkv_load_stats<C>(st, lse2, negd, step0 * C::BMQ, a.Lq, tid);
        dkv_store_stats<C>(st, stage0, tid);
        dkv_load_step<C>(st, a, qbase, qbbase, dobase, step0 * C::BMQ, tid);
        dkv_store_step<C>(st, a, stage0, tid);
    }
    __syncthreads();

    // Additive mask: the values of a step (16 per lane and 32 x 32 block) are requested one step
    // ahead and added by the FMA that applies the softmax scale.
    f32x16_t mk[C::MASK ? C::QBLK : 1][C::MASK ? C::KBW : 1], mkn[C::MASK ? C::QBLK : 1][C::MASK ? C::KBW : 1];
    auto load_mask = [&](f32x16_t (&dst)[C::MASK ? C::QBLK : 1][C::MASK ? C::KBW : 1], int m0) {
#pragma unroll
        for (int qb = 0; qb < C::QBLK; ++qb)
#pragma unroll
            for (int kb = 0; kb < C::KBW; ++kb)
                mask_block_queries<T>(a.mask, mbase, m0 + qb * 32, g, wk0 + kb * 32 + c, a.Lq, a.Lk, dst[qb][kb]);
    };
    const bool mtile = C::MTILE && direct.mtile; // else the mask values travel through registers
    if constexpr (C::MASK) {
        if (step0 < nsteps && !mtile) load_mask(mk, step0 * C::BMQ);
    }

    int cur = 0; // stage of the current step
    for (int step = step0; step < nsteps; ++step) {
        const int m0 = step * C::BMQ;
        const bool more = step + 1 < nsteps;
        const int nxt = cur == C::NSTAGE - 1 ? 0 : cur + 1;
        if constexpr (C::MASK) {
            if (more && !mtile) load_mask(mkn, m0 + C::BMQ);
        }
        if constexpr (C::VEC) {
            if (step + AHEAD < nsteps) {
                const int tgt = (cur + AHEAD) % C::NSTAGE; // the stage that step - 1 has left
                direct.issue(a, stage0 + tgt * C::STAGE_ELEMS, m0 + AHEAD * C::BMQ, a.Lq);
            }
            direct.fix_ragged(stage0 + cur * C::STAGE_ELEMS, m0, a.Lq, tid);
        } else if (more) {
            dkv_load_stats<C>(st, lse2, negd, m0 + C::BMQ, a.Lq, tid);
            dkv_load_step<C>(st, a, qbase, qbbase, dobase, m0 + C::BMQ, tid);
        }
        const uint16_t *sQ = stage0 + cur * C::STAGE_ELEMS;
        const uint16_t *sdO = sQ + C::SQ;
        const float *sStat = reinterpret_cast<const float *>(sdO + C::SDO);
        const uint16_t *sM = sdO + C::SDO + 4 * C::BMQ;

        const bool visible = !(a.causal && wk0 > m0 + C::BMQ - 1) && wk0 < a.Lk;
        if (visible) {
#pragma unroll
            for (int qb = 0; qb < C::QBLK; ++qb) {
                u32x4_t qa[C::NK], da[C::NKD];
#pragma unroll
                for (int t = 0; t < C::NK; ++t)
                    qa[t] = *reinterpret_cast<const u32x4_t *>(sQ + swz_off<C::ROWCH>(qb * 32 + c, 2 * t + g));
#pragma unroll
                for (int t = 0; t < (C::DO_DK ? C::NKD : 0); ++t)
                    da[t] = *reinterpret_cast<const u32x4_t *>(sdO + swz_off<C::ROWCHO>(qb * 32 + c, 2 * t + g));
                u32x4_t pp[C::KBW][2], pds[C::KBW][2]; // P and dS, packed, per 16-query step
#pragma unroll
                for (int kb = 0; kb < C::KBW; ++kb) {
                    const int key = wk0 + kb * 32 + c;
                    f32x16_t s, dp;
                    float lse2[16];
                    // per-register query statistics: query = qb*32 + 8*(v/4) + 4g + v%4
#pragma unroll
                    for (int bq = 0; bq < 4; ++bq) {
                        const f32x4_t l4 = *reinterpret_cast<const f32x4_t *>(sStat + qb * 32 + 8 * bq + 4 * g);
                        const f32x4_t d4 =
                            *reinterpret_cast<const f32x4_t *>(sStat + C::BMQ + qb * 32 + 8 * bq + 4 * g);
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            lse2[4 * bq + e] = l4[e];
                            dp[4 * bq + e] = d4[e];
                        }
                    }
#pragma unroll
                    for (int v = 0; v < 16; ++v) s[v] = 0.f;
#pragma unroll
                    for (int t = 0; t < C::NKD; ++t) s = T::mfma(qa[t], kreg[kb][t], s);
#pragma unroll
                    for (int t = 0; t < (C::DO_DK ? C::NKD : 0); ++t) dp = T::mfma(da[t], vreg[kb][t], dp);
                    f32x16_t mval; // additive mask of this block, added by the FMA that applies the scale
                    if constexpr (C::MASK) {
                        if (mtile) { // column `key`, rows in C-layout order: four transposing reads
                            if constexpr (C::MTILE) {
                                const int col = (wave * C::KBW + kb) * 32 + 16 * (c >> 4) + 4 * (c & 3);
#pragma unroll
                                for (int j = 0; j < 4; ++j) {
                                    const int row = qb * 32 + 8 * j + 4 * g + ((c & 15) >> 2);
                                    const u32x2_t x = lds_read_tr4(sM + swz_off<C::MROWCH>(row, col >> 3) + (col & 7));
                                    mval[4 * j + 0] = T::to_float((uint16_t)(x[0] & 0xffffu));
                                    mval[4 * j + 1] = T::to_float((uint16_t)(x[0] >> 16));
                                    mval[4 * j + 2] = T::to_float((uint16_t)(x[1] & 0xffffu));
                                    mval[4 * j + 3] = T::to_float((uint16_t)(x[1] >> 16));
                                }
                            }
                        } else {
                            mval = mk[C::MASK ? qb : 0][C::MASK ? kb : 0];
                        }
                    }
                    // the softmax scale multiplies the fp32 q k^T accumulator before the bias steps
                    // (one chain keeps this kernel at three waves per SIMD)
                    if constexpr (!C::FOLD) {
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            s[v] = C::MASK ? __builtin_fmaf(s[v], a.scale, mval[v]) : s[v] * a.scale;
                    }
#pragma unroll
                    for (int t = C::NKD; t < C::NK; ++t) s = T::mfma(qa[t], kreg[kb][t], s);
                    const bool edge = (wk0 + kb * 32 + 32 > a.Lk) || (a.causal && wk0 + kb * 32 + 31 > m0 + qb * 32);
                    if (edge) {
                        int query0 = m0 + qb * 32 + 4 * g;
                        asm volatile("" : "+v"(query0)); // (computed here, not kept in registers across the loop)
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const int query = query0 + 8 * (v >> 2) + (v & 3);
                            if (key >= a.Lk || (a.causal && key > query)) s[v] = -INFINITY;
                        }
                    }
#pragma unroll
                    for (int v = 0; v < 16; v += 2) {
                        const float p0 = fast_exp2(__builtin_fmaf(s[v], to_log2, -lse2[v]));
                        const float p1 = fast_exp2(__builtin_fmaf(s[v + 1], to_log2, -lse2[v + 1]));
                        if constexpr (C::DO_DV) pp[kb][v >> 3][(v & 7) >> 1] = T::pack2(p0, p1);
                        if constexpr (C::DO_DK) pds[kb][v >> 3][(v & 7) >> 1] = T::pack2(p0 * dp[v], p1 * dp[v + 1]);
                    }
                }
                // dV^T += dout^T P ; [dK|dK_b]^T += [Q|Q_b]^T dS  (contraction over this block's queries)
#pragma unroll
                for (int t = 0; t < 2; ++t) {
#pragma unroll
                    for (int n = 0; n < (C::DO_DV ? C::NDV : 0); ++n) {
                        const u32x4_t dot = lds_read_a_tr<C::ROWCHO>(sdO, qb * 32 + 16 * t, 32 * n, c, g);
#pragma unroll
                        for (int kb = 0; kb < C::KBW; ++kb) acc_dv[kb][n] = T::mfma(dot, pp[kb][t], acc_dv[kb][n]);
                    }
#pragma unroll
                    for (int n = C::MB0; n < C::MB1; ++n) {
                        const u32x4_t qt = lds_read_a_tr<C::ROWCH>(sQ, qb * 32 + 16 * t, 32 * n, c, g);
#pragma unroll
                        for (int kb = 0; kb < C::KBW; ++kb)
                            acc_dk[kb][n - C::MB0] = T::mfma(qt, pds[kb][t], acc_dk[kb][n - C::MB0]);
                    }
                }
            }
        }
        if constexpr (C::VEC) {
            // the next step's tiles must have landed; the one after may still be in flight
            if (AHEAD == 2 && step + AHEAD < nsteps)
                direct.template wait_older<true>();
            else
                direct.template wait_older<false>();
            barrier_lds();
        } else {
            if (more) {
                dkv_store_stats<C>(st, stage0 + nxt * C::STAGE_ELEMS, tid);
                dkv_store_step<C>(st, a, stage0 + nxt * C::STAGE_ELEMS, tid);
            }
            __syncthreads();
        }
        cur = nxt;
        if constexpr (C::MASK) {
#pragma unroll
            for (int qb = 0; qb < C::QBLK; ++qb)
#pragma unroll
                for (int kb = 0; kb < C::KBW; ++kb) mk[qb][kb] = mkn[qb][kb];
        }
    }

    // ---- epilogue of this batch entry: dv and dk (times scale) for this lane's keys
    dkv_store<T, C, false>(a, acc_dv, acc_dk, b, h, wk0, c, g);
    } // batch entries of the group

    // ---- dk_bias, summed over the group's batch entries
    if constexpr (C::NKR > 0 && C::DO_DK) {
        if (a.dkb.ptr) { // (null: the caller does not want the factor gradients)
            const int lane_end = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
            dkv_store<T, C, true>(a, acc_dv, acc_dk, bg, h, wk0, lane_end & 31, lane_end >> 5);
        }
    }
}

template <class T, class C>
__global__ __launch_bounds__(C::NTHREADS) __attribute__((amdgpu_waves_per_eu(C::WAVES_EU, C::WAVES_EU + 1))) void
bwd_dkv_kernel(const BwdArgs a) {
    bwd_dkv_body<T, C>(a, blockIdx.x);
}

template <class T, int NKD, int NKR, int NDV, bool VEC, bool MASK, int PART, bool FOLD, bool BG = true>
static hipError_t launch_dkv_part(const BwdArgs &a0, hipStream_t stream) {
    typedef DkvCfg<T, NKD, NKR, NDV, VEC, MASK, PART, FOLD, BG> C;
    BwdArgs a = a0;
    a.ntiles_n = (a.Lk + C::BN - 1) / C::BN;
    auto kern = bwd_dkv_kernel<T, C>;
    static KernelOnce once;
    const hipError_t e = allow_lds(kern, C::LDS_BYTES, once);
    if (e != hipSuccess) return e;
    const int group = a.group > 1 ? a.group : 1;
    return launch_flat(kern, (int64_t)a.ntiles_n * ((a.B + group - 1) / group) * a.H, C::NTHREADS, C::LDS_BYTES, stream, a);
}

// One pass, or (head dims above 64, aligned tensors) two or three passes that each keep a part
// of the accumulators.
template <class T, int NKD, int NKR, int NDV, bool VEC, bool MASK, bool FOLD = false>
static hipError_t launch_dkv_vec(const BwdArgs &a, hipStream_t stream) {
    if constexpr (NKD > 4 && VEC) {
        if constexpr (NKR <= 2 && !MASK) {
            // two passes, dv and then all of [dk | dk_bias]: 44 MFMAs per 32 x 32 block (three passes: 61;
            // dv with the lower half of dk, then the upper half: 52, measured 15-24 % slower than this)
            const hipError_t e = launch_dkv_part<T, NKD, NKR, NDV, VEC, MASK, 1, FOLD>(a, stream);
            if (e != hipSuccess) return e;
            return launch_dkv_part<T, NKD, NKR, NDV, VEC, MASK, 2, FOLD>(a, stream);
        } else { // larger ranks and masked calls: all of dk would spill at 256 registers
            hipError_t e = launch_dkv_part<T, NKD, NKR, NDV, VEC, MASK, 1, FOLD>(a, stream);
            if (e != hipSuccess) return e;
            e = launch_dkv_part<T, NKD, NKR, NDV, VEC, MASK, 3, FOLD>(a, stream);
            if (e != hipSuccess) return e;
        }
        return launch_dkv_part<T, NKD, NKR, NDV, VEC, MASK, 4, FOLD>(a, stream);
    } else {
        // head dim 32, aligned, unmasked, no dk_bias wanted: the instantiation without its products
        if constexpr (NKD == 2 && NKR > 0 && NKR <= 2 && VEC && !MASK) {
            if (!a.dkb.ptr) return launch_dkv_part<T, NKD, NKR, NDV, VEC, MASK, 0, FOLD, false>(a, stream);
        }
        return launch_dkv_part<T, NKD, NKR, NDV, VEC, MASK, 0, FOLD>(a, stream);
    }
}

} // namespace fb
#include "fb_bwd_dkv_lean.h"
namespace fb {

template <class T, int NKD, int NKR, int NDV>
static hipError_t launch_dkv_cfg(const BwdArgs &a, hipStream_t stream) {
    // the direct loader keeps the byte distance between two steps' rows in 32 bits
    const int64_t lim = (int64_t)1 << 24;
    const bool vec = a.q.vec_ok && a.k.vec_ok && a.v.vec_ok && a.dout.vec_ok && a.d % 8 == 0 &&
                     (a.r == 0 || (a.qb.vec_ok && a.kb.vec_ok && a.r % 8 == 0)) && a.q.ss < lim && a.dout.ss < lim &&
                     (a.r == 0 || a.qb.ss < lim);
    if (a.mask.type)
        return vec ? launch_dkv_vec<T, NKD, NKR, NDV, true, true>(a, stream)
                   : launch_dkv_vec<T, NKD, NKR, NDV, false, true>(a, stream);
    if constexpr (NKD == 2 && NKR <= 1 && NDV == 1) {
        // the streamlined kernel: same 128-key workgroups as the general one, and ahead of it at every
        // grid size (measured at B2 H4: 0.019 against 0.023 ms at L=1024, 0.063 against 0.082 at 4096,
        // 0.73 against 0.82 at 16384)
        if (dkv_streamlined(a)) {
            if constexpr (NKR > 0) {
                if (!a.dkb.ptr) return launch_dkv_lean<T, NKR, false>(a, stream);
            }
            return launch_dkv_lean<T, NKR>(a, stream);
        }
    }
    if constexpr (NKR <= 2) {
        if (vec && fold_scale_ok<T>(a.scale, a.r, a.Lq)) return launch_dkv_vec<T, NKD, NKR, NDV, true, false, true>(a, stream);
    }
    return vec ? launch_dkv_vec<T, NKD, NKR, NDV, true, false>(a, stream)
               : launch_dkv_vec<T, NKD, NKR, NDV, false, false>(a, stream);
}

template <class T, int NKD, int NDV>
static hipError_t launch_dkv_r(const BwdArgs &a, hipStream_t stream) {
    switch (nkr_of(a.r)) {
    case 0: return launch_dkv_cfg<T, NKD, 0, NDV>(a, stream);
    case 1: return launch_dkv_cfg<T, NKD, 1, NDV>(a, stream);
    case 2: return launch_dkv_cfg<T, NKD, 2, NDV>(a, stream);
    case 4: return launch_dkv_cfg<T, NKD, 4, NDV>(a, stream);
    default: return launch_dkv_cfg<T, NKD, 8, NDV>(a, stream);
    }
}

// Compiled once per (element type, head-dim bucket), see Makefile.  (FB_BODIES_ONLY: included by the unit that
// builds the mixed dq + dk/dv launch, which wants the kernels' bodies and not this entry point.)
#ifndef FB_BODIES_ONLY
#define FB_CAT2(a, b) a##b
#define FB_CAT(a, b) FB_CAT2(a, b)
hipError_t FB_CAT(launch_bwd_dkv_, FB_SUFFIX)(const BwdArgs &a, hipStream_t stream) {
    return launch_dkv_r<FB_T, FB_NKD, FB_NDV>(a, stream);
}
#endif

} // namespace fb
