// Backward FlashBias attention for gfx950, part 2 of 2: dq and dq_bias.
// Together with fb_bwd_dkv.hip this replaces _bwd_kernel of the reference
// (flash_bias/flash_bias_triton.py:450-1097); this kernel covers the dq / dq_bias updates of
// :725-817 without their global read-modify-write or atomics.
//
// Query-stationary, like the forward: one workgroup (4 waves) owns 256 consecutive queries of
// one (batch, head), each wave 64 of them (two 32-blocks); keys are streamed in tiles of 64
// through double-buffered LDS.  With lane = query, register = key (transposed products):
//
//   S^T  = [K | K_b] [scale Q | Q_b]^T        A = key rows (LDS),        B = query registers
//   dP^T = V dO^T                             A = value rows (LDS),      B = dO registers
//   P^T  = exp(S^T - lse)                     lse is a per-lane scalar
//   dS^T = P^T * (dP^T - delta)               -delta is the initial value of the dP^T accumulator
//   [dQ | dQ_b]^T += [K | K_b]^T dS^T         A = key tile read column-wise (LDS), B = dS^T registers
//
// so dS^T goes from the accumulator layout straight into the next MFMA and [dQ | dQ_b]^T stays
// in registers for the whole key loop: each output element is written exactly once, in a fixed
// summation order (bit-reproducible).  The softmax scale multiplies the fp32 q k^T accumulator as
// in the forward; dq is multiplied by the scale in the epilogue, dq_bias is not (:728-732).
#include "fb_kernels.h"

namespace fb {

// QB2_: allow two query blocks per wave (the launcher turns it off for small grids).
// FOLD_: the scores are scale * (q k^T + (q_b / scale) k_b^T), one MFMA chain and no FMA per
// score for the scale (the launcher says when that is exact).
// KB1_: 32-key tiles (half the LDS per stage: two workgroups per CU at head dims above 64).
// BG_: also accumulate dq_bias (false: the caller does not want the factor gradients; the accumulator blocks that
// hold nothing but dq_bias are then left out of the products).
template <class T, int NKD_, int NKR_, bool VEC_, bool MASK_, bool QB2_ = true, bool FOLD_ = false, bool KB1_ = false,
          bool BG_ = true>
struct DqCfg {
    static constexpr bool FOLD = FOLD_;
    static_assert(!FOLD_ || (VEC_ && !MASK_), "folded scale: direct loader, no additive mask");
    // folded scale with r <= 8: the K_b columns 8..15 of a tile hold a second copy of k_b, the
    // partner of the low parts of q_b / scale in the query operand
    static __device__ __forceinline__ bool low_parts(const BwdArgs &a) { return FOLD_ && NKR_ == 1 && a.r <= 8 && a.scale != 1.f; }
    static constexpr int NKD = NKD_, NKR = NKR_;
    static constexpr bool VEC = VEC_, MASK = MASK_;
    static constexpr int NWAVES = 4, NTHREADS = 64 * NWAVES;
    static constexpr int NK = NKD + NKR;
    static constexpr int MB = (NK + 1) / 2; // 32-row blocks of [dQ | dQ_b]^T
    static constexpr int MBE = BG_ ? MB : (NKD + 1) / 2; // ... of which the key loop accumulates the first MBE
    static constexpr int QBLK = (QB2_ && NK <= 3 && !MASK_) ? 2 : 1; // the mask values need the registers of the second block
    static constexpr int BM = NWAVES * QBLK * 32;
    static constexpr int KBLK = KB1_ ? 1 : 2, BN = 32 * KBLK;
    static constexpr bool ONECHAIN = KB1_ && !MASK_; // scale between the d steps and the r steps of one MFMA chain
    // sK row: [K | K_b] of one key in ROWCH swizzled 16-byte chunks; the one copy is read
    // row-wise for S^T and column-wise for [dQ | dQ_b]^T
    static constexpr int ROWCH = 2 * NK <= 8 ? 8 : 2 * NK <= 16 ? 16 : 32;
    static constexpr int ROWCHV = 2 * NKD <= 8 ? 8 : 16; // sV row: V of one key, same chunk swizzle
    static constexpr int SK = BN * ROWCH * 8, SV = BN * ROWCHV * 8;
    // masked, aligned instantiations also stage the tile's BM x BN block of a 16-bit matrix mask
    static constexpr bool MTILE = VEC_ && MASK_;
    static constexpr int MROWCH = BN / 8; // chunks per mask-tile row
    static constexpr int SM = MTILE ? BM * BN : 0;
    static constexpr int STAGE = SK + SV + SM;
    // direct loader: three stages, two tiles ahead; with a mask tile (or the element-wise loader)
    // two stages, one ahead
    static constexpr int AHEAD = (VEC_ && !MASK_) ? 2 : 1;
    static constexpr int NSTAGE = AHEAD + 1;
    static constexpr int LDS_BYTES = NSTAGE * STAGE * 2;
    // loader: 8-channel chunks of K, K_b and V, one key row each
    static constexpr int CD = 2 * NKD, CR = 2 * NKR;
    static constexpr int K_TASKS = BN * (CD + CR), V_TASKS = BN * CD;
    static constexpr int K_PT = (K_TASKS + NTHREADS - 1) / NTHREADS;
    static constexpr int V_PT = (V_TASKS + NTHREADS - 1) / NTHREADS;
    static constexpr int WAVES_EU = (NK <= (MASK_ ? 6 : 8) || KB1_) ? 2 : 1;
};

template <class C>
struct DqStage { // register staging of one tile, used by the element-wise loader only
    u32x4_t k[C::VEC ? 1 : C::K_PT];
    u32x4_t v[C::VEC ? 1 : C::V_PT];
};

// Element-wise loader (tensors that are not 16-byte aligned, d or r not a multiple of 8):
// clamped loads into registers, written to LDS after the tile's arithmetic.
template <class C>
struct DqLoader {
    // K task: one key row x one 8-channel chunk of K (chunk < CD) or K_b
    __device__ static __forceinline__ void ktask(int task, int &row, int &ch, bool &is_b) {
        row = task % C::BN;
        const int cc = task / C::BN;
        is_b = cc >= C::CD;
        ch = is_b ? cc - C::CD : cc;
    }

    __device__ static __forceinline__ void load(DqStage<C> &st, const BwdArgs &a, const uint16_t *kbase,
                                                const uint16_t *kbbase, const uint16_t *vbase, int n0, int tid) {
#pragma unroll
        for (int i = 0; i < (C::VEC ? 1 : C::K_PT); ++i) {
            const int task = tid + i * C::NTHREADS;
            int row, ch;
            bool is_b;
            ktask(task, row, ch, is_b);
            const uint16_t *base = is_b ? kbbase : kbase;
            const int64_t ld = is_b ? a.kb.ss : a.k.ss;
            const int ncols = is_b ? a.r : a.d;
            st.k[i] = u32x4_t{0u, 0u, 0u, 0u};
            if (C::K_TASKS % C::NTHREADS == 0 || task < C::K_TASKS)
                st.k[i] = load_chunk<false>(base, ld, n0 + row, a.Lk, ch * 8, ncols);
        }
#pragma unroll
        for (int i = 0; i < (C::VEC ? 1 : C::V_PT); ++i) {
            const int task = tid + i * C::NTHREADS;
            st.v[i] = u32x4_t{0u, 0u, 0u, 0u};
            if (C::V_TASKS % C::NTHREADS == 0 || task < C::V_TASKS)
                st.v[i] = load_chunk<false>(vbase, a.v.ss, n0 + task % C::BN, a.Lk, (task / C::BN) * 8, a.d);
        }
    }

    // chunks in the zero padding of the channel dimension are never written (LDS cleared once)
    __device__ static __forceinline__ void store(const DqStage<C> &st, const BwdArgs &a, uint16_t *stage, int tid) {
        uint16_t *sK = stage, *sV = sK + C::SK;
#pragma unroll
        for (int i = 0; i < (C::VEC ? 1 : C::K_PT); ++i) {
            const int task = tid + i * C::NTHREADS;
            int row, ch;
            bool is_b;
            ktask(task, row, ch, is_b);
            if (task < C::K_TASKS && ch * 8 < (is_b ? a.r : a.d))
                *reinterpret_cast<u32x4_t *>(sK + swz_off<C::ROWCH>(row, (is_b ? 2 * C::NKD : 0) + ch)) = st.k[i];
        }
#pragma unroll
        for (int i = 0; i < (C::VEC ? 1 : C::V_PT); ++i) {
            const int task = tid + i * C::NTHREADS;
            if (task < C::V_TASKS && (task / C::BN) * 8 < a.d)
                *reinterpret_cast<u32x4_t *>(sV + swz_off<C::ROWCHV>(task % C::BN, task / C::BN)) = st.v[i];
        }
    }
};

// Direct loader (16-byte aligned tensors, d and r multiples of 8): the [K | K_b] and V tiles of
// a key tile, copied straight into an LDS stage.
template <class C>
struct DqDirect {
    TileDma<C::BN, C::ROWCH, C::NWAVES, (C::NKR > 0)> k;
    TileDma<C::BN, C::ROWCHV, C::NWAVES, false> v;
    TileDma<C::BM, C::MROWCH, C::NWAVES, false> m; // mask tile (masked instantiations, 16-bit matrix masks)
    bool mtile = false;
    static constexpr int N = decltype(k)::NINST + decltype(v)::NINST;

    __device__ __forceinline__ void init(const BwdArgs &a, const uint16_t *kbase, const uint16_t *kbbase,
                                         const uint16_t *vbase, int wave, int lane) {
        k.init(kbase, a.k.ss, a.d, 2 * C::NKD, C::NKR > 0 ? kbbase : nullptr, C::NKR > 0 ? a.kb.ss : 0, a.r, wave, lane, 0,
               C::low_parts(a));
        v.init(vbase, a.v.ss, a.d, C::ROWCHV, nullptr, 0, 0, wave, lane, 0);
    }

    // Rows [m0, m0 + BM) of the (batch, head) mask matrix, 16-bit elements; the tiles follow each
    // other along the rows (BN keys at a time).
    __device__ __forceinline__ void init_mask(const BwdArgs &a, const uint8_t *mbase, int m0, int wave, int lane) {
        mtile = true;
        m0_ = m0;
        m.init(reinterpret_cast<const uint16_t *>(mbase), a.mask.sm, C::BN, C::MROWCH, nullptr, 0, 0, wave, lane, m0);
    }

    __device__ __forceinline__ void issue(const BwdArgs &a, uint16_t *stage, int n0, int Lk) {
        const uint32_t base = lds_addr_of(stage);
        k.issue(base, n0, Lk, a.k.ss, C::NKR > 0 ? a.kb.ss : 0, 2 * C::NKD);
        v.issue(base + 2 * C::SK, n0, Lk, a.v.ss, 0, C::ROWCHV);
        if constexpr (C::MTILE) { // full tiles only: a ragged last tile takes the element path
            if (mtile && n0 + C::BN <= Lk)
                m.issue_step(base + 2 * (C::SK + C::SV), m0_, a.Lq, a.mask.sm, 0, C::MROWCH, 2 * C::BN, 0);
        }
    }
    int m0_ = 0; // first query of the workgroup (set by init_mask)
};

// Epilogue stores of the dq kernel: the dq part (BIAS = false, times the softmax scale, batch row
// `brow` of dq) or the dq_bias part (BIAS = true, batch row `brow` of dq_bias) of the accumulators.
// Block n holds channels [32 n, 32 n + 32) of [dQ | dQ_b]; dQ_b starts at channel 16 NKD (a multiple
// of 16, so a 16-channel half of a block is all dq or all dq_bias).
template <class T, class C, bool BIAS>
__device__ __forceinline__ void dq_store(const BwdArgs &a, const f32x16_t (&acc)[C::QBLK][C::MB], int brow, int h, int wq0,
                                         int c, int g) {
    const Tensor &t = BIAS ? a.dqb : a.dq;
    const float mul = BIAS ? 1.f : a.scale;
    const int ncols = BIAS ? a.r : a.d;
    constexpr int CH0 = BIAS ? 16 * C::NKD : 0; // first channel of this part in [dQ | dQ_b]
#pragma unroll
    for (int qb = 0; qb < C::QBLK; ++qb) {
        int query = wq0 + qb * 32 + c;
        asm volatile("" : "+v"(query)); // (keeps the address arithmetic below the key loop: its registers are all taken)
        const bool ok = query < a.Lq;
        uint16_t *row = const_cast<uint16_t *>(t.ptr) + brow * t.sb + h * t.sh + (int64_t)(ok ? query : 0) * t.ss;
#pragma unroll
        for (int n = 0; n < C::MB; ++n) {
            constexpr int END = BIAS ? 32 * C::MB : 16 * C::NKD; // one past the last channel of this part
            const int lo_ch = 32 * n, hi_ch = 32 * n + 32;
            if (hi_ch <= CH0 || lo_ch >= END) continue; // the block has nothing of this part
            if (lo_ch >= CH0 && hi_ch <= END) {
                store_acc_rows<T, C::VEC>(row + (lo_ch - CH0), ok, t.vec_ok, acc[qb][n], mul, ncols - (lo_ch - CH0), g);
            } else { // the block straddles: channels [32 n, 32 n + 16) are dq, the rest dq_bias
                f32x16_t half;
#pragma unroll
                for (int v = 0; v < 8; ++v) {
                    half[v] = acc[qb][n][BIAS ? 8 + v : v];
                    half[8 + v] = 0.f;
                }
                const int off = BIAS ? 0 : lo_ch;
                store_acc_rows<T, C::VEC>(row + off, ok, t.vec_ok, half, mul, min(ncols - off, 16), g);
            }
        }
    }
}

// The whole dq / dq_bias computation of one workgroup; the kernel below is nothing else.
template <class T, class C>
__device__ __forceinline__ void bwd_dq_body(const BwdArgs &a, int wg) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint16_t *stage0 = reinterpret_cast<uint16_t *>(smem);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 31, g = lane >> 5;

    // One workgroup serves `group` consecutive batch entries of its (head, query tile), one after the
    // other: dq is written per entry, the dq_bias accumulators run on and are written once, as row
    // b / group of the dq_bias tensor (factors shared by the batch: their gradient is the sum).
    const int group = a.group > 1 ? a.group : 1;
    const int nbg = (a.B + group - 1) / group;
    const int total = a.ntiles_m * nbg * a.H;
    int bgh, tile_m;
    work_order(wg, a.ntiles_m, total, a.causal, bgh, tile_m);
    if (a.causal) tile_m = a.ntiles_m - 1 - tile_m; // the last query tile sees the most keys
    const int bg = bgh / a.H, h = bgh % a.H;
    const int m0 = tile_m * C::BM;
    const int wq0 = m0 + wave * (32 * C::QBLK);

    {   // clear the stages once: the zero padding of the channel dimension is never rewritten
        u32x4_t *z = reinterpret_cast<u32x4_t *>(smem);
        for (int i = tid; i < C::LDS_BYTES / 16; i += C::NTHREADS) z[i] = u32x4_t{0u, 0u, 0u, 0u};
    }
    __syncthreads();

    f32x16_t acc[C::QBLK][C::MB];
#pragma unroll
    for (int qb = 0; qb < C::QBLK; ++qb)
#pragma unroll
        for (int n = 0; n < C::MB; ++n)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[qb][n][v] = 0.f;
    int turn = __builtin_amdgcn_readfirstlane(cu_slot());
    // the query-side factor operand outlives a batch entry when the batch shares the factor (stride 0)
    u32x4_t qbr[C::QBLK][C::NKR > 0 ? C::NKR : 1];

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
    const uint8_t *mbase = nullptr;
    if constexpr (C::MASK)
        mbase = reinterpret_cast<const uint8_t *>(a.mask.ptr) +
                (b * a.mask.sb + h * a.mask.sh) * (a.mask.is_f32 ? 4 : 2);

    // ---- query-side operands, resident in registers
    u32x4_t qr[C::QBLK][C::NKD];
    u32x4_t dor[C::QBLK][C::NKD];
    float lse2[C::QBLK]; // lse * log2(e) of this lane's queries
    // -delta of this lane's query in all 16 registers of an accumulator block: the initial value
    // of every dP^T chain (lane = query, so it is the same for every key), no add per score
    f32x16_t negd[C::QBLK];
#pragma unroll
    for (int qb = 0; qb < C::QBLK; ++qb) {
        const int query = wq0 + qb * 32 + c;
#pragma unroll
        for (int t = 0; t < C::NKD; ++t) {
            qr[qb][t] = load_chunk<C::VEC>(qbase, a.q.ss, query, a.Lq, 16 * t + 8 * g, a.d);
            dor[qb][t] = load_chunk<C::VEC>(dobase, a.dout.ss, query, a.Lq, 16 * t + 8 * g, a.d);
        }
        if constexpr (C::NKR > 0) {
            if (bi == 0 || a.qb.sb != 0) {
#pragma unroll
                for (int t = 0; t < C::NKR; ++t) {
                    const bool low = C::low_parts(a) && g == 1;
                    qbr[qb][t] = load_chunk<C::VEC>(qbbase, a.qb.ss, query, a.Lq, low ? 0 : 16 * t + 8 * g, a.r);
                    if (C::FOLD && a.scale != 1.f) qbr[qb][t] = fold_scale_chunk<T>(qbr[qb][t], 1.f / a.scale, C::low_parts(a), low);
                }
            }
        }
        const bool ok = query < a.Lq;
        const int64_t sidx = (int64_t)bh * a.Lq + (ok ? query : a.Lq - 1);
        float nd, l2;
        if (a.stats_here) {
            // delta = rowsum(o * dO) of this lane's query (flash_bias_triton.py:358-400) from the dO
            // chunks it holds and the same chunks of o; the other half of the channels is with lane ^ 32.
            // -delta and lse * log2(e) also go to the scratch buffer, for the dk/dv kernel that follows.
            const uint16_t *obase = a.o.ptr + b * a.o.sb + h * a.o.sh;
            // (summed in the order of the preprocess kernel: per 8-channel chunk, then a pairwise tree
            // over the chunks, so that both ways of running the backward give the same bits)
            float cs[C::NKD];
#pragma unroll
            for (int t = 0; t < C::NKD; ++t) {
                const u32x4_t oc = load_chunk<C::VEC>(obase, a.o.ss, query, a.Lq, 16 * t + 8 * g, a.d);
                float acc1 = 0.f;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    acc1 = __builtin_fmaf(T::to_float((uint16_t)(oc[e] & 0xffffu)),
                                          T::to_float((uint16_t)(dor[qb][t][e] & 0xffffu)), acc1);
                    acc1 = __builtin_fmaf(T::to_float((uint16_t)(oc[e] >> 16)), T::to_float((uint16_t)(dor[qb][t][e] >> 16)),
                                          acc1);
                }
                cs[t] = acc1 + __shfl_xor(acc1, 32, 64); // chunks 2t and 2t + 1
            }
#pragma unroll
            for (int m = 1; m < C::NKD; m <<= 1)
#pragma unroll
                for (int t = 0; t + m < C::NKD; t += 2 * m) cs[t] += cs[t + m];
            const float part = cs[0];
            nd = ok ? -part : 0.f;
            l2 = ok ? a.lse[sidx] * kLog2e : INFINITY;
            if (ok && g == 0) {
                const int64_t rows = (int64_t)a.B * a.H * a.Lq;
                a.delta[sidx] = nd;
                a.delta[rows + sidx] = l2;
                if (a.stat_chunks) reinterpret_cast<u32x4_t *>(a.delta + stat_offset(rows))[sidx] = stat_chunk<T>(nd, l2);
            }
        } else {
            // the preprocess step left -delta and lse * log2(e) in the scratch buffer
            l2 = ok ? a.delta[(int64_t)a.B * a.H * a.Lq + sidx] : INFINITY;
            nd = ok ? a.delta[sidx] : 0.f;
        }
        lse2[qb] = l2; // rows past the end: P = exp2(-inf) = 0
#pragma unroll
        for (int v = 0; v < 16; ++v) negd[qb][v] = nd;
        // (element v of block n is channel 32 n + 8 (v / 4) + 4 g + v % 4: below 16 NKD it belongs to dq)
#pragma unroll
        for (int n = 0; n < C::MB; ++n)
#pragma unroll
            for (int v = 0; v < 16; ++v)
                if (32 * n + 8 * (v >> 2) < 16 * C::NKD) acc[qb][n][v] = 0.f;
    }

    const float to_log2 = C::FOLD ? a.scale * kLog2e : kLog2e; // the scores are in units of 1 / scale when folded

    int k_end = a.Lk;
    if (a.causal && m0 + C::BM < k_end) k_end = m0 + C::BM; // keys past the last query are hidden
    const int ntiles_k = (k_end + C::BN - 1) / C::BN;

    // Tile t is computed from stage t % NSTAGE.  Direct loader: tile t + 2 is requested at the top
    // of tile t; element-wise loader: tile t + 1 goes through registers.  Keys past the end of a
    // ragged last tile hold copies of the last key; their scores are set to -inf below.
    constexpr int AHEAD = C::AHEAD;
    DqDirect<C> direct;
    DqStage<C> st;
    if constexpr (C::VEC) {
        direct.init(a, kbase, kbbase, vbase, wave, lane);
        if constexpr (C::MTILE) {
            // a 16-bit matrix mask whose rows allow 16-byte copies goes through the LDS stages
            if (a.mask.vec_ok && !a.mask.is_f32 && a.Lk % 8 == 0 && a.mask.sm % 8 == 0 && // (a vector mask: row stride 0)
                a.mask.sm < (1 << 24) && reinterpret_cast<uintptr_t>(mbase) % 16 == 0)
                direct.init_mask(a, mbase, m0, wave, lane);
        }
#pragma unroll
        for (int k = 0; k < AHEAD; ++k)
            if (k < ntiles_k) direct.issue(a, stage0 + k * C::STAGE, k * C::BN, a.Lk);
        if (AHEAD == 2 && 1 < ntiles_k)
            wait_vmcnt<DqDirect<C>::N>(); // the first tile has landed, the second may be in flight
        else
            wait_vmcnt<0>();
    } else {
        DqLoader<C>::load(st, a, kbase, kbbase, vbase, 0, tid);
        DqLoader<C>::store(st, a, stage0, tid);
    }
    __syncthreads();

    int cur = 0; // stage of the current tile
    take_turn(turn, a.slots);
    for (int it = 0; it < ntiles_k; ++it) {
        const int n0 = it * C::BN;
        const bool more = it + 1 < ntiles_k;
        const int nxt = cur == C::NSTAGE - 1 ? 0 : cur + 1;
        if constexpr (C::VEC) {
            if (it + AHEAD < ntiles_k)
                direct.issue(a, stage0 + ((cur + AHEAD) % C::NSTAGE) * C::STAGE, n0 + AHEAD * C::BN, a.Lk);
        } else if (more) {
            DqLoader<C>::load(st, a, kbase, kbbase, vbase, n0 + C::BN, tid);
        }

        const uint16_t *sK = stage0 + cur * C::STAGE, *sV = sK + C::SK;
        const bool visible = !(a.causal && n0 > wq0 + 32 * C::QBLK - 1) && wq0 < a.Lq;
        if (visible) {
#pragma unroll
            for (int kb = 0; kb < C::KBLK; ++kb) {
                u32x4_t ka[C::NK], va[C::NKD];
#pragma unroll
                for (int t = 0; t < C::NK; ++t)
                    ka[t] = *reinterpret_cast<const u32x4_t *>(sK + swz_off<C::ROWCH>(kb * 32 + c, 2 * t + g));
#pragma unroll
                for (int t = 0; t < C::NKD; ++t)
                    va[t] = *reinterpret_cast<const u32x4_t *>(sV + swz_off<C::ROWCHV>(kb * 32 + c, 2 * t + g));
                u32x4_t dsp[C::QBLK][2]; // dS^T, packed, per 16-key step
#pragma unroll
                for (int qb = 0; qb < C::QBLK; ++qb) {
                    f32x16_t s, dp;
                    const int query = wq0 + qb * 32 + c;
#pragma unroll
                    for (int v = 0; v < 16; ++v) s[v] = 0.f;
                    // q k^T and q_b k_b^T: two independent MFMA chains, joined by one FMA per score
                    // that applies the softmax scale in fp32 (:638-641); an additive mask is the
                    // initial value of the bias chain
                    if constexpr (C::NKR > 0 || C::MASK) {
                        f32x16_t sb;
                        if constexpr (C::MASK) {
                            if (C::MTILE && direct.mtile && n0 + C::BN <= a.Lk) {
                                // this lane's query row of the staged tile, keys in C-layout order
                                const uint16_t *sM = sV + C::SV;
                                const int row = wave * 32 + c;
#pragma unroll
                                for (int j = 0; j < 4; ++j) {
                                    const u32x2_t x = *reinterpret_cast<const u32x2_t *>(
                                        sM + swz_off<C::MROWCH>(row, 4 * kb + j) + 4 * g);
                                    sb[4 * j + 0] = T::to_float((uint16_t)(x[0] & 0xffffu));
                                    sb[4 * j + 1] = T::to_float((uint16_t)(x[0] >> 16));
                                    sb[4 * j + 2] = T::to_float((uint16_t)(x[1] & 0xffffu));
                                    sb[4 * j + 3] = T::to_float((uint16_t)(x[1] >> 16));
                                }
                            } else {
                                const uint8_t *mrow =
                                    mbase + (a.mask.type == 2 ? (int64_t)min(query, a.Lq - 1) * a.mask.sm : 0) *
                                                (a.mask.is_f32 ? 4 : 2);
                                mask_block_keys<T>(a.mask, mrow, n0 + kb * 32, g, a.Lk, sb);
                            }
                        } else {
#pragma unroll
                            for (int v = 0; v < 16; ++v) sb[v] = 0.f;
                        }
#pragma unroll
                        for (int t = 0; t < C::NKD; ++t) s = T::mfma(ka[t], qr[qb][t], s);
                        if constexpr (C::ONECHAIN && !C::FOLD) { // (a second accumulator would spill here)
#pragma unroll
                            for (int v = 0; v < 16; ++v) s[v] *= a.scale;
                        }
#pragma unroll
                        for (int t = C::NKD; t < C::NK; ++t) {
                            if constexpr (C::FOLD || C::ONECHAIN)
                                s = T::mfma(ka[t], qbr[qb][t - C::NKD], s);
                            else
                                sb = T::mfma(ka[t], qbr[qb][t - C::NKD], sb);
                        }
                        if constexpr (!C::FOLD && !C::ONECHAIN) {
#pragma unroll
                            for (int v = 0; v < 16; ++v) s[v] = __builtin_fmaf(s[v], a.scale, sb[v]);
                        }
                    } else {
#pragma unroll
                        for (int t = 0; t < C::NKD; ++t) s = T::mfma(ka[t], qr[qb][t], s);
                        if constexpr (!C::FOLD) {
#pragma unroll
                            for (int v = 0; v < 16; ++v) s[v] *= a.scale;
                        }
                    }
#pragma unroll
                    for (int t = 0; t < C::NKD; ++t) dp = T::mfma(va[t], dor[qb][t], t == 0 ? negd[qb] : dp);
                    // (bitwise on purpose: a short-circuit evaluation puts a small block of scalar code between the last
                    // MFMA and the branch, which the branch's other edge skips, and the compiler then counts the
                    // wait states between an MFMA and the first reader of its result along the longer path only)
                    const bool edge = (n0 + kb * 32 + 32 > a.Lk) | ((a.causal != 0) & (n0 + kb * 32 + 31 > wq0 + qb * 32));
                    if (edge) {
                        int key0 = n0 + kb * 32 + 4 * g;
                        asm volatile("" : "+v"(key0)); // (computed here, not kept in 16 registers across the loop)
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const int key = key0 + 8 * (v >> 2) + (v & 3);
                            if (key >= a.Lk || (a.causal && key > query)) s[v] = -INFINITY;
                        }
                    }
#pragma unroll
                    for (int v = 0; v < 16; v += 2) {
                        const float p0 = fast_exp2(__builtin_fmaf(s[v], to_log2, -lse2[qb]));
                        const float p1 = fast_exp2(__builtin_fmaf(s[v + 1], to_log2, -lse2[qb]));
                        dsp[qb][v >> 3][(v & 7) >> 1] = T::pack2(p0 * dp[v], p1 * dp[v + 1]);
                    }
                }
                // [dQ | dQ_b]^T += [K | K_b]^T dS^T over this block's 32 keys
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int n = 0; n < C::MBE; ++n) {
                        const u32x4_t kt = lds_read_a_tr<C::ROWCH>(sK, kb * 32 + 16 * t, 32 * n, c, g);
#pragma unroll
                        for (int qb = 0; qb < C::QBLK; ++qb) acc[qb][n] = T::mfma(kt, dsp[qb][t], acc[qb][n]);
                    }
            }
        }
        if constexpr (C::VEC) {
            if (AHEAD == 2 && it + AHEAD < ntiles_k)
                wait_vmcnt<DqDirect<C>::N>(); // the next tile has landed, the one after may be in flight
            else
                wait_vmcnt<0>();
            barrier_lds();
        } else {
            if (more) DqLoader<C>::store(st, a, stage0 + nxt * C::STAGE, tid);
            __syncthreads();
        }
        cur = nxt;
        take_turn(turn, a.slots); // (next to the barrier: the compiler moves nothing across either)
    }

    // ---- epilogue of this batch entry: dq = scale * acc rows [0, d)
    dq_store<T, C, false>(a, acc, b, h, wq0, c, g);
    } // batch entries of the group

    // ---- dq_bias = acc rows [16 NKD, 16 NKD + r), summed over the group's batch entries
    if constexpr (C::NKR > 0) {
        if (a.dqb.ptr) { // (null: the caller does not want the factor gradients)
            const int lane_end = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
            dq_store<T, C, true>(a, acc, bg, h, wq0, lane_end & 31, lane_end >> 5);
        }
    }
}

// (One query block per wave and at most four operand steps fit 168 registers: a third wave per SIMD, which the
// upper bound of the attribute has to allow; 768 x 4 rows of 768 tokens at rank 32: 0.80 -> 0.71 ms.)
template <class T, class C>
__global__ __launch_bounds__(C::NTHREADS) __attribute__((amdgpu_waves_per_eu(C::WAVES_EU + (C::QBLK == 1 && C::NK <= 4 && C::VEC && !C::MASK ? 1 : 0), C::WAVES_EU + (C::QBLK == 1 && C::NK <= 4 ? 1 : 0)))) void
bwd_dq_kernel(const BwdArgs a) {
    bwd_dq_body<T, C>(a, blockIdx.x);
}

template <class T, int NKD, int NKR, bool VEC, bool MASK, bool QB2, bool FOLD, bool KB1, bool BG>
static hipError_t launch_dq_qb_bg(const BwdArgs &a0, hipStream_t stream) {
    typedef DqCfg<T, NKD, NKR, VEC, MASK, QB2, FOLD, KB1, BG> C;
    BwdArgs a = a0;
    a.ntiles_m = (a.Lq + C::BM - 1) / C::BM;
    auto kern = bwd_dq_kernel<T, C>;
    static KernelOnce once;
    const hipError_t e = allow_lds(kern, C::LDS_BYTES, once);
    if (e != hipSuccess) return e;
    const int group = a.group > 1 ? a.group : 1;
    const int64_t total = (int64_t)a.ntiles_m * ((a.B + group - 1) / group) * a.H;
    a.slots = slots_per_cu(kern, C::NTHREADS, C::LDS_BYTES, total, once);
    return launch_flat(kern, total, C::NTHREADS, C::LDS_BYTES, stream, a);
}

template <class T, int NKD, int NKR, bool VEC, bool MASK, bool QB2, bool FOLD, bool KB1 = false>
static hipError_t launch_dq_qb(const BwdArgs &a, hipStream_t stream) {
    // head dim 32, aligned, unmasked, no dq_bias wanted: the instantiation without its products
    if constexpr (NKD == 2 && NKR > 0 && NKR <= 2 && VEC && !MASK && !KB1) {
        if (!a.dqb.ptr) return launch_dq_qb_bg<T, NKD, NKR, VEC, MASK, QB2, FOLD, KB1, false>(a, stream);
    }
    return launch_dq_qb_bg<T, NKD, NKR, VEC, MASK, QB2, FOLD, KB1, true>(a, stream);
}

// 256-query workgroups (two blocks per wave) once every compute unit has two of them (three under
// a causal mask: B1 H50 d32 r16 at L=4096 0.162 -> 0.153 ms with the large ones, equal at L=8192 and
// L=16384), 128-query workgroups below that and for short sequences whose last 256-query
// workgroup would be half empty (8192 x 16 windows of 128 tokens: 2.59 -> 1.76 ms): as in the forward
// launcher.
template <class T, int NKD, int NKR, bool VEC, bool MASK, bool FOLD = false>
static hipError_t launch_dq_vec(const BwdArgs &a, hipStream_t stream) {
    if constexpr (DqCfg<T, NKD, NKR, VEC, MASK, true>::QBLK == 2) {
        const int64_t wgs = (int64_t)a.B * a.H * ((a.Lq + 255) / 256);
        if (wgs < (int64_t)(a.causal ? 3 : 2) * num_cus() || half_empty_256(a.Lq))
            return launch_dq_qb<T, NKD, NKR, VEC, MASK, false, FOLD>(a, stream);
    }
    // head dims above 64, aligned, unmasked, rank <= 32: 32-key tiles fit two workgroups per CU
    // (measured 20-35 % faster without and 35-40 % faster with a causal mask at head dim 128;
    // larger ranks spill at 256 registers and keep 64-key tiles at one wave per SIMD)
    if constexpr (NKD > 4 && NKR <= 2 && VEC && !MASK)
        return launch_dq_qb<T, NKD, NKR, VEC, MASK, true, FOLD, true>(a, stream);
    return launch_dq_qb<T, NKD, NKR, VEC, MASK, true, FOLD>(a, stream);
}

} // namespace fb
#include "fb_bwd_dq_lean.h"
namespace fb {

template <class T, int NKD, int NKR>
static hipError_t launch_dq_cfg(const BwdArgs &a, hipStream_t stream) {
    // the direct loader keeps the byte distance between two tiles' rows in 32 bits
    const int64_t lim = (int64_t)1 << 24;
    const bool vec = a.q.vec_ok && a.k.vec_ok && a.v.vec_ok && a.dout.vec_ok && a.d % 8 == 0 &&
                     (a.r == 0 || (a.qb.vec_ok && a.kb.vec_ok && a.r % 8 == 0)) && a.k.ss < lim && a.v.ss < lim &&
                     (a.r == 0 || a.kb.ss < lim) && (!a.stats_here || a.o.vec_ok);
    if (a.mask.type)
        return vec ? launch_dq_vec<T, NKD, NKR, true, true>(a, stream) : launch_dq_vec<T, NKD, NKR, false, true>(a, stream);
    if constexpr (NKD == 2 && NKR <= 1) {
        if (dq_streamlined(a)) {
            if constexpr (NKR > 0) {
                if (!a.dqb.ptr) return launch_dq_lean<T, NKR, false>(a, stream);
            }
            return launch_dq_lean<T, NKR>(a, stream);
        }
    }
    if constexpr (NKR <= 2) {
        if (vec && fold_scale_ok<T>(a.scale, a.r, a.Lk)) return launch_dq_vec<T, NKD, NKR, true, false, true>(a, stream);
    }
    return vec ? launch_dq_vec<T, NKD, NKR, true, false>(a, stream) : launch_dq_vec<T, NKD, NKR, false, false>(a, stream);
}

template <class T, int NKD>
static hipError_t launch_dq_r(const BwdArgs &a, hipStream_t stream) {
    switch (nkr_of(a.r)) {
    case 0: return launch_dq_cfg<T, NKD, 0>(a, stream);
    case 1: return launch_dq_cfg<T, NKD, 1>(a, stream);
    case 2: return launch_dq_cfg<T, NKD, 2>(a, stream);
    case 4: return launch_dq_cfg<T, NKD, 4>(a, stream);
    default: return launch_dq_cfg<T, NKD, 8>(a, stream);
    }
}

// Compiled once per (element type, head-dim bucket), see Makefile.  (FB_BODIES_ONLY: included by the unit that
// builds the mixed dq + dk/dv launch, which wants the kernels' bodies and not this entry point.)
#ifndef FB_BODIES_ONLY
#define FB_CAT2(a, b) a##b
#define FB_CAT(a, b) FB_CAT2(a, b)
hipError_t FB_CAT(launch_bwd_dq_, FB_SUFFIX)(const BwdArgs &a, hipStream_t stream) {
    return launch_dq_r<FB_T, FB_NKD>(a, stream);
}
#endif

} // namespace fb
