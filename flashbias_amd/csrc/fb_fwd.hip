// Forward FlashBias attention for gfx950:  o = softmax(scale q k^T + q_b k_b^T + mask) v, lse.
// Replaces _fwd_kernel of the reference (flash_bias/flash_bias_triton.py:62-355).
//
// One workgroup (4 waves) owns BM = 128 or 256 consecutive queries of one (batch, head); each
// wave owns one or two blocks of 32 of them.  Keys are streamed in tiles of BN = 64 or 128
// through double-buffered LDS.
// Everything is computed transposed so that a lane owns one query:
//
//   S^T (keys x queries) = [K | K_b] [scale Q | Q_b]^T     A = key tile from LDS, B = query regs
//   O^T (d x queries)   += V^T P^T                         A = V^T tile from LDS, B = P^T regs
//
// In the C layout a lane holds one query column and 16 keys of it, so the row max of the
// online softmax is an in-lane reduction plus one exchange with lane ^ 32, the rescale factor
// is a per-lane scalar, and P^T is already in the B-operand layout of the second MFMA (no LDS
// round trip for P).  The contraction runs over the concatenated channels [d | r],
// zero-padded to 16-wide MFMA steps.
//
// Softmax scale: the reference multiplies the fp32 q k^T accumulator by the scale and never
// scales the bias product (flash_bias_triton.py:246-256).  General case here: q k^T and q_b k_b^T
// are two separate (and therefore independent, shorter) MFMA chains, joined by one fp32 FMA per
// score.  (Folding the scale into the query operand needs a second, low-order MFMA per step and
// measured slower: the matrix pipe is the scarcer resource when two waves share a SIMD.)
// FOLD instantiations (no mask; no factors, or bf16 factors with a power-of-two scale or r <= 8,
// see fold_scale_ok) instead divide q_b by the scale once, keep the scores in units of 1 / scale
// in one MFMA chain, and apply the scale inside the FMA that feeds exp2: one FMA per score less.
//
// Per score the VALU does: [fma (scale),] max3, fma + exp2, convert, add (row sum); the running
// reference of the softmax only moves when a row maximum grows by more than 2^8 (then
// p <= 256, exact enough in fp32 / 16-bit), so the accumulator rescale is rare.
#include "fb_kernels.h"

namespace fb {

// VEC: every streamed tensor is 16-byte aligned (base and strides) and d, r are multiples of 8.
// QB2_: allow two query blocks per wave (the launcher turns it off for small grids).
// FOLD_: the scores are scale * (q k^T + (q_b / scale) k_b^T), one MFMA chain and no FMA per
// score for the scale (see the launcher for when that is exact).
template <class T, int NKD_, int NKR_, int NDV_, bool VEC_, bool MASK_, bool QB2_ = true, bool FOLD_ = false>
struct FwdCfg {
    static constexpr int NKD = NKD_, NKR = NKR_, NDV = NDV_;
    static constexpr bool VEC = VEC_, MASK = MASK_, FOLD = FOLD_;
    static_assert(!FOLD_ || !MASK_, "the additive mask is not divided by the scale");
    static constexpr int NWAVES = 4, NTHREADS = 64 * NWAVES;
    // query blocks (of 32) per wave: two where the registers allow (head dim <= 32, rank <= 32:
    // 219-247 registers at four operand steps), so that every key / value fragment read from LDS
    // feeds two blocks and two waves per SIMD carry four softmax streams (768 x 4 rows of 768
    // tokens at rank 32: 0.77 -> 0.64 ms)
    static constexpr int QB = (QB2_ && NKD_ + NKR_ <= 4 && NDV_ == 1 && VEC_ && !MASK_) ? 2 : 1;
    static constexpr int BM = NWAVES * 32 * QB;
    static constexpr int NK = NKD + NKR;
    // A wave computes KBLK * 32 keys at a time; an LDS tile (one barrier) holds SUBS such groups.
    static constexpr int KBLK = 2, BSUB = 32 * KBLK;
    // two groups per tile where three workgroups of that size still fit the 160 KB of a CU
    static constexpr int LDS2 = 2 * 2 * (2 * BSUB * (16 * NK + 8) + 32 * NDV_ * (2 * BSUB + 8));
    // (masked, aligned instantiations also stage a BM x BN mask tile: one group per tile)
    static constexpr bool MTILE = VEC_ && MASK_;
    static constexpr int SUBS = (!MTILE && NK <= 4 && NDV_ <= 2 && 3 * LDS2 <= 160 * 1024) ? 2 : 1;
    static constexpr int BN = BSUB * SUBS;
    static constexpr int DKP = 16 * NK + 8; // LDS row of [K | K_b], elements (16 B of padding)
    static constexpr int DV = 32 * NDV;
    static constexpr int BNP = BN + 8; // LDS row of V^T
    static constexpr int SK_ELEMS = BN * DKP, SV_ELEMS = DV * BNP;
    static constexpr int MROWCH = BN / 8;                    // 16-byte chunks per mask-tile row
    static constexpr int SM_ELEMS = MTILE ? BM * BN : 0;      // 16-bit matrix mask tile, swizzled chunks
    static constexpr int LDS_BYTES = 2 * (SK_ELEMS + SV_ELEMS + SM_ELEMS) * 2;
    // cooperative loader: 8-channel chunks of K and K_b (one key row each), (4 keys x 4
    // channels) blocks of V.  Consecutive threads take the consecutive chunks of one row, then the
    // next row: a load instruction then asks for whole 64-byte rows (one request each) instead of
    // a quarter of 64 different rows (Swin windows: forward 1.65 -> 1.55 ms; head dim 64, rank 16,
    // L=4096: 0.92 -> 0.80; causal rank 16 at L=8192: 0.59 -> 0.52), at the price of two-way bank
    // conflicts in the transposing stores of V.
    static constexpr int CD = 2 * NKD, CR = 2 * NKR;
    static constexpr int K_TASKS = BN * CD, KB_TASKS = BN * CR, V_TASKS = (BN / 4) * (DV / 4);
    static constexpr int K_PT = (K_TASKS + NTHREADS - 1) / NTHREADS;
    static constexpr int KB_PT = (KB_TASKS + NTHREADS - 1) / NTHREADS;
    static constexpr int V_PT = (V_TASKS + NTHREADS - 1) / NTHREADS;
    // registers: three waves per SIMD for the configurations that need at most 168 (six operand steps
    // with head dims up to 64: 158-166; the attribute is a cap the hardware honours, so a kernel that
    // would fit three waves runs two unless it says three), one (512 registers) where the
    // mask values or an unaligned head dim of 128 would spill at 256, else two
    static constexpr bool BIG = (MASK_ && (NDV_ >= 2 || NKD_ + NKR_ >= 5)) || (!VEC_ && NDV_ == 4) ||
                                2 * LDS_BYTES > 160 * 1024; // (one workgroup per CU anyway)
    static constexpr int WAVES_EU = QB == 2 ? 2 : BIG ? 1 : (NK <= 6 && NDV <= 2) ? 3 : 2;
    // LDS fragments requested ahead of their use: all key steps of a group when they are few,
    // and the V^T fragments of a group when the head dimension is one MFMA block
    static constexpr int KPRE = NK <= 4 ? NK : 0;
    static constexpr bool VPRE = NDV == 1;
};

template <class C>
struct FwdStage { // one key tile in flight from HBM to LDS
    u32x4_t k[C::K_PT];
    u32x4_t kb[C::KB_PT > 0 ? C::KB_PT : 1];
    u32x2_t v[C::V_PT][4];
};

// Four consecutive channels [col0, col0 + 4) of one row, zero outside the matrix.
template <bool VEC>
__device__ __forceinline__ u32x2_t load_half(const uint16_t *base, int64_t ld, int row, int nrows, int col0,
                                             int ncols) {
    const bool row_ok = row < nrows;
    const uint16_t *rp = base + (int64_t)(row_ok ? row : nrows - 1) * ld;
    u32x2_t out;
    if constexpr (VEC) {
        const bool ok = row_ok && col0 < ncols;
        out = *reinterpret_cast<const u32x2_t *>(rp + (col0 < ncols ? col0 : 0));
        out[0] = ok ? out[0] : 0u;
        out[1] = ok ? out[1] : 0u;
    } else {
        uint32_t e[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int col = col0 + i;
            uint32_t val = rp[col < ncols ? col : ncols - 1];
            asm volatile("" : "+v"(val));
            e[i] = (row_ok && col < ncols) ? val : 0u;
        }
        out[0] = e[0] | (e[1] << 16);
        out[1] = e[2] | (e[3] << 16);
    }
    return out;
}

// Per-thread constants of the cooperative loader: which rows / chunks this thread copies, as
// 32-bit element offsets from the (wave-uniform) base of a key tile, so that the per-tile
// address is "scalar base + lane offset" and costs no vector ALU work.
template <class C>
struct FwdLoader {
    uint32_t koff[C::K_PT], kboff[C::KB_PT > 0 ? C::KB_PT : 1], voff[C::V_PT][4];
    uint32_t kdst[C::K_PT], kbdst[C::KB_PT > 0 ? C::KB_PT : 1], vdst[C::V_PT];
    bool kok[C::K_PT], kbok[C::KB_PT > 0 ? C::KB_PT : 1], vok[C::V_PT];

    // Folded scale with r <= 8: columns 8..15 of the bias step hold a second copy of k_b, the
    // partner of the low parts of q_b / scale in the query operand.
    static __device__ __forceinline__ bool low_parts(const FwdArgs &a) { return C::FOLD && C::NKR == 1 && a.r <= 8 && a.scale != 1.f; }
    static __device__ __forceinline__ int bias_src_chunk(const FwdArgs &a, int ch) {
        return (low_parts(a) && ch == 1) ? 0 : ch;
    }

    __device__ __forceinline__ void init(const FwdArgs &a, int tid) {
#pragma unroll
        for (int i = 0; i < C::K_PT; ++i) {
            const int task = tid + i * C::NTHREADS;
            const int row = task / C::CD, ch = task % C::CD; // (consecutive lanes: the consecutive chunks of one row)
            kok[i] = task < C::K_TASKS && ch * 8 < a.d;
            koff[i] = kok[i] ? (uint32_t)(row * a.k.ss + ch * 8) : 0u;
            kdst[i] = row * C::DKP + ch * 8;
        }
#pragma unroll
        for (int i = 0; i < C::KB_PT; ++i) {
            const int task = tid + i * C::NTHREADS;
            const int row = task / C::CR, ch = task % C::CR;
            const int src = bias_src_chunk(a, ch);
            kbok[i] = task < C::KB_TASKS && src * 8 < a.r;
            kboff[i] = kbok[i] ? (uint32_t)(row * a.kb.ss + src * 8) : 0u;
            kbdst[i] = row * C::DKP + 16 * C::NKD + ch * 8;
        }
#pragma unroll
        for (int i = 0; i < C::V_PT; ++i) {
            const int task = (C::NTHREADS - 1 - tid) + i * C::NTHREADS;
            const int hc = task % (C::DV / 4), quad = task / (C::DV / 4); // (consecutive lanes: one row's channels)
            vok[i] = task < C::V_TASKS && hc * 4 < a.d;
#pragma unroll
            for (int j = 0; j < 4; ++j) voff[i][j] = vok[i] ? (uint32_t)((quad * 4 + j) * a.v.ss + hc * 4) : 0u;
            vdst[i] = (hc * 4) * C::BNP + slot_of(quad * 4); // 4 keys stay adjacent, quads are permuted
        }
    }

    // Tile fully inside the sequence, 16-byte aligned tensors: plain loads, nothing else.
    __device__ __forceinline__ void load_fast(FwdStage<C> &st, const uint16_t *kt, const uint16_t *kbt,
                                              const uint16_t *vt) const {
#pragma unroll
        for (int i = 0; i < C::K_PT; ++i) st.k[i] = *reinterpret_cast<const u32x4_t *>(kt + koff[i]);
        if constexpr (C::NKR > 0) {
#pragma unroll
            for (int i = 0; i < C::KB_PT; ++i) st.kb[i] = *reinterpret_cast<const u32x4_t *>(kbt + kboff[i]);
        }
#pragma unroll
        for (int i = 0; i < C::V_PT; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) st.v[i][j] = *reinterpret_cast<const u32x2_t *>(vt + voff[i][j]);
    }

    // Any tile: rows past the end and columns past d / r read a clamped address and become 0.
    __device__ __forceinline__ void load_safe(FwdStage<C> &st, const FwdArgs &a, const uint16_t *kbase,
                                              const uint16_t *kbbase, const uint16_t *vbase, int n0, int tid) const {
#pragma unroll
        for (int i = 0; i < C::K_PT; ++i) {
            const int task = tid + i * C::NTHREADS;
            st.k[i] = load_chunk<C::VEC>(kbase, a.k.ss, n0 + task / C::CD, a.Lk, (task % C::CD) * 8, a.d);
        }
        if constexpr (C::NKR > 0) {
#pragma unroll
            for (int i = 0; i < C::KB_PT; ++i) {
                const int task = tid + i * C::NTHREADS;
                st.kb[i] = load_chunk<C::VEC>(kbbase, a.kb.ss, n0 + task / C::CR, a.Lk,
                                              bias_src_chunk(a, task % C::CR) * 8, a.r);
            }
        }
#pragma unroll
        for (int i = 0; i < C::V_PT; ++i) {
            const int task = (C::NTHREADS - 1 - tid) + i * C::NTHREADS;
            const int hc = task % (C::DV / 4), quad = task / (C::DV / 4); // (consecutive lanes: one row's channels)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                st.v[i][j] = load_half<C::VEC>(vbase, a.v.ss, n0 + quad * 4 + j, a.Lk, hc * 4, a.d);
        }
    }

    // Registers -> LDS.  Threads whose chunk lies in the zero padding of the channel dimension
    // never store: those LDS columns are cleared once before the loop.
    __device__ __forceinline__ void store(const FwdStage<C> &st, uint16_t *sK, uint16_t *sVt) const {
#pragma unroll
        for (int i = 0; i < C::K_PT; ++i)
            if (kok[i]) *reinterpret_cast<u32x4_t *>(sK + kdst[i]) = st.k[i];
        if constexpr (C::NKR > 0) {
#pragma unroll
            for (int i = 0; i < C::KB_PT; ++i)
                if (kbok[i]) *reinterpret_cast<u32x4_t *>(sK + kbdst[i]) = st.kb[i];
        }
#pragma unroll
        for (int i = 0; i < C::V_PT; ++i) {
            if (vok[i]) {
#pragma unroll
                for (int e = 0; e < 4; ++e) { // channel hc*4 + e gets its four keys as one 8-byte store
                    const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;
                    u32x2_t pk;
                    pk[0] = __builtin_amdgcn_perm(st.v[i][1][e >> 1], st.v[i][0][e >> 1], sel);
                    pk[1] = __builtin_amdgcn_perm(st.v[i][3][e >> 1], st.v[i][2][e >> 1], sel);
                    *reinterpret_cast<u32x2_t *>(sVt + vdst[i] + e * C::BNP) = pk;
                }
            }
        }
    }
};

// The whole forward of one workgroup (C::BM queries of one (batch, head)); the kernel below is
// nothing else, and the streamlined kernel (fb_fwd_lean.h) calls it for a workgroup whose row sums
// left the range that its fixed reference point covers.
template <class T, class C>
__device__ __forceinline__ void fwd_body(const FwdArgs &a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint16_t *sKbuf = reinterpret_cast<uint16_t *>(smem);
    uint16_t *sVbuf = sKbuf + 2 * C::SK_ELEMS;
    uint16_t *sMbuf = sVbuf + 2 * C::SV_ELEMS;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6); // scalar: branches on it are uniform
    const int c = lane & 31, g = lane >> 5;

    const int total = a.ntiles_m * a.B * a.H;
    int bh, tile_m;
    work_order(blockIdx.x, a.ntiles_m, total, a.causal, bh, tile_m);
    if (a.causal) tile_m = a.ntiles_m - 1 - tile_m; // the last query tile sees the most keys
    const int b = bh / a.H, h = bh % a.H;
    const int m0 = tile_m * C::BM;
    const int wq0 = m0 + wave * (32 * C::QB); // first query of this wave

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

    // ---- query operands, resident in registers for the whole key loop
    u32x4_t qr[C::QB][C::NKD], qbr[C::QB][C::NKR > 0 ? C::NKR : 1];
    f32x16_t acc_o[C::QB][C::NDV];
    float m_ref[C::QB]; // reference of the exponentials (natural units), lags the true row max
    float m2[C::QB];    // m_ref * log2(e), 0 while the row has seen no finite score
    float l_run[C::QB]; // per-lane partial row sum (the two lanes of a query are added at the end)
#pragma unroll
    for (int qb = 0; qb < C::QB; ++qb) {
        const int query = wq0 + 32 * qb + c;
#pragma unroll
        for (int t = 0; t < C::NKD; ++t)
            qr[qb][t] = load_chunk<C::VEC>(qbase, a.q.ss, query, a.Lq, 16 * t + 8 * g, a.d);
        if constexpr (C::NKR > 0) {
#pragma unroll
            for (int t = 0; t < C::NKR; ++t) {
                const bool low = FwdLoader<C>::low_parts(a) && g == 1;
                qbr[qb][t] = load_chunk<C::VEC>(qbbase, a.qb.ss, query, a.Lq, low ? 0 : 16 * t + 8 * g, a.r);
                if (C::FOLD && a.scale != 1.f) qbr[qb][t] = fold_scale_chunk<T>(qbr[qb][t], 1.f / a.scale, FwdLoader<C>::low_parts(a), low);
            }
        }
#pragma unroll
        for (int n = 0; n < C::NDV; ++n)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc_o[qb][n][v] = 0.f;
        m_ref[qb] = -INFINITY;
        m2[qb] = 0.f;
        l_run[qb] = 0.f;
    }
    // m_ref and the scores are in natural units, or in units of 1 / scale when the scale is folded
    const float to_log2 = C::FOLD ? a.scale * kLog2e : kLog2e;
    const float lag = 8.0f / to_log2; // let the row max run ahead of m_ref by up to 2^8

    // causal: tiles past the last query of this workgroup are never visible (:202)
    int k_end = a.Lk;
    if (a.causal && m0 + C::BM < k_end) k_end = m0 + C::BM;
    const int ntiles_k = (k_end + C::BN - 1) / C::BN;

    FwdLoader<C> ld;
    ld.init(a, tid);
    {   // clear both LDS buffers once: the zero padding of the channel dimension is never rewritten
        u32x4_t *z = reinterpret_cast<u32x4_t *>(smem);
        for (int i = tid; i < C::LDS_BYTES / 16; i += C::NTHREADS) z[i] = u32x4_t{0u, 0u, 0u, 0u};
    }
    __syncthreads();
    auto load_tile = [&](FwdStage<C> &stg, int n0) {
        if (C::VEC && n0 + C::BN <= a.Lk)
            ld.load_fast(stg, kbase + (int64_t)n0 * a.k.ss, C::NKR > 0 ? kbbase + (int64_t)n0 * a.kb.ss : nullptr,
                         vbase + (int64_t)n0 * a.v.ss);
        else
            ld.load_safe(stg, a, kbase, kbbase, vbase, n0, tid);
    };
    // Masked, aligned instantiations: a 16-bit matrix mask whose rows allow 16-byte copies travels
    // as a BM x BN tile straight into LDS, one tile ahead like K and V (full key tiles only; a
    // ragged last tile and every other kind of mask take the loads of mask_block_keys).
    TileDma<C::BM, C::MROWCH, C::NWAVES, false> mdma;
    bool mtile = false;
    if constexpr (C::MTILE) {
        static_assert(C::QB == 1, "one query block per wave in masked instantiations");
        if (a.mask.vec_ok && !a.mask.is_f32 && a.Lk % 8 == 0 && a.mask.sm % 8 == 0 && // (a vector mask: row stride 0)
            a.mask.sm < (1 << 24) && reinterpret_cast<uintptr_t>(mbase) % 16 == 0) {
            mtile = true;
            mdma.init(reinterpret_cast<const uint16_t *>(mbase), a.mask.sm, C::BN, C::MROWCH, nullptr, 0, 0, wave, lane, m0);
            if (C::BN <= a.Lk) mdma.issue_step(lds_addr_of(sMbuf), m0, a.Lq, a.mask.sm, 0, C::MROWCH, 2 * C::BN, 0);
        }
    }
    FwdStage<C> st;
    load_tile(st, 0);
    ld.store(st, sKbuf, sVbuf);
    if constexpr (C::MTILE) wait_vmcnt<0>();
    __syncthreads();

    int turn = __builtin_amdgcn_readfirstlane(cu_slot());
    for (int it = 0; it < ntiles_k; ++it) {
        const int cur = it & 1;
        take_turn(turn, a.slots);
        const int n0 = it * C::BN;
        const bool more = it + 1 < ntiles_k;
        if constexpr (C::MTILE) {
            if (mtile && more && n0 + 2 * C::BN <= a.Lk)
                mdma.issue_step(lds_addr_of(sMbuf + (cur ^ 1) * C::SM_ELEMS), m0, a.Lq, a.mask.sm, 0, C::MROWCH,
                                2 * C::BN, 0);
        }
        if (more) load_tile(st, n0 + C::BN);

        const uint16_t *sK = sKbuf + cur * C::SK_ELEMS;
        const uint16_t *sVt = sVbuf + cur * C::SV_ELEMS;
        int nsubs = C::SUBS;
        if constexpr (C::MTILE || C::SUBS == 1) asm volatile("" : "+s"(nsubs)); // keeps the loop a loop (without it the masked code spills)
#pragma nounroll
        for (int sub = 0; sub < nsubs; ++sub) {
            const int ns = n0 + sub * C::BSUB;
            // the group is hidden from every query of this wave: so are all later ones
            if ((a.causal && ns > wq0 + 32 * C::QB - 1) || wq0 >= a.Lq || ns >= k_end) break;
            // all key fragments of the group are requested before the first MFMA (one LDS wait)
            // and serve every query block of the wave
            u32x4_t ka[C::KBLK][C::KPRE > 0 ? C::KPRE : 1];
#pragma unroll
            for (int kb = 0; kb < C::KBLK; ++kb)
#pragma unroll
                for (int t = 0; t < C::KPRE; ++t)
                    ka[kb][t] = *reinterpret_cast<const u32x4_t *>(sK + (sub * C::BSUB + kb * 32 + c) * C::DKP +
                                                                   16 * t + 8 * g);
            // the V^T fragments travel from LDS while the first row maximum is formed
            u32x4_t va[C::VPRE ? C::KBLK * 2 : 1];
            if constexpr (C::VPRE) {
#pragma unroll
                for (int kb = 0; kb < C::KBLK; ++kb)
#pragma unroll
                    for (int t = 0; t < 2; ++t)
                        va[kb * 2 + t] = *reinterpret_cast<const u32x4_t *>(sVt + c * C::BNP + sub * C::BSUB + kb * 32 +
                                                                            16 * t + 8 * g);
            }
#pragma unroll
            for (int qb = 0; qb < C::QB; ++qb) {
                const int bq0 = wq0 + 32 * qb; // first query of the block
                const int query = bq0 + c;
                // wave-uniform skip of a block the whole group is hidden from (it also keeps the
                // instruction streams of the two blocks apart, which the register allocation needs)
                if (C::QB > 1 && a.causal && ns > bq0 + 31) continue;
                // ---- S^T = [K | K_b] [scale Q | Q_b]^T
                f32x16_t s[C::KBLK];
                // additive mask: requested up front, it is the initial value of the bias chain
                f32x16_t mk[C::MASK ? C::KBLK : 1];
                if constexpr (C::MASK) {
                    const uint8_t *mrow = mbase + (a.mask.type == 2 ? (int64_t)min(query, a.Lq - 1) * a.mask.sm : 0) *
                                                      (a.mask.is_f32 ? 4 : 2);
                    if (C::MTILE && mtile && n0 + C::BN <= a.Lk) {
                        // this lane's query row of the staged tile, keys in C-layout order
                        const uint16_t *sM = sMbuf + cur * C::SM_ELEMS;
                        const int row = wave * 32 + c;
#pragma unroll
                        for (int kb = 0; kb < C::KBLK; ++kb)
#pragma unroll
                            for (int j = 0; j < 4; ++j) {
                                const u32x2_t x = *reinterpret_cast<const u32x2_t *>(
                                    sM + swz_off<C::MROWCH>(row, 4 * kb + j) + 4 * g);
                                mk[kb][4 * j + 0] = T::to_float((uint16_t)(x[0] & 0xffffu));
                                mk[kb][4 * j + 1] = T::to_float((uint16_t)(x[0] >> 16));
                                mk[kb][4 * j + 2] = T::to_float((uint16_t)(x[1] & 0xffffu));
                                mk[kb][4 * j + 3] = T::to_float((uint16_t)(x[1] >> 16));
                            }
                    } else {
#pragma unroll
                        for (int kb = 0; kb < C::KBLK; ++kb)
                            mask_block_keys<T>(a.mask, mrow, ns + kb * 32, g, a.Lk, mk[kb]);
                    }
                }
#pragma unroll
                for (int kb = 0; kb < C::KBLK; ++kb) {
                    // the q k^T part and the bias part are two independent MFMA chains, joined by
                    // one FMA per score that applies the softmax scale in fp32 (:246-256)
                    f32x16_t acc, accb;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        acc[v] = 0.f;
                        accb[v] = C::MASK ? mk[C::MASK ? kb : 0][v] : 0.f;
                    }
#pragma unroll
                    for (int t = 0; t < C::NK; ++t) {
                        const u32x4_t kf = t < C::KPRE ? ka[kb][t < C::KPRE ? t : 0]
                                                       : *reinterpret_cast<const u32x4_t *>(
                                                             sK + (sub * C::BSUB + kb * 32 + c) * C::DKP + 16 * t + 8 * g);
                        if (t < C::NKD)
                            acc = T::mfma(kf, qr[qb][t], acc);
                        else if (C::FOLD)
                            acc = T::mfma(kf, qbr[qb][t - C::NKD], acc);
                        else
                            accb = T::mfma(kf, qbr[qb][t - C::NKD], accb);
                    }
                    if constexpr (!C::FOLD) {
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            acc[v] = (C::NKR > 0 || C::MASK) ? __builtin_fmaf(acc[v], a.scale, accb[v]) : acc[v] * a.scale;
                    }
                    s[kb] = acc;
                }
                // ---- -inf for keys past the end and causal-hidden pairs
                const bool ragged = ns + C::BSUB > a.Lk;
                const bool diag = a.causal && (ns + C::BSUB - 1 > bq0);
                if (ragged || diag) {
                    int key0 = ns + 4 * g;
                    asm volatile("" : "+v"(key0)); // (computed here, not kept in registers across the loop)
#pragma unroll
                    for (int kb = 0; kb < C::KBLK; ++kb)
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const int key = key0 + kb * 32 + 8 * (v >> 2) + (v & 3);
                            if (key >= a.Lk || (a.causal && key > query)) s[kb][v] = -INFINITY;
                        }
                }
                // ---- online softmax, one query per lane (two lanes share a query)
                float mx = s[0][0];
#pragma unroll
                for (int kb = 0; kb < C::KBLK; ++kb)
#pragma unroll
                    for (int v = (kb == 0 ? 1 : 0); v < 16; ++v) mx = fmaxf(mx, s[kb][v]);
                mx = half_wave_max(mx);
                const bool grow = mx > m_ref[qb] + lag; // also true for the first finite score of a row
                if (__any(grow)) {
                    const float m_new = grow ? mx : m_ref[qb];
                    const float alpha = grow ? fast_exp2((m_ref[qb] - m_new) * to_log2) : 1.f; // exp2(-inf) = 0
                    l_run[qb] *= alpha;
#pragma unroll
                    for (int n = 0; n < C::NDV; ++n)
#pragma unroll
                        for (int v = 0; v < 16; ++v) acc_o[qb][n][v] *= alpha;
                    m_ref[qb] = m_new;
                    m2[qb] = (m_new == -INFINITY) ? 0.f : m_new * to_log2;
                }
                // ---- P^T = exp(S^T - m_ref), row sums (of the fp32 values, :271), O^T += V^T P^T
#pragma unroll
                for (int kb = 0; kb < C::KBLK; ++kb)
#pragma unroll
                    for (int t = 0; t < 2; ++t) {
                        u32x4_t pb;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float p0 = fast_exp2(__builtin_fmaf(s[kb][8 * t + 2 * e], to_log2, -m2[qb]));
                            const float p1 = fast_exp2(__builtin_fmaf(s[kb][8 * t + 2 * e + 1], to_log2, -m2[qb]));
                            pb[e] = T::pack2(p0, p1);
                            l_run[qb] += p0 + p1;
                        }
                        if constexpr (C::VPRE) {
                            acc_o[qb][0] = T::mfma(va[kb * 2 + t], pb, acc_o[qb][0]);
                        } else {
#pragma unroll
                            for (int n = 0; n < C::NDV; ++n) {
                                const u32x4_t vf = *reinterpret_cast<const u32x4_t *>(
                                    sVt + (32 * n + c) * C::BNP + sub * C::BSUB + kb * 32 + 16 * t + 8 * g);
                                acc_o[qb][n] = T::mfma(vf, pb, acc_o[qb][n]);
                            }
                        }
                    }
            }
        }
        if (more) ld.store(st, sKbuf + (cur ^ 1) * C::SK_ELEMS, sVbuf + (cur ^ 1) * C::SV_ELEMS);
        if constexpr (C::MTILE) wait_vmcnt<0>(); // the mask tile copies are not known to the compiler
        __syncthreads();
    }

    // ---- epilogue: o = acc / l, lse = m_ref + ln(l)
    uint16_t *obase = const_cast<uint16_t *>(a.o.ptr) + b * a.o.sb + h * a.o.sh;
#pragma unroll
    for (int qb = 0; qb < C::QB; ++qb) {
        int query = wq0 + 32 * qb + c;
        asm volatile("" : "+v"(query)); // (keeps the address arithmetic below the key loop)
        const float l = l_run[qb] + __shfl_xor(l_run[qb], 32, 64);
        const float inv = 1.f / l;
        const bool ok = query < a.Lq;
        if (ok && g == 0) a.lse[(int64_t)bh * a.Lq + query] = m_ref[qb] * (C::FOLD ? a.scale : 1.f) + __builtin_amdgcn_logf(l) * kLn2;
        uint16_t *orow = obase + (int64_t)(ok ? query : 0) * a.o.ss;
#pragma unroll
        for (int n = 0; n < C::NDV; ++n) store_acc_rows<T, C::VEC>(orow + 32 * n, ok, true, acc_o[qb][n], inv, a.d - 32 * n, g);
    }
}

template <class T, class C>
__global__ __launch_bounds__(C::NTHREADS) __attribute__((amdgpu_waves_per_eu(C::WAVES_EU == 1 ? 1 : 2, C::WAVES_EU))) void fwd_kernel(
    const FwdArgs a) {
    fwd_body<T, C>(a);
}

} // namespace fb
#include "fb_fwd_lean.h"
namespace fb {

template <class T, int NKD, int NKR, int NDV, bool VEC, bool MASK, bool QB2, bool FOLD>
static hipError_t launch_fwd_qb(const FwdArgs &a0, hipStream_t stream) {
    typedef FwdCfg<T, NKD, NKR, NDV, VEC, MASK, QB2, FOLD> C;
    FwdArgs a = a0;
    a.ntiles_m = (a.Lq + C::BM - 1) / C::BM;
    auto kern = fwd_kernel<T, C>;
    static KernelOnce once;
    const hipError_t e = allow_lds(kern, C::LDS_BYTES, once);
    if (e != hipSuccess) return e;
    const int64_t total = (int64_t)a.ntiles_m * a.B * a.H;
    a.slots = slots_per_cu(kern, C::NTHREADS, C::LDS_BYTES, total, once);
    return launch_flat(kern, total, C::NTHREADS, C::LDS_BYTES, stream, a);
}

// Two query blocks per wave (256 queries per workgroup) pay once every compute unit has two such
// workgroups; below that, 128-query workgroups at three waves per SIMD fill the chip better
// (measured: 35 % faster at a quarter of that grid, 10 % slower at twice it).  Under a causal mask the
// workgroups differ in length; with every XCD's share started longest first (work_order, fb_order.h) three
// per compute unit are enough (B1 H50 d32 r16: 0.453 -> 0.434 ms at L=8192, 0.127 -> 0.125 at L=4096; while the
// grid was walked head by head the small workgroups stayed ahead up to seven per compute unit).
// Short sequences whose last 256-query workgroup would be half
// empty also take the small ones (8192 x 16 windows of 128 tokens: 1.94 -> 1.41 ms).
template <class T, int NKD, int NKR, int NDV, bool VEC, bool MASK, bool FOLD = false>
static hipError_t launch_fwd_vec(const FwdArgs &a, hipStream_t stream) {
    if constexpr (FwdCfg<T, NKD, NKR, NDV, VEC, MASK, true>::QB == 2) {
        const int64_t wgs = (int64_t)a.B * a.H * ((a.Lq + 255) / 256);
        if (wgs < (int64_t)(a.causal ? 3 : 2) * num_cus() || half_empty_256(a.Lq))
            return launch_fwd_qb<T, NKD, NKR, NDV, VEC, MASK, false, FOLD>(a, stream);
    }
    return launch_fwd_qb<T, NKD, NKR, NDV, VEC, MASK, true, FOLD>(a, stream);
}

template <class T, int NKD, int NKR, int NDV>
static hipError_t launch_fwd_cfg(const FwdArgs &a, hipStream_t stream) {
    // the fast loader keeps the element offset of a tile row in 32 bits
    const int64_t lim = (int64_t)1 << 24;
    const bool vec = a.q.vec_ok && a.k.vec_ok && a.v.vec_ok && a.o.vec_ok && a.d % 8 == 0 &&
                     (a.r == 0 || (a.qb.vec_ok && a.kb.vec_ok && a.r % 8 == 0)) && a.k.ss < lim && a.v.ss < lim &&
                     (a.r == 0 || a.kb.ss < lim);
    if (a.mask.type)
        return vec ? launch_fwd_vec<T, NKD, NKR, NDV, true, true>(a, stream)
                   : launch_fwd_vec<T, NKD, NKR, NDV, false, true>(a, stream);
    if constexpr (NKD == 2 && NKR <= 1 && NDV == 1) {
        // The streamlined kernel: 256-query workgroups (two query blocks per wave) where they give every
        // SIMD of the chip a wave, 128-query workgroups (one block per wave) below that.
        const int64_t wgs = (int64_t)a.B * a.H * ((a.Lq + 255) / 256);
        // On grids that fill the chip a loop of at least 512 keys pays for the kernel's pipeline (4096 x 16
        // windows, general against streamlined: 1.91 against 2.82 ms at 128 keys, 1.79 against 1.88 at 256,
        // 1.38 against 1.21 at 512); small grids take it at every length.
        if (vec && fwd_lean_ok(a) && (a.Lk >= 512 || small_grid(a.B, a.H, a.Lq))) {
            if (a.causal) return launch_fwd_lean<T, NKR, 1, true>(a, stream);
            return wgs >= num_cus() && !half_empty_256(a.Lq) ? launch_fwd_lean<T, NKR, 2>(a, stream)
                                                             : launch_fwd_lean<T, NKR, 1>(a, stream);
        }
    }
    if constexpr (NKR <= 2) {
        if (vec && fold_scale_ok<T>(a.scale, a.r, a.Lk)) return launch_fwd_vec<T, NKD, NKR, NDV, true, false, true>(a, stream);
    }
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
