// Backward FlashBias attention for gfx950, window regime: all five gradients of one (batch, head)
// in one workgroup when the whole sequence fits it (Lq, Lk <= 256: the window attention of
// 2_Vision_Transformer/swin_transformer_v2.py:178-203).  Replaces the key-block loop of
// _bwd_kernel_one_col_block (flash_bias/flash_bias_triton.py:575-869) including its dq / dq_bias
// updates (:725-817), which the reference adds with atomics and the long-sequence kernels of this
// library (fb_bwd_dkv.hip, fb_bwd_dq.hip) recompute in a second, query-stationary kernel.
//
// Sequences this short are bound by memory, not by arithmetic: the two-kernel backward reads q, k,
// v, o, dO twice and recomputes S and dP.  Here a workgroup of 8 waves holds the window's [Q | Q_b],
// dO and [K | K_b] in LDS (copied there once, straight from global memory; the query-side tiles of the next
// window are requested while the current one finishes) and wave w owns keys [32 w, 32 w + 32) with K, K_b, V
// in registers.  The per-query statistics (delta = rowsum(o * dO), lse * log2 e) are formed by the workgroup
// itself at the top of a window: no preprocess launch, no scratch buffer.  Per step of 128 queries:
//
//   phase 1 (lane = key, as in the dk/dv kernel): S, P = exp(S - lse), dP = dO V^T - delta,
//           dS = P * dP; dV^T += dO^T P, [dK | dK_b]^T += [Q | Q_b]^T dS with P and dS fed from
//           registers; dS also goes to LDS as a (256 keys x 128 queries) tile
//   phase 2 (lane = query): [dQ | dQ_b]^T (64 channels x 128 queries) = [K | K_b]^T dS^T, a small GEMM
//           over the 256 keys with both operands read column-wise from LDS (transposing reads):
//           eight 32 x 32 output blocks, one per wave.  The four dq blocks are written at once; the
//           four dq_bias blocks stay in registers, and since the step's dq_bias blocks go to waves
//           4 step .. 4 step + 3, every wave ends up holding exactly one of the window's eight.
//
// dq needs no sum across workgroups because the workgroup sees every key.  As in the other backward
// kernels a workgroup walks `group` consecutive batch entries and keeps the factor gradients in
// registers across them (factors shared by the batch).  All sums have a fixed order: the results
// are bit-reproducible.
#define FB_BODIES_ONLY
#include "fb_bwd_dkv.hip"

namespace fb {

// NKR_: 16-wide steps of the rank (0, 1, 2).  FOLD_: the scores are scale * (q k^T + q_b k_b^T), no multiply per
// score for the scale (no factors, or a scale of exactly 1).  BG_: also form dq_bias and dk_bias.
template <class T, int NKR_, bool FOLD_, bool BG_>
struct WinCfg {
    static constexpr int NKD = 2, NKR = NKR_, NK = NKD + NKR_, NDV = 1, KBW = 1;
    static constexpr bool FOLD = FOLD_, BG = BG_ && NKR_ > 0, VEC = true, DO_DV = true, DO_DK = true;
    static constexpr int NWAVES = 8, NTHREADS = 64 * NWAVES;
    static constexpr int BN = 32 * NWAVES, LQ = 256, BMQ = 128, QBLK = BMQ / 32;
    static constexpr int ROWCH = 8;   // 128-byte rows: [Q | Q_b], [K | K_b]
    static constexpr int ROWCHS = 16; // 256-byte rows: the 128 queries of a key's dS
    static constexpr int MB = (NK + 1) / 2, MB0 = 0, MB1 = BG ? MB : 1; // 32-row blocks of [dK | dK_b]^T
    // 16-bit elements; the dO tile is a dense region of 64-byte rows (fb_lean_tiles.h)
    static constexpr int SQ = LQ * 64, SDO = LQ * 32, SK = BN * 64, SDS = BN * 128;
    static constexpr int STAT_FLOATS = 2 * LQ;
    static constexpr int LDS_BYTES = 2 * (SQ + SDO + SK + SDS) + 4 * STAT_FLOATS;
    static_assert(LDS_BYTES <= 160 * 1024, "");
};

template <class T, class C>
__global__ __launch_bounds__(C::NTHREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void bwd_win_kernel(const BwdArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint16_t *sQ = reinterpret_cast<uint16_t *>(smem), *sdO = sQ + C::SQ, *sK = sdO + C::SDO, *sdS = sK + C::SK;
    float *sStat = reinterpret_cast<float *>(sdS + C::SDS);
    // (LDS byte addresses of the tiles for the copy instructions, taken here once from the array itself)
    const uint32_t lds_q = lds_addr_of(smem), lds_do = lds_q + 2 * C::SQ, lds_k = lds_do + 2 * C::SDO;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // A workgroup walks `group` consecutive batch entries (the next one's tiles travel while this one computes).
    // With a.group > 1 their factor gradients are summed into row bg of the gradient tensors; otherwise the walk
    // is the launcher's choice (a.walk) and every entry's factor gradients are stored as its own rows.
    const bool summed = a.group > 1;
    const int group = summed ? a.group : (a.walk > 1 ? a.walk : 1);
    const int nbg = (a.B + group - 1) / group;
    const int work = xcd_remap(blockIdx.x, nbg * a.H);
    const int bg = work / a.H, h = work % a.H;
    const int wk0 = wave * 32; // first key of this wave
    const int nb = wave & 3;   // phase 2: this wave's query block of the step

    {   // clear LDS once: channel padding, and the dS rows of waves whose keys do not exist, are never written
        u32x4_t *z = reinterpret_cast<u32x4_t *>(smem);
        for (int i = tid; i < C::LDS_BYTES / 16; i += C::NTHREADS) z[i] = u32x4_t{0u, 0u, 0u, 0u};
    }
    __syncthreads();

    f32x16_t acc_dv[1][1], acc_dk[1][C::MB1], acc_dqb;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
#pragma unroll
        for (int n = 0; n < C::MB1; ++n) acc_dk[0][n][v] = 0.f;
        acc_dqb[v] = 0.f;
    }

    // The copies of a window, in halves of 128 rows so that a half can be refilled as soon as its step is over: per
    // half and wave two instructions (16 rows) of Q, two of Q_b, two of K, two of K_b and one (16 rows) of dO.
    typedef TileDma<128, C::ROWCH, C::NWAVES, (C::NKR > 0)> Copy;
    Copy cq;
    cq.init(a.q.ptr, a.q.ss, a.d, 2 * C::NKD, C::NKR > 0 ? a.qb.ptr : nullptr, C::NKR > 0 ? a.qb.ss : 0, a.r, wave, lane, 0);
    uint32_t do_off[2]; // (rows past the end step back to the last one)
    {
        int row, chunk;
        lean_copy_place<4>(lane, row, chunk);
#pragma unroll
        for (int hf = 0; hf < 2; ++hf)
            do_off[hf] = (uint32_t)(min(128 * hf + 16 * wave + row, a.Lq - 1) * (int)(a.dout.ss * 2) + chunk * 16);
    }
    // One tensor's two instructions for rows [128 hf, 128 hf + 128) of a [X | X_b] tile (second: the factor part).
    auto copy_half = [&](const Copy &cp, const uint16_t *base, int64_t ld, uint32_t lds_tile, int hf, int nrows, bool second) {
        const uint8_t *src = reinterpret_cast<const uint8_t *>(base) + (int64_t)(128 * hf) * ld * 2;
#pragma unroll
        for (int j = 0; j < Copy::NI; ++j) {
            uint32_t off = cp.off[j];
            if (128 * hf + 128 > nrows) { // a ragged half: rows past the end re-read the last row
                const int r = ((wave * Copy::NI + j) * 64 + (int)(threadIdx.x & 63)) / C::ROWCH;
                off -= (uint32_t)max(128 * hf + r - (nrows - 1), 0) * (uint32_t)(ld * 2);
            }
            // (the LDS address is wave-uniform; said again for the compiler, which must hand the copy a scalar)
            const uint32_t dst = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds_tile + hf * 16384 + (wave * Copy::NI + j) * 1024));
            lds_dma16_lanes(off, src, dst, second ? cp.lanes_b[j] : cp.lanes_a[j]);
        }
    };

    const float to_log2 = C::FOLD ? a.scale * kLog2e : kLog2e;
    const int nsteps = (a.Lq + C::BMQ - 1) / C::BMQ;
    const bool visible = wk0 < a.Lk;

    // What a window needs from global memory, requested piece by piece while the previous window computes (a wave
    // that issues many copies at once waits for the memory pipeline to take them):
    //   queries(b, hf, part): rows [128 hf, 128 hf + 128) of Q (part 0), Q_b (1), dO (2) into their tiles
    //   operands(b):          K, K_b and V of this lane's key into registers (B operands of S and dP; the [K | K_b] tile
    //                         that phase 2 reads column-wise is written from them)
    //   stat_inputs(b):       for the statistics of the 32 queries whose dO rows this wave copies: 16 channels of o
    //                         per lane, and the lse
    u32x4_t kreg[C::NK], vreg[C::NKD], so[2];
    float slse;
    // the query whose statistics this lane helps with: one of the rows of dO that its wave copies (16 of each half)
    const int srow = 128 * (lane >> 5) + 16 * wave + ((lane >> 1) & 15);
    auto queries = [&](int b, int hf, int part) {
        if (128 * hf >= a.Lq) return;
        if (part == 0) copy_half(cq, a.q.ptr + b * a.q.sb + h * a.q.sh, a.q.ss, lds_q, hf, a.Lq, false);
        if constexpr (C::NKR > 0) {
            if (part == 1) copy_half(cq, a.qb.ptr + b * a.qb.sb + h * a.qb.sh, a.qb.ss, lds_q, hf, a.Lq, true);
        }
        if (part == 2) {
            // (wave-uniform by construction; said again for the compiler, which must hand the copy a scalar base)
            const uint64_t db = reinterpret_cast<uint64_t>(a.dout.ptr + b * a.dout.sb + h * a.dout.sh);
            const void *dobase = reinterpret_cast<const void *>(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(db >> 32)) << 32) |
                                                                (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)db));
            lds_dma16_all(do_off[hf], dobase, (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds_do + (8 * hf + wave) * 1024)));
        }
    };
    // (plain loads, nothing that would make the wave wait for them here: keys past the end read the last key, whose
    // scores are hidden later, and factor channels past the rank read chunk 0 and are cleared where the window starts)
    auto operands = [&](int b) {
        const int key = min(wk0 + (int)(threadIdx.x & 31), a.Lk - 1), g = (threadIdx.x >> 5) & 1;
        const uint16_t *krow = a.k.ptr + b * a.k.sb + h * a.k.sh + (int64_t)key * a.k.ss + 8 * g;
        const uint16_t *vrow = a.v.ptr + b * a.v.sb + h * a.v.sh + (int64_t)key * a.v.ss + 8 * g;
#pragma unroll
        for (int t = 0; t < C::NKD; ++t) {
            kreg[t] = *reinterpret_cast<const u32x4_t *>(krow + 16 * t);
            vreg[t] = *reinterpret_cast<const u32x4_t *>(vrow + 16 * t);
        }
        if constexpr (C::NKR > 0) {
            const uint16_t *kbrow = a.kb.ptr + b * a.kb.sb + h * a.kb.sh + (int64_t)key * a.kb.ss;
#pragma unroll
            for (int t = 0; t < C::NKR; ++t) kreg[C::NKD + t] = *reinterpret_cast<const u32x4_t *>(kbrow + (16 * t + 8 * g < a.r ? 16 * t + 8 * g : 0));
        }
    };
    auto stat_inputs = [&](int b) {
        const int rr = min(srow, a.Lq - 1), ch = 16 * (threadIdx.x & 1);
        const uint16_t *orow = a.o.ptr + b * a.o.sb + h * a.o.sh + (int64_t)rr * a.o.ss + ch;
#pragma unroll
        for (int j = 0; j < 2; ++j) so[j] = *reinterpret_cast<const u32x4_t *>(orow + 8 * j);
        slse = a.lse[((int64_t)b * a.H + h) * a.Lq + rr];
    };
    // dk_bias (one accumulator block per wave, its keys) and dq_bias (one block per wave: queries
    // 128 (wave / 4) + 32 (wave % 4) ..) into row `row_b` of the gradient tensors
    auto factor_gradients = [&](int row_b) {
        if constexpr (C::BG) {
            const int lane_end = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
            const int c = lane_end & 31, g = lane_end >> 5;
            dkv_store<T, C, true>(a, acc_dv, acc_dk, row_b, h, wk0, c, g);
            const int query = C::BMQ * (wave >> 2) + 32 * nb + c;
            const bool ok = query < a.Lq;
            uint16_t *row = const_cast<uint16_t *>(a.dqb.ptr) + row_b * a.dqb.sb + h * a.dqb.sh + (int64_t)(ok ? query : 0) * a.dqb.ss;
            store_acc_rows<T, true>(row, ok, a.dqb.vec_ok, acc_dqb, 1.f, a.r, g);
        }
    };
    if (bg * group < a.B) { // the first window of the workgroup: everything at once
        const int b0 = __builtin_amdgcn_readfirstlane(bg * group);
#pragma unroll
        for (int hf = 0; hf < 2; ++hf)
#pragma unroll
            for (int part = 0; part < 3; ++part) queries(b0, hf, part);
        operands(b0);
        stat_inputs(b0);
    }

    for (int bi = 0; bi < group; ++bi) {
        const int b = __builtin_amdgcn_readfirstlane(bg * group + bi);
        if (b >= a.B) break;
        int tid_again = threadIdx.x; // (opaque: what derives from the lane id is recomputed per window, not kept in registers)
        asm volatile("" : "+v"(tid_again));
        const int tid = tid_again, lane = tid & 63, c = lane & 31, g = lane >> 5;
        const int key = wk0 + c;

        // ---- this window.  The first half of its query-side tiles, its register operands and the inputs of its
        // statistics were requested during the previous window (or above); every wave has left the previous window's
        // [K | K_b] and dS tiles and its statistics (the barrier that ends a step).
        const bool next = bi + 1 < group && b + 1 < a.B;
        const int bn = __builtin_amdgcn_readfirstlane(b + 1);
        // Everything requested for this window has landed (what this waits for beyond that are the few stores of the
        // previous window's last step).
        wait_vmcnt<0>();
        {   // the per-query statistics (_bwd_preprocess_do_o_dot, flash_bias_triton.py:358-400) of the 32 queries whose dO
            // rows this wave copied itself (so that it may read them without a barrier): lanes 2 i and 2 i + 1 sum the
            // channels [0, 16) and [16, 32) of o * dO of one query and add up; lse * log2(e) and -delta go to LDS.
            // Queries past the end get P = 0.
            const int half = tid & 1;
            const bool ok = srow < a.Lq;
            float sum = 0.f;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const u32x4_t sd = lds_load16(lds_do + lean_chunk_off<4>(srow, 2 * half + j));
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    sum = __builtin_fmaf(T::to_float((uint16_t)(so[j][e] & 0xffffu)), T::to_float((uint16_t)(sd[e] & 0xffffu)), sum);
                    sum = __builtin_fmaf(T::to_float((uint16_t)(so[j][e] >> 16)), T::to_float((uint16_t)(sd[e] >> 16)), sum);
                }
            }
            const float other = __shfl_xor(sum, 1, 64);
            const float delta = half == 0 ? sum + other : other + sum; // (the same order in both lanes)
            if (half == 0) {
                sStat[srow] = ok ? slse * kLog2e : INFINITY;
                sStat[C::LQ + srow] = ok ? -delta : 0.f;
            }
        }
        // the [K | K_b] tile, row `key` from this lane's register operands (factor channels past the rank cleared
        // first; keys past the end hold the last key, whose dS is zero)
        if constexpr (C::NKR > 0) {
#pragma unroll
            for (int t = 0; t < C::NKR; ++t)
                if (16 * t + 8 * g >= a.r) kreg[C::NKD + t] = u32x4_t{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int t = 0; t < C::NK; ++t) *reinterpret_cast<u32x4_t *>(sK + swz_off<C::ROWCH>(key, 2 * t + g)) = kreg[t];
        barrier_lds();
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            acc_dv[0][0][v] = 0.f;
            acc_dk[0][0][v] = 0.f; // (block 0 is dk; block 1, dk_bias, runs on over the group)
        }
        const uint32_t do_lds = lds_do;
        const uint32_t do_row[2] = {do_lds + lean_row_addr<4>(c, g), do_lds + lean_row_addr<4>(c, 2 + g)};
        const uint32_t do_col[2] = {do_lds + lean_tr_addr4(c, g, 0), do_lds + lean_tr_addr4(c, g, 1)};

#pragma unroll 1
        for (int step = 0; step < nsteps; ++step) {
            const int m0 = step * C::BMQ;
            // ---- phase 1: this wave's 32 keys against the step's 128 queries
            {
#pragma unroll 1
                for (int qb = 0; qb < C::QBLK; ++qb) {
                    const int r0 = m0 + qb * 32;
                    // a slice of the copies that may run now: during the second step the first half of the next window's
                    // query-side tiles (its rows are no longer read)
                    if (step == 1 && next && qb < 3) queries(bn, 0, qb);
                    if (!visible || r0 >= a.Lq) continue;
                    u32x4_t qa[C::NK], da[C::NKD];
#pragma unroll
                    for (int t = 0; t < C::NK; ++t) qa[t] = *reinterpret_cast<const u32x4_t *>(sQ + swz_off<C::ROWCH>(r0 + c, 2 * t + g));
#pragma unroll
                    for (int t = 0; t < C::NKD; ++t) da[t] = lds_load16(do_row[t] + (r0 >> 5) * 2048);
                    f32x16_t s, dp;
                    float lse2[16];
#pragma unroll
                    for (int bq = 0; bq < 4; ++bq) { // register v <-> query r0 + 8 (v / 4) + 4 g + v % 4
                        const f32x4_t l4 = *reinterpret_cast<const f32x4_t *>(sStat + r0 + 8 * bq + 4 * g);
                        const f32x4_t d4 = *reinterpret_cast<const f32x4_t *>(sStat + C::LQ + r0 + 8 * bq + 4 * g);
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            lse2[4 * bq + e] = l4[e];
                            dp[4 * bq + e] = d4[e];
                        }
                    }
#pragma unroll
                    for (int v = 0; v < 16; ++v) s[v] = 0.f;
#pragma unroll
                    for (int t = 0; t < C::NKD; ++t) s = T::mfma(qa[t], kreg[t], s);
#pragma unroll
                    for (int t = 0; t < C::NKD; ++t) dp = T::mfma(da[t], vreg[t], dp);
                    if constexpr (!C::FOLD) { // the softmax scale multiplies q k^T only (flash_bias_triton.py:248)
#pragma unroll
                        for (int v = 0; v < 16; ++v) s[v] *= a.scale;
                    }
#pragma unroll
                    for (int t = C::NKD; t < C::NK; ++t) s = T::mfma(qa[t], kreg[t], s);
                    if (wk0 + 32 > a.Lk) {
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            if (key >= a.Lk) s[v] = -INFINITY;
                    }
                    // (The vector instructions below read what the matrix instructions above have just written, which
                    // takes wait states that the compiler inserts along straight-line code; here the two can meet
                    // across the loop's branches, where it was seen to leave them out: they are spelt out.)
                    asm volatile("s_nop 11" : "+v"(s), "+v"(dp));
                    u32x4_t pp[2], pds[2]; // P and dS, packed, per 16-query step
#pragma unroll
                    for (int v = 0; v < 16; v += 2) {
                        const float p0 = fast_exp2(__builtin_fmaf(s[v], to_log2, -lse2[v]));
                        const float p1 = fast_exp2(__builtin_fmaf(s[v + 1], to_log2, -lse2[v + 1]));
                        pp[v >> 3][(v & 7) >> 1] = T::pack2(p0, p1);
                        pds[v >> 3][(v & 7) >> 1] = T::pack2(p0 * dp[v], p1 * dp[v + 1]);
                    }
                    // dS of (this key, queries r0 + 16 t + 8 half + 4 g + 0..3) -> row `key` of the dS tile
#pragma unroll
                    for (int t = 0; t < 2; ++t)
#pragma unroll
                        for (int half = 0; half < 2; ++half)
                            *reinterpret_cast<u32x2_t *>(sdS + swz_off<C::ROWCHS>(key, 4 * qb + 2 * t + half) + 4 * g) =
                                u32x2_t{pds[t][2 * half], pds[t][2 * half + 1]};
                    // dV^T += dO^T P ; [dK | dK_b]^T += [Q | Q_b]^T dS  (contraction over this block's queries)
#pragma unroll
                    for (int t = 0; t < 2; ++t) {
                        const u32x4_t dot = lds_load_tr(do_col[0] + ((r0 >> 4) + t) * 1024, do_col[1] + ((r0 >> 4) + t) * 1024);
                        acc_dv[0][0] = T::mfma(dot, pp[t], acc_dv[0][0]);
#pragma unroll
                        for (int n = 0; n < C::MB1; ++n) {
                            const u32x4_t qt = lds_read_a_tr<C::ROWCH>(sQ, r0 + 16 * t, 32 * n, c, g);
                            acc_dk[0][n] = T::mfma(qt, pds[t], acc_dk[0][n]);
                        }
                    }
                }
            }
            barrier_lds(); // the step's dS tile is complete
            if (step == nsteps - 1) {
                // dv and dk (times scale) of this window are final and K, K_b, V in registers no longer needed: the
                // next window's are requested now and arrive during phase 2
                dkv_store<T, C, false>(a, acc_dv, acc_dk, b, h, wk0, c, g);
                if (next) {
                    operands(bn);
                    // the rows of the second half of the query-side tiles are free as well (with a single step: those
                    // of the first half, which had no second step to be spread over)
#pragma unroll
                    for (int part = 0; part < 3; ++part) queries(bn, nsteps == 1 ? 0 : 1, part);
                }
            }
            if (step == 0 && next) stat_inputs(bn);
            // ---- phase 2: one 32 x 32 block of [dQ | dQ_b]^T per wave, over all keys: queries m0 + 32 nb ..; the
            // step's dq_bias blocks (channels 32 ..) go to waves 4 step .. 4 step + 3, its dq blocks to the other four
            const bool bias_block = (wave >> 2) == step;
            if ((!bias_block || C::BG) && m0 + 32 * nb < a.Lq) {
                f32x16_t acc2;
#pragma unroll
                for (int v = 0; v < 16; ++v) acc2[v] = bias_block ? acc_dqb[v] : 0.f;
                const int col0 = bias_block ? 32 : 0;
#pragma unroll 4
                for (int key0 = 0; key0 < a.Lk; key0 += 16) {
                    const u32x4_t ka = lds_read_a_tr<C::ROWCH>(sK, key0, col0, c, g);
                    const u32x4_t db = lds_read_a_tr<C::ROWCHS>(sdS, key0, 32 * nb, c, g);
                    acc2 = T::mfma(ka, db, acc2);
                }
                asm volatile("s_nop 11" : "+v"(acc2)); // (as above: the loop's exit lies between the last product and its first reader)
                if (bias_block) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc_dqb[v] = acc2[v];
                } else {
                    const int query = m0 + 32 * nb + c;
                    const bool ok = query < a.Lq;
                    uint16_t *row = const_cast<uint16_t *>(a.dq.ptr) + b * a.dq.sb + h * a.dq.sh + (int64_t)(ok ? query : 0) * a.dq.ss;
                    store_acc_rows<T, true>(row, ok, a.dq.vec_ok, acc2, a.scale, a.d, g);
                }
            }
            barrier_lds(); // everyone has read the dS tile
        }
        if constexpr (C::BG) {
            if (!summed && a.dkb.ptr) { // this entry's own factor gradients; the accumulators start the next entry at zero
                factor_gradients(b);
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    acc_dqb[v] = 0.f;
#pragma unroll
                    for (int n = 1; n < C::MB1; ++n) acc_dk[0][n][v] = 0.f;
                }
            }
        }
    }

    // ---- the factor gradients, summed over the group's batch entries
    if constexpr (C::BG) {
        if (summed && a.dkb.ptr) factor_gradients(bg);
    }
}

template <class T, int NKR, bool FOLD, bool BG>
static hipError_t launch_win_cfg(const BwdArgs &a, hipStream_t stream) {
    typedef WinCfg<T, NKR, FOLD, BG> C;
    auto kern = bwd_win_kernel<T, C>;
    static KernelOnce once;
    const hipError_t e = allow_lds(kern, C::LDS_BYTES, once);
    if (e != hipSuccess) return e;
    BwdArgs b = a;
    b.walk = 1;
    if (a.group <= 1) // nothing to sum: walk as many entries as leave four workgroups per compute unit
        for (int w = 32; w > 1; w /= 2)
            if ((int64_t)((a.B + w - 1) / w) * a.H >= 4 * (int64_t)num_cus()) {
                b.walk = w;
                break;
            }
    const int group = a.group > 1 ? a.group : b.walk;
    return launch_flat(kern, (int64_t)((a.B + group - 1) / group) * a.H, C::NTHREADS, C::LDS_BYTES, stream, b);
}

template <class T, int NKR>
static hipError_t launch_win_r(const BwdArgs &a, hipStream_t stream) {
    const bool fold = a.r == 0 || a.scale == 1.f;
    const bool bg = NKR > 0 && a.dqb.ptr;
    if (fold) return bg ? launch_win_cfg<T, NKR, true, true>(a, stream) : launch_win_cfg<T, NKR, true, false>(a, stream);
    return bg ? launch_win_cfg<T, NKR, false, true>(a, stream) : launch_win_cfg<T, NKR, false, false>(a, stream);
}

// Compiled once per element type for head dim 32 (see Makefile).  When fb_bwd takes this path is decided by
// window_backward() in fb_kernels.h; the statistics must be in the scratch buffer (preprocess step).
#define FB_CAT2(a, b) a##b
#define FB_CAT(a, b) FB_CAT2(a, b)
hipError_t FB_CAT(launch_bwd_win_, FB_SUFFIX)(const BwdArgs &a, hipStream_t stream) {
    switch (nkr_of(a.r)) {
    case 0: return launch_win_r<FB_T, 0>(a, stream);
    case 1: return launch_win_r<FB_T, 1>(a, stream);
    default: return launch_win_r<FB_T, 2>(a, stream);
    }
}

} // namespace fb
