// Streamlined dk / dv / dk_bias kernel for the shapes the benchmark family lives on: aligned
// tensors, no additive mask, head dim 32, rank 8 (or no factors).  Included by fb_bwd_dkv.hip after
// the general kernel, whose algebra it shares (key-stationary, lane = key, register = query); what
// differs is the arithmetic per score and the way tiles reach LDS:
//
//   * the softmax scale and log2(e) are folded into the resident key operand (k -> rn(k * scale *
//     log2 e), k_b -> hi + lo parts of k_b * log2 e against two copies of q_b), so the chain of
//     MFMAs delivers the exponent of 2 directly;
//   * -lse * log2(e) and -delta enter the two chains as one more MFMA step: every query row carries
//     a 16-byte statistics chunk (stat_chunk, written by the dq kernel or the preprocess step)
//     whose parts face ones in a constant key-side operand.  No per-score FMA, no statistics in
//     registers: the VALU is left with exp2, one multiply and the two converts per score;
//   * every block step is a fixed sequence of 13 slots, each one MFMA followed by four VALU
//     instructions and at most one LDS request: the two chains of the next 32 x 32 block, the
//     second half of the previous block's accumulation and the first half of this one's are spread
//     between the exponentials of this block, so that both pipes always have independent work
//     within one wave, and every LDS fragment is requested at least six slots before its use;
//   * [Q], [Q_b | Q_b], dO and the statistics chunks of 64 queries are copied straight from global
//     memory into a ring of six dense LDS stages, three tiles ahead, by whole-wave copies.
#pragma once
#include <type_traits>

#include "fb_lean_tiles.h"

namespace fb {

// BG_: also accumulate and store dk_bias (false: the caller does not want the factor gradients, and the block
// step keeps its slots but two of them carry no MFMA and no transposing read).
template <class T, int NKR_, bool BG_ = true>
struct DkvLeanCfg {
    static constexpr int NKR = NKR_;
    static constexpr bool BG = BG_ && NKR_ > 0;
    static_assert(NKR_ <= 1, "rank 8 or none");
    static constexpr int NWAVES = 4, NTHREADS = 256, BN = 128, BM = 64;
    static constexpr int Q_BYTES = BM * 64, B_BYTES = BM * 32, AUX_BYTES = BM * 16, DO_BYTES = BM * 64;
    static constexpr int B_OFF = Q_BYTES, AUX_OFF = B_OFF + B_BYTES, DO_OFF = AUX_OFF + AUX_BYTES;
    static constexpr int STAGE_BYTES = DO_OFF + DO_BYTES;
    static constexpr int NSTAGE = 6;
    static constexpr int LDS_BYTES = NSTAGE * STAGE_BYTES;
    // copy instructions per wave and tile: one of Q (16 rows), one of dO, and one of Q_b (waves 0
    // and 1, 32 rows each) or of the statistics (wave 2, all 64 rows; wave 3 repeats it: every
    // wave then waits for the same count).  Without factors waves 0 and 1 copy statistics too.
    static constexpr int NDMA = 3;
    // the general configuration a workgroup falls back to (same 128 keys per workgroup)
    typedef DkvCfg<T, 2, NKR_, 1, true, false, 0, false> General;
    static_assert(General::BN == BN && General::LDS_BYTES <= LDS_BYTES, "");
};

template <class T, class C>
__device__ __attribute__((noinline)) void dkv_lean_retry(const void *kernargs, int wg) {
    const BwdArgs a = uniform_kernargs<BwdArgs>(kernargs);
    bwd_dkv_body<T, typename C::General>(a, __builtin_amdgcn_readfirstlane(wg));
}

// The whole streamlined dk/dv computation of workgroup `wg` of the launch (the kernel below is nothing else; a
// launch that mixes dq and dk/dv workgroups calls it with its own numbering).  `kernargs`: where the kernel's
// argument block lives, for the out-of-line fallback.
template <class T, class C>
__device__ __forceinline__ void bwd_dkv_lean_body(const BwdArgs &a, int wg, const void *kernargs) {
    constexpr int NKR = C::NKR;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 31, g = lane >> 5;

    const int total = a.ntiles_n * a.B * a.H;
    int bh, tile_n; // (causal: the first key tile sees the most queries)
    work_order(wg, a.ntiles_n, total, a.causal, bh, tile_n);
    const int b = bh / a.H, h = bh % a.H;
    const int n0 = tile_n * C::BN;
    const int key = n0 + 32 * wave + c; // this lane's key

    const uint8_t *qptr = reinterpret_cast<const uint8_t *>(a.q.ptr + b * a.q.sb + h * a.q.sh);
    const uint8_t *doptr = reinterpret_cast<const uint8_t *>(a.dout.ptr + b * a.dout.sb + h * a.dout.sh);
    const uint8_t *qbptr = nullptr;
    if constexpr (NKR > 0) qbptr = reinterpret_cast<const uint8_t *>(a.qb.ptr + b * a.qb.sb + h * a.qb.sh);
    const int64_t rows_all = (int64_t)a.B * a.H * a.Lq;
    const uint8_t *auxptr = reinterpret_cast<const uint8_t *>(a.delta + stat_offset(rows_all)) + (int64_t)bh * a.Lq * 16;

    // ---- resident key operands (keys past the end are zero; their lanes store nothing)
    const float cq = a.scale * kLog2e;
    u32x4_t kr[2], vr[2], kbr = {0u, 0u, 0u, 0u};
    bool bad = false; // a folded operand that left the 16-bit range: the general kernel takes the tile
    {
        const uint16_t *kbase = a.k.ptr + b * a.k.sb + h * a.k.sh;
        const uint16_t *vbase = a.v.ptr + b * a.v.sb + h * a.v.sh;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const u32x4_t raw = load_chunk<true>(kbase, a.k.ss, key, a.Lk, 16 * t + 8 * g, a.d);
            kr[t] = fold_scale_chunk<T>(raw, cq, false, false);
            bad |= chunk_has_inf<T>(kr[t]) && !chunk_has_inf<T>(raw);
            vr[t] = load_chunk<true>(vbase, a.v.ss, key, a.Lk, 16 * t + 8 * g, a.d);
        }
        if constexpr (NKR > 0) { // columns 8..15 of the bias step face the second copy of q_b: low-order parts
            const u32x4_t raw = load_chunk<true>(a.kb.ptr + b * a.kb.sb + h * a.kb.sh, a.kb.ss, key, a.Lk, 0, a.r);
            kbr = fold_scale_chunk<T>(raw, kLog2e, true, g == 1);
            bad |= chunk_has_inf<T>(kbr) && !chunk_has_inf<T>(raw);
        }
    }
    if (__syncthreads_or(bad)) {
        dkv_lean_retry<T, C>(kernargs, wg);
        return;
    }
    // ones against the parts of -lse * log2(e) (k-slots 0..2) and of -delta (k-slots 3..5)
    const uint32_t one = T::from_float(1.f);
    const u32x4_t ones_lse = g == 0 ? u32x4_t{one | (one << 16), one, 0u, 0u} : u32x4_t{0u, 0u, 0u, 0u};
    const u32x4_t ones_del = g == 0 ? u32x4_t{0u, one << 16, one | (one << 16), 0u} : u32x4_t{0u, 0u, 0u, 0u};

    // causal: the first query tile that can see this key tile (flash_bias_triton.py:498)
    const int tile0 = a.causal ? n0 / C::BM : 0;
    const int ntiles_m = (a.Lq + C::BM - 1) / C::BM;

    // ---- the copies.  Whole tiles take their source offsets from three registers; a ragged last
    // tile recomputes them with the rows past the end stepped back to the last one.
    const uint32_t lds0 = lds_addr_of(smem);
    const bool copies_b = NKR > 0 && wave < 2; // this wave's third copy: Q_b rows, else the statistics
    LeanCopy4<C::BM> cp_q, cp_do;
    LeanCopy2<C::BM> cp_b;
    cp_q.init(wave, lane, a.q.ss);
    cp_do.init(wave, lane, a.dout.ss);
    if constexpr (NKR > 0) cp_b.init(wave, lane, a.qb.ss);
    const uint32_t off3 = copies_b ? cp_b.off : (uint32_t)(lane * 16);
    auto issue = [&](int stage, int it) { // query tile `it` into a stage; exactly NDMA copy instructions
        const int m0 = it * C::BM, left = a.Lq - m0;
        const uint32_t sb = lds0 + stage * C::STAGE_BYTES;
        const uint8_t *src3 = copies_b ? qbptr + (int64_t)m0 * cp_b.pitch : auxptr + (int64_t)m0 * 16;
        const uint32_t dst3 = copies_b ? sb + C::B_OFF + wave * 1024 : sb + C::AUX_OFF;
        if (left >= C::BM) {
            lds_dma16_all(cp_q.off[0], qptr + (int64_t)m0 * cp_q.pitch, sb + wave * 1024);
            lds_dma16_all(cp_do.off[0], doptr + (int64_t)m0 * cp_do.pitch, sb + C::DO_OFF + wave * 1024);
            lds_dma16_all(off3, src3, dst3);
        } else {
            int l = lane;
            asm volatile("" : "+v"(l)); // (nothing of this path is worth a register across the loop)
            cp_q.issue(qptr + (int64_t)m0 * cp_q.pitch, sb, wave, l, left);
            cp_do.issue(doptr + (int64_t)m0 * cp_do.pitch, sb + C::DO_OFF, wave, l, left);
            if (copies_b) {
                if constexpr (NKR > 0) cp_b.issue(qbptr + (int64_t)m0 * cp_b.pitch, sb + C::B_OFF, wave, l, left);
            } else {
                lds_dma16_all((uint32_t)(min(l, left - 1) * 16), src3, dst3);
            }
        }
    };
    // at most `tiles` tiles' worth of this wave's copies still in flight
    auto wait_tiles = [&](int tiles) {
        if (tiles <= 0) wait_vmcnt<0>();
        else if (tiles == 1) wait_vmcnt<C::NDMA>();
        else wait_vmcnt<2 * C::NDMA>();
    };
    static_assert(C::NSTAGE == 6, "wait_tiles covers up to two tiles in flight behind the one awaited");
    // Tile tile0 + j lives in stage j % NSTAGE.  The first NSTAGE - 2 tiles are requested here, tile
    // t + NSTAGE - 2 at the barrier that opens tile t, into the stage of tile t - 2: every LDS read
    // of that stage was consumed by an MFMA during tile t - 1 at the latest, so the barrier need
    // not wait for this wave's LDS reads in flight (which would drain the fragment pipeline).
#pragma unroll
    for (int j = 0; j < C::NSTAGE - 2; ++j)
        if (tile0 + j < ntiles_m) issue(j, tile0 + j);
    wait_tiles(min(2, ntiles_m - 1 - tile0)); // (waiting for more than asked is harmless)
    __syncthreads();

    // ---- this lane's read addresses (absolute LDS bytes); block and step are immediates.  Rows
    // are read one tile ahead of columns, so the two sets move through the stages separately.
    uint32_t rq[2], rb = 0, ra, tq[2], tb[2][2];
#pragma unroll
    for (int t = 0; t < 2; ++t) rq[t] = lds0 + lean_row_addr<4>(c, 2 * t + g);
    ra = lds0 + C::AUX_OFF + 16 * c;
#pragma unroll
    for (int hi = 0; hi < 2; ++hi) tq[hi] = lds0 + lean_tr_addr4(c, g, hi);
    if constexpr (NKR > 0) {
        rb = lds0 + C::B_OFF + lean_row_addr<2>(c, g);
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int hi = 0; hi < 2; ++hi) tb[t][hi] = lds0 + C::B_OFF + lean_tr_addr2(c, g, hi, t);
    }
    auto rows_next_stage = [&](int delta) {
        ra += delta;
        rq[0] += delta;
        rq[1] += delta;
        if constexpr (NKR > 0) rb += delta;
    };
    auto cols_next_stage = [&](int delta) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            tq[t] += delta;
            if constexpr (NKR > 0) {
                tb[t][0] += delta;
                tb[t][1] += delta;
            }
        }
    };

    // row fragments of one 32-query block (A operands of the chains): Q (2), Q_b | Q_b, the
    // statistics chunk, dO (2); column fragments of one 16-query step (A operands of the
    // accumulation): dO^T, Q^T, [Q_b | Q_b]^T
    u32x4_t fq[2], fqb = {0u, 0u, 0u, 0u}, faux, fd[2];
    u32x4_t cd = {0u, 0u, 0u, 0u}, cq4 = {0u, 0u, 0u, 0u}, cqb = {0u, 0u, 0u, 0u};
    auto read_rows_s = [&](int qb) {
#pragma unroll
        for (int t = 0; t < 2; ++t) fq[t] = lds_load16(rq[t] + qb * 2048);
        if constexpr (NKR > 0) fqb = lds_load16(rb + qb * 1024);
    };
    auto read_rows_aux = [&](int qb) { faux = lds_load16(ra + qb * 512); };
    auto read_rows_d = [&](int qb) {
#pragma unroll
        for (int t = 0; t < 2; ++t) fd[t] = lds_load16(rq[t] + C::DO_OFF + qb * 2048);
    };
    auto read_col_d = [&](int qb, int t) { cd = lds_load_tr(tq[0] + C::DO_OFF + (2 * qb + t) * 1024, tq[1] + C::DO_OFF + (2 * qb + t) * 1024); };
    auto read_col_q = [&](int qb, int t) { cq4 = lds_load_tr(tq[0] + (2 * qb + t) * 1024, tq[1] + (2 * qb + t) * 1024); };
    auto read_col_b = [&](int qb, int t) {
        if constexpr (C::BG) cqb = lds_load_tr(tb[t][0] + qb * 1024, tb[t][1] + qb * 1024);
    };
    const f32x16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // -inf (p = 0) for queries past the end and pairs that a causal mask hides
    auto hide = [&](f32x16_t &s, int q0) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int query = q0 + 8 * (v >> 2) + 4 * g + (v & 3);
            if (query >= a.Lq || (a.causal && key > query)) s[v] = -INFINITY;
        }
    };
    // The 24 VALU instructions of one 16-query step t of a block, i = 0..23: eight exponentials
    // P = 2^s, the four converts of P, eight products dS = P dp (dp is the last thing the chains
    // deliver, so they come late), the four converts of dS.
    float pe[8];
    auto vop = [&](const f32x16_t &s, const f32x16_t &dp, int t, int i, u32x4_t &pp, u32x4_t &pds) {
        if (i < 8) pe[i] = fast_exp2(s[8 * t + i]);
        else if (i < 12) pp[i - 8] = T::pack2(pe[2 * (i - 8)], pe[2 * (i - 8) + 1]);
        else if (i < 20) pe[i - 12] *= dp[8 * t + i - 12];
        else pds[i - 20] = T::pack2(pe[2 * (i - 20)], pe[2 * (i - 20) + 1]);
    };

    f32x16_t acc_dv = zero16, acc_dk = zero16, acc_dkb = zero16;
    u32x4_t pp0, pds0, pp1 = {0u, 0u, 0u, 0u}, pds1 = {0u, 0u, 0u, 0u};
    f32x16_t s0, dp0, s1, dp1;
    if (tile0 < ntiles_m) { // the chains of the very first block, and the row fragments of the second
        read_rows_s(0);
        read_rows_aux(0);
        read_rows_d(0);
        s0 = T::mfma(fq[0], kr[0], zero16);
        s0 = T::mfma(fq[1], kr[1], s0);
        if constexpr (NKR > 0) s0 = T::mfma(fqb, kbr, s0);
        s0 = T::mfma(faux, ones_lse, s0);
        dp0 = T::mfma(faux, ones_del, zero16);
        dp0 = T::mfma(fd[0], vr[0], dp0);
        dp0 = T::mfma(fd[1], vr[1], dp0);
        read_rows_s(1);
        read_rows_aux(1);
        read_rows_d(1);
    }
    rows_next_stage(C::STAGE_BYTES); // from here on the rows are those of the next tile

#define FB_SLOT_END __builtin_amdgcn_sched_barrier(0)
    // One block step: 13 slots of one MFMA, four VALU instructions and at most one LDS request.
    // (s, dp): this block, chains done; (sn, dpn): the next block, chains run here; pp1 / pds1 and
    // the column fragments hold the second half of the previous block on entry and of this block
    // on exit.  Row requests are for the block after the next (same block index, next tile's stage).
    auto block = [&](const f32x16_t &s, const f32x16_t &dp, f32x16_t &sn, f32x16_t &dpn, int qb) {
        auto v4 = [&](int t, int i0, u32x4_t &pp, u32x4_t &pds) {
#pragma unroll
            for (int i = i0; i < i0 + 4; ++i) vop(s, dp, t, i, pp, pds);
        };
        mfma_into<T>(acc_dv, cd, pp1);
        read_col_d(qb, 0);
        v4(0, 0, pp0, pds0);
        FB_SLOT_END;
        sn = T::mfma(fq[0], kr[0], zero16);
        v4(0, 4, pp0, pds0);
        FB_SLOT_END;
        mfma_into<T>(acc_dk, cq4, pds1);
        read_col_q(qb, 0);
        v4(0, 8, pp0, pds0);
        FB_SLOT_END;
        sn = T::mfma(fq[1], kr[1], sn);
        v4(0, 12, pp0, pds0);
        FB_SLOT_END;
        if constexpr (C::BG) mfma_into<T>(acc_dkb, cqb, pds1);
        read_col_b(qb, 0);
        v4(0, 16, pp0, pds0);
        FB_SLOT_END;
        if constexpr (NKR > 0) sn = T::mfma(fqb, kbr, sn);
        v4(0, 20, pp0, pds0);
        read_rows_s(qb);
        FB_SLOT_END;
        mfma_into<T>(acc_dv, cd, pp0);
        read_col_d(qb, 1);
        v4(1, 0, pp1, pds1);
        FB_SLOT_END;
        sn = T::mfma(faux, ones_lse, sn);
        v4(1, 4, pp1, pds1);
        FB_SLOT_END;
        mfma_into<T>(acc_dk, cq4, pds0);
        read_col_q(qb, 1);
        v4(1, 8, pp1, pds1);
        FB_SLOT_END;
        dpn = T::mfma(faux, ones_del, zero16);
        v4(1, 12, pp1, pds1);
        read_rows_aux(qb);
        FB_SLOT_END;
        if constexpr (C::BG) mfma_into<T>(acc_dkb, cqb, pds0);
        read_col_b(qb, 1);
        v4(1, 16, pp1, pds1);
        FB_SLOT_END;
        dpn = T::mfma(fd[0], vr[0], dpn);
        v4(1, 20, pp1, pds1);
        FB_SLOT_END;
        dpn = T::mfma(fd[1], vr[1], dpn);
        read_rows_d(qb);
        FB_SLOT_END;
    };

    int it = tile0, stg = 0; // stg: the stage of tile `it` (columns); the rows are one stage ahead
    int turn = __builtin_amdgcn_readfirstlane(cu_slot());
    auto tile = [&](auto edge_tag) {
        constexpr bool EDGE = decltype(edge_tag)::value;
        const int m0 = it * C::BM;
        // tile it + 1 has landed (its rows are read from here on), everyone has left tile it - 1 and
        // has used what it read of tile it - 2
        wait_tiles(min(2, ntiles_m - 2 - it));
        asm volatile("s_barrier" ::: "memory");
        take_turn(turn, a.slots); // (the two workgroups of a compute unit swap wave priority at every tile, as in the forward)
        if (it + C::NSTAGE - 2 < ntiles_m) issue(stg < 2 ? stg + C::NSTAGE - 2 : stg - 2, it + C::NSTAGE - 2);
        if (EDGE) hide(s0, m0);
        FB_SLOT_END;
        block(s0, dp0, s1, dp1, 0);
        if (EDGE) hide(s1, m0 + 32);
        FB_SLOT_END;
        block(s1, dp1, s0, dp0, 1);
        cols_next_stage(stg == C::NSTAGE - 1 ? -(C::NSTAGE - 1) * C::STAGE_BYTES : C::STAGE_BYTES);
        rows_next_stage(stg == C::NSTAGE - 2 ? -(C::NSTAGE - 1) * C::STAGE_BYTES : C::STAGE_BYTES);
        stg = stg == C::NSTAGE - 1 ? 0 : stg + 1;
        ++it;
    };
    // Only the tiles on the diagonal of a causal call and a ragged last tile hide anything.
    const int ntiles_full = a.Lq / C::BM;
    const int diag_end = a.causal ? min(tile0 + C::BN / C::BM, ntiles_m) : tile0;
    while (it < diag_end) tile(std::true_type{});
#pragma unroll 1
    while (it < ntiles_full) tile(std::false_type{});
    if (it < ntiles_m) tile(std::true_type{});
    // the second half of the last block
    mfma_into<T>(acc_dv, cd, pp1);
    mfma_into<T>(acc_dk, cq4, pds1);
    if constexpr (C::BG) mfma_into<T>(acc_dkb, cqb, pds1);
#undef FB_SLOT_END

    // ---- epilogue: dv, dk (times scale), dk_bias of this lane's key.  (The wait states let the
    // last accumulating MFMAs, which the compiler does not see as such, finish writing.)
    if constexpr (C::BG)
        asm volatile("s_nop 15\n\ts_nop 15" : "+v"(acc_dv), "+v"(acc_dk), "+v"(acc_dkb));
    else
        asm volatile("s_nop 15\n\ts_nop 15" : "+v"(acc_dv), "+v"(acc_dk));
    const bool ok = key < a.Lk;
    const int64_t krow = ok ? key : 0;
    store_acc_rows<T, true>(const_cast<uint16_t *>(a.dv.ptr) + b * a.dv.sb + h * a.dv.sh + krow * a.dv.ss, ok, a.dv.vec_ok, acc_dv, 1.f,
                            32, g);
    store_acc_rows<T, true>(const_cast<uint16_t *>(a.dk.ptr) + b * a.dk.sb + h * a.dk.sh + krow * a.dk.ss, ok, a.dk.vec_ok, acc_dk,
                            a.scale, 32, g);
    if constexpr (C::BG) // rows 0..7 of the third accumulator block (8..15 repeat them)
        store_acc_rows<T, true>(const_cast<uint16_t *>(a.dkb.ptr) + b * a.dkb.sb + h * a.dkb.sh + krow * a.dkb.ss, ok, a.dkb.vec_ok,
                                acc_dkb, 1.f, 8, g);
}

template <class T, class C>
__global__ __launch_bounds__(C::NTHREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void bwd_dkv_lean_kernel(const BwdArgs a) {
    bwd_dkv_lean_body<T, C>(a, blockIdx.x, (const void *)__builtin_amdgcn_kernarg_segment_ptr());
}

template <class T, int NKR, bool BG = true>
static hipError_t launch_dkv_lean(const BwdArgs &a0, hipStream_t stream) {
    typedef DkvLeanCfg<T, NKR, BG> C;
    BwdArgs a = a0;
    a.ntiles_n = (a.Lk + C::BN - 1) / C::BN;
    auto kern = bwd_dkv_lean_kernel<T, C>;
    static KernelOnce once;
    const hipError_t e = allow_lds(kern, C::LDS_BYTES, once);
    if (e != hipSuccess) return e;
    const int64_t total = (int64_t)a.ntiles_n * a.B * a.H;
    a.slots = slots_per_cu(kern, C::NTHREADS, C::LDS_BYTES, total, once);
    return launch_flat(kern, total, C::NTHREADS, C::LDS_BYTES, stream, a);
}

} // namespace fb
