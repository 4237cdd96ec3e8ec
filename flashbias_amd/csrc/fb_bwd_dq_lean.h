// Streamlined dq / dq_bias kernel for the shapes the benchmark family lives on: aligned tensors, no
// additive mask, head dim 32, rank 8 (or no factors).  Included by fb_bwd_dq.hip after the general
// kernel, whose algebra it shares (query-stationary, lane = query, register = key); it differs in
// the same ways as the streamlined dk/dv kernel (fb_bwd_dkv_lean.h):
//
//   * the softmax scale and log2(e) are folded into the resident query operand (q -> rn(q * scale *
//     log2 e), q_b -> hi + lo parts of q_b * log2 e against two copies of k_b), and the two chains
//     start from accumulator blocks that hold -lse * log2(e) and -delta of the lane's query (the
//     same for every key): the MFMAs deliver the exponent of 2 and dP - delta directly, the VALU is
//     left with exp2, one multiply and half a convert per score;
//   * every block step is a fixed sequence of 9 slots, each one MFMA followed by four VALU
//     instructions and at most one LDS request: the two chains of the next 32 x 32 block, the second
//     half of the previous block's accumulation and the first half of this one's alternate between
//     the exponentials of this block, and every LDS fragment is requested four to seven slots
//     before its use;
//   * [K], [K_b | K_b] and V of 64 keys are copied straight from global memory into a ring of six
//     dense LDS stages, three tiles ahead, by whole-wave copies.
#pragma once
#include <type_traits>

#include "fb_lean_tiles.h"

namespace fb {

// BG_: also accumulate and store dq_bias (false: the caller does not want the factor gradients).
template <class T, int NKR_, bool BG_ = true>
struct DqLeanCfg {
    static constexpr int NKR = NKR_;
    static constexpr bool BG = BG_ && NKR_ > 0;
    static_assert(NKR_ <= 1, "rank 8 or none");
    static constexpr int NWAVES = 4, NTHREADS = 256, BM = 128, BN = 64;
    static constexpr int K_BYTES = BN * 64, B_BYTES = BN * 32, V_BYTES = BN * 64;
    static constexpr int B_OFF = K_BYTES, V_OFF = B_OFF + B_BYTES, STAGE_BYTES = V_OFF + V_BYTES;
    static constexpr int NSTAGE = 6;
    static constexpr int LDS_BYTES = NSTAGE * STAGE_BYTES;
    // copy instructions per wave and tile: one of K (16 rows), one of V, one of K_b (32 rows: waves
    // 2 and 3 repeat the copies of waves 0 and 1, so that every wave waits for the same count)
    static constexpr int NDMA = 2 + (NKR_ ? 1 : 0);
    // the general configuration a workgroup falls back to (same 128 queries per workgroup)
    typedef DqCfg<T, 2, NKR_, true, false, false, false, false> General;
    static_assert(General::BM == BM && General::LDS_BYTES <= LDS_BYTES, "");
};

template <class T, class C>
__device__ __attribute__((noinline)) void dq_lean_retry(const void *kernargs, int wg) {
    const BwdArgs a = uniform_kernargs<BwdArgs>(kernargs);
    bwd_dq_body<T, typename C::General>(a, __builtin_amdgcn_readfirstlane(wg));
}

// The whole streamlined dq computation of workgroup `wg` of the launch (the kernel below is nothing else; a
// launch that mixes dq and dk/dv workgroups calls it with its own numbering).  `kernargs`: where the kernel's
// argument block lives, for the out-of-line fallback.
template <class T, class C>
__device__ __forceinline__ void bwd_dq_lean_body(const BwdArgs &a, int wg, const void *kernargs) {
    constexpr int NKR = C::NKR;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 31, g = lane >> 5;

    const int total = a.ntiles_m * a.B * a.H;
    int bh, tile_m;
    work_order(wg, a.ntiles_m, total, a.causal, bh, tile_m);
    if (a.causal) tile_m = a.ntiles_m - 1 - tile_m; // the last query tile sees the most keys
    const int b = bh / a.H, h = bh % a.H;
    const int m0 = tile_m * C::BM;
    const int query = m0 + 32 * wave + c; // this lane's query
    const bool ok = query < a.Lq;

    const uint8_t *kptr = reinterpret_cast<const uint8_t *>(a.k.ptr + b * a.k.sb + h * a.k.sh);
    const uint8_t *vptr = reinterpret_cast<const uint8_t *>(a.v.ptr + b * a.v.sb + h * a.v.sh);
    const uint8_t *kbptr = nullptr;
    if constexpr (NKR > 0) kbptr = reinterpret_cast<const uint8_t *>(a.kb.ptr + b * a.kb.sb + h * a.kb.sh);

    // ---- resident query operands (queries past the end are zero; their lanes store nothing)
    const float cq = a.scale * kLog2e;
    u32x4_t qr[2], dor[2], qbr = {0u, 0u, 0u, 0u};
    bool bad = false; // a folded operand that left the 16-bit range: the general kernel takes the tile
    {
        const uint16_t *qbase = a.q.ptr + b * a.q.sb + h * a.q.sh;
        const uint16_t *dobase = a.dout.ptr + b * a.dout.sb + h * a.dout.sh;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const u32x4_t raw = load_chunk<true>(qbase, a.q.ss, query, a.Lq, 16 * t + 8 * g, a.d);
            qr[t] = fold_scale_chunk<T>(raw, cq, false, false);
            bad |= chunk_has_inf<T>(qr[t]) && !chunk_has_inf<T>(raw);
            dor[t] = load_chunk<true>(dobase, a.dout.ss, query, a.Lq, 16 * t + 8 * g, a.d);
        }
        if constexpr (NKR > 0) { // columns 8..15 of the bias step face the second copy of k_b: low-order parts
            const u32x4_t raw = load_chunk<true>(a.qb.ptr + b * a.qb.sb + h * a.qb.sh, a.qb.ss, query, a.Lq, 0, a.r);
            qbr = fold_scale_chunk<T>(raw, kLog2e, true, g == 1);
            bad |= chunk_has_inf<T>(qbr) && !chunk_has_inf<T>(raw);
        }
    }
    if (__syncthreads_or(bad)) {
        dq_lean_retry<T, C>(kernargs, wg);
        return;
    }
    // -lse * log2(e) and -delta of this lane's query
    float nd, l2;
    {
        const int64_t sidx = (int64_t)bh * a.Lq + (ok ? query : a.Lq - 1);
        if (a.stats_here) {
            // delta = rowsum(o * dO) (flash_bias_triton.py:358-400) from the dO chunks the lane holds and
            // the same chunks of o; the other half of the channels is with lane ^ 32.  Summed in the
            // order of the preprocess kernel (per 8-channel chunk, then pairwise over the chunks), so
            // that both ways of running the backward give the same bits.  Both values also go to the
            // scratch buffer, for the dk/dv kernel that follows.
            const uint16_t *obase = a.o.ptr + b * a.o.sb + h * a.o.sh;
            float cs[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const u32x4_t oc = load_chunk<true>(obase, a.o.ss, query, a.Lq, 16 * t + 8 * g, a.d);
                float acc1 = 0.f;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    acc1 = __builtin_fmaf(T::to_float((uint16_t)(oc[e] & 0xffffu)), T::to_float((uint16_t)(dor[t][e] & 0xffffu)), acc1);
                    acc1 = __builtin_fmaf(T::to_float((uint16_t)(oc[e] >> 16)), T::to_float((uint16_t)(dor[t][e] >> 16)), acc1);
                }
                cs[t] = acc1 + __shfl_xor(acc1, 32, 64); // chunks 2t and 2t + 1
            }
            cs[0] += cs[1];
            nd = ok ? -cs[0] : 0.f;
            l2 = ok ? a.lse[sidx] * kLog2e : INFINITY;
            if (ok && g == 0) {
                const int64_t rows = (int64_t)a.B * a.H * a.Lq;
                a.delta[sidx] = nd;
                a.delta[rows + sidx] = l2;
                if (a.stat_chunks) reinterpret_cast<u32x4_t *>(a.delta + stat_offset(rows))[sidx] = stat_chunk<T>(nd, l2);
            }
        } else { // the preprocess step left them in the scratch buffer
            l2 = ok ? a.delta[(int64_t)a.B * a.H * a.Lq + sidx] : INFINITY;
            nd = ok ? a.delta[sidx] : 0.f;
        }
    }
    // the initial values of the two chains, the same for every key (queries past the end: P = 0)
    f32x16_t init_s, init_dp;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        init_s[v] = -l2;
        init_dp[v] = nd;
    }

    int k_end = a.Lk;
    if (a.causal && m0 + C::BM < k_end) k_end = m0 + C::BM; // keys past the last query are hidden
    const int ntiles_k = (k_end + C::BN - 1) / C::BN;

    // ---- the copies.  Whole tiles take their source offsets from three registers; a ragged last
    // tile recomputes them with the rows past the end stepped back to the last one.
    const uint32_t lds0 = lds_addr_of(smem);
    LeanCopy4<C::BN> cp_k, cp_v;
    LeanCopy2<C::BN> cp_b;
    cp_k.init(wave, lane, a.k.ss);
    cp_v.init(wave, lane, a.v.ss);
    if constexpr (NKR > 0) cp_b.init(wave & 1, lane, a.kb.ss);
    auto issue = [&](int stage, int it) { // key tile `it` into a stage; exactly NDMA copy instructions
        const int n0 = it * C::BN, left = a.Lk - n0;
        const uint32_t sb = lds0 + stage * C::STAGE_BYTES;
        if (left >= C::BN) {
            lds_dma16_all(cp_k.off[0], kptr + (int64_t)n0 * cp_k.pitch, sb + wave * 1024);
            lds_dma16_all(cp_v.off[0], vptr + (int64_t)n0 * cp_v.pitch, sb + C::V_OFF + wave * 1024);
            if constexpr (NKR > 0) lds_dma16_all(cp_b.off, kbptr + (int64_t)n0 * cp_b.pitch, sb + C::B_OFF + (wave & 1) * 1024);
        } else {
            int l = lane;
            asm volatile("" : "+v"(l)); // (nothing of this path is worth a register across the loop)
            cp_k.issue(kptr + (int64_t)n0 * cp_k.pitch, sb, wave, l, left);
            cp_v.issue(vptr + (int64_t)n0 * cp_v.pitch, sb + C::V_OFF, wave, l, left);
            if constexpr (NKR > 0) cp_b.issue(kbptr + (int64_t)n0 * cp_b.pitch, sb + C::B_OFF, wave & 1, l, left);
        }
    };
    // at most `tiles` tiles' worth of this wave's copies still in flight
    auto wait_tiles = [&](int tiles) {
        if (tiles <= 0) wait_vmcnt<0>();
        else if (tiles == 1) wait_vmcnt<C::NDMA>();
        else wait_vmcnt<2 * C::NDMA>();
    };
    static_assert(C::NSTAGE == 6, "wait_tiles covers up to two tiles in flight behind the one awaited");
    // Tile j lives in stage j % NSTAGE.  The first NSTAGE - 2 tiles are requested here, tile
    // t + NSTAGE - 2 at the barrier that opens tile t, into the stage of tile t - 2: every LDS read
    // of that stage was consumed by an MFMA during tile t - 1 at the latest, so the barrier need
    // not wait for this wave's LDS reads in flight.
#pragma unroll
    for (int j = 0; j < C::NSTAGE - 2; ++j)
        if (j < ntiles_k) issue(j, j);
    wait_tiles(min(2, ntiles_k - 1)); // (waiting for more than asked is harmless)
    __syncthreads();

    // ---- this lane's read addresses (absolute LDS bytes); block and step are immediates.  Rows
    // are read one tile ahead of columns, so the two sets move through the stages separately.
    uint32_t rk[2], rb = 0, tq[2], tb[2][2];
#pragma unroll
    for (int t = 0; t < 2; ++t) rk[t] = lds0 + lean_row_addr<4>(c, 2 * t + g);
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
        rk[0] += delta;
        rk[1] += delta;
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

    // row fragments of one 32-key block (A operands of the chains): K (2), K_b | K_b, V (2); column
    // fragments of one 16-key step (A operands of the accumulation): K^T, [K_b | K_b]^T
    u32x4_t fk[2], fkb = {0u, 0u, 0u, 0u}, fv[2];
    u32x4_t ck = {0u, 0u, 0u, 0u}, ckb = {0u, 0u, 0u, 0u};
    auto read_rows_k = [&](int kb) {
#pragma unroll
        for (int t = 0; t < 2; ++t) fk[t] = lds_load16(rk[t] + kb * 2048);
        if constexpr (NKR > 0) fkb = lds_load16(rb + kb * 1024);
    };
    auto read_rows_v = [&](int kb) {
#pragma unroll
        for (int t = 0; t < 2; ++t) fv[t] = lds_load16(rk[t] + C::V_OFF + kb * 2048);
    };
    auto read_col_k = [&](int kb, int t) { ck = lds_load_tr(tq[0] + (2 * kb + t) * 1024, tq[1] + (2 * kb + t) * 1024); };
    auto read_col_b = [&](int kb, int t) {
        if constexpr (C::BG) ckb = lds_load_tr(tb[t][0] + kb * 1024, tb[t][1] + kb * 1024);
    };
    // -inf (p = 0) for keys past the end and pairs that a causal mask hides
    auto hide = [&](f32x16_t &s, int k0) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int key = k0 + 8 * (v >> 2) + 4 * g + (v & 3);
            if (key >= a.Lk || (a.causal && key > query)) s[v] = -INFINITY;
        }
    };
    // The 20 VALU instructions of one 16-key step t of a block, i = 0..19: eight exponentials
    // P = 2^s, eight products dS = P dp (dp is the last thing the chains deliver, so they come
    // late), the four converts of dS.
    float pe[8];
    auto vop = [&](const f32x16_t &s, const f32x16_t &dp, int t, int i, u32x4_t &pds) {
        if (i < 8) pe[i] = fast_exp2(s[8 * t + i]);
        else if (i < 16) pe[i - 8] *= dp[8 * t + i - 8];
        else pds[i - 16] = T::pack2(pe[2 * (i - 16)], pe[2 * (i - 16) + 1]);
    };

    const f32x16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    f32x16_t acc_dq = zero16, acc_dqb = zero16;
    u32x4_t pds0, pds1 = {0u, 0u, 0u, 0u};
    f32x16_t s0, dp0, s1, dp1;
    if (0 < ntiles_k) { // the chains of the very first block, and the row fragments of the second
        read_rows_k(0);
        read_rows_v(0);
        s0 = T::mfma(fk[0], qr[0], init_s);
        s0 = T::mfma(fk[1], qr[1], s0);
        if constexpr (NKR > 0) s0 = T::mfma(fkb, qbr, s0);
        dp0 = T::mfma(fv[0], dor[0], init_dp);
        dp0 = T::mfma(fv[1], dor[1], dp0);
        read_rows_k(1);
        read_rows_v(1);
    }
    rows_next_stage(C::STAGE_BYTES); // from here on the rows are those of the next tile

#define FB_SLOT_END __builtin_amdgcn_sched_barrier(0)
    // One block step: 9 slots of one MFMA, four VALU instructions and at most one LDS request.
    // (s, dp): this block, chains done; (sn, dpn): the next block, chains run here; pds1 and the
    // column fragments hold the second half of the previous block on entry and of this block on
    // exit.  Row requests are for the block after the next (same block index, next tile's stage).
    // A converted dS is never read by the MFMA of the slot that follows its conversion: the
    // accumulating MFMAs are opaque to the compiler's hazard handling (mfma_into).
    auto block = [&](const f32x16_t &s, const f32x16_t &dp, f32x16_t &sn, f32x16_t &dpn, int kb) {
        auto v4 = [&](int t, int i0, int n, u32x4_t &pds) {
#pragma unroll
            for (int i = i0; i < i0 + n; ++i) vop(s, dp, t, i, pds);
        };
        sn = T::mfma(fk[0], qr[0], init_s);
        v4(0, 0, 4, pds0);
        FB_SLOT_END;
        mfma_into<T>(acc_dq, ck, pds1);
        read_col_k(kb, 0);
        v4(0, 4, 4, pds0);
        FB_SLOT_END;
        sn = T::mfma(fk[1], qr[1], sn);
        v4(0, 8, 4, pds0);
        FB_SLOT_END;
        if constexpr (C::BG) mfma_into<T>(acc_dqb, ckb, pds1);
        read_col_b(kb, 0);
        v4(0, 12, 4, pds0);
        FB_SLOT_END;
        if constexpr (NKR > 0) sn = T::mfma(fkb, qbr, sn);
        v4(0, 16, 4, pds0);
        read_rows_k(kb);
        FB_SLOT_END;
        dpn = T::mfma(fv[0], dor[0], init_dp);
        v4(1, 0, 4, pds1);
        FB_SLOT_END;
        mfma_into<T>(acc_dq, ck, pds0);
        read_col_k(kb, 1);
        v4(1, 4, 4, pds1);
        FB_SLOT_END;
        dpn = T::mfma(fv[1], dor[1], dpn);
        v4(1, 8, 4, pds1);
        read_rows_v(kb);
        FB_SLOT_END;
        if constexpr (C::BG) mfma_into<T>(acc_dqb, ckb, pds0);
        read_col_b(kb, 1);
        v4(1, 12, 8, pds1);
        FB_SLOT_END;
    };

    int it = 0, stg = 0; // stg: the stage of tile `it` (columns); the rows are one stage ahead
    int turn = __builtin_amdgcn_readfirstlane(cu_slot());
    auto tile = [&](auto edge_tag) {
        constexpr bool EDGE = decltype(edge_tag)::value;
        const int n0 = it * C::BN;
        // tile it + 1 has landed (its rows are read from here on), everyone has left tile it - 1 and
        // has used what it read of tile it - 2
        wait_tiles(min(2, ntiles_k - 2 - it));
        asm volatile("s_barrier" ::: "memory");
        take_turn(turn, a.slots); // (the two workgroups of a compute unit swap wave priority at every tile, as in the forward)
        if (it + C::NSTAGE - 2 < ntiles_k) issue(stg < 2 ? stg + C::NSTAGE - 2 : stg - 2, it + C::NSTAGE - 2);
        if (EDGE) hide(s0, n0);
        FB_SLOT_END;
        block(s0, dp0, s1, dp1, 0);
        if (EDGE) hide(s1, n0 + 32);
        FB_SLOT_END;
        block(s1, dp1, s0, dp0, 1);
        cols_next_stage(stg == C::NSTAGE - 1 ? -(C::NSTAGE - 1) * C::STAGE_BYTES : C::STAGE_BYTES);
        rows_next_stage(stg == C::NSTAGE - 2 ? -(C::NSTAGE - 1) * C::STAGE_BYTES : C::STAGE_BYTES);
        stg = stg == C::NSTAGE - 1 ? 0 : stg + 1;
        ++it;
    };
    // Whole tiles below the diagonal first; the tiles on the diagonal of a causal call and a ragged
    // last tile, which hide something, come last.
    int nplain = a.Lk / C::BN;
    if (a.causal) nplain = min(nplain, m0 / C::BN);
    nplain = min(nplain, ntiles_k);
#pragma unroll 1
    while (it < nplain) tile(std::false_type{});
#pragma unroll 1
    while (it < ntiles_k) tile(std::true_type{});
    // the second half of the last block (two wait states after its conversion)
    asm volatile("s_nop 1" : "+v"(pds1));
    mfma_into<T>(acc_dq, ck, pds1);
    if constexpr (C::BG) mfma_into<T>(acc_dqb, ckb, pds1);
#undef FB_SLOT_END

    // ---- epilogue: dq (times scale) and dq_bias of this lane's query.  (The wait states let the
    // last accumulating MFMAs, which the compiler does not see as such, finish writing.)
    if constexpr (C::BG)
        asm volatile("s_nop 15\n\ts_nop 15" : "+v"(acc_dq), "+v"(acc_dqb));
    else
        asm volatile("s_nop 15\n\ts_nop 15" : "+v"(acc_dq));
    const int64_t qrow = ok ? query : 0;
    store_acc_rows<T, true>(const_cast<uint16_t *>(a.dq.ptr) + b * a.dq.sb + h * a.dq.sh + qrow * a.dq.ss, ok, a.dq.vec_ok, acc_dq,
                            a.scale, 32, g);
    if constexpr (C::BG) // rows 0..7 of the second accumulator block (8..15 repeat them)
        store_acc_rows<T, true>(const_cast<uint16_t *>(a.dqb.ptr) + b * a.dqb.sb + h * a.dqb.sh + qrow * a.dqb.ss, ok, a.dqb.vec_ok,
                                acc_dqb, 1.f, 8, g);
}

template <class T, class C>
__global__ __launch_bounds__(C::NTHREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void bwd_dq_lean_kernel(const BwdArgs a) {
    bwd_dq_lean_body<T, C>(a, blockIdx.x, (const void *)__builtin_amdgcn_kernarg_segment_ptr());
}

template <class T, int NKR, bool BG = true>
static hipError_t launch_dq_lean(const BwdArgs &a0, hipStream_t stream) {
    typedef DqLeanCfg<T, NKR, BG> C;
    BwdArgs a = a0;
    a.ntiles_m = (a.Lq + C::BM - 1) / C::BM;
    auto kern = bwd_dq_lean_kernel<T, C>;
    static KernelOnce once;
    const hipError_t e = allow_lds(kern, C::LDS_BYTES, once);
    if (e != hipSuccess) return e;
    const int64_t total = (int64_t)a.ntiles_m * a.B * a.H;
    a.slots = slots_per_cu(kern, C::NTHREADS, C::LDS_BYTES, total, once);
    return launch_flat(kern, total, C::NTHREADS, C::LDS_BYTES, stream, a);
}

} // namespace fb
