// Device-side building blocks shared by the forward and backward kernels (gfx950 only).
//
// MFMA tile used everywhere: v_mfma_f32_32x32x16_{bf16,f16}.  For a wave of 64 lanes with
// g = lane / 32 and c = lane % 32:
//   A operand (32 x 16): lane holds row c, eight consecutive k-slots of group g
//   B operand (16 x 32): lane holds column c, eight consecutive k-slots of group g
//   C / D    (32 x 32): lane holds column c, register v holds row 8*(v/4) + 4*g + v%4
// Only the C layout is relied on; the pairing of k-slots between A and B is whatever the
// hardware does, identical on both sides.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "fb_order.h"

namespace fb {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 f16x2_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2_t;

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct BF16 {
    typedef uint16_t raw;
    static __device__ __forceinline__ f32x16_t mfma(u32x4_t a, u32x4_t b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                       __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        bf16x2_t p;
        p[0] = (__bf16)lo;
        p[1] = (__bf16)hi;
        return __builtin_bit_cast(uint32_t, p);
    }
    static __device__ __forceinline__ float to_float(uint16_t x) {
        return __builtin_bit_cast(float, (uint32_t)x << 16);
    }
    static __device__ __forceinline__ uint16_t from_float(float x) {
        return __builtin_bit_cast(uint16_t, (__bf16)x);
    }
    static constexpr uint16_t kOne = 0x3f80;
    static constexpr bool kWideRange = true; // the exponent range of fp32
};

struct F16 {
    typedef uint16_t raw;
    static __device__ __forceinline__ f32x16_t mfma(u32x4_t a, u32x4_t b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a),
                                                      __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        f16x2_t p;
        p[0] = (_Float16)lo;
        p[1] = (_Float16)hi;
        return __builtin_bit_cast(uint32_t, p);
    }
    static __device__ __forceinline__ float to_float(uint16_t x) {
        return (float)__builtin_bit_cast(_Float16, x);
    }
    static __device__ __forceinline__ uint16_t from_float(float x) {
        return __builtin_bit_cast(uint16_t, (_Float16)x);
    }
    static constexpr uint16_t kOne = 0x3c00;
    static constexpr bool kWideRange = false;
};

// A (batch, seq, heads, channels) tensor as the kernels see it: 16-bit elements, channel
// stride 1, everything else through element strides.
struct Tensor {
    const uint16_t *ptr;
    int64_t sb, sh, ss;
    int vec_ok; // base pointer and all strides are multiples of 16 bytes
};

struct MaskDesc {
    const void *ptr;
    int64_t sb, sh, sm;
    int type;   // 0 none, 1 vector, 2 matrix
    int is_f32; // else same 16-bit type as the inputs
    int vec_ok; // base and strides allow aligned loads of four consecutive keys
};

// Eight consecutive channels [col0, col0 + 8) of row `row` of a (rows x ncols) matrix with row
// stride `ld`; zero beyond ncols and for row >= nrows.  Branch-free: out-of-range lanes read a
// clamped (valid) address and the result is zeroed by a select.  VEC = one 16-byte load
// (requires 16-byte aligned base / strides and ncols % 8 == 0), else eight 2-byte loads.
template <bool VEC>
__device__ __forceinline__ u32x4_t load_chunk(const uint16_t *base, int64_t ld, int row, int nrows, int col0,
                                              int ncols) {
    const bool row_ok = row < nrows;
    const uint16_t *rp = base + (int64_t)(row_ok ? row : nrows - 1) * ld;
    u32x4_t out;
    if constexpr (VEC) {
        const bool ok = row_ok && col0 < ncols;
        out = *reinterpret_cast<const u32x4_t *>(rp + (col0 < ncols ? col0 : 0));
#pragma unroll
        for (int i = 0; i < 4; ++i) out[i] = ok ? out[i] : 0u;
    } else {
        uint32_t e[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int col = col0 + i;
            uint32_t val = rp[col < ncols ? col : ncols - 1];
            asm volatile("" : "+v"(val)); // keep the load unconditional (no per-lane branch)
            e[i] = (row_ok && col < ncols) ? val : 0u;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) out[i] = e[2 * i] | (e[2 * i + 1] << 16);
    }
    return out;
}

// Kernels that fold the softmax scale into the contraction compute scale * (q k^T + q_b' k_b^T)
// with q_b' = q_b / scale (or k_b' = k_b / scale), the operand that stays in registers.  This
// turns eight 16-bit values x into rn(x * inv) or, with `split`, into two parts of x * inv: the
// high part hi (x * inv truncated to 16 bits) or, for `low`, the remainder rn(x * inv - hi).  A
// lane that owns otherwise unused (zero-padded) columns of the MFMA step carries the low parts
// there, against a second copy of the other operand's columns, which leaves a relative error of
// 2^-16 in the product.  Both parts have the sign of x and the low part of a non-zero value is
// never zero, so that a product with an infinite entry of the other operand (a key-padding
// column of -inf) is the same infinity in both halves instead of inf - inf or 0 * inf.
template <class T>
__device__ __forceinline__ u32x4_t fold_scale_chunk(u32x4_t x, float inv, bool split, bool low) {
    u32x4_t out;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        uint32_t w = 0;
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const float f = T::to_float((uint16_t)(hf ? x[e] >> 16 : x[e] & 0xffffu)) * inv;
            uint16_t hi = T::from_float(f);
            if (split) {
                if (fabsf(T::to_float(hi)) > fabsf(f)) hi -= 1; // one step towards zero (sign-magnitude encoding)
                if (low) {
                    const float h = T::to_float(hi);
                    uint16_t lo = (fabsf(h) == INFINITY) ? (uint16_t)0 : T::from_float(f - h);
                    if ((lo & 0x7fffu) == 0 && fabsf(h) != INFINITY) lo = T::from_float(h * 0x1p-24f);
                    hi = lo;
                }
            }
            w |= (uint32_t)hi << (16 * hf);
        }
        out[e] = w;
    }
    return out;
}

// True if any of the eight 16-bit values of a chunk is +-inf (or NaN).
template <class T>
__device__ __forceinline__ bool chunk_has_inf(u32x4_t x) {
    bool bad = false;
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const float f = T::to_float((uint16_t)(hf ? x[e] >> 16 : x[e] & 0xffffu));
            bad |= !(fabsf(f) <= 3.0e38f);
        }
    return bad;
}

// Per-query statistics of the backward pass as one 16-byte chunk of eight 16-bit values:
// -lse * log2(e) in k-slots 0..2 and -delta in k-slots 3..5, each as three parts (the value
// rounded to 16 bits, then twice the rounded remainder: 24 significant bits for bf16), zeros in
// slots 6, 7.  An MFMA step against ones in slots 0..2 (or 3..5) adds the value to an accumulator,
// which is how the streamlined backward kernels subtract lse and delta without touching the VALU.
// nd = -delta, l2 = lse * log2(e).
template <class T>
__device__ __forceinline__ u32x4_t stat_chunk(float nd, float l2) {
    uint32_t p[6];
    // (the values as they are stored in fp32, not an expression the compiler may still fuse into the
    // subtractions below: every writer of the scratch buffer must produce the same bits)
    asm volatile("" : "+v"(nd), "+v"(l2));
    float x = -l2;
#pragma unroll
    for (int i = 0; i < 6; ++i) {
        if (i == 3) x = nd;
        const uint16_t hi = T::from_float(x);
        p[i] = hi;
        x -= T::to_float(hi);
    }
    return u32x4_t{p[0] | (p[1] << 16), p[2] | (p[3] << 16), p[4] | (p[5] << 16), 0u};
}

// Position of key (or query) `x` of a 16-group inside an LDS row that feeds the A operand
// of an MFMA whose B operand comes straight from a C-layout register block: C rows
// 8b + 4g + c (b, g in {0,1}) must sit at slot 8g + 4b + c, i.e. bits 2 and 3 swap.
__device__ __forceinline__ int slot_of(int x) {
    return (x & ~12) | ((x & 4) << 1) | ((x & 8) >> 1);
}

// LDS tiles that are read both row-wise (16-byte chunk of one row per lane: A operand with
// rows = tile rows) and column-wise (ds_read_b64_tr_b16: A operand with rows = tile columns)
// keep one row-major copy whose 16-byte chunks are XOR-swizzled by row, so that both access
// patterns are free of bank conflicts.  ROWCH = chunks per row (8 -> 128-byte rows).
template <int ROWCH>
__device__ __forceinline__ int swz_of(int row) {
    // 128-byte rows: row bit 0 already selects the bank half, bits 1, 2, 3 swizzle three chunk
    // bits; longer rows are a multiple of all 64 banks, so bit 0 swizzles a fourth chunk bit
    const int s3 = ((row & 2) << 1) | ((row >> 2) & 1) | ((row >> 2) & 2);
    return ROWCH == 8 ? s3 : s3 | ((row & 1) << 3);
}
template <int ROWCH>
__device__ __forceinline__ int swz_off(int row, int chunk) { // element offset of a chunk
    return (row * ROWCH + (chunk ^ swz_of<ROWCH>(row))) * 8;
}

// Transposing LDS read.  Within each group of 16 lanes, lane 4a + b receives as element j the
// b-th 16-bit element of the 8 bytes that lane 4j + a points at.  With lane 4j + a pointing at
// tile[k0 + j][c0 + 4a ..], lane 4a + b gets tile[k0 .. k0 + 3][c0 + 4a + b]: four consecutive
// rows of one column.
__device__ __forceinline__ u32x2_t lds_read_tr4(const uint16_t *p) {
    typedef short v4s_t __attribute__((ext_vector_type(4)));
    const v4s_t r = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (v4s_t __attribute__((address_space(3))) *)(__attribute__((address_space(3))) const void *)p);
    return __builtin_bit_cast(u32x2_t, r);
}

// A operand (rows = 32 tile columns starting at col0, contraction over 16 tile rows starting
// at row0) for a B operand that comes straight from a C-layout register block: C-layout
// element i of half-wave g is row 8 (i / 4) + 4 g + i % 4 of the 16, so each lane needs two
// runs of four consecutive rows.
template <int ROWCH>
__device__ __forceinline__ u32x4_t lds_read_a_tr(const uint16_t *tile, int row0, int col0, int c, int g) {
    const int chunk = (col0 >> 3) + 2 * (c >> 4) + ((c & 3) >> 1), within = 4 * (c & 1);
    const int r = row0 + 4 * g + ((c & 15) >> 2);
    const u32x2_t lo = lds_read_tr4(tile + swz_off<ROWCH>(r, chunk) + within);
    const u32x2_t hi = lds_read_tr4(tile + swz_off<ROWCH>(r + 8, chunk) + within);
    return u32x4_t{lo[0], lo[1], hi[0], hi[1]};
}

// Direct global -> LDS copies (global_load_lds): lane i of the wave writes its 16 (or 4) bytes at
// LDS byte address `lds` + 16 i (4 i); `lds` must be wave-uniform; switched-off lanes write
// nothing.  They are issued through inline assembly so that the compiler's wait-count pass does
// not know them: it would make every later LDS read wait for all of them, and the point is to
// keep them in flight for more than one step.  The price: they count in vmcnt like any load, in
// issue order, and the kernel must wait for them itself (wait_vmcnt) before the barrier that
// publishes the data.
__device__ __forceinline__ uint32_t lds_addr_of(const void *p) {
    return (uint32_t)(size_t)(__attribute__((address_space(3))) const void *)p;
}
__device__ __forceinline__ void lds_dma16(const void *g, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds), "v"(g) : "memory");
}
// 16 bytes per lane from base + off (base wave-uniform, off a 32-bit byte offset per lane), with
// only the given lanes switched on.  All lanes of the wave must be active at the call.
__device__ __forceinline__ void lds_dma16_lanes(uint32_t off, const void *base, uint32_t lds, uint64_t lanes) {
    uint64_t saved;
    // (the base is wave-uniform by contract; said again here for pointers that run through nested loops, which the
    // compiler may keep in vector registers: a scalar operand is what the instruction takes)
    const uint64_t bb = reinterpret_cast<uint64_t>(base);
    // (readfirstlane returns a signed int: each half goes through uint32_t, or a low half with its top bit set
    // would sign-extend over the high half of the address)
    const uint64_t ub = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(bb >> 32)) << 32) |
                        (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)bb);
    asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, %4\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\t"
                 "global_load_lds_dwordx4 %1, %2\n\ts_mov_b64 exec, %0"
                 : "=&s"(saved)
                 : "v"(off), "s"(ub), "s"(lds), "s"(lanes)
                 : "memory");
}
__device__ __forceinline__ void lds_dma4(const void *g, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(lds), "v"(g) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() { // at most N vector memory loads of this wave still in flight
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
// Workgroup barrier that only waits for this wave's LDS operations (not for loads in flight).
__device__ __forceinline__ void barrier_lds() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// One wave's share of the direct copies that fill a swizzled LDS tile of ROWS rows x ROWCH
// 16-byte chunks from one or (HASB) two row-major tensors: chunks [0, split) of a tile row come
// from tensor A (channels 8 * chunk ..), chunks from `split` on from tensor B.  One copy
// instruction fills 64 consecutive chunk positions of the tile, each lane fetching the global
// chunk that the swizzle puts at its position; with two tensors there is one instruction per
// tensor and group of 64 positions, each with only that tensor's lanes switched on.  Lanes whose
// position is channel padding are never switched on (those chunks keep the zeros of the initial
// clear); rows past the end of the tensor re-read its last row.
//
// Addressing: the tensor's running tile pointer lives in scalar registers and each lane adds a
// 32-bit offset that does not change from tile to tile, so a copy costs no vector arithmetic.
// Tiles must be copied in sequence (rows r0, r0 + ROWS, ...).  The NWAVES waves of the workgroup
// issue equal shares, and every instruction has lanes switched on (each tile row starts with a
// valid chunk of every tensor), so a wave always issues exactly NINST of them per tile: the
// kernels' vmcnt waits count on that.
template <int ROWS, int ROWCH, int NWAVES, bool HASB>
struct TileDma {
    static constexpr int NI = ROWS * ROWCH / 64 / NWAVES; // groups of 64 chunk positions per wave
    static constexpr int NINST = NI * (HASB ? 2 : 1);     // copy instructions per wave and tile
    static_assert(NI * 64 * NWAVES == ROWS * ROWCH, "tile must split evenly over the waves");
    uint32_t off[NI];             // this lane's chunk: bytes from its tensor's tile pointer
    uint64_t lanes_a[NI], lanes_b[NI];
    const uint8_t *pa, *pb;       // first row of the next tile in A and B (wave-uniform)
    int wave, lane;

    // r0: first row of the first tile that issue() will copy.  Row strides below 2^24 elements.
    // twice_b: chunk 1 of the B part of a row is a second copy of chunk 0 (kernels that fold the
    // softmax scale pair it with the low-order half of the other operand, see fold_scale_chunk).
    __device__ __forceinline__ void init(const uint16_t *a, int64_t lda, int ncols_a, int split, const uint16_t *b,
                                         int64_t ldb, int ncols_b, int wave_, int lane_, int r0, bool twice_b = false) {
        wave = wave_;
        lane = lane_;
        pa = reinterpret_cast<const uint8_t *>(a) + (int64_t)r0 * lda * 2;
        pb = HASB ? reinterpret_cast<const uint8_t *>(b) + (int64_t)r0 * ldb * 2 : nullptr;
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int p = (wave * NI + j) * 64 + lane;
            const int r = p / ROWCH, pos = p % ROWCH;
            const int chunk = pos ^ swz_of<ROWCH>(r);
            const bool is_b = chunk >= split;
            const int cc = is_b ? ((twice_b && chunk - split == 1) ? 0 : chunk - split) : chunk;
            lanes_a[j] = __builtin_amdgcn_ballot_w64(!is_b && cc * 8 < ncols_a);
            lanes_b[j] = HASB ? __builtin_amdgcn_ballot_w64(is_b && cc * 8 < ncols_b) : 0;
            off[j] = (uint32_t)r * (uint32_t)((is_b ? ldb : lda) * 2) + cc * 16;
        }
    }

    // Copies the next tile, rows [r0, r0 + ROWS) clamped to nrows - 1, and moves on to the one
    // after it.  lda / ldb as given to init(); all lanes of the wave must be active.
    __device__ __forceinline__ void issue(uint32_t lds_tile, int r0, int nrows, int64_t lda, int64_t ldb, int split) {
        issue_step(lds_tile, r0, nrows, lda, ldb, split, lda * (2 * ROWS), ldb * (2 * ROWS));
    }

    // The same with the byte distance to the next tile given by the caller (a sequence of tiles
    // that runs along the rows of the tensor instead of down its columns).
    __device__ __forceinline__ void issue_step(uint32_t lds_tile, int r0, int nrows, int64_t lda, int64_t ldb, int split,
                                               int64_t step_a, int64_t step_b) {
        if (r0 + ROWS <= nrows) {
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                lds_dma16_lanes(off[j], pa, lds_tile + (wave * NI + j) * 1024, lanes_a[j]);
                if constexpr (HASB) lds_dma16_lanes(off[j], pb, lds_tile + (wave * NI + j) * 1024, lanes_b[j]);
            }
        } else { // the ragged last tile: rows past the end step back to the last row
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                const int p = (wave * NI + j) * 64 + lane;
                const int r = p / ROWCH, pos = p % ROWCH;
                const bool is_b = (pos ^ swz_of<ROWCH>(r)) >= split;
                const int over = max(r0 + r - (nrows - 1), 0);
                const uint32_t o = off[j] - (uint32_t)over * (uint32_t)((is_b ? ldb : lda) * 2);
                lds_dma16_lanes(o, pa, lds_tile + (wave * NI + j) * 1024, lanes_a[j]);
                if constexpr (HASB) lds_dma16_lanes(o, pb, lds_tile + (wave * NI + j) * 1024, lanes_b[j]);
            }
        }
        pa += step_a;
        if constexpr (HASB) pb += step_b;
    }
};

// Additive-mask values for the 16 scores that one lane holds of a 32 x 32 block, in C-layout
// register order, as fp32.  They are used as the initial value of an accumulator (or as the
// addend of the FMA that applies the softmax scale), so the mask costs no add per score.
//
// Lane = query (forward, dq kernel): register v <-> key k0 + 8 (v / 4) + 4 g + v % 4 of the
// lane's own mask row `row` (byte pointer; the same row for every lane of a vector mask): four
// runs of four consecutive keys, one aligned load each when the mask allows it.  Keys past Lk
// read as 0 (their scores are set to -inf afterwards).
template <class T>
__device__ __forceinline__ void mask_block_keys(const MaskDesc &m, const uint8_t *row, int k0, int g, int Lk,
                                                f32x16_t &out) {
    if (m.vec_ok && k0 + 32 <= Lk) {
        if (m.is_f32) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const f32x4_t x = *reinterpret_cast<const f32x4_t *>(row + (int64_t)(k0 + 8 * j + 4 * g) * 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) out[4 * j + e] = x[e];
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const u32x2_t x = *reinterpret_cast<const u32x2_t *>(row + (int64_t)(k0 + 8 * j + 4 * g) * 2);
                out[4 * j + 0] = T::to_float((uint16_t)(x[0] & 0xffffu));
                out[4 * j + 1] = T::to_float((uint16_t)(x[0] >> 16));
                out[4 * j + 2] = T::to_float((uint16_t)(x[1] & 0xffffu));
                out[4 * j + 3] = T::to_float((uint16_t)(x[1] >> 16));
            }
        }
    } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int key = k0 + 8 * (v >> 2) + 4 * g + (v & 3);
            const int kc = key < Lk ? key : Lk - 1;
            const float x = m.is_f32 ? reinterpret_cast<const float *>(row)[kc]
                                     : T::to_float(reinterpret_cast<const uint16_t *>(row)[kc]);
            out[v] = key < Lk ? x : 0.f;
        }
    }
}

// Lane = key (dk/dv kernel): register v <-> query q0 + 8 (v / 4) + 4 g + v % 4, all of key `key`:
// sixteen element loads, consecutive lanes reading consecutive keys of a row.  `base` is the
// byte pointer of the (batch, head) mask.  Out-of-range pairs read as 0.
template <class T>
__device__ __forceinline__ void mask_block_queries(const MaskDesc &m, const uint8_t *base, int q0, int g, int key, int Lq,
                                                   int Lk, f32x16_t &out) {
    const int kc = key < Lk ? key : Lk - 1;
    if (m.type == 1) { // vector mask: one value per key, i.e. per lane
        const float x = m.is_f32 ? reinterpret_cast<const float *>(base)[kc]
                                 : T::to_float(reinterpret_cast<const uint16_t *>(base)[kc]);
#pragma unroll
        for (int v = 0; v < 16; ++v) out[v] = key < Lk ? x : 0.f;
        return;
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int q = q0 + 8 * (v >> 2) + 4 * g + (v & 3);
        const int qc = q < Lq ? q : Lq - 1;
        const int64_t off = (m.type == 2 ? (int64_t)qc * m.sm : 0) + kc;
        const float x = m.is_f32 ? reinterpret_cast<const float *>(base)[off]
                                 : T::to_float(reinterpret_cast<const uint16_t *>(base)[off]);
        out[v] = (q < Lq && key < Lk) ? x : 0.f;
    }
}

// Grid id -> logical work id such that the workgroups that land on one XCD (hardware hands
// consecutive ids to the 8 XCDs round-robin) cover a contiguous range of logical ids and so
// share K/V of the same (batch, head) in that XCD's L2.
__device__ __forceinline__ int xcd_remap(int wg, int total) {
    int work, none;
    work_order(wg, 1, total, false, work, none); // (fb_order.h: the shares of any total, walked in order)
    return work;
}

// max(x of this lane, x of lane ^ 32): v_permlane32_swap exchanges the upper half of its first
// operand with the lower half of its second, so both copies end up holding one half's value in
// every lane.  A VALU exchange: no trip through the LDS crossbar.
__device__ __forceinline__ float half_wave_max(float x) {
    float lo = x, hi = x;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
    return fmaxf(lo, hi);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Epilogue store of one 32 x 32 accumulator block whose lanes are rows: lane (c, g) holds, for
// bq = 0..3, the channels ch0 + 8 bq + 4 g + {0..3} of row c in acc[4 bq .. 4 bq + 3] (what the
// 32x32 MFMA leaves with the row operand as B).  `row` points at channel ch0 of this lane's row,
// `ncols` counts the channels from ch0 that exist, `mul` scales the values.  With 16-byte aligned
// rows (`vec`, ncols a multiple of 8) the two lanes of a row first exchange halves
// (v_permlane32_swap: the upper half of one register against the lower half of another), so that
// each stores 16 contiguous bytes and the pair a 32-byte piece of the row: half the store
// instructions and write requests of 8-byte stores.  Must be called by all lanes (the exchange is
// outside the row test).
template <class T, bool VEC>
__device__ __forceinline__ void store_acc_rows(uint16_t *row, bool row_ok, bool vec, const f32x16_t &acc, float mul,
                                               int ncols, int g) {
    if (VEC && vec) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            uint32_t e0 = T::pack2(acc[8 * j] * mul, acc[8 * j + 1] * mul), e1 = T::pack2(acc[8 * j + 2] * mul, acc[8 * j + 3] * mul);
            uint32_t o0 = T::pack2(acc[8 * j + 4] * mul, acc[8 * j + 5] * mul), o1 = T::pack2(acc[8 * j + 6] * mul, acc[8 * j + 7] * mul);
            // lower half-wave: (e, o) = channels 16 j + {0..3, 4..7}; upper: channels 16 j + {8..11, 12..15}
            asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\tv_permlane32_swap_b32 %2, %3\n\ts_nop 1"
                         : "+v"(e0), "+v"(o0), "+v"(e1), "+v"(o1));
            const int col = 16 * j + 8 * g;
            if (row_ok && col + 8 <= ncols) *reinterpret_cast<u32x4_t *>(row + col) = u32x4_t{e0, e1, o0, o1};
        }
    } else if (row_ok) {
#pragma unroll
        for (int bq = 0; bq < 4; ++bq)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int col = 8 * bq + 4 * g + e;
                if (col < ncols) row[col] = T::from_float(acc[4 * bq + e] * mul);
            }
    }
}

// Turn-taking between the workgroups that share a CU.  The instruction arbiter serves the oldest
// wave of a SIMD first, so of two resident workgroups the older one runs at the speed it would
// have alone and the younger one only fills its stalls: their progress differs by a third, and
// whenever the older one ends the other is left alone with a SIMD it cannot fill.  Raising the
// wave priority of a different workgroup at every step evens the progress out.  Measured at
// B2 H4 d32 r8: forward 5 % faster at L = 8192 and 16384, 4 % at 32768; dq kernel 2 % at 16384;
// the streamlined dq and dk/dv kernels (two workgroups per CU, a turn per 64-row tile) 0.6 % and 1 %;
// the general dk/dv kernel (three workgroups per CU, one 32-query step per turn) gained nothing from
// any rotation tried and does not take turns.
//
// cu_slot(): which of the CU's equally sized LDS allocations this workgroup holds (0, 1, ...),
// read from the LDS_ALLOC hardware register (id 6: base in bits 11:0, size in bits 23:12, same
// units).  Workgroups of one launch get disjoint allocations at multiples of their size, and a new
// workgroup inherits the place of the one that ended.  Only a scheduling hint depends on it.
__device__ __forceinline__ int cu_slot() {
    const uint32_t r = __builtin_amdgcn_s_getreg((31 << 11) | 6);
    const uint32_t base = r & 0xfffu, size = (r >> 12) & 0xfffu;
    return size ? (int)(base / size) : 0;
}

// Called once per step: the workgroup whose turn it is runs at wave priority 1, the others at 0.
// `turn` starts as the workgroup's slot and counts round the `nslots` workgroups that share a CU
// in this launch (wave-uniform values).
__device__ __forceinline__ void take_turn(int &turn, int nslots) {
    if (nslots > 1) {
        if (turn == 0) __builtin_amdgcn_s_setprio(1);
        else __builtin_amdgcn_s_setprio(0);
        turn = turn + 1 >= nslots ? 0 : turn + 1;
    }
}

} // namespace fb
