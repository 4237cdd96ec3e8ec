// LDS tiles of the streamlined kernels (head dim 32, rank 8 or no factors): dense regions filled by
// whole-wave direct copies, read with per-lane base addresses plus immediates.
//
// A region holds ROWS rows of CPR 16-byte chunks (CPR = 4: a 32-channel row of q, k, v or dO;
// CPR = 2: a bias-factor row and its second copy; CPR = 1: one chunk of per-row statistics) as a
// dense array of 128-byte lines of eight chunks: row r sits in line r / (8 / CPR) at slot
// (r % (8 / CPR)) * CPR + chunk, and a slot's position inside its line is slot ^ ((line >> 1) & 3).
// With that swizzle the row-wise 16-byte reads (lane = row, one chunk column) and the transposing
// 8-byte reads (lds_read_tr4) of 4-chunk regions touch every LDS bank once per pass.
//
// A copy instruction (global_load_lds_dwordx4) fills 64 consecutive positions = 8 lines of one
// region, every lane fetching the chunk that belongs at its position: all lanes on, one tensor per
// instruction, nothing to set up but the scalar base and m0.
#pragma once
#include <type_traits>

#include "fb_device.h"

namespace fb {

// 16 bytes per lane from base + off (base wave-uniform, off a 32-bit byte offset per lane) to LDS
// byte address lds + 16 * lane; every lane of the wave takes part.
__device__ __forceinline__ void lds_dma16_all(uint32_t off, const void *base, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"(lds) : "memory");
}

// Which (row, chunk) of a region with CPR chunks per row belongs at position `lane` of a copy
// instruction's 8 lines (the instruction starts at a multiple of 8 lines, which leaves the swizzle
// term a function of the lane alone).  row is relative to the instruction's first row.
template <int CPR>
__device__ __forceinline__ void lean_copy_place(int lane, int &row, int &chunk) {
    const int line = lane >> 3, slot = (lane & 7) ^ ((lane >> 4) & 3);
    row = line * (8 / CPR) + slot / CPR;
    chunk = slot % CPR;
}

// Byte offset inside a region of chunk `chunk` of row `row`.
template <int CPR>
__device__ __forceinline__ uint32_t lean_chunk_off(int row, int chunk) {
    const int line = row / (8 / CPR), slot = (row % (8 / CPR)) * CPR + chunk;
    return (uint32_t)(line * 128 + ((slot ^ ((line >> 1) & 3)) * 16));
}

// Row-wise A / B operand: lane (c, g) reads chunk 2 t + g of row c.  Rows c + 32 k of the same
// region are at + k * 32 * CPR * 16 bytes (the swizzle term repeats every 16 lines).
template <int CPR>
__device__ __forceinline__ uint32_t lean_row_addr(int c, int chunk) {
    return lean_chunk_off<CPR>(c, chunk);
}

// Column-wise (transposing) A operand of a 4-chunk region for a B operand that comes straight from
// a C-layout register block: the address this lane hands to ds_read_b64_tr_b16 for the low (hi = 0)
// and high (hi = 1) half of a 16-row contraction step starting at row 0, columns [0, 32).  Step
// starts at rows 16 k are at + k * 16 * 64 bytes.  The lane receives tile[4 g + 8 hi + 0..3 ...]
// of its own column c: rows {0..3, 8..11} + 4 g of the step, the order of the C layout.
__device__ __forceinline__ uint32_t lean_tr_addr4(int c, int g, int hi) {
    const int r = 4 * g + ((c & 15) >> 2) + 8 * hi, chunk = 2 * (c >> 4) + ((c & 3) >> 1);
    return lean_chunk_off<4>(r, chunk) + 8 * (c & 1);
}
// The same for a 2-chunk region (16 columns) and the step that starts at row 16 t (t = 0, 1: the
// swizzle term differs between them); lanes 16..31 repeat columns 0..15 (the rows of the product
// that they feed are never used).  Steps 32 k rows further on are at + k * 32 * 32 bytes.
__device__ __forceinline__ uint32_t lean_tr_addr2(int c, int g, int hi, int t) {
    const int r = 16 * t + 4 * g + ((c & 15) >> 2) + 8 * hi, chunk = (c & 3) >> 1;
    return lean_chunk_off<2>(r, chunk) + 8 * (c & 1);
}

// Reads at absolute LDS byte addresses (a per-lane register plus an immediate).
__device__ __forceinline__ u32x4_t lds_load16(uint32_t addr) {
    return *(const __attribute__((address_space(3))) u32x4_t *)addr;
}
__device__ __forceinline__ u32x4_t lds_load_tr(uint32_t lo, uint32_t hi) {
    typedef short v4s_t __attribute__((ext_vector_type(4)));
    const u32x2_t a = __builtin_bit_cast(u32x2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s_t __attribute__((address_space(3))) *)lo));
    const u32x2_t b = __builtin_bit_cast(u32x2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((v4s_t __attribute__((address_space(3))) *)hi));
    return u32x4_t{a[0], a[1], b[0], b[1]};
}

__device__ __forceinline__ u32x4_t lean_read_tr(const uint8_t *lo, const uint8_t *hi) {
    const u32x2_t a = lds_read_tr4(reinterpret_cast<const uint16_t *>(lo));
    const u32x2_t b = lds_read_tr4(reinterpret_cast<const uint16_t *>(hi));
    return u32x4_t{a[0], a[1], b[0], b[1]};
}

// One wave's copies of a 4-chunk region (32-channel rows): the workgroup's 4 waves copy
// ROWS = 64 or 128 rows per tile, this wave rows [ROWS / 4 * wave, ...), 16 rows per instruction.
template <int ROWS>
struct LeanCopy4 {
    static constexpr int NI = ROWS / 64; // instructions per wave and tile
    uint32_t off[NI];
    int pitch; // bytes between rows of the tensor
    __device__ __forceinline__ void init(int wave, int lane, int64_t ld_elems) {
        pitch = (int)ld_elems * 2;
        int row, chunk;
        lean_copy_place<4>(lane, row, chunk);
#pragma unroll
        for (int j = 0; j < NI; ++j) off[j] = (uint32_t)(((ROWS / 4) * wave + 16 * j + row) * pitch + chunk * 16);
    }
    // tile = first row of the tile in the tensor (wave-uniform), region = LDS byte address of the
    // region; rows_left = rows of the tensor from the tile's first row on (>= 1): rows past the end
    // re-read the last one
    __device__ __forceinline__ void issue(const uint8_t *tile, uint32_t region, int wave, int lane, int rows_left) const {
        if (rows_left >= ROWS) {
#pragma unroll
            for (int j = 0; j < NI; ++j) lds_dma16_all(off[j], tile, region + (NI * wave + j) * 1024);
        } else {
            int row, chunk;
            lean_copy_place<4>(lane, row, chunk);
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                const int over = max((ROWS / 4) * wave + 16 * j + row - (rows_left - 1), 0);
                lds_dma16_all(off[j] - (uint32_t)(over * pitch), tile, region + (NI * wave + j) * 1024);
            }
        }
    }
};

// The same for a 2-chunk region whose two chunks are both the tensor's one chunk (a rank-8 factor
// row and its second copy): 32 rows per instruction, ROWS / 128 instructions per wave (one for
// ROWS = 128; for ROWS = 64 only waves 0 and 1 copy).
template <int ROWS>
struct LeanCopy2 {
    uint32_t off;
    int pitch;
    __device__ __forceinline__ void init(int wave, int lane, int64_t ld_elems) {
        pitch = (int)ld_elems * 2;
        int row, chunk;
        lean_copy_place<2>(lane, row, chunk);
        off = (uint32_t)((32 * wave + row) * pitch);
    }
    __device__ __forceinline__ void issue(const uint8_t *tile, uint32_t region, int wave, int lane, int rows_left) const {
        if (ROWS < 128 && wave >= ROWS / 32) return; // (wave-uniform)
        if (rows_left >= ROWS) {
            lds_dma16_all(off, tile, region + wave * 1024);
        } else {
            int row, chunk;
            lean_copy_place<2>(lane, row, chunk);
            const int over = max(32 * wave + row - (rows_left - 1), 0);
            lds_dma16_all(off - (uint32_t)(over * pitch), tile, region + wave * 1024);
        }
    }
    // copy instructions this wave issues per tile
    __device__ __forceinline__ static int count(int wave) { return (ROWS < 128 && wave >= ROWS / 32) ? 0 : 1; }
};

// The kernel arguments as a function called by the kernel may read them: a function's pointer
// argument arrives in vector registers, which would make every value loaded through it look
// divergent (vector loads, no scalar operands for the copy instructions); made wave-uniform again
// and typed as constant memory it is read with scalar loads like the kernel's own copy.
template <class A>
__device__ __forceinline__ A uniform_kernargs(const void *p) {
    static_assert(sizeof(A) % 4 == 0, "");
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint64_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint64_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
    const __attribute__((address_space(4))) uint32_t *w = (const __attribute__((address_space(4))) uint32_t *)((hi << 32) | lo);
    union {
        A a;
        uint32_t u[sizeof(A) / 4];
    } x;
#pragma unroll
    for (unsigned i = 0; i < sizeof(A) / 4; ++i) x.u[i] = w[i];
    return x.a;
}

// acc += A B with the accumulator tied to the result register block (the compiler's own choice
// often is a second block and a copy).  The compiler does not see an MFMA here, so the caller owes
// the two wait states between a VALU write of a or b and this instruction (the block step below
// converts P and dS at least one slot before their use) and the wait for the last result before
// anything but another such MFMA reads acc.
template <class T>
__device__ __forceinline__ void mfma_into(f32x16_t &acc, const u32x4_t &a, const u32x4_t &b) {
    if constexpr (std::is_same<T, BF16>::value)
        asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
    else
        asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
}

} // namespace fb
