/*
 * flashbias.h -- C ABI of the MI355X (gfx950) FlashBias attention library.
 *
 * The library is the device side of the reference's operator
 *     flash_bias_func(q, k, v, q_bias, k_bias, mask, causal, softmax_scale)
 * (flash_bias/flash_bias_triton.py:1345-1405).  Each entry point below names the reference
 * function it replaces.  Conventions shared by all of them:
 *
 *   - Nothing here allocates or frees device memory: every buffer, including scratch
 *     (lse, delta), is owned by the caller, as in the reference where
 *     torch allocates o/lse/tmp/delta/dq_accum (flash_bias_triton.py:1145-1148, :1212-1219).
 *   - Launches are asynchronous on the given hipStream_t (passed as void*); no autotuning side
 *     effects.  The only process-wide state are write-once caches (compute units per device,
 *     per-kernel occupancy and LDS limit; atomics, safe under concurrent first calls) and the
 *     scratch array of fb_bwd_static.
 *   - Return value: FB_OK (0) or a negative fb_status; fb_last_error() gives the text of the
 *     last failure on the calling thread.  No C++ exception crosses the boundary.
 *   - Tensors use the reference layout (batch, seq, heads, channels) with the channel
 *     dimension contiguous (stride 1: the ABI has no channel stride, a caller with another one
 *     must make the tensor contiguous first, as the reference does, :1357-1360); batch / head /
 *     seq are addressed through element strides, the way the Triton launchers pass them
 *     (flash_bias_triton.py:1163-1177).  Sequence strides of 2^24 elements or more are correct
 *     but take slower instantiations (the fast loaders keep a tile row's offset in 32 bits).
 */
#ifndef FLASHBIAS_H
#define FLASHBIAS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FB_VERSION 3
#define FB_MAX_HEADDIM 128 /* flash_bias_triton.py:1106 */
#define FB_MAX_RANK 128
/* Size of the library-owned scratch buffer used by fb_bwd_static (one copy per GPU, held until the
 * process ends): enough for B * H * Lq <= 1398101 query rows (24 bytes each). */
#define FB_STATIC_SCRATCH_BYTES (32u << 20)

typedef enum fb_status {
    FB_OK = 0,
    FB_ERR_NULL = -1,       /* required pointer missing */
    FB_ERR_SHAPE = -2,      /* non-positive size, d > 128, r > 128, B * H * ceil(L / 32) >= 2^31 */
    FB_ERR_DTYPE = -3,      /* only fp16 / bf16 inputs (flash_bias_triton.py:1108) */
    FB_ERR_STRIDE = -4,     /* stride would alias gradient rows / negative stride */
    FB_ERR_MASK = -5,       /* bad mask type / dtype */
    FB_ERR_RESERVED = -6,
    FB_ERR_ABI = -7,        /* fb_params.size does not match this library */
    FB_ERR_LAUNCH = -8,     /* HIP reported a launch error */
    FB_ERR_SCALE = -9       /* softmax scale not finite or zero (negative scales are accepted) */
} fb_status;

typedef enum fb_dtype { FB_F16 = 0, FB_BF16 = 1, FB_F32 = 2 /* mask only */ } fb_dtype;

/* flash_bias_triton.py:1112-1123 */
typedef enum fb_mask_type { FB_MASK_NONE = 0, FB_MASK_VECTOR = 1, FB_MASK_MATRIX = 2 } fb_mask_type;

/* A (batch, seq, heads, channels) tensor with contiguous channels.  Strides are in elements.
 * For the mask, which is (batch, heads, Lq|1, Lk), stride_s is the stride of the query row
 * (0 for the vector type) and stride_b / stride_h may be 0 (broadcast). */
typedef struct fb_tensor {
    void *ptr;
    int64_t stride_b, stride_h, stride_s;
} fb_tensor;

typedef struct fb_params {
    uint32_t size; /* sizeof(fb_params) as seen by the caller */
    int32_t dtype; /* fb_dtype of q, k, v, factors, o and all gradients */
    int32_t B, H, Lq, Lk;
    int32_t d;     /* head dim, 1..128 */
    int32_t r;     /* bias rank, 0 = no factors (plain attention, flash_bias_triton.py:1359) */
    int32_t causal;     /* top-left aligned: key j visible from query i iff j <= i (:262) */
    int32_t mask_type;  /* fb_mask_type */
    int32_t mask_dtype; /* dtype or FB_F32 (:1115) */
    float scale;        /* softmax scale, applied to q k^T only, never to the bias (:248) */

    fb_tensor q, k, v;        /* in */
    fb_tensor q_bias, k_bias; /* in; stride_b / stride_h = 0 broadcasts (:1135-1136) */
    fb_tensor mask;           /* in, additive, no gradient (:1371) */
    fb_tensor o;              /* fwd: out; bwd: in */
    float *lse;               /* (B, H, Lq) fp32, natural log; fwd: out; bwd: in (:323) */

    fb_tensor dout;             /* bwd in: upstream gradient of o */
    fb_tensor dq, dk, dv;       /* bwd out */
    fb_tensor dq_bias, dk_bias; /* bwd out, full (B, L, H, r) shape: the caller reduces over
                                   broadcast dims (but see bias_grad_group).  Both pointers NULL: the
                                   factor gradients are not wanted (constant factors) and are neither
                                   stored nor, in the streamlined kernels, computed; the reference
                                   always computes them (flash_bias_triton.py:718-719, :725-817) */
    float *delta;               /* backward scratch of fb_bwd_workspace_bytes() bytes, 16-byte aligned, written by the
                                   backward: -delta and lse * log2(e) per query row, as fp32 and as 16-bit parts */
    int32_t bias_grad_group;    /* 0 or 1: as above.  g > 1, for factors that the batch shares (stride_b = 0, the
                                   window attention of swin_transformer_v2.py:178-203): dq_bias and dk_bias have
                                   ceil(B / g) batch rows and row i receives the sum of the gradients of batch
                                   entries [i g, (i + 1) g), accumulated in fp32 inside the kernels and rounded
                                   once; the caller reduces the remaining rows.  (The reference accumulates the factor
                                   gradients with atomic adds into fp32 buffers laid out like the factors
                                   themselves, flash_bias_triton.py:1219-1231, :1342.) */
} fb_params;

/* Library / ABI version. */
int fb_version(void);

/* Optional set-up for the current device: looks up the address of the static scratch array that
 * fb_bwd_static uses (one hipGetSymbolAddress per device, cached), so that no later call has to.
 * fb_bwd_static does the same on its first call on a device; a caller that wants that first call
 * inside a HIP graph capture calls fb_init() (or fb_bwd_static once, eagerly) on the device
 * beforehand, because a symbol lookup is not a stream operation and must not happen while a
 * stream is capturing.  Launches nothing, allocates nothing.  No counterpart in the reference. */
int fb_init(void);

/* Text of the last error on this thread ("" if none). */
const char *fb_last_error(void);

/* Argument checks of _flash_attn_forward / _flash_attn_backward
 * (flash_bias_triton.py:1102-1129, :1201-1225) without touching the GPU.
 * pass: 0 = forward, 1 = backward. */
int fb_check(const fb_params *p, int pass);

/* The bias_grad_group this library recommends for a backward call: 1 unless both factors are shared by
 * the batch (stride_b = 0) and the call is a large batch of short sequences (the window attention of
 * swin_transformer_v2.py:178-203), where writing the full-shape factor gradients and summing them
 * afterwards costs more than the attention itself saves; then the largest of 8, 4, 2 (32, 16, ... for whole
 * sequences of at most 256 positions at head dim 32, which one workgroup per batch entry and head serves) that still
 * leaves every compute unit several workgroups.  Reads the sizes, the causal flag, the mask type and the factors' strides only.
 * No counterpart in the reference. */
int fb_suggest_bias_grad_group(const fb_params *p);

/* Bytes of the backward's scratch buffer fb_params.delta for these sizes (24 per query row: two
 * floats and one 16-byte chunk of 16-bit parts, the second array starting on a 16-byte boundary;
 * the reference allocates delta, dq_accum and dq_bias_accum itself, flash_bias_triton.py:1212-1219).
 * Only B, H and Lq are read; returns 0 for a null pointer or non-positive sizes. */
size_t fb_bwd_workspace_bytes(const fb_params *p);

/* Replaces _flash_attn_forward + _fwd_kernel (flash_bias_triton.py:1100-1194, :62-355):
 * o = softmax(scale q k^T + q_bias k_bias^T + mask) v and lse. */
int fb_fwd(const fb_params *p, void *stream);

/* Replaces _flash_attn_backward (flash_bias_triton.py:1197-1342).  Two launches on the stream: the
 * query-stationary kernel (dq, dq_bias), which also forms delta = rowsum(o * dout) for its own
 * queries and leaves -delta and lse * log2(e) in the scratch buffer, then the key-stationary kernel
 * (dk, dv, dk_bias) that reads them.  (On grids that would give each of these kernels at most one
 * workgroup per compute unit: the preprocess phase, then a single launch that holds the workgroups of
 * both kernels side by side.)  The results of these are bit-identical to the three phases below
 * called one by one.  Whole sequences of at most 256 positions (head dim 32, rank a multiple of 8 up to
 * 32, aligned tensors, no additive or causal mask, at least one (batch, head) pair per compute unit: the
 * window attention of swin_transformer_v2.py:178-203) take a single launch instead in which one
 * workgroup forms delta and all five gradients of a (batch, head) pair, dq summed inside the workgroup;
 * it leaves the scratch buffer untouched and its results equal the phases' up to the rounding of other
 * summation orders.  Unlike the reference there is no fp32 dq_accum buffer, no atomics and no final
 * cast on any of these paths (:1212-1219, :1340-1342): dq and dq_bias are accumulated in registers
 * (or, for windows, in a fixed order through LDS) and written once, so every gradient is
 * bit-reproducible. */
int fb_bwd(const fb_params *p, void *stream);

/* fb_bwd for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose
 * backward allocates its scratch through torch (flash_bias_triton.py:1212-1219).  Same inputs,
 * outputs and results as fb_bwd, except that fb_params.delta is ignored: the scratch lives in a
 * static device array of FB_STATIC_SCRATCH_BYTES inside the library.  Neither this call nor
 * anything it calls allocates or frees memory.  Returns FB_ERR_SHAPE when
 * fb_bwd_workspace_bytes(p) exceeds FB_STATIC_SCRATCH_BYTES.  All calls on one GPU share that
 * GPU's array: calls that overlap in time on one GPU (two streams, two threads) race; calls
 * ordered on one stream are safe.  Nothing in the array has to be cleared between calls.  The
 * first call on a device looks the array's address up (see fb_init): make it, or fb_init(), outside
 * graph capture. */
int fb_bwd_static(const fb_params *p, void *stream);

/* The last step of the backward for factors that every batch entry shares: the kernels write such
 * a factor's gradient in full (B, L, H, r) shape, and this sums it over the batch:
 * out[j] = sum_b full[b * batch_stride + j] for j < n = L * H * r, accumulated in fp32 in a fixed
 * order (bit-reproducible), written in the input dtype or (out_dtype = FB_F32) in fp32.  The
 * reference has no such step: it hands the kernels the un-expanded tensors with expanded strides
 * (flash_bias_triton.py:1227-1231), so every batch entry overwrites the same gradient rows.
 * n and batch_stride must be multiples of 8 elements, full 16-byte aligned (FB_ERR_STRIDE else). */
int fb_sum_over_batch(const void *full, void *out, int dtype, int out_dtype, int64_t B, int64_t n,
                      int64_t batch_stride, void *stream);

/* Factors of a rank that is no multiple of 8 (ALiBi: 2, a distance bias in three dimensions: 5) have rows the
 * kernels' 16-byte loads cannot take; their owner, or the operator on every call, pads them with zero columns,
 * which change nothing in q_bias k_bias^T.  out[row][c] = c < min(r_in, r_out) ? in[row][c] : 0 for `rows`
 * contiguous rows of 16-bit elements (either dtype): r_out > r_in pads, r_out < r_in takes the original columns of
 * a gradient back out.  One launch.  The reference pads inside its kernels instead (BLOCK_RANKDIM, the next power
 * of two of at least 16, with masked loads: flash_bias_triton.py:1137, :195-200). */
int fb_resize_rank(const void *in, void *out, int64_t rows, int r_in, int r_out, void *stream);

/* The backward in three phases, exported so that a harness can time them separately (call them in
 * this order: the two main kernels read what the preprocess wrote).
 *   fb_bwd_preprocess: delta = rowsum(o * dout)       (_bwd_preprocess_do_o_dot, :358-400); fills the
 *                      scratch with -delta (first B*H*Lq floats), lse * log2(e) (next B*H*Lq) and, from the
 *                      next 16-byte boundary on, both once more per query row as three 16-bit parts each
 *                      (what the streamlined dk/dv kernel feeds to its MFMAs; written only for the calls
 *                      that kernel takes: aligned, unmasked, head dim 32, rank 8 or 0)
 *   fb_bwd_dkv:        recompute P from lse; dk, dv, dk_bias, one workgroup per key tile
 *                      (_bwd_kernel / _bwd_kernel_one_col_block, :450-1097, minus dq)
 *   fb_bwd_dq:         recompute P from lse; dq, dq_bias, one workgroup per query tile
 *                      (the dq / dq_bias updates of :725-817) */
int fb_bwd_preprocess(const fb_params *p, void *stream);
int fb_bwd_dkv(const fb_params *p, void *stream);
int fb_bwd_dq(const fb_params *p, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FLASHBIAS_H */
