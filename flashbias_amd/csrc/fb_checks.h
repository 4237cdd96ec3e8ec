// Error reporting and the scratch-buffer layout shared by the two halves of the C ABI
// (fb_checks.cpp, fb_api.hip) and the kernels.
#pragma once
#include <cstddef>
#include <cstdint>

#ifdef __HIPCC__
#define FB_HOST_DEVICE __host__ __device__
#else
#define FB_HOST_DEVICE
#endif

namespace fb {
// Stores the formatted text as the calling thread's last error and returns `code`.
int api_fail(int code, const char *fmt, ...);
void api_clear_error();

// Layout of the backward's scratch buffer, in floats from its (16-byte aligned) start: rows =
// B * H * Lq values of -delta, rows values of lse * log2(e), and from stat_offset(rows) on one
// 16-byte chunk per query row (stat_chunk, fb_device.h) holding both as 16-bit parts.
FB_HOST_DEVICE inline int64_t stat_offset(int64_t rows) { return (2 * rows + 3) & ~(int64_t)3; }
inline size_t bwd_scratch_bytes(int64_t rows) { return (size_t)(stat_offset(rows) + 4 * rows) * sizeof(float); }
} // namespace fb
