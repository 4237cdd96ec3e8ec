// Error reporting shared by the two halves of the C ABI (fb_checks.cpp, fb_api.hip).
#pragma once

namespace fb {
// Stores the formatted text as the calling thread's last error and returns `code`.
int api_fail(int code, const char *fmt, ...);
void api_clear_error();
} // namespace fb
