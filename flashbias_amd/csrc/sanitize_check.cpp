// Sanitizer driver for the argument checks and size queries of the C ABI (fb_checks.cpp), built
// under AddressSanitizer and UBSan by `make sanitize` and called with well-formed and with
// deliberately malformed parameter blocks, and for the launch order of the kernels (fb_order.h).  No GPU is
// involved.  Exit status 0 = clean.
#include <cstdio>
#include <cstring>
#include <vector>

#include "fb_order.h"
#include "flashbias.h"

// Every (unit, position) pair exactly once; under a causal mask every XCD's share longest first.
static bool launch_order_ok(int units, int ntiles, bool causal) {
    const int total = units * ntiles;
    std::vector<int> seen(total, 0);
    std::vector<int> last(8, 0); // the position of the previous workgroup of each XCD's sequence
    std::vector<int> lo(8, total), hi(8, -1); // the range of the unit-major numbering each XCD serves
    for (int wg = 0; wg < total; ++wg) {
        int unit = -1, pos = -1;
        fb::work_order(wg, ntiles, total, causal, unit, pos);
        if (unit < 0 || unit >= units || pos < 0 || pos >= ntiles) return false;
        if (seen[unit * ntiles + pos]++) return false;
        if (unit * ntiles + pos < lo[wg % 8]) lo[wg % 8] = unit * ntiles + pos;
        if (unit * ntiles + pos > hi[wg % 8]) hi[wg % 8] = unit * ntiles + pos;
        if (causal) {
            int &prev = last[wg % 8];
            if (pos < prev) return false;
            prev = pos;
        }
    }
    int count = 0; // the shares are contiguous: their extents add up to the total
    for (int x = 0; x < 8; ++x)
        if (hi[x] >= 0) count += hi[x] - lo[x] + 1;
    return count == total;
}

static fb_params good(int pass) {
    alignas(16) static char buf[64]; // (never dereferenced by the checks)
    fb_params p;
    std::memset(&p, 0, sizeof(p));
    p.size = sizeof(p);
    p.dtype = FB_BF16;
    p.B = 2; p.H = 4; p.Lq = 128; p.Lk = 96; p.d = 32; p.r = 8;
    p.scale = 0.25f;
    auto t = [&](int c) { return fb_tensor{buf, (int64_t)128 * 4 * c, c, 4 * c}; };
    p.q = t(32); p.k = t(32); p.v = t(32); p.o = t(32);
    p.q_bias = t(8); p.k_bias = t(8);
    p.lse = reinterpret_cast<float *>(buf);
    if (pass) {
        p.dout = t(32); p.dq = t(32); p.dk = t(32); p.dv = t(32);
        p.dq_bias = t(8); p.dk_bias = t(8);
        p.delta = reinterpret_cast<float *>(buf);
    }
    return p;
}

int main() {
    int bad = 0;
    auto expect = [&](int got, int want, const char *what) {
        if (got != want) {
            std::fprintf(stderr, "%s: got %d, want %d (%s)\n", what, got, want, fb_last_error());
            bad = 1;
        }
    };
    for (int pass = 0; pass < 2; ++pass) {
        fb_params p = good(pass);
        expect(fb_check(&p, pass), FB_OK, "well-formed block");
        p = good(pass); p.size = 8;                     expect(fb_check(&p, pass), FB_ERR_ABI, "size");
        p = good(pass); p.dtype = FB_F32;               expect(fb_check(&p, pass), FB_ERR_DTYPE, "dtype");
        p = good(pass); p.d = 129;                      expect(fb_check(&p, pass), FB_ERR_SHAPE, "d");
        p = good(pass); p.Lk = -5;                      expect(fb_check(&p, pass), FB_ERR_SHAPE, "Lk");
        p = good(pass); p.B = 1 << 20; p.H = 1 << 12;   expect(fb_check(&p, pass), FB_ERR_SHAPE, "grid");
        p = good(pass); p.scale = 0.f;                  expect(fb_check(&p, pass), FB_ERR_SCALE, "scale");
        p = good(pass); p.q.ptr = nullptr;              expect(fb_check(&p, pass), FB_ERR_NULL, "q");
        p = good(pass); p.v.stride_s = -1;              expect(fb_check(&p, pass), FB_ERR_STRIDE, "v stride");
        p = good(pass); p.mask_type = 7;                expect(fb_check(&p, pass), FB_ERR_MASK, "mask type");
        if (pass) {
            p = good(pass); p.delta = reinterpret_cast<float *>(reinterpret_cast<char *>(p.delta) + 4);
            expect(fb_check(&p, pass), FB_ERR_STRIDE, "scratch alignment");
        }
    }
    expect(fb_check(nullptr, 0), FB_ERR_NULL, "null block");
    fb_params p = good(1);
    if (fb_bwd_workspace_bytes(&p) != (size_t)2 * 4 * 128 * (2 * sizeof(float) + 16)) bad = 1; // per query row: two floats, one chunk
    p.B = 0;
    if (fb_bwd_workspace_bytes(&p) != 0 || fb_bwd_workspace_bytes(nullptr) != 0) bad = 1;
    for (int units : {1, 2, 3, 7, 8, 9, 16, 50, 64})
        for (int ntiles : {1, 2, 3, 5, 8, 16, 31, 32, 64, 100, 128})
            for (int causal = 0; causal < 2; ++causal)
                if (!launch_order_ok(units, ntiles, causal != 0)) {
                    std::fprintf(stderr, "launch order: %d units x %d tiles, causal %d\n", units, ntiles, causal);
                    bad = 1;
                }
    if (!bad) std::puts("sanitize_check: clean");
    return bad;
}
