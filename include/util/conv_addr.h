// Integer arithmetic of the convolution kernels' prologues (csrc/gemm_pipe.hpp, csrc/gemm_wide.hpp),
// kept in a header that also compiles on the host so that it can be checked exhaustively there
// (tests/conv_addr_check.cpp).
#pragma once

#if defined(__HIPCC__)
#define GP_CA_HD __host__ __device__ inline
#else
#define GP_CA_HD inline
#endif

namespace gp {

// a / b for 0 <= a < 2^22, 0 < b <= a range: a float multiply by a reciprocal taken once
// (rcp_b = 1.0f / (float)b), and one correction step either way.  The integer division of MI355X
// is some sixty instructions per lane, and every lane of a convolution tile needs two of them to
// turn an output row index into (image, row, column).
GP_CA_HD int small_div(int a, int b, float rcp_b) {
    int q = (int)((float)a * rcp_b);
    const int r = a - q * b;
    q += (r >= b) - (r < 0);
    return q;
}
constexpr int kSmallDivLimit = 1 << 22;

// Which taps of an R x S window whose origin is (h0, w0) (it may lie outside) fall inside an H x W
// image: bit r * S + s is set for tap (r, s).  Needs R * S <= 32 and S < 32.
GP_CA_HD unsigned window_tap_mask(int h0, int w0, int H, int W, int R, int S) {
    const int s_lo = w0 < 0 ? -w0 : 0, s_hi = W - w0 < S ? W - w0 : S;
    if (s_hi <= s_lo) return 0u;
    const unsigned smask = ((1u << s_hi) - 1u) & ~((1u << s_lo) - 1u);
    unsigned mask = 0;
    for (int r = 0; r < R; ++r)
        if ((unsigned)(h0 + r) < (unsigned)H) mask |= smask << (r * S);
    return mask;
}

}  // namespace gp
