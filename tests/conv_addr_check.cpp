// Host check of include/util/conv_addr.h: the reciprocal division against the integer division over
// its whole domain of use, and the window tap mask against a tap-by-tap loop.
#include <cstdio>
#include <cstdlib>
#include "util/conv_addr.h"

int main() {
    using namespace gp;
    long checked = 0;
    // every divisor up to 4096 (pixels per image and row lengths of real layers), dividends at and around the
    // multiples of the divisor, the range ends, and a stride through the rest
    for (int b = 1; b <= 4096; ++b) {
        const float rcp = 1.0f / (float)b;
        for (long a = 0; a < kSmallDivLimit; a += (a < 70000 ? 1 : 997)) {
            if (small_div((int)a, b, rcp) != (int)(a / b)) { std::printf("small_div(%ld, %d) = %d\n", a, b, small_div((int)a, b, rcp)); return 1; }
            ++checked;
        }
        for (long q = 0; q * b < kSmallDivLimit; q += 1 + q / 64) {
            for (long d = -1; d <= 1; ++d) {
                const long a = q * b + d;
                if (a < 0 || a >= kSmallDivLimit) continue;
                if (small_div((int)a, b, rcp) != (int)(a / b)) { std::printf("small_div(%ld, %d) = %d\n", a, b, small_div((int)a, b, rcp)); return 1; }
                ++checked;
            }
        }
    }
    // large divisors (images of up to 2^22 pixels)
    for (int b = 4097; b < kSmallDivLimit; b += 1 + b / 300) {
        const float rcp = 1.0f / (float)b;
        for (long a = 0; a < kSmallDivLimit; a += 1 + b / 7) {
            if (small_div((int)a, b, rcp) != (int)(a / b)) { std::printf("small_div(%ld, %d)\n", a, b); return 1; }
            ++checked;
        }
        const long edge[] = {b - 1L, b, b + 1L, kSmallDivLimit - 1L, (kSmallDivLimit - 1L) / b * b, (kSmallDivLimit - 1L) / b * b - 1};
        for (long a : edge)
            if (a >= 0 && a < kSmallDivLimit && small_div((int)a, b, rcp) != (int)(a / b)) { std::printf("small_div(%ld, %d)\n", a, b); return 1; }
    }
    long masks = 0;
    for (int R = 1; R <= 7; ++R)
        for (int S = 1; S <= 7 && R * S <= 32; ++S)
            for (int H = 1; H <= 9; ++H)
                for (int W = 1; W <= 9; ++W)
                    for (int h0 = -8; h0 <= 10; ++h0)
                        for (int w0 = -8; w0 <= 10; ++w0) {
                            unsigned ref = 0;
                            for (int r = 0; r < R; ++r)
                                for (int s = 0; s < S; ++s)
                                    if (h0 + r >= 0 && h0 + r < H && w0 + s >= 0 && w0 + s < W) ref |= 1u << (r * S + s);
                            if (window_tap_mask(h0, w0, H, W, R, S) != ref) { std::printf("mask h0 %d w0 %d H %d W %d R %d S %d\n", h0, w0, H, W, R, S); return 1; }
                            ++masks;
                        }
    std::printf("ok %ld divisions %ld masks\n", checked, masks);
    return 0;
}
