"""The int8 quantiser divides a whole 32-row block by one f16 scale. The kernels do the divisor's share of an f32
division once (reciprocal estimate + one refinement) and per quotient only the remaining steps (fa_sage_quant.h). This
checks that sequence on the CPU, in C with fused multiply-adds, against the division itself: every positive finite f16
divisor, the reciprocal estimate exact and off by one ulp either way, and numerators both spread over many binades
and placed within a few ulps of (k + 1/2) * scale, the quantiser's rounding boundaries. Bit-equal quotients are
required, which is more than the quantiser needs."""
import os
import subprocess
import tempfile

SRC = r"""
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>
static float f16_value(uint16_t h) {
    const uint32_t e = (h >> 10) & 31, m = h & 1023;
    return e == 0 ? ldexpf((float)m, -24) : ldexpf((float)(m + 1024), (int)e - 25);
}
static float step(float x, int d) { uint32_t u; memcpy(&u, &x, 4); u += (uint32_t)d; float y; memcpy(&y, &u, 4); return y; }
int main(void) {
    unsigned long long bad = 0, n = 0;
    uint32_t seed = 12345;
    for (uint32_t h = 1; h < 0x7c00; ++h) {
        const float d = f16_value((uint16_t)h);
        for (int off = -1; off <= 1; ++off) {
            const float r0 = step(1.0f / d, off);           /* the hardware's estimate is within one ulp */
            const float r = fmaf(fmaf(-d, r0, 1.0f), r0, r0);
            for (int t = 0; t < 200; ++t) {
                seed = seed * 1664525u + 1013904223u; const uint32_t a = seed;
                seed = seed * 1664525u + 1013904223u;
                float x;
                if (t & 1) x = step(((float)((int)(a % 300) - 150) + 0.5f) * d, (int)(seed % 7) - 3);
                else x = ldexpf((float)(a >> 8) / 16777216.0f * 2.0f - 1.0f, (int)(seed % 40) - 30) * d * 256.0f;
                const float q0 = x * r;
                const float q1 = fmaf(fmaf(-d, q0, x), r, q0);
                const float q2 = fmaf(fmaf(-d, q1, x), r, q1);
                const float got = isfinite(q0) ? q2 : q0, want = x / d;
                ++n;
                if (!(got == want) && !(isnan(got) && isnan(want))) { if (bad < 5) printf("d=%a x=%a got=%a want=%a\n", d, x, got, want); ++bad; }
            }
        }
    }
    printf("checked %llu bad %llu\n", n, bad);
    return bad != 0;
}
"""


def test_shared_divisor_sequence_equals_division():
    with tempfile.TemporaryDirectory() as tmp:
        src, exe = os.path.join(tmp, "t.c"), os.path.join(tmp, "t")
        with open(src, "w") as fh:
            fh.write(SRC)
        subprocess.run(["gcc", "-O2", "-ffp-contract=off", "-o", exe, src, "-lm"], check=True)
        out = subprocess.run([exe], capture_output=True, text=True)
        assert out.returncode == 0, out.stdout[-800:]
        assert "bad 0" in out.stdout
