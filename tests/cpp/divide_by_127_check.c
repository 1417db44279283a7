/* The device quantizer's short route divides by 127 as q = a * c, r = fma(-127, q, a), d = fma(r, c, q), c = fl32(1 / 127)
 * (nihilus_amd/csrc/q8_0_device.h, quantize_block_lane).  This program checks on the host that the result equals the correctly
 * rounded quotient a / 127.f for every fp32 mantissa, at the two ends of the exponent range the route accepts and three exponents
 * between (powers of two scale exactly within the normal range, so the mantissa is what matters).  Prints the number of
 * mismatches; exit status 0 only if there are none. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

int main(void) {
	const float c = 1.0f / 127.0f;
	long bad	  = 0;
	for (int e = -2; e <= 2; ++e) {
		for (uint32_t m = 0; m < (1u << 23); ++m) {
			const uint32_t bits = ((uint32_t)(127 + e * 30) << 23) | m; /* 2^-60, 2^-30, 1, 2^30, 2^60 times [1, 2) */
			float a;
			memcpy(&a, &bits, 4);
			volatile float q	= a * c;
			volatile float r	= fmaf(-127.0f, q, a);
			volatile float d	= fmaf(r, c, q);
			volatile float want = a / 127.0f;
			if (d != want) {
				if (bad < 5) {
					printf("mismatch a=%a got %a want %a\n", a, d, want);
				}
				++bad;
			}
		}
	}
	printf("mismatches %ld\n", bad);
	return bad == 0 ? 0 : 1;
}
