/*
 * q8_0_oracle.c -- CPU restatement of the Q8_0 mat-mul arithmetic.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker that the GPU kernels are compared against.  Nothing that ships
 * (the HIP library, its host wrappers) may call into it; only tests, the smoke check and
 * the cpu_baseline leg of the benchmark do.
 *
 * It is written from the behaviour of the reference's (commented-out) AVX2 code, in plain
 * scalar C, with the SIMD lane structure spelled out so that the fp32 summation order is
 * the reference's.  Every function names the reference lines it restates
 * (paths relative to include/nihilus-incl/).
 *
 * Pinning status (what, besides this file, fixes each function's answers):
 *   nho_fp16_to_fp32 / nho_fp32_to_fp16  exhaustive 65536-value round trip, all midpoints between
 *                                        neighbouring halves (ties-to-even), numpy.float16 as an
 *                                        independent converter, F16C hardware in q8_0_avx2.c.
 *   layout (nho_block_*)                 the reference's tensor dumps Leaf_Data_0.json (byte sizes,
 *                                        first blocks of real Q8_0 tensors: every real block has
 *                                        max|q| == 127, which fails if d/qs offsets are wrong).
 *   nho_quantize_row_q8_0                closed-form invariants (zero block, amax -> +-127, odd
 *                                        symmetry, power-of-two scaling, constructed .5 ties go to
 *                                        even, trailing k%32 ignored) and an independent numpy
 *                                        evaluation.  No reference-held vector exists: the
 *                                        reference has no test of this function.
 *   nho_dequantize_row / nho_get_rows    independent numpy evaluation (numpy's own float16), real ggml blocks from
 *                                        the reference's dumps used as an embedding table, a table whose row r
 *                                        decodes to the constant r (index order), out-of-range ids.  The
 *                                        reference's dump of this op's output (inp_embd) covers a vocabulary row
 *                                        whose bytes are not in the dumps, so it cannot be replayed end to end.
 *   nho_rms_norm_*                       the reference's rms_norm has no live body and an ISA-dependent sqrtf_fast:
 *                                        pinned against float64 (sum of squares, scale, normalised row), by exact
 *                                        invariance under scaling the row by powers of two (eps = 0), and by
 *                                        constant rows whose answer is known in closed form.
 *   nho_expf / nho_silu_mul              no reference body exists (its silu kernels are empty): pinned against the
 *                                        correctly rounded double-precision value, <= 2 ulp over a dense sweep of
 *                                        the whole clamped range plus the special points; silu against float64.
 *   nho_block_sum_i32                    int64 brute force; extreme blocks (+-127 -> +-516128).
 *   nho_vec_dot_q8_f32 / nho_scalar_dot_q8_f32 / nho_mul_mat_q8_f32
 *                                        (fp32 activations, no activation quantize) float64 evaluation, d == 1 with integer
 *                                        activations gives exact integers, the two reference orders agree to rounding,
 *                                        equality with dequantize-then-dot in float64.
 *   nho_vec_dot_* / gemv / gemm          float64 evaluation (<= ~1e-6 rel), d == 1 gives exact
 *                                        integers, tiny hand-checkable shapes, gemm == M gemvs.
 *   The reference holds no golden vector for quantize or dot (its tests only print tok/s), and its
 *   own source for this path sits inside a block comment (cpu/avx_2.hpp:229-5666) and cannot be
 *   compiled, so there is no oracle/_ref build for it.
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math (see Makefile).  -ffp-contract=off matters:
 * the reference multiplies by the reciprocal and rounds in separate instructions.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define NHO_QK 32 /* Q_SIZE, common/data_types.hpp:28 */
#define NHO_BLOCK_BYTES 34 /* sizeof(block_q8_0<half>), common/data_types.hpp:38-44 */

/* ---------------------------------------------------------------- bits */

static inline uint32_t f32_bits(float f) {
	uint32_t u;
	memcpy(&u, &f, 4);
	return u;
}
static inline float bits_f32(uint32_t u) {
	float f;
	memcpy(&f, &u, 4);
	return f;
}

/* ---------------------------------------------------------------- fp16 */

/* fp16 -> fp32, exact.  Restates what vcvtph2ps does (cpu/common.hpp:219-221). */
float nho_fp16_to_fp32(uint16_t h) {
	const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
	const uint32_t exp	= (h >> 10) & 0x1Fu;
	const uint32_t man	= h & 0x3FFu;
	if (exp == 0x1Fu) { /* inf / nan */
		return bits_f32(sign | 0x7F800000u | (man << 13));
	}
	if (exp == 0) {
		if (man == 0) {
			return bits_f32(sign);
		}
		/* subnormal: man * 2^-24, exactly representable */
		float v = (float)man * bits_f32(0x33800000u); /* 2^-24 */
		return bits_f32(f32_bits(v) | sign);
	}
	return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* fp32 -> fp16, round to nearest even, subnormals kept, overflow -> inf, nan -> quiet nan.
 * Semantics of vcvtps2ph with _MM_FROUND_TO_NEAREST_INT (cpu/common.hpp:215-217); the dead
 * quantizer calls a software twin meant to equal it (cpu/avx_2.hpp:4418-4437).  Written here
 * as explicit integer rounding rather than the float-add trick, so the two cannot share a bug. */
uint16_t nho_fp32_to_fp16(float f) {
	const uint32_t w	= f32_bits(f);
	const uint16_t sign = (uint16_t)((w >> 16) & 0x8000u);
	const uint32_t a	= w & 0x7FFFFFFFu;
	if (a > 0x7F800000u) {
		return (uint16_t)(sign | 0x7E00u);
	}
	if (a >= 0x47800000u) { /* >= 65536: inf (65520..65536 handled by rounding below) */
		return (uint16_t)(sign | 0x7C00u);
	}
	const int32_t e = (int32_t)(a >> 23) - 127; /* unbiased */
	uint32_t m		= (a & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
	if ((a >> 23) == 0) {
		return sign; /* fp32 subnormal: far below half of the smallest fp16 subnormal */
	}
	int shift; /* number of low bits to drop from the 24-bit significand */
	uint32_t base;
	if (e >= -14) {
		shift = 13;
		base  = (uint32_t)(e + 15) << 10;
		m &= 0x7FFFFFu; /* hidden bit is carried by the exponent field */
	} else {
		shift = 13 + (-14 - e);
		base  = 0;
		if (shift > 25) {
			return sign; /* < 2^-26: rounds to zero */
		}
	}
	const uint32_t keep = m >> shift;
	const uint32_t rem	= m & ((1u << shift) - 1u);
	const uint32_t half = 1u << (shift - 1);
	uint32_t r			= base + keep;
	if (rem > half || (rem == half && (r & 1u))) {
		r += 1; /* may carry into the exponent, up to 0x7C00 = inf: both are correct */
	}
	return (uint16_t)(sign | r);
}

/* ---------------------------------------------------------------- layout */

/* A row of blocks is a packed byte stream: block b at byte 34*b = { u16 d (LE); i8 qs[32] }.
 * common/data_types.hpp:38-44, common/type_traits.hpp:185-193. */
static inline uint16_t blk_d(const uint8_t* row, int64_t b) {
	const uint8_t* p = row + b * NHO_BLOCK_BYTES;
	return (uint16_t)(p[0] | ((uint16_t)p[1] << 8));
}
static inline const int8_t* blk_qs(const uint8_t* row, int64_t b) {
	return (const int8_t*)(row + b * NHO_BLOCK_BYTES + 2);
}

uint16_t nho_block_d(const void* row, int64_t b) {
	return blk_d((const uint8_t*)row, b);
}
void nho_block_qs(const void* row, int64_t b, int8_t* out32) {
	memcpy(out32, blk_qs((const uint8_t*)row, b), NHO_QK);
}

/* total bytes of a [rows x k] Q8_0 tensor: type_traits<...>::total_byte_size, type_traits.hpp:38-61 */
int64_t nho_q8_0_bytes(int64_t rows, int64_t k) {
	return rows * (k / NHO_QK) * NHO_BLOCK_BYTES;
}

/* y = d * q, the live token-embedding dequant (cpu/avx_2.hpp:40-66; dead twin :4290-4302) */
void nho_dequantize_row_q8_0(const void* vx, float* y, int64_t k) {
	const uint8_t* row = (const uint8_t*)vx;
	const int64_t nb   = k / NHO_QK;
	for (int64_t b = 0; b < nb; ++b) {
		const float d	 = nho_fp16_to_fp32(blk_d(row, b));
		const int8_t* qs = blk_qs(row, b);
		for (int j = 0; j < NHO_QK; ++j) {
			y[b * NHO_QK + j] = (float)qs[j] * d;
		}
	}
}

/* Token-embedding lookup: row ids[t] of the [n_rows x k] block matrix, dequantized, for every token
 * (cpu/avx_2.hpp:80-103 prompt phase, :112-135 eval phase; per-op form :1241-1294).  The reference reads any row an
 * id names; the GPU library defines an id outside [0, n_rows) as a row of zeros, restated here so both can be
 * compared on such inputs.  Returns the number of such ids. */
int64_t nho_get_rows_q8_0(const void* vw, const int32_t* ids, float* out, int64_t n_tokens, int64_t n_rows, int64_t k) {
	const uint8_t* w	   = (const uint8_t*)vw;
	const int64_t row_size = (k / NHO_QK) * NHO_BLOCK_BYTES;
	int64_t invalid		   = 0;
	for (int64_t t = 0; t < n_tokens; ++t) {
		const int64_t id = ids[t];
		if (id < 0 || id >= n_rows) {
			for (int64_t j = 0; j < k; ++j) {
				out[t * k + j] = 0.0f;
			}
			++invalid;
			continue;
		}
		nho_dequantize_row_q8_0(w + id * row_size, out + t * k, k);
	}
	return invalid;
}

/* ---------------------------------------------------------------- RMS norm */

/* 1 / sqrt(mean(x^2) + eps) with the sum of squares taken in the order of the GPU kernels' 1024-thread workgroup:
 * the row's G = k / 128 groups are cut into 16 contiguous runs (q = G / 16 groups each, the first G % 16 runs one more);
 * lane l of wave w folds the float4s l, l + 64, ... of run w by fma; each 64-lane wave is reduced by an xor butterfly
 * over lane distances 32, 16, ..., 1; the 16 wave sums are added in wave order.  The rms_norm node of the reference's
 * graph (infra/core_traits.hpp:570, :971, :1186); its dead CPU attempt (cpu/avx_2.hpp:5331-5347) sums 8 AVX lanes and
 * calls sqrtf_fast, which is vsqrt on NEON and a bit trick elsewhere (cpu/common.hpp:310, :448): here the square root
 * and the divides are the IEEE ones.  k % 128 == 0. */
float nho_rms_norm_scale(const float* x, int64_t k, float eps) {
	float wave_sum[16];
	const int64_t groups = k / 128, q = groups / 16, r = groups % 16;
	for (int w = 0; w < 16; ++w) {
		const int64_t g0 = w * q + (w < r ? w : r);
		const int64_t n4 = (q + (w < r ? 1 : 0)) * 32;
		const float* run = x + g0 * 128;
		float lane[64], next[64];
		for (int l = 0; l < 64; ++l) {
			float p = 0.0f;
			for (int64_t j = l; j < n4; j += 64) {
				for (int e = 0; e < 4; ++e) {
					p = fmaf(run[4 * j + e], run[4 * j + e], p);
				}
			}
			lane[l] = p;
		}
		for (int off = 32; off >= 1; off >>= 1) {
			for (int l = 0; l < 64; ++l) {
				volatile float s = lane[l] + lane[l ^ off];
				next[l]			 = s;
			}
			memcpy(lane, next, sizeof(lane));
		}
		wave_sum[w] = lane[0];
	}
	volatile float sum = wave_sum[0];
	for (int w = 1; w < 16; ++w) {
		sum = sum + wave_sum[w];
	}
	volatile float mean = sum / (float)k;
	volatile float arg	= mean + eps;
	volatile float root = sqrtf(arg);
	return 1.0f / root;
}

/* y_i = (x_i * scale) * w_i: the rms_norm node, then the mul node with the norm weight (infra/core_traits.hpp:570-573) */
void nho_rms_norm_mul_row(const float* x, const float* w, float eps, float* y, int64_t k) {
	const float scale = nho_rms_norm_scale(x, k, eps);
	for (int64_t i = 0; i < k; ++i) {
		volatile float t = x[i] * scale;
		y[i]			 = t * w[i];
	}
}

void nho_quantize_row_q8_0(const float* x, void* vy, int64_t k);

/* xq[m] = quantize_row_q8_0(rms_norm(x[m]) * w), m rows of k */
void nho_rms_norm_quantize_rows_q8_0(const float* x, const float* w, float eps, void* vy, int64_t m, int64_t k, float* scratch_row) {
	uint8_t* y = (uint8_t*)vy;
	for (int64_t r = 0; r < m; ++r) {
		nho_rms_norm_mul_row(x + r * k, w, eps, scratch_row, k);
		nho_quantize_row_q8_0(scratch_row, y + r * (k / NHO_QK) * NHO_BLOCK_BYTES, k);
	}
}

/* ---------------------------------------------------------------- FFN activation */

void nho_quantize_row_q8_0(const float* x, void* vy, int64_t k);

/* exp(x) as a fixed sequence of correctly rounded fp32 operations: n = rne(x * log2 e), two-part ln 2 reduction by
 * fma, degree-5 polynomial (Cephes single-precision coefficients) by fma, 2^n by exponent insertion; argument clamped
 * to [-87, 88].  Not a restatement of reference code (the reference's silu kernels are empty, cpu/avx_2.hpp:1946-2075):
 * it exists so that the GPU and this checker evaluate the model's SiLU with the same bits.  Pinned against the
 * correctly rounded value (double exp) to <= 2 ulp over a dense sweep. */
float nho_expf(float x) {
	x				 = fminf(fmaxf(x, -87.0f), 88.0f);
	volatile float t = x * 1.44269504088896341f;
	const float n	 = nearbyintf(t);
	float r			 = fmaf(n, -0.693359375f, x);
	r				 = fmaf(n, 2.12194440e-4f, r);
	float p			 = 1.9875691500e-4f;
	p				 = fmaf(p, r, 1.3981999507e-3f);
	p				 = fmaf(p, r, 8.3334519073e-3f);
	p				 = fmaf(p, r, 4.1665795894e-2f);
	p				 = fmaf(p, r, 1.6666665459e-1f);
	p				 = fmaf(p, r, 5.0000001201e-1f);
	volatile float r2 = r * r;
	volatile float e  = fmaf(p, r2, r);
	e				  = e + 1.0f;
	union {
		uint32_t u;
		float f;
	} two_n;
	two_n.u = (uint32_t)((int32_t)n + 127) << 23;
	return e * two_n.f;
}

/* silu(g) * u with silu(g) = g / (1 + exp(-g)): ffn_silu then ffn_gate_par (mul) of the reference's graph
 * (infra/core_traits.hpp:982-986); IEEE divide, separate multiply. */
float nho_silu_mul(float g, float u) {
	volatile float den = 1.0f + nho_expf(-g);
	volatile float s   = g / den;
	return s * u;
}

/* xq = quantize_row_q8_0(silu(gate) * up), m rows of k */
void nho_silu_mul_quantize_rows_q8_0(const float* gate, const float* up, void* vy, int64_t m, int64_t k) {
	float act[NHO_QK];
	uint8_t* y		 = (uint8_t*)vy;
	const int64_t nb = k / NHO_QK;
	for (int64_t r = 0; r < m; ++r) {
		for (int64_t b = 0; b < nb; ++b) {
			for (int j = 0; j < NHO_QK; ++j) {
				act[j] = nho_silu_mul(gate[r * k + b * NHO_QK + j], up[r * k + b * NHO_QK + j]);
			}
			nho_quantize_row_q8_0(act, y + (r * nb + b) * NHO_BLOCK_BYTES, NHO_QK);
		}
	}
}

/* ---------------------------------------------------------------- quantize */

/* cpu/avx_2.hpp:4439-4489 (twin :671-721).
 *   amax  = max |x_i| over the block                                   (:4449-4458)
 *   d     = amax / 127.f in fp32, stored as fp16 RNE                   (:4460-4461)
 *   id    = amax != 0 ? 127.f / amax : 0                               (:4462)
 *   q_i   = (int8) round_half_even(x_i * id), product rounded to fp32 first   (:4465-4478)
 *   packs are saturating (:4480-4482) -- for finite input |x_i*id| <= 127 unless 127/amax overflows (see below).
 *   nb = k / 32; a trailing partial block is ignored                   (:4440)                */
void nho_quantize_row_q8_0(const float* x, void* vy, int64_t k) {
	uint8_t* y		 = (uint8_t*)vy;
	const int64_t nb = k / NHO_QK;
	for (int64_t b = 0; b < nb; ++b) {
		const float* xb = x + b * NHO_QK;
		float amax		= 0.0f;
		for (int j = 0; j < NHO_QK; ++j) {
			const float a = fabsf(xb[j]);
			if (a > amax) {
				amax = a;
			}
		}
		const float d	   = amax / 127.0f;
		const uint16_t dh  = nho_fp32_to_fp16(d);
		const float id	   = (amax != 0.0f) ? 127.0f / amax : 0.0f;
		uint8_t* out	   = y + b * NHO_BLOCK_BYTES;
		out[0]			   = (uint8_t)(dh & 0xFFu);
		out[1]			   = (uint8_t)(dh >> 8);
		for (int j = 0; j < NHO_QK; ++j) {
			volatile float p = xb[j] * id; /* one fp32 rounding, never fused with anything */
			float r			 = nearbyintf(p); /* default rounding mode: ties to even */
			/* cvtps_epi32 (:4475-4478) returns the "integer indefinite" 0x80000000 for NaN and for values outside
			 * int32; that only happens when 127/amax overflows to inf (amax below ~3.7e-37): inf and 0*inf = NaN
			 * then both saturate to -128 in the packs. */
			int32_t q = (r >= -2147483648.0f && r < 2147483648.0f) ? (int32_t)r : INT32_MIN;
			if (q > 127) {
				q = 127;
			}
			if (q < -128) {
				q = -128;
			}
			out[2 + j] = (uint8_t)(int8_t)q;
		}
	}
}

void nho_quantize_rows_q8_0(const float* x, void* vy, int64_t m, int64_t k) {
	const int64_t row_bytes = (k / NHO_QK) * NHO_BLOCK_BYTES;
	for (int64_t i = 0; i < m; ++i) {
		nho_quantize_row_q8_0(x + i * k, (uint8_t*)vy + i * row_bytes, k);
	}
}

/* ---------------------------------------------------------------- integer block dot */

/* mul_sum_i8_pairs_float, cpu/avx_2.hpp:4509-4524: lane j (0..7) = sum_{i=4j..4j+3} x_i*y_i as
 * int32 (maddubs pair sums <= 2*127^2 never saturate for quants in [-127,127]), then cvtepi32_ps,
 * which is exact because |lane| <= 4*127*127 = 64516 < 2^24. */
static inline void lanes8_i32(const int8_t* x, const int8_t* y, int32_t lane[8]) {
	for (int j = 0; j < 8; ++j) {
		int32_t s = 0;
		for (int i = 0; i < 4; ++i) {
			s += (int32_t)x[4 * j + i] * (int32_t)y[4 * j + i];
		}
		lane[j] = s;
	}
}

int32_t nho_block_sum_i32(const void* vx, int64_t bx, const void* vy, int64_t by) {
	int32_t lane[8];
	lanes8_i32(blk_qs((const uint8_t*)vx, bx), blk_qs((const uint8_t*)vy, by), lane);
	int32_t s = 0;
	for (int j = 0; j < 8; ++j) {
		s += lane[j];
	}
	return s;
}

/* sums[n*nb + b] for a weight matrix against one quantized activation row */
void nho_block_sums_gemv(const void* w, const void* xq, int32_t* sums, int64_t n_rows, int64_t k) {
	const int64_t nb		= k / NHO_QK;
	const int64_t row_bytes = nb * NHO_BLOCK_BYTES;
	for (int64_t n = 0; n < n_rows; ++n) {
		const uint8_t* wr = (const uint8_t*)w + n * row_bytes;
		for (int64_t b = 0; b < nb; ++b) {
			sums[n * nb + b] = nho_block_sum_i32(wr, b, xq, b);
		}
	}
}

/* ---------------------------------------------------------------- fp32 dot, reference order */

typedef struct {
	float v[8];
} lanes8_f;

static inline lanes8_f l8_zero(void) {
	lanes8_f r;
	for (int j = 0; j < 8; ++j) {
		r.v[j] = 0.0f;
	}
	return r;
}
static inline lanes8_f l8_add(lanes8_f a, lanes8_f b) {
	lanes8_f r;
	for (int j = 0; j < 8; ++j) {
		r.v[j] = a.v[j] + b.v[j];
	}
	return r;
}
/* acc = fmadd(d, q, acc) per lane, cpu/avx_2.hpp:4567, :4610-4611, :4667-4670 */
static inline lanes8_f l8_fma_block(lanes8_f acc, const uint8_t* x, const uint8_t* y, int64_t b) {
	const float d = nho_fp16_to_fp32(blk_d(x, b)) * nho_fp16_to_fp32(blk_d(y, b)); /* one fp32 rounding (exact in fact: 11x11 bits) */
	int32_t lane[8];
	lanes8_i32(blk_qs(x, b), blk_qs(y, b), lane);
	for (int j = 0; j < 8; ++j) {
		acc.v[j] = fmaf(d, (float)lane[j], acc.v[j]);
	}
	return acc;
}
/* hsum_float_8, cpu/avx_2.hpp:4526-4532: hi128+lo128, then [0]+=[2],[1]+=[3], then [0]+[1] */
static inline float l8_hsum(lanes8_f x) {
	float r[4];
	for (int j = 0; j < 4; ++j) {
		r[j] = x.v[j + 4] + x.v[j];
	}
	const float r0 = r[0] + r[2];
	const float r1 = r[1] + r[3];
	return r0 + r1;
}

/* scalar form for fewer than 4 blocks, cpu/avx_2.hpp:4536-4553: sumf += sumi * (dx*dy), the
 * multiply and the add taken as two roundings (the C abstract machine; a compiler allowed to
 * contract would fuse them -- the reference leaves that to its build flags, so inputs that reach
 * this branch are checked with a tolerance, never bit-exactly). */
static float dot_scalar(const uint8_t* x, const uint8_t* y, int64_t n) {
	float sumf = 0.0f;
	for (int64_t b = 0; b < n; ++b) {
		int64_t sumi	 = 0;
		const int8_t* qx = blk_qs(x, b);
		const int8_t* qy = blk_qs(y, b);
		for (int j = 0; j < NHO_QK; ++j) {
			sumi += (int64_t)qx[j] * (int64_t)qy[j];
		}
		const float dd		= nho_fp16_to_fp32(blk_d(x, b)) * nho_fp16_to_fp32(blk_d(y, b));
		volatile float prod = (float)sumi * dd;
		sumf				= sumf + prod;
	}
	return sumf;
}

/* vec_dot_q8_0_q8_0<n>::impl for compile-time n, all branches, cpu/avx_2.hpp:4536-4747. */
static float dot_fixed(const uint8_t* x, const uint8_t* y, int64_t n) {
	if (n <= 0) {
		return 0.0f;
	}
	if (n < 4) {
		return dot_scalar(x, y, n); /* :4536-4553 */
	}
	if (n == 4) { /* :4555-4572, one accumulator */
		lanes8_f acc = l8_zero();
		for (int b = 0; b < 4; ++b) {
			acc = l8_fma_block(acc, x, y, b);
		}
		return l8_hsum(acc);
	}
	if (n < 8) { /* :4574-4587 */
		float s = dot_fixed(x, y, 4);
		s		= s + dot_fixed(x + 4 * NHO_BLOCK_BYTES, y + 4 * NHO_BLOCK_BYTES, n - 4);
		return s;
	}
	if (n == 8) { /* :4589-4617, two accumulators, even/odd blocks */
		lanes8_f a0 = l8_zero(), a1 = l8_zero();
		for (int b = 0; b < 8; b += 2) {
			a0 = l8_fma_block(a0, x, y, b);
			a1 = l8_fma_block(a1, x, y, b + 1);
		}
		return l8_hsum(l8_add(a0, a1));
	}
	if (n < 16) { /* :4619-4632 */
		float s = dot_fixed(x, y, 8);
		s		= s + dot_fixed(x + 8 * NHO_BLOCK_BYTES, y + 8 * NHO_BLOCK_BYTES, n - 8);
		return s;
	}
	if (n == 16) { /* :4634-4677, four accumulators, block b -> acc[b%4] */
		lanes8_f a[4] = { l8_zero(), l8_zero(), l8_zero(), l8_zero() };
		for (int b = 0; b < 16; b += 4) {
			for (int t = 0; t < 4; ++t) {
				a[t] = l8_fma_block(a[t], x, y, b + t);
			}
		}
		return l8_hsum(l8_add(l8_add(a[0], a[1]), l8_add(a[2], a[3])));
	}
	/* n > 16, :4715-4747: chunks of 16 added left to right, then the remainder chunk */
	const int64_t total_chunks = (n + 15) / 16;
	const int64_t rem		   = n % 16;
	float total				   = 0.0f;
	for (int64_t c = 0; c < total_chunks - 1; ++c) {
		total = total + dot_fixed(x + c * 16 * NHO_BLOCK_BYTES, y + c * 16 * NHO_BLOCK_BYTES, 16);
	}
	const int64_t last = total_chunks - 1;
	total = total + dot_fixed(x + last * 16 * NHO_BLOCK_BYTES, y + last * 16 * NHO_BLOCK_BYTES, rem == 0 ? 16 : rem);
	return total;
}

float nho_vec_dot_q8_0_q8_0(int64_t n_blocks, const void* vx, const void* vy) {
	return dot_fixed((const uint8_t*)vx, (const uint8_t*)vy, n_blocks);
}

/* Runtime-length variant vec_dot_q8_0_q8_0_impl, cpu/avx_2.hpp:4749-4780: one 8-lane accumulator
 * over all blocks, one hsum.  n is the element count (k), as in the reference. */
float nho_vec_dot_q8_0_q8_0_rt(int64_t n, const void* vx, const void* vy) {
	const int64_t nb = n / NHO_QK;
	lanes8_f acc	 = l8_zero();
	for (int64_t b = 0; b < nb; ++b) {
		acc = l8_fma_block(acc, (const uint8_t*)vx, (const uint8_t*)vy, b);
	}
	return l8_hsum(acc);
}

/* float64 evaluation of the same sum: the error-budget yardstick, order-free to ~1e-16. */
double nho_vec_dot_f64(int64_t n_blocks, const void* vx, const void* vy) {
	double s = 0.0;
	for (int64_t b = 0; b < n_blocks; ++b) {
		const double dd = (double)nho_fp16_to_fp32(blk_d((const uint8_t*)vx, b)) * (double)nho_fp16_to_fp32(blk_d((const uint8_t*)vy, b));
		s += dd * (double)nho_block_sum_i32(vx, b, vy, b);
	}
	return s;
}

/* ---------------------------------------------------------------- mat-vec / mat-mat */

/* y[n] = dot(W row n, xq); the GEMV the dead dispatcher intends (cpu/avx_2.hpp:1371-1444 shape,
 * leaf :4715-4747).  W is [n_rows][k/32] blocks row-major, xq is [k/32] blocks. */
void nho_gemv_q8_0(const void* w, const void* xq, float* y, int64_t n_rows, int64_t k) {
	const int64_t nb		= k / NHO_QK;
	const int64_t row_bytes = nb * NHO_BLOCK_BYTES;
	for (int64_t n = 0; n < n_rows; ++n) {
		y[n] = dot_fixed((const uint8_t*)w + n * row_bytes, (const uint8_t*)xq, nb);
	}
}

void nho_gemv_q8_0_f64(const void* w, const void* xq, double* y, int64_t n_rows, int64_t k) {
	const int64_t nb		= k / NHO_QK;
	const int64_t row_bytes = nb * NHO_BLOCK_BYTES;
	for (int64_t n = 0; n < n_rows; ++n) {
		y[n] = nho_vec_dot_f64(nb, (const uint8_t*)w + n * row_bytes, xq);
	}
}

/* C[m*N + n]: n fastest, as ggml's dst[ir1*nr0 + ir0] (cpu/avx_2.hpp:4934, :4959).
 * Output dims [ne0 = N, ne1 = M] (common/kernel_traits.hpp:393-417). */
void nho_gemm_q8_0(const void* w, const void* aq, float* c, int64_t m_rows, int64_t n_rows, int64_t k) {
	const int64_t nb		= k / NHO_QK;
	const int64_t row_bytes = nb * NHO_BLOCK_BYTES;
	for (int64_t m = 0; m < m_rows; ++m) {
		nho_gemv_q8_0(w, (const uint8_t*)aq + m * row_bytes, c + m * n_rows, n_rows, k);
	}
}

/* ---------------------------------------------------------------- synthetic inputs */

/* Counter-based generator shared (by specification, not by code) with the GPU fill kernels, so the
 * CPU and the GPU see the same bytes without either depending on a library's random stream.
 *   h(seed, i) = splitmix64 finaliser of seed + (i+1)*golden
 *   gauss(seed, i): twelve 16-bit uniforms from three hashes, summed (Irwin-Hall, variance 1):
 *                   g = (sum - 393210) / 65536 exactly in fp32
 *   weight block t: qs[j] = ((u16 * 255) >> 16) - 127  -> uniform over [-127,127];
 *                   d = fp16(|gauss| * 0.01f)                                                  */
/* ---- fp32 activations against Q8_0 weights, no activation quantize (the one mul_mat with a body in the reference) ---- */

/* cpu/avx_2.hpp:4798-4816 (one block: sum of x_i * float(q_i) in element order, then times the scale) summed block after
 * block as :4834-4851 does for a row of whole blocks; the eval_time dispatcher calls it per output row (:4978-5004). */
float nho_vec_dot_q8_f32(const float* x, const void* vw, int64_t n_blocks) {
	const uint8_t* w = (const uint8_t*)vw;
	float sum		 = 0.0f;
	for (int64_t b = 0; b < n_blocks; ++b) {
		const float scale = nho_fp16_to_fp32(blk_d(w, b));
		const int8_t* qs  = blk_qs(w, b);
		float s			  = 0.0f;
		for (int i = 0; i < NHO_QK; ++i) {
			s += x[b * NHO_QK + i] * (float)qs[i];
		}
		sum += s * scale;
	}
	return sum;
}

/* cpu/avx_2.hpp:4881-4900, the prompt_eval_time dispatcher's leaf: sum += x * (float(q) * scale), element after element. */
float nho_scalar_dot_q8_f32(const float* x, const void* vw, int64_t n_blocks) {
	const uint8_t* w = (const uint8_t*)vw;
	float sum		 = 0.0f;
	for (int64_t b = 0; b < n_blocks; ++b) {
		const float scale = nho_fp16_to_fp32(blk_d(w, b));
		const int8_t* qs  = blk_qs(w, b);
		for (int i = 0; i < NHO_QK; ++i) {
			sum += x[b * NHO_QK + i] * ((float)qs[i] * scale);
		}
	}
	return sum;
}

double nho_dot_q8_f32_f64(const float* x, const void* vw, int64_t n_blocks) {
	const uint8_t* w = (const uint8_t*)vw;
	double sum		 = 0.0;
	for (int64_t b = 0; b < n_blocks; ++b) {
		const double scale = (double)nho_fp16_to_fp32(blk_d(w, b));
		const int8_t* qs   = blk_qs(w, b);
		double s		   = 0.0;
		for (int i = 0; i < NHO_QK; ++i) {
			s += (double)x[b * NHO_QK + i] * (double)qs[i];
		}
		sum += s * scale;
	}
	return sum;
}

/* y[m][n] (n fastest, :4934 / :4959): order 0 = the eval_time leaf for every row, 1 = the prompt_eval_time leaf. */
void nho_mul_mat_q8_f32(const void* vw, const float* x, float* y, int64_t m_rows, int64_t n_rows, int64_t k, int order) {
	const uint8_t* w = (const uint8_t*)vw;
	const int64_t nb = k / NHO_QK;
	for (int64_t m = 0; m < m_rows; ++m) {
		for (int64_t n = 0; n < n_rows; ++n) {
			const uint8_t* row = w + n * nb * NHO_BLOCK_BYTES;
			y[m * n_rows + n]  = order ? nho_scalar_dot_q8_f32(x + m * k, row, nb) : nho_vec_dot_q8_f32(x + m * k, row, nb);
		}
	}
}

void nho_mul_mat_q8_f32_f64(const void* vw, const float* x, double* y, int64_t m_rows, int64_t n_rows, int64_t k) {
	const uint8_t* w = (const uint8_t*)vw;
	const int64_t nb = k / NHO_QK;
	for (int64_t m = 0; m < m_rows; ++m) {
		for (int64_t n = 0; n < n_rows; ++n) {
			y[m * n_rows + n] = nho_dot_q8_f32_f64(x + m * k, w + n * nb * NHO_BLOCK_BYTES, nb);
		}
	}
}

static inline uint64_t nho_hash(uint64_t seed, uint64_t i) {
	uint64_t z = seed + (i + 1) * 0x9E3779B97F4A7C15ull;
	z		   = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
	z		   = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
	return z ^ (z >> 31);
}
static inline float nho_gauss(uint64_t seed, uint64_t i) {
	int32_t s = 0;
	for (int t = 0; t < 3; ++t) {
		uint64_t h = nho_hash(seed, 3 * i + (uint64_t)t);
		s += (int32_t)(h & 0xFFFF) + (int32_t)((h >> 16) & 0xFFFF) + (int32_t)((h >> 32) & 0xFFFF) + (int32_t)((h >> 48) & 0xFFFF);
	}
	return (float)(s - 393210) * (1.0f / 65536.0f);
}

void nho_fill_activations(uint64_t seed, float* x, int64_t count) {
	for (int64_t i = 0; i < count; ++i) {
		x[i] = nho_gauss(seed ^ 0xA5A5A5A5A5A5A5A5ull, (uint64_t)i);
	}
}

/* n_blocks consecutive 34-byte blocks starting at global block index first_block */
void nho_fill_weight_blocks(uint64_t seed, void* out, int64_t first_block, int64_t n_blocks) {
	uint8_t* p = (uint8_t*)out;
	for (int64_t t = 0; t < n_blocks; ++t) {
		const uint64_t blk = (uint64_t)(first_block + t);
		volatile float ds  = fabsf(nho_gauss(seed ^ 0x5EED5EED5EED5EEDull, blk)) * 0.01f;
		const uint16_t dh  = nho_fp32_to_fp16(ds);
		uint8_t* o		   = p + t * NHO_BLOCK_BYTES;
		o[0]			   = (uint8_t)(dh & 0xFF);
		o[1]			   = (uint8_t)(dh >> 8);
		for (int g = 0; g < 8; ++g) {
			uint64_t h = nho_hash(seed, blk * 8 + (uint64_t)g);
			for (int j = 0; j < 4; ++j) {
				const uint32_t u = (uint32_t)((h >> (16 * j)) & 0xFFFF);
				o[2 + 4 * g + j] = (uint8_t)(int8_t)((int32_t)((u * 255u) >> 16) - 127);
			}
		}
	}
}
