/*
 * q8_0_avx2.c -- AVX2/FMA/F16C restatement of the same arithmetic, for the timed CPU baseline.
 * TEST INFRASTRUCTURE ONLY (see q8_0_oracle.c): used by tests (to cross-check the scalar
 * restatement bit for bit) and by the benchmark's cpu_baseline leg.  Never linked into the product.
 *
 * The reference's own AVX2 source for this path cannot be built (it sits inside a block comment,
 * cpu/avx_2.hpp:229-5666, and uses aligned 256-bit loads on the 2-byte-aligned qs field,
 * :4565, :4602, :4654); this file performs the same operations in the same order with unaligned
 * loads.  Row work is handed out in chunks through one atomic counter, the reference's live
 * work-splitting pattern (cpu/avx_2.hpp:92-99).
 *
 * Build: gcc -O3 -mavx2 -mfma -mf16c -ffp-contract=off -pthread
 * (the reference's AVX2 flag set, cmake/detection/nihilus_detect_cpu_properties.cmake:175-180).
 */
#define _GNU_SOURCE
#include <immintrin.h>
#include <pthread.h>
#include <sched.h>
#include <stdatomic.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#define QK 32
#define BLK 34

/* cpu/common.hpp:215-221 */
uint16_t nha_fp32_to_fp16(float f) {
	return (uint16_t)_mm_extract_epi16(_mm_cvtps_ph(_mm_set_ss(f), _MM_FROUND_TO_NEAREST_INT), 0);
}
float nha_fp16_to_fp32(uint16_t h) {
	return _mm_cvtss_f32(_mm_cvtph_ps(_mm_cvtsi32_si128(h)));
}

static inline uint16_t ld_d(const uint8_t* blk) {
	uint16_t d;
	memcpy(&d, blk, 2);
	return d;
}

/* cpu/avx_2.hpp:4439-4489 */
void nha_quantize_row_q8_0(const float* x, void* vy, int64_t k) {
	uint8_t* y		 = (uint8_t*)vy;
	const int64_t nb = k / QK;
	for (int64_t i = 0; i < nb; ++i) {
		__m256 v0 = _mm256_loadu_ps(x);
		__m256 v1 = _mm256_loadu_ps(x + 8);
		__m256 v2 = _mm256_loadu_ps(x + 16);
		__m256 v3 = _mm256_loadu_ps(x + 24);
		x += 32;
		const __m256 sign = _mm256_set1_ps(-0.0f);
		__m256 mx		  = _mm256_andnot_ps(sign, v0);
		mx				  = _mm256_max_ps(mx, _mm256_andnot_ps(sign, v1));
		mx				  = _mm256_max_ps(mx, _mm256_andnot_ps(sign, v2));
		mx				  = _mm256_max_ps(mx, _mm256_andnot_ps(sign, v3));
		__m128 m4		  = _mm_max_ps(_mm256_extractf128_ps(mx, 1), _mm256_castps256_ps128(mx));
		m4				  = _mm_max_ps(m4, _mm_movehl_ps(m4, m4));
		m4				  = _mm_max_ss(m4, _mm_movehdup_ps(m4));
		const float amax  = _mm_cvtss_f32(m4);

		const float d	  = amax / 127.0f;
		const uint16_t dh = nha_fp32_to_fp16(d);
		const float id	  = (amax != 0.0f) ? 127.0f / amax : 0.0f;
		const __m256 mul  = _mm256_set1_ps(id);
		uint8_t* out	  = y + i * BLK;
		memcpy(out, &dh, 2);

		v0 = _mm256_round_ps(_mm256_mul_ps(v0, mul), _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
		v1 = _mm256_round_ps(_mm256_mul_ps(v1, mul), _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
		v2 = _mm256_round_ps(_mm256_mul_ps(v2, mul), _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
		v3 = _mm256_round_ps(_mm256_mul_ps(v3, mul), _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
		__m256i i0 = _mm256_cvtps_epi32(v0);
		__m256i i1 = _mm256_cvtps_epi32(v1);
		__m256i i2 = _mm256_cvtps_epi32(v2);
		__m256i i3 = _mm256_cvtps_epi32(v3);
		i0		   = _mm256_packs_epi32(i0, i1);
		i2		   = _mm256_packs_epi32(i2, i3);
		i0		   = _mm256_packs_epi16(i0, i2);
		i0		   = _mm256_permutevar8x32_epi32(i0, _mm256_setr_epi32(0, 4, 1, 5, 2, 6, 3, 7));
		_mm256_storeu_si256((__m256i*)(out + 2), i0);
	}
}

void nha_quantize_rows_q8_0(const float* x, void* vy, int64_t m, int64_t k) {
	const int64_t row_bytes = (k / QK) * BLK;
	for (int64_t i = 0; i < m; ++i) {
		nha_quantize_row_q8_0(x + i * k, (uint8_t*)vy + i * row_bytes, k);
	}
}

/* cpu/avx_2.hpp:4509-4524 */
static inline __m256 mul_sum_i8_pairs_float(__m256i x, __m256i y) {
	const __m256i ax  = _mm256_sign_epi8(x, x);
	const __m256i sy  = _mm256_sign_epi8(y, x);
	const __m256i dot = _mm256_maddubs_epi16(ax, sy);
	return _mm256_cvtepi32_ps(_mm256_madd_epi16(_mm256_set1_epi16(1), dot));
}
/* cpu/avx_2.hpp:4526-4532 */
static inline float hsum8(__m256 x) {
	__m128 r = _mm256_extractf128_ps(x, 1);
	r		 = _mm_add_ps(r, _mm256_castps256_ps128(x));
	r		 = _mm_add_ps(r, _mm_movehl_ps(r, r));
	r		 = _mm_add_ss(r, _mm_movehdup_ps(r));
	return _mm_cvtss_f32(r);
}
static inline __m256 fma_block(__m256 acc, const uint8_t* x, const uint8_t* y) {
	const __m256 d	 = _mm256_set1_ps(nha_fp16_to_fp32(ld_d(x)) * nha_fp16_to_fp32(ld_d(y)));
	const __m256i qx = _mm256_loadu_si256((const __m256i*)(x + 2));
	const __m256i qy = _mm256_loadu_si256((const __m256i*)(y + 2));
	return _mm256_fmadd_ps(d, mul_sum_i8_pairs_float(qx, qy), acc);
}

/* 16-block chunk, cpu/avx_2.hpp:4634-4677 */
static inline float dot16(const uint8_t* x, const uint8_t* y) {
	__m256 a0 = _mm256_setzero_ps(), a1 = a0, a2 = a0, a3 = a0;
	for (int b = 0; b < 16; b += 4) {
		a0 = fma_block(a0, x + (b + 0) * BLK, y + (b + 0) * BLK);
		a1 = fma_block(a1, x + (b + 1) * BLK, y + (b + 1) * BLK);
		a2 = fma_block(a2, x + (b + 2) * BLK, y + (b + 2) * BLK);
		a3 = fma_block(a3, x + (b + 3) * BLK, y + (b + 3) * BLK);
	}
	return hsum8(_mm256_add_ps(_mm256_add_ps(a0, a1), _mm256_add_ps(a2, a3)));
}

/* Only block counts that are multiples of 16 (every LLaMA shape on this path is); the
 * general-n branches live in the scalar restatement. cpu/avx_2.hpp:4715-4747 */
float nha_vec_dot_q8_0_q8_0_x16(int64_t n_blocks, const void* vx, const void* vy) {
	const uint8_t* x = (const uint8_t*)vx;
	const uint8_t* y = (const uint8_t*)vy;
	float total		 = 0.0f;
	for (int64_t c = 0; c < n_blocks / 16; ++c) {
		total = total + dot16(x + c * 16 * BLK, y + c * 16 * BLK);
	}
	return total;
}

/* ------------------------------------------------------------------ threaded GEMV / GEMM */

/* The t-th CPU of the mask this process may run on (a job is often confined to a subset of the machine's cores, so "core t"
 * is not a valid target in general); -1 if the mask holds fewer. */
static int nth_allowed_cpu(int t) {
	cpu_set_t set;
	if (sched_getaffinity(0, sizeof(set), &set) != 0) {
		return -1;
	}
	for (int c = 0; c < CPU_SETSIZE; ++c) {
		if (CPU_ISSET(c, &set) && t-- == 0) {
			return c;
		}
	}
	return -1;
}

typedef struct {
	const uint8_t* w;
	const uint8_t* aq;
	float* c;
	int64_t m_rows, n_rows, nb;
	int64_t chunk_rows;
	atomic_long* next_chunk;
	int cpu;
} job_t;

static void* worker(void* p) {
	job_t* j = (job_t*)p;
	if (j->cpu >= 0) {
		cpu_set_t set;
		CPU_ZERO(&set);
		CPU_SET(j->cpu, &set);
		pthread_setaffinity_np(pthread_self(), sizeof(set), &set); /* cpu/thread_pool.hpp:34-56 pins workers */
	}
	const int64_t row_bytes = j->nb * BLK;
	const int64_t n_chunks	= (j->n_rows + j->chunk_rows - 1) / j->chunk_rows;
	for (;;) {
		const long c = atomic_fetch_add(j->next_chunk, 1); /* chunk claiming, cpu/avx_2.hpp:92-99 */
		if (c >= n_chunks) {
			break;
		}
		const int64_t n0 = c * j->chunk_rows;
		const int64_t n1 = n0 + j->chunk_rows < j->n_rows ? n0 + j->chunk_rows : j->n_rows;
		for (int64_t n = n0; n < n1; ++n) {
			const uint8_t* wr = j->w + n * row_bytes;
			for (int64_t m = 0; m < j->m_rows; ++m) {
				j->c[m * j->n_rows + n] = nha_vec_dot_q8_0_q8_0_x16(j->nb, wr, j->aq + m * row_bytes);
			}
		}
	}
	return 0;
}

/* C[m*N+n] = dot(W row n, Aq row m); threads <= 0 means 1.  Returns 0, or -1 if k/32 % 16 != 0. */
int nha_gemm_q8_0_mt(const void* w, const void* aq, float* c, int64_t m_rows, int64_t n_rows, int64_t k, int threads, int pin) {
	const int64_t nb = k / QK;
	if (nb % 16 != 0) {
		return -1;
	}
	if (threads < 1) {
		threads = 1;
	}
	atomic_long next;
	atomic_init(&next, 0);
	job_t* jobs	   = (job_t*)malloc(sizeof(job_t) * (size_t)threads);
	pthread_t* tid = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)threads);
	for (int t = 0; t < threads; ++t) {
		jobs[t] = (job_t){ (const uint8_t*)w, (const uint8_t*)aq, c, m_rows, n_rows, nb, 16, &next, pin ? nth_allowed_cpu(t) : -1 };
	}
	for (int t = 0; t < threads; ++t) { /* the caller's own thread is left alone so its affinity is never changed */
		pthread_create(&tid[t], 0, worker, &jobs[t]);
	}
	for (int t = 0; t < threads; ++t) {
		pthread_join(tid[t], 0);
	}
	free(jobs);
	free(tid);
	return 0;
}

/* ------------------------------------------------------------------ timed baseline */

typedef struct {
	const uint8_t* w_all;
	int64_t n_mats, wsz;
	const float* x;
	uint8_t* xq;
	float* y;
	int64_t n_rows, k, nb;
	int iters;
	atomic_long* counters; /* one chunk counter per iteration, zeroed up front */
	pthread_barrier_t* bar;
	int tid, cpu;
} tjob_t;

static void* timed_worker(void* p) {
	tjob_t* j = (tjob_t*)p;
	if (j->cpu >= 0) {
		cpu_set_t set;
		CPU_ZERO(&set);
		CPU_SET(j->cpu, &set);
		pthread_setaffinity_np(pthread_self(), sizeof(set), &set);
	}
	const int64_t row_bytes	 = j->nb * BLK;
	const int64_t chunk_rows = 16;
	const int64_t n_chunks	 = (j->n_rows + chunk_rows - 1) / chunk_rows;
	for (int it = 0; it < j->iters; ++it) {
		if (j->tid == 0) {
			nha_quantize_row_q8_0(j->x, j->xq, j->k); /* once per activation row, as the reference intends */
		}
		pthread_barrier_wait(j->bar);
		const uint8_t* w = j->w_all + (int64_t)(it % j->n_mats) * j->wsz;
		for (;;) {
			const long c = atomic_fetch_add(&j->counters[it], 1);
			if (c >= n_chunks) {
				break;
			}
			const int64_t n0 = c * chunk_rows;
			const int64_t n1 = n0 + chunk_rows < j->n_rows ? n0 + chunk_rows : j->n_rows;
			for (int64_t n = n0; n < n1; ++n) {
				j->y[n] = nha_vec_dot_q8_0_q8_0_x16(j->nb, w + n * row_bytes, j->xq);
			}
		}
		pthread_barrier_wait(j->bar);
	}
	return 0;
}

/* Times `iters` passes of quantize(x) + GEMV with a persistent set of `threads` workers (created once,
 * outside the timed region is not possible with one call, so creation is amortised over iters), over
 * `n_mats` distinct weight matrices laid end to end: rotation keeps the last-level cache from serving
 * them.  Returns seconds per GEMV, or -1 on a shape this file does not handle. */
double nha_time_gemv(const void* w_all, int64_t n_mats, const float* x, float* y, int64_t n_rows, int64_t k, int threads, int pin, int iters) {
	const int64_t nb = k / QK;
	if (nb % 16 != 0 || iters < 1 || n_mats < 1) {
		return -1.0;
	}
	if (threads < 1) {
		threads = 1;
	}
	uint8_t* xq			  = (uint8_t*)aligned_alloc(64, (size_t)((nb * BLK + 63) / 64 * 64));
	atomic_long* counters = (atomic_long*)calloc((size_t)iters, sizeof(atomic_long));
	pthread_barrier_t bar;
	pthread_barrier_init(&bar, 0, (unsigned)threads);
	tjob_t* jobs   = (tjob_t*)malloc(sizeof(tjob_t) * (size_t)threads);
	pthread_t* tid = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)threads);
	for (int t = 0; t < threads; ++t) {
		jobs[t] = (tjob_t){ (const uint8_t*)w_all, n_mats, n_rows * nb * BLK, x, xq, y, n_rows, k, nb, iters, counters, &bar, t, pin ? nth_allowed_cpu(t) : -1 };
	}
	struct timespec t0, t1;
	clock_gettime(CLOCK_MONOTONIC, &t0);
	for (int t = 0; t < threads; ++t) {
		pthread_create(&tid[t], 0, timed_worker, &jobs[t]);
	}
	for (int t = 0; t < threads; ++t) {
		pthread_join(tid[t], 0);
	}
	clock_gettime(CLOCK_MONOTONIC, &t1);
	pthread_barrier_destroy(&bar);
	free(jobs);
	free(tid);
	free(counters);
	free(xq);
	return ((double)(t1.tv_sec - t0.tv_sec) + 1e-9 * (double)(t1.tv_nsec - t0.tv_nsec)) / (double)iters;
}
