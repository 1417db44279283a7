// Do the matrix pipe and the VALU of a gfx950 SIMD overlap?  The Q8_0 mat-mat spends one int8 MFMA per (32 x 32 tile,
// 32-quant block) and, because both operands carry a scale per block, 16 conversions + 16 multiply-adds per lane on its
// result before the next block: whether those two kinds of work run side by side or one after the other decides the
// kernel's ceiling.  One workgroup on one CU, 1 / 2 / 4 waves per SIMD, every wave the same loop; per iteration and wave
//   matrix part: 4 x v_mfma_i32_32x32x32_i8,   VALU part: 64 x v_cvt_f32_i32 + 64 x v_fmac_f32
// in five arrangements: matrix only; VALU only; both with the VALU work independent of the MFMA results; both with the
// VALU folding the PREVIOUS MFMA's result (software-pipelined by one); both with the VALU folding the MFMA just issued
// (the mat-mat's loop as written).  Instruction order is pinned with sched_barrier.  Reported: clocks of SIMD time per
// wave-iteration (clock64 of the slowest wave / iterations / waves per SIMD).  Overlap would give max(matrix, VALU) for
// "both"; no overlap gives their sum.  A measurement tool beside the tests; prints one JSON object.
#include <hip/hip_runtime.h>

#include <cstdio>

#define CK(x)                                                         \
	do {                                                              \
		hipError_t e_ = (x);                                          \
		if (e_ != hipSuccess) {                                       \
			std::printf("FAILED %s: %s\n", #x, hipGetErrorString(e_)); \
			return 1;                                                 \
		}                                                             \
	} while (0)

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

enum arrangement : int { MATRIX_ONLY = 0, VALU_ONLY = 1, BOTH_INDEPENDENT = 2, BOTH_FOLD_PREVIOUS = 3, BOTH_FOLD_CURRENT = 4, ARRANGEMENTS = 5 };

__device__ __forceinline__ void fold(v16f& acc, const v16i& sums, float scale) {
#pragma unroll
	for (int e = 0; e < 16; ++e) {
		acc[e] = fmaf(static_cast<float>(sums[e]), scale, acc[e]);
	}
}
__device__ __forceinline__ v16i block_sums(v4i& a, const v4i& b, const v16i& c) {
	asm volatile("" : "+v"(a)); // a fresh operand each time: the compiler may not merge or hoist the MFMAs
	return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
}

template<int MODE> __global__ void probe(float* out, long long* cycles, int iterations) {
	v4i a = { static_cast<int>(threadIdx.x), 2, 3, 4 }, b = { 1, 1, static_cast<int>(threadIdx.x), 1 };
	const v16i zero = { 0 };
	v16i r[4]	   = { zero, zero, zero, zero };
	v16f f[2]	   = { { 0 }, { 0 } };
	v16i k[2];
	for (int e = 0; e < 16; ++e) {
		k[0][e] = threadIdx.x + e;
		k[1][e] = threadIdx.x * 3 + e;
	}
	const float scale = 1.0f + threadIdx.x * 1e-3f;
	__syncthreads();
	const long long t0 = clock64();
	for (int it = 0; it < iterations; ++it) {
		if constexpr (MODE == MATRIX_ONLY) {
#pragma unroll
			for (int q = 0; q < 4; ++q) {
				r[q] = block_sums(a, b, r[q]);
			}
		} else if constexpr (MODE == VALU_ONLY) {
#pragma unroll
			for (int q = 0; q < 4; ++q) {
				asm volatile("" : "+v"(k[q & 1]));
				fold(f[q & 1], k[q & 1], scale);
			}
		} else if constexpr (MODE == BOTH_INDEPENDENT) {
#pragma unroll
			for (int q = 0; q < 4; ++q) {
				r[q] = block_sums(a, b, r[q]);
				__builtin_amdgcn_sched_barrier(0);
				asm volatile("" : "+v"(k[0]));
				fold(f[0], k[0], scale);
				__builtin_amdgcn_sched_barrier(0);
			}
		} else if constexpr (MODE == BOTH_FOLD_PREVIOUS) {
#pragma unroll
			for (int q = 0; q < 4; ++q) {
				r[q & 1] = block_sums(a, b, zero);
				__builtin_amdgcn_sched_barrier(0);
				fold(f[q & 1], r[(q + 1) & 1], scale); // the result of the MFMA before this one
				__builtin_amdgcn_sched_barrier(0);
			}
		} else {
#pragma unroll
			for (int q = 0; q < 4; ++q) {
				r[0] = block_sums(a, b, zero);
				__builtin_amdgcn_sched_barrier(0);
				fold(f[0], r[0], scale);
				__builtin_amdgcn_sched_barrier(0);
			}
		}
	}
	const long long t1 = clock64();
	float s			   = 0;
	for (int e = 0; e < 16; ++e) {
		s += f[0][e] + f[1][e] + r[0][e] + r[1][e] + r[2][e] + r[3][e];
	}
	out[threadIdx.x] = s;
	if ((threadIdx.x & 63) == 0) {
		cycles[threadIdx.x >> 6] = t1 - t0;
	}
}

static int run(int mode, int threads, float* out, long long* cyc, int iterations) {
	switch (mode) {
		case MATRIX_ONLY:
			probe<MATRIX_ONLY><<<1, threads>>>(out, cyc, iterations);
			break;
		case VALU_ONLY:
			probe<VALU_ONLY><<<1, threads>>>(out, cyc, iterations);
			break;
		case BOTH_INDEPENDENT:
			probe<BOTH_INDEPENDENT><<<1, threads>>>(out, cyc, iterations);
			break;
		case BOTH_FOLD_PREVIOUS:
			probe<BOTH_FOLD_PREVIOUS><<<1, threads>>>(out, cyc, iterations);
			break;
		default:
			probe<BOTH_FOLD_CURRENT><<<1, threads>>>(out, cyc, iterations);
			break;
	}
	CK(hipGetLastError());
	CK(hipDeviceSynchronize());
	return 0;
}

int main() {
	float* out	   = nullptr;
	long long* cyc = nullptr;
	CK(hipMalloc(&out, 1024 * 4));
	CK(hipMalloc(&cyc, 16 * 8));
	const int iterations = 20000;
	const char* names[ARRANGEMENTS] = { "matrix_only", "valu_only", "both_valu_independent", "both_fold_previous_result", "both_fold_current_result" };
	double simd_clocks[3][ARRANGEMENTS];
	for (int wi = 0; wi < 3; ++wi) {
		const int waves_per_simd = 1 << wi;
		const int threads		 = 256 * waves_per_simd;
		for (int mode = 0; mode < ARRANGEMENTS; ++mode) {
			long long h[16] = { 0 };
			for (int rep = 0; rep < 2; ++rep) { // the second run is the one read
				if (run(mode, threads, out, cyc, iterations)) {
					return 1;
				}
			}
			CK(hipMemcpy(h, cyc, sizeof(long long) * 4 * waves_per_simd, hipMemcpyDeviceToHost));
			long long slowest = 0;
			for (int w = 0; w < 4 * waves_per_simd; ++w) {
				slowest = h[w] > slowest ? h[w] : slowest;
			}
			simd_clocks[wi][mode] = static_cast<double>(slowest) / iterations / waves_per_simd;
		}
	}
	std::printf("{\"per_wave_iteration\": {\"int8_mfma_32x32x32\": 4, \"valu_instructions\": 128}, \"iterations\": %d, \"simd_clocks_per_wave_iteration\": {", iterations);
	for (int mode = 0; mode < ARRANGEMENTS; ++mode) {
		std::printf("%s\"%s\": [%.1f, %.1f, %.1f]", mode ? ", " : "", names[mode], simd_clocks[0][mode], simd_clocks[1][mode], simd_clocks[2][mode]);
	}
	const double m = simd_clocks[2][MATRIX_ONLY], v = simd_clocks[2][VALU_ONLY], both = simd_clocks[2][BOTH_FOLD_CURRENT];
	std::printf("}, \"waves_per_simd\": [1, 2, 4], \"clocks_per_mfma\": %.2f, \"clocks_per_valu_instruction\": %.3f, \"at_four_waves\": {\"if_overlapped\": %.1f, \"if_added\": %.1f, "
				"\"measured\": %.1f, \"fraction_of_sum\": %.3f}}\n",
		m / 4, v / 128, m > v ? m : v, m + v, both, both / (m + v));
	return 0;
}
