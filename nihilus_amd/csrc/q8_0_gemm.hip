// Prefill mat-mat C[m][n] = dot(W row n, Aq row m) for Q8_0 operands, gfx950, int8 MFMA.
//
// Same arithmetic as the mat-vec (reference vec_dot_q8_0_q8_0, cpu/avx_2.hpp:4534-4747) for M activation
// rows; output is [M][N] with n fastest (reference cpu/avx_2.hpp:4934; dims [ne0 = N, ne1 = M],
// common/kernel_traits.hpp:393-417).
//
// One v_mfma_i32_32x32x32_i8 covers exactly one 32-quant block of 32 activation rows x 32 weight rows, so its
// int32 result is the exact per-block sum for 1024 (m, n) pairs.  Because both operands carry a scale per
// block, the accumulator cannot run across blocks: every MFMA result is converted and folded into an fp32
// accumulator with the factor f32(dA[m][b]) * f32(dW[n][b]) (exact in fp32: two 11-bit significands).
//
// Operand lanes: lane l supplies row (l % 32), quants 16*(l/32)..+15 of the block -- the tiled layout stores
// tiles in exactly that order, so operands go from memory to the MFMA with one 16-byte load per lane and no
// shuffle.  Result lanes: register i of lane l is C[m = 8*(i/4) + 4*(l/32) + i%4][n = l % 32].
#include "q8_0_device.h"

namespace nh {

constexpr int GEMM_WAVES_M = 2; // waves along M in a workgroup
constexpr int GEMM_WAVES_N = 2; // waves along N
constexpr int GEMM_TM	   = 2; // 32-row MFMA tiles per wave along M
constexpr int GEMM_TN	   = 2; // along N
constexpr int GEMM_BM	   = GEMM_WAVES_M * GEMM_TM * 32; // 128
constexpr int GEMM_BN	   = GEMM_WAVES_N * GEMM_TN * 32; // 128
constexpr int GEMM_THREADS = GEMM_WAVES_M * GEMM_WAVES_N * 64;

// 16 operand bytes for (row strip, block b): lane supplies row strip*32 + lane%32, half lane/32.
template<bool TILED> __device__ __forceinline__ v4i load_operand(const uint8_t* base, int rows, int nb, int strip, int b, int lane) {
	if constexpr (TILED) {
		return *reinterpret_cast<const v4i*>(base + macro_offset(strip, b / GROUP_BLOCKS, nb / GROUP_BLOCKS) + (b % GROUP_BLOCKS) * TILE_BYTES + 16 * lane);
	} else {
		const int row = min(strip * STRIP_ROWS + (lane & 31), rows - 1); // padding rows re-read the last row; dropped at the store
		return load16_unaligned(base + (static_cast<int64_t>(row) * nb + b) * BLOCK_BYTES + 2 + 16 * (lane >> 5));
	}
}
template<bool TILED> __device__ __forceinline__ float load_scale(const uint8_t* base, int rows, int nb, int row, int b) {
	if constexpr (TILED) {
		return half_bits_to_float(load_u16(base + macro_offset(row / STRIP_ROWS, b / GROUP_BLOCKS, nb / GROUP_BLOCKS) + MACRO_D_OFFSET + 8 * (row % STRIP_ROWS) + 2 * (b % GROUP_BLOCKS)));
	} else {
		return half_bits_to_float(load_u16(base + (static_cast<int64_t>(min(row, rows - 1)) * nb + b) * BLOCK_BYTES));
	}
}

template<bool TILED, bool DUMP>
__global__ __launch_bounds__(GEMM_THREADS) void gemm_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ A, float* __restrict__ C, int32_t* __restrict__ sums, int M, int N, int K) {
	__shared__ float a_scale[GROUP_BLOCKS][GEMM_BM]; // f32(dA) for this workgroup's rows, current 4 blocks
	__shared__ float w_scale[GROUP_BLOCKS][GEMM_BN];

	const int nb	   = K / QK;
	const int m_strips = (M + 31) / 32;
	const int n_strips = (N + 31) / 32;
	const int tid	   = threadIdx.x;
	const int lane	   = tid & 63;
	const int wave	   = tid >> 6;
	const int wm	   = wave / GEMM_WAVES_N;
	const int wn	   = wave % GEMM_WAVES_N;
	const int half	   = lane >> 5;
	const int m0	   = blockIdx.y * GEMM_BM; // first activation row of the workgroup
	const int n0	   = blockIdx.x * GEMM_BN;

	float acc[GEMM_TM][GEMM_TN][16];
#pragma unroll
	for (int i = 0; i < GEMM_TM; ++i) {
#pragma unroll
		for (int j = 0; j < GEMM_TN; ++j) {
#pragma unroll
			for (int e = 0; e < 16; ++e) {
				acc[i][j][e] = 0.0f;
			}
		}
	}

	for (int b0 = 0; b0 < nb; b0 += GROUP_BLOCKS) {
		// ---- scales of the next four blocks for all rows of the workgroup tile, as fp32, via LDS ----
		__syncthreads();
		for (int i = tid; i < GROUP_BLOCKS * GEMM_BM; i += GEMM_THREADS) {
			const int t = i / GEMM_BM, rr = i % GEMM_BM;
			const int b = b0 + t, row = m0 + rr;
			a_scale[t][rr] = (b < nb && row < m_strips * 32 && (TILED || row < M)) ? load_scale<TILED>(A, M, nb, row, b) : 0.0f;
		}
		for (int i = tid; i < GROUP_BLOCKS * GEMM_BN; i += GEMM_THREADS) {
			const int t = i / GEMM_BN, rr = i % GEMM_BN;
			const int b = b0 + t, row = n0 + rr;
			w_scale[t][rr] = (b < nb && row < n_strips * 32 && (TILED || row < N)) ? load_scale<TILED>(W, N, nb, row, b) : 0.0f;
		}
		__syncthreads();

#pragma unroll
		for (int t = 0; t < GROUP_BLOCKS; ++t) {
			const int b = b0 + t;
			if (b >= nb) {
				break;
			}
			v4i a[GEMM_TM], w[GEMM_TN];
#pragma unroll
			for (int i = 0; i < GEMM_TM; ++i) {
				const int strip = m0 / 32 + wm * GEMM_TM + i;
				a[i]			= strip < m_strips ? load_operand<TILED>(A, M, nb, strip, b, lane) : v4i{ 0, 0, 0, 0 };
			}
#pragma unroll
			for (int j = 0; j < GEMM_TN; ++j) {
				const int strip = n0 / 32 + wn * GEMM_TN + j;
				w[j]			= strip < n_strips ? load_operand<TILED>(W, N, nb, strip, b, lane) : v4i{ 0, 0, 0, 0 };
			}
#pragma unroll
			for (int i = 0; i < GEMM_TM; ++i) {
#pragma unroll
				for (int j = 0; j < GEMM_TN; ++j) {
					const v16i zero = { 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 };
					const v16i s	= __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], w[j], zero, 0, 0, 0);
					const int ml	= (wm * GEMM_TM + i) * 32; // tile's first row inside the workgroup tile
					const int nl	= (wn * GEMM_TN + j) * 32 + (lane & 31);
					const float dw	= w_scale[t][nl];
#pragma unroll
					for (int e = 0; e < 16; ++e) {
						const int mr = ml + 8 * (e >> 2) + 4 * half + (e & 3);
						if constexpr (DUMP) {
							const int m = m0 + mr, n = n0 + nl;
							if (m < M && n < N) {
								sums[(static_cast<int64_t>(m) * N + n) * nb + b] = s[e];
							}
						} else {
							acc[i][j][e] = fmaf(static_cast<float>(s[e]), a_scale[t][mr] * dw, acc[i][j][e]);
						}
					}
				}
			}
		}
	}

	if constexpr (!DUMP) {
#pragma unroll
		for (int i = 0; i < GEMM_TM; ++i) {
#pragma unroll
			for (int j = 0; j < GEMM_TN; ++j) {
				const int n = n0 + (wn * GEMM_TN + j) * 32 + (lane & 31);
#pragma unroll
				for (int e = 0; e < 16; ++e) {
					const int m = m0 + (wm * GEMM_TM + i) * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
					if (m < M && n < N) {
						C[static_cast<int64_t>(m) * N + n] = acc[i][j][e];
					}
				}
			}
		}
	}
}

__global__ void zero_c_kernel(float* __restrict__ c, int64_t n) {
	const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
	if (i < n) {
		c[i] = 0.0f;
	}
}

hipError_t launch_gemm(const void* W, const void* Aq, float* C, int32_t* sums, int64_t M, int64_t N, int64_t K, bool tiled, hipStream_t s) {
	if (M == 0 || N == 0) {
		return hipSuccess;
	}
	if (K == 0) {
		if (!sums) {
			zero_c_kernel<<<dim3(static_cast<unsigned>((M * N + 255) / 256)), dim3(256), 0, s>>>(C, M * N);
		}
		return hipGetLastError();
	}
	const dim3 grid(static_cast<unsigned>((N + GEMM_BN - 1) / GEMM_BN), static_cast<unsigned>((M + GEMM_BM - 1) / GEMM_BM));
	const uint8_t* w = static_cast<const uint8_t*>(W);
	const uint8_t* a = static_cast<const uint8_t*>(Aq);
	const int m = static_cast<int>(M), n = static_cast<int>(N), k = static_cast<int>(K);
	if (tiled) {
		if (sums) {
			gemm_kernel<true, true><<<grid, dim3(GEMM_THREADS), 0, s>>>(w, a, C, sums, m, n, k);
		} else {
			return launch_kernel(KIND_GEMM, gemm_kernel<true, false>, grid, dim3(GEMM_THREADS), 0, s, w, a, C, sums, m, n, k);
		}
	} else {
		if (sums) {
			gemm_kernel<false, true><<<grid, dim3(GEMM_THREADS), 0, s>>>(w, a, C, sums, m, n, k);
		} else {
			return launch_kernel(KIND_GEMM, gemm_kernel<false, false>, grid, dim3(GEMM_THREADS), 0, s, w, a, C, sums, m, n, k);
		}
	}
	return hipGetLastError();
}

} // namespace nh
