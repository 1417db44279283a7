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

// ---------------------------------------------------------------------------------------------------------
// The prefill kernel for the tiled layout.
//
// Both operands carry a scale per 32-quant block, so each 32x32x32 int8 MFMA result (1024 exact block sums, 16 per
// lane) has to be converted and folded into the fp32 accumulator before the next block: 16 conversions + 16
// multiply-adds per lane per MFMA.  Measured on this part, a SIMD retires one wave64 VALU instruction per ~2.4 cycles
// once it holds two or more waves (a lone wave issues one per ~5), and MFMA and VALU work does not overlap: a
// (tile, block) costs 32 + 32 matrix-pipe cycles plus 32 x 2.4 VALU cycles, ~141 cycles against the 32 of the int8
// MFMA alone.  That is the ceiling (~22 % of the int8 MFMA peak); the kernel is shaped to add as little as possible:
//   * the scale products f32(dA[m][b]) * f32(dW[n][b]) are formed on the matrix pipe: one v_mfma_f32_32x32x8_f16 whose
//     operands are the two blocks' fp16 scales as stored, each in the k = 0 slot ({d, 0, 0, 0}; lanes 32..63 supply
//     the k = 4..7 slots = 0).  The product of two fp16 values is exact in fp32 (fp16 subnormals included) and lands
//     in the int8 MFMA's own accumulator layout: no conversion, broadcast or cross-lane move of a scale, ever;
//   * only the operand that is shared goes through LDS.  A workgroup is four waves; wave w owns weight strip
//     4*blockIdx.x + w and loads its tiles straight from global memory into registers (one coalesced 16-byte-per-lane
//     load per tile, already an MFMA operand, a whole 128-quant group ahead of use); all four waves share the same
//     TM activation strips, copied global -> LDS one group ahead (double-buffered, one barrier per group, the copy
//     spread over the four waves) and read back as conflict-free 16-byte-per-lane operand images plus one half-word
//     read per scale;
//   * latency is hidden by occupancy, not by a software pipeline: one result-register set per tile keeps the kernel
//     at <= 128 VGPRs, four workgroups per CU, four waves per SIMD.  (A two-result-set, software-pipelined variant
//     at two waves per SIMD measured 8 % slower: with so few waves the SIMD falls back to the lone-wave issue rate
//     whenever one of them waits.)
template<int TM, bool DUMP, int KS = 1>
__global__ __launch_bounds__(256 * KS, 4) void gemm_tiled_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ A, float* C, const float* R, int32_t* __restrict__ sums, int M, int N,
	int groups) {
	constexpr int DATA_BYTES  = TM * MACRO_BYTES;
	constexpr int STAGE_BYTES = DATA_BYTES + 16;
	// KS > 1: the workgroup holds KS sets of four waves; set kr walks groups [kr * groups / KS, (kr + 1) * groups / KS) with its
	// own activation stages, and the sets' results are added to the first's through LDS at the end (set order, fixed).  A
	// grid too small to give every SIMD its four waves gets them this way without a second pass over memory.
	__shared__ __align__(16) uint8_t lds_all[KS][2 * STAGE_BYTES];
	__shared__ float red[KS > 1 ? 4 * TM * 16 * 64 : 1];
	typedef _Float16 v4h __attribute__((ext_vector_type(4)));
	typedef float v16f __attribute__((ext_vector_type(16)));

	const int tid	   = threadIdx.x;
	const int lane	   = tid & 63;
	const int wave_all = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int wave	   = wave_all & 3; // which of the workgroup's four weight strips
	const int kr	   = wave_all >> 2; // which K range
	uint8_t* lds	   = lds_all[kr];
	const int g_len	   = groups / KS; // the host launches KS > 1 only when it divides
	const int g_base   = kr * g_len;
	const int half	   = lane >> 5;
	const int m_strips = (M + 31) / 32;
	const int n_strips = (N + 31) / 32;
	const int ms0	   = blockIdx.y * TM;
	const int ns	   = blockIdx.x * 4 + wave;
	if ((tid & 255) < 8) {
		*reinterpret_cast<uint32_t*>(lds + ((tid & 255) >> 2) * STAGE_BYTES + DATA_BYTES + 4 * (tid & 3)) = 0u;
	}
	const uint8_t* w_src = W + macro_offset(min(ns, n_strips - 1), g_base, groups);
	struct w_regs {
		v4i q[GROUP_BLOCKS];
		v2u d;
	};
	auto fetch_w = [&](int g, w_regs& r) {
		const uint8_t* p = w_src + static_cast<int64_t>(g) * MACRO_BYTES;
#pragma unroll
		for (int k = 0; k < GROUP_BLOCKS; ++k) {
			r.q[k] = *reinterpret_cast<const v4i*>(p + k * TILE_BYTES + 16 * lane);
		}
		r.d = *reinterpret_cast<const v2u*>(p + MACRO_D_OFFSET + 8 * (lane & 31));
	};
	// activations: global -> registers -> LDS, shared out over the four waves: wave w moves tiles TM*w .. TM*w+TM-1 of the
	// TM*4 tiles of a group, waves 0..TM-1 also the 256-byte scale table of strip w
	const uint8_t* a_src[TM];
	int a_dst[TM];
#pragma unroll
	for (int j = 0; j < TM; ++j) {
		const int u = TM * wave + j;
		a_src[j]	= A + macro_offset(min(ms0 + u / 4, m_strips - 1), g_base, groups) + (u % 4) * TILE_BYTES + 16 * lane;
		a_dst[j]	= (u / 4) * MACRO_BYTES + (u % 4) * TILE_BYTES + 16 * lane;
	}
	const bool sc_copier   = wave < TM;
	const uint8_t* sc_src = A + macro_offset(min(ms0 + min(wave, TM - 1), m_strips - 1), g_base, groups) + MACRO_D_OFFSET + 4 * lane;
	const int sc_dst	   = min(wave, TM - 1) * MACRO_BYTES + MACRO_D_OFFSET + 4 * lane;
	struct a_regs {
		v4i q[TM];
		uint32_t d;
	};
	auto fetch_a = [&](int g, a_regs& r) {
#pragma unroll
		for (int j = 0; j < TM; ++j) {
			r.q[j] = *reinterpret_cast<const v4i*>(a_src[j] + static_cast<int64_t>(g) * MACRO_BYTES);
		}
		if (sc_copier) {
			r.d = *reinterpret_cast<const uint32_t*>(sc_src + static_cast<int64_t>(g) * MACRO_BYTES);
		}
	};
	auto stash_a = [&](int stage, const a_regs& r) {
		uint8_t* p = lds + stage * STAGE_BYTES;
#pragma unroll
		for (int j = 0; j < TM; ++j) {
			*reinterpret_cast<v4i*>(p + a_dst[j]) = r.q[j];
		}
		if (sc_copier) {
			*reinterpret_cast<uint32_t*>(p + sc_dst) = r.d;
		}
	};
	v16f acc[TM];
#pragma unroll
	for (int i = 0; i < TM; ++i) {
		acc[i] = v16f{ 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 };
	}
	const int a_sc_rel = half ? DATA_BYTES : MACRO_D_OFFSET + 8 * (lane & 31);

	w_regs wa, wb;
	a_regs pre;
	fetch_w(0, wa);
	fetch_a(0, pre);
	stash_a(0, pre);
	__syncthreads();
	auto trip = [&](int g, w_regs& cur, w_regs& nxt) {
		const bool more = g + 1 < g_len;
		if (more) {
			fetch_w(g + 1, nxt);
			fetch_a(g + 1, pre);
		}
		if (half) {
			cur.d = v2u{ 0u, 0u };
		}
		const uint8_t* stage = lds + (g & 1) * STAGE_BYTES;
#pragma unroll
		for (int t = 0; t < GROUP_BLOCKS; ++t) {
			const uint32_t wd = (t < 2) ? cur.d.x : cur.d.y;
			const v2u w_sc	  = v2u{ (t & 1) ? (wd >> 16) : (wd & 0xFFFFu), 0u };
#pragma unroll
			for (int i = 0; i < TM; ++i) {
				asm volatile("" ::: "memory");
				const v4i a		= *reinterpret_cast<const v4i*>(stage + i * MACRO_BYTES + t * TILE_BYTES + 16 * lane);
				const v2u a_sc	= v2u{ *reinterpret_cast<const uint16_t*>(stage + (half ? 0 : i * MACRO_BYTES) + a_sc_rel + 2 * t), 0u };
				const v16i zi	= { 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 };
				const v16f zf	= { 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 };
				const v16i sv	= __builtin_amdgcn_mfma_i32_32x32x32_i8(a, cur.q[t], zi, 0, 0, 0);
				if constexpr (DUMP) {
					const int n = ns * 32 + (lane & 31);
#pragma unroll
					for (int e = 0; e < 16; ++e) {
						const int m = (ms0 + i) * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
						if (m < M && n < N) {
							sums[(static_cast<int64_t>(m) * N + n) * (groups * GROUP_BLOCKS) + (g_base + g) * GROUP_BLOCKS + t] = sv[e];
						}
					}
				} else {
					const v16f pv = __builtin_amdgcn_mfma_f32_32x32x8f16(__builtin_bit_cast(v4h, a_sc), __builtin_bit_cast(v4h, w_sc), zf, 0, 0, 0);
#pragma unroll
					for (int e = 0; e < 16; ++e) {
						acc[i][e] = fmaf(static_cast<float>(sv[e]), pv[e], acc[i][e]);
					}
					asm volatile("" : "+v"(acc[i]));
				}
			}
		}
		if (more) {
			stash_a((g + 1) & 1, pre);
		}
		__syncthreads();
	};
	for (int g = 0; g < g_len; g += 2) {
		trip(g, wa, wb);
		if (g + 1 < g_len) {
			trip(g + 1, wb, wa);
		}
	}
	if constexpr (KS > 1 && !DUMP) {
		// sets 1 .. KS-1 park their tiles one after the other in the same LDS buffer, set 0 adds them (set order, fixed)
		float* slot = red + wave * (TM * 16 * 64);
#pragma unroll
		for (int k = 1; k < KS; ++k) {
			if (kr == k) {
#pragma unroll
				for (int i = 0; i < TM; ++i) {
#pragma unroll
					for (int e = 0; e < 16; ++e) {
						slot[(i * 16 + e) * 64 + lane] = acc[i][e];
					}
				}
			}
			__syncthreads();
			if (kr == 0) {
#pragma unroll
				for (int i = 0; i < TM; ++i) {
#pragma unroll
					for (int e = 0; e < 16; ++e) {
						acc[i][e] += slot[(i * 16 + e) * 64 + lane];
					}
				}
			}
			if (k + 1 < KS) {
				__syncthreads();
			}
		}
		if (kr > 0) {
			return;
		}
	}
	if constexpr (!DUMP) {
		const int n = ns * 32 + (lane & 31);
#pragma unroll
		for (int i = 0; i < TM; ++i) {
#pragma unroll
			for (int e = 0; e < 16; ++e) {
				const int m = (ms0 + i) * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
				if (m < M && n < N) {
					const int64_t at = static_cast<int64_t>(m) * N + n;
					C[at]			 = R ? acc[i][e] + R[at] : acc[i][e]; // R may be C: read before the write, by the same thread
				}
			}
		}
	}
}

template<int TM> static hipError_t launch_gemm_tiled_t(const uint8_t* w, const uint8_t* a, float* C, const float* R, int32_t* sums, int m, int n, int k, hipStream_t s) {
	const int groups   = k / GROUP_K;
	const int m_strips = (m + 31) / 32, n_strips = (n + 31) / 32;
	const dim3 grid(static_cast<unsigned>((n_strips + 3) / 4), static_cast<unsigned>((m_strips + TM - 1) / TM));
	if (sums) {
		gemm_tiled_kernel<TM, true><<<grid, dim3(256), 0, s>>>(w, a, C, R, sums, m, n, groups);
		return hipGetLastError();
	}
	// a grid that leaves SIMDs short of their four waves: K sets inside the workgroup (8 or 16 waves) make up for it
	int ks = 1;
	while (ks < 4 && static_cast<int64_t>(grid.x) * grid.y * 4 * ks * 2 <= 4096 && groups % (ks * 2) == 0 && groups / (ks * 2) >= 4) {
		ks *= 2;
	}
	if (ks == 4) {
		return launch_kernel(KIND_GEMM, gemm_tiled_kernel<TM, false, 4>, grid, dim3(1024), 0, s, w, a, C, R, sums, m, n, groups);
	}
	if (ks == 2) {
		return launch_kernel(KIND_GEMM, gemm_tiled_kernel<TM, false, 2>, grid, dim3(512), 0, s, w, a, C, R, sums, m, n, groups);
	}
	return launch_kernel(KIND_GEMM, gemm_tiled_kernel<TM, false>, grid, dim3(256), 0, s, w, a, C, R, sums, m, n, groups);
}

// Tile choice.  One wave alone issues a VALU instruction only every ~5 cycles (two or more per SIMD reach ~2.4), so
// the grid must give every SIMD at least two waves: 64-row workgroup tiles (half the LDS and L2 traffic per MFMA) when
// that still leaves >= 512 workgroups, 32-row tiles otherwise.
static hipError_t launch_gemm_tiled(const uint8_t* w, const uint8_t* a, float* C, const float* R, int32_t* sums, int m, int n, int k, hipStream_t s) {
	const int64_t ms = (m + 31) / 32;
	// Two activation strips per wave whenever there are two: every weight tile fetched is used twice, which halves what a CU
	// has to take in per MFMA (that intake, not the MFMA rate, bounds the one-strip form); the K sets below give back the
	// waves the halved grid loses.
	if (ms >= 2) {
		return launch_gemm_tiled_t<2>(w, a, C, R, sums, m, n, k, s);
	}
	return launch_gemm_tiled_t<1>(w, a, C, R, sums, m, n, k, s);
}

__global__ void zero_c_kernel(float* c, const float* src, int64_t n) {
	const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
	if (i < n) {
		c[i] = src ? src[i] : 0.0f;
	}
}

hipError_t launch_gemm(const void* W, const void* Aq, float* C, int32_t* sums, int64_t M, int64_t N, int64_t K, bool tiled, hipStream_t s, const float* residual) {
	if (M == 0 || N == 0) {
		return hipSuccess;
	}
	if (K == 0) { // empty dot products: C = residual, or 0
		if (!sums) {
			zero_c_kernel<<<dim3(static_cast<unsigned>((M * N + 255) / 256)), dim3(256), 0, s>>>(C, residual, M * N);
		}
		return hipGetLastError();
	}
	const dim3 grid(static_cast<unsigned>((N + GEMM_BN - 1) / GEMM_BN), static_cast<unsigned>((M + GEMM_BM - 1) / GEMM_BM));
	const uint8_t* w = static_cast<const uint8_t*>(W);
	const uint8_t* a = static_cast<const uint8_t*>(Aq);
	const int m = static_cast<int>(M), n = static_cast<int>(N), k = static_cast<int>(K);
	if (tiled) {
		// Few rows: the weights are read once and the kernel is HBM-bound.  Somewhat more rows than that, but so few
		// 128-row x 32-row tiles that the tile kernel would leave most SIMDs with one wave or none (measured: it needs
		// more than one workgroup per CU to pay): the same streaming kernel over groups of 64 rows, K split over the
		// waves of a workgroup, the weights coming from cache after the first group.
		const int64_t tile_workgroups = ((N + 127) / 128) * ((M + 31) / 32);
		if (M <= GEMM_SKINNY_MAX_M || tile_workgroups <= 256) {
			return launch_gemm_skinny(W, Aq, C, sums, M, N, K, s, residual);
		}
		return launch_gemm_tiled(w, a, C, residual, sums, m, n, k, s);
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
