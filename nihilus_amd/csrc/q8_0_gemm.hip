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
#include <type_traits>

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
// lane) has to be converted and folded into the fp32 accumulator before the next block.  That makes the kernel
// VALU-bound, not MFMA-bound: 16 conversions + 16 multiply-adds per lane per MFMA is 128 VALU cycles against 32
// MFMA cycles on the same SIMD, so the design goal is to spend NOTHING else on the VALU:
//   * the scale products f32(dA[m][b]) * f32(dW[n][b]) are formed on the matrix pipe too: one v_mfma_f32_32x32x8_f16
//     whose A operand is the lane's four fp16 block scales as stored (row l%32, k = block within the group) and whose
//     B operand is the weight row's four scales with all but block b masked off.  The product of two fp16 values is
//     exact in fp32 (fp16 subnormals included), and it lands in the int8 MFMA's own accumulator layout, so the scales
//     never need a conversion, a broadcast or a cross-lane move;
//   * operands reach the waves through LDS: a workgroup copies whole 4352-byte macro-tiles (four blocks of 32 rows
//     plus their scales) global -> registers -> LDS, double-buffered, one barrier per 128-quant group; waves read
//     their 32x32 tiles back as conflict-free 16-byte-per-lane reads that already are MFMA operands.
// Workgroup = 4 waves in a 2 x 2 arrangement, each wave TM x TN tiles of 32 x 32.
template<int TM, int TN, bool DUMP>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ A, float* __restrict__ C, int32_t* __restrict__ sums, int M, int N,
	int groups) {
	constexpr int SA		  = 2 * TM; // A strips per workgroup
	constexpr int SW		  = 2 * TN; // W strips per workgroup
	constexpr int STRIPS	  = SA + SW;
	constexpr int DATA_BYTES  = STRIPS * MACRO_BYTES;
	constexpr int STAGE_BYTES = DATA_BYTES + 16; // + 16 zero bytes: what lanes 32..63 feed the scale MFMA (k = 4..7)
	extern __shared__ __align__(16) uint8_t lds[]; // [2][STAGE_BYTES]
	if (threadIdx.x < 8) {
		*reinterpret_cast<uint32_t*>(lds + (threadIdx.x >> 2) * STAGE_BYTES + DATA_BYTES + 4 * (threadIdx.x & 3)) = 0u; // made visible by the first barrier below
	}

	typedef _Float16 v4h __attribute__((ext_vector_type(4)));
	typedef float v16f __attribute__((ext_vector_type(16)));

	const int tid	   = threadIdx.x;
	const int lane	   = tid & 63;
	const int wave	   = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int wm	   = wave >> 1;
	const int wn	   = wave & 1;
	const int half	   = lane >> 5;
	const int m_strips = (M + 31) / 32;
	const int n_strips = (N + 31) / 32;
	const int ms0	   = blockIdx.y * SA; // first A strip of the workgroup
	const int ns0	   = blockIdx.x * SW;

	// Global -> LDS copy: whole macro-tiles, one per wave at a time (wave w moves strips w, w+4, ...).  4352 bytes are
	// 64 lanes x (4 x 16 B + 4 B): every lane is live in every load, so the copy needs no predicate and no zero fill.
	// Strips past the matrix edge are clamped to the last real one: their products are computed and never stored.
	constexpr int COPIES = (STRIPS + 3) / 4;
	const uint8_t* src[COPIES];
#pragma unroll
	for (int c = 0; c < COPIES; ++c) {
		const int strip = min(wave + 4 * c, STRIPS - 1); // the last round may repeat a strip: same bytes, same place
		const uint8_t* base;
		if (strip < SA) {
			base = A + macro_offset(min(ms0 + strip, m_strips - 1), 0, groups);
		} else {
			base = W + macro_offset(min(ns0 + strip - SA, n_strips - 1), 0, groups);
		}
		src[c] = base;
	}
	struct copy_regs {
		v4i q[COPIES][4];
		uint32_t d[COPIES];
	};
	auto fetch = [&](int g, copy_regs& r) {
#pragma unroll
		for (int c = 0; c < COPIES; ++c) {
			const uint8_t* p = src[c] + static_cast<int64_t>(g) * MACRO_BYTES;
#pragma unroll
			for (int k = 0; k < 4; ++k) {
				r.q[c][k] = *reinterpret_cast<const v4i*>(p + k * TILE_BYTES + 16 * lane);
			}
			r.d[c] = *reinterpret_cast<const uint32_t*>(p + MACRO_D_OFFSET + 4 * lane);
		}
	};
	auto stash = [&](int stage, const copy_regs& r) {
#pragma unroll
		for (int c = 0; c < COPIES; ++c) {
			uint8_t* p = lds + stage * STAGE_BYTES + min(wave + 4 * c, STRIPS - 1) * MACRO_BYTES;
#pragma unroll
			for (int k = 0; k < 4; ++k) {
				*reinterpret_cast<v4i*>(p + k * TILE_BYTES + 16 * lane) = r.q[c][k];
			}
			*reinterpret_cast<uint32_t*>(p + MACRO_D_OFFSET + 4 * lane) = r.d[c];
		}
	};

	v16f acc[TM][TN];
#pragma unroll
	for (int i = 0; i < TM; ++i) {
#pragma unroll
		for (int j = 0; j < TN; ++j) {
			acc[i][j] = v16f{ 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 };
		}
	}

	// One block's worth of matrix-pipe work for this wave: TM*TN int8 MFMAs (block sums) and as many f16 MFMAs (scale
	// products), results in sv / pv.  Everything an MFMA needs comes out of LDS in its final form, so this half costs
	// the VALU nothing: the quants as 16-byte operand images, the scales as single zero-extended half-word reads
	// ({d, 0, 0, 0} in the k = 0..3 slots; lanes 32..63, the k = 4..7 slots, read the stage's zero bytes instead).
	// The compiler fence pins the LDS reads -- and with them the MFMAs that depend on them -- behind the previous
	// pipeline step; without it every MFMA of a group is hoisted to the front and the result registers overflow.
	const int sc_rel = half ? DATA_BYTES : MACRO_D_OFFSET + 8 * (lane & 31); // + strip*MACRO_BYTES for live lanes, see below
	auto issue = [&](const uint8_t* stage, auto t_const, v16i(&sv)[TM][TN], v16f(&pv)[TM][TN]) {
		constexpr int t = decltype(t_const)::value;
		asm volatile("" ::: "memory");
		v4i a[TM], w[TN];
		v2u a_sc[TM], w_sc[TN];
#pragma unroll
		for (int i = 0; i < TM; ++i) {
			const int strip = wm * TM + i;
			a[i]			= *reinterpret_cast<const v4i*>(stage + strip * MACRO_BYTES + t * TILE_BYTES + 16 * lane);
			a_sc[i]			= v2u{ *reinterpret_cast<const uint16_t*>(stage + (half ? 0 : strip * MACRO_BYTES) + sc_rel + 2 * t), 0u };
		}
#pragma unroll
		for (int j = 0; j < TN; ++j) {
			const int strip = SA + wn * TN + j;
			w[j]			= *reinterpret_cast<const v4i*>(stage + strip * MACRO_BYTES + t * TILE_BYTES + 16 * lane);
			w_sc[j]			= v2u{ *reinterpret_cast<const uint16_t*>(stage + (half ? 0 : strip * MACRO_BYTES) + sc_rel + 2 * t), 0u };
		}
#pragma unroll
		for (int j = 0; j < TN; ++j) {
#pragma unroll
			for (int i = 0; i < TM; ++i) {
				const v16i zi = { 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 };
				const v16f zf = { 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 };
				sv[i][j]	  = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], w[j], zi, 0, 0, 0);
				if constexpr (!DUMP) {
					pv[i][j] = __builtin_amdgcn_mfma_f32_32x32x8f16(__builtin_bit_cast(v4h, a_sc[i]), __builtin_bit_cast(v4h, w_sc[j]), zf, 0, 0, 0);
				}
			}
		}
	};
	// The VALU half: convert the block sums and fold them into the accumulators with their scale products.
	auto fold = [&](int block, const v16i(&sv)[TM][TN], const v16f(&pv)[TM][TN]) {
#pragma unroll
		for (int i = 0; i < TM; ++i) {
#pragma unroll
			for (int j = 0; j < TN; ++j) {
				if constexpr (DUMP) {
					const int n = (ns0 + wn * TN + j) * 32 + (lane & 31);
#pragma unroll
					for (int e = 0; e < 16; ++e) {
						const int m = (ms0 + wm * TM + i) * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
						if (m < M && n < N) {
							sums[(static_cast<int64_t>(m) * N + n) * (groups * GROUP_BLOCKS) + block] = sv[i][j][e];
						}
					}
				} else {
#pragma unroll
					for (int e = 0; e < 16; ++e) {
						acc[i][j][e] = fmaf(static_cast<float>(sv[i][j][e]), pv[i][j][e], acc[i][j][e]);
					}
					// pins this fold in program order (no instruction is emitted): the arithmetic above has no side effect, and
					// left free it is sunk to the end of the loop, behind every MFMA of the group
					asm volatile("" : "+v"(acc[i][j]));
				}
			}
		}
	};
	using t0 = std::integral_constant<int, 0>;
	using t1 = std::integral_constant<int, 1>;
	using t2 = std::integral_constant<int, 2>;
	using t3 = std::integral_constant<int, 3>;

	copy_regs pre;
	fetch(0, pre);
	stash(0, pre);
	__syncthreads();

	// Software pipeline, one block deep: while the VALU folds block b, the matrix pipe already works on block b+1
	// (two register sets, s0/p0 and s1/p1).  The scheduling fences keep the compiler from hoisting more than that:
	// left alone it moves every MFMA of a group to the front and the result registers overflow the file.
	v16i s0[TM][TN], s1[TM][TN];
	v16f p0[TM][TN], p1[TM][TN];
	issue(lds, t0{}, s0, p0);
	__builtin_amdgcn_sched_barrier(0);
	for (int g = 0; g < groups; ++g) {
		const bool more = g + 1 < groups;
		if (more) {
			fetch(g + 1, pre); // global loads in flight across the next three folds
		}
		const uint8_t* stage = lds + (g & 1) * STAGE_BYTES;
		const int b0		 = g * GROUP_BLOCKS;
		issue(stage, t1{}, s1, p1);
		fold(b0 + 0, s0, p0);
		__builtin_amdgcn_sched_barrier(0);
		issue(stage, t2{}, s0, p0);
		fold(b0 + 1, s1, p1);
		__builtin_amdgcn_sched_barrier(0);
		issue(stage, t3{}, s1, p1);
		fold(b0 + 2, s0, p0);
		__builtin_amdgcn_sched_barrier(0);
		if (more) {
			// the other stage was last read during the previous trip, and a barrier has passed since
			stash((g + 1) & 1, pre);
		}
		__syncthreads(); // every wave is done reading this stage's tiles (all four issues are behind it) and the next stage is complete
		if (more) {
			const uint8_t* next = lds + ((g + 1) & 1) * STAGE_BYTES;
			issue(next, t0{}, s0, p0);
		}
		fold(b0 + 3, s1, p1);
		__builtin_amdgcn_sched_barrier(0);
	}

	if constexpr (!DUMP) {
#pragma unroll
		for (int i = 0; i < TM; ++i) {
#pragma unroll
			for (int j = 0; j < TN; ++j) {
				const int n = (ns0 + wn * TN + j) * 32 + (lane & 31);
#pragma unroll
				for (int e = 0; e < 16; ++e) {
					const int m = (ms0 + wm * TM + i) * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
					if (m < M && n < N) {
						C[static_cast<int64_t>(m) * N + n] = acc[i][j][e];
					}
				}
			}
		}
	}
}

template<int TM, int TN> static hipError_t launch_gemm_tiled_t(const uint8_t* w, const uint8_t* a, float* C, int32_t* sums, int m, int n, int k, hipStream_t s) {
	const int groups   = k / GROUP_K;
	const int m_strips = (m + 31) / 32, n_strips = (n + 31) / 32;
	const dim3 grid(static_cast<unsigned>((n_strips + 2 * TN - 1) / (2 * TN)), static_cast<unsigned>((m_strips + 2 * TM - 1) / (2 * TM)));
	const size_t shmem = 2 * (static_cast<size_t>(2 * TM + 2 * TN) * MACRO_BYTES + 16);
	hipError_t e	   = hipSuccess;
	if (shmem > 64 * 1024) { // more than the default dynamic-LDS limit: opt in once per kernel
		static bool raised_plain = false, raised_dump = false;
		bool& raised = sums ? raised_dump : raised_plain;
		if (!raised) {
			e = sums ? hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_tiled_kernel<TM, TN, true>), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(shmem))
					 : hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_tiled_kernel<TM, TN, false>), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(shmem));
			if (e != hipSuccess) {
				return e;
			}
			raised = true;
		}
	}
	if (sums) {
		gemm_tiled_kernel<TM, TN, true><<<grid, dim3(256), shmem, s>>>(w, a, C, sums, m, n, groups);
		return hipGetLastError();
	}
	return launch_kernel(KIND_GEMM, gemm_tiled_kernel<TM, TN, false>, grid, dim3(256), shmem, s, w, a, C, sums, m, n, groups);
}

// Tile choice.  The kernel is bound by VALU issue, and one wave alone issues a VALU instruction only every ~5 cycles
// (two or more per SIMD reach ~2.4), so occupancy matters more than operand reuse: 64 x 64 workgroup tiles (TM = TN = 1,
// ~120 VGPRs, 35 KB LDS: four workgroups per CU) measured faster than 64 x 128 at every prefill shape tried.
static hipError_t launch_gemm_tiled(const uint8_t* w, const uint8_t* a, float* C, int32_t* sums, int m, int n, int k, hipStream_t s) {
	return launch_gemm_tiled_t<1, 1>(w, a, C, sums, m, n, k, s);
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
		if (M <= GEMM_SKINNY_MAX_M) {
			return launch_gemm_skinny(W, Aq, C, sums, M, N, K, s); // few rows: weights are read once, the kernel is HBM-bound
		}
		return launch_gemm_tiled(w, a, C, sums, m, n, k, s);
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
