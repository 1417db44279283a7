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
#include "q8_0_plan.h"

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
// multiply-adds per lane per MFMA.  Measured on this part, a SIMD retires one wave64 VALU instruction per ~2.5 cycles
// once it holds two or more waves (a lone wave issues one per ~4-5), and MFMA and VALU time add on a SIMD, also across
// waves: a (tile, block) costs 32 + 32 matrix-pipe cycles plus 32 x 2.5 VALU cycles, ~145 cycles against the 32 of the int8
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
//   * every global address is a wave-uniform base in scalar registers plus a 32-bit lane offset (the addressing mode of
//     global_load with a scalar base): no 64-bit address arithmetic on the VALU, which is the pipe the fold saturates,
//     and ~10 fewer registers than per-lane pointers (the difference between spilling and not at two activation strips);
//   * latency is hidden by occupancy, not by a software pipeline: one result-register set per tile keeps the kernel
//     at <= 128 VGPRs, four workgroups per CU, four waves per SIMD.  (A two-result-set, software-pipelined variant
//     at two waves per SIMD measured 8 % slower: with so few waves the SIMD falls back to the lone-wave issue rate
//     whenever one of them waits.)
// a 64-bit offset that the compiler may keep in scalar registers (it is the same for every lane of the wave)
__device__ __forceinline__ int64_t uniform_i64(int64_t v) {
	const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v)), hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(static_cast<uint64_t>(v) >> 32));
	return static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo);
}

typedef const __attribute__((address_space(1))) uint8_t* gptr_u8;
// base + wave-uniform offset as a pointer the compiler must keep in scalar registers (and cannot fold the lane offset into)
__device__ __forceinline__ gptr_u8 scalar_base(const uint8_t* base, int64_t uniform_off) {
	gptr_u8 p = (gptr_u8)(base) + uniform_off;
	asm volatile("" : "+s"(p));
	return p;
}
template<typename T, bool NT> __device__ __forceinline__ T load_sv(gptr_u8 p, uint32_t lane_off) {
	typedef const __attribute__((address_space(1))) T* gp;
	if constexpr (NT) {
		return __builtin_nontemporal_load(reinterpret_cast<gp>(p + lane_off));
	} else {
		return *reinterpret_cast<gp>(p + lane_off);
	}
}

// GATE_UP: the prefill FFN's first half as ONE launch (the reference's mega_ffn composite: ffn_gate and ffn_up mul_mat -> silu ->
// mul -> activation operand of ffn_down, infra/core_traits.hpp:976-989).  Waves 0, 1 of a workgroup take strips 2 * blockIdx.x + {0, 1}
// of W (gate), waves 2, 3 the SAME strips of W2 (up), all four against the one activation image in LDS; the loop is the plain
// kernel's.  Behind it the up waves hand their tiles to the gate waves through LDS, and those apply silu(g) * u and quantize: a
// 32-value block of the down projection's activation is one activation row against one 32-row weight strip, i.e. one (register,
// half-wave) of an MFMA result tile -- 32 lanes hold it, its maximum is five cross-lane steps, and the quants go out in the tiled
// operand layout (through an LDS image of the tile, one 16-byte store per lane).  The two fp32 [M x N] intermediates are never
// written, the activation is read once for both matrices, and two launches (the second mat-mat and the SiLU * up quantizer) are gone.
// The arithmetic per value is that of the stand-alone kernels (same fp32 sums, silu_mul, quantize_row_q8_0), so the bytes are theirs.
// C / C2 (optional, inspection): the fp32 gate / up tiles as the launch computed them.
template<int TM, bool DUMP, int KS, bool STREAM, bool SPLIT, bool GATE_UP>
__device__ __forceinline__ void gemm_tiled_body(const uint8_t* __restrict__ W, const uint8_t* __restrict__ A, float* C, const float* R, int32_t* __restrict__ sums, int M, int N, int groups,
	float* __restrict__ partials, unsigned* __restrict__ counters, const uint8_t* __restrict__ W2, uint8_t* __restrict__ act_out, float* __restrict__ C2) {
	static_assert(!SPLIT || (KS > 1 && !DUMP), "K over several workgroups continues the K sets' sum");
	static_assert(!GATE_UP || (KS == 1 && !DUMP && !SPLIT && !STREAM), "the fused gate/up form runs one K set per workgroup");
	constexpr int DATA_BYTES  = TM * MACRO_BYTES;
	constexpr int STAGE_BYTES = DATA_BYTES + 16;
	constexpr int SET_BYTES	   = 2 * STAGE_BYTES + 256; // + 256: where waves that copy no scale table put theirs
	constexpr int PARK_BYTES   = KS > 1 ? KS * 4 * (KS - 1) * (16 * TM / KS) * 64 * 4 : 0; // the final sum over the K sets, below
	// GATE_UP epilogue: two up tiles per activation strip as fp32, then per gate wave TM tile images and TM x 32 scales
	constexpr int XCH_BYTES	   = GATE_UP ? 2 * TM * 16 * 64 * 4 : 0;
	constexpr int FUSE_BYTES   = GATE_UP ? XCH_BYTES + 2 * TM * (TILE_BYTES + 64) : 0;
	constexpr int LDS_BASE	   = KS * SET_BYTES > PARK_BYTES ? KS * SET_BYTES : PARK_BYTES;
	constexpr int LDS_BYTES	   = LDS_BASE > FUSE_BYTES ? LDS_BASE : FUSE_BYTES;
	__shared__ __align__(16) uint8_t lds_raw[LDS_BYTES];
	typedef _Float16 v4h __attribute__((ext_vector_type(4)));
	typedef float v16f __attribute__((ext_vector_type(16)));

	const int tid	   = threadIdx.x;
	const int lane	   = tid & 63;
	const int wave_all = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int wave	   = wave_all & 3; // which of the workgroup's four weight strips
	const int kr	   = wave_all >> 2; // which K range
	uint8_t* lds	   = lds_raw + kr * SET_BYTES;
	// the host launches KS > 1, and K over gridDim.z workgroups, only when they divide
	const int g_len	   = SPLIT ? groups / (KS * static_cast<int>(gridDim.z)) : groups / KS;
	const int g_base   = SPLIT ? (static_cast<int>(blockIdx.z) * KS + kr) * g_len : kr * g_len;
	const int half	   = lane >> 5;
	const int m_strips = (M + 31) / 32;
	const int n_strips = (N + 31) / 32;
	const int ms0	   = blockIdx.y * TM;
	const int ns	   = GATE_UP ? blockIdx.x * 2 + (wave & 1) : blockIdx.x * 4 + wave;
	const uint8_t* Wm  = (GATE_UP && wave >= 2) ? W2 : W; // wave-uniform
	if ((tid & 255) < 8) {
		*reinterpret_cast<uint32_t*>(lds + ((tid & 255) >> 2) * STAGE_BYTES + DATA_BYTES + 4 * (tid & 3)) = 0u;
	}
	// every address below is a wave-uniform part (scalar registers, advanced by scalar adds) plus one of three lane constants
	const uint32_t lane16 = 16u * lane;
	const int64_t w_off	  = uniform_i64(macro_offset(min(ns, n_strips - 1), g_base, groups));
	struct w_regs {
		v4i q[GROUP_BLOCKS];
		v2u d;
	};
	// activations: global -> registers -> LDS, shared out over the four waves: wave w moves tiles TM*w .. TM*w+TM-1 of the
	// TM*4 tiles of a group, waves 0..TM-1 also the 256-byte scale table of strip w
	int64_t a_off[TM];
	uint32_t a_dst[TM];
#pragma unroll
	for (int j = 0; j < TM; ++j) {
		const int u = TM * wave + j;
		a_off[j]	= uniform_i64(macro_offset(min(ms0 + u / 4, m_strips - 1), g_base, groups) + (u % 4) * TILE_BYTES);
		a_dst[j]	= (u / 4) * MACRO_BYTES + (u % 4) * TILE_BYTES; // + 16 * lane at the store
	}
	// every wave copies a dword per lane of a scale table (waves >= TM: strip TM-1's again, stored nowhere), so that all waves
	// issue the same loads
	const int64_t sc_off  = uniform_i64(macro_offset(min(ms0 + min(wave, TM - 1), m_strips - 1), g_base, groups) + MACRO_D_OFFSET);
	const uint32_t sc_dst = wave < TM ? wave * MACRO_BYTES + MACRO_D_OFFSET : 2 * STAGE_BYTES; // + 4 * lane at the store
	const uint32_t sc_stage = wave < TM ? STAGE_BYTES : 0; // the spare area is not staged
	struct a_regs {
		v4i q[TM];
		uint32_t d;
	};
	auto fetch_a = [&](int g, a_regs& r) {
		const int64_t adv = static_cast<int64_t>(g) * MACRO_BYTES;
		uint32_t l16 = lane16;
		asm volatile("" : "+v"(l16));
		const uint32_t l4 = l16 >> 2;
#pragma unroll
		for (int j = 0; j < TM; ++j) {
			r.q[j] = load_sv<v4i, false>(scalar_base(A, a_off[j] + adv), l16);
		}
		r.d = load_sv<uint32_t, false>(scalar_base(A, sc_off + adv), l4);
	};
	auto stash_a = [&](int stage, const a_regs& r) {
		uint8_t* p	 = lds + stage * STAGE_BYTES;
		uint32_t l16 = lane16;
		asm volatile("" : "+v"(l16)); // wave-uniform offsets stay in scalar registers, added here, instead of one more lane constant each
#pragma unroll
		for (int j = 0; j < TM; ++j) {
			*reinterpret_cast<v4i*>(p + a_dst[j] + l16) = r.q[j];
		}
		*reinterpret_cast<uint32_t*>(lds + stage * sc_stage + sc_dst + (l16 >> 2)) = r.d;
	};
	auto fetch_w = [&](int g, w_regs& r) {
		const int64_t at = w_off + static_cast<int64_t>(g) * MACRO_BYTES;
		const gptr_u8 p	 = scalar_base(Wm, at);
		uint32_t l16 = lane16;
		asm volatile("" : "+v"(l16));
		const uint32_t l8 = (l16 & 0x1F0u) >> 1; // the widening of a lane offset has to stay beside its loads for scalar base + 32-bit lane offset to be picked as the addressing mode
#pragma unroll
		for (int k = 0; k < GROUP_BLOCKS; ++k) {
			r.q[k] = load_sv<v4i, STREAM>(p + k * TILE_BYTES, l16);
		}
		r.d = load_sv<v2u, STREAM>(scalar_base(Wm, at + MACRO_D_OFFSET), l8);
	};
	// load number p of a group's set (PIECES of them: TM activation tiles, their scale dword, four weight tiles, their scales);
	// the same loads as fetch_a and fetch_w, which the prologue issues in one go
	constexpr int PIECES = TM + 2 + GROUP_BLOCKS;
	auto fetch_piece = [&](int p, int g, a_regs& ra, w_regs& rw) {
		uint32_t l16 = lane16;
		asm volatile("" : "+v"(l16));
		if (p < TM) {
			ra.q[p] = load_sv<v4i, false>(scalar_base(A, a_off[p] + static_cast<int64_t>(g) * MACRO_BYTES), l16);
		} else if (p == TM) {
			ra.d = load_sv<uint32_t, false>(scalar_base(A, sc_off + static_cast<int64_t>(g) * MACRO_BYTES), l16 >> 2);
		} else if (p < TM + 1 + GROUP_BLOCKS) {
			const int k = p - TM - 1;
			rw.q[k] = load_sv<v4i, STREAM>(scalar_base(Wm, w_off + static_cast<int64_t>(g) * MACRO_BYTES + k * TILE_BYTES), l16);
		} else {
			rw.d = load_sv<v2u, STREAM>(scalar_base(Wm, w_off + static_cast<int64_t>(g) * MACRO_BYTES + MACRO_D_OFFSET), (l16 & 0x1F0u) >> 1);
		}
	};
	v16f acc[TM];
#pragma unroll
	for (int i = 0; i < TM; ++i) {
		acc[i] = v16f{ 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 };
	}
	const int a_sc_rel = half ? DATA_BYTES : MACRO_D_OFFSET + 8 * (lane & 31);
	const int last	   = g_len - 1;

	w_regs wa, wb;
	a_regs pre;
	fetch_a(0, pre);
	fetch_w(0, wa);
	stash_a(0, pre);
	__syncthreads();
	// One trip = one 128-quant group.  Requested during it: the next group's activation tiles, then its weight tiles -- in
	// that order, because loads return in issue order: the (cached) activations are needed at the trip's end, for the barrier,
	// and must not queue behind weights that have until the next trip to arrive.  The requests are spread over the trip's
	// units, one or two behind each unit's LDS read: issued together at the trip's start, the sixteen waves of a CU that
	// leave the barrier at the same moment queue at the memory pipeline (0.4 to 2 k cycles per wave and trip before its first
	// MFMA).  Past the end the last group is requested again (a cache hit that nobody uses): every trip issues the same
	// loads, so every wait the compiler places is a count (a load under a condition makes it wait for everything
	// outstanding instead).
	auto trip = [&](int g, w_regs& cur, w_regs& nxt) {
		const int gn = min(g + 1, last);
		if (half) {
			cur.d = v2u{ 0u, 0u };
		}
		const uint8_t* stage = lds + (g & 1) * STAGE_BYTES;
		// the operand of unit u + 1 is read from LDS before unit u's arithmetic starts: one exposed LDS latency per trip, not eight
		constexpr int UNITS = GROUP_BLOCKS * TM;
		auto read_a = [&](int u, v4i& a, uint32_t& sc) {
			const int t = u / TM, i = u % TM;
			a  = *reinterpret_cast<const v4i*>(stage + i * MACRO_BYTES + t * TILE_BYTES + 16 * lane);
			sc = *reinterpret_cast<const uint16_t*>(stage + (half ? 0 : i * MACRO_BYTES) + a_sc_rel + 2 * t);
		};
		v4i a_cur;
		uint32_t s_cur;
		read_a(0, a_cur, s_cur);
#pragma unroll
		for (int u = 0; u < UNITS; ++u) {
			const int t = u / TM, i = u % TM;
			v4i a_nxt		= a_cur;
			uint32_t s_nxt	= s_cur;
			if (u + 1 < UNITS) {
				read_a(u + 1, a_nxt, s_nxt);
			}
			__builtin_amdgcn_sched_barrier(0);
#pragma unroll
			for (int pc = u * PIECES / UNITS; pc < (u + 1) * PIECES / UNITS; ++pc) {
				fetch_piece(pc, gn, pre, nxt);
			}
			__builtin_amdgcn_sched_barrier(0);
			const uint32_t wd = (t < 2) ? cur.d.x : cur.d.y;
			const v2u w_sc	  = v2u{ (t & 1) ? (wd >> 16) : (wd & 0xFFFFu), 0u };
			const v2u a_sc	  = v2u{ s_cur, 0u };
			const v16i zi	  = { 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 };
			const v16f zf	  = { 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 };
			const v16i sv	  = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_cur, cur.q[t], zi, 0, 0, 0);
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
			__builtin_amdgcn_sched_barrier(0);
			a_cur = a_nxt;
			s_cur = s_nxt;
		}
		stash_a((g + 1) & 1, pre);
		__syncthreads();
	};
	for (int g = 0; g < g_len; g += 2) {
		trip(g, wa, wb);
		if (g + 1 < g_len) {
			trip(g + 1, wb, wa);
		}
	}
	if constexpr (KS > 1 && !DUMP) {
		// The K sets' tiles are summed by all of them at once: set q keeps PER = 16 / KS of a lane's 16 values per strip (with
		// four sets: rows 8q .. 8q+7 of every 32-row strip), parks the other sets' shares in LDS, and after one barrier adds what
		// the others parked for it, in set order (s0 + s1 + s2 + s3 whatever q is, so the result does not depend on who adds),
		// and stores its own rows.  One set adding the others' whole tiles in turn took 12 % of the launch at M=512, N=K=4096.
		constexpr int PER = 16 / KS;
		__syncthreads(); // every set is through with its stages
		float* park = reinterpret_cast<float*>(lds_raw);
		auto slot	= [&](int q, int src) { // where set src parks its share of part q (src != q), this wave's strip
			return park + ((((q * 4 + wave) * (KS - 1)) + (src < q ? src : src - 1)) * (PER * TM)) * 64 + lane;
		};
#pragma unroll
		for (int q = 0; q < KS; ++q) {
			if (q != kr) {
				float* dst = slot(q, kr);
#pragma unroll
				for (int i = 0; i < TM; ++i) {
#pragma unroll
					for (int e = 0; e < PER; ++e) {
						dst[(i * PER + e) * 64] = acc[i][q * PER + e];
					}
				}
			}
		}
		__syncthreads();
		const int n = ns * 32 + (lane & 31);
		float mine[TM * PER]; // this wave's rows of the workgroup's tile (SPLIT: of its share of K)
#pragma unroll
		for (int q = 0; q < KS; ++q) {
			if (q == kr) {
#pragma unroll
				for (int i = 0; i < TM; ++i) {
#pragma unroll
					for (int e = 0; e < PER; ++e) {
						float v = 0.0f;
#pragma unroll
						for (int src = 0; src < KS; ++src) {
							const float part = src == q ? acc[i][q * PER + e] : slot(q, src)[(i * PER + e) * 64];
							v				 = src == 0 ? part : v + part;
						}
						mine[i * PER + e] = v;
					}
				}
			}
		}
		if constexpr (SPLIT) {
			// K over gridDim.z workgroups: every one leaves its tile in the scratch (each wave its own rows, as it holds them),
			// counts itself in, and the last to arrive adds the tiles in z order -- whoever that is -- and stores
			__shared__ int last_flag;
			const int kz_count = static_cast<int>(gridDim.z);
			const int unit	   = static_cast<int>(blockIdx.y * gridDim.x + blockIdx.x);
			constexpr int TILE_FLOATS = 4 * KS * TM * PER * 64; // = TM * 4096: a workgroup's tile
			float* tile = partials + (static_cast<int64_t>(unit) * kz_count) * TILE_FLOATS + wave_all * (TM * PER * 64) + lane;
			float* dst	= tile + static_cast<int64_t>(blockIdx.z) * TILE_FLOATS;
#pragma unroll
			for (int j = 0; j < TM * PER; ++j) {
				__hip_atomic_store(&dst[j * 64], mine[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
			}
			wait_stores_acknowledged();
			__syncthreads();
			if (tid == 0) {
				const unsigned prev = __hip_atomic_fetch_add(&counters[unit], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
				const int last		= (prev == static_cast<unsigned>(kz_count - 1));
				if (last) {
					__hip_atomic_store(&counters[unit], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); // ready for the next launch
				}
				last_flag = last;
			}
			__syncthreads();
			if (!last_flag) {
				return;
			}
#pragma unroll
			for (int j = 0; j < TM * PER; ++j) {
				mine[j] = 0.0f;
			}
			for (int z = 0; z < kz_count; ++z) {
				float got[TM * PER];
#pragma unroll
				for (int j = 0; j < TM * PER; ++j) {
					got[j] = __hip_atomic_load(&tile[static_cast<int64_t>(z) * TILE_FLOATS + j * 64], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
				}
#pragma unroll
				for (int j = 0; j < TM * PER; ++j) {
					mine[j] = z == 0 ? got[j] : mine[j] + got[j];
				}
			}
		}
#pragma unroll
		for (int i = 0; i < TM; ++i) {
#pragma unroll
			for (int e = 0; e < PER; ++e) {
				const int ee = kr * PER + e;
				const int m	 = (ms0 + i) * 32 + 8 * (ee >> 2) + 4 * half + (ee & 3);
				if (m < M && n < N) {
					const int64_t at = static_cast<int64_t>(m) * N + n;
					const float v	 = mine[i * PER + e];
					C[at]			 = R ? v + R[at] : v; // R may be C: read before the write, by the same thread
				}
			}
		}
		return;
	}
	if constexpr (GATE_UP) {
		// Every wave is through with the stages (the last trip ended in a barrier).  The gate wave and the up wave of a strip share
		// the work behind the loop: registers 0..7 of every tile are finished by the gate wave, 8..15 by the up wave, each handing
		// the other the half it does not finish (the exp and the divides of SiLU and of the quantizer are a quarter of the loop's
		// VALU work; on two of the four waves alone they cost the launch 6 %).
		const int pair	 = wave & 1;
		const bool is_up = wave >= 2;
		float* xch		 = reinterpret_cast<float*>(lds_raw); // [pair][TM][16][64]: slot (i, e) holds the value of the wave that does not finish it
#pragma unroll
		for (int i = 0; i < TM; ++i) {
#pragma unroll
			for (int e = 0; e < 8; ++e) {
				const int give						  = is_up ? e : e + 8;
				xch[((pair * TM + i) * 16 + give) * 64 + lane] = acc[i][give];
			}
		}
		float* dbg = is_up ? C2 : C; // inspection copies of the fp32 tiles
		if (dbg) {
			const int n = ns * 32 + (lane & 31);
#pragma unroll
			for (int i = 0; i < TM; ++i) {
#pragma unroll
				for (int e = 0; e < 16; ++e) {
					const int m = (ms0 + i) * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
					if (m < M && n < N) {
						dbg[static_cast<int64_t>(m) * N + n] = acc[i][e];
					}
				}
			}
		}
		__syncthreads();
		uint8_t* image = lds_raw + XCH_BYTES + pair * TM * (TILE_BYTES + 64); // the pair's TM tile images, each followed by its 32 scales
		const int j	   = lane & 31; // the lane's weight row = quant j of the block
#pragma unroll
		for (int i = 0; i < TM; ++i) {
			uint8_t* tile	 = image + i * (TILE_BYTES + 64);
			uint16_t* scales = reinterpret_cast<uint16_t*>(tile + TILE_BYTES);
#pragma unroll
			for (int e8 = 0; e8 < 8; ++e8) {
				const int e		  = is_up ? e8 + 8 : e8;
				const float other = xch[((pair * TM + i) * 16 + e) * 64 + lane];
				const float v	  = is_up ? silu_mul(other, acc[i][e]) : silu_mul(acc[i][e], other);
				// the block = this register over the 32 lanes of the half-wave: quantize_row_q8_0 on it
				float amax = fabsf(v);
#pragma unroll
				for (int off = 16; off >= 1; off >>= 1) {
					amax = fmaxf(amax, __shfl_xor(amax, off));
				}
				const float d  = __fdiv_rn(amax, 127.0f);
				const float id = (amax != 0.0f) ? __fdiv_rn(127.0f, amax) : 0.0f;
				const int r	   = 8 * (e >> 2) + 4 * half + (e & 3); // row within the activation strip
				tile[16 * (r + 32 * (j >> 4)) + (j & 15)] = static_cast<uint8_t>(quantize_value(v, id));
				if (j == 0) {
					scales[r] = float_to_half_bits(d);
				}
			}
		}
		__syncthreads(); // both waves of a pair have filled its images
		// tile i of the pair goes out through the gate wave (even i) or the up wave (odd i): one 16-byte store per lane
		const int out_groups = N / GROUP_K; // the activation is [M x N]: N / 128 groups per strip, this strip's block is ns
		if (ns < n_strips) {
#pragma unroll
			for (int i = 0; i < TM; ++i) {
				if ((i & 1) == (is_up ? 1 : 0) && ms0 + i < m_strips) {
					const uint8_t* tile = image + i * (TILE_BYTES + 64);
					uint8_t* macro		= act_out + macro_offset(ms0 + i, ns / GROUP_BLOCKS, out_groups);
					*reinterpret_cast<v4i*>(macro + (ns % GROUP_BLOCKS) * TILE_BYTES + 16 * lane) = *reinterpret_cast<const v4i*>(tile + 16 * lane);
					if (lane < STRIP_ROWS) {
						*reinterpret_cast<uint16_t*>(macro + MACRO_D_OFFSET + 8 * lane + 2 * (ns % GROUP_BLOCKS)) = reinterpret_cast<const uint16_t*>(tile + TILE_BYTES)[lane];
					}
				}
			}
		}
		return;
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

template<int TM, bool DUMP, int KS = 1, bool STREAM = false, bool SPLIT = false>
__global__ __launch_bounds__(256 * KS, 4) void gemm_tiled_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ A, float* C, const float* R, int32_t* __restrict__ sums, int M, int N,
	int groups, float* __restrict__ partials, unsigned* __restrict__ counters) {
	gemm_tiled_body<TM, DUMP, KS, STREAM, SPLIT, false>(W, A, C, R, sums, M, N, groups, partials, counters, nullptr, nullptr, nullptr);
}

// the fused gate / up form (GATE_UP above): N = rows of each of the two matrices; gate_out / up_out optional
template<int TM>
__global__ __launch_bounds__(256, 4) void gemm_gate_up_kernel(const uint8_t* __restrict__ W_gate, const uint8_t* __restrict__ W_up, const uint8_t* __restrict__ A, uint8_t* __restrict__ act_out,
	float* __restrict__ gate_out, float* __restrict__ up_out, int M, int N, int groups) {
	gemm_tiled_body<TM, false, 1, false, false, true>(W_gate, A, gate_out, nullptr, nullptr, M, N, groups, nullptr, nullptr, W_up, act_out, up_out);
}

// Executes a cut made by plan_gemm_tile (q8_0_plan.h): TM activation strips per wave, KS sets of four waves per workgroup,
// and, with non-temporal weights, K over kz workgroups per tile whose tiles are added through the scratch.
template<int TM, bool STREAM> static hipError_t launch_gemm_tiled_t(const gemm_tile_cut& cut, const uint8_t* w, const uint8_t* a, float* C, const float* R, int32_t* sums, int m, int n, int k, hipStream_t s) {
	const int groups = k / GROUP_K;
	const dim3 grid(cut.grid_x, cut.grid_y);
	if (sums) {
		gemm_tiled_kernel<TM, true><<<grid, dim3(256), 0, s>>>(w, a, C, R, sums, m, n, groups, nullptr, nullptr);
		return hipGetLastError();
	}
	const int ks = cut.ks;
	if constexpr (STREAM) {
		if (cut.kz > 1) {
			float* partials	   = nullptr;
			unsigned* counters = nullptr;
			const hipError_t e = acquire_gemm_split_scratch(&partials, &counters, s);
			if (e != hipSuccess) {
				return e;
			}
			return launch_kernel(KIND_GEMM, gemm_tiled_kernel<TM, false, 4, true, true>, dim3(grid.x, grid.y, static_cast<unsigned>(cut.kz)), dim3(1024), 0, s, w, a, C, R, sums, m, n, groups, partials,
				counters);
		}
	}
	if (ks == 4) {
		return launch_kernel(KIND_GEMM, gemm_tiled_kernel<TM, false, 4, STREAM>, grid, dim3(1024), 0, s, w, a, C, R, sums, m, n, groups, static_cast<float*>(nullptr), static_cast<unsigned*>(nullptr));
	}
	if (ks == 2) {
		return launch_kernel(KIND_GEMM, gemm_tiled_kernel<TM, false, 2, STREAM>, grid, dim3(512), 0, s, w, a, C, R, sums, m, n, groups, static_cast<float*>(nullptr), static_cast<unsigned*>(nullptr));
	}
	return launch_kernel(KIND_GEMM, gemm_tiled_kernel<TM, false, 1, STREAM>, grid, dim3(256), 0, s, w, a, C, R, sums, m, n, groups, static_cast<float*>(nullptr), static_cast<unsigned*>(nullptr));
}

// stream: the weights are read once and not again (a batch of decode rows against a large matrix), so their loads bypass the caches.
static hipError_t launch_gemm_tiled(const gemm_tile_cut& cut, const uint8_t* w, const uint8_t* a, float* C, const float* R, int32_t* sums, int m, int n, int k, hipStream_t s, bool stream) {
	if (stream) {
		return cut.tm == 2 ? launch_gemm_tiled_t<2, true>(cut, w, a, C, R, sums, m, n, k, s) : launch_gemm_tiled_t<1, true>(cut, w, a, C, R, sums, m, n, k, s);
	}
	return cut.tm == 2 ? launch_gemm_tiled_t<2, false>(cut, w, a, C, R, sums, m, n, k, s) : launch_gemm_tiled_t<1, false>(cut, w, a, C, R, sums, m, n, k, s);
}

// act_out (tiled, [M x n_ff]) = quantize_row_q8_0(silu(W_gate . Aq) * (W_up . Aq)); gate_dbg / up_dbg: optional fp32 copies of the two
// mat-mats' outputs.  workspace: 2 * M * n_ff floats for shapes the fused form does not take (plan_gate_up_fused), else unused.
hipError_t launch_gemm_gate_up_silu(const void* w_gate, const void* w_up, const void* aq, void* act_out, float* gate_dbg, float* up_dbg, float* workspace, int64_t M, int64_t n_ff, int64_t K,
	hipStream_t s) {
	if (M == 0 || n_ff == 0) {
		return hipSuccess;
	}
	gemm_tile_cut cut{};
	if (plan_gate_up_fused(M, n_ff, K, &cut)) {
		const uint8_t* wg = static_cast<const uint8_t*>(w_gate);
		const uint8_t* wu = static_cast<const uint8_t*>(w_up);
		const uint8_t* a  = static_cast<const uint8_t*>(aq);
		uint8_t* out	  = static_cast<uint8_t*>(act_out);
		const int m = static_cast<int>(M), n = static_cast<int>(n_ff), groups = static_cast<int>(K / GROUP_K);
		const dim3 grid(cut.grid_x, cut.grid_y);
		if (cut.tm == 2) {
			return launch_kernel(KIND_GEMM, gemm_gate_up_kernel<2>, grid, dim3(256), 0, s, wg, wu, a, out, gate_dbg, up_dbg, m, n, groups);
		}
		return launch_kernel(KIND_GEMM, gemm_gate_up_kernel<1>, grid, dim3(256), 0, s, wg, wu, a, out, gate_dbg, up_dbg, m, n, groups);
	}
	float* gate = gate_dbg ? gate_dbg : workspace;
	float* up	= up_dbg ? up_dbg : workspace + M * n_ff;
	hipError_t e = launch_gemm(w_gate, aq, gate, nullptr, M, n_ff, K, true, s);
	if (e != hipSuccess) {
		return e;
	}
	e = launch_gemm(w_up, aq, up, nullptr, M, n_ff, K, true, s);
	if (e != hipSuccess) {
		return e;
	}
	return launch_silu_mul_quantize(gate, up, act_out, M, n_ff, true, s);
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
		if (sums) { // the inspection variant runs on the plain tile kernel, whatever the shape
			return launch_gemm_tiled(plan_gemm_tile(M, N, K, false), w, a, C, residual, sums, m, n, k, s, false);
		}
		const gemm_plan plan = plan_gemm(M, N, K); // which kernel and how it cuts the work: q8_0_plan.h
		if (plan.kernel == MM_GEMM_SKINNY) {
			return launch_gemm_skinny(W, Aq, C, sums, M, N, K, s, residual);
		}
		return launch_gemm_tiled(plan.tile, w, a, C, residual, sums, m, n, k, s, plan.kernel == MM_GEMM_TILE_STREAM);
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
