// Batched decode with up to sixteen activation rows on the matrix cores: y[m][n] = dot(W row n, quantize(x row m)), gfx950.
//
// The streaming mat-vec once more (q8_0_gemv.hip, q8_0_gemv_rows.hip): one workgroup of sixteen waves per (32-row weight strip,
// K split), every wave puts the weight loads of its K range in flight before it waits for anything, and quantizes its slice of
// the activation rows on the spot from fp32 while they fly (the stand-alone quantize kernel's arithmetic, reference
// quantize_row_q8_0, cpu/avx_2.hpp:4439-4489) -- no quantize launch in front, no quantized copy of the activations in memory.
// What differs from the few-row kernel is the inner product: there every lane reads each row's 16 quants from LDS and runs a
// v_dot4 chain per row, and from four rows on the CU's LDS port is what the launch waits for (one 1 KB read per wave, block and
// row).  Here the quantized slices go to LDS as an MFMA operand -- a 32 x 32 tile of which rows 0..R-1 (R = 8 or 16) are the
// activation rows and the rest one shared row of zeros -- so a block costs one 16-byte LDS read per lane and one
// v_mfma_i32_32x32x32_i8 whatever the number of rows, and of the 16 sums a lane gets back only the R / 2 that belong to real rows are
// scaled and accumulated.
// Arithmetic per output element: exact int32 block sums, each times d_w * d_x in fp32, accumulated per wave in block order, then
// over the waves and K splits in fixed order (reference vec_dot_q8_0_q8_0, cpu/avx_2.hpp:4534-4747); output [M][N], n fastest
// (cpu/avx_2.hpp:4934).
#include "q8_0_plan.h"

namespace nh {

// R: activation rows a launch takes, 8 or 16.  One k-half of a block's operand tile: rows 0..R-1 and the row of zeros, 16 quants each.
template<int R> constexpr int rows_a_half = (R + 1) * 16;
template<int R> constexpr int rows_a_tile = 2 * rows_a_half<R>;

// One chunk of a wave's K range: groups [gc, gc + CNT).  CNT is a template parameter for the reason given at gemv_chunk_n.
// a_tiles: this wave's LDS operand tiles, one per block of the chunk; a_scales: [block][R] fp32 activation scales.
template<int R, int TILES, int CNT>
__device__ __forceinline__ void rows8_chunk_n(const uint8_t* __restrict__ w_strip, const float* __restrict__ x, int64_t K, int M, uint8_t* a_tiles, float* a_scales, int gc, int lane,
	float (&acc)[R / 2]) {
	constexpr int cnt	 = CNT;
	constexpr int ROWS8 = R, ROWS8_A_HALF = rows_a_half<R>, ROWS8_A_TILE = rows_a_tile<R>;
	constexpr int BLOCKS = cnt * GROUP_BLOCKS; // blocks of the chunk, per row
	const int r			 = lane & 31;
	const int half		 = lane >> 5;

	// ---- 1. the activation slices, requested first (loads return in issue order): item v = lane + 64 i is float4 v % 8 of
	// block (v / 8) % BLOCKS of row (v / 8) / BLOCKS, so that eight consecutive lanes hold one block ----
	constexpr int X_LOADS = cnt > 0 ? ROWS8 * BLOCKS * 8 / 64 : 1;
	float4 xf[X_LOADS];
#pragma unroll
	for (int i = 0; i < X_LOADS; ++i) {
		const int v = lane + 64 * i, blk = (v >> 3) % (BLOCKS > 0 ? BLOCKS : 1), m = (v >> 3) / (BLOCKS > 0 ? BLOCKS : 1);
		xf[i] = cnt > 0 && m < M ? reinterpret_cast<const float4*>(x + static_cast<int64_t>(m) * K + static_cast<int64_t>(gc) * GROUP_K + blk * QK)[v & 7] : make_float4(0.f, 0.f, 0.f, 0.f);
	}

	// ---- 2. every weight byte of the chunk, in flight at once ----
	v4i q[TILES][GROUP_BLOCKS];
	v2u dd[TILES];
	const uint8_t* macro0 = w_strip + static_cast<int64_t>(gc) * MACRO_BYTES;
#pragma unroll
	for (int t = 0; t < TILES; ++t) {
		if (t < cnt) {
			const uint8_t* macro = macro0 + t * MACRO_BYTES;
#pragma unroll
			for (int j = 0; j < GROUP_BLOCKS; ++j) {
				q[t][j] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(macro + j * TILE_BYTES + 16 * lane));
			}
			dd[t] = __builtin_nontemporal_load(reinterpret_cast<const v2u*>(macro + MACRO_D_OFFSET + 8 * r));
		}
	}

	// ---- 3. quantize the slices into the operand tiles: dword f of row m's block goes to k-half f / 4, row m, bytes 4 (f % 4) ----
#pragma unroll
	for (int i = 0; i < X_LOADS; ++i) {
		const int v = lane + 64 * i, blk = (v >> 3) % (BLOCKS > 0 ? BLOCKS : 1), m = (v >> 3) / (BLOCKS > 0 ? BLOCKS : 1), f = v & 7;
		// load i holds rows [i * ROWS_PER_LOAD, + ROWS_PER_LOAD) in every lane: past M there is nothing to quantize (wave-uniform),
		// zeros with scale 0 go out instead
		constexpr int ROWS_PER_LOAD = BLOCKS >= 8 ? 1 : 8 / (BLOCKS > 0 ? BLOCKS : 8);
		uint16_t dh		= 0;
		uint32_t packed = 0u;
		if (i * ROWS_PER_LOAD < M) {
			packed = quantize_block_lane(xf[i], &dh); // a row past M within the load holds zeros and quantizes to zeros with scale 0
		}
		if (cnt > 0) {
			*reinterpret_cast<uint32_t*>(a_tiles + blk * ROWS8_A_TILE + (f >> 2) * ROWS8_A_HALF + m * 16 + 4 * (f & 3)) = packed;
			if (f == 0) {
				a_scales[blk * ROWS8 + m] = half_bits_to_float(dh);
			}
		}
	}
	__builtin_amdgcn_wave_barrier(); // wave-local hand-off: the same wave wrote and reads; the LDS counter wait orders it

	// ---- 4. one MFMA per block as the tiles land; lane (r, half) gets the sums of column r for rows 8 i + 4 half + (0..3) in s[4 i .. 4 i + 3] ----
	const int a_row = r < ROWS8 ? r : ROWS8; // operand rows past the last real one: the row of zeros
#pragma unroll
	for (int t = 0; t < TILES; ++t) {
		if (t < cnt) {
			const float dw[GROUP_BLOCKS] = { half_bits_to_float(static_cast<uint16_t>(dd[t].x & 0xFFFFu)), half_bits_to_float(static_cast<uint16_t>(dd[t].x >> 16)),
				half_bits_to_float(static_cast<uint16_t>(dd[t].y & 0xFFFFu)), half_bits_to_float(static_cast<uint16_t>(dd[t].y >> 16)) };
#pragma unroll
			for (int j = 0; j < GROUP_BLOCKS; ++j) {
				const int blk	= t * GROUP_BLOCKS + j;
				const v4i a		= *reinterpret_cast<const v4i*>(a_tiles + blk * ROWS8_A_TILE + half * ROWS8_A_HALF + a_row * 16);
				const v16i zi	= { 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 };
				const v16i s	= __builtin_amdgcn_mfma_i32_32x32x32_i8(a, q[t][j], zi, 0, 0, 0);
#pragma unroll
				for (int e4 = 0; e4 < R / 8; ++e4) { // sums 4 e4 .. 4 e4 + 3: rows 8 e4 + 4 half + (0..3)
					const float4 dx = *reinterpret_cast<const float4*>(a_scales + blk * ROWS8 + 8 * e4 + 4 * half);
					acc[4 * e4 + 0] = fmaf(static_cast<float>(s[4 * e4 + 0]), dw[j] * dx.x, acc[4 * e4 + 0]);
					acc[4 * e4 + 1] = fmaf(static_cast<float>(s[4 * e4 + 1]), dw[j] * dx.y, acc[4 * e4 + 1]);
					acc[4 * e4 + 2] = fmaf(static_cast<float>(s[4 * e4 + 2]), dw[j] * dx.z, acc[4 * e4 + 2]);
					acc[4 * e4 + 3] = fmaf(static_cast<float>(s[4 * e4 + 3]), dw[j] * dx.w, acc[4 * e4 + 3]);
				}
			}
		}
	}
}

template<int R, int TILES>
__device__ __forceinline__ void rows8_chunk(const uint8_t* __restrict__ w_strip, const float* __restrict__ x, int64_t K, int M, uint8_t* a_tiles, float* a_scales, int gc, int cnt, int lane,
	float (&acc)[R / 2]) {
	switch (cnt) { // wave-uniform
		case 1:
			rows8_chunk_n<R, TILES, 1>(w_strip, x, K, M, a_tiles, a_scales, gc, lane, acc);
			break;
		case 2:
			if constexpr (TILES >= 2) {
				rows8_chunk_n<R, TILES, 2>(w_strip, x, K, M, a_tiles, a_scales, gc, lane, acc);
			}
			break;
		default: // 0: an idle wave (still takes part in the reduction)
			break;
	}
}

template<int R, int TILES, bool LOOP>
__global__ __launch_bounds__(GEMV_WAVES * 64) void gemv_rows8_kernel(const uint8_t* __restrict__ W, const float* __restrict__ x, float* y, const float* residual, uint64_t* __restrict__ tagged,
	unsigned epoch, int M, int N, int groups, int split_shift) {
	constexpr int ROWS8 = R, ROWS8_A_HALF = rows_a_half<R>, ROWS8_A_TILE = rows_a_tile<R>;
	__shared__ __align__(16) uint8_t a_tiles[GEMV_WAVES][TILES * GROUP_BLOCKS * ROWS8_A_TILE];
	__shared__ __align__(16) float a_scales[GEMV_WAVES][TILES * GROUP_BLOCKS * ROWS8];
	__shared__ float red[R / 2][GEMV_WAVES][64];
	const int tid	 = threadIdx.x;
	const int lane	 = tid & 63;
	const int wave	 = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int splits = 1 << split_shift;
	const int strip	 = static_cast<int>(blockIdx.x >> split_shift);
	const int split	 = static_cast<int>(blockIdx.x) & (splits - 1);
	int g0, g1; // this wave's share of the strip's K range
	wave_k_range(groups, split_shift, split, GEMV_WAVES, wave, g0, g1);
	const int64_t K = static_cast<int64_t>(groups) * GROUP_K;

	// the row of zeros of every operand tile of this wave (the quantizer only ever writes rows 0..R-1)
	for (int i = lane; i < TILES * GROUP_BLOCKS * 2 * 4; i += 64) {
		*reinterpret_cast<uint32_t*>(&a_tiles[wave][(i >> 3) * ROWS8_A_TILE + ((i >> 2) & 1) * ROWS8_A_HALF + ROWS8 * 16 + 4 * (i & 3)]) = 0u;
	}
	__builtin_amdgcn_wave_barrier();

	const uint8_t* w_strip = W + macro_offset(strip, 0, groups);
	float acc[R / 2];
#pragma unroll
	for (int e = 0; e < R / 2; ++e) {
		acc[e] = 0.0f;
	}
	if constexpr (!LOOP) {
		rows8_chunk<R, TILES>(w_strip, x, K, M, a_tiles[wave], a_scales[wave], g0, g1 - g0, lane, acc);
	} else {
		for (int gc = g0; gc < g1; gc += TILES) {
			rows8_chunk<R, TILES>(w_strip, x, K, M, a_tiles[wave], a_scales[wave], gc, min(TILES, g1 - gc), lane, acc);
			__builtin_amdgcn_wave_barrier(); // the next chunk overwrites this wave's tiles
		}
	}

	// ---- one reduction per workgroup, fixed order: thread 32 * m + l owns output (row m, strip row l) ----
#pragma unroll
	for (int e = 0; e < R / 2; ++e) {
		red[e][wave][lane] = acc[e];
	}
	__syncthreads();
	const int m = tid >> 5, l = tid & 31;
	if (m >= M || m >= R) {
		return;
	}
	float total = 0.0f;
#pragma unroll
	for (int w = 0; w < GEMV_WAVES; ++w) {
		total += red[4 * (m >> 3) + (m & 3)][w][32 * ((m >> 2) & 1) + l]; // row m = 8 e4 + 4 half + i sits in lanes of that half, sum 4 e4 + i
	}
	const int row	= strip * STRIP_ROWS + l;
	float* ym		= y + static_cast<int64_t>(m) * N;
	const float* rm = residual ? residual + static_cast<int64_t>(m) * N : nullptr; // may be ym: read before the write, by the same thread
	if (splits == 1) {
		if (row < N) {
			ym[row] = rm ? total + rm[row] : total;
		}
		return;
	}
	split_k_finish(tagged, epoch, strip * R + m, splits, split, l, total, ym, row, N, rm);
}

template<int R, int TILES, bool LOOP> static hipError_t launch_rows8_n(const gemv_plan& p, const uint8_t* W, const float* x, float* y, const float* r, int M, int N, const gemv_scratch& sc, hipStream_t s) {
	const dim3 grid(static_cast<unsigned>(p.strips * p.splits)), block(GEMV_WAVES * 64);
	int shift = 0;
	while ((1 << shift) < p.splits) {
		++shift;
	}
	return launch_kernel(KIND_GEMV, gemv_rows8_kernel<R, TILES, LOOP>, grid, block, 0, s, W, x, y, r, sc.tagged, sc.epoch, M, N, p.groups, shift);
}

// 1 <= M <= 16 fp32 activation rows [M][K] against a tiled weight [N][K]; y is [M][N].  K % 128 == 0 (checked by the caller).
hipError_t launch_gemv_rows_mfma(const void* W, const float* x, float* y, int64_t M, int64_t N, int64_t K, hipStream_t s, const float* residual) {
	const int64_t strips = (N + STRIP_ROWS - 1) / STRIP_ROWS;
	if (M < 1 || M > GEMV_ROWS_MFMA_MAX) {
		return hipErrorInvalidValue;
	}
	if (strips == 0) {
		return hipSuccess;
	}
	const int rows	  = M <= 8 ? 8 : 16;
	const gemv_plan p = plan_gemv_rows_mfma(strips, K, rows, stream_is_capturing(s));
	gemv_scratch sc;
	if (p.splits > 1) {
		const hipError_t e = get_gemv_scratch(&sc, true, s);
		if (e != hipSuccess) {
			return e;
		}
	}
	const uint8_t* w = static_cast<const uint8_t*>(W);
	const int m = static_cast<int>(M), n = static_cast<int>(N);
	if (rows == 16) { // one group per wave and step: sixteen rows of two groups would not fit the registers
		return p.tiles > 1 ? launch_rows8_n<16, 1, true>(p, w, x, y, residual, m, n, sc, s) : launch_rows8_n<16, 1, false>(p, w, x, y, residual, m, n, sc, s);
	}
	if (p.tiles > 2) {
		return launch_rows8_n<8, 2, true>(p, w, x, y, residual, m, n, sc, s);
	}
	return p.tiles <= 1 ? launch_rows8_n<8, 1, false>(p, w, x, y, residual, m, n, sc, s) : launch_rows8_n<8, 2, false>(p, w, x, y, residual, m, n, sc, s);
}

} // namespace nh
