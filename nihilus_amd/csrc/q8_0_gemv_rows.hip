// Batched decode with two or three activation rows (2 <= M <= GEMV_ROWS_MAX): y[m][n] = dot(W row n, quantize(x row m)), gfx950.
//
// The streaming mat-vec again (q8_0_gemv.hip): one workgroup of sixteen waves per (32-row weight strip, K split), every
// wave puts all the weight loads of its K range in flight before it waits for anything, the activation slice is quantized
// on the spot from fp32 (same arithmetic as the stand-alone quantize kernel, reference quantize_row_q8_0,
// cpu/avx_2.hpp:4439-4489) while the weights fly.  The only difference is that the wave stages MR activation slices
// instead of one and runs MR dot products against every weight tile it fetched, so the weights are still read exactly
// once and no quantize launch, no quantized copy of the activations and no 32-row MFMA tile (30 of whose rows would be
// padding at M = 2) is involved.  The integer dots and the quantizer cost MR times those of the mat-vec (every strip's
// workgroup quantizes the rows again), which an HBM-bound kernel can afford for two or three rows.  From four rows on every lane's
// LDS reads of the rows' quants (one 16-byte read per lane, block and row) are what a CU waits for ([4096 x 4096]: 4.6 us at two
// rows, 8.1 us at four): there the rows go to the matrix cores instead (q8_0_gemv_rows_mfma.hip on small matrices, the quantize
// launch and the MFMA kernels otherwise).
// Arithmetic per output element: exact int32 block sums, fp32 scale-and-accumulate in the mat-vec's fixed order
// (reference vec_dot_q8_0_q8_0, cpu/avx_2.hpp:4534-4747); output [M][N] with n fastest (cpu/avx_2.hpp:4934).
#include "q8_0_gemv_tiled.h"

namespace nh {

// One chunk of a wave's K range for MR activation rows: groups [gc, gc + CNT).  CNT is a template parameter for the
// reason given at gemv_chunk_n: the waits in front of the quantizer can only leave the weight loads in flight if the
// compiler can count them.
template<int TILES, int MR, int CNT>
__device__ __forceinline__ void gemv_rows_chunk_n(const uint8_t* __restrict__ w_strip, const float* __restrict__ x, int64_t K, uint8_t (*xs_q)[TILES * GROUP_K], float (*xs_d)[TILES * GROUP_BLOCKS],
	int gc, int lane, float (&acc)[MR]) {
	constexpr int cnt = CNT;
	const int r		  = lane & 31;
	const int half	  = lane >> 5;

	// ---- 1. the MR activation slices, requested first (loads return in issue order) ----
	constexpr int XF_LOADS = (TILES * 32 + 63) / 64; // float4 per lane and row: 128 floats per group = 32 float4
	float4 xf[MR][XF_LOADS];
#pragma unroll
	for (int m = 0; m < MR; ++m) {
		const float4* x4 = reinterpret_cast<const float4*>(x + m * K + static_cast<int64_t>(gc) * GROUP_K);
#pragma unroll
		for (int i = 0; i < XF_LOADS; ++i) {
			const int v = lane + 64 * i;
			xf[m][i]	= v < cnt * 32 ? x4[v] : make_float4(0.f, 0.f, 0.f, 0.f);
		}
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

	// ---- 3. quantize the slices into this wave's LDS: quants 16-byte aligned per half block, scales as fp32 ----
#pragma unroll
	for (int m = 0; m < MR; ++m) {
#pragma unroll
		for (int i = 0; i < XF_LOADS; ++i) {
			const int v = lane + 64 * i;
			uint16_t dh;
			const uint32_t packed = quantize_block_lane(xf[m][i], &dh); // all lanes take part; lanes past the slice hold zeros
			if (v < cnt * 32) {
				*reinterpret_cast<uint32_t*>(xs_q[m] + 4 * v) = packed; // block v/8 at 32*(v/8), dword v%8
				if ((v & 7) == 0) {
					xs_d[m][v >> 3] = half_bits_to_float(dh); // the fp16-rounded scale, exactly what a stored block would hold
				}
			}
		}
	}
	__builtin_amdgcn_wave_barrier(); // wave-local hand-off: the same wave wrote and reads; the LDS counter wait orders it

	// ---- 4. MR dot products per weight tile, as the tiles land ----
#pragma unroll
	for (int t = 0; t < TILES; ++t) {
		if (t < cnt) {
			const float dw[GROUP_BLOCKS] = { half_bits_to_float(static_cast<uint16_t>(dd[t].x & 0xFFFFu)), half_bits_to_float(static_cast<uint16_t>(dd[t].x >> 16)),
				half_bits_to_float(static_cast<uint16_t>(dd[t].y & 0xFFFFu)), half_bits_to_float(static_cast<uint16_t>(dd[t].y >> 16)) };
#pragma unroll
			for (int j = 0; j < GROUP_BLOCKS; ++j) {
				const int jj = t * GROUP_BLOCKS + j;
#pragma unroll
				for (int m = 0; m < MR; ++m) {
					const v4i xv = *reinterpret_cast<const v4i*>(xs_q[m] + jj * QK + 16 * half);
					const int s	 = dot16(q[t][j], xv);
					acc[m]		 = fmaf(static_cast<float>(s), dw[j] * xs_d[m][jj], acc[m]);
				}
			}
		}
	}
}

template<int TILES, int MR>
__device__ __forceinline__ void gemv_rows_chunk(const uint8_t* __restrict__ w_strip, const float* __restrict__ x, int64_t K, uint8_t (*xs_q)[TILES * GROUP_K], float (*xs_d)[TILES * GROUP_BLOCKS], int gc,
	int cnt, int lane, float (&acc)[MR]) {
	switch (cnt) { // wave-uniform
		case 1:
			gemv_rows_chunk_n<TILES, MR, 1>(w_strip, x, K, xs_q, xs_d, gc, lane, acc);
			break;
		case 2:
			if constexpr (TILES >= 2) {
				gemv_rows_chunk_n<TILES, MR, 2>(w_strip, x, K, xs_q, xs_d, gc, lane, acc);
			}
			break;
		default: // 0: an idle wave (still takes part in the reduction)
			break;
	}
}

// TILES <= 2 groups per wave and chunk: MR slices of fp32 activations sit in registers next to the weight tiles (two rows fit
// in 64 registers = two workgroups per CU; three take 65 and run as one, which measured faster than spilling to stay at two).
template<int TILES, int MR, bool LOOP>
__global__ __launch_bounds__(GEMV_WAVES * 64) void gemv_rows_kernel(const uint8_t* __restrict__ W, const float* __restrict__ x, float* y, const float* residual, uint64_t* __restrict__ tagged, unsigned epoch,
	int N, int groups, int split_shift) {
	__shared__ __align__(16) uint8_t xs_q[GEMV_WAVES][MR][TILES * GROUP_K]; // each wave's quantized slices, block jj of row m at 32*jj
	__shared__ float xs_d[GEMV_WAVES][MR][TILES * GROUP_BLOCKS];
	__shared__ float red[MR][GEMV_WAVES][64];
	const int tid	 = threadIdx.x;
	const int lane	 = tid & 63;
	const int wave	 = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int splits = 1 << split_shift;
	const int strip	 = static_cast<int>(blockIdx.x >> split_shift);
	const int split	 = static_cast<int>(blockIdx.x) & (splits - 1);
	int g0, g1; // this wave's share of the strip's K range
	wave_k_range(groups, split_shift, split, GEMV_WAVES, wave, g0, g1);
	const int64_t K	 = static_cast<int64_t>(groups) * GROUP_K;

	const uint8_t* w_strip = W + macro_offset(strip, 0, groups);
	float acc[MR];
#pragma unroll
	for (int m = 0; m < MR; ++m) {
		acc[m] = 0.0f;
	}
	if constexpr (!LOOP) {
		gemv_rows_chunk<TILES, MR>(w_strip, x, K, xs_q[wave], xs_d[wave], g0, g1 - g0, lane, acc);
	} else {
		for (int gc = g0; gc < g1; gc += TILES) {
			gemv_rows_chunk<TILES, MR>(w_strip, x, K, xs_q[wave], xs_d[wave], gc, min(TILES, g1 - gc), lane, acc);
			__builtin_amdgcn_wave_barrier(); // the next chunk overwrites this wave's LDS slices
		}
	}

	// ---- one reduction per workgroup, fixed order: thread 32 * m + l owns output (row m, strip row l) ----
#pragma unroll
	for (int m = 0; m < MR; ++m) {
		red[m][wave][lane] = acc[m];
	}
	__syncthreads();
	if (tid >= MR * STRIP_ROWS) {
		return;
	}
	const int m = tid >> 5, l = tid & 31;
	float total = 0.0f;
#pragma unroll
	for (int w = 0; w < GEMV_WAVES; ++w) {
		total += red[m][w][l] + red[m][w][32 + l];
	}
	const int row = strip * STRIP_ROWS + l;
	float* ym		= y + static_cast<int64_t>(m) * N;
	const float* rm = residual ? residual + static_cast<int64_t>(m) * N : nullptr; // may be ym: read before the write, by the same thread
	if (splits == 1) {
		if (row < N) {
			ym[row] = rm ? total + rm[row] : total;
		}
		return;
	}
	split_k_finish(tagged, epoch, strip * MR + m, splits, split, l, total, ym, row, N, rm);
}

template<int TILES, int MR, bool LOOP> static hipError_t launch_rows_n(const gemv_plan& p, const uint8_t* W, const float* x, float* y, const float* r, int N, const gemv_scratch& sc, hipStream_t s) {
	const dim3 grid(static_cast<unsigned>(p.strips * p.splits)), block(GEMV_WAVES * 64);
	int shift = 0;
	while ((1 << shift) < p.splits) {
		++shift;
	}
	return launch_kernel(KIND_GEMV, gemv_rows_kernel<TILES, MR, LOOP>, grid, block, 0, s, W, x, y, r, sc.tagged, sc.epoch, N, p.groups, shift);
}

template<int MR> static hipError_t launch_rows_m(const gemv_plan& p, const uint8_t* W, const float* x, float* y, const float* r, int N, const gemv_scratch& sc, hipStream_t s) {
	if (p.tiles > 2) {
		return launch_rows_n<2, MR, true>(p, W, x, y, r, N, sc, s);
	}
	return p.tiles <= 1 ? launch_rows_n<1, MR, false>(p, W, x, y, r, N, sc, s) : launch_rows_n<2, MR, false>(p, W, x, y, r, N, sc, s);
}

hipError_t launch_gemv_rows(const void* W, const float* x, float* y, int64_t M, int64_t N, int64_t K, hipStream_t s, const float* residual) {
	const int64_t strips = (N + STRIP_ROWS - 1) / STRIP_ROWS;
	if (strips == 0 || M < 2 || M > GEMV_ROWS_MAX) {
		return M < 2 || M > GEMV_ROWS_MAX ? hipErrorInvalidValue : hipSuccess;
	}
	// K is cut until a wave owns at most two groups (the register budget above); the split scratch holds one unit per
	// (strip, activation row, split)
	gemv_plan p;
	p.strips	   = static_cast<int>(strips);
	p.groups	   = static_cast<int>(K / GROUP_K);
	p.splits	   = 1;
	auto tiles_for = [&](int sp) { return (p.groups + GEMV_WAVES * sp - 1) / (GEMV_WAVES * sp); };
	while (tiles_for(p.splits) > 2 && strips * M * p.splits * 2 <= GEMV_MAX_SPLIT_UNITS) {
		p.splits *= 2;
	}
	// few strips (k/v-sized outputs): keep cutting K while the launch would leave half the CUs without a workgroup and a wave
	// still owns more than one group
	while (strips * p.splits < 128 && tiles_for(p.splits) > 1 && strips * M * p.splits * 2 <= GEMV_MAX_SPLIT_UNITS) {
		p.splits *= 2;
	}
	if (p.splits > 1 && stream_is_capturing(s)) { // replay-safe form: no K split, chunked walk instead
		p.splits = 1;
	}
	p.tiles = tiles_for(p.splits);
	gemv_scratch sc;
	if (p.splits > 1) {
		const hipError_t e = get_gemv_scratch(&sc, true, s);
		if (e != hipSuccess) {
			return e;
		}
	}
	const uint8_t* w = static_cast<const uint8_t*>(W);
	const int n		 = static_cast<int>(N);
	return M == 2 ? launch_rows_m<2>(p, w, x, y, residual, n, sc, s) : launch_rows_m<3>(p, w, x, y, residual, n, sc, s);
}

} // namespace nh
