// Which kernel a mul_mat call runs, and how that kernel cuts the work: decided here, on the host, in one place, from the
// shape alone.  The launchers execute the plan they get from these functions and decide nothing themselves, so a test can
// ask (nh_q8_0_debug_plan_mul_mat, no GPU needed) what a shape will run and pin it.
//
// The rules are measurements, not a model: each threshold below names the shapes it was fitted on.  A shape between the
// measured ones follows the nearest rule; the plan says which, so it can at least be seen and tested.
#pragma once
#include "q8_0_gemv_tiled.h"

namespace nh {

// values are part of the debug C entry's contract (include/nihilus_amd/q8_0_abi.h: nh_q8_0_debug_plan_mul_mat)
enum mul_mat_kernel : int {
	MM_NOTHING			= 0, // an empty problem: nothing, or a fill of the output
	MM_GEMV				= 1, // M == 1: quantize inside the streaming mat-vec (gemv_tiled_kernel)
	MM_GEMV_ROWS		= 2, // 2, 3 rows: the streaming mat-vec with one dot product per row (gemv_rows_kernel), quantize inside
	MM_GEMM_SKINNY		= 3, // quantize launch + weight-streaming MFMA kernel (gemm_skinny_kernel)
	MM_GEMM_TILE_STREAM = 4, // quantize launch + MFMA tile kernel with non-temporal weight loads (batched decode on large matrices)
	MM_GEMM_TILE		= 5, // quantize launch + MFMA tile kernel (prefill)
	MM_GEMV_ROWS_MFMA	= 6, // 4..16 rows on small matrices: the streaming mat-vec with the rows as an MFMA operand (gemv_rows8_kernel), quantize inside
};

constexpr int SK_WAVES			  = 8; // waves per workgroup of the weight-streaming MFMA kernel
constexpr int SK_MAX_SPLIT_UNITS  = 2048; // strips * splits when splits > 1
constexpr int SK_MAX_SPLIT_STRIPS = 512;
constexpr int GEMM_SPLIT_MIN_TRIPS = 2; // K goes over more workgroups only while each K set keeps this many 128-quant groups
constexpr int GEMM_STREAM_TILE_MIN_COLUMN_BLOCKS = 192; // 128-row column blocks from which the tile kernel also takes the few-row (batched decode) shapes

// The MFMA tile kernel's cut: TM activation strips per wave; KS sets of four waves per workgroup, each on a share of K (grids
// that would leave SIMDs short of their four waves); with non-temporal weights also K over kz workgroups per tile (grids short
// of one workgroup per CU), their tiles added through the scratch by the last to arrive.
struct gemm_tile_cut {
	int tm, ks, kz;
	unsigned grid_x, grid_y;
};
inline gemm_tile_cut plan_gemm_tile(int64_t M, int64_t N, int64_t K, bool stream) {
	gemm_tile_cut c{};
	const int64_t m_strips = (M + 31) / 32, n_strips = (N + 31) / 32;
	const int groups	   = static_cast<int>(K / GROUP_K);
	// two activation strips per wave whenever there are two: every weight tile fetched is used twice (the one-strip form,
	// with twice the weight loads per MFMA, measured 8 to 60 % slower at M = 512)
	c.tm	 = m_strips >= 2 ? 2 : 1;
	c.grid_x = static_cast<unsigned>((n_strips + 3) / 4);
	c.grid_y = static_cast<unsigned>((m_strips + c.tm - 1) / c.tm);
	c.ks	 = 1;
	while (c.ks < 4 && static_cast<int64_t>(c.grid_x) * c.grid_y * 4 * c.ks * 2 <= 4096 && groups % (c.ks * 2) == 0 && groups / (c.ks * 2) >= 4) {
		c.ks *= 2;
	}
	c.kz = 1;
	if (stream) {
		const int64_t wgs = static_cast<int64_t>(c.grid_x) * c.grid_y;
		while (c.ks == 4 && wgs * c.kz * 2 <= 256 && groups % (c.ks * c.kz * 2) == 0 && groups / (c.ks * c.kz * 2) >= GEMM_SPLIT_MIN_TRIPS &&
			wgs * c.kz * 2 * c.tm * 4096 <= GEMM_SPLIT_SCRATCH_FLOATS && wgs <= GEMM_SPLIT_MAX_UNITS) {
			c.kz *= 2;
		}
	}
	return c;
}

// The weight-streaming MFMA kernel's cut: MS activation strips per workgroup, K of a strip over `splits` workgroups.
struct gemm_skinny_cut {
	int ms, splits;
};
inline gemm_skinny_cut plan_gemm_skinny(int64_t M, int64_t N, int64_t K) {
	gemm_skinny_cut c{};
	const int groups	 = static_cast<int>(K / GROUP_K);
	const int64_t strips = (N + STRIP_ROWS - 1) / STRIP_ROWS, m_strips = (M + STRIP_ROWS - 1) / STRIP_ROWS;
	// Two activation strips per workgroup halve the weight traffic per row, but only pay once the grid fills the chip
	// without them: 64 rows against 128 weight strips are better off as 256 workgroups of one strip each.
	c.ms				= (m_strips <= 1 || strips * ((m_strips + 1) / 2) < 256) ? 1 : 2;
	const int64_t units = strips * ((m_strips + c.ms - 1) / c.ms);
	c.splits			= 1;
	// The hand-off between workgroups is expensive here (a partial tile of 16 values per lane and strip, an arrival counter,
	// the last arriver reading every share): K goes over several workgroups only until every CU has one (and every wave
	// keeps at least two groups, one step of the kernel's walk: [4096 x 4096] at M = 32 12.1 -> 10.8 us, [1024 x 8192] at M = 64
	// 14.9 -> 13.2 us against keeping four), or when a wave would otherwise walk more than sixteen groups.  Measured on
	// [8192 x 28672] at M = 16: 68 us with eight workgroups per strip, 51 us with two.
	while (units * c.splits < 256 && groups >= 4 * SK_WAVES * c.splits && units * c.splits * 2 <= SK_MAX_SPLIT_UNITS && units <= SK_MAX_SPLIT_STRIPS) {
		c.splits *= 2;
	}
	while (groups > 16 * SK_WAVES * c.splits && units * c.splits * 2 <= SK_MAX_SPLIT_UNITS && units <= SK_MAX_SPLIT_STRIPS) {
		c.splits *= 2;
	}
	return c;
}

// A mat-mat on tiled, already quantized operands (nh_q8_0_gemm_tiled, and the second half of nh_q8_0_mul_mat wherever the activations are quantized by a launch of their own).
struct gemm_plan {
	int kernel; // MM_GEMM_SKINNY, MM_GEMM_TILE_STREAM or MM_GEMM_TILE (MM_NOTHING for an empty problem)
	gemm_tile_cut tile; // when a tile kernel runs
	gemm_skinny_cut skinny; // when the streaming kernel runs
};
inline gemm_plan plan_gemm(int64_t M, int64_t N, int64_t K) {
	gemm_plan p{};
	if (M <= 0 || N <= 0 || K <= 0) {
		p.kernel = MM_NOTHING;
		return p;
	}
	// Few rows: the weights are read once and the kernel is HBM-bound.  Somewhat more rows than that, but so few
	// 128-row x 32-row tiles that the tile kernel would leave most SIMDs with one wave or none (measured: it needs
	// more than one workgroup per CU to pay): the same streaming kernel over groups of 64 rows, K split over the
	// waves of a workgroup, the weights coming from cache after the first group.
	const int64_t column_blocks	  = (N + 127) / 128;
	const int64_t tile_workgroups = column_blocks * ((M + 31) / 32);
	const int64_t weights		  = N * K;
	bool stream_tile			  = false;
	if (M <= GEMM_SKINNY_MAX_M) {
		// A matrix with enough 128-row column blocks to occupy the chip by itself takes the tile kernel at any M: its four
		// waves share each activation tile through LDS, where the streaming kernel's eight waves fetch one each from L2 --
		// at 32 to 64 rows that is one to two times the weight bytes in extra traffic into every CU ([28672 x 8192] at
		// M = 16 / 32 / 64: 50 / 55 / 75 us streaming, 44 / 44 / 69 us on the tile kernel; [128256 x 8192]: 193 / - / 298
		// against 182 / - / 221 us).  Below that the tile kernel's grid leaves CUs idle ([14336 x 4096] at M = 64: 30 us
		// against 23 us) and the streaming kernel, which can split K over workgroups, stays.
		if (column_blocks >= GEMM_STREAM_TILE_MIN_COLUMN_BLOCKS) {
			stream_tile = true;
		} else if (M > 32 ? (column_blocks >= 32 && weights >= (48ll << 20)) : (M >= 16 && column_blocks >= 64 && weights >= (64ll << 20))) {
			// Between the two, with K long enough to cut: the tile kernel with K over several workgroups per tile as well, so
			// that 32 to 191 column blocks still put a workgroup on every CU.  Measured against the streaming kernel:
			// [8192 x 28672] M = 64 / 32 / 16: 52 / 46 / 46 against 70 / 52 / 48 us; [8192 x 8192]: 23.7 / 18.0 / 17.6 against
			// 24.1 / 19.0 / 18.4; [14336 x 4096] M = 64: 20.5 against 22.9 (M = 32: 16.8 against 16.2, left where it was);
			// [4096 x 14336] M = 64: 24.0 against 26.2 (M = 16: 19.8 against 18.0); [1024 x 8192] M = 64: 13.5 against 11.7;
			// [4096 x 4096] M = 64: 13.6 against 10.3.  So: two row strips from 48 Mi weights on, one (16 rows or more) from
			// 64 Mi.  The rule only holds where that K split is actually possible: a shape whose groups do not divide (kz
			// stays 1) would run the tile kernel on 32 to 191 workgroups, the form measured slower than the streaming kernel
			// ([14336 x 4096] at M = 64 unsplit: 30 against 23 us), and stays with the streaming kernel.
			stream_tile = plan_gemm_tile(M, N, K, true).kz > 1;
		}
	}
	if (stream_tile) {
		p.kernel = MM_GEMM_TILE_STREAM;
		p.tile	 = plan_gemm_tile(M, N, K, true);
	} else if (M <= GEMM_SKINNY_MAX_M || tile_workgroups <= 256) {
		p.kernel = MM_GEMM_SKINNY;
		p.skinny = plan_gemm_skinny(M, N, K);
	} else {
		p.kernel = MM_GEMM_TILE;
		p.tile	 = plan_gemm_tile(M, N, K, false);
	}
	return p;
}

// The prefill FFN's gate and up mat-mats with SiLU * up and the quantizer behind them: one launch of the tile kernel's fused form
// where each matrix alone would take the prefill tile kernel and the doubled grid runs one K set per workgroup; otherwise the two
// mat-mats and the quantizer as launches of their own (through an fp32 workspace).
inline bool plan_gate_up_fused(int64_t M, int64_t n_ff, int64_t K, gemm_tile_cut* cut = nullptr) {
	if (M <= 0 || n_ff <= 0 || K <= 0 || n_ff % GROUP_K != 0 || K % GROUP_K != 0) {
		return false;
	}
	if (plan_gemm(M, n_ff, K).kernel != MM_GEMM_TILE) {
		return false;
	}
	const gemm_tile_cut c = plan_gemm_tile(M, 2 * n_ff, K, false); // grid_x = n_ff / 64 workgroups of two gate and two up strips
	if (c.ks != 1) {
		return false;
	}
	if (cut) {
		*cut = c;
	}
	return true;
}

// The MFMA mat-vec's cut (q8_0_gemv_rows_mfma.hip): K over workgroups until a wave owns at most two groups (one with the
// sixteen-row operand: its register budget), within the split scratch's units (one per strip, activation row and split); matrices with few strips are cut
// further so that the launch reaches the CUs.  Under HIP graph capture: no K split (a replay could not renew the hand-off's epoch),
// a chunked walk instead.
constexpr int GEMV_ROWS_MFMA_MAX = 16;
// Where it is the fastest form (measured against what ran before, quantize launch included; us, new / old):
//   [4096 x 4096]   17.8 MB   M = 4:  5.2 /  8.1 (dot-product kernel)   M = 8:  6.8 / 12.2   M = 16:  8.6 / 11.7 (quantize + streaming MFMA kernel)
//   [1024 x 8192]    8.9 MB   M = 4:  5.6 /  7.3                        M = 16:  9.1 / 14.3
//   [14336 x 4096]  62.4 MB   M = 4: 13.7 / 15.6                        M = 8:  19.3 / 15.7
//   [8192 x 8192]   71.3 MB   M = 4: 17.4 / 21.2
//   [28672 x 8192]   250 MB   M = 4: 51   / 43.6;  [128256 x 8192]: 199 / 167
// Every strip's workgroup quantizes all the rows again, which costs in proportion to M and to the matrix: up to sixteen rows on
// matrices of at most 40 MB, four on matrices of at most 80 MB.  (Two and three rows stay on the dot-product kernel.)
inline bool gemv_rows_mfma_suits(int64_t M, int64_t N, int64_t K) {
	const int64_t weight_bytes = N * (K / QK) * BLOCK_BYTES;
	return M >= 4 && M <= GEMV_ROWS_MFMA_MAX && (weight_bytes <= (int64_t{ 40 } << 20) || (M == 4 && weight_bytes <= (int64_t{ 80 } << 20)));
}
inline gemv_plan plan_gemv_rows_mfma(int64_t strips, int64_t K, int rows, bool capturing) { // rows: 8 or 16, the kernel's operand rows
	gemv_plan p;
	p.strips	   = static_cast<int>(strips);
	p.groups	   = static_cast<int>(K / GROUP_K);
	p.splits	   = 1;
	auto tiles_for = [&](int sp) { return (p.groups + GEMV_WAVES * sp - 1) / (GEMV_WAVES * sp); };
	auto room	   = [&](int sp) { return strips * rows * sp <= GEMV_MAX_SPLIT_UNITS; };
	const int fit  = rows <= 8 ? 2 : 1; // groups of a wave's K range that its registers hold at once
	while (tiles_for(p.splits) > fit && room(p.splits * 2)) {
		p.splits *= 2;
	}
	// (a workgroup per CU, not per two as in the dot-product kernel: every workgroup quantizes its K range of all the rows, and that
	// work is what the launch waits for -- [4096 x 4096] at 8 rows: 9.8 us with 128 workgroups, 7.5 us with 256)
	while (strips * p.splits < 256 && tiles_for(p.splits) > 1 && room(p.splits * 2)) {
		p.splits *= 2;
	}
	if (capturing) {
		p.splits = 1;
	}
	p.tiles = tiles_for(p.splits);
	return p;
}

// nh_q8_0_mul_mat: fp32 activations [M][K] against a tiled weight [N][K].
struct mul_mat_plan {
	int kernel; // mul_mat_kernel
	int quantize_launch; // 1: the activations are quantized by a launch of their own into the caller's workspace
	gemv_plan gemv; // MM_GEMV, MM_GEMV_ROWS: strips, groups, K splits, groups per wave
	int gemv_row_parts; // MM_GEMV: workgroups that share a strip by rows (unsplit launches with fewer strips than CUs)
	gemm_plan gemm; // the MFMA kernels
};
// row parts per strip of an unsplit mat-vec launch: fewer strips than CUs (the 4096-row projections have 128, k/v 32) are cut
// into 2 or 4 row parts so that the launch reaches that many more CUs; what a single CU takes in per microsecond is limited,
// so half a chip cannot stream at the full HBM rate however many loads it has in flight.  (Between 129 and 255 strips -- q+k+v's 192 --
// two parts measured slower: 8.3 against 7.1 us with the norm in front.)
inline int plan_gemv_row_parts(const gemv_plan& p) {
	if (p.splits != 1 || p.tiles > 4) {
		return 1;
	}
	return p.strips * 2 <= 256 ? (p.strips * 4 <= 256 ? 4 : 2) : 1;
}
inline mul_mat_plan plan_mul_mat(int64_t M, int64_t N, int64_t K) {
	mul_mat_plan p{};
	if (M <= 0 || N <= 0 || K <= 0) {
		p.kernel = MM_NOTHING;
		return p;
	}
	if (M == 1) {
		p.kernel		 = MM_GEMV;
		p.gemv			 = plan_gemv((N + STRIP_ROWS - 1) / STRIP_ROWS, K);
		p.gemv_row_parts = plan_gemv_row_parts(p.gemv);
		return p;
	}
	if (gemv_rows_mfma_suits(M, N, K)) {
		p.kernel		 = MM_GEMV_ROWS_MFMA;
		p.gemv			 = plan_gemv_rows_mfma((N + STRIP_ROWS - 1) / STRIP_ROWS, K, M <= 8 ? 8 : 16, false);
		p.gemv_row_parts = 1;
		return p;
	}
	if (gemv_rows_suits(M, N, K)) {
		p.kernel		 = MM_GEMV_ROWS;
		p.gemv_row_parts = 1;
		return p;
	}
	p.quantize_launch = 1;
	p.gemm			  = plan_gemm(M, N, K);
	p.kernel		  = p.gemm.kernel;
	return p;
}

} // namespace nh
