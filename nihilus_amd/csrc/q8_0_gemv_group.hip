// Several INDEPENDENT mat-vecs as one launch: y_i = W_i . Q(x_i), each with its own activation row, K and N, gfx950.
//
// A decode-sized mat-vec is a few tens of MB: 8-17 us of HBM time behind ~2 us in which the chip fills with
// workgroups and the first bytes arrive, and ~1 us in which the last sums are reduced and handed over.  Mat-vecs that
// share their activation row already run as one launch (q/k/v, gate/up: gemv_tiled_kernel's segments).  This kernel
// does the same for mat-vecs that share nothing, provided none of them reads or overwrites what another one writes
// (the caller, or the batch runner's hazard check, vouches for that): the workgroups of all of them form one grid, so
// the ramp and the tail are paid once per group instead of once per matrix.
//
// Every matrix keeps the cut it would have as a launch of its own (plan_gemv on its strips and K: workgroups per
// strip, groups per wave, K ranges), so its result is the one the single launch gives, bit for bit, whenever that
// launch would not use the row split.  The activation quantize is inside, as in the single launch.
#include "q8_0_gemv_tiled.h"

namespace nh {

struct gemv_group {
	const uint8_t* W[GEMV_GROUP_MAX];
	const float* x[GEMV_GROUP_MAX];
	float* y[GEMV_GROUP_MAX];
	const float* residual[GEMV_GROUP_MAX];
	int rows[GEMV_GROUP_MAX];
	int groups[GEMV_GROUP_MAX]; // K / 128
	int split_shift[GEMV_GROUP_MAX]; // workgroups per strip = 1 << split_shift
	int wg_end[GEMV_GROUP_MAX]; // running total of workgroups
	int unit0[GEMV_GROUP_MAX]; // the matrix's first (strip, split) slot in the tagged partial sums
};

template<int TILES> __global__ __launch_bounds__(GEMV_WAVES * 64) void gemv_group_kernel(gemv_group g, uint64_t* __restrict__ tagged, unsigned epoch) {
	__shared__ __align__(16) uint8_t xs_q[GEMV_WAVES][TILES * GROUP_K];
	__shared__ float xs_d[GEMV_WAVES][TILES * GROUP_BLOCKS];
	__shared__ float red[GEMV_WAVES][64];
	const int tid  = threadIdx.x;
	const int lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int wg   = static_cast<int>(blockIdx.x);
	int m		   = 0; // which matrix (all scalar)
#pragma unroll
	for (int i = 0; i < GEMV_GROUP_MAX - 1; ++i) {
		m += wg >= g.wg_end[i] ? 1 : 0;
	}
	const int local	 = wg - (m == 0 ? 0 : g.wg_end[m - 1]);
	const int shift	 = g.split_shift[m];
	const int splits = 1 << shift;
	const int strip	 = local >> shift;
	const int split	 = local & (splits - 1);
	const int groups = g.groups[m];
	const int N		 = g.rows[m];
	int g0, g1;
	wave_k_range(groups, shift, split, GEMV_WAVES, wave, g0, g1);

	const uint8_t* w_strip = g.W[m] + macro_offset(strip, 0, groups);
	const int row_l		   = strip * STRIP_ROWS + (lane & 31);
	// the host only groups matrices whose waves own at most TILES groups: every load of the wave in flight at once
	const float acc = gemv_chunk<TILES, X_F32, DUMP_NONE>(w_strip, g.x[m], nullptr, xs_q[wave], xs_d[wave], g0, g1 - g0, groups, lane, row_l, N, false);

	red[wave][lane] = acc;
	__syncthreads();
	float total = 0.0f;
	if (tid < STRIP_ROWS) {
#pragma unroll
		for (int w = 0; w < GEMV_WAVES; ++w) {
			total += red[w][tid] + red[w][32 + tid];
		}
	}
	const int row	 = strip * STRIP_ROWS + tid;
	float* y		 = g.y[m];
	const float* res = g.residual[m];
	if (splits == 1) {
		if (tid < STRIP_ROWS && row < N) {
			y[row] = res ? total + res[row] : total;
		}
		return;
	}
	if (tid < STRIP_ROWS) {
		split_k_finish(tagged + static_cast<int64_t>(g.unit0[m]) * STRIP_ROWS, epoch, strip, splits, split, tid, total, y, row, N, res);
	}
}

// The cut of one matrix inside a group, or splits = 0 when it cannot join one (a wave would own more than four groups:
// long K on a capturing stream, or more strips than the K split serves).
static gemv_plan plan_for_group(int64_t N, int64_t K, bool capturing) {
	gemv_plan p = plan_gemv((N + STRIP_ROWS - 1) / STRIP_ROWS, K);
	if (p.splits > 1 && capturing) {
		p.splits = 1;
		p.tiles	 = (p.groups + GEMV_WAVES - 1) / GEMV_WAVES;
	}
	if (p.tiles > 4) {
		p.splits = 0;
	}
	return p;
}

// count in [1, GEMV_GROUP_MAX]; every op: N > 0, K > 0, K % 128 == 0, gemv_can_group(N, K).  The ops must be independent.
hipError_t launch_gemv_group(const gemv_group_op* ops, int count, hipStream_t s) {
	const bool capturing = stream_is_capturing(s);
	if (count < 1 || count > GEMV_GROUP_MAX) {
		return hipErrorInvalidValue;
	}
	// Matrices whose K is split over workgroups go first: their partial sums are handed over while the others still stream,
	// instead of at the very end of the launch with nothing left to overlap the hand-off.
	gemv_plan plans[GEMV_GROUP_MAX];
	int order[GEMV_GROUP_MAX];
	int n = 0;
	for (int pass = 0; pass < 2; ++pass) {
		for (int i = 0; i < count; ++i) {
			if (pass == 0) {
				plans[i] = plan_for_group(ops[i].N, ops[i].K, capturing);
				if (plans[i].splits <= 0) {
					return hipErrorInvalidValue;
				}
			}
			if ((plans[i].splits > 1) == (pass == 0)) {
				order[n++] = i;
			}
		}
	}
	gemv_group g{};
	int wgs = 0, units = 0, tiles = 1;
	for (int j = 0; j < GEMV_GROUP_MAX; ++j) {
		if (j < count) {
			const gemv_group_op& o = ops[order[j]];
			const gemv_plan& p	   = plans[order[j]];
			int shift			   = 0;
			while ((1 << shift) < p.splits) {
				++shift;
			}
			g.W[j]			 = static_cast<const uint8_t*>(o.W);
			g.x[j]			 = o.x;
			g.y[j]			 = o.y;
			g.residual[j]	 = o.residual;
			g.rows[j]		 = static_cast<int>(o.N);
			g.groups[j]		 = p.groups;
			g.split_shift[j] = shift;
			g.unit0[j]		 = units;
			wgs += p.strips * p.splits;
			if (p.splits > 1) {
				units += p.strips * p.splits;
			}
			tiles = p.tiles > tiles ? p.tiles : tiles;
		}
		g.wg_end[j] = wgs;
	}
	if (units > GEMV_MAX_SPLIT_UNITS) {
		return hipErrorInvalidValue;
	}
	gemv_scratch sc;
	if (units > 0) {
		const hipError_t e = get_gemv_scratch(&sc, true, s);
		if (e != hipSuccess) {
			return e;
		}
	}
	const dim3 grid(static_cast<unsigned>(wgs)), block(GEMV_WAVES * 64);
	if (tiles <= 2) {
		return launch_kernel(KIND_GEMV, gemv_group_kernel<2>, grid, block, 0, s, g, sc.tagged, sc.epoch);
	}
	return launch_kernel(KIND_GEMV, gemv_group_kernel<4>, grid, block, 0, s, g, sc.tagged, sc.epoch);
}

// Any number of independent mat-vecs in as few launches as their shapes allow: runs of groupable ones go out as groups
// of up to GEMV_GROUP_MAX (and within the scratch's partial-sum slots), the rest one by one.  A lone matrix takes the
// single launch, which may cut a small one by rows.
hipError_t launch_gemv_independent(const gemv_group_op* ops, int64_t count, hipStream_t s) {
	const bool capturing = stream_is_capturing(s);
	auto single			 = [&](const gemv_group_op& o) {
		 const void* w[1]  = { o.W };
		 float* y[1]	   = { o.y };
		 const float* r[1] = { o.residual };
		 return o.N > 0 ? launch_gemv_tiled_multi(w, y, &o.N, 1, o.x, true, o.K, s, nullptr, 0.0f, o.residual ? r : nullptr) : hipSuccess;
	};
	int64_t i = 0;
	while (i < count) {
		int n = 0, units = 0;
		while (i + n < count && n < GEMV_GROUP_MAX) {
			const gemv_group_op& o = ops[i + n];
			if (o.N <= 0 || o.K <= 0) {
				break;
			}
			const gemv_plan p = plan_for_group(o.N, o.K, capturing);
			const int u		  = p.splits > 1 ? p.strips * p.splits : 0;
			if (p.splits <= 0 || units + u > GEMV_MAX_SPLIT_UNITS) {
				break;
			}
			units += u;
			++n;
		}
		const hipError_t e = n >= 2 ? launch_gemv_group(ops + i, n, s) : single(ops[i]);
		if (e != hipSuccess) {
			return e;
		}
		i += n >= 2 ? n : 1;
	}
	return hipSuccess;
}

} // namespace nh
