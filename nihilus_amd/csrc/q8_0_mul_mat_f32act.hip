// fp32 activations against Q8_0 weights WITHOUT quantizing the activations, gfx950:
//   y[m][n] = sum_b f32(d_w[n][b]) * sum_i x[m][32 b + i] * float(q_w[n][b][i])
//
// The one mul_mat with a body in the reference (cpu/avx_2.hpp:4782-4852 leaf, :4978-5004 eval_time and :4854-4976
// prompt_eval_time dispatchers, key <float, block_q8_0<half>, float>).  It is not the path the model runs -- that one
// quantizes the activations and multiplies integers -- and is kept as what it is there: a plain, correct form.  It streams the
// tiled weights like the mat-vec (16 waves per 32-row strip, every weight byte once per activation row), converts the quants
// to fp32 and multiplies in fp32; a lane holds half a block (16 quants) of one weight row and reads the matching 16 activations
// as LDS broadcasts.  One workgroup per (strip, activation row): M rows read the weights M times, which is what the reference's
// loop does too.
#include "q8_0_gemv_tiled.h"

namespace nh {

constexpr int F32ACT_WAVES = 16;

// GC groups per step: every load of the step (weights, scales, activation slice) is issued before the first one is waited
// for, so a wave has GC * 4 KiB in flight; a group past the wave's range repeats the last one (a cache hit, not used).
template<int GC> __global__ __launch_bounds__(F32ACT_WAVES * 64, GC <= 2 ? 8 : 4) void mul_mat_f32act_kernel(const uint8_t* __restrict__ W, const float* __restrict__ x, float* __restrict__ y, int N, int groups, int split_shift,
	uint64_t* __restrict__ tagged, unsigned epoch) {
	__shared__ __align__(16) float xs[F32ACT_WAVES][GC][GROUP_K];
	__shared__ float red[F32ACT_WAVES][64];
	const int tid	= threadIdx.x;
	const int lane	= tid & 63;
	const int wave	= __builtin_amdgcn_readfirstlane(tid >> 6);
	// split_shift > 0 (one activation row only): 1 << split_shift workgroups share a strip's K range and hand their partial
	// sums over as the mat-vec does
	const int splits = 1 << split_shift;
	const int strip	 = static_cast<int>(blockIdx.x >> split_shift);
	const int split	 = static_cast<int>(blockIdx.x) & (splits - 1);
	const int64_t m	 = blockIdx.y;
	const int half	= lane >> 5;
	const int r		= lane & 31;
	int g0, g1;
	wave_k_range(groups, split_shift, split, F32ACT_WAVES, wave, g0, g1);
	const float* xrow	   = x + m * static_cast<int64_t>(groups) * GROUP_K;
	const uint8_t* w_strip = W + macro_offset(strip, 0, groups);
	float acc			   = 0.0f;
	// GC == 2 is launched only where a wave has at most two groups: one step, no loop state
	for (int g = g0; g < g1; g += (GC == 2 ? (1 << 30) : GC)) {
		v4i q[GC][GROUP_BLOCKS];
		v2u dd[GC];
		// the activation slices go from memory straight into LDS, two groups (64 lanes x 16 bytes) per transfer, no registers
#pragma unroll
		for (int c = 0; c < GC; c += 2) {
			const int gg = min(g + c + half, g1 - 1);
			load_global_to_lds_b128(xrow + static_cast<int64_t>(gg) * GROUP_K + 4 * r, &xs[wave][c][0]);
		}
		asm volatile("" ::: "memory"); // the loads below are issued after the transfers
#pragma unroll
		for (int c = 0; c < GC; ++c) {
			dd[c] = __builtin_nontemporal_load(reinterpret_cast<const v2u*>(w_strip + static_cast<int64_t>(min(g + c, g1 - 1)) * MACRO_BYTES + MACRO_D_OFFSET + 8 * r));
		}
#pragma unroll
		for (int c = 0; c < GC; ++c) {
			const uint8_t* macro = w_strip + static_cast<int64_t>(min(g + c, g1 - 1)) * MACRO_BYTES;
#pragma unroll
			for (int j = 0; j < GROUP_BLOCKS; ++j) {
				q[c][j] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(macro + j * TILE_BYTES + 16 * lane));
			}
		}
		// loads complete in issue order: once the first scale load (issued after the transfers) is there, so are the slices; the
		// LDS reads below may not move above this point
		asm volatile("" ::"v"(dd[0].x) : "memory");
#pragma unroll
		for (int c = 0; c < GC; ++c) {
			if (c == 0 || g + c < g1) {
				const float dw[GROUP_BLOCKS] = { half_bits_to_float(static_cast<uint16_t>(dd[c].x & 0xFFFFu)), half_bits_to_float(static_cast<uint16_t>(dd[c].x >> 16)),
					half_bits_to_float(static_cast<uint16_t>(dd[c].y & 0xFFFFu)), half_bits_to_float(static_cast<uint16_t>(dd[c].y >> 16)) };
#pragma unroll
				for (int j = 0; j < GROUP_BLOCKS; ++j) {
					const float* xb = &xs[wave][c][j * QK + 16 * half];
					float s			= 0.0f;
#pragma unroll
					for (int k = 0; k < 4; ++k) {
						const float4 xv = *reinterpret_cast<const float4*>(xb + 4 * k);
						const int word	= q[c][j][k];
						s				= fmaf(xv.x, static_cast<float>(static_cast<int8_t>(word & 0xFF)), s);
						s				= fmaf(xv.y, static_cast<float>(static_cast<int8_t>((word >> 8) & 0xFF)), s);
						s				= fmaf(xv.z, static_cast<float>(static_cast<int8_t>((word >> 16) & 0xFF)), s);
						s				= fmaf(xv.w, static_cast<float>(static_cast<int8_t>((word >> 24) & 0xFF)), s);
					}
					acc = fmaf(s, dw[j], acc);
				}
			}
		}
		asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // this step's LDS reads are done before the next step's transfers overwrite the slices
	}
	red[wave][lane] = acc;
	__syncthreads();
	if (tid < STRIP_ROWS) {
		float total = 0.0f;
#pragma unroll
		for (int w = 0; w < F32ACT_WAVES; ++w) {
			total += red[w][tid] + red[w][32 + tid];
		}
		const int row = strip * STRIP_ROWS + tid;
		if (splits > 1) {
			split_k_finish(tagged, epoch, strip, splits, split, tid, total, y, row, N, nullptr);
		} else if (row < N) {
			y[m * N + row] = total;
		}
	}
}

// K % 128 == 0; M, N > 0 checked by the caller.
hipError_t launch_mul_mat_f32act(const void* W_tiled, const float* x, float* y, int64_t M, int64_t N, int64_t K, hipStream_t s) {
	if (M == 0 || N == 0) {
		return hipSuccess;
	}
	const int strips = static_cast<int>((N + STRIP_ROWS - 1) / STRIP_ROWS);
	const int groups = static_cast<int>(K / GROUP_K);
	// One row: K goes over several workgroups per strip where the mat-vec's plan says so (long rows, few strips), except on a
	// capturing stream (the hand-off's epoch would be the same in every replay).
	int shift		   = 0;
	gemv_scratch sc;
	if (M == 1 && !stream_is_capturing(s)) {
		const gemv_plan p = plan_gemv(strips, K);
		if (p.splits > 1) {
			while ((1 << shift) < p.splits) {
				++shift;
			}
			const hipError_t e = get_gemv_scratch(&sc, true, s);
			if (e != hipSuccess) {
				return e;
			}
		}
	}
	// two groups per step where a wave owns at most two (one step, two workgroups per CU), else four per step
	const int per_split = (groups + (1 << shift) - 1) >> shift; // the longest K range of a workgroup, in groups
	const auto kernel	= (per_split + F32ACT_WAVES - 1) / F32ACT_WAVES <= 2 ? mul_mat_f32act_kernel<2> : mul_mat_f32act_kernel<4>;
	// the grid's second dimension holds at most 65535 rows: walk M in slabs
	for (int64_t m0 = 0; m0 < M; m0 += 65535) {
		const int64_t rows = M - m0 < 65535 ? M - m0 : 65535;
		const hipError_t e = launch_kernel(KIND_GEMV, kernel, dim3(static_cast<unsigned>(strips) << shift, static_cast<unsigned>(rows)), dim3(F32ACT_WAVES * 64), 0, s,
			static_cast<const uint8_t*>(W_tiled), x + m0 * K, y + m0 * N, static_cast<int>(N), groups, shift, sc.tagged, sc.epoch);
		if (e != hipSuccess) {
			return e;
		}
	}
	return hipSuccess;
}

} // namespace nh
