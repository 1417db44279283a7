// The decode-time FFN as ONE launch: y = W_down . Q(silu(W_gate . Q(x)) * (W_up . Q(x))) [+ residual], gfx950.
//
// Stands for the eval_time body of the reference's mega_ffn core (ffn_gate/ffn_up mul_mat -> silu -> mul -> ffn_down
// mul_mat -> residual add, infra/core_traits.hpp:971-995; its GPU dispatcher is empty, cuda/cuda_12.hpp:806-916).
// Every Q() is quantize_row_q8_0 done inside the consuming mat-vec, so no activation is ever written in quantized form.
//
// Why one launch: the three mat-vecs are HBM-bound and each launch pays a ramp (first bytes ~2 us after the launch
// starts) and a tail (the last workgroups run on a mostly idle chip).  Here the workgroups of the down projection are
// part of the same grid, placed after those of gate and up.  A down-projection wave puts all its weight loads in flight
// the moment it starts -- while gate/up workgroups are still streaming -- and only then waits for the activation
// blocks that cover its slice, so HBM never idles between the two phases.
//
// A producer workgroup computes the SAME 32-row strip of gate (waves 0-7) and of up (waves 8-15): those 32 + 32 outputs
// are exactly what one 32-value block of the down projection's activation needs, so the producer applies silu(g) * u,
// quantizes the block (the quantize kernel's arithmetic) and publishes 34 bytes; consumers never evaluate an exp and
// read 1/7.5 of what the fp32 vectors would cost them.
//
// Progress: workgroups are dispatched in index order within each XCD's share of the grid, and producers all precede
// consumers, so a waiting consumer never keeps a producer from being scheduled; producers wait for nothing.  The wait
// is bounded all the same (see gemv_chunk).  Hand-off: a producer publishes its block as nine 64-bit words, each the
// launch's epoch beside 32 bits of the block, with device-scope stores; a consumer reads the words of its slice until
// all carry the epoch.  One trip through memory each way (with a flag beside the data it was two each way, and under
// the weight stream every trip costs 2-3 us); nothing is reset between launches (epochs only move forward).
#include "q8_0_gemv_tiled.h"

namespace nh {

struct ffn_args {
	const uint8_t* w_gate;
	const uint8_t* w_up;
	const uint8_t* w_down;
	const float* x; // [K]
	const float* norm_w; // [K] or null: RMS norm * weight applied to x in front of the gate/up quantizer
	float norm_eps;
	const float* residual; // [n_out] or null
	float* y; // [n_out]
	float* gate_up; // scratch: g at [0, n_ff), u at [FFN_MAX_HIDDEN, FFN_MAX_HIDDEN + n_ff), kept for inspection
	uint64_t* act_words; // scratch: the activation, PUBLISHED_WORDS {epoch, payload} words per block
	unsigned epoch;
	uint64_t* tagged; // scratch: tagged partial sums of the down projection's K split
	int n_ff, n_out;
	int groups_p, groups_c; // K / 128, n_ff / 128
	int producers; // n_ff / 32
	int p_per_slot, p_rem; // a producer strip's K range over the 8 waves of one matrix
	int split_shift; // a consumer strip's K range goes over (1 << split_shift) workgroups of 16 waves
	unsigned* error_word; // device-visible host word: set when a consumer gives up waiting for a producer
	int spin_limit; // polls before it does
	uint64_t* x_words; // scratch (NORM): the normalised, quantized input row, published by the first producer workgroup for the others; null: each works it out
};

// PAIR: every producer wave takes a K range of BOTH matrices (the strip's rows of gate and of up against one staged slice of
// the input row), sixteen ranges per workgroup, instead of eight waves per matrix each staging the same eight slices: the row
// (and the norm weights) are fetched and quantized once per workgroup instead of twice.  For K up to 2 groups per wave.
template<int TILES, bool LOOP, bool NORM, bool PAIR = false> __global__ __launch_bounds__(GEMV_WAVES * 64) void ffn_decode_kernel(ffn_args a) {
	__shared__ __align__(16) uint8_t xs_q[GEMV_WAVES][TILES * GROUP_K];
	__shared__ float xs_d[GEMV_WAVES][TILES * GROUP_BLOCKS];
	__shared__ float red[GEMV_WAVES][64];
	__shared__ float red_up[PAIR ? GEMV_WAVES : 1][64];

	const int tid  = threadIdx.x;
	const int lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int wg   = static_cast<int>(blockIdx.x);

	if (wg < a.producers) {
		// ---- rows [32 * wg, 32 * wg + 32) of gate (waves 0-7) and of up (waves 8-15) -> activation block wg ----
		__shared__ __align__(16) float act_f[STRIP_ROWS];
		__shared__ float norm_red[16];
		__shared__ float4 xs_w[NORM ? GEMV_WAVES : 1][NORM ? TILES * 32 : 1];
		const int matrix	   = PAIR ? 0 : wave >> 3;
		const int slot		   = PAIR ? wave : wave & 7;
		const int strip		   = wg;
		const int g0		   = slot * a.p_per_slot + min(slot, a.p_rem);
		const int g1		   = g0 + a.p_per_slot + (slot < a.p_rem ? 1 : 0);
		const uint8_t* w_strip = (matrix ? a.w_up : a.w_gate) + macro_offset(strip, 0, a.groups_p);
		const uint8_t* w_other = PAIR ? a.w_up + macro_offset(strip, 0, a.groups_p) : nullptr;
		const int row_l		   = strip * STRIP_ROWS + (lane & 31);
		float acc			   = 0.0f;
		[[maybe_unused]] float acc_up = 0.0f;
		auto walk = [&]<int XMODE, bool WITH_NORM>(const void* x_from, void* dump_to, gemv_norm* norm) {
			if constexpr (PAIR) {
				return gemv_chunk<2, XMODE, DUMP_NONE, WITH_NORM, 1, 2>(w_strip, x_from, dump_to, xs_q[wave], xs_d[wave], g0, g1 - g0, a.groups_p, lane, row_l, a.n_ff, false, a.epoch, norm, 0, a.spin_limit,
					w_other, &acc_up);
			} else if constexpr (!LOOP) {
				return gemv_chunk<TILES, XMODE, DUMP_NONE, WITH_NORM>(w_strip, x_from, dump_to, xs_q[wave], xs_d[wave], g0, g1 - g0, a.groups_p, lane, row_l, a.n_ff, false, a.epoch, norm, 0, a.spin_limit);
			} else {
				float sum = 0.0f;
				for (int gc = g0; gc < g1; gc += TILES) {
					sum += gemv_chunk<TILES, XMODE, DUMP_NONE, WITH_NORM>(w_strip, x_from, dump_to, xs_q[wave], xs_d[wave], gc, min(TILES, g1 - gc), a.groups_p, lane, row_l, a.n_ff, false, a.epoch, norm, 0,
						a.spin_limit);
					__builtin_amdgcn_wave_barrier();
				}
				return sum;
			}
		};
		if constexpr (NORM) {
			// one row, one norm: the first producer workgroup works the normalised, quantized row out (its gate waves cover all of K
			// between them and publish what they stage), the others read it from there
			if (!a.x_words || wg == 0) {
				gemv_norm norm_state; // the row's scale first (a workgroup barrier inside)
				gemv_norm_begin(norm_state, a.x, a.norm_w, xs_w[NORM ? wave : 0], norm_red, a.norm_eps, a.groups_p * GROUP_K, lane, wave);
				norm_state.publish = matrix == 0 ? a.x_words : nullptr;
				norm_state.epoch   = a.epoch;
				acc				   = walk.template operator()<X_F32, true>(a.x, nullptr, &norm_state);
			} else {
				acc = walk.template operator()<X_PUBLISHED_EARLY_WATCH, false>(a.x_words, a.error_word, nullptr);
			}
		} else if constexpr (PAIR) {
			acc = walk.template operator()<X_F32, false>(a.x, nullptr, nullptr);
		} else if constexpr (!LOOP) {
			acc = gemv_chunk<TILES, X_F32, DUMP_NONE, false>(w_strip, a.x, nullptr, xs_q[wave], xs_d[wave], g0, g1 - g0, a.groups_p, lane, row_l, a.n_ff, false, 0, nullptr);
		} else {
			for (int gc = g0; gc < g1; gc += TILES) {
				acc += gemv_chunk<TILES, X_F32, DUMP_NONE, false>(w_strip, a.x, nullptr, xs_q[wave], xs_d[wave], gc, min(TILES, g1 - gc), a.groups_p, lane, row_l, a.n_ff, false, 0, nullptr);
				__builtin_amdgcn_wave_barrier();
			}
		}
		if constexpr (PAIR) {
			red_up[wave][lane] = acc_up;
		}
		red[wave][lane] = acc;
		__syncthreads();
		if (wave == 0) {
			if (lane < STRIP_ROWS) {
				float g = 0.0f, u = 0.0f;
				if constexpr (PAIR) {
#pragma unroll
					for (int w = 0; w < GEMV_WAVES; ++w) {
						g += red[w][lane] + red[w][32 + lane];
						u += red_up[w][lane] + red_up[w][32 + lane];
					}
				} else {
#pragma unroll
					for (int w = 0; w < GEMV_WAVES / 2; ++w) {
						g += red[w][lane] + red[w][32 + lane];
						u += red[GEMV_WAVES / 2 + w][lane] + red[GEMV_WAVES / 2 + w][32 + lane];
					}
				}
				act_f[lane]									 = silu_mul(g, u);
				a.gate_up[strip * STRIP_ROWS + lane]				 = g; // inspection copies, not read by this launch
				a.gate_up[FFN_MAX_HIDDEN + strip * STRIP_ROWS + lane] = u;
			}
			__builtin_amdgcn_wave_barrier();
			// the block as eight float4 in lanes 0..7; every lane runs the quantizer (lanes 8.. on zeros)
			const float4 v = lane < 8 ? *reinterpret_cast<const float4*>(&act_f[4 * lane]) : make_float4(0.f, 0.f, 0.f, 0.f);
			uint16_t dh;
			const uint32_t packed = quantize_block_lane(v, &dh);
			// lanes 0..7 hold the quants and the block's scale; lane 8 stores the scale: nine self-tagged words, no
			// acknowledgement to wait for
			const uint32_t d_bits = __builtin_amdgcn_readfirstlane(__float_as_uint(half_bits_to_float(dh)));
			if (lane <= 8) {
				const uint32_t payload = lane < 8 ? packed : d_bits;
				__hip_atomic_store(&a.act_words[strip * PUBLISHED_WORDS + lane], (static_cast<uint64_t>(a.epoch) << 32) | payload, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
			}
		}
		return;
	}

	// ---- a (32-row strip, K split) of the down projection; its activation blocks come from the producers ----
	const int c		 = wg - a.producers;
	const int splits = 1 << a.split_shift;
	// K part first, strip second: the workgroups of the first K part come first in dispatch order, and their activation blocks come
	// from the first producers, which are done by the time these start; ordered strip first, every other early workgroup held its
	// CU waiting for the last producers (measured at the LLaMA-3-8B shapes: 30.9 -> 30.55 us, with the norm 33.15 -> 32.5 us; at the
	// LLaMA-3-70B shapes, four K parts, 113.8 -> 109.6 us; K
	// over four or eight parts instead of two, ordered either way, measured 31.7 and 32.6 to 34.4 us; uneven parts -- 40/40/32,
	// 64/48, 32/40/40 of the 112 groups and others -- 31.0 to 32.7 us)
	const int strips_c = (a.n_out + STRIP_ROWS - 1) / STRIP_ROWS;
	const int split	   = c / strips_c;
	const int gstrip   = c - split * strips_c;
	int g0, g1;
	wave_k_range(a.groups_c, a.split_shift, split, GEMV_WAVES, wave, g0, g1);

	const uint8_t* w_strip = a.w_down + macro_offset(gstrip, 0, a.groups_c);
	const int row_l		   = gstrip * STRIP_ROWS + (lane & 31);
	float acc			   = 0.0f;
	if constexpr (!LOOP) {
		acc = gemv_chunk<TILES, X_PUBLISHED, DUMP_NONE>(w_strip, a.act_words, a.error_word, xs_q[wave], xs_d[wave], g0, g1 - g0, a.groups_c, lane, row_l, a.n_out, false, a.epoch, nullptr, 0, a.spin_limit);
	} else {
		for (int gc = g0; gc < g1; gc += TILES) {
			acc += gemv_chunk<TILES, X_PUBLISHED, DUMP_NONE>(w_strip, a.act_words, a.error_word, xs_q[wave], xs_d[wave], gc, min(TILES, g1 - gc), a.groups_c, lane, row_l, a.n_out, false, a.epoch, nullptr, 0, a.spin_limit);
			__builtin_amdgcn_wave_barrier();
		}
	}

	red[wave][lane] = acc;
	__syncthreads();
	float total = 0.0f;
	if (tid < STRIP_ROWS) {
#pragma unroll
		for (int w = 0; w < GEMV_WAVES; ++w) {
			total += red[w][tid] + red[w][32 + tid];
		}
	}
	const int row = gstrip * STRIP_ROWS + tid;
	if (splits == 1) {
		if (tid < STRIP_ROWS && row < a.n_out) {
			a.y[row] = a.residual ? total + a.residual[row] : total;
		}
		return;
	}
	// K split over several workgroups: as in the plain mat-vec
	if (tid < STRIP_ROWS) {
		split_k_finish(a.tagged, a.epoch, gstrip, splits, split, tid, total, a.y, row, a.n_out, a.residual);
	}
}

// an empty inner dimension anywhere makes the activation zero: y = residual (or 0)
__global__ void ffn_empty_kernel(float* __restrict__ y, const float* __restrict__ residual, int64_t n) {
	const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
	if (i < n) {
		y[i] = residual ? residual[i] : 0.0f;
	}
}

template<int TILES, bool LOOP, bool PAIR = false> static hipError_t launch_ffn_t(const ffn_args& a, unsigned grid, hipStream_t s) {
	if (a.norm_w) {
		return launch_kernel(KIND_GEMV, ffn_decode_kernel<TILES, LOOP, true, PAIR>, dim3(grid), dim3(GEMV_WAVES * 64), 0, s, a);
	}
	return launch_kernel(KIND_GEMV, ffn_decode_kernel<TILES, LOOP, false, PAIR>, dim3(grid), dim3(GEMV_WAVES * 64), 0, s, a);
}

// n_ff % 128 == 0, K % 128 == 0, n_ff <= FFN_MAX_HIDDEN (checked by the caller).
hipError_t launch_ffn_decode(const void* w_gate, const void* w_up, const void* w_down, const float* x, const float* norm_w, float norm_eps, const float* residual, float* y, int64_t n_ff,
	int64_t K, int64_t n_out, hipStream_t s) {
	if (n_out == 0) {
		return hipSuccess;
	}
	if (n_ff == 0 || K == 0) {
		ffn_empty_kernel<<<dim3(static_cast<unsigned>((n_out + 255) / 256)), dim3(256), 0, s>>>(y, residual, n_out);
		return hipGetLastError();
	}
	gemv_scratch sc;
	const hipError_t e = get_gemv_scratch(&sc, true, s);
	if (e != hipSuccess) {
		return e;
	}
	if (stream_is_capturing(s) || !in_kernel_waits_enabled()) {
		// (Also what a caller gets who has switched waits between the workgroups of a launch off.)
		// A replayed graph runs the kernel with the epoch it was captured with, so the published blocks of one replay would
		// pass for those of the next.  Under capture the step is three launches instead, none of which keeps state between
		// launches: gate/up mat-vecs (norm inside) -> SiLU * up -> quantize -> down mat-vec (+ residual).  The gate / up
		// values land where the one-launch form leaves its inspection copies.
		const void* w2[2] = { w_gate, w_up };
		float* y2[2]	  = { sc.gate_up, sc.gate_up + FFN_MAX_HIDDEN };
		const int64_t n2[2] = { n_ff, n_ff };
		hipError_t e2		= launch_gemv_tiled_multi(w2, y2, n2, 2, x, true, K, s, norm_w, norm_eps);
		if (e2 != hipSuccess) {
			return e2;
		}
		e2 = launch_silu_mul_quantize(sc.gate_up, sc.gate_up + FFN_MAX_HIDDEN, sc.act_blocks, 1, n_ff, false, s);
		if (e2 != hipSuccess) {
			return e2;
		}
		const void* w1[1]		= { w_down };
		float* y1[1]			= { y };
		const float* r1[1]		= { residual };
		return launch_gemv_tiled_multi(w1, y1, &n_out, 1, sc.act_blocks, false, n_ff, s, nullptr, 0.0f, r1);
	}
	// the down projection: K over as many workgroups per strip as it takes for a wave to own at most 4 groups
	const int strips_c = static_cast<int>((n_out + STRIP_ROWS - 1) / STRIP_ROWS);
	const int groups_c = static_cast<int>(n_ff / GROUP_K);
	int splits		   = 1;
	auto tiles_for	   = [&](int sp) { return (groups_c + GEMV_WAVES * sp - 1) / (GEMV_WAVES * sp); };
	while (tiles_for(splits) > 4 && strips_c <= GEMV_MAX_SPLIT_STRIPS && strips_c * splits * 2 <= GEMV_MAX_SPLIT_UNITS) {
		splits *= 2;
	}
	ffn_args a{};
	a.w_gate	 = static_cast<const uint8_t*>(w_gate);
	a.w_up		 = static_cast<const uint8_t*>(w_up);
	a.w_down	 = static_cast<const uint8_t*>(w_down);
	a.x			 = x;
	a.norm_w	 = norm_w;
	a.norm_eps	 = norm_eps;
	a.residual	 = residual;
	a.y			 = y;
	a.gate_up	 = sc.gate_up;
	a.act_words	 = sc.act_words;
	a.epoch		 = sc.epoch;
	a.tagged	 = sc.tagged;
	a.error_word = sc.error_word;
	a.spin_limit = sc.spin_limit;
	a.n_ff		 = static_cast<int>(n_ff);
	a.n_out		 = static_cast<int>(n_out);
	a.groups_p	 = static_cast<int>(K / GROUP_K);
	a.groups_c	 = groups_c;
	a.producers	 = static_cast<int>(n_ff / STRIP_ROWS);
	a.x_words	 = norm_w && a.producers >= FFN_SHARED_X_MIN_PRODUCERS && K <= GEMV_SHARED_X_MAX_K ? sc.x_words : nullptr;
	// up to two groups per wave when the row is cut sixteen ways: every producer wave takes both matrices (PAIR)
	// ... where the eight-and-eight form would need the four-group kernel anyway (the two-group kernel fits two workgroups per
	// CU and is left alone), and not with the chunked walk
	const int tiles_8_8 = (a.groups_p + GEMV_WAVES / 2 - 1) / (GEMV_WAVES / 2);
	// Measured at the LLaMA-3-8B shapes: with the norm in front 34.2 -> 33.1 us (the row AND the norm weights once instead of twice
	// per workgroup), without it 31.2 -> 31.3 us (the row alone stays in the CU's L1 between the two halves): used with a norm only.
	const bool pair		= norm_w && (a.groups_p + GEMV_WAVES - 1) / GEMV_WAVES <= 2 && tiles_for(splits) <= 4 && (tiles_8_8 > 2 || tiles_for(splits) > 2);
	const int p_slots  = pair ? GEMV_WAVES : GEMV_WAVES / 2;
	a.p_per_slot	   = a.groups_p / p_slots;
	a.p_rem			   = a.groups_p % p_slots;
	int shift	 = 0;
	while ((1 << shift) < splits) {
		++shift;
	}
	a.split_shift		= shift;
	const int tiles_p	= pair ? 2 : (a.groups_p + GEMV_WAVES / 2 - 1) / (GEMV_WAVES / 2); // LDS slice per wave, in groups
	const int tiles_c	= tiles_for(splits);
	const int tiles		= tiles_p > tiles_c ? tiles_p : tiles_c;
	const unsigned grid = static_cast<unsigned>(a.producers + strips_c * splits);
	if (pair) {
		return launch_ffn_t<4, false, true>(a, grid, s);
	}
	if (tiles > 4) {
		// the chunked walk in chunks of two groups: chunks of four leave the kernel at 128 registers with up to 14 spilled (the norm's
		// registers on top of 72 for weights), and a spill's reload queues behind the weight loads like any other load.  Measured at
		// the LLaMA-3-70B shapes: 133.0 -> 122.7 us with the norm in front, 116.3 -> 113.5 us without.  (Every wave taking both
		// matrices, two groups of each at a time -- what the chained block's launch does with these shapes -- measured 124.2 and
		// 117.1 us here: two spilled registers again.)
		return launch_ffn_t<2, true>(a, grid, s);
	}
	if (tiles <= 1) {
		return launch_ffn_t<1, false>(a, grid, s);
	}
	if (tiles <= 2) {
		return launch_ffn_t<2, false>(a, grid, s);
	}
	return launch_ffn_t<4, false>(a, grid, s);
}

// parity hook: the gate and up projections' outputs of the last fused launch on this device
hipError_t copy_ffn_gate_up(float* gate_out, float* up_out, int64_t n_ff, hipStream_t s) {
	gemv_scratch sc;
	hipError_t e = get_gemv_scratch(&sc);
	if (e != hipSuccess) {
		return e;
	}
	e = hipMemcpyAsync(gate_out, sc.gate_up, static_cast<size_t>(n_ff) * 4, hipMemcpyDeviceToDevice, s);
	if (e != hipSuccess) {
		return e;
	}
	return hipMemcpyAsync(up_out, sc.gate_up + FFN_MAX_HIDDEN, static_cast<size_t>(n_ff) * 4, hipMemcpyDeviceToDevice, s);
}

} // namespace nh
