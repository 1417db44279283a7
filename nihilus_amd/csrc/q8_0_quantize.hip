// Activation quantize, fp32 -> Q8_0, for gfx950.
//
// Restates quantize_row_q8_0 (reference cpu/avx_2.hpp:4439-4489) with bit-exact results:
//   amax = max|x_i| over 32 values; d = fp16_rne(amax / 127.f) with an IEEE fp32 divide;
//   id = amax != 0 ? 127.f / amax : 0;  q_i = int8(round_half_even(fl32(x_i * id))).
// The multiply, the rounding and the divide are kept as separate correctly rounded fp32 operations
// (__fmul_rn / __fdiv_rn / v_rndne_f32): contracting x*id into anything else would change ties.
//
// Memory-bound: 4 bytes read + 1.0625 bytes written per element.  Eight lanes share one block, each
// loads one float4 (a wavefront reads 1 KiB contiguous), the block maximum is a three-step
// cross-lane max inside the 8-lane group.
#include "q8_0_device.h"

namespace nh {

//
// SILU_MUL: the value quantized is silu(x) * u (the FFN activation in front of the down projection, computed from the
// gate and up projections' outputs), so the fp32 activation never makes a round trip through memory.
template<bool TILED, bool SILU_MUL>
__global__ __launch_bounds__(256) void quantize_kernel(const float* __restrict__ x, const float* __restrict__ u, uint8_t* __restrict__ out, int64_t M, int64_t rows_out, int64_t K) {
	const int64_t nb = K / QK;
	const int64_t t	 = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
	const int j		 = static_cast<int>(t & 7); // which float4 of the block
	// Eight lanes per block either way.  Tiled output: a wave takes one block column of eight consecutive rows, so that its
	// stores fill two whole 128-byte lines of the tile (8 rows x 16 bytes per half) instead of sixteen 16-byte pieces of
	// eight different tiles; rows_out is a multiple of 32 there.  Blocks output: a wave takes eight consecutive blocks of a row.
	int64_t m, b;
	bool in_range;
	if constexpr (TILED) {
		const int64_t unit = t >> 6; // (8-row group, block column)
		in_range		   = unit < (rows_out / 8) * nb;
		const int64_t rg   = in_range ? unit / nb : 0;
		b				   = in_range ? unit - rg * nb : 0;
		m				   = rg * 8 + ((t >> 3) & 7);
	} else {
		const int64_t blk = t >> 3; // block index over rows_out * nb
		in_range		  = blk < rows_out * nb; // whole 8-lane groups agree, so the shuffles below stay converged per group
		m				  = in_range ? blk / nb : 0;
		b				  = in_range ? blk - m * nb : 0;
	}

	float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
	if (in_range && m < M) {
		v = *reinterpret_cast<const float4*>(x + m * K + b * QK + 4 * j);
		if constexpr (SILU_MUL) {
			v = silu_mul4(v, *reinterpret_cast<const float4*>(u + m * K + b * QK + 4 * j));
		}
	}
	uint16_t dh;
	const uint32_t packed = quantize_block_lane(v, &dh);

	if (!in_range) {
		return;
	}
	if constexpr (TILED) {
		const int64_t strip = m / STRIP_ROWS;
		const int r			= static_cast<int>(m % STRIP_ROWS);
		const int64_t g		= b / GROUP_BLOCKS;
		const int tq		= static_cast<int>(b % GROUP_BLOCKS);
		uint8_t* macro		= out + macro_offset(strip, g, K / GROUP_K);
		const int lane		= r + 32 * (j >> 2); // quants 0..15 live in lanes 0..31, 16..31 in lanes 32..63
		*reinterpret_cast<uint32_t*>(macro + tq * TILE_BYTES + 16 * lane + 4 * (j & 3)) = packed;
		if (j == 0) {
			*reinterpret_cast<uint16_t*>(macro + MACRO_D_OFFSET + 8 * r + 2 * tq) = dh;
		}
	} else {
		uint8_t* o = out + (m * nb + b) * BLOCK_BYTES;
		// the qs field sits at a 2-byte-aligned address: two half-word stores per lane
		*reinterpret_cast<uint16_t*>(o + 2 + 4 * j)		= static_cast<uint16_t>(packed & 0xFFFFu);
		*reinterpret_cast<uint16_t*>(o + 2 + 4 * j + 2) = static_cast<uint16_t>(packed >> 16);
		if (j == 0) {
			*reinterpret_cast<uint16_t*>(o) = dh;
		}
	}
}

// RMS norm * weight fused into the quantizer (the prologue of the q/k/v, gate/up and output projections in prefill):
// one 1024-thread workgroup per row; the row's scale first (fixed-order sum of squares, see rms_scale_workgroup), then
// every thread normalises and quantizes its float4s.  The row is read twice, the second time from cache.
template<bool TILED>
__global__ __launch_bounds__(1024) void rms_norm_quantize_kernel(const float* __restrict__ x, const float* __restrict__ norm_w, float eps, uint8_t* __restrict__ out, int64_t M, int K) {
	__shared__ float red[16];
	const int tid	  = threadIdx.x;
	const int lane	  = tid & 63;
	const int wave	  = tid >> 6;
	const int64_t m	  = blockIdx.x; // row of the output, padding rows of a tiled output included
	const int n4	  = K / 4;
	const bool real	  = m < M;
	const float4* x4  = reinterpret_cast<const float4*>(x + (real ? m : 0) * K);
	const float4* w4  = reinterpret_cast<const float4*>(norm_w);
	const float p = real ? rms_run_sumsq(x + m * K, K / GROUP_K, wave, lane) : 0.0f;
	const float scale = rms_scale_workgroup(p, red, wave, lane, K, eps);
	const int nb	  = K / QK;
	for (int j0 = 0; j0 < n4; j0 += 1024) { // uniform trip count: whole 8-lane groups stay together in the quantizer
		const int j = j0 + tid;
		float4 v	= make_float4(0.f, 0.f, 0.f, 0.f);
		if (real && j < n4) {
			v = norm_mul4(x4[j], scale, w4[j]);
		}
		uint16_t dh;
		const uint32_t packed = quantize_block_lane(v, &dh);
		if (j >= n4) {
			continue;
		}
		const int b	 = j >> 3;
		const int jj = j & 7;
		if constexpr (TILED) {
			const int64_t strip = m / STRIP_ROWS;
			const int r			= static_cast<int>(m % STRIP_ROWS);
			uint8_t* macro		= out + macro_offset(strip, b / GROUP_BLOCKS, K / GROUP_K);
			const int tq		= b % GROUP_BLOCKS;
			const int l			= r + 32 * (jj >> 2);
			*reinterpret_cast<uint32_t*>(macro + tq * TILE_BYTES + 16 * l + 4 * (jj & 3)) = packed;
			if (jj == 0) {
				*reinterpret_cast<uint16_t*>(macro + MACRO_D_OFFSET + 8 * r + 2 * tq) = dh;
			}
		} else {
			uint8_t* o										 = out + (m * nb + b) * BLOCK_BYTES;
			*reinterpret_cast<uint16_t*>(o + 2 + 4 * jj)	 = static_cast<uint16_t>(packed & 0xFFFFu);
			*reinterpret_cast<uint16_t*>(o + 2 + 4 * jj + 2) = static_cast<uint16_t>(packed >> 16);
			if (jj == 0) {
				*reinterpret_cast<uint16_t*>(o) = dh;
			}
		}
	}
}

hipError_t launch_rms_norm_quantize(const float* x, const float* norm_w, float eps, void* out, int64_t M, int64_t K, bool tiled, hipStream_t s) {
	const int64_t rows_out = tiled ? (M + STRIP_ROWS - 1) / STRIP_ROWS * STRIP_ROWS : M;
	if (rows_out == 0 || K == 0) {
		return hipSuccess;
	}
	const dim3 g(static_cast<unsigned>(rows_out)), b(1024);
	if (tiled) {
		return launch_kernel(KIND_QUANTIZE, rms_norm_quantize_kernel<true>, g, b, 0, s, x, norm_w, eps, static_cast<uint8_t*>(out), M, static_cast<int>(K));
	}
	return launch_kernel(KIND_QUANTIZE, rms_norm_quantize_kernel<false>, g, b, 0, s, x, norm_w, eps, static_cast<uint8_t*>(out), M, static_cast<int>(K));
}

template<bool SILU_MUL> static hipError_t launch_quantize_t(const float* x, const float* u, void* out, int64_t M, int64_t K, bool tiled, hipStream_t s) {
	const int64_t rows_out = tiled ? (M + STRIP_ROWS - 1) / STRIP_ROWS * STRIP_ROWS : M;
	const int64_t threads  = rows_out * (K / QK) * 8;
	if (threads == 0) {
		return hipSuccess;
	}
	const int64_t grid = (threads + 255) / 256;
	const dim3 g(static_cast<unsigned>(grid)), b(256);
	if (tiled) {
		return launch_kernel(KIND_QUANTIZE, quantize_kernel<true, SILU_MUL>, g, b, 0, s, x, u, static_cast<uint8_t*>(out), M, rows_out, K);
	}
	return launch_kernel(KIND_QUANTIZE, quantize_kernel<false, SILU_MUL>, g, b, 0, s, x, u, static_cast<uint8_t*>(out), M, rows_out, K);
}

hipError_t launch_quantize(const float* x, void* out, int64_t M, int64_t K, bool tiled, hipStream_t s) {
	return launch_quantize_t<false>(x, nullptr, out, M, K, tiled, s);
}

hipError_t launch_silu_mul_quantize(const float* gate, const float* up, void* out, int64_t M, int64_t K, bool tiled, hipStream_t s) {
	return launch_quantize_t<true>(gate, up, out, M, K, tiled, s);
}

} // namespace nh
