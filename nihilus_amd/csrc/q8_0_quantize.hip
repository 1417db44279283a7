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

// rows from which the norm + quantize takes eight rows per workgroup (a workgroup per CU; with fewer the one-row form's 1024-thread
// workgroups reach more CUs: [512 x 4096] 5.8 against 9.3 us, [2048 x 4096] 18.7 against 13.9 us)
constexpr int64_t RMS_ROWS8_MIN_ROWS = 2048;
constexpr int64_t QUANTIZE_TWO_PASS_MIN_THREADS = int64_t{ 1 } << 20; // float4s from which a thread takes two
constexpr int QUANTIZE_PASSES = 2;

// SILU_MUL: the value quantized is silu(x) * u (the FFN activation in front of the down projection, computed from the
// gate and up projections' outputs), so the fp32 activation never makes a round trip through memory.
// PASSES: float4s per thread, `stride` threads apart (two from 2^20 float4s on: twice the bytes in flight per CU, which is what
// a streaming launch of this kernel is short of -- [8192 x 4096]: 34.0 -> 31.0 us, [32768 x 4096]: 132 -> 123 us, 5.1 -> 5.5 TB/s;
// four measured the same as two).
template<bool TILED, bool SILU_MUL, int PASSES>
__global__ __launch_bounds__(256) void quantize_kernel(const float* __restrict__ x, const float* __restrict__ u, uint8_t* __restrict__ out, int64_t M, int64_t rows_out, int64_t K, int64_t stride) {
	const int64_t nb = K / QK;
	const int64_t t0 = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
	const int j		 = static_cast<int>(t0 & 7); // which float4 of the block (stride is a multiple of 64)
	// Eight lanes per block either way.  Tiled output: a wave takes one block column of eight consecutive rows, so that its
	// stores fill two whole 128-byte lines of the tile (8 rows x 16 bytes per half) instead of sixteen 16-byte pieces of
	// eight different tiles; rows_out is a multiple of 32 there.  Blocks output: a wave takes eight consecutive blocks of a row.
	int64_t m[PASSES], b[PASSES];
	bool in_range[PASSES];
	float4 v[PASSES];
#pragma unroll
	for (int p = 0; p < PASSES; ++p) {
		const int64_t t = t0 + p * stride;
		if constexpr (TILED) {
			const int64_t unit = t >> 6; // (8-row group, block column)
			in_range[p]		   = unit < (rows_out / 8) * nb;
			const int64_t rg   = in_range[p] ? unit / nb : 0;
			b[p]			   = in_range[p] ? unit - rg * nb : 0;
			m[p]			   = rg * 8 + ((t >> 3) & 7);
		} else {
			const int64_t blk = t >> 3; // block index over rows_out * nb
			in_range[p]		  = blk < rows_out * nb; // whole 8-lane groups agree, so the shuffles below stay converged per group
			m[p]			  = in_range[p] ? blk / nb : 0;
			b[p]			  = in_range[p] ? blk - m[p] * nb : 0;
		}
		v[p] = make_float4(0.f, 0.f, 0.f, 0.f);
		if (in_range[p] && m[p] < M) {
			v[p] = *reinterpret_cast<const float4*>(x + m[p] * K + b[p] * QK + 4 * j);
			if constexpr (SILU_MUL) {
				v[p] = silu_mul4(v[p], *reinterpret_cast<const float4*>(u + m[p] * K + b[p] * QK + 4 * j));
			}
		}
	}
#pragma unroll
	for (int p = 0; p < PASSES; ++p) {
		uint16_t dh;
		const uint32_t packed = quantize_block_lane(v[p], &dh);
		if (!in_range[p]) {
			continue;
		}
		if constexpr (TILED) {
			const int64_t strip = m[p] / STRIP_ROWS;
			const int r			= static_cast<int>(m[p] % STRIP_ROWS);
			const int64_t g		= b[p] / GROUP_BLOCKS;
			const int tq		= static_cast<int>(b[p] % GROUP_BLOCKS);
			uint8_t* macro		= out + macro_offset(strip, g, K / GROUP_K);
			const int lane		= r + 32 * (j >> 2); // quants 0..15 live in lanes 0..31, 16..31 in lanes 32..63
			*reinterpret_cast<uint32_t*>(macro + tq * TILE_BYTES + 16 * lane + 4 * (j & 3)) = packed;
			if (j == 0) {
				*reinterpret_cast<uint16_t*>(macro + MACRO_D_OFFSET + 8 * r + 2 * tq) = dh;
			}
		} else {
			uint8_t* o = out + (m[p] * nb + b[p]) * BLOCK_BYTES;
			// the qs field sits at a 2-byte-aligned address: two half-word stores per lane
			*reinterpret_cast<uint16_t*>(o + 2 + 4 * j)		= static_cast<uint16_t>(packed & 0xFFFFu);
			*reinterpret_cast<uint16_t*>(o + 2 + 4 * j + 2) = static_cast<uint16_t>(packed >> 16);
			if (j == 0) {
				*reinterpret_cast<uint16_t*>(o) = dh;
			}
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

// The same for the tiled output and rows of up to 8192 values, EIGHT rows per 1024-thread workgroup.  What bounds the one-row form
// at prefill sizes is not its reads but its stores: a row owns 16 bytes of every 128-byte line of the operand tiles, so a row at a
// time writes nothing but sixteenth-of-a-wave pieces ([8192 x 4096]: 65 us; the same launch without its stores 22 us).  Eight
// consecutive rows own whole lines.  Waves 2r and 2r + 1 take row r: runs 8 (w % 2) .. + 7 of the fixed-order sum of squares,
// each lane the float4s that the 16-wave form gives lane `lane` of wave `run` -- the same per-lane sums, butterflies and order
// of the sixteen run sums, hence the same scale and the same bytes -- kept in registers for the quantizer, so the rows are read
// once (non-temporal loads of the rows measured no different: the launch is bound by its stores).  The quants and scales go to an LDS image of the eight rows' share of the tiles ([group][tile][half][row][16 bytes], then
// [group][row][4 scales]) and from there to memory as whole lines, 16 bytes per lane.  F4: float4s per lane and run.
template<int F4>
__global__ __launch_bounds__(1024, F4 == 1 ? 8 : 4) void rms_norm_quantize_rows8_kernel(const float* __restrict__ x, const float* __restrict__ norm_w, float eps, uint8_t* __restrict__ out, int64_t M, int K) {
	__shared__ __align__(16) uint8_t image[F4 * 4096 * 8 + F4 * 32 * 64]; // K * 8 bytes of quants, then K / 128 * 64 bytes of scales (K <= 4096 F4)
	__shared__ float red[8][16];
	const int tid	 = threadIdx.x;
	const int lane	 = tid & 63;
	const int wave	 = __builtin_amdgcn_readfirstlane(tid >> 6); // wave-uniform: the runs' bounds stay in scalar registers
	const int row8	 = wave >> 1; // which of the workgroup's eight rows
	const int64_t m0 = static_cast<int64_t>(blockIdx.x) * 8;
	const int64_t m	 = m0 + row8;
	const bool real	 = m < M; // rows past M are the padding of the last strip: zeros
	const int groups = K / GROUP_K;
	const int q = groups / 16, r = groups % 16;
	const float4* x4 = reinterpret_cast<const float4*>(x + (real ? m : 0) * K);
	const float4* w4 = reinterpret_cast<const float4*>(norm_w);
	float4 v[8][F4];
	int first[8], n4[8];
#pragma unroll
	for (int rr = 0; rr < 8; ++rr) {
		const int run = 8 * (wave & 1) + rr;
		first[rr]	  = (run * q + min(run, r)) * 32; // the run's first float4
		n4[rr]		  = (q + (run < r ? 1 : 0)) * 32; // and how many it has (a multiple of 32: whole blocks)
#pragma unroll
		for (int i = 0; i < F4; ++i) {
			const int j = lane + 64 * i;
			v[rr][i]	= (real && j < n4[rr]) ? x4[first[rr] + j] : make_float4(0.f, 0.f, 0.f, 0.f);
		}
	}
#pragma unroll
	for (int rr = 0; rr < 8; ++rr) {
		float p = 0.0f;
#pragma unroll
		for (int i = 0; i < F4; ++i) {
			if (lane + 64 * i < n4[rr]) {
				p = sumsq_fold(p, v[rr][i]);
			}
		}
		p = wave_sum_butterfly(p);
		if (lane == 0) {
			red[row8][8 * (wave & 1) + rr] = p;
		}
	}
	__syncthreads();
	float sum = red[row8][0];
#pragma unroll
	for (int k = 1; k < 16; ++k) {
		sum = __fadd_rn(sum, red[row8][k]);
	}
	const float scale = __fdiv_rn(1.0f, sqrtf(__fadd_rn(__fdiv_rn(sum, static_cast<float>(K)), eps)));
	uint8_t* image_d  = image + static_cast<size_t>(K) * 8;
#pragma unroll
	for (int rr = 0; rr < 8; ++rr) {
#pragma unroll
		for (int i = 0; i < F4; ++i) {
			const int jr	= lane + 64 * i;
			const bool have = jr < n4[rr]; // whole 8-lane groups agree
			const int j		= first[rr] + (have ? jr : 0);
			const float4 y	= (real && have) ? norm_mul4(v[rr][i], scale, w4[j]) : make_float4(0.f, 0.f, 0.f, 0.f);
			uint16_t dh;
			const uint32_t packed = quantize_block_lane(y, &dh);
			if (!have) {
				continue;
			}
			const int b	 = j >> 3; // block of the row: group b / 4, tile b % 4
			const int jj = j & 7; // float4 of the block: quants 4 jj .. 4 jj + 3, i.e. half jj / 4 of the tile
			*reinterpret_cast<uint32_t*>(image + ((b * 2 + (jj >> 2)) * 8 + row8) * 16 + 4 * (jj & 3)) = packed;
			if (jj == 0) {
				*reinterpret_cast<uint16_t*>(image_d + ((b / GROUP_BLOCKS) * 8 + row8) * 8 + 2 * (b % GROUP_BLOCKS)) = dh;
			}
		}
	}
	__syncthreads();
	// the image out: line (block b, half h) = 128 bytes at tile b % 4 of group b / 4, rows r0 .. r0 + 7 of half h; eight lanes per line
	const int64_t strip = m0 / STRIP_ROWS;
	const int r0		= static_cast<int>(m0 % STRIP_ROWS);
	const int lines		= (K / QK) * 2;
	for (int t = tid; t < lines * 8; t += 1024) {
		const int line = t >> 3, piece = t & 7;
		const int b = line >> 1, h = line & 1;
		uint8_t* macro = out + macro_offset(strip, b / GROUP_BLOCKS, groups);
		*reinterpret_cast<v4i*>(macro + (b % GROUP_BLOCKS) * TILE_BYTES + 16 * (r0 + 32 * h + piece)) = *reinterpret_cast<const v4i*>(image + line * 128 + piece * 16);
	}
	for (int t = tid; t < groups * 4; t += 1024) { // 64 bytes of scales per group: rows r0 .. r0 + 7, four lanes each
		const int g = t >> 2, piece = t & 3;
		uint8_t* macro = out + macro_offset(strip, g, groups);
		*reinterpret_cast<v4i*>(macro + MACRO_D_OFFSET + 8 * r0 + 16 * piece) = *reinterpret_cast<const v4i*>(image_d + g * 64 + piece * 16);
	}
}

hipError_t launch_rms_norm_quantize(const float* x, const float* norm_w, float eps, void* out, int64_t M, int64_t K, bool tiled, hipStream_t s) {
	const int64_t rows_out = tiled ? (M + STRIP_ROWS - 1) / STRIP_ROWS * STRIP_ROWS : M;
	if (rows_out == 0 || K == 0) {
		return hipSuccess;
	}
	if (tiled && K <= 8192 && rows_out >= RMS_ROWS8_MIN_ROWS) {
		// a run has at most ceil(K / 128 / 16) groups of 32 float4s: 64 float4s (one per lane) up to K = 4096, 128 up to 8192
		const dim3 g8(static_cast<unsigned>(rows_out / 8)), b8(1024);
		uint8_t* o		 = static_cast<uint8_t*>(out);
		if (K <= 4096) {
			return launch_kernel(KIND_QUANTIZE, rms_norm_quantize_rows8_kernel<1>, g8, b8, 0, s, x, norm_w, eps, o, M, static_cast<int>(K));
		}
		return launch_kernel(KIND_QUANTIZE, rms_norm_quantize_rows8_kernel<2>, g8, b8, 0, s, x, norm_w, eps, o, M, static_cast<int>(K));
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
	const int passes	 = (!SILU_MUL && threads >= QUANTIZE_TWO_PASS_MIN_THREADS) ? QUANTIZE_PASSES : 1; // (SiLU * up, two inputs per value already: 14.3 -> 15.6 us at [2048 x 4096] with two)
	const int64_t grid	 = ((threads + passes - 1) / passes + 255) / 256;
	const int64_t stride = grid * 256;
	const dim3 g(static_cast<unsigned>(grid)), b(256);
	uint8_t* o = static_cast<uint8_t*>(out);
	if (passes == 1) {
		return tiled ? launch_kernel(KIND_QUANTIZE, quantize_kernel<true, SILU_MUL, 1>, g, b, 0, s, x, u, o, M, rows_out, K, stride)
					 : launch_kernel(KIND_QUANTIZE, quantize_kernel<false, SILU_MUL, 1>, g, b, 0, s, x, u, o, M, rows_out, K, stride);
	}
	return tiled ? launch_kernel(KIND_QUANTIZE, quantize_kernel<true, SILU_MUL, QUANTIZE_PASSES>, g, b, 0, s, x, u, o, M, rows_out, K, stride)
				 : launch_kernel(KIND_QUANTIZE, quantize_kernel<false, SILU_MUL, QUANTIZE_PASSES>, g, b, 0, s, x, u, o, M, rows_out, K, stride);
}

hipError_t launch_quantize(const float* x, void* out, int64_t M, int64_t K, bool tiled, hipStream_t s) {
	return launch_quantize_t<false>(x, nullptr, out, M, K, tiled, s);
}

hipError_t launch_silu_mul_quantize(const float* gate, const float* up, void* out, int64_t M, int64_t K, bool tiled, hipStream_t s) {
	return launch_quantize_t<true>(gate, up, out, M, K, tiled, s);
}

} // namespace nh
