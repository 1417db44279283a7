// Decode mat-vec y = W . xq for Q8_0 weights and a Q8_0-quantized activation row, gfx950.
//
// Computes vec_dot_q8_0_q8_0 (reference cpu/avx_2.hpp:4534-4747) for every weight row:
//   y[n] = sum_b f32(dW[n][b]) * f32(dx[b]) * (sum_j W.qs[n][b][j] * x.qs[b][j])
// with exact int32 block sums (v_dot4_i32_i8) and fp32 scale-and-accumulate.
//
// HBM-bound: 34 bytes of weight per 32 multiply-adds, read exactly once.
//   * one workgroup per 32-row strip; its waves split the strip's K range into 128-quant groups and
//     walk them interleaved, so the workgroup streams one contiguous span of the tiled matrix;
//   * per group a lane issues four 16-byte loads (one KiB per wavefront each, fully coalesced in the
//     tiled layout) plus one 8-byte load of its row's four block scales;
//   * the activation row is staged once in LDS (quants as 16-byte chunks, scales as fp32); each lane
//     reads its 16-byte chunk as a two-address broadcast;
//   * lane l accumulates row (l%32), quants 16*(l/32).. of every block: no cross-lane reduction in the
//     loop; halves and waves are combined once through LDS, in a fixed order (run-to-run bit-stable).
// The same kernel reads the reference's packed 34-byte blocks directly (TILED = false) with unaligned
// 16-byte loads; that is the drop-in-on-raw-bytes form and the parity twin of the tiled one.
#include "q8_0_device.h"

namespace nh {

template<int WAVES, bool TILED, bool DUMP>
__global__ __launch_bounds__(WAVES * 64) void gemv_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ xq, float* __restrict__ y, int32_t* __restrict__ sums, int N, int K) {
	extern __shared__ __align__(16) uint8_t smem[];
	const int nb	 = K / QK;
	const int groups = (nb + GROUP_BLOCKS - 1) / GROUP_BLOCKS;
	uint8_t* xs_q	 = smem; // [K] quants, block b at 32*b
	float* xs_d		 = reinterpret_cast<float*>(smem + K); // [nb]
	float* red		 = xs_d + nb; // [WAVES][64]

	const int tid	= threadIdx.x;
	const int lane	= tid & 63;
	const int wave	= tid >> 6;
	const int strip = blockIdx.x;
	const int r		= lane & 31;
	const int half	= lane >> 5;
	const int row	= strip * STRIP_ROWS + r;
	const int row_c = min(row, N - 1); // rows past the end re-read the last row; their results are dropped

	// ---- stage the activation row: dword j of block b <- two half-word loads (qs is 2-byte aligned) ----
	for (int i = tid; i < nb * 8; i += WAVES * 64) {
		const int b		   = i >> 3;
		const int j		   = i & 7;
		const uint8_t* src = xq + static_cast<int64_t>(b) * BLOCK_BYTES;
		const uint32_t q   = static_cast<uint32_t>(load_u16(src + 2 + 4 * j)) | (static_cast<uint32_t>(load_u16(src + 4 + 4 * j)) << 16);
		*reinterpret_cast<uint32_t*>(xs_q + b * QK + 4 * j) = q;
		if (j == 0) {
			xs_d[b] = half_bits_to_float(load_u16(src));
		}
	}
	__syncthreads();

	const int64_t row_bytes = static_cast<int64_t>(nb) * BLOCK_BYTES;
	const uint8_t* w_row	= W + row_c * row_bytes; // blocks layout
	const uint8_t* w_strip	= W + macro_offset(strip, 0, groups); // tiled layout

	float acc = 0.0f;
#pragma unroll 2
	for (int g = wave; g < groups; g += WAVES) {
		v4i q[GROUP_BLOCKS];
		float dw[GROUP_BLOCKS];
		if constexpr (TILED) {
			const uint8_t* macro = w_strip + static_cast<int64_t>(g) * MACRO_BYTES;
#pragma unroll
			for (int t = 0; t < GROUP_BLOCKS; ++t) {
				q[t] = *reinterpret_cast<const v4i*>(macro + t * TILE_BYTES + 16 * lane);
			}
			const uint2 dd = *reinterpret_cast<const uint2*>(macro + MACRO_D_OFFSET + 8 * r);
			dw[0]		   = half_bits_to_float(static_cast<uint16_t>(dd.x & 0xFFFFu));
			dw[1]		   = half_bits_to_float(static_cast<uint16_t>(dd.x >> 16));
			dw[2]		   = half_bits_to_float(static_cast<uint16_t>(dd.y & 0xFFFFu));
			dw[3]		   = half_bits_to_float(static_cast<uint16_t>(dd.y >> 16));
		} else {
#pragma unroll
			for (int t = 0; t < GROUP_BLOCKS; ++t) {
				const int b		   = min(g * GROUP_BLOCKS + t, nb - 1); // ragged last group: clamped, masked below
				const uint8_t* blk = w_row + static_cast<int64_t>(b) * BLOCK_BYTES;
				q[t]			   = load16_unaligned(blk + 2 + 16 * half);
				dw[t]			   = half_bits_to_float(load_u16(blk));
			}
		}
#pragma unroll
		for (int t = 0; t < GROUP_BLOCKS; ++t) {
			const int b = g * GROUP_BLOCKS + t;
			if (TILED || b < nb) {
				const v4i xv = *reinterpret_cast<const v4i*>(xs_q + b * QK + 16 * half);
				const int s	 = dot16(q[t], xv);
				if constexpr (DUMP) {
					const int full = s + __shfl_xor(s, 32);
					if (half == 0 && row < N) {
						sums[static_cast<int64_t>(row) * nb + b] = full;
					}
				} else {
					acc = fmaf(static_cast<float>(s), dw[t] * xs_d[b], acc);
				}
			}
		}
	}

	if constexpr (!DUMP) {
		red[wave * 64 + lane] = acc;
		__syncthreads();
		if (tid < STRIP_ROWS) {
			float total = 0.0f;
#pragma unroll
			for (int w = 0; w < WAVES; ++w) {
				total += red[w * 64 + tid] + red[w * 64 + 32 + tid];
			}
			if (strip * STRIP_ROWS + tid < N) {
				y[strip * STRIP_ROWS + tid] = total;
			}
		}
	}
}

// y <- 0 for an empty inner dimension (a fill kernel rather than a memset node, so the call can be graph-captured)
__global__ void zero_f32_kernel(float* __restrict__ y, int64_t n) {
	const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
	if (i < n) {
		y[i] = 0.0f;
	}
}

template<int WAVES, bool TILED> static hipError_t launch_gemv_t(const uint8_t* W, const uint8_t* xq, float* y, int32_t* sums, int N, int K, hipStream_t s) {
	const int strips   = (N + STRIP_ROWS - 1) / STRIP_ROWS;
	const size_t shmem = static_cast<size_t>(K) + static_cast<size_t>(K / QK) * 4 + WAVES * 64 * 4;
	if (sums) {
		gemv_kernel<WAVES, TILED, true><<<dim3(strips), dim3(WAVES * 64), shmem, s>>>(W, xq, y, sums, N, K);
		return hipGetLastError();
	}
	return launch_kernel(KIND_GEMV, gemv_kernel<WAVES, TILED, false>, dim3(strips), dim3(WAVES * 64), shmem, s, W, xq, y, sums, N, K);
}

hipError_t launch_gemv(const void* W, const void* xq_blocks, float* y, int32_t* sums, int64_t N, int64_t K, bool tiled, hipStream_t s) {
	if (N == 0 || K == 0) {
		if (N > 0 && !sums) {
			zero_f32_kernel<<<dim3(static_cast<unsigned>((N + 255) / 256)), dim3(256), 0, s>>>(y, N); // empty dot product
			return hipGetLastError();
		}
		return hipSuccess;
	}
	const uint8_t* w = static_cast<const uint8_t*>(W);
	const uint8_t* x = static_cast<const uint8_t*>(xq_blocks);
	if (tiled) {
		return launch_gemv_t<4, true>(w, x, y, sums, static_cast<int>(N), static_cast<int>(K), s);
	}
	return launch_gemv_t<4, false>(w, x, y, sums, static_cast<int>(N), static_cast<int>(K), s);
}

} // namespace nh
