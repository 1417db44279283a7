// Token-embedding lookup: out[t][j] = f32(d[id_t][j / 32]) * f32(q[id_t][j]) for Q8_0 rows, gfx950.
//
// The reference's live kernel on both of its backends (cpu/avx_2.hpp:40-66 with the per-token loop at :80-103 and
// :112-135; per-op form :1241-1294; CUDA cuda/cuda_12.hpp:560-601).  One fp32 multiply per element, so the result is
// bit-exact against the CPU.  The reference's CUDA eval-time kernel (cuda/cuda_12.hpp:691-722) never reads the token id
// and always dequantizes row 0; here both phases go through the same kernel and always index by the id.
//
// HBM-bound: 34 bytes read per 128 bytes written.  One thread per four quants (one 16-byte store); the eight threads
// of a block read its scale once each (same address: one request).
#include "q8_0_device.h"

namespace nh {

template<bool TILED>
__global__ __launch_bounds__(256) void get_rows_kernel(const uint8_t* __restrict__ W, const int32_t* __restrict__ ids, float* __restrict__ out, int32_t* __restrict__ invalid, int64_t n_rows,
	int K) {
	const int token	  = blockIdx.y;
	const int t		  = blockIdx.x * 256 + threadIdx.x; // this thread's group of four quants
	const int64_t row = ids[token]; // block-uniform
	if (4 * t >= K) {
		return;
	}
	float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
	if (row >= 0 && row < n_rows) {
		const int b	 = t >> 3; // block of the row
		const int q0 = 4 * (t & 7); // first quant inside the block
		uint32_t quads;
		uint16_t dh;
		if constexpr (TILED) {
			const uint8_t* m = W + macro_offset(row / STRIP_ROWS, b / GROUP_BLOCKS, K / GROUP_K);
			const int r		 = static_cast<int>(row % STRIP_ROWS);
			quads			 = *reinterpret_cast<const uint32_t*>(m + (b % GROUP_BLOCKS) * TILE_BYTES + 16 * (r + 32 * (q0 >> 4)) + (q0 & 15));
			dh				 = load_u16(m + MACRO_D_OFFSET + 8 * r + 2 * (b % GROUP_BLOCKS));
		} else {
			const uint8_t* p = W + (row * (K / QK) + b) * BLOCK_BYTES;
			dh				 = load_u16(p);
			quads			 = static_cast<uint32_t>(load_u16(p + 2 + q0)) | (static_cast<uint32_t>(load_u16(p + 4 + q0)) << 16); // qs is only 2-byte aligned
		}
		const float d = half_bits_to_float(dh);
		v.x			  = d * static_cast<float>(static_cast<int8_t>(quads & 0xFF));
		v.y			  = d * static_cast<float>(static_cast<int8_t>((quads >> 8) & 0xFF));
		v.z			  = d * static_cast<float>(static_cast<int8_t>((quads >> 16) & 0xFF));
		v.w			  = d * static_cast<float>(static_cast<int8_t>(quads >> 24));
	} else if (invalid && t == 0) {
		atomicAdd(invalid, 1);
	}
	*reinterpret_cast<float4*>(out + static_cast<int64_t>(token) * K + 4 * t) = v;
}

hipError_t launch_get_rows(const void* W, const int32_t* ids, float* out, int32_t* invalid, int64_t n_tokens, int64_t n_rows, int64_t K, bool tiled, hipStream_t s) {
	if (n_tokens == 0 || K == 0) {
		return hipSuccess;
	}
	const unsigned chunks = static_cast<unsigned>((K / 4 + 255) / 256);
	for (int64_t first = 0; first < n_tokens; first += 65535) { // grid.y limit
		const unsigned count = static_cast<unsigned>(n_tokens - first < 65535 ? n_tokens - first : 65535);
		const dim3 grid(chunks, count);
		const hipError_t e = tiled
			? launch_kernel(KIND_GET_ROWS, get_rows_kernel<true>, grid, dim3(256), 0, s, static_cast<const uint8_t*>(W), ids + first, out + first * K, invalid, n_rows, static_cast<int>(K))
			: launch_kernel(KIND_GET_ROWS, get_rows_kernel<false>, grid, dim3(256), 0, s, static_cast<const uint8_t*>(W), ids + first, out + first * K, invalid, n_rows, static_cast<int>(K));
		if (e != hipSuccess) {
			return e;
		}
	}
	return hipSuccess;
}

} // namespace nh
