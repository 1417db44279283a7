// Layout conversion (packed 34-byte blocks <-> tiled device layout) and the synthetic-input generator.
//
// The reference keeps weights as rows of packed block_q8_0 (common/data_types.hpp:38-44) and copies them
// into its device arena at load time (infra/model_parser.hpp:151-154).  tile_kernel is that copy with a byte
// permutation: after it, one 64-lane wavefront reads a 32-row x 32-quant tile as one contiguous KiB.
// Both directions are lossless; one thread moves four quants.
#include "q8_0_device.h"

namespace nh {

// Address of the dword holding quants 4j..4j+3 of (row, block b) in the tiled layout.
__device__ __forceinline__ int64_t tiled_q_offset(int64_t row, int64_t b, int j, int64_t groups) {
	const int64_t strip = row / STRIP_ROWS;
	const int r			= static_cast<int>(row % STRIP_ROWS);
	const int lane		= r + 32 * (j >> 2);
	return macro_offset(strip, b / GROUP_BLOCKS, groups) + (b % GROUP_BLOCKS) * TILE_BYTES + 16 * lane + 4 * (j & 3);
}
__device__ __forceinline__ int64_t tiled_d_offset(int64_t row, int64_t b, int64_t groups) {
	return macro_offset(row / STRIP_ROWS, b / GROUP_BLOCKS, groups) + MACRO_D_OFFSET + 8 * (row % STRIP_ROWS) + 2 * (b % GROUP_BLOCKS);
}

__global__ __launch_bounds__(256) void tile_kernel(const uint8_t* __restrict__ blocks, uint8_t* __restrict__ tiled, int64_t rows, int64_t rows_padded, int64_t K) {
	const int64_t nb  = K / QK;
	const int64_t t	  = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
	const int64_t blk = t >> 3;
	const int j		  = static_cast<int>(t & 7);
	if (blk >= rows_padded * nb) {
		return;
	}
	const int64_t row = blk / nb;
	const int64_t b	  = blk - row * nb;
	uint32_t q		  = 0;
	uint16_t d		  = 0;
	if (row < rows) {
		const uint8_t* src = blocks + blk * BLOCK_BYTES;
		q				   = static_cast<uint32_t>(load_u16(src + 2 + 4 * j)) | (static_cast<uint32_t>(load_u16(src + 4 + 4 * j)) << 16);
		d				   = load_u16(src);
	}
	*reinterpret_cast<uint32_t*>(tiled + tiled_q_offset(row, b, j, K / GROUP_K)) = q;
	if (j == 0) {
		*reinterpret_cast<uint16_t*>(tiled + tiled_d_offset(row, b, K / GROUP_K)) = d;
	}
}

__global__ __launch_bounds__(256) void untile_kernel(const uint8_t* __restrict__ tiled, uint8_t* __restrict__ blocks, int64_t rows, int64_t K) {
	const int64_t nb  = K / QK;
	const int64_t t	  = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
	const int64_t blk = t >> 3;
	const int j		  = static_cast<int>(t & 7);
	if (blk >= rows * nb) {
		return;
	}
	const int64_t row = blk / nb;
	const int64_t b	  = blk - row * nb;
	const uint32_t q  = *reinterpret_cast<const uint32_t*>(tiled + tiled_q_offset(row, b, j, K / GROUP_K));
	uint8_t* dst	  = blocks + blk * BLOCK_BYTES;
	*reinterpret_cast<uint16_t*>(dst + 2 + 4 * j) = static_cast<uint16_t>(q & 0xFFFFu);
	*reinterpret_cast<uint16_t*>(dst + 4 + 4 * j) = static_cast<uint16_t>(q >> 16);
	if (j == 0) {
		*reinterpret_cast<uint16_t*>(dst) = load_u16(tiled + tiled_d_offset(row, b, K / GROUP_K));
	}
}

hipError_t launch_tile(const void* blocks, void* tiled, int64_t rows, int64_t K, hipStream_t s) {
	const int64_t rows_padded = (rows + STRIP_ROWS - 1) / STRIP_ROWS * STRIP_ROWS;
	const int64_t threads	  = rows_padded * (K / QK) * 8;
	if (threads == 0) {
		return hipSuccess;
	}
	tile_kernel<<<dim3(static_cast<unsigned>((threads + 255) / 256)), dim3(256), 0, s>>>(static_cast<const uint8_t*>(blocks), static_cast<uint8_t*>(tiled), rows, rows_padded, K);
	return hipGetLastError();
}

hipError_t launch_untile(const void* tiled, void* blocks, int64_t rows, int64_t K, hipStream_t s) {
	const int64_t threads = rows * (K / QK) * 8;
	if (threads == 0) {
		return hipSuccess;
	}
	untile_kernel<<<dim3(static_cast<unsigned>((threads + 255) / 256)), dim3(256), 0, s>>>(static_cast<const uint8_t*>(tiled), static_cast<uint8_t*>(blocks), rows, K);
	return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------------
// Synthetic inputs.  Counter-based, so the same (seed, index) gives the same bytes on any device or host:
//   h(seed, i)  = splitmix64 finaliser of seed + (i+1)*0x9E3779B97F4A7C15
//   gauss(s, i) = (sum of twelve 16-bit fields of h(s,3i..3i+2) - 393210) / 65536   (Irwin-Hall, variance 1; exact in fp32)
//   weight block t: qs[4g+j] = ((16-bit field j of h(seed, 8t+g)) * 255 >> 16) - 127;  d = fp16(|gauss(seed^W, t)| * 0.01f)
//   activation i:   gauss(seed^A, i)

__device__ __forceinline__ uint64_t mix_hash(uint64_t seed, uint64_t i) {
	uint64_t z = seed + (i + 1) * 0x9E3779B97F4A7C15ull;
	z		   = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
	z		   = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
	return z ^ (z >> 31);
}
__device__ __forceinline__ float gauss12(uint64_t seed, uint64_t i) {
	int s = 0;
#pragma unroll
	for (int t = 0; t < 3; ++t) {
		const uint64_t h = mix_hash(seed, 3 * i + t);
		s += static_cast<int>(h & 0xFFFF) + static_cast<int>((h >> 16) & 0xFFFF) + static_cast<int>((h >> 32) & 0xFFFF) + static_cast<int>((h >> 48) & 0xFFFF);
	}
	return __fmul_rn(static_cast<float>(s - 393210), 1.0f / 65536.0f);
}

__global__ __launch_bounds__(256) void fill_weights_kernel(uint8_t* __restrict__ blocks, uint64_t seed, int64_t first_block, int64_t n_blocks) {
	const int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
	const int64_t i = t >> 3;
	const int g		= static_cast<int>(t & 7);
	if (i >= n_blocks) {
		return;
	}
	const uint64_t blk = static_cast<uint64_t>(first_block + i);
	const uint64_t h   = mix_hash(seed, blk * 8 + g);
	uint32_t packed	   = 0;
#pragma unroll
	for (int j = 0; j < 4; ++j) {
		const uint32_t u = static_cast<uint32_t>((h >> (16 * j)) & 0xFFFF);
		const int q		 = static_cast<int>((u * 255u) >> 16) - 127;
		packed |= (static_cast<uint32_t>(q) & 0xFFu) << (8 * j);
	}
	uint8_t* o = blocks + i * BLOCK_BYTES;
	*reinterpret_cast<uint16_t*>(o + 2 + 4 * g) = static_cast<uint16_t>(packed & 0xFFFFu);
	*reinterpret_cast<uint16_t*>(o + 4 + 4 * g) = static_cast<uint16_t>(packed >> 16);
	if (g == 0) {
		float ds = __fmul_rn(fabsf(gauss12(seed ^ 0x5EED5EED5EED5EEDull, blk)), 0.01f);
		// Keep the fp32 product and the fp16 conversion as two roundings: without this barrier the compiler merges
		// them into one v_fma_mixlo_f16 (a single rounding), which differs from the two-step host arithmetic.
		asm volatile("" : "+v"(ds));
		*reinterpret_cast<uint16_t*>(o) = float_to_half_bits(ds);
	}
}

__global__ __launch_bounds__(256) void fill_activations_kernel(float* __restrict__ x, uint64_t seed, int64_t count) {
	const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
	if (i < count) {
		x[i] = gauss12(seed ^ 0xA5A5A5A5A5A5A5A5ull, static_cast<uint64_t>(i));
	}
}

hipError_t launch_fill_weights(void* blocks, uint64_t seed, int64_t first_block, int64_t n_blocks, hipStream_t s) {
	if (n_blocks == 0) {
		return hipSuccess;
	}
	const int64_t threads = n_blocks * 8;
	fill_weights_kernel<<<dim3(static_cast<unsigned>((threads + 255) / 256)), dim3(256), 0, s>>>(static_cast<uint8_t*>(blocks), seed, first_block, n_blocks);
	return hipGetLastError();
}

hipError_t launch_fill_activations(float* x, uint64_t seed, int64_t count, hipStream_t s) {
	if (count == 0) {
		return hipSuccess;
	}
	fill_activations_kernel<<<dim3(static_cast<unsigned>((count + 255) / 256)), dim3(256), 0, s>>>(x, seed, count);
	return hipGetLastError();
}

} // namespace nh
