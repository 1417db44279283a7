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
#include "q8_0_device.h"

namespace nh {

constexpr int F32ACT_WAVES = 16;

__global__ __launch_bounds__(F32ACT_WAVES * 64) void mul_mat_f32act_kernel(const uint8_t* __restrict__ W, const float* __restrict__ x, float* __restrict__ y, int N, int groups) {
	__shared__ __align__(16) float xs[F32ACT_WAVES][GROUP_K];
	__shared__ float red[F32ACT_WAVES][64];
	const int tid	= threadIdx.x;
	const int lane	= tid & 63;
	const int wave	= __builtin_amdgcn_readfirstlane(tid >> 6);
	const int strip = static_cast<int>(blockIdx.x);
	const int64_t m = blockIdx.y;
	const int half	= lane >> 5;
	const int r		= lane & 31;
	int g0, g1;
	wave_k_range(groups, 0, 0, F32ACT_WAVES, wave, g0, g1);
	const float* xrow = x + m * static_cast<int64_t>(groups) * GROUP_K;
	float acc		  = 0.0f;
	for (int g = g0; g < g1; ++g) {
		const uint8_t* macro = W + macro_offset(strip, g, groups);
		v4i q[GROUP_BLOCKS];
#pragma unroll
		for (int j = 0; j < GROUP_BLOCKS; ++j) {
			q[j] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(macro + j * TILE_BYTES + 16 * lane));
		}
		const v2u dd = __builtin_nontemporal_load(reinterpret_cast<const v2u*>(macro + MACRO_D_OFFSET + 8 * r));
		if (lane < GROUP_K / 4) {
			*reinterpret_cast<float4*>(&xs[wave][4 * lane]) = *reinterpret_cast<const float4*>(xrow + static_cast<int64_t>(g) * GROUP_K + 4 * lane);
		}
		__builtin_amdgcn_wave_barrier(); // wave-local: the same wave wrote and reads
		const float dw[GROUP_BLOCKS] = { half_bits_to_float(static_cast<uint16_t>(dd.x & 0xFFFFu)), half_bits_to_float(static_cast<uint16_t>(dd.x >> 16)),
			half_bits_to_float(static_cast<uint16_t>(dd.y & 0xFFFFu)), half_bits_to_float(static_cast<uint16_t>(dd.y >> 16)) };
#pragma unroll
		for (int j = 0; j < GROUP_BLOCKS; ++j) {
			const float* xb = &xs[wave][j * QK + 16 * half];
			float s			= 0.0f;
#pragma unroll
			for (int c = 0; c < 4; ++c) {
				const float4 xv = *reinterpret_cast<const float4*>(xb + 4 * c);
				const int word	= q[j][c];
				s				= fmaf(xv.x, static_cast<float>(static_cast<int8_t>(word & 0xFF)), s);
				s				= fmaf(xv.y, static_cast<float>(static_cast<int8_t>((word >> 8) & 0xFF)), s);
				s				= fmaf(xv.z, static_cast<float>(static_cast<int8_t>((word >> 16) & 0xFF)), s);
				s				= fmaf(xv.w, static_cast<float>(static_cast<int8_t>((word >> 24) & 0xFF)), s);
			}
			acc = fmaf(s, dw[j], acc);
		}
		__builtin_amdgcn_wave_barrier(); // the next group overwrites this wave's slice
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
		if (row < N) {
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
	// the grid's second dimension holds at most 65535 rows: walk M in slabs
	for (int64_t m0 = 0; m0 < M; m0 += 65535) {
		const int64_t rows = M - m0 < 65535 ? M - m0 : 65535;
		const hipError_t e = launch_kernel(KIND_GEMV, mul_mat_f32act_kernel, dim3(static_cast<unsigned>(strips), static_cast<unsigned>(rows)), dim3(F32ACT_WAVES * 64), 0, s,
			static_cast<const uint8_t*>(W_tiled), x + m0 * K, y + m0 * N, static_cast<int>(N), static_cast<int>(K / GROUP_K));
		if (e != hipSuccess) {
			return e;
		}
	}
	return hipSuccess;
}

} // namespace nh
