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

#include <mutex>

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

// ---------------------------------------------------------------------------------------------------------
// The streaming form for the tiled layout: the kernel the decode path runs.
//
// A 62 MB weight matrix is 7.8 us of HBM time; what decides the achieved bandwidth is how quickly the whole
// chip has loads in flight and how little happens after the last byte lands.  So:
//   * sixteen waves per workgroup, one workgroup per (32-row strip, K split); every wave owns at most TILES
//     128-quant groups and issues ALL of its weight loads (TILES x (4 x 16 B + 8 B) per lane, non-temporal)
//     before it waits for anything: no loop, no workgroup barrier in front of the loads;
//   * its slice of the activation row is staged wave-locally: the loads for it go out first, are re-aligned
//     from the packed 34-byte blocks into LDS as the weight loads fly, and are read back as 16-byte
//     two-address broadcasts (only the wave's own lgkm counter is waited on, never a barrier);
//   * one LDS reduction per workgroup; when K is split over several workgroups (few rows, long K) each writes
//     32 partial sums and the last to arrive adds them in split order -- fixed order, so results do not
//     depend on arrival order.
constexpr int GEMV_WAVES = 16;

template<int TILES, bool DUMP>
__global__ __launch_bounds__(GEMV_WAVES * 64) void gemv_tiled_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ xq, float* __restrict__ y, int32_t* __restrict__ sums,
	float* __restrict__ partials, unsigned* __restrict__ counters, int N, int groups, int splits) {
	__shared__ __align__(16) uint8_t xs_q[GEMV_WAVES][TILES * GROUP_K]; // this wave's activation quants, block jj at 32*jj
	__shared__ float xs_d[GEMV_WAVES][TILES * GROUP_BLOCKS];
	__shared__ float red[GEMV_WAVES][64];
	__shared__ int last_flag;

	const int tid	= threadIdx.x;
	const int lane	= tid & 63;
	const int wave	= tid >> 6;
	const int strip = blockIdx.x / splits;
	const int split = blockIdx.x - strip * splits;
	const int slots = splits * GEMV_WAVES;
	const int slot	= split * GEMV_WAVES + wave;
	const int g0	= static_cast<int>((static_cast<int64_t>(groups) * slot) / slots);
	const int g1	= static_cast<int>((static_cast<int64_t>(groups) * (slot + 1)) / slots);
	const int cnt	= g1 - g0; // <= TILES (the host picks splits so)
	const int r		= lane & 31;
	const int half	= lane >> 5;

	// ---- 1. activation slice: raw dwords of blocks [4*g0, 4*g1), 34 dwords per group, issued first ----
	const uint32_t* x_raw = reinterpret_cast<const uint32_t*>(xq + static_cast<int64_t>(g0) * (GROUP_BLOCKS * BLOCK_BYTES));
	constexpr int X_DWORDS = TILES * 34;
	constexpr int X_LOADS  = (X_DWORDS + 63) / 64;
	uint32_t xr[X_LOADS];
#pragma unroll
	for (int i = 0; i < X_LOADS; ++i) {
		const int sidx = lane + 64 * i;
		xr[i]		   = sidx < cnt * 34 ? x_raw[sidx] : 0u;
	}

	// ---- 2. every weight byte this wave will ever need, in flight at once ----
	v4i q[TILES][GROUP_BLOCKS];
	v2u dd[TILES];
	const uint8_t* macro0 = W + macro_offset(strip, g0, groups);
#pragma unroll
	for (int t = 0; t < TILES; ++t) {
		if (t < cnt) {
			const uint8_t* macro = macro0 + static_cast<int64_t>(t) * MACRO_BYTES;
#pragma unroll
			for (int j = 0; j < GROUP_BLOCKS; ++j) {
				q[t][j] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(macro + j * TILE_BYTES + 16 * lane));
			}
			dd[t] = __builtin_nontemporal_load(reinterpret_cast<const v2u*>(macro + MACRO_D_OFFSET + 8 * r));
		}
	}

	// ---- 3. re-align the activation slice into LDS: half-word hw of the raw stream is scale (hw%17 == 0) or a quant pair ----
#pragma unroll
	for (int i = 0; i < X_LOADS; ++i) {
		const int sidx = lane + 64 * i;
		if (sidx < cnt * 34) {
#pragma unroll
			for (int h = 0; h < 2; ++h) {
				const int hw	   = 2 * sidx + h;
				const int jj	   = hw / 17;
				const int o		   = hw - 17 * jj;
				const uint16_t val = static_cast<uint16_t>(h ? (xr[i] >> 16) : (xr[i] & 0xFFFFu));
				if (o == 0) {
					xs_d[wave][jj] = half_bits_to_float(val);
				} else {
					*reinterpret_cast<uint16_t*>(&xs_q[wave][jj * QK + 2 * (o - 1)]) = val;
				}
			}
		}
	}
	__builtin_amdgcn_wave_barrier(); // wave-local hand-off: same wave wrote and reads, the LDS counter wait orders it

	// ---- 4. dot products as the tiles land ----
	float acc = 0.0f;
#pragma unroll
	for (int t = 0; t < TILES; ++t) {
		if (t < cnt) {
			const float dw[GROUP_BLOCKS] = { half_bits_to_float(static_cast<uint16_t>(dd[t].x & 0xFFFFu)), half_bits_to_float(static_cast<uint16_t>(dd[t].x >> 16)),
				half_bits_to_float(static_cast<uint16_t>(dd[t].y & 0xFFFFu)), half_bits_to_float(static_cast<uint16_t>(dd[t].y >> 16)) };
#pragma unroll
			for (int j = 0; j < GROUP_BLOCKS; ++j) {
				const int jj = t * GROUP_BLOCKS + j;
				const v4i xv = *reinterpret_cast<const v4i*>(&xs_q[wave][jj * QK + 16 * half]);
				const int s	 = dot16(q[t][j], xv);
				if constexpr (DUMP) {
					const int full = s + __shfl_xor(s, 32);
					const int row  = strip * STRIP_ROWS + r;
					if (half == 0 && row < N) {
						sums[static_cast<int64_t>(row) * (groups * GROUP_BLOCKS) + (g0 * GROUP_BLOCKS + jj)] = full;
					}
				} else {
					acc = fmaf(static_cast<float>(s), dw[j] * xs_d[wave][jj], acc);
				}
			}
		}
	}
	if constexpr (DUMP) {
		return;
	}

	// ---- 5. one reduction per workgroup, fixed order ----
	red[wave][lane] = acc;
	__syncthreads();
	float total = 0.0f;
	if (tid < STRIP_ROWS) {
#pragma unroll
		for (int w = 0; w < GEMV_WAVES; ++w) {
			total += red[w][tid] + red[w][32 + tid];
		}
	}
	const int row = strip * STRIP_ROWS + tid;
	if (splits == 1) {
		if (tid < STRIP_ROWS && row < N) {
			y[row] = total;
		}
		return;
	}

	// ---- 6. K split over several workgroups: publish partial sums, the last arriver adds them in split order ----
	// Each XCD has its own L2, so data that crosses workgroups goes through device-scope atomic stores and loads
	// (written through to / read from the memory side).  A device-wide fence would also order them, but it writes
	// back and invalidates the whole L2 under the other workgroups' streaming loads; waiting for the stores to be
	// acknowledged before the arrival count is bumped is all the ordering this hand-off needs.
	if (tid < STRIP_ROWS) {
		__hip_atomic_store(&partials[(static_cast<int64_t>(strip) * splits + split) * STRIP_ROWS + tid], total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
	}
	__builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup"); // s_waitcnt only: the stores above have completed
	__syncthreads();
	if (tid == 0) {
		const unsigned prev = __hip_atomic_fetch_add(&counters[strip], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		const int last		= (prev == static_cast<unsigned>(splits - 1));
		if (last) {
			__hip_atomic_store(&counters[strip], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); // all arrived: ready for the next launch
		}
		last_flag = last;
	}
	__syncthreads();
	if (last_flag && tid < STRIP_ROWS && row < N) {
		float sum = 0.0f;
		for (int sp = 0; sp < splits; ++sp) {
			sum += __hip_atomic_load(&partials[(static_cast<int64_t>(strip) * splits + sp) * STRIP_ROWS + tid], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		}
		y[row] = sum;
	}
}

// Scratch of the K-split path: partial sums and arrival counters, one allocation per device, made on first use
// and kept for the life of the process.  Calls that overlap on one GPU (different streams) and both split K race on it.
constexpr int GEMV_MAX_SPLIT_UNITS = 8192; // strips * splits when splits > 1
constexpr int GEMV_MAX_SPLIT_STRIPS = 512;
struct gemv_scratch {
	float* partials	   = nullptr;
	unsigned* counters = nullptr;
};
static hipError_t get_gemv_scratch(gemv_scratch* out) {
	static std::mutex lock;
	static gemv_scratch per_device[64];
	int dev = 0;
	hipError_t e = hipGetDevice(&dev);
	if (e != hipSuccess) {
		return e;
	}
	if (dev < 0 || dev >= 64) {
		return hipErrorInvalidDevice;
	}
	std::lock_guard<std::mutex> g(lock);
	gemv_scratch& sc = per_device[dev];
	if (!sc.partials) {
		void* p			   = nullptr;
		const size_t bytes = static_cast<size_t>(GEMV_MAX_SPLIT_UNITS) * STRIP_ROWS * 4 + GEMV_MAX_SPLIT_STRIPS * 4;
		e				   = hipMalloc(&p, bytes);
		if (e != hipSuccess) {
			return e;
		}
		e = hipMemset(p, 0, bytes); // synchronous, once: counters start at zero and every launch leaves them at zero
		if (e != hipSuccess) {
			(void)hipFree(p);
			return e;
		}
		sc.partials = static_cast<float*>(p);
		sc.counters = reinterpret_cast<unsigned*>(sc.partials + static_cast<size_t>(GEMV_MAX_SPLIT_UNITS) * STRIP_ROWS);
	}
	*out = sc;
	return hipSuccess;
}

// How a [N x K] tiled mat-vec is cut: `splits` workgroups per strip, each of 16 waves owning <= `tiles` groups.
struct gemv_plan {
	int strips, groups, splits, tiles;
};
static gemv_plan plan_gemv(int64_t N, int64_t K) {
	gemv_plan p;
	p.strips = static_cast<int>((N + STRIP_ROWS - 1) / STRIP_ROWS);
	p.groups = static_cast<int>(K / GROUP_K);
	p.splits = 1;
	auto tiles_for = [&](int s) { return (p.groups + GEMV_WAVES * s - 1) / (GEMV_WAVES * s); };
	// split further while a wave would own more than 4 groups, or while the grid cannot cover the chip and waves still own > 1 group
	while ((tiles_for(p.splits) > 4 || (p.strips * p.splits < 256 && GEMV_WAVES * p.splits < p.groups)) && p.strips * p.splits * 2 <= GEMV_MAX_SPLIT_UNITS && p.strips <= GEMV_MAX_SPLIT_STRIPS) {
		p.splits *= 2;
	}
	p.tiles = tiles_for(p.splits);
	return p;
}

template<int TILES> static hipError_t launch_gemv_tiled_t(const gemv_plan& p, const uint8_t* W, const uint8_t* xq, float* y, int32_t* sums, const gemv_scratch& sc, int N, hipStream_t s) {
	const dim3 grid(static_cast<unsigned>(p.strips * p.splits)), block(GEMV_WAVES * 64);
	if (sums) {
		gemv_tiled_kernel<TILES, true><<<grid, block, 0, s>>>(W, xq, y, sums, sc.partials, sc.counters, N, p.groups, p.splits);
		return hipGetLastError();
	}
	return launch_kernel(KIND_GEMV, gemv_tiled_kernel<TILES, false>, grid, block, 0, s, W, xq, y, sums, sc.partials, sc.counters, N, p.groups, p.splits);
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
		const gemv_plan p = plan_gemv(N, K);
		if (p.tiles <= 4) {
			gemv_scratch sc;
			if (p.splits > 1) {
				const hipError_t e = get_gemv_scratch(&sc);
				if (e != hipSuccess) {
					return e;
				}
			}
			const int n = static_cast<int>(N);
			switch (p.tiles) {
				case 1:
					return launch_gemv_tiled_t<1>(p, w, x, y, sums, sc, n, s);
				case 2:
					return launch_gemv_tiled_t<2>(p, w, x, y, sums, sc, n, s);
				default:
					return launch_gemv_tiled_t<4>(p, w, x, y, sums, sc, n, s);
			}
		}
		// K too long to split within the scratch limits: the looping kernel takes it
		return launch_gemv_t<4, true>(w, x, y, sums, static_cast<int>(N), static_cast<int>(K), s);
	}
	return launch_gemv_t<4, false>(w, x, y, sums, static_cast<int>(N), static_cast<int>(K), s);
}

} // namespace nh
