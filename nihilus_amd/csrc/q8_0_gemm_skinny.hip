// Batched-decode mat-mat for a handful of activation rows (M <= 64): C[m][n] = dot(W row n, Aq row m), gfx950.
//
// With so few rows the weights are read once and nothing is reused enough to leave the HBM roofline, so this is the
// streaming mat-vec again -- one workgroup per (32-row weight strip, K split), waves splitting the strip's K range,
// all of a chunk's loads issued before anything is waited for, one fixed-order reduction at the end -- with the
// v_dot4 inner product replaced by the int8 MFMA: the weight tile a wave fetches (one coalesced 16-byte-per-lane load
// in the tiled layout) is the B operand as it stands, the matching activation tile (served by L2: the activations
// are M*K bytes) is the A operand, and one v_mfma_i32_32x32x32_i8 yields the exact block sums of 32 rows x 32
// columns.  Scale products come from a v_mfma_f32_32x32x8_f16 on the blocks' fp16 scales (exact, same register layout),
// then one convert + one multiply-add per value.  Same arithmetic as the prefill kernel (reference
// vec_dot_q8_0_q8_0, cpu/avx_2.hpp:4534-4747; output [M][N], n fastest, cpu/avx_2.hpp:4934).
#include "q8_0_plan.h"

#include <mutex>

namespace nh {

typedef _Float16 sk_v4h __attribute__((ext_vector_type(4)));
typedef float sk_v16f __attribute__((ext_vector_type(16)));

// fp16 scale of block t (0..3) from a row's four packed scales, as the f16 MFMA's k = 0 slot: {d_t, 0, 0, 0}
__device__ __forceinline__ v2u scale_slot(v2u four, int t) {
	const uint32_t dword = (t < 2) ? four.x : four.y;
	return v2u{ (t & 1) ? (dword >> 16) : (dword & 0xFFFFu), 0u };
}

template<int MS, bool DUMP, int GC>
__global__ __launch_bounds__(SK_WAVES * 64, DUMP ? 2 : 4) void gemm_skinny_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ A, float* C, const float* R, int32_t* __restrict__ sums,
	float* __restrict__ partials, unsigned* __restrict__ counters, int M, int N, int groups, int split_shift) {
	__shared__ float red[SK_WAVES / 2][MS][16][64];
	__shared__ int last_flag;

	const int tid	 = threadIdx.x;
	const int lane	 = tid & 63;
	const int wave	 = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int splits = 1 << split_shift;
	const int strip	 = static_cast<int>(blockIdx.x >> split_shift);
	const int split	 = static_cast<int>(blockIdx.x) & (splits - 1);
	const int mg	 = static_cast<int>(blockIdx.y); // group of MS activation strips (more than 32 * MS rows: the weights are read once per group, from cache after the first)
	const int unit	 = mg * static_cast<int>(gridDim.x >> split_shift) + strip; // index of this (row group, weight strip) in the split scratch
	int g0, g1; // this wave's share of the strip's K range
	wave_k_range(groups, split_shift, split, SK_WAVES, wave, g0, g1);
	const int r		 = lane & 31;
	const int half	 = lane >> 5;

	sk_v16f acc[MS];
#pragma unroll
	for (int i = 0; i < MS; ++i) {
		acc[i] = sk_v16f{ 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 };
	}

	const uint8_t* w_strip = W + macro_offset(strip, 0, groups);
	struct w_regs {
		v4i q[GROUP_BLOCKS];
		v2u d;
	};
	struct a_regs {
		v4i q[MS][GROUP_BLOCKS];
		v2u d[MS];
	};
	auto issue_w = [&](int g, w_regs& b) {
		const uint8_t* macro = w_strip + static_cast<int64_t>(g) * MACRO_BYTES;
#pragma unroll
		for (int j = 0; j < GROUP_BLOCKS; ++j) {
			b.q[j] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(macro + j * TILE_BYTES + 16 * lane));
		}
		b.d = __builtin_nontemporal_load(reinterpret_cast<const v2u*>(macro + MACRO_D_OFFSET + 8 * r));
	};
	// Activation rows beyond M are zero padding in the tiled operand.  Their lanes all read the strip's last row instead of
	// their own (zeros as well, since a strip with any padding ends in it): one cache line per load instead of one per four
	// lanes, so a batch of 4 rows costs a fraction of the cache traffic of a full strip, with no extra registers or branches.
	int a_q_off[MS], a_d_off[MS];
#pragma unroll
	for (int i = 0; i < MS; ++i) {
		const bool real = (mg * MS + i) * STRIP_ROWS + r < M;
		a_q_off[i]		= real ? 16 * lane : 16 * (STRIP_ROWS - 1);
		a_d_off[i]		= real ? 8 * r : 8 * (STRIP_ROWS - 1);
	}
	auto issue_a = [&](int g, a_regs& b) {
#pragma unroll
		for (int i = 0; i < MS; ++i) {
			const uint8_t* am = A + macro_offset(mg * MS + i, g, groups);
#pragma unroll
			for (int j = 0; j < GROUP_BLOCKS; ++j) {
				b.q[i][j] = *reinterpret_cast<const v4i*>(am + j * TILE_BYTES + a_q_off[i]);
			}
			b.d[i] = *reinterpret_cast<const v2u*>(am + MACRO_D_OFFSET + a_d_off[i]);
		}
	};
	auto compute = [&](int g, const w_regs& w, const a_regs& a) {
		// lanes 32..63 feed the k = 4..7 slots of the scale MFMA: zero
		const v2u wdz = half ? v2u{ 0u, 0u } : w.d;
#pragma unroll
		for (int j = 0; j < GROUP_BLOCKS; ++j) {
			const v2u ws = scale_slot(wdz, j);
#pragma unroll
			for (int i = 0; i < MS; ++i) {
				const sk_v16f zf = { 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 };
				const v16i zi	 = { 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 };
				const v16i s	 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a.q[i][j], w.q[j], zi, 0, 0, 0);
				if constexpr (DUMP) {
					const int n = strip * STRIP_ROWS + r;
#pragma unroll
					for (int e = 0; e < 16; ++e) {
						const int m = (mg * MS + i) * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
						if (m < M && n < N) {
							sums[(static_cast<int64_t>(m) * N + n) * (groups * GROUP_BLOCKS) + (g * GROUP_BLOCKS + j)] = s[e];
						}
					}
				} else {
					const v2u as	= scale_slot(half ? v2u{ 0u, 0u } : a.d[i], j);
					const sk_v16f p = __builtin_amdgcn_mfma_f32_32x32x8f16(__builtin_bit_cast(sk_v4h, as), __builtin_bit_cast(sk_v4h, ws), zf, 0, 0, 0);
#pragma unroll
					for (int e = 0; e < 16; ++e) {
						acc[i][e] = fmaf(static_cast<float>(s[e]), p[e], acc[i][e]);
					}
				}
			}
		}
	};
	// GC groups per step: their loads are issued, then waited for together (loads complete in issue order, so a
	// short-latency activation load queued behind a weight load returns no earlier than it: prefetching one kind deeper
	// than the other buys nothing), then computed.  (The compiler sinks the second group's loads into the branch that
	// uses them, behind the first group's MFMAs; holding them in front, and one group per step, both measured the same
	// within 0.3 us on every shape of the crossover and 70B tables: the eight waves of two workgroups per CU are what
	// keeps bytes in flight, not the depth of one wave.)
	for (int g = g0; g < g1; g += GC) {
		w_regs w[GC];
		a_regs a[GC];
#pragma unroll
		for (int c = 0; c < GC; ++c) {
			issue_w(min(g + c, g1 - 1), w[c]); // past the end: the last group again (a cache hit, never used) so that the waits stay countable
		}
#pragma unroll
		for (int c = 0; c < GC; ++c) {
			issue_a(min(g + c, g1 - 1), a[c]);
		}
		__builtin_amdgcn_sched_barrier(0); // every load of the step before the first MFMA (left alone, the compiler interleaves them: measured slower)
#pragma unroll
		for (int c = 0; c < GC; ++c) {
			if (c == 0 || g + c < g1) {
				compute(g + c, w[c], a[c]);
			}
		}
	}
	if constexpr (DUMP) {
		return;
	}

	// ---- fixed-order tree reduction over the workgroup's waves ----
#pragma unroll
	for (int s = SK_WAVES / 2; s >= 1; s >>= 1) {
		if (wave >= s && wave < 2 * s) {
#pragma unroll
			for (int i = 0; i < MS; ++i) {
#pragma unroll
				for (int e = 0; e < 16; ++e) {
					red[wave - s][i][e][lane] = acc[i][e];
				}
			}
		}
		__syncthreads();
		if (wave < s) {
#pragma unroll
			for (int i = 0; i < MS; ++i) {
#pragma unroll
				for (int e = 0; e < 16; ++e) {
					acc[i][e] += red[wave][i][e][lane];
				}
			}
		}
		__syncthreads();
	}

	const int n = strip * STRIP_ROWS + r;
	if (splits == 1) {
		if (wave == 0 && n < N) {
#pragma unroll
			for (int i = 0; i < MS; ++i) {
#pragma unroll
				for (int e = 0; e < 16; ++e) {
					const int m = (mg * MS + i) * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
					if (m < M) {
						const int64_t at = static_cast<int64_t>(m) * N + n;
						C[at]			 = R ? acc[i][e] + R[at] : acc[i][e]; // R may be C: read before the write, by the same thread
					}
				}
			}
		}
		return;
	}

	// ---- K split over several workgroups: partial tiles through device-scope atomics, last arriver adds in split order ----
	float* mine = partials + (static_cast<int64_t>(unit) * splits + split) * (MS * 16 * 64);
	if (wave == 0) {
#pragma unroll
		for (int i = 0; i < MS; ++i) {
#pragma unroll
			for (int e = 0; e < 16; ++e) {
				__hip_atomic_store(&mine[(i * 16 + e) * 64 + lane], acc[i][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
			}
		}
	}
	wait_stores_acknowledged();
	__syncthreads();
	if (tid == 0) {
		const unsigned prev = __hip_atomic_fetch_add(&counters[unit], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		const int last		= (prev == static_cast<unsigned>(splits - 1));
		if (last) {
			__hip_atomic_store(&counters[unit], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		}
		last_flag = last;
	}
	__syncthreads();
	if (last_flag && wave == 0 && n < N) {
		// two splits' worth of partial tiles requested at a time (32 loads per lane in flight), added in split order
		sk_v16f sum[MS];
#pragma unroll
		for (int i = 0; i < MS; ++i) {
			sum[i] = sk_v16f{ 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 };
		}
		const float* base = partials + static_cast<int64_t>(unit) * splits * (MS * 16 * 64) + lane;
#pragma unroll
		for (int i = 0; i < MS; ++i) {
			for (int sp0 = 0; sp0 < splits; sp0 += 2) {
				float v[2][16];
#pragma unroll
				for (int u = 0; u < 2; ++u) {
#pragma unroll
					for (int e = 0; e < 16; ++e) {
						v[u][e] = (sp0 + u < splits) ? __hip_atomic_load(&base[(static_cast<int64_t>(sp0 + u) * (MS * 16) + (i * 16 + e)) * 64], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0.0f;
					}
				}
#pragma unroll
				for (int u = 0; u < 2; ++u) {
					if (sp0 + u < splits) {
#pragma unroll
						for (int e = 0; e < 16; ++e) {
							sum[i][e] += v[u][e];
						}
					}
				}
			}
#pragma unroll
			for (int e = 0; e < 16; ++e) {
				const int m = (mg * MS + i) * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
				if (m < M) {
					const int64_t at = static_cast<int64_t>(m) * N + n;
					C[at]			 = R ? sum[i][e] + R[at] : sum[i][e];
				}
			}
		}
	}
}

// Scratch of the K-split path (partial 32x32 tiles and arrival counters): one allocation per device on first use.
static_assert(GEMM_SPLIT_SCRATCH_FLOATS == SK_MAX_SPLIT_UNITS * 2 * 16 * 64 && GEMM_SPLIT_MAX_UNITS == SK_MAX_SPLIT_STRIPS, "one scratch, two users");
struct skinny_scratch {
	float* partials	   = nullptr;
	unsigned* counters = nullptr;
	hipStream_t user   = nullptr; // stream of the last K-split launch
	bool has_user	   = false;
};
// launching = true: a K-split launch on `s` is about to use the scratch.  It serves one stream at a time: if the previous such
// launch went to another stream that has not drained, hipErrorNotReady comes back (NH_ERR_BUSY at the C ABI).  Not checked for
// capturing streams or after a launch on the null stream (neither may be queried safely).
static hipError_t get_skinny_scratch(skinny_scratch* out, bool launching = false, hipStream_t s = nullptr) {
	static std::mutex lock;
	static skinny_scratch per_device[64];
	int dev		 = 0;
	hipError_t e = hipGetDevice(&dev);
	if (e != hipSuccess) {
		return e;
	}
	if (dev < 0 || dev >= 64) {
		return hipErrorInvalidDevice;
	}
	std::lock_guard<std::mutex> g(lock);
	skinny_scratch& sc = per_device[dev];
	if (!sc.partials) {
		void* p			   = nullptr;
		const size_t tiles = static_cast<size_t>(SK_MAX_SPLIT_UNITS) * 2 * 16 * 64 * 4; // two 32-row activation strips at most
		const size_t bytes = tiles + SK_MAX_SPLIT_STRIPS * 4;
		e				   = hipMalloc(&p, bytes);
		if (e != hipSuccess) {
			return e;
		}
		e = hipMemset(p, 0, bytes);
		if (e != hipSuccess) {
			(void)hipFree(p);
			return e;
		}
		sc.partials = static_cast<float*>(p);
		sc.counters = reinterpret_cast<unsigned*>(static_cast<uint8_t*>(p) + tiles);
	}
	if (launching && !stream_is_capturing(s)) {
		if (sc.has_user && sc.user != s && sc.user != nullptr && !stream_is_capturing(sc.user)) {
			const hipError_t q = query_stream_any_capture_mode(sc.user);
			if (q == hipErrorNotReady) {
				return q;
			}
			if (q != hipSuccess) {
				(void)hipGetLastError();
			}
		}
		sc.user		= s;
		sc.has_user = true;
	}
	*out = sc;
	return hipSuccess;
}

// The same scratch for the tile kernel's K split over workgroups (GEMM_SPLIT_SCRATCH_FLOATS floats of tiles, GEMM_SPLIT_MAX_UNITS
// counters that every launch leaves at zero); same one-stream rule.
hipError_t acquire_gemm_split_scratch(float** partials, unsigned** counters, hipStream_t s) {
	skinny_scratch sc;
	const hipError_t e = get_skinny_scratch(&sc, true, s);
	if (e != hipSuccess) {
		return e;
	}
	*partials = sc.partials;
	*counters = sc.counters;
	return hipSuccess;
}

hipError_t prepare_gemm_scratch() {
	skinny_scratch sc;
	return get_skinny_scratch(&sc);
}

template<int MS> static hipError_t launch_skinny_t(int splits, const uint8_t* w, const uint8_t* a, float* C, const float* R, int32_t* sums, int m, int n, int groups, hipStream_t s) {
	const int strips   = (n + STRIP_ROWS - 1) / STRIP_ROWS;
	const int m_groups = ((m + STRIP_ROWS - 1) / STRIP_ROWS + MS - 1) / MS;
	skinny_scratch sc;
	if (splits > 1) {
		const hipError_t e = get_skinny_scratch(&sc, true, s);
		if (e != hipSuccess) {
			return e;
		}
	}
	int shift = 0;
	while ((1 << shift) < splits) {
		++shift;
	}
	const dim3 grid(static_cast<unsigned>(strips * splits), static_cast<unsigned>(m_groups)), block(SK_WAVES * 64);
	if (sums) {
		gemm_skinny_kernel<MS, true, 1><<<grid, block, 0, s>>>(w, a, C, R, sums, sc.partials, sc.counters, m, n, groups, shift);
		return hipGetLastError();
	}
	return launch_kernel(KIND_GEMM, gemm_skinny_kernel<MS, false, 2>, grid, block, 0, s, w, a, C, R, sums, sc.partials, sc.counters, m, n, groups, shift);
}

hipError_t launch_gemm_skinny(const void* W, const void* Aq, float* C, int32_t* sums, int64_t M, int64_t N, int64_t K, hipStream_t s, const float* residual) {
	const uint8_t* w = static_cast<const uint8_t*>(W);
	const uint8_t* a = static_cast<const uint8_t*>(Aq);
	const int groups = static_cast<int>(K / GROUP_K);
	const gemm_skinny_cut cut = plan_gemm_skinny(M, N, K); // activation strips per workgroup, workgroups per strip: q8_0_plan.h
	if (cut.ms == 1) {
		return launch_skinny_t<1>(cut.splits, w, a, C, residual, sums, static_cast<int>(M), static_cast<int>(N), groups, s);
	}
	return launch_skinny_t<2>(cut.splits, w, a, C, residual, sums, static_cast<int>(M), static_cast<int>(N), groups, s);
}

} // namespace nh
