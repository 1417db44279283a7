// Decode mat-vec y = W . xq for Q8_0 weights and a Q8_0-quantized activation row, gfx950.
//
// Computes vec_dot_q8_0_q8_0 (reference cpu/avx_2.hpp:4534-4747) for every weight row:
//   y[n] = sum_b f32(dW[n][b]) * f32(dx[b]) * (sum_j W.qs[n][b][j] * x.qs[b][j])
// with exact int32 block sums (v_dot4_i32_i8) and fp32 scale-and-accumulate.  HBM-bound: 34 bytes of weight
// per 32 multiply-adds, each read exactly once.
//
// Two kernels:
//   gemv_blocks_kernel  reads the reference's packed 34-byte blocks as they are (unaligned 16-byte loads):
//                       the drop-in-on-raw-bytes form, and the parity twin of the streaming kernel;
//   gemv_tiled_kernel   the streaming kernel on the tiled layout -- the one the decode path runs.
// In both, lane l accumulates row (l % 32), quants 16*(l/32).. of every block, so the loop needs no cross-lane
// reduction; halves and waves are combined once through LDS in a fixed order (run-to-run bit-stable).
#include "q8_0_plan.h"

#include <atomic>
#include <mutex>

namespace nh {

template<int WAVES, bool DUMP>
__global__ __launch_bounds__(WAVES * 64) void gemv_blocks_kernel(const uint8_t* __restrict__ W, const uint8_t* __restrict__ xq, float* __restrict__ y, int32_t* __restrict__ sums, int N, int K) {
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
	const uint8_t* w_row	= W + row_c * row_bytes;

	float acc = 0.0f;
	for (int g = wave; g < groups; g += WAVES) {
		v4i q[GROUP_BLOCKS];
		float dw[GROUP_BLOCKS];
#pragma unroll
		for (int t = 0; t < GROUP_BLOCKS; ++t) {
			const int b		   = min(g * GROUP_BLOCKS + t, nb - 1); // ragged last group: clamped, masked below
			const uint8_t* blk = w_row + static_cast<int64_t>(b) * BLOCK_BYTES;
			q[t]			   = load16_unaligned(blk + 2 + 16 * half);
			dw[t]			   = half_bits_to_float(load_u16(blk));
		}
#pragma unroll
		for (int t = 0; t < GROUP_BLOCKS; ++t) {
			const int b = g * GROUP_BLOCKS + t;
			if (b < nb) {
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
//   * its slice of the activation row is staged wave-locally while the weight loads fly, either re-aligned
//     from packed 34-byte blocks (XF32 = false) or quantized on the spot from the fp32 activations with the
//     very arithmetic of the stand-alone quantize kernel (XF32 = true: no separate quantize launch, no
//     round trip of the quantized row through memory); it is read back as 16-byte two-address broadcasts
//     (only the wave's own LDS counter is waited on, never a barrier);
//   * one LDS reduction per workgroup; when K is split over several workgroups (few rows, long K) each writes
//     32 partial sums and the last to arrive adds them in split order -- fixed order, so results do not
//     depend on arrival order;
//   * up to three weight matrices that share K and the activation row (q/k/v, gate/up) run as one launch:
//     a bigger launch amortises the ramp-up and the tail.
//   * RS > 1: a strip is shared by RS workgroups that own 32 / RS of its rows each and all of K (see gemv_chunk_n): how a
//     matrix with few rows reaches every CU without partial sums.
template<int TILES, bool XF32, int DUMP, bool LOOP, bool NORM, int RS = 1>
__global__ __launch_bounds__(GEMV_WAVES * 64) void gemv_tiled_kernel(gemv_segments seg, const void* __restrict__ xin, void* __restrict__ dump, uint64_t* __restrict__ tagged,
	unsigned epoch, int groups, int split_shift, const float* __restrict__ norm_w, float norm_eps, uint64_t* __restrict__ x_words, unsigned* error_word, int spin_limit) {
	__shared__ __align__(16) uint8_t xs_q[GEMV_WAVES][TILES * GROUP_K]; // each wave's activation quants, block jj at 32*jj
	__shared__ float norm_red[16];
	__shared__ float4 xs_w[NORM ? GEMV_WAVES : 1][NORM ? TILES * 32 : 1]; // each wave's slice of the norm weights
	__shared__ float xs_d[GEMV_WAVES][TILES * GROUP_BLOCKS];
	__shared__ float red[GEMV_WAVES][64];
	const int tid	 = threadIdx.x;
	const int lane	 = tid & 63;
	const int wave	 = __builtin_amdgcn_readfirstlane(tid >> 6); // wave-uniform by construction: keep it (and all that follows from it) scalar
	const int splits  = RS > 1 ? 1 : 1 << split_shift; // a power of two: no integer division anywhere on the way to the first load
	const int gstrip  = RS > 1 ? static_cast<int>(blockIdx.x / RS) : static_cast<int>(blockIdx.x >> split_shift); // strip index over all segments
	const int split	  = RS > 1 ? 0 : static_cast<int>(blockIdx.x) & (splits - 1);
	const int rowpart = RS > 1 ? static_cast<int>(blockIdx.x % RS) : 0; // which 32 / RS rows of the strip
	const int sidx	 = (gstrip >= seg.strip_end[0]) + (gstrip >= seg.strip_end[1]);
	const int strip	 = gstrip - (sidx == 0 ? 0 : seg.strip_end[sidx - 1]);
	const int N		 = seg.rows[sidx];
	int g0, g1; // this wave's share of the strip's K range
	wave_k_range(groups, RS > 1 ? 0 : split_shift, split, GEMV_WAVES, wave, g0, g1);

	const uint8_t* w_strip = DUMP == DUMP_X ? nullptr : seg.W[sidx] + macro_offset(strip, 0, groups);
	const int row_l		   = strip * STRIP_ROWS + (lane & 31);
	float acc			   = 0.0f;
	// the wave's K range, in one piece when the host picked splits so that g1 - g0 <= TILES (straight-line code, every load of the
	// wave in flight at once), else walked in chunks of TILES groups (K too long for that within the host's scratch limits)
	auto walk = [&]<int XMODE, bool WITH_NORM>(const void* x_from, void* dump_to, gemv_norm* norm) {
		if constexpr (!LOOP) {
			return gemv_chunk<TILES, XMODE, DUMP, WITH_NORM, RS>(w_strip, x_from, dump_to, xs_q[wave], xs_d[wave], g0, g1 - g0, groups, lane, row_l, N, gstrip == 0, epoch, norm, rowpart, spin_limit);
		} else {
			float sum = 0.0f;
			for (int gc = g0; gc < g1; gc += TILES) {
				sum += gemv_chunk<TILES, XMODE, DUMP, WITH_NORM, RS>(w_strip, x_from, dump_to, xs_q[wave], xs_d[wave], gc, min(TILES, g1 - gc), groups, lane, row_l, N, gstrip == 0, epoch, norm, rowpart, spin_limit);
				__builtin_amdgcn_wave_barrier(); // the next chunk overwrites this wave's LDS slice
			}
			return sum;
		}
	};
	if constexpr (NORM) {
		// RMS norm * weight in front of the quantizer.  With x_words the row is normalised and quantized once per launch: by the
		// workgroups of the first strip (one per K split, each on its K range; the first workgroup alone when strips are cut by
		// rows), which publish what they stage; everybody else reads it from there.
		bool works_it_out = true;
		if constexpr (DUMP == DUMP_NONE) { // (the inspection variants never share)
			works_it_out = !x_words || (RS > 1 ? blockIdx.x == 0 : gstrip == 0);
		}
		if (works_it_out) {
			gemv_norm norm_state; // the row's scale first (a workgroup barrier inside)
			gemv_norm_begin(norm_state, static_cast<const float*>(xin), norm_w, xs_w[NORM ? wave : 0], norm_red, norm_eps, groups * GROUP_K, lane, wave);
			norm_state.publish = x_words;
			norm_state.epoch   = epoch;
			acc				   = walk.template operator()<XF32 ? X_F32 : X_BLOCKS, true>(xin, dump, &norm_state);
		} else if constexpr (DUMP == DUMP_NONE) {
			acc = walk.template operator()<X_PUBLISHED_EARLY_WATCH, false>(x_words, error_word, nullptr);
		}
	} else if constexpr (!LOOP) {
		acc = gemv_chunk<TILES, XF32, DUMP, false, RS>(w_strip, xin, dump, xs_q[wave], xs_d[wave], g0, g1 - g0, groups, lane, row_l, N, gstrip == 0, 0, nullptr, rowpart);
	} else {
		for (int gc = g0; gc < g1; gc += TILES) {
			acc += gemv_chunk<TILES, XF32, DUMP, false, RS>(w_strip, xin, dump, xs_q[wave], xs_d[wave], gc, min(TILES, g1 - gc), groups, lane, row_l, N, gstrip == 0, 0, nullptr, rowpart);
			__builtin_amdgcn_wave_barrier(); // the next chunk overwrites this wave's LDS slice
		}
	}
	if constexpr (DUMP != DUMP_NONE) {
		return;
	}

	// ---- one reduction per workgroup, fixed order ----
	red[wave][lane] = acc;
	__syncthreads();
	constexpr int PART_ROWS = STRIP_ROWS / RS; // rows this workgroup owns: 64 / PART_ROWS lanes of every wave hold a share of each
	float total				= 0.0f;
	if (tid < PART_ROWS) {
#pragma unroll
		for (int w = 0; w < GEMV_WAVES; ++w) {
			float part = 0.0f; // this wave's shares of the row, then the waves in order
#pragma unroll
			for (int c = 0; c < 64 / PART_ROWS; ++c) {
				part += red[w][c * PART_ROWS + tid];
			}
			total += part;
		}
	}
	const int row = strip * STRIP_ROWS + rowpart * PART_ROWS + tid;
	float* y		  = seg.y[sidx];
	const float* res  = seg.residual[sidx];
	if (splits == 1) {
		if (tid < PART_ROWS && row < N) {
			y[row] = res ? total + res[row] : total;
		}
		return;
	}

	// ---- K split over several workgroups ----
	if (tid < STRIP_ROWS) {
		split_k_finish(tagged, epoch, gstrip, splits, split, tid, total, y, row, N, res);
	}
}

namespace {
	struct scratch_state {
		gemv_scratch sc;
		hipStream_t user = nullptr; // stream of the last launch that used the scratch
		bool has_user	 = false;
	};
	std::mutex scratch_lock;
	scratch_state scratch_per_device[64];
	int published_spin_limit = PUBLISHED_SPIN_LIMIT;

	// hipErrorNotReady when `prev` still has work in flight; anything else (a destroyed stream, a capturing one) counts as drained
	hipError_t stream_drained(hipStream_t prev) {
		if (stream_is_capturing(prev)) {
			return hipSuccess; // must not be queried; its launches take forms that keep no state in the scratch
		}
		const hipError_t q = query_stream_any_capture_mode(prev);
		if (q == hipErrorNotReady) {
			return q;
		}
		if (q != hipSuccess) {
			(void)hipGetLastError();
		}
		return hipSuccess;
	}
} // namespace

hipError_t get_gemv_scratch(gemv_scratch* out, bool next_epoch, hipStream_t s) {
	int dev		 = 0;
	hipError_t e = hipGetDevice(&dev);
	if (e != hipSuccess) {
		return e;
	}
	if (dev < 0 || dev >= 64) {
		return hipErrorInvalidDevice;
	}
	std::lock_guard<std::mutex> g(scratch_lock);
	scratch_state& st = scratch_per_device[dev];
	gemv_scratch& sc  = st.sc;
	if (!sc.tagged) {
		void* p			   = nullptr;
		const size_t blocks_end = static_cast<size_t>(GEMV_MAX_SPLIT_UNITS) * STRIP_ROWS * 8 + 2 * FFN_MAX_HIDDEN * 4 + (FFN_MAX_HIDDEN / STRIP_ROWS) * PUBLISHED_WORDS * 8 + (FFN_MAX_HIDDEN / QK) * BLOCK_BYTES;
		const size_t x_words_at = (blocks_end + 255) / 256 * 256;
		const size_t rows_at	= x_words_at + static_cast<size_t>(GEMV_SHARED_X_MAX_K / QK) * PUBLISHED_WORDS * 8; // a multiple of 256
		const size_t next_at	= rows_at + 2 * static_cast<size_t>(CHAIN_MAX_EMBD) * 8;
		const size_t bytes		= next_at + static_cast<size_t>(CHAIN_MAX_EMBD / QK) * PUBLISHED_WORDS * 8;
		e				   = hipMalloc(&p, bytes);
		if (e != hipSuccess) {
			return e;
		}
		e = hipMemset(p, 0, bytes); // synchronous, once: every tag and flag starts at epoch 0, which no launch uses
		void* word = nullptr;
		if (e == hipSuccess) {
			e = hipHostMalloc(&word, 64, hipHostMallocDefault); // pinned, device-visible under the same address
		}
		if (e != hipSuccess) {
			(void)hipFree(p);
			return e;
		}
		*static_cast<volatile unsigned*>(word) = DEVICE_ERROR_NONE;
		sc.tagged	  = static_cast<uint64_t*>(p);
		sc.gate_up	  = reinterpret_cast<float*>(sc.tagged + static_cast<size_t>(GEMV_MAX_SPLIT_UNITS) * STRIP_ROWS);
		sc.act_words  = reinterpret_cast<uint64_t*>(sc.gate_up + 2 * FFN_MAX_HIDDEN);
		sc.act_blocks = reinterpret_cast<uint8_t*>(sc.act_words + (FFN_MAX_HIDDEN / STRIP_ROWS) * PUBLISHED_WORDS); // 16-byte aligned: every part before it is a multiple of 16 bytes
		sc.x_words	  = reinterpret_cast<uint64_t*>(static_cast<uint8_t*>(p) + x_words_at);
		sc.row_tagged[0] = reinterpret_cast<uint64_t*>(static_cast<uint8_t*>(p) + rows_at);
		sc.row_tagged[1] = sc.row_tagged[0] + CHAIN_MAX_EMBD;
		sc.x_words_next	 = reinterpret_cast<uint64_t*>(static_cast<uint8_t*>(p) + next_at);
		sc.error_word = static_cast<unsigned*>(word);
	}
	if (next_epoch) {
		if (!stream_is_capturing(s)) {
			if (st.has_user && st.user != s && st.user != nullptr) {
				e = stream_drained(st.user);
				if (e != hipSuccess) {
					return e; // hipErrorNotReady: another stream's launch may still be using the scratch
				}
			}
			st.user		= s;
			st.has_user = true;
		}
		++sc.epoch; // tags start at zero and the first epoch handed out is 1
		if (sc.epoch == 0) {
			++sc.epoch;
		}
	}
	sc.spin_limit = published_spin_limit;
	*out		  = sc;
	return hipSuccess;
}

unsigned read_device_error(bool clear) {
	int dev = 0;
	if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
		(void)hipGetLastError();
		return DEVICE_ERROR_NONE;
	}
	std::lock_guard<std::mutex> g(scratch_lock);
	unsigned* word = scratch_per_device[dev].sc.error_word;
	if (!word) {
		return DEVICE_ERROR_NONE;
	}
	return clear ? __atomic_exchange_n(word, static_cast<unsigned>(DEVICE_ERROR_NONE), __ATOMIC_RELAXED) : __atomic_load_n(word, __ATOMIC_RELAXED);
}

namespace {
	std::atomic<bool> in_kernel_waits{ true };
}
bool in_kernel_waits_enabled() {
	return in_kernel_waits.load(std::memory_order_relaxed);
}
bool set_in_kernel_waits(bool enabled) {
	return in_kernel_waits.exchange(enabled, std::memory_order_relaxed);
}

void set_published_spin_limit(int limit) {
	std::lock_guard<std::mutex> g(scratch_lock);
	published_spin_limit = limit < 1 ? 1 : (limit > PUBLISHED_SPIN_LIMIT ? PUBLISHED_SPIN_LIMIT : limit);
}

hipError_t prepare_gemv_scratch() {
	gemv_scratch sc;
	return get_gemv_scratch(&sc);
}

// ---- the mat-vec for callers that must not allocate -------------------------------------------------------------
// Same kernels, same cut, same hand-off; the tagged partial sums of a K split live in a device array that is part of the
// code object instead of a buffer made with hipMalloc.  Every GPU the library runs on holds its own copy of the array
// at its own address for the life of the process; its name below is only the host-side handle for hipGetSymbolAddress.
constexpr int NOALLOC_MAX_SPLIT_UNITS = 2048; // (strip, split) slots: 512 KiB
static __device__ __align__(256) uint64_t scratch[NOALLOC_MAX_SPLIT_UNITS * STRIP_ROWS];

__global__ void clear_tags_kernel(uint64_t* __restrict__ p, int n) {
	const int i = static_cast<int>(blockIdx.x * blockDim.x + threadIdx.x);
	if (i < n) {
		p[i] = 0ull;
	}
}

// The array's device address and the next epoch, per device.  First use on a device (that device current): look the
// address up, then set every tag to zero, the one value no launch uses as its epoch (a fill kernel, not a memset node).
// Calls that overlap on one GPU share the array and would race on it, like the calls that share the allocated scratch: the
// same one-stream-at-a-time rule applies (hipErrorNotReady while the previous user's stream, a different one, has work in
// flight; the query allocates nothing).
static hipError_t get_noalloc_scratch(gemv_scratch* out, hipStream_t s) {
	struct state {
		uint64_t* ptr  = nullptr;
		unsigned epoch = 0;
		hipStream_t user = nullptr; // stream of the last launch that used the array
		bool has_user	 = false;
	};
	static std::mutex lock;
	static state per_device[64];
	int dev		 = 0;
	hipError_t e = hipGetDevice(&dev);
	if (e != hipSuccess) {
		return e;
	}
	if (dev < 0 || dev >= 64) {
		return hipErrorInvalidDevice;
	}
	std::lock_guard<std::mutex> g(lock);
	state& st = per_device[dev];
	if (!stream_is_capturing(s)) {
		if (st.has_user && st.user != s && st.user != nullptr) {
			e = stream_drained(st.user); // also covers the first use's tag clearing, which went to that stream
			if (e != hipSuccess) {
				return e;
			}
		}
		st.user		= s;
		st.has_user = true;
	}
	if (!st.ptr) {
		void* p = nullptr;
		e		= hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
		if (e != hipSuccess) {
			return e;
		}
		if (!p) {
			return hipErrorInvalidSymbol;
		}
		constexpr int n = NOALLOC_MAX_SPLIT_UNITS * STRIP_ROWS;
		clear_tags_kernel<<<dim3((n + 255) / 256), dim3(256), 0, s>>>(static_cast<uint64_t*>(p), n); // stream order puts it ahead of the launch that follows
		e = hipGetLastError();
		if (e != hipSuccess) {
			return e;
		}
		st.ptr = static_cast<uint64_t*>(p);
	}
	++st.epoch;
	if (st.epoch == 0) {
		++st.epoch;
	}
	*out		= gemv_scratch{};
	out->tagged = st.ptr;
	out->epoch	= st.epoch;
	return hipSuccess;
}

bool gemv_noalloc_fits(int64_t N, int64_t K) {
	const gemv_plan p = plan_gemv((N + STRIP_ROWS - 1) / STRIP_ROWS, K);
	return p.splits == 1 || static_cast<int64_t>(p.strips) * p.splits <= NOALLOC_MAX_SPLIT_UNITS;
}

// whether a launch with a norm has its first strip's workgroups work the row out for the others (rs: row parts per strip)
static bool gemv_shares_x(const gemv_plan& p, int rs) {
	return static_cast<int64_t>(p.strips) * p.splits * rs >= GEMV_SHARED_X_MIN_WORKGROUPS && static_cast<int64_t>(p.groups) * GROUP_K <= GEMV_SHARED_X_MAX_K;
}

template<int TILES, bool XF32, bool LOOP, bool NORM, int RS = 1> static hipError_t launch_gemv_tiled_n(const gemv_plan& p, const gemv_segments& seg, const void* x, void* dump, int dump_mode, const gemv_scratch& sc, const float* norm_w, float norm_eps, hipStream_t s) {
	const dim3 grid(static_cast<unsigned>(p.strips * p.splits * RS)), block(GEMV_WAVES * 64);
	// a norm in a launch of more than one strip, with a fresh epoch in hand: the first strip's workgroups work the row out for all
	uint64_t* shared_x = NORM && sc.epoch != 0 && gemv_shares_x(p, RS) ? sc.x_words : nullptr;
	if constexpr (RS > 1) { // row split (unsplit K, production only): RS workgroups per strip, nothing handed over
		return launch_kernel(KIND_GEMV, gemv_tiled_kernel<TILES, XF32, DUMP_NONE, LOOP, NORM, RS>, grid, block, 0, s, seg, x, dump, sc.tagged, sc.epoch, p.groups, 0, norm_w, norm_eps, shared_x, sc.error_word,
			sc.spin_limit);
	} else {
		int shift = 0;
		while ((1 << shift) < p.splits) {
			++shift;
		}
		if (dump_mode == DUMP_SUMS) {
			gemv_tiled_kernel<TILES, XF32, DUMP_SUMS, LOOP, NORM><<<grid, block, 0, s>>>(seg, x, dump, sc.tagged, sc.epoch, p.groups, shift, norm_w, norm_eps, nullptr, nullptr, 0);
			return hipGetLastError();
		}
		if (dump_mode == DUMP_X) {
			gemv_tiled_kernel<TILES, XF32, DUMP_X, LOOP, NORM><<<grid, block, 0, s>>>(seg, x, dump, sc.tagged, sc.epoch, p.groups, shift, norm_w, norm_eps, nullptr, nullptr, 0);
			return hipGetLastError();
		}
		return launch_kernel(KIND_GEMV, gemv_tiled_kernel<TILES, XF32, DUMP_NONE, LOOP, NORM>, grid, block, 0, s, seg, x, dump, sc.tagged, sc.epoch, p.groups, shift, norm_w, norm_eps, shared_x, sc.error_word,
			sc.spin_limit);
	}
}

template<int TILES, bool XF32, bool LOOP, int RS = 1> static hipError_t launch_gemv_tiled_t(const gemv_plan& p, const gemv_segments& seg, const void* x, void* dump, int dump_mode, const gemv_scratch& sc, const float* norm_w, float norm_eps, hipStream_t s) {
	if constexpr (XF32) {
		if (norm_w) {
			return launch_gemv_tiled_n<TILES, XF32, LOOP, true, RS>(p, seg, x, dump, dump_mode, sc, norm_w, norm_eps, s);
		}
	}
	return launch_gemv_tiled_n<TILES, XF32, LOOP, false, RS>(p, seg, x, dump, dump_mode, sc, nullptr, 0.0f, s);
}

// unsplit, at most four groups per wave, production: RS row parts per strip
template<int RS, bool XF32> static hipError_t launch_gemv_tiled_rs(int tiles, const gemv_plan& p, const gemv_segments& seg, const void* x, const gemv_scratch& sc, const float* norm_w, float norm_eps, hipStream_t s) {
	switch (tiles) {
		case 1:
			return launch_gemv_tiled_t<1, XF32, false, RS>(p, seg, x, nullptr, DUMP_NONE, sc, norm_w, norm_eps, s);
		case 2:
			return launch_gemv_tiled_t<2, XF32, false, RS>(p, seg, x, nullptr, DUMP_NONE, sc, norm_w, norm_eps, s);
		default:
			return launch_gemv_tiled_t<4, XF32, false, RS>(p, seg, x, nullptr, DUMP_NONE, sc, norm_w, norm_eps, s);
	}
}

static hipError_t launch_gemv_tiled_any(const void* const* W, float* const* y, const int64_t* N, int count, const void* x, bool x_is_f32, int64_t K, void* dump, int dump_mode, hipStream_t s,
	const float* norm_w = nullptr, float norm_eps = 0.0f, const float* const* residual = nullptr, bool noalloc = false) {
	gemv_segments seg{};
	int64_t strips = 0;
	for (int i = 0; i < GEMV_MAX_SEGMENTS; ++i) {
		if (i < count) {
			seg.W[i]	= static_cast<const uint8_t*>(W[i]);
			seg.y[i]	= y ? y[i] : nullptr;
			seg.rows[i] = static_cast<int>(N[i]);
			seg.residual[i] = residual ? residual[i] : nullptr;
			strips += (N[i] + STRIP_ROWS - 1) / STRIP_ROWS;
		}
		seg.strip_end[i] = static_cast<int>(strips);
	}
	if (strips == 0) {
		return hipSuccess;
	}
	gemv_plan p = plan_gemv(strips, K);
	if (p.splits > 1 && stream_is_capturing(s)) { // replay-safe form: every workgroup walks all of K (slower on long-K shapes, no per-launch state)
		p.splits = 1;
		p.tiles	 = (p.groups + GEMV_WAVES - 1) / GEMV_WAVES;
	}
	gemv_scratch sc;
	if (p.splits == 1 && norm_w && x_is_f32 && dump_mode == DUMP_NONE && !noalloc && gemv_shares_x(p, 1) && !stream_is_capturing(s) && in_kernel_waits_enabled()) {
		// the normalised, quantized row goes from the first strip's workgroups to the others through the scratch, tagged with a
		// fresh epoch; not under capture, where a replay could not renew the epoch: there every workgroup works the row out
		const hipError_t e = get_gemv_scratch(&sc, true, s);
		if (e != hipSuccess) {
			return e;
		}
	}
	if (p.splits > 1) {
		if (noalloc && p.strips * p.splits > NOALLOC_MAX_SPLIT_UNITS) {
			return hipErrorInvalidValue; // the caller checks gemv_noalloc_fits first
		}
		const hipError_t e = noalloc ? get_noalloc_scratch(&sc, s) : get_gemv_scratch(&sc, true, s);
		if (e != hipSuccess) {
			return e;
		}
	}
	if (p.tiles > 4) { // K too long to keep every load in flight within the scratch limits: chunked walk
		if (x_is_f32 && norm_w) {
			// chunks of two groups: with the norm's registers on top, chunks of four do not fit the 128 registers of a 1024-thread
			// workgroup and the compiler spills, and a spill's reload queues behind the weight loads like any other load
			return launch_gemv_tiled_t<2, true, true>(p, seg, x, dump, dump_mode, sc, norm_w, norm_eps, s);
		}
		return x_is_f32 ? launch_gemv_tiled_t<4, true, true>(p, seg, x, dump, dump_mode, sc, norm_w, norm_eps, s) : launch_gemv_tiled_t<4, false, true>(p, seg, x, dump, dump_mode, sc, norm_w, norm_eps, s);
	}
	const int tiles = p.tiles <= 1 ? 1 : (p.tiles <= 2 ? 2 : 4);
	if (dump_mode == DUMP_NONE && p.splits == 1) {
		const int rs = plan_gemv_row_parts(p); // fewer strips than CUs: row parts per strip (q8_0_plan.h)
		if (rs == 4) {
			return x_is_f32 ? launch_gemv_tiled_rs<4, true>(tiles, p, seg, x, sc, norm_w, norm_eps, s) : launch_gemv_tiled_rs<4, false>(tiles, p, seg, x, sc, norm_w, norm_eps, s);
		}
		if (rs == 2) {
			return x_is_f32 ? launch_gemv_tiled_rs<2, true>(tiles, p, seg, x, sc, norm_w, norm_eps, s) : launch_gemv_tiled_rs<2, false>(tiles, p, seg, x, sc, norm_w, norm_eps, s);
		}
	}
	if (x_is_f32) {
		switch (tiles) {
			case 1:
				return launch_gemv_tiled_t<1, true, false>(p, seg, x, dump, dump_mode, sc, norm_w, norm_eps, s);
			case 2:
				return launch_gemv_tiled_t<2, true, false>(p, seg, x, dump, dump_mode, sc, norm_w, norm_eps, s);
			default:
				return launch_gemv_tiled_t<4, true, false>(p, seg, x, dump, dump_mode, sc, norm_w, norm_eps, s);
		}
	}
	switch (tiles) {
		case 1:
			return launch_gemv_tiled_t<1, false, false>(p, seg, x, dump, dump_mode, sc, norm_w, norm_eps, s);
		case 2:
			return launch_gemv_tiled_t<2, false, false>(p, seg, x, dump, dump_mode, sc, norm_w, norm_eps, s);
		default:
			return launch_gemv_tiled_t<4, false, false>(p, seg, x, dump, dump_mode, sc, norm_w, norm_eps, s);
	}
}

// y <- 0 for an empty inner dimension (a fill kernel rather than a memset node, so the call can be graph-captured)
__global__ void copy_or_zero_f32_kernel(float* y, const float* src, int64_t n) {
	const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
	if (i < n) {
		y[i] = src ? src[i] : 0.0f;
	}
}

__global__ void zero_f32_kernel(float* __restrict__ y, int64_t n) {
	const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
	if (i < n) {
		y[i] = 0.0f;
	}
}

template<int WAVES> static hipError_t launch_gemv_blocks_t(const uint8_t* W, const uint8_t* xq, float* y, int32_t* sums, int N, int K, hipStream_t s) {
	const int strips   = (N + STRIP_ROWS - 1) / STRIP_ROWS;
	const size_t shmem = static_cast<size_t>(K) + static_cast<size_t>(K / QK) * 4 + WAVES * 64 * 4;
	if (sums) {
		gemv_blocks_kernel<WAVES, true><<<dim3(strips), dim3(WAVES * 64), shmem, s>>>(W, xq, y, sums, N, K);
		return hipGetLastError();
	}
	return launch_kernel(KIND_GEMV, gemv_blocks_kernel<WAVES, false>, dim3(strips), dim3(WAVES * 64), shmem, s, W, xq, y, sums, N, K);
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
		const void* wl[1] = { W };
		float* yl[1]	  = { y };
		return launch_gemv_tiled_any(wl, yl, &N, 1, xq_blocks, false, K, sums, sums ? DUMP_SUMS : DUMP_NONE, s);
	}
	return launch_gemv_blocks_t<4>(w, x, y, sums, static_cast<int>(N), static_cast<int>(K), s);
}

hipError_t launch_gemv_tiled_multi(const void* const* W, float* const* y, const int64_t* N, int count, const void* x, bool x_is_f32, int64_t K, hipStream_t s, const float* norm_w, float norm_eps,
	const float* const* residual) {
	if (K == 0) { // empty dot products: y = residual, or 0
		for (int i = 0; i < count; ++i) {
			if (N[i] > 0) {
				copy_or_zero_f32_kernel<<<dim3(static_cast<unsigned>((N[i] + 255) / 256)), dim3(256), 0, s>>>(y[i], residual ? residual[i] : nullptr, N[i]);
			}
		}
		return hipGetLastError();
	}
	return launch_gemv_tiled_any(W, y, N, count, x, x_is_f32, K, nullptr, DUMP_NONE, s, x_is_f32 ? norm_w : nullptr, norm_eps, residual);
}

hipError_t launch_gemv_tiled_f32_noalloc(const void* W, const float* x, float* y, int64_t N, int64_t K, hipStream_t s) {
	if (K == 0) {
		if (N > 0) {
			zero_f32_kernel<<<dim3(static_cast<unsigned>((N + 255) / 256)), dim3(256), 0, s>>>(y, N); // empty dot product
		}
		return hipGetLastError();
	}
	const void* wl[1] = { W };
	float* yl[1]	  = { y };
	return launch_gemv_tiled_any(wl, yl, &N, 1, x, true, K, nullptr, DUMP_NONE, s, nullptr, 0.0f, nullptr, true);
}

hipError_t launch_gemv_dump_staged_x(const float* x, void* xq_blocks_out, int64_t K, hipStream_t s, const float* norm_w, float norm_eps) {
	const void* wl[1] = { nullptr }; // the dump variant never touches the weights
	const int64_t n	  = STRIP_ROWS;
	return launch_gemv_tiled_any(wl, nullptr, &n, 1, x, true, K, xq_blocks_out, DUMP_X, s, norm_w, norm_eps);
}

} // namespace nh
