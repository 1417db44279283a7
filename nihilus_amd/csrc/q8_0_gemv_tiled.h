// The streaming mat-vec on the tiled layout: pieces shared by the plain decode kernel and the fused FFN kernel.
#pragma once
#include "q8_0_device.h"

namespace nh {

constexpr int GEMV_WAVES = 16;

struct gemv_segments {
	const uint8_t* W[GEMV_MAX_SEGMENTS];
	float* y[GEMV_MAX_SEGMENTS];
	int rows[GEMV_MAX_SEGMENTS];
	int strip_end[GEMV_MAX_SEGMENTS]; // running total of strips
	const float* residual[GEMV_MAX_SEGMENTS]; // per matrix, or null: added to the finished row (one fp32 add after the sum)
};

enum gemv_dump : int { DUMP_NONE = 0, DUMP_SUMS = 1, DUMP_X = 2 };

// One chunk of a wave's K range: groups [gc, gc + cnt), cnt <= TILES, all wave-uniform (scalar registers).
// xs_q / xs_d are this wave's private LDS slices.  Returns the lane's partial dot product over the chunk.
//
// XMODE says where the activation slice comes from:
//   X_BLOCKS    packed Q8_0 blocks (xin), re-aligned into LDS;
//   X_F32       fp32 values (xin), quantized on the spot;
//   X_PUBLISHED quantized blocks that OTHER workgroups of the same launch produce.  xin = PUBLISHED_WORDS 64-bit words
//               per block, each {epoch, payload}: eight dwords of quants and the fp32 scale.  A 64-bit store is seen
//               whole or not at all, so the data carries its own "ready" mark: the producer needs no acknowledgement
//               and no flag, the consumer no second read.  The wave first puts all its weight loads in flight, then
//               reads the 4 * cnt blocks of its slice with device-scope loads until every word carries `epoch`.  The
//               wait is bounded: after `spin_limit` polls the wave gives up, returns NaN and stores a non-zero code
//               in the device-visible error word that `dump` names in this mode (host memory that the next
//               nh_stream_sync / nh_q8_0_last_error reads), so the kernel always drains and the failure reaches the host.
//   X_PUBLISHED_EARLY_WATCH  X_PUBLISHED_EARLY for waves that may wait long for a row that ONE workgroup publishes: after two polls of the
//               whole slice a waiting wave watches a single word of it until that carries the epoch (8 bytes per poll instead of 72 per block)
//   X_PUBLISHED_WATCH  X_PUBLISHED with the same watching (a slice of several producers whose last block is the last to come)
//   X_PUBLISHED_EARLY  the same, with a first read of the words ahead of the weight loads: for slices that are usually there
//               already when the workgroup starts (a launch's input row, published by its first workgroups).
enum gemv_xmode : int { X_BLOCKS = 0, X_F32 = 1, X_PUBLISHED = 2, X_PUBLISHED_EARLY = 3, X_PUBLISHED_EARLY_WATCH = 4, X_PUBLISHED_WATCH = 5 };
constexpr int PUBLISHED_SPIN_LIMIT = 1 << 20;
constexpr int PUBLISHED_FULL_POLLS = 2; // polls of a whole slice before a waiting wave starts watching one word of it
constexpr int PUBLISHED_WORDS	   = 9; // per block: quant dwords 0..7, then the scale
// codes a kernel leaves in the device-visible error word (nh_q8_0_last_error reports them as NH_ERR_DEVICE_TIMEOUT)
enum device_error : unsigned { DEVICE_ERROR_NONE = 0, DEVICE_ERROR_PUBLISH_TIMEOUT = 1 };

// RMS norm * weight in front of the quantizer (X_F32 only).  The row's scale needs every element, so the workgroup works it
// out first, from the row itself (16 KB at K = 4096, served by cache for all but the first workgroups; fixed order of the sum of
// squares: rms_run_* in q8_0_device.h; one workgroup barrier), before its weight loads go out.  Taking the sum from the waves'
// own activation slices instead -- they are loaded anyway, and an unsplit launch cuts K over its 16 waves exactly as the
// fixed order cuts the row -- saves that read but puts the barrier behind the slice loads, with the weight stream already
// queued around them: measured 3-4 % slower ([14336 x 4096] 12.4 against 11.9 us), and it was the more fragile form.
// Loads return in issue order, so what the staging needs (the slice and its norm weights) is requested BEFORE the weight
// stream: a load issued after it would only come back behind it.  The norm weights go from memory straight into LDS (no
// destination registers: the kernel stays at two workgroups per CU).
// One row, one norm: in a launch of many workgroups only those of the first strip do this (`publish` below); as they stage their
// slices they also write them out as tagged words, and every other workgroup takes its slice from there (X_PUBLISHED_EARLY)
// instead of reading the row, the norm weights and working the same blocks out again -- which, norm weights and all, cost the
// one-launch FFN 3 us of its 34.
struct gemv_norm {
	const float* w; // norm weight, fp32 [K]
	float4* xs_w; // this wave's LDS slice for the norm weights of its activation slice (TILES * 32 float4)
	float scale; // the row's 1 / rms
	uint64_t* publish; // non-null: where the staged blocks also go, PUBLISHED_WORDS {epoch, payload} words per block, indexed by block of the row
	unsigned epoch;
};
// red: 16 floats of LDS.  Contains a workgroup barrier: every thread of the workgroup must call it.
__device__ __forceinline__ void gemv_norm_begin(gemv_norm& n, const float* x, const float* w, float4* xs_w, float* red, float eps, int K, int lane, int wave) {
	n.w		  = w;
	n.xs_w	  = xs_w;
	n.publish = nullptr;
	n.epoch	  = 0;
	n.scale	  = rms_scale_workgroup(rms_run_sumsq(x, K / GROUP_K, wave, lane), red, wave, lane, K, eps);
}

//
// CNT, the number of groups, is a template parameter although only the wave knows it at run time (gemv_chunk below
// switches on it): loads complete in issue order and a wait names how many later ones may still be outstanding, so
// the compiler can wait for the activation slice alone, with the weight loads still in flight, only where it can
// count the weight loads.  With a run-time count it has to wait for everything, and the quantizer runs after the last
// weight byte has landed instead of under the stream.
//
// RS > 1 ("row split"): the workgroup owns only 32 / RS rows of its strip (part `rowpart`), and RS workgroups share the
// strip.  A 1 KiB tile is two 512-byte halves (k 0..15 / 16..31) of 32 rows x 16 bytes, so the rows of one part are a
// run of 512 / RS bytes in each half: whole 128-byte lines for RS <= 4.  One 16-byte-per-lane load then covers RS
// blocks instead of one (a group takes 4 / RS loads per lane) and the lane's block and half follow from its number.
// A matrix with fewer strips than the chip has CUs spreads over RS times as many of them this way, with nothing to
// hand over between workgroups.
// MATS == 2: two weight strips (w_strip, w_strip2: the same rows of two matrices that share the activation, gate and up)
// against ONE staged slice: the slice is fetched, quantized and read back from LDS once for both; the second matrix's
// sum comes back through acc2.
template<int TILES, int XMODE, int DUMP, bool NORM, int CNT, int RS = 1, int MATS = 1>
__device__ __forceinline__ float gemv_chunk_n(const uint8_t* __restrict__ w_strip, const void* __restrict__ xin, void* __restrict__ dump, uint8_t* xs_q, float* xs_d, int gc, int groups,
	int lane, int row, int N, bool dump_this_strip, unsigned epoch, gemv_norm* norm, int rowpart = 0, int spin_limit = PUBLISHED_SPIN_LIMIT, const uint8_t* __restrict__ w_strip2 = nullptr,
	float* acc2 = nullptr) {
	static_assert(MATS == 1 || (MATS == 2 && RS == 1 && DUMP == DUMP_NONE), "two matrices: whole strips, production form");
	constexpr int cnt	= CNT;
	constexpr bool XF32 = XMODE == X_F32; // the slice is quantized here, from fp32
	constexpr bool WATCH = XMODE == X_PUBLISHED_EARLY_WATCH || XMODE == X_PUBLISHED_WATCH;
	constexpr bool EARLY = XMODE == X_PUBLISHED_EARLY || XMODE == X_PUBLISHED_EARLY_WATCH; // ... with a first look before the weight loads go out
	constexpr bool XPUB = XMODE == X_PUBLISHED || XMODE == X_PUBLISHED_WATCH || EARLY; // the slice is read as tagged words
	static_assert(RS == 1 || RS == 2 || RS == 4, "a strip splits into 1, 2 or 4 row parts");
	static_assert(RS == 1 || DUMP == DUMP_NONE, "the inspection variants run on whole strips");
	constexpr int PART_ROWS = STRIP_ROWS / RS; // rows this workgroup owns
	constexpr int W_LOADS	= GROUP_BLOCKS / RS; // 16-byte loads per lane and group
	const int r	   = RS == 1 ? (lane & 31) : rowpart * PART_ROWS + (lane & (PART_ROWS - 1)); // row within the strip
	const int half = RS == 1 ? (lane >> 5) : ((lane / PART_ROWS) & 1); // which 16 quants of its block the lane holds
	const int blk0 = RS == 1 ? 0 : (lane / PART_ROWS) >> 1; // block of the lane's first load within the group; load j: blk0 + j * RS

	// ---- 1. activation slice loads, issued first ----
	constexpr int XQ_LOADS = (TILES * 34 + 63) / 64; // raw dwords of blocks [4*gc, 4*(gc+cnt)): 34 dwords per group
	constexpr int XF_LOADS = (TILES * 32 + 63) / 64; // float4 per lane: 128 floats per group = 32 float4
	uint32_t xr[XQ_LOADS];
	float4 xf[XF_LOADS];
	if constexpr (XMODE == X_F32) {
		if constexpr (NORM) {
			// memory -> LDS, no destination registers; issued before the slice loads, which the quantizer waits for:
			// loads complete in issue order, so once the slice is there these are too
			const float4* w4 = reinterpret_cast<const float4*>(norm->w + static_cast<int64_t>(gc) * GROUP_K);
#pragma unroll
			for (int i = 0; i < XF_LOADS; ++i) {
				const int v = lane + 64 * i;
				if (v < cnt * 32) { // 16 bytes per lane, lane l of the wave lands at xs_w[64 * i + l]
					load_global_to_lds_b128(w4 + v, norm->xs_w + 64 * i);
				}
			}
			asm volatile("" ::: "memory"); // the slice loads below are issued after these
		}
		const float4* x4 = reinterpret_cast<const float4*>(static_cast<const float*>(xin) + static_cast<int64_t>(gc) * GROUP_K);
#pragma unroll
		for (int i = 0; i < XF_LOADS; ++i) {
			const int v = lane + 64 * i; // float4 index in the slice; block = v / 8
			xf[i]		= v < cnt * 32 ? x4[v] : make_float4(0.f, 0.f, 0.f, 0.f);
		}
	} else if constexpr (XMODE == X_BLOCKS) {
		const uint32_t* x_raw = reinterpret_cast<const uint32_t*>(static_cast<const uint8_t*>(xin) + static_cast<int64_t>(gc) * (GROUP_BLOCKS * BLOCK_BYTES));
#pragma unroll
		for (int i = 0; i < XQ_LOADS; ++i) {
			const int v = lane + 64 * i;
			xr[i]		= v < cnt * 34 ? x_raw[v] : 0u;
		}
	}

	// device-scope loads: the producers ran on other XCDs, whose L2 this one does not snoop
	constexpr int PW_LOADS = XPUB ? (TILES * GROUP_BLOCKS * PUBLISHED_WORDS + 63) / 64 : 1;
	const uint64_t* pw	   = XPUB ? static_cast<const uint64_t*>(xin) + static_cast<int64_t>(gc) * (GROUP_BLOCKS * PUBLISHED_WORDS) : nullptr;
	const int n_words	   = cnt * GROUP_BLOCKS * PUBLISHED_WORDS;
	uint64_t pv[PW_LOADS];
	if constexpr (EARLY) {
		// a first look ahead of the weight loads: a workgroup that starts after the publishers are through finds every word
		// there and has its slice staged while its weights are still arriving
#pragma unroll
		for (int i = 0; i < PW_LOADS; ++i) {
			const int v = lane + 64 * i;
			pv[i]		= v < n_words ? __hip_atomic_load(pw + v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : (static_cast<uint64_t>(epoch) << 32);
		}
	}

	// ---- 2. every weight byte of the chunk, in flight at once ----
	v4i q[TILES][W_LOADS];
	v2u dd[TILES];
	if constexpr (DUMP != DUMP_X) {
		const uint8_t* macro0 = w_strip + static_cast<int64_t>(gc) * MACRO_BYTES;
		// byte offset of the lane's 16 quants inside its first tile: RS == 1 is the tile as stored (16 * lane)
		const int lane_off = RS == 1 ? 16 * lane : blk0 * TILE_BYTES + half * (TILE_BYTES / 2) + 16 * r;
#pragma unroll
		for (int t = 0; t < TILES; ++t) {
			if (t < cnt) {
				const uint8_t* macro = macro0 + t * MACRO_BYTES;
#pragma unroll
				for (int j = 0; j < W_LOADS; ++j) {
					q[t][j] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(macro + j * (RS * TILE_BYTES) + lane_off));
				}
				dd[t] = __builtin_nontemporal_load(reinterpret_cast<const v2u*>(macro + MACRO_D_OFFSET + 8 * r));
			}
		}
	}
	v4i q2[MATS == 2 ? TILES : 1][W_LOADS];
	v2u dd2[MATS == 2 ? TILES : 1];
	if constexpr (MATS == 2) {
		const uint8_t* macro0 = w_strip2 + static_cast<int64_t>(gc) * MACRO_BYTES;
#pragma unroll
		for (int t = 0; t < TILES; ++t) {
			if (t < cnt) {
				const uint8_t* macro = macro0 + t * MACRO_BYTES;
#pragma unroll
				for (int j = 0; j < W_LOADS; ++j) {
					q2[t][j] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(macro + j * TILE_BYTES + 16 * lane));
				}
				dd2[t] = __builtin_nontemporal_load(reinterpret_cast<const v2u*>(macro + MACRO_D_OFFSET + 8 * r));
			}
		}
	}

	// ---- 2b. the slice comes from this launch's own producers: read it until every word is this launch's ----
	bool timed_out = false;
	if constexpr (XPUB) {
		int spins	= 0;
		bool looked = EARLY; // the first set of words is already on its way
		bool watched = !WATCH; // the slice's last word has been seen to be this launch's
		for (;;) {
			if (!looked) {
#pragma unroll
				for (int i = 0; i < PW_LOADS; ++i) {
					const int v = lane + 64 * i;
					pv[i]		= v < n_words ? __hip_atomic_load(pw + v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : (static_cast<uint64_t>(epoch) << 32);
				}
			}
			looked	   = false;
			bool fresh = true;
#pragma unroll
			for (int i = 0; i < PW_LOADS; ++i) {
				fresh = fresh && static_cast<unsigned>(pv[i] >> 32) == epoch;
			}
			if (__builtin_amdgcn_ballot_w64(!fresh) == 0) {
				break;
			}
			// Not there yet: watch ONE word of the slice (its last; the same address in every lane, one request per poll) until it is
			// this launch's, then read the whole slice again.  A wave that waits long -- a workgroup that became resident well before
			// its producers are done -- polls 8 bytes at a time instead of the slice's 72 per block.  Once that word has come the
			// rest is polled as a whole (a slice with several producers: watching one word first would put a second round trip
			// into every further poll).
			if (++spins >= spin_limit) {
				timed_out = true;
			}
			__builtin_amdgcn_s_sleep(8);
			while (!watched && !timed_out && spins > PUBLISHED_FULL_POLLS) {
				const uint64_t last = __hip_atomic_load(pw + (n_words - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
				if (static_cast<unsigned>(last >> 32) == epoch) {
					watched = true;
				} else if (++spins >= spin_limit) {
					timed_out = true;
				} else {
					__builtin_amdgcn_s_sleep(8);
				}
			}
			if (timed_out) {
				// tell the host (an ordinary vector store to pinned host memory).  Done here, not where the NaN is set: kept for
				// the end of the function the pointer and the branch cost the hot path 25 registers
				if (lane == 0 && dump) {
					__hip_atomic_store(static_cast<unsigned*>(dump), static_cast<unsigned>(DEVICE_ERROR_PUBLISH_TIMEOUT), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
				}
				break;
			}
		}
#pragma unroll
		for (int i = 0; i < PW_LOADS; ++i) {
			const int v = lane + 64 * i;
			if (v < n_words) {
				const int blk = v / PUBLISHED_WORDS, j = v - blk * PUBLISHED_WORDS;
				const uint32_t payload = static_cast<uint32_t>(pv[i]);
				if (j < 8) {
					*reinterpret_cast<uint32_t*>(xs_q + blk * QK + 4 * j) = payload;
				} else {
					xs_d[blk] = __uint_as_float(payload);
				}
			}
		}
	}

	// ---- 3. stage the activation slice in LDS: quants 16-byte aligned per half block, scales as fp32 ----
	if constexpr (XF32) {
		if constexpr (NORM) {
			// a use of the last slice register that a load fills (the ones past the slice hold constants): the compiler has
			// to wait for the slice here, which (issue order) covers the memory -> LDS loads; the LDS reads below may not
			// move above this point
			constexpr int LAST_LOADED = cnt > 0 ? (cnt * 32 - 1) / 64 : 0;
			asm volatile("" ::"v"(xf[LAST_LOADED].w) : "memory");
#pragma unroll
			for (int i = 0; i < XF_LOADS; ++i) {
				const int v = lane + 64 * i;
				if (v < cnt * 32) {
					xf[i] = norm_mul4(xf[i], norm->scale, norm->xs_w[v]);
				}
			}
		}
#pragma unroll
		for (int i = 0; i < XF_LOADS; ++i) {
			const int v = lane + 64 * i;
			uint16_t dh;
			const uint32_t packed = quantize_block_lane(xf[i], &dh); // all lanes take part; lanes past the slice hold zeros
			if (v < cnt * 32) {
				*reinterpret_cast<uint32_t*>(xs_q + 4 * v) = packed; // block v/8 at 32*(v/8), dword v%8
				if ((v & 7) == 0) {
					xs_d[v >> 3] = half_bits_to_float(dh); // the fp16-rounded scale, exactly what a stored block would hold
				}
			}
		}
	} else if constexpr (XMODE == X_BLOCKS) {
		// half-word hw of the raw stream is a scale (hw % 17 == 0) or a quant pair
#pragma unroll
		for (int i = 0; i < XQ_LOADS; ++i) {
			const int v = lane + 64 * i;
			if (v < cnt * 34) {
#pragma unroll
				for (int h = 0; h < 2; ++h) {
					const int hw	   = 2 * v + h;
					const int jj	   = hw / 17;
					const int o		   = hw - 17 * jj;
					const uint16_t val = static_cast<uint16_t>(h ? (xr[i] >> 16) : (xr[i] & 0xFFFFu));
					if (o == 0) {
						xs_d[jj] = half_bits_to_float(val);
					} else {
						*reinterpret_cast<uint16_t*>(xs_q + jj * QK + 2 * (o - 1)) = val;
					}
				}
			}
		}
	}
	__builtin_amdgcn_wave_barrier(); // wave-local hand-off: the same wave wrote and reads; the LDS counter wait orders it

	if constexpr (XF32 && NORM) {
		if (norm->publish) {
			// the slice as staged, for the workgroups that do not work it out themselves: self-tagged 64-bit words, device-scope
			// stores, nothing waited for (a reader takes a word only with this launch's epoch in it)
			uint64_t* out			= norm->publish + static_cast<int64_t>(gc) * (GROUP_BLOCKS * PUBLISHED_WORDS);
			constexpr int OUT_WORDS = cnt * GROUP_BLOCKS * PUBLISHED_WORDS;
#pragma unroll
			for (int i = 0; i < (OUT_WORDS + 63) / 64; ++i) {
				const int v = lane + 64 * i;
				if (v < OUT_WORDS) {
					const int blk		   = v / PUBLISHED_WORDS, j = v - blk * PUBLISHED_WORDS;
					const uint32_t payload = j < 8 ? *reinterpret_cast<const uint32_t*>(xs_q + blk * QK + 4 * j) : __float_as_uint(xs_d[blk]);
					__hip_atomic_store(out + v, (static_cast<uint64_t>(norm->epoch) << 32) | payload, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
				}
			}
		}
	}

	if constexpr (DUMP == DUMP_X) {
		// parity hook: what was staged, written back as packed blocks (the first strip of the launch covers all of K)
		if (dump_this_strip) {
			uint8_t* out = static_cast<uint8_t*>(dump) + static_cast<int64_t>(gc) * (GROUP_BLOCKS * BLOCK_BYTES);
			for (int jj = lane; jj < cnt * GROUP_BLOCKS; jj += 64) {
				uint8_t* o						= out + jj * BLOCK_BYTES;
				*reinterpret_cast<uint16_t*>(o) = float_to_half_bits(xs_d[jj]); // exact: the value came from fp16
				for (int i = 0; i < 16; ++i) {
					*reinterpret_cast<uint16_t*>(o + 2 + 2 * i) = *reinterpret_cast<const uint16_t*>(xs_q + jj * QK + 2 * i);
				}
			}
		}
		return 0.0f;
	}

	// ---- 4. dot products as the tiles land ----
	float acc = 0.0f;
	[[maybe_unused]] float second = 0.0f;
#pragma unroll
	for (int t = 0; t < TILES; ++t) {
		if (t < cnt) {
			if constexpr (RS == 1) {
				const float dw[GROUP_BLOCKS] = { half_bits_to_float(static_cast<uint16_t>(dd[t].x & 0xFFFFu)), half_bits_to_float(static_cast<uint16_t>(dd[t].x >> 16)),
					half_bits_to_float(static_cast<uint16_t>(dd[t].y & 0xFFFFu)), half_bits_to_float(static_cast<uint16_t>(dd[t].y >> 16)) };
#pragma unroll
				for (int j = 0; j < GROUP_BLOCKS; ++j) {
					const int jj = t * GROUP_BLOCKS + j;
					const v4i xv = *reinterpret_cast<const v4i*>(xs_q + jj * QK + 16 * half);
					const int s	 = dot16(q[t][j], xv);
					if constexpr (DUMP == DUMP_SUMS) {
						const int full = s + __shfl_xor(s, 32);
						if (half == 0 && row < N) {
							static_cast<int32_t*>(dump)[static_cast<int64_t>(row) * (groups * GROUP_BLOCKS) + (gc * GROUP_BLOCKS + jj)] = full;
						}
					} else {
						acc = fmaf(static_cast<float>(s), dw[j] * xs_d[jj], acc);
					}
					if constexpr (MATS == 2) {
						const uint32_t dp2 = (j & 2) ? dd2[t].y : dd2[t].x;
						const float dw2	   = half_bits_to_float(static_cast<uint16_t>((j & 1) ? (dp2 >> 16) : (dp2 & 0xFFFFu)));
						second			   = fmaf(static_cast<float>(dot16(q2[t][j], xv)), dw2 * xs_d[jj], second);
					}
				}
			} else {
#pragma unroll
				for (int j = 0; j < W_LOADS; ++j) {
					const int b		  = blk0 + j * RS; // the lane's block within the group
					const int jj	  = t * GROUP_BLOCKS + b;
					const uint32_t dp = (b & 2) ? dd[t].y : dd[t].x;
					const float dw	  = half_bits_to_float(static_cast<uint16_t>((b & 1) ? (dp >> 16) : (dp & 0xFFFFu)));
					const v4i xv	  = *reinterpret_cast<const v4i*>(xs_q + jj * QK + 16 * half);
					const int s		  = dot16(q[t][j], xv);
					acc				  = fmaf(static_cast<float>(s), dw * xs_d[jj], acc);
				}
			}
		}
	}
	if constexpr (XPUB) {
		if (timed_out) {
			acc	   = __uint_as_float(0x7FC00000u); // a producer never published: make the failure visible in the output as well
			second = acc;
		}
	}
	if constexpr (MATS == 2) {
		*acc2 = second;
	}
	return acc;
}

template<int TILES, int XMODE, int DUMP, bool NORM = false, int RS = 1, int MATS = 1>
__device__ __forceinline__ float gemv_chunk(const uint8_t* __restrict__ w_strip, const void* __restrict__ xin, void* __restrict__ dump, uint8_t* xs_q, float* xs_d, int gc, int cnt,
	int groups, int lane, int row, int N, bool dump_this_strip, unsigned epoch = 0, gemv_norm* norm = nullptr, int rowpart = 0, int spin_limit = PUBLISHED_SPIN_LIMIT,
	const uint8_t* __restrict__ w_strip2 = nullptr, float* acc2 = nullptr) {
#define NH_CHUNK_CASE(C)                                                                                                                                              \
	case C:                                                                                                                                                           \
		if constexpr (C <= TILES) {                                                                                                                                   \
			return gemv_chunk_n<TILES, XMODE, DUMP, NORM, (C <= TILES ? C : 0), RS, MATS>(w_strip, xin, dump, xs_q, xs_d, gc, groups, lane, row, N, dump_this_strip, epoch, norm, rowpart,   \
				spin_limit, w_strip2, acc2);                                                                                                                          \
		}                                                                                                                                                             \
		break;
	switch (cnt) { // wave-uniform
		NH_CHUNK_CASE(1)
		NH_CHUNK_CASE(2)
		NH_CHUNK_CASE(3)
		NH_CHUNK_CASE(4)
		NH_CHUNK_CASE(5)
		NH_CHUNK_CASE(6)
		NH_CHUNK_CASE(7)
		NH_CHUNK_CASE(8)
		default:
			break;
	}
#undef NH_CHUNK_CASE
	// an idle wave (still takes part in barriers)
	return gemv_chunk_n<TILES, XMODE, DUMP, NORM, 0, RS, MATS>(w_strip, xin, dump, xs_q, xs_d, gc, groups, lane, row, N, dump_this_strip, epoch, norm, rowpart, spin_limit, w_strip2, acc2);
}

// K split over several workgroups: each publishes the 32 partial sums of its share, tagged with the launch's epoch
// (one 64-bit device-scope store per row: tag and value can never be seen apart), waits for the acknowledgement, then
// reads every share of its strip.  A row whose shares all carry the epoch is summed in split order and stored; the
// workgroup whose store was performed last is certain to see them all, an earlier one may too and then writes the
// same bits.  Two memory round trips, no counter, no barrier, nothing to reset (epochs only move forward), and the
// result does not depend on arrival order.
// Each XCD has its own L2, so data that crosses workgroups goes through device-scope stores and loads (written through
// to / read from the memory side).  A device-wide fence would also order them, but it writes back and invalidates the
// whole L2 under the other workgroups' streaming loads.
// Call from the first 32 threads of the workgroup (one wave), total = the row's partial sum over this split.
__device__ __forceinline__ void split_k_finish(uint64_t* __restrict__ tagged, unsigned epoch, int gstrip, int splits, int split, int lane, float total, float* __restrict__ y, int row,
	int N, const float* __restrict__ residual) {
	uint64_t* mine = tagged + static_cast<int64_t>(gstrip) * splits * STRIP_ROWS + lane;
	// The residual may be y itself, and more than one workgroup may store the row: each takes its copy of the residual before
	// it publishes its own share.  Nobody can have stored the row by then (that takes every share, this one included), so all
	// of them add the same value, whoever stores first.
	float res = 0.0f;
	if (residual && row < N) {
		res = residual[row];
	}
	asm volatile("" : "+v"(res)::"memory"); // the value is in a register (the load has returned) before the share goes out
	__hip_atomic_store(&mine[split * STRIP_ROWS], (static_cast<uint64_t>(epoch) << 32) | __float_as_uint(total), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
	wait_stores_acknowledged();
	bool all  = true;
	float sum = 0.0f;
	for (int sp0 = 0; sp0 < splits; sp0 += 8) { // every share requested before the first is waited for
		uint64_t v[8];
#pragma unroll
		for (int u = 0; u < 8; ++u) {
			v[u] = (sp0 + u < splits) ? __hip_atomic_load(&mine[(sp0 + u) * STRIP_ROWS], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0ull;
		}
#pragma unroll
		for (int u = 0; u < 8; ++u) {
			if (sp0 + u < splits) {
				all = all && static_cast<unsigned>(v[u] >> 32) == epoch;
				sum += __uint_as_float(static_cast<uint32_t>(v[u]));
			}
		}
	}
	if (all && row < N) {
		y[row] = residual ? sum + res : sum;
	}
}

// Scratch of the K-split path (tagged partial sums) and of the fused FFN launch (the gate and up
// projections' outputs and one "published" word per producer strip): one allocation per device, made on first use and
// kept for the life of the process.  Calls that overlap on one GPU (different streams) and both use it race on it.
constexpr int GEMV_MAX_SPLIT_UNITS	= 8192; // strips * splits when splits > 1
constexpr int GEMV_MAX_SPLIT_STRIPS = 512;
constexpr int FFN_MAX_HIDDEN		= 65536; // rows of the gate / up projections in a fused FFN launch
constexpr int CHAIN_MAX_EMBD			= 8192; // longest hidden state the chained decode layer takes (a wave of its norm workgroups holds its share of the row in registers)
constexpr int GEMV_SHARED_X_MAX_K	= 65536; // longest input row that a launch with a norm shares between its workgroups (longer: each works it out)
// Sharing makes every other workgroup wait for the first strip's: a chain of row read, norm, quantize, publish and read-back
// of ~3 us that the first round of workgroups sits out.  It pays once a launch runs several rounds, each of which would
// otherwise spend its first 1.5 us on the norm instead of on its loads: measured, lm_head [128256 x 4096] 88.6 -> 84.9 us,
// gate+up [2 x 28672 x 8192] 84.1 -> 81.0 us, the one-launch FFN at those shapes 155 -> 133 us; but q+k+v [6144 x 4096]
// 8.0 -> 9.6 us and nothing gained on gate+up [2 x 14336 x 4096] or its FFN (34.2 -> 34.0 us).
constexpr int GEMV_SHARED_X_MIN_WORKGROUPS = 1024; // mat-vec launches
constexpr int FFN_SHARED_X_MIN_PRODUCERS   = 768; // producer workgroups of a one-launch FFN
struct gemv_scratch {
	uint64_t* tagged   = nullptr; // [GEMV_MAX_SPLIT_UNITS][32] {epoch, partial sum}
	float* gate_up	   = nullptr; // [2][FFN_MAX_HIDDEN]: the gate and up outputs (kept for inspection only)
	uint64_t* act_words = nullptr; // [FFN_MAX_HIDDEN / 32][PUBLISHED_WORDS] {epoch, payload}: the quantized activation of the down projection
	uint8_t* act_blocks = nullptr; // [FFN_MAX_HIDDEN / 32] packed 34-byte blocks: the activation of the three-launch form used under graph capture
	uint64_t* x_words	= nullptr; // [GEMV_SHARED_X_MAX_K / 32][PUBLISHED_WORDS] {epoch, payload}: a launch's normalised, quantized input row, from its first strip's workgroups to the rest
	// the chained decode layer (q8_0_decode_layer.hip): the fp32 rows that one stage hands to the next as {epoch, value} words, and
	// the second normalised, quantized row of the launch
	uint64_t* row_tagged[2] = { nullptr, nullptr }; // [CHAIN_MAX_EMBD] each: attn_out + residual, then down + residual
	uint64_t* x_words_next	= nullptr; // [CHAIN_MAX_EMBD / 32][PUBLISHED_WORDS]
	unsigned epoch	   = 0; // with next_epoch = true: a value no earlier launch on this device has used
	unsigned* error_word = nullptr; // 4 bytes of pinned host memory the device can write: non-zero once a kernel has given up a bounded wait
	int spin_limit	   = PUBLISHED_SPIN_LIMIT; // polls before a consumer of published blocks gives up (lowered only by tests)
};
// next_epoch = true is what a launch that hands data between workgroups through the scratch asks for; `s` is the stream it is
// about to launch on.  The scratch serves one stream at a time: if the previous such launch went to a different stream and that
// stream has not drained, hipErrorNotReady comes back (NH_ERR_BUSY at the C ABI) instead of a launch that would corrupt both.
// The check is skipped for capturing streams and when the previous user was the null stream (which may not be queried while
// another stream captures).
hipError_t get_gemv_scratch(gemv_scratch* out, bool next_epoch = false, hipStream_t s = nullptr);
// Reads the current device's error word (DEVICE_ERROR_NONE if no scratch exists yet); clear = true also resets it.
unsigned read_device_error(bool clear);
void set_published_spin_limit(int limit);
// Whether launches may contain workgroups that wait for other workgroups of the same launch (the one-launch FFN, the chained block,
// the norm row shared between the workgroups of a large mat-vec).  On by default; off, those calls take the forms a capturing
// stream gets: several launches, or every workgroup working the row out itself.  Process-wide.
bool in_kernel_waits_enabled();
bool set_in_kernel_waits(bool enabled); // returns the previous setting

// How a tiled mat-vec launch is cut: `splits` workgroups per strip, each of 16 waves owning <= `tiles` groups.
struct gemv_plan {
	int strips, groups, splits, tiles;
};
inline gemv_plan plan_gemv(int64_t total_strips, int64_t K) {
	gemv_plan p;
	p.strips	   = static_cast<int>(total_strips);
	p.groups	   = static_cast<int>(K / GROUP_K);
	p.splits	   = 1;
	auto tiles_for = [&](int s) { return (p.groups + GEMV_WAVES * s - 1) / (GEMV_WAVES * s); };
	// K goes over several workgroups only when it has to: the hand-off between workgroups costs 1-2 us, more than an
	// idle half of the chip costs a matrix of a few MB.  So: split until a wave owns at most 4 groups (every load of the
	// wave in flight at once), and, once splitting anyway, one step further to 2 groups per wave (measured best on the
	// long-K down projections).
	const bool room = p.strips <= GEMV_MAX_SPLIT_STRIPS;
	while (tiles_for(p.splits) > 4 && room && p.strips * p.splits * 2 <= GEMV_MAX_SPLIT_UNITS) {
		p.splits *= 2;
	}
	if (p.splits > 1 && tiles_for(p.splits) > 2 && p.strips * p.splits * 2 <= GEMV_MAX_SPLIT_UNITS) {
		p.splits *= 2;
	}
	// few strips (k/v-sized outputs with a long K): keep cutting while the launch would leave CUs without a workgroup and a
	// workgroup still gets a dozen groups ([1024 x 14336]: 6.7 us with 4 workgroups per strip, 5.4 us with 8)
	while (p.splits > 1 && p.strips * p.splits < 256 && p.groups >= 24 * p.splits && p.strips * p.splits * 2 <= GEMV_MAX_SPLIT_UNITS) {
		p.splits *= 2;
	}
	p.tiles = tiles_for(p.splits);
	return p;
}


} // namespace nh
