// One transformer block's decode-time mat-vecs behind the attention, and the next block's in front of it, as ONE launch, gfx950:
//
//   ffn_inp = W_o . Q(attn) + layer_in                                        attn_out mul_mat -> residual add   (mega_attention_apply)
//   l_out   = W_down . Q(silu(W_gate . Q(n1)) * (W_up . Q(n1))) + ffn_inp,    n1 = rms_norm(ffn_inp) * ffn_norm   (mega_ffn)
//   y_i     = W_next[i] . Q(n2),  i < count,                                   n2 = rms_norm(l_out) * next_norm    (the next block's q / k / v
//                                                                              of mega_qkv_prep_and_cache_publish, or the logits of final_norm_and_sampling)
//
// In the reference these are three cores of the per-block fold (cuda/thread_pool.hpp:46-67; graphs at infra/core_traits.hpp:768-772,
// :971-995, :570-594, :1186-1193), each a synchronous launch.  The attention itself sits between q / k / v and attn_out, so a launch can
// run from one attention to the next: per token one launch per block instead of three.
//
// Why one launch: every launch pays ~3 us beyond its bytes (first bytes ~2 us after the launch starts, a tail on a mostly idle chip).
// Here the five stages are ranges of one grid, in data-flow order -- attn_out strips, one norm workgroup, gate/up strips, down strips,
// one norm workgroup, the next projections' strips -- and a workgroup of a later stage puts its weight loads in flight the moment it
// is resident, then waits for its activation, so HBM stays busy across the seams.
//
// Hand-offs (all through self-tagged 64-bit words {epoch, 32 bits of payload}, device-scope stores and loads: a 64-bit store is seen
// whole or not at all, so the data is its own "ready" mark, nobody waits for an acknowledgement, nothing is reset between launches):
//   * attn_out and down workgroups publish their finished rows (the residual already added) as fp32 words;
//   * a norm workgroup reads that whole row (each of its sixteen waves the run of the fixed-order sum of squares that it also
//     quantizes), works out the scale, multiplies by the norm weight, quantizes, and publishes the row as Q8_0 blocks (nine words per
//     block): the arithmetic of rms_norm_quantize_kernel, bit for bit;
//   * every gate/up / next-projection workgroup stages its slices from those blocks; the down workgroups take theirs from the blocks
//     that the gate/up workgroups publish (as in the one-launch FFN), and their residual from the published attn_out row.
// Progress: every workgroup waits only for workgroups with lower indices, and workgroups are dispatched in index order within each
// XCD's share of the grid, so the lowest unfinished workgroup can always run; every wait is bounded all the same (the wave gives
// up, leaves NaN and a code in the device-visible error word).
#include "q8_0_gemv_tiled.h"

namespace nh {

constexpr int CHAIN_TILES = 4; // groups a wave stages at once: LDS slices are sized for it
constexpr int CHAIN_DOWN_ROWS_TILES = 8; // ... in the down stage when it is cut by rows (half-size groups)
constexpr int CHAIN_NORM_F4 = CHAIN_MAX_EMBD / GROUP_K / GEMV_WAVES * 32 / 64; // float4 per lane of a norm workgroup's wave: 2

struct layer_args {
	// attn_out
	const uint8_t* w_o;
	const float* attn; // [n_embd]
	const float* layer_in; // [n_embd]: the residual
	float* ffn_inp; // [n_embd]
	// ffn
	const float* ffn_norm_w;
	const uint8_t* w_gate;
	const uint8_t* w_up;
	const uint8_t* w_down;
	float* l_out; // [n_embd]
	// the projections behind the next norm
	const float* next_norm_w;
	gemv_segments next; // weights, outputs, rows, running strip totals
	float eps;
	int n_embd, n_ff;
	int groups_e, groups_f; // n_embd / 128, n_ff / 128
	// grid: [0, first_norm) attn_out, first_norm, [first_producer, first_consumer) gate/up, [first_consumer, second_norm) down,
	// second_norm, [first_next, grid) next projections (second_norm == grid: no such stage)
	int first_norm, first_producer, first_consumer, second_norm, first_next;
	int p_per_slot, p_rem; // a producer strip's K range over its waves
	int split_shift; // a down strip's K range goes over (1 << split_shift) workgroups
	int down_by_rows; // instead: two workgroups per down strip, each 16 rows and all of K (nothing to hand over)
	// scratch
	uint64_t* attn_row; // [n_embd] {epoch, fp32}: ffn_inp as published
	uint64_t* x_words; // [n_embd / 32][9]: Q(n1)
	float* gate_up; // inspection copies of the gate / up outputs
	uint64_t* act_words; // [n_ff / 32][9]: the down projection's activation
	uint64_t* tagged; // K-split partial sums of the down projection
	uint64_t* down_row; // [n_embd] {epoch, fp32}: l_out as published
	uint64_t* x_words_next; // [n_embd / 32][9]: Q(n2)
	unsigned epoch;
	unsigned* error_word;
	int spin_limit;
};

// Bounded wait of one wave for `count` (<= 4 per lane and step) tagged words: true once every word carries the epoch.
__device__ __forceinline__ bool give_up(int& spins, int limit, unsigned* error_word, int lane) {
	if (++spins >= limit) {
		if (lane == 0 && error_word) {
			__hip_atomic_store(error_word, static_cast<unsigned>(DEVICE_ERROR_PUBLISH_TIMEOUT), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
		}
		return true;
	}
	__builtin_amdgcn_s_sleep(8);
	return false;
}

// The norm workgroup: the fp32 row `row` (tagged words, written by the workgroups of the stage before) -> (row * scale) * norm_w
// -> quantize_row_q8_0 -> published blocks.  Sixteen waves; wave w takes run w of the fixed-order sum of squares (q8_0_device.h),
// lane l the float4s l, l + 64, ... of that run -- for the sum and for the quantizer alike, so the row is read once, into registers.
// The same sequence of fp32 operations as rms_norm_quantize_kernel and the mat-vec kernels' own norm, hence the same bytes.
__device__ __forceinline__ void norm_workgroup(const uint64_t* __restrict__ row, const float* __restrict__ norm_w, uint64_t* __restrict__ out, int groups, float eps, unsigned epoch,
	unsigned* error_word, int spin_limit, float* red, int lane, int wave) {
	const int q = groups / GEMV_WAVES, r = groups % GEMV_WAVES;
	const int g0 = wave * q + min(wave, r);
	const int n4 = (q + (wave < r ? 1 : 0)) * 32; // float4s in this wave's run
	const float4* w4 = reinterpret_cast<const float4*>(norm_w) + g0 * 32;
	float4 wv[CHAIN_NORM_F4], xf[CHAIN_NORM_F4];
#pragma unroll
	for (int i = 0; i < CHAIN_NORM_F4; ++i) {
		const int v = lane + 64 * i;
		wv[i]		= v < n4 ? w4[v] : make_float4(0.f, 0.f, 0.f, 0.f);
	}
	const uint64_t* mine = row + static_cast<int64_t>(g0) * GROUP_K;
	int spins			 = 0;
	for (;;) {
		bool fresh = true;
#pragma unroll
		for (int i = 0; i < CHAIN_NORM_F4; ++i) {
			const int v = lane + 64 * i;
			uint64_t t[4];
#pragma unroll
			for (int c = 0; c < 4; ++c) {
				t[c] = v < n4 ? __hip_atomic_load(mine + 4 * v + c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : (static_cast<uint64_t>(epoch) << 32);
			}
#pragma unroll
			for (int c = 0; c < 4; ++c) {
				fresh = fresh && static_cast<unsigned>(t[c] >> 32) == epoch;
			}
			xf[i] = make_float4(__uint_as_float(static_cast<uint32_t>(t[0])), __uint_as_float(static_cast<uint32_t>(t[1])), __uint_as_float(static_cast<uint32_t>(t[2])),
				__uint_as_float(static_cast<uint32_t>(t[3])));
		}
		if (__builtin_amdgcn_ballot_w64(!fresh) == 0) {
			break;
		}
		if (give_up(spins, spin_limit, error_word, lane)) {
			// the stage before never delivered: what is published below is NaN, and everything downstream inherits it
#pragma unroll
			for (int i = 0; i < CHAIN_NORM_F4; ++i) {
				const float nan = __uint_as_float(0x7FC00000u);
				xf[i]			= make_float4(nan, nan, nan, nan);
			}
			break;
		}
	}
	float p = 0.0f;
#pragma unroll
	for (int i = 0; i < CHAIN_NORM_F4; ++i) {
		if (lane + 64 * i < n4) {
			p = sumsq_fold(p, xf[i]);
		}
	}
	const float scale = rms_scale_workgroup(p, red, wave, lane, groups * GROUP_K, eps); // a workgroup barrier inside
#pragma unroll
	for (int i = 0; i < CHAIN_NORM_F4; ++i) {
		const int v = lane + 64 * i;
		uint16_t dh;
		const uint32_t packed = quantize_block_lane(norm_mul4(xf[i], scale, wv[i]), &dh); // every lane takes part; lanes past the run hold zeros
		if (v < n4) {
			uint64_t* blk = out + (static_cast<int64_t>(g0) * GROUP_BLOCKS + (v >> 3)) * PUBLISHED_WORDS;
			__hip_atomic_store(blk + (v & 7), (static_cast<uint64_t>(epoch) << 32) | packed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
			if ((v & 7) == 0) {
				__hip_atomic_store(blk + 8, (static_cast<uint64_t>(epoch) << 32) | __float_as_uint(half_bits_to_float(dh)), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
			}
		}
	}
}

// A finished row goes out twice: as the plain output tensor (read by later launches) and as a tagged word for this launch's next stage.
__device__ __forceinline__ void store_row(float* __restrict__ y, uint64_t* __restrict__ y_tagged, unsigned epoch, int row, float v) {
	y[row] = v;
	__hip_atomic_store(&y_tagged[row], (static_cast<uint64_t>(epoch) << 32) | __float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Every gate/up wave takes a K range of both matrices (one staged slice of the input row for the two), two groups of each at a time:
// CHUNKS = 1 for hidden states up to 4096 values (a wave's whole share in one go), 2 up to 8192.
template<int CHUNKS> __global__ __launch_bounds__(GEMV_WAVES * 64) void decode_layer_kernel(layer_args a) {
	__shared__ __align__(16) uint8_t xs_q[GEMV_WAVES][CHAIN_DOWN_ROWS_TILES * GROUP_K];
	__shared__ float xs_d[GEMV_WAVES][CHAIN_DOWN_ROWS_TILES * GROUP_BLOCKS];
	__shared__ float red[GEMV_WAVES][64];
	__shared__ float red_up[GEMV_WAVES][64];
	__shared__ float norm_red[16];
	__shared__ __align__(16) float act_f[STRIP_ROWS];

	const int tid  = threadIdx.x;
	const int lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int wg   = static_cast<int>(blockIdx.x);
	if (wg < a.first_norm) {
		// ---- attn_out: rows of W_o against Q(attn), + layer_in ----
		const int strip = wg;
		int g0, g1;
		wave_k_range(a.groups_e, 0, 0, GEMV_WAVES, wave, g0, g1);
		const uint8_t* w_strip = a.w_o + macro_offset(strip, 0, a.groups_e);
		const int row_l		   = strip * STRIP_ROWS + (lane & 31);
		const float acc		   = gemv_chunk<CHAIN_TILES, X_F32, DUMP_NONE, false>(w_strip, a.attn, nullptr, xs_q[wave], xs_d[wave], g0, g1 - g0, a.groups_e, lane, row_l, a.n_embd, false, 0, nullptr);
		red[wave][lane] = acc;
		__syncthreads();
		if (tid < STRIP_ROWS) {
			float total = 0.0f;
#pragma unroll
			for (int w = 0; w < GEMV_WAVES; ++w) {
				total += red[w][tid] + red[w][32 + tid];
			}
			const int row = strip * STRIP_ROWS + tid;
			if (row < a.n_embd) {
				store_row(a.ffn_inp, a.attn_row, a.epoch, row, total + a.layer_in[row]);
			}
		}
		return;
	}
	if (wg == a.first_norm) {
		norm_workgroup(a.attn_row, a.ffn_norm_w, a.x_words, a.groups_e, a.eps, a.epoch, a.error_word, a.spin_limit, norm_red, lane, wave);
		return;
	}
	if (wg < a.first_consumer) {
		// ---- rows [32 * strip, + 32) of gate and of up against Q(n1) -> silu(g) * u -> activation block `strip` ----
		const int strip		   = wg - a.first_producer;
		const int g0		   = wave * a.p_per_slot + min(wave, a.p_rem);
		const int g1		   = g0 + a.p_per_slot + (wave < a.p_rem ? 1 : 0);
		const uint8_t* w_strip = a.w_gate + macro_offset(strip, 0, a.groups_e);
		const uint8_t* w_other = a.w_up + macro_offset(strip, 0, a.groups_e);
		const int row_l		   = strip * STRIP_ROWS + (lane & 31);
		float acc = 0.0f, acc_up = 0.0f;
		if constexpr (CHUNKS == 1) {
			acc = gemv_chunk<2, X_PUBLISHED_EARLY_WATCH, DUMP_NONE, false, 1, 2>(w_strip, a.x_words, a.error_word, xs_q[wave], xs_d[wave], g0, g1 - g0, a.groups_e, lane, row_l, a.n_ff, false, a.epoch, nullptr, 0,
				a.spin_limit, w_other, &acc_up);
		} else {
			for (int gc = g0; gc < g1; gc += 2) {
				float up_chunk = 0.0f;
				acc += gemv_chunk<2, X_PUBLISHED_EARLY, DUMP_NONE, false, 1, 2>(w_strip, a.x_words, a.error_word, xs_q[wave], xs_d[wave], gc, min(2, g1 - gc), a.groups_e, lane, row_l, a.n_ff, false, a.epoch,
					nullptr, 0, a.spin_limit, w_other, &up_chunk);
				acc_up += up_chunk;
				__builtin_amdgcn_wave_barrier(); // the next chunk overwrites this wave's LDS slices
			}
		}
		red_up[wave][lane] = acc_up;
		red[wave][lane] = acc;
		__syncthreads();
		if (wave == 0) {
			if (lane < STRIP_ROWS) {
				float g = 0.0f, u = 0.0f;
#pragma unroll
				for (int w = 0; w < GEMV_WAVES; ++w) {
					g += red[w][lane] + red[w][32 + lane];
					u += red_up[w][lane] + red_up[w][32 + lane];
				}
				act_f[lane]									  = silu_mul(g, u);
				a.gate_up[strip * STRIP_ROWS + lane]				  = g; // inspection copies, not read by this launch
				a.gate_up[FFN_MAX_HIDDEN + strip * STRIP_ROWS + lane] = u;
			}
			__builtin_amdgcn_wave_barrier();
			const float4 v = lane < 8 ? *reinterpret_cast<const float4*>(&act_f[4 * lane]) : make_float4(0.f, 0.f, 0.f, 0.f);
			uint16_t dh;
			const uint32_t packed = quantize_block_lane(v, &dh);
			const uint32_t d_bits = __builtin_amdgcn_readfirstlane(__float_as_uint(half_bits_to_float(dh)));
			if (lane <= 8) {
				const uint32_t payload = lane < 8 ? packed : d_bits;
				__hip_atomic_store(&a.act_words[strip * PUBLISHED_WORDS + lane], (static_cast<uint64_t>(a.epoch) << 32) | payload, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
			}
		}
		return;
	}
	if (wg < a.second_norm) {
		const int c = wg - a.first_consumer;
		if (a.down_by_rows) {
			// ---- 16 rows of a down strip against the whole published activation, + ffn_inp: the row is complete in this workgroup, so
			// what the next stage waits for leaves without the two trips through memory of a K-split hand-off ----
			const int gstrip = c >> 1, rowpart = c & 1;
			int g0, g1;
			wave_k_range(a.groups_f, 0, 0, GEMV_WAVES, wave, g0, g1);
			const uint8_t* w_strip = a.w_down + macro_offset(gstrip, 0, a.groups_f);
			const int row_l		   = gstrip * STRIP_ROWS + (lane & 31);
			const float acc = gemv_chunk<CHAIN_DOWN_ROWS_TILES, X_PUBLISHED_WATCH, DUMP_NONE, false, 2>(w_strip, a.act_words, a.error_word, xs_q[wave], xs_d[wave], g0, g1 - g0, a.groups_f, lane, row_l, a.n_embd, false,
				a.epoch, nullptr, rowpart, a.spin_limit);
			red[wave][lane] = acc;
			__syncthreads();
			if (tid < STRIP_ROWS / 2) {
				float total = 0.0f;
#pragma unroll
				for (int w = 0; w < GEMV_WAVES; ++w) {
					float part = 0.0f;
#pragma unroll
					for (int q = 0; q < 4; ++q) {
						part += red[w][q * (STRIP_ROWS / 2) + tid];
					}
					total += part;
				}
				const int row = gstrip * STRIP_ROWS + rowpart * (STRIP_ROWS / 2) + tid;
				if (row < a.n_embd) {
					const uint64_t t = __hip_atomic_load(&a.attn_row[row], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
					const float res	 = static_cast<unsigned>(t >> 32) == a.epoch ? __uint_as_float(static_cast<uint32_t>(t)) : __uint_as_float(0x7FC00000u);
					store_row(a.l_out, a.down_row, a.epoch, row, total + res);
				}
			}
			return;
		}
		// ---- a (32-row strip, K split) of the down projection against the published activation, + ffn_inp ----
		// (K part first, strip second: the first K part's activation blocks come from the first gate/up workgroups, so the down
		// workgroups that are dispatched first can finish instead of holding their CUs until the last gate/up workgroup is done:
		// a LLaMA-3-70B block 150.2 -> 145.5 us; no difference at the LLaMA-3-8B shapes, two K parts)
		const int splits   = 1 << a.split_shift;
		const int strips_d = (a.n_embd + STRIP_ROWS - 1) / STRIP_ROWS;
		const int split	   = c / strips_d;
		const int gstrip   = c - split * strips_d;
		int g0, g1;
		wave_k_range(a.groups_f, a.split_shift, split, GEMV_WAVES, wave, g0, g1);
		const uint8_t* w_strip = a.w_down + macro_offset(gstrip, 0, a.groups_f);
		const int row_l		   = gstrip * STRIP_ROWS + (lane & 31);
		const float acc = gemv_chunk<CHAIN_TILES, X_PUBLISHED, DUMP_NONE>(w_strip, a.act_words, a.error_word, xs_q[wave], xs_d[wave], g0, g1 - g0, a.groups_f, lane, row_l, a.n_embd, false, a.epoch, nullptr, 0,
			a.spin_limit);
		red[wave][lane] = acc;
		__syncthreads();
		if (tid >= STRIP_ROWS) {
			return;
		}
		float total = 0.0f;
#pragma unroll
		for (int w = 0; w < GEMV_WAVES; ++w) {
			total += red[w][tid] + red[w][32 + tid];
		}
		const int row = gstrip * STRIP_ROWS + tid;
		// the residual is this launch's own attn_out row.  Its words are final: this workgroup's activation exists only because the
		// norm workgroup read all of them.  (A word that does not carry the epoch all the same poisons the row.)
		float res = 0.0f;
		if (row < a.n_embd) {
			const uint64_t t = __hip_atomic_load(&a.attn_row[row], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
			res				 = static_cast<unsigned>(t >> 32) == a.epoch ? __uint_as_float(static_cast<uint32_t>(t)) : __uint_as_float(0x7FC00000u);
		}
		if (splits == 1) {
			if (row < a.n_embd) {
				store_row(a.l_out, a.down_row, a.epoch, row, total + res);
			}
			return;
		}
		// K over several workgroups: tagged shares, everybody reads them all, who sees them all stores (split_k_finish's protocol)
		uint64_t* mine = a.tagged + static_cast<int64_t>(gstrip) * splits * STRIP_ROWS + tid;
		asm volatile("" : "+v"(res)::"memory");
		__hip_atomic_store(&mine[split * STRIP_ROWS], (static_cast<uint64_t>(a.epoch) << 32) | __float_as_uint(total), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		wait_stores_acknowledged();
		bool all  = true;
		float sum = 0.0f;
		for (int sp0 = 0; sp0 < splits; sp0 += 8) {
			uint64_t v[8];
#pragma unroll
			for (int u = 0; u < 8; ++u) {
				v[u] = (sp0 + u < splits) ? __hip_atomic_load(&mine[(sp0 + u) * STRIP_ROWS], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0ull;
			}
#pragma unroll
			for (int u = 0; u < 8; ++u) {
				if (sp0 + u < splits) {
					all = all && static_cast<unsigned>(v[u] >> 32) == a.epoch;
					sum += __uint_as_float(static_cast<uint32_t>(v[u]));
				}
			}
		}
		if (all && row < a.n_embd) {
			store_row(a.l_out, a.down_row, a.epoch, row, sum + res);
		}
		return;
	}
	if (wg == a.second_norm) {
		norm_workgroup(a.down_row, a.next_norm_w, a.x_words_next, a.groups_e, a.eps, a.epoch, a.error_word, a.spin_limit, norm_red, lane, wave);
		return;
	}
	// ---- the projections behind the next norm: rows of W_next[i] against Q(n2) ----
	{
		const int gstrip = wg - a.first_next;
		const int sidx	 = (gstrip >= a.next.strip_end[0]) + (gstrip >= a.next.strip_end[1]);
		const int strip	 = gstrip - (sidx == 0 ? 0 : a.next.strip_end[sidx - 1]);
		const int N		 = a.next.rows[sidx];
		int g0, g1;
		wave_k_range(a.groups_e, 0, 0, GEMV_WAVES, wave, g0, g1);
		const uint8_t* w_strip = a.next.W[sidx] + macro_offset(strip, 0, a.groups_e);
		const int row_l		   = strip * STRIP_ROWS + (lane & 31);
		const float acc = gemv_chunk<CHAIN_TILES, CHUNKS == 1 ? X_PUBLISHED_EARLY_WATCH : X_PUBLISHED_EARLY, DUMP_NONE>(w_strip, a.x_words_next, a.error_word, xs_q[wave], xs_d[wave], g0, g1 - g0, a.groups_e, lane, row_l, N, false, a.epoch, nullptr, 0,
			a.spin_limit);
		red[wave][lane] = acc;
		__syncthreads();
		if (tid < STRIP_ROWS) {
			float total = 0.0f;
#pragma unroll
			for (int w = 0; w < GEMV_WAVES; ++w) {
				total += red[w][tid] + red[w][32 + tid];
			}
			const int row = strip * STRIP_ROWS + tid;
			if (row < N) {
				a.next.y[sidx][row] = total;
			}
		}
	}
}

// Whether the shape takes the one-launch form; otherwise (and under HIP graph capture, where a replay could not renew the epoch) the
// layer runs as its three launches.
bool decode_layer_chains(int64_t n_embd, int64_t n_ff, int64_t next_strips) {
	if (n_embd <= 0 || n_ff <= 0 || n_embd % GROUP_K != 0 || n_ff % GROUP_K != 0 || n_embd > CHAIN_MAX_EMBD || n_ff > FFN_MAX_HIDDEN) {
		return false;
	}
	const int64_t strips_e = n_embd / STRIP_ROWS, groups_f = n_ff / GROUP_K;
	// the down projection's K split must bring a wave's share to four groups within the scratch
	int splits = 1;
	while ((groups_f + GEMV_WAVES * splits - 1) / (GEMV_WAVES * splits) > CHAIN_TILES && strips_e <= GEMV_MAX_SPLIT_STRIPS && strips_e * splits * 2 <= GEMV_MAX_SPLIT_UNITS) {
		splits *= 2;
	}
	if ((groups_f + GEMV_WAVES * splits - 1) / (GEMV_WAVES * splits) > CHAIN_TILES) {
		return false;
	}
	return next_strips >= 0 && next_strips < (1 << 20);
}

hipError_t launch_decode_layer(const void* w_o, const float* attn, const float* layer_in, float* ffn_inp, const void* w_gate, const void* w_up, const void* w_down, const float* ffn_norm_w,
	float* l_out, const void* const* w_next, float* const* y_next, const int64_t* n_next, int count_next, const float* next_norm_w, float eps, int64_t n_embd, int64_t n_ff, hipStream_t s) {
	int64_t next_strips = 0;
	for (int i = 0; i < count_next; ++i) {
		next_strips += (n_next[i] + STRIP_ROWS - 1) / STRIP_ROWS;
	}
	if (!decode_layer_chains(n_embd, n_ff, next_strips) || stream_is_capturing(s) || !in_kernel_waits_enabled()) {
		// the same three steps as launches of their own
		const void* w1[1]  = { w_o };
		float* y1[1]	   = { ffn_inp };
		const float* r1[1] = { layer_in };
		hipError_t e	   = launch_gemv_tiled_multi(w1, y1, &n_embd, 1, attn, true, n_embd, s, nullptr, 0.0f, r1);
		if (e != hipSuccess) {
			return e;
		}
		e = launch_ffn_decode(w_gate, w_up, w_down, ffn_inp, ffn_norm_w, eps, ffn_inp, l_out, n_ff, n_embd, n_embd, s);
		if (e != hipSuccess || next_strips == 0) {
			return e;
		}
		return launch_gemv_tiled_multi(w_next, y_next, n_next, count_next, l_out, true, n_embd, s, next_norm_w, eps);
	}
	gemv_scratch sc;
	const hipError_t e = get_gemv_scratch(&sc, true, s);
	if (e != hipSuccess) {
		return e;
	}
	layer_args a{};
	a.w_o		 = static_cast<const uint8_t*>(w_o);
	a.attn		 = attn;
	a.layer_in	 = layer_in;
	a.ffn_inp	 = ffn_inp;
	a.ffn_norm_w = ffn_norm_w;
	a.w_gate	 = static_cast<const uint8_t*>(w_gate);
	a.w_up		 = static_cast<const uint8_t*>(w_up);
	a.w_down	 = static_cast<const uint8_t*>(w_down);
	a.l_out		 = l_out;
	a.next_norm_w = next_norm_w;
	int64_t strips = 0;
	for (int i = 0; i < GEMV_MAX_SEGMENTS; ++i) {
		if (i < count_next) {
			a.next.W[i]	   = static_cast<const uint8_t*>(w_next[i]);
			a.next.y[i]	   = y_next[i];
			a.next.rows[i] = static_cast<int>(n_next[i]);
			strips += (n_next[i] + STRIP_ROWS - 1) / STRIP_ROWS;
		}
		a.next.strip_end[i] = static_cast<int>(strips);
	}
	a.eps	   = eps;
	a.n_embd   = static_cast<int>(n_embd);
	a.n_ff	   = static_cast<int>(n_ff);
	a.groups_e = static_cast<int>(n_embd / GROUP_K);
	a.groups_f = static_cast<int>(n_ff / GROUP_K);
	const int strips_e = static_cast<int>(n_embd / STRIP_ROWS);
	// attn_out: whole strips.  As a launch of its own a matrix with fewer strips than CUs is cut by rows so that it reaches them all;
	// here the gate/up workgroups behind it fill the other CUs and have their weights on the way at once, and the CUs that start
	// on attn_out run a few microseconds ahead of the rest from then on, so the chip's workgroups do not change rounds in lock-step
	// (measured at the LLaMA-3-8B block: 43.1 us against 44.0 us with half strips).
	// gate/up: sixteen K ranges per workgroup, both matrices per wave, two groups of each at a time: one such chunk covers a wave's
	// share up to 4096 values of hidden state, two up to 8192 (CHAIN_MAX_EMBD).  (Up to 8192 the stage used to give eight waves to each
	// matrix, four groups at a time: 128 registers and spills, the LLaMA-3-70B block 160.8 us against 150.3 us in this form.)
	const bool one_chunk = (a.groups_e + GEMV_WAVES - 1) / GEMV_WAVES <= 2;
	a.p_per_slot		 = a.groups_e / GEMV_WAVES;
	a.p_rem				 = a.groups_e % GEMV_WAVES;
	int splits = 1;
	while ((a.groups_f + GEMV_WAVES * splits - 1) / (GEMV_WAVES * splits) > CHAIN_TILES) {
		splits *= 2;
	}
	while ((1 << a.split_shift) < splits) {
		++a.split_shift;
	}
	// Down cut by rows instead of K where two workgroups per strip are what the K split would make anyway, they put a workgroup on
	// every CU and a wave can hold its whole share of K (the LLaMA-3-8B block: 256 workgroups of 16 rows, seven half-size groups per
	// wave): a finished row then leaves its workgroup directly, without the K-split hand-off's two trips through memory, on the path
	// that ends the launch.  Measured at that block: 42.6 against 43.1 us (the stage behind the down projection 6.2 against 6.8 us).
	// As a launch of its own, or in the one-launch FFN, the same cut measured no different from the K split.
	a.down_by_rows = splits == 2 && strips_e * 2 <= 256 && (a.groups_f + GEMV_WAVES - 1) / GEMV_WAVES <= CHAIN_DOWN_ROWS_TILES;
	a.first_norm	 = strips_e;
	a.first_producer = a.first_norm + 1;
	a.first_consumer = a.first_producer + static_cast<int>(n_ff / STRIP_ROWS);
	a.second_norm	 = a.first_consumer + strips_e * splits;
	a.first_next	 = a.second_norm + 1;
	const unsigned grid = static_cast<unsigned>(next_strips > 0 ? a.first_next + next_strips : a.second_norm);
	a.attn_row		= sc.row_tagged[0];
	a.x_words		= sc.x_words;
	a.gate_up		= sc.gate_up;
	a.act_words		= sc.act_words;
	a.tagged		= sc.tagged;
	a.down_row		= sc.row_tagged[1];
	a.x_words_next	= sc.x_words_next;
	a.epoch			= sc.epoch;
	a.error_word	= sc.error_word;
	a.spin_limit	= sc.spin_limit;
	const dim3 block(GEMV_WAVES * 64);
	return one_chunk ? launch_kernel(KIND_GEMV, decode_layer_kernel<1>, dim3(grid), block, 0, s, a) : launch_kernel(KIND_GEMV, decode_layer_kernel<2>, dim3(grid), block, 0, s, a);
}

} // namespace nh
