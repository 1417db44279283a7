// mega_dispatch.hpp -- the gfx950 specialisations of the reference's LIVE kernel specialisation point.
//
// The reference's scheduler reaches every kernel through one class template (paths relative to include/nihilus-incl/):
//
//   template<typename config_type, typename core_traits_type, device_types, uint64_t arch, core_types, processing_phases>
//   struct kernel_dispatcher_impl;                                                      common/kernel_traits.hpp:382-383
//
// picked by kernel_dispatcher<config, phase, core_type>::impl(params[, current_block]) (infra/monolithic_dispatcher.hpp:41-66)
// from per_block_thread_function (infra/behavioral_axes.hpp:399-416).  One specialisation exists per "mega" core of the
// model graph and phase; the reference's GPU ones are models of the calling convention with empty bodies
// (cuda/cuda_12.hpp:803-952: arch 4, impl(core_traits_type& params[, int64_t current_block]), operands looked up through
// params.values / get_adjacent_value, pointers handed over in params.data_ptrs).  This header supplies the same four
// specialisations for device_types::gpu, arch index 5 (= gfx950), both phases, with the Q8_0 mat-mul path as their bodies:
//
//   core_types::mega_qkv_prep_and_cache_publish   rms_norm -> mul(attn_norm) -> q, k, v mul_mat        infra/core_traits.hpp:570-594
//   core_types::mega_attention_apply              attn_out mul_mat -> residual add                     infra/core_traits.hpp:768-772
//   core_types::mega_ffn                          rms_norm -> mul(ffn_norm) -> gate, up mul_mat -> silu -> mul -> down mul_mat -> residual add
//                                                                                                      infra/core_traits.hpp:971-995
//   core_types::final_norm_and_sampling           rms_norm -> mul(output_norm) -> logits mul_mat      infra/core_traits.hpp:1186-1193
//
// eval_time: the mat-vecs from one attention to the next are ONE launch (nh_q8_0_decode_layer_f32): mega_attention_apply runs the
// attention hook and leaves its attn_out projection to mega_ffn, whose launch is [attn_out + residual -> norm -> gate/up -> SiLU * up ->
// down + residual -> norm -> the NEXT block's q / k / v] (behind the last block: -> the logits); mega_qkv_prep_and_cache_publish of the
// next block and final_norm_and_sampling then find their mat-vecs done and run only their hooks.  Per token: the first block's q / k / v
// plus one launch per block, where the reference's fold makes three synchronous launches per block (cuda/thread_pool.hpp:46-67).  A
// config that needs every core's outputs complete when that core returns declares `static constexpr bool amd_decode_per_core_launches
// = true` and gets one launch per core instead (the quantize, the norm, SiLU * up and the residual add inside the mat-vec kernels).
// prompt_eval_time bodies quantize into a workspace and run the int8-MFMA mat-mat.
//
// What those cores hold besides mat-muls is outside this path and is reached through three customisation points that a
// config MUST specialise: without them a model runs and produces garbage (no rope, no cache write, q standing in for the
// attention output, no sampled token).  The primary templates therefore refuse to compile, unless the config declares
// `static constexpr bool amd_matmul_only = true` -- what a benchmark or a test of the mat-mul path alone does -- in which case
// they do the minimum that keeps the data flowing:
//   amd_qkv_epilogue<config>    rope on q and k, the k / v cache write              (reshape/rope/copy nodes, core_traits.hpp:596-616)
//   amd_attention<config>       k.q, softmax, .v, merge: produces the attn_out operand  (core_traits.hpp:743-766)
//   amd_sampling<config>        logit bias, penalties, top-k/p, sample               (core_traits.hpp:1195-1227)
//
// Operand conventions of the bodies: Q8_0 weight pointers (get_data(current_block) of attn_q, attn_k, attn_v, attn_output,
// ffn_gate, ffn_up, ffn_down, get_data() of output) name the TILED copy made at load time with nh_q8_0_tile, where the
// reference copies weights into its device arena (infra/model_parser.hpp:151-154); norm weights and activations are fp32.
// A layer's input is the token-embedding output for block 0 and the previous block's l_out after that.
//
// This header sees no HIP header.  Inside the reference tree: define NIHILUS_AMD_WITH_REFERENCE_HEADERS and include the
// reference's headers first; stand-alone, reference_mirror.hpp declares the same names.
#pragma once

#include "mul_mat_dispatch.hpp"

#include <mutex>

namespace nihilus {

	namespace amd_detail {

		// Device memory the bodies need beyond the graph's own tensors: quantized activations of the prompt phase, the k / v
		// projections in front of the cache write, the fp32 gate / up outputs of a prompt-phase FFN, the logits.  The
		// reference's kernels never allocate: its arena is sized once from a compile-time plan over the graph nodes
		// (infra/behavioral_axes.hpp:61-90, infra/model.hpp:241).  Here the same happens in amd_prepare (below): every slot is
		// sized once for the longest sequence the config allows, and the dispatchers only check capacity.  One host thread
		// drives the GPU (cuda/thread_pool.hpp:46-67).
		enum workspace_slot : int { slot_quantized = 0, slot_k, slot_v, slot_activation, slot_gate_up, slot_attention, slot_logits, slot_count };
		struct workspace_entry {
			void* ptr{};
			int64_t bytes{};
		};
		template<typename config_type> struct workspace_pool {
			workspace_entry slots[slot_count]{};
			std::mutex lock{};
			int64_t allocations{}; // nh_malloc calls made for this config so far (a test reads it: none after amd_prepare)
			static workspace_pool& get() {
				static workspace_pool pool{};
				return pool;
			}
		};
		// A slot of at least `bytes`.  Allocates nothing: a slot that amd_prepare did not make large enough is an error.
		template<typename config_type> inline void* workspace(int slot, int64_t bytes, const std::source_location where = std::source_location::current()) {
			auto& pool = workspace_pool<config_type>::get();
			std::lock_guard<std::mutex> guard{ pool.lock };
			const workspace_entry& e = pool.slots[slot];
			if (e.bytes < bytes) {
				check<config_type>(NH_ERR_TOO_LARGE, "workspace: call nihilus::amd_prepare<config, model_traits>(max_sequence_length) first, with a sequence length that covers this call", where);
				return nullptr;
			}
			return e.ptr;
		}
		template<typename config_type> inline void reserve_slot(int slot, int64_t bytes, const std::source_location where = std::source_location::current()) {
			auto& pool = workspace_pool<config_type>::get();
			std::lock_guard<std::mutex> guard{ pool.lock };
			workspace_entry& e = pool.slots[slot];
			bytes			   = (bytes + 255) / 256 * 256;
			if (e.bytes < bytes) {
				check<config_type>(nh_stream_sync(nullptr), "amd_prepare: stream sync", where); // the old buffer may still be in use by enqueued work
				check<config_type>(nh_free(e.ptr), "amd_prepare: free", where);
				e = workspace_entry{};
				check<config_type>(nh_malloc(&e.ptr, bytes), "amd_prepare: alloc", where);
				e.bytes = bytes;
				++pool.allocations;
			}
		}

		// get_data() of a graph node, per transformer block or global as the node's data strategy says.
		template<typename op_type> inline auto* data_of(op_type& op, int64_t current_block) {
			if constexpr (op_type::data_strategy_type == data_strategy_types::per_block) {
				return op.get_data(static_cast<uint64_t>(current_block));
			} else {
				return op.get_data();
			}
		}

		// The reference waits for the device after every launch (cuda/cuda_12.hpp:679) and looks at the error state only in dev
		// builds (:650-655); launches on one stream are ordered without that, so the wait is kept for dev builds only.
		template<typename config_type> inline void after_launch(const std::source_location where = std::source_location::current()) {
			if constexpr (config_type::dev) {
				check<config_type>(nh_stream_sync(nullptr), "stream sync", where);
			}
		}

		// A config that runs the mat-mul path alone (benchmarks, tests) says so; only then do the primary customisation points compile.
		template<typename config_type> inline constexpr bool matmul_only = [] {
			if constexpr (requires { config_type::amd_matmul_only; }) {
				return static_cast<bool>(config_type::amd_matmul_only);
			} else {
				return false;
			}
		}();

		// eval_time chains a block's mat-vecs into one launch unless the config asks for one launch per core.
		template<typename config_type> inline constexpr bool chains_decode = [] {
			if constexpr (requires { config_type::amd_decode_per_core_launches; }) {
				return !static_cast<bool>(config_type::amd_decode_per_core_launches);
			} else {
				return true;
			}
		}();
		// What the eval_time cores hand to each other when they chain (one host thread drives the GPU, cuda/thread_pool.hpp:46-67):
		// the attn_out projection that mega_attention_apply left to mega_ffn, and which mat-vecs a launch has already done for the
		// core that comes next.
		template<typename config_type> struct decode_chain_state {
			int64_t attn_block{ -1 }; // block whose attn_out projection is pending; its operands:
			const void* w_o{};
			const float* attn{};
			const float* layer_in{};
			float* ffn_inp{};
			int64_t qkv_done_block{ -1 }; // block whose q / k / v the previous block's launch has computed
			bool logits_done{}; // the last block's launch has computed the logits
			static decode_chain_state& get() {
				static decode_chain_state state{};
				return state;
			}
		};

		// The input of transformer block `current_block`: token embeddings for the first, the previous block's l_out afterwards.
		template<typename core_traits_type> inline const float* layer_input(core_traits_type& params, int64_t current_block) {
			using config_type = typename core_traits_type::config_type;
			if (current_block == 0) {
				auto& token_embd_core = get_adjacent_value<config_type, core_types::token_embeddings>::impl(params);
				return token_embd_core.values.template get_core<token_embeddings_types, token_embeddings_types::get_rows>().template get_data<float>();
			}
			auto& ffn_core = get_adjacent_value<config_type, core_types::mega_ffn>::impl(params);
			return ffn_core.values.template get_core<mega_ffn_types, mega_ffn_types::l_out>().template get_data<float>();
		}

	} // namespace amd_detail

	// ---- set-up ---------------------------------------------------------------------------------------------------------

	// Sizes every device buffer the dispatchers below need beyond the graph's tensors, once, for sequences of up to
	// `max_sequence_length` rows, and has the library make its own per-device scratch (nh_q8_0_prepare).  Call it after the
	// model's memory is set up and before the first impl: from then on no impl allocates, frees or waits for the device on
	// behalf of memory (a sequence longer than prepared for is reported through the config's error convention).  Stands for
	// the reference's compile-time memory plan (infra/behavioral_axes.hpp:61-90).  model_traits_type: the mtt of the config's
	// core traits (embedding_length, feed_forward_length, n_embd_kv_gqa, vocab_size).
	template<typename config_type, typename model_traits_type> inline void amd_prepare(uint64_t max_sequence_length = config_type::max_sequence_length) {
		const int64_t rows	 = max_sequence_length < 1 ? 1 : static_cast<int64_t>(max_sequence_length);
		const int64_t n_embd = model_traits_type::embedding_length, n_ff = model_traits_type::feed_forward_length, n_kv = model_traits_type::n_embd_kv_gqa;
		int64_t quantized	 = nh_q8_0_tiled_bytes(rows, n_embd);
		const int64_t other	 = nh_q8_0_mul_mat_workspace_bytes(rows, n_embd);
		quantized			 = other > quantized ? other : quantized;
		amd_detail::reserve_slot<config_type>(amd_detail::slot_quantized, quantized); // activations quantized along the embedding
		amd_detail::reserve_slot<config_type>(amd_detail::slot_k, rows * n_kv * 4);
		amd_detail::reserve_slot<config_type>(amd_detail::slot_v, rows * n_kv * 4);
		amd_detail::reserve_slot<config_type>(amd_detail::slot_activation, nh_q8_0_tiled_bytes(rows, n_ff)); // the down projection's quantized activation
		// fp32 gate / up outputs of prompts too short for the fused gate / up kernel (longer ones need none)
		int64_t gate_up = 0;
		for (int64_t r = 1; r <= rows; ++r) {
			const int64_t need = nh_q8_0_gate_up_silu_workspace_bytes(r, n_ff, n_embd);
			gate_up			   = need > gate_up ? need : gate_up;
		}
		amd_detail::reserve_slot<config_type>(amd_detail::slot_gate_up, gate_up);
		amd_detail::reserve_slot<config_type>(amd_detail::slot_attention, rows * n_embd * 4);
		amd_detail::reserve_slot<config_type>(amd_detail::slot_logits, static_cast<int64_t>(model_traits_type::vocab_size) * 4);
		amd_detail::check<config_type>(nh_q8_0_prepare(), "amd_prepare: library scratch");
	}
	// How many device allocations amd_prepare has made for this config (a later amd_prepare with a longer sequence adds to it; impl never does).
	template<typename config_type> inline int64_t amd_workspace_allocations() {
		auto& pool = amd_detail::workspace_pool<config_type>::get();
		std::lock_guard<std::mutex> guard{ pool.lock };
		return pool.allocations;
	}

	// ---- customisation points for the nodes of a mega core that are not mat-muls --------------------------------------

	// After the q / k / v projections: q [sequence_length][embedding_length] sits in the core's q_out tensor, k and v
	// [sequence_length][n_embd_kv_gqa] in scratch.  A config's specialisation applies rope to q and k and writes k / v into
	// the cache (params.data_ptrs holds inp_pos, rope_freqs, cache_k, cache_v).  Primary (amd_matmul_only configs): nothing.
	template<typename config_type> struct amd_qkv_epilogue {
		template<typename core_traits_type>
		static void impl(core_traits_type&, int64_t /*current_block*/, uint64_t /*sequence_length*/, float* /*q*/, const float* /*k*/, const float* /*v*/, void* /*stream*/) {
			static_assert(amd_detail::matmul_only<config_type>,
				"specialise nihilus::amd_qkv_epilogue<config> (rope on q and k, k / v cache write), or declare config::amd_matmul_only = true to run the mat-mul path alone");
		}
	};

	// In front of the attn_out projection: returns the attention output, fp32 [sequence_length][embedding_length].  A config's
	// specialisation runs k.q, softmax, .v and the head merge into `scratch` and returns it.  Primary (amd_matmul_only configs):
	// the q tensor itself (attention over a single cached position with v = q), which keeps shapes and data flow those of the model.
	template<typename config_type> struct amd_attention {
		template<typename core_traits_type>
		static const float* impl(core_traits_type& params, int64_t /*current_block*/, uint64_t /*sequence_length*/, float* /*scratch*/, void* /*stream*/) {
			static_assert(amd_detail::matmul_only<config_type>,
				"specialise nihilus::amd_attention<config> (k.q, softmax, .v, head merge), or declare config::amd_matmul_only = true to run the mat-mul path alone");
			return params.data_ptrs.template get_q_input_data<float>();
		}
	};

	// Behind the logits mat-vec: logits fp32 [vocab_size] of the last token.  A config's specialisation applies the sampling
	// chain and writes params.data_ptrs.get_result_token_id_data, which the reference's generation loop reads next.  Primary
	// (amd_matmul_only configs): nothing (the logits stay in the scratch slot, no token id is written).
	template<typename config_type> struct amd_sampling {
		template<typename core_traits_type> static void impl(core_traits_type&, const float* /*logits*/, void* /*stream*/) {
			static_assert(amd_detail::matmul_only<config_type>,
				"specialise nihilus::amd_sampling<config> (sampling chain, writes result_token_id), or declare config::amd_matmul_only = true to run the mat-mul path alone");
		}
	};

	// ---- mega_qkv_prep_and_cache_publish --------------------------------------------------------------------------------

	template<typename config_type, typename core_traits_type, processing_phases processing_phase>
	struct kernel_dispatcher_impl<config_type, core_traits_type, device_types::gpu, gfx950_arch_index, core_types::mega_qkv_prep_and_cache_publish, processing_phase> {
		static void impl(core_traits_type& params, int64_t current_block) {
			using mtt					   = typename core_traits_type::mtt;
			using cfg					   = typename core_traits_type::config_type;
			static constexpr int64_t n_embd = mtt::embedding_length;
			static constexpr int64_t n_kv   = mtt::n_embd_kv_gqa;
			static_assert(n_embd % 128 == 0, "the tiled weight layout needs the embedding length to be a multiple of 128");

			auto& q_out_op		 = params.values.template get_core<mega_qkv_prep_and_cache_publish_types, mega_qkv_prep_and_cache_publish_types::q_out>();
			auto& weights_core	 = get_adjacent_value<cfg, core_types::weights>::impl(params);
			auto& inputs_core	 = get_adjacent_value<cfg, core_types::global_inputs>::impl(params);
			auto& attn_norm_w_op = weights_core.values.template get_core<weight_types, weight_types::attn_norm>();
			auto& attn_q_w_op	 = weights_core.values.template get_core<weight_types, weight_types::attn_q>();
			auto& attn_k_w_op	 = weights_core.values.template get_core<weight_types, weight_types::attn_k>();
			auto& attn_v_w_op	 = weights_core.values.template get_core<weight_types, weight_types::attn_v>();
			auto& rope_freqs_op	 = weights_core.values.template get_core<weight_types, weight_types::rope_freqs>();
			auto& inp_pos_op	 = inputs_core.values.template get_core<global_input_types, global_input_types::inp_pos>();
			auto& cache_k_op	 = inputs_core.values.template get_core<global_input_types, global_input_types::cache_k>();
			auto& cache_v_op	 = inputs_core.values.template get_core<global_input_types, global_input_types::cache_v>();

			const uint64_t sequence_length = q_out_op.get_seq_length_dim();
			params.data_ptrs.set_ptrs(q_out_op.get_data(), amd_detail::layer_input(params, current_block), amd_detail::data_of(attn_norm_w_op, current_block),
				amd_detail::data_of(attn_q_w_op, current_block), amd_detail::data_of(attn_k_w_op, current_block), amd_detail::data_of(attn_v_w_op, current_block),
				amd_detail::data_of(inp_pos_op, current_block), amd_detail::data_of(rope_freqs_op, current_block), amd_detail::data_of(cache_k_op, current_block),
				amd_detail::data_of(cache_v_op, current_block));
			if (sequence_length == 0) {
				return; // the reference launches nothing for an empty sequence (cuda/cuda_12.hpp:657)
			}
			auto ptrs			  = params.data_ptrs; // the pack travels by value, as it does into the reference's kernels (cuda/cuda_12.hpp:648)
			const int64_t rows	  = processing_phase == processing_phases::eval_time ? 1 : static_cast<int64_t>(sequence_length);
			float* q			  = ptrs.template get_q_output_data<float>();
			float* k			  = static_cast<float*>(amd_detail::workspace<config_type>(amd_detail::slot_k, rows * n_kv * 4));
			float* v			  = static_cast<float*>(amd_detail::workspace<config_type>(amd_detail::slot_v, rows * n_kv * 4));
			const float* x		  = ptrs.template get_inp_embd_data<float>();
			const float* norm_w	  = ptrs.template get_attn_norm_w_data<float>();
			const void* weights[3] = { ptrs.template get_attn_q_w_data<void>(), ptrs.template get_attn_k_w_data<void>(), ptrs.template get_attn_v_w_data<void>() };
			float* outputs[3]	  = { q, k, v };
			const int64_t ns[3]	  = { n_embd, n_kv, n_kv };
			if constexpr (processing_phase == processing_phases::eval_time) {
				auto& chain = amd_detail::decode_chain_state<config_type>::get();
				if (amd_detail::chains_decode<config_type> && chain.qkv_done_block == current_block) {
					// the previous block's launch ended in this block's norm + q / k / v (same operands, same outputs): only the hook is left
				} else {
					amd_detail::check<config_type>(nh_q8_0_gemv_tiled_multi_norm_f32(weights, outputs, ns, 3, x, norm_w, mtt::layer_norm_rms_epsilon, n_embd, nullptr),
						"mega_qkv eval_time: norm + q/k/v mat-vec");
				}
				chain.qkv_done_block = -1;
			} else {
				amd_detail::decode_chain_state<config_type>::get() = {}; // a prompt pass ends whatever a decode step had pending
				void* xq = amd_detail::workspace<config_type>(amd_detail::slot_quantized, nh_q8_0_tiled_bytes(rows, n_embd));
				amd_detail::check<config_type>(nh_q8_0_rms_norm_quantize_tiled(x, norm_w, mtt::layer_norm_rms_epsilon, xq, rows, n_embd, nullptr), "mega_qkv prompt_eval_time: norm + quantize");
				for (int i = 0; i < 3; ++i) {
					amd_detail::check<config_type>(nh_q8_0_gemm_tiled(weights[i], xq, outputs[i], rows, ns[i], n_embd, nullptr), "mega_qkv prompt_eval_time: q/k/v mat-mat");
				}
			}
			amd_qkv_epilogue<config_type>::impl(params, current_block, static_cast<uint64_t>(rows), q, k, v, nullptr);
			amd_detail::after_launch<config_type>();
		}
	};

	// ---- mega_attention_apply -------------------------------------------------------------------------------------------

	template<typename config_type, typename core_traits_type, processing_phases processing_phase>
	struct kernel_dispatcher_impl<config_type, core_traits_type, device_types::gpu, gfx950_arch_index, core_types::mega_attention_apply, processing_phase> {
		static void impl(core_traits_type& params, int64_t current_block) {
			using mtt					   = typename core_traits_type::mtt;
			using cfg					   = typename core_traits_type::config_type;
			static constexpr int64_t n_embd = mtt::embedding_length;

			auto& ffn_inp_op	   = params.values.template get_core<mega_attention_apply_types, mega_attention_apply_types::ffn_inp>();
			auto& weights_core	   = get_adjacent_value<cfg, core_types::weights>::impl(params);
			auto& inputs_core	   = get_adjacent_value<cfg, core_types::global_inputs>::impl(params);
			auto& qkv_core		   = get_adjacent_value<cfg, core_types::mega_qkv_prep_and_cache_publish>::impl(params);
			auto& q_out_op		   = qkv_core.values.template get_core<mega_qkv_prep_and_cache_publish_types, mega_qkv_prep_and_cache_publish_types::q_out>();
			auto& attn_output_w_op = weights_core.values.template get_core<weight_types, weight_types::attn_output>();
			auto& cache_k_op	   = inputs_core.values.template get_core<global_input_types, global_input_types::cache_k>();
			auto& cache_v_op	   = inputs_core.values.template get_core<global_input_types, global_input_types::cache_v>();
			auto& kq_mask_op	   = inputs_core.values.template get_core<global_input_types, global_input_types::kq_mask>();

			const uint64_t sequence_length = ffn_inp_op.get_seq_length_dim();
			params.data_ptrs.set_ptrs(ffn_inp_op.get_data(), q_out_op.get_data(), amd_detail::data_of(cache_k_op, current_block), amd_detail::data_of(cache_v_op, current_block),
				amd_detail::data_of(kq_mask_op, current_block), amd_detail::data_of(attn_output_w_op, current_block), amd_detail::layer_input(params, current_block));
			if (sequence_length == 0) {
				return;
			}
			auto ptrs			 = params.data_ptrs;
			const int64_t rows	 = processing_phase == processing_phases::eval_time ? 1 : static_cast<int64_t>(sequence_length);
			float* scratch		 = static_cast<float*>(amd_detail::workspace<config_type>(amd_detail::slot_attention, rows * n_embd * 4));
			const float* attn	 = amd_attention<config_type>::impl(params, current_block, static_cast<uint64_t>(rows), scratch, nullptr);
			const float* residual = ptrs.template get_inp_embd_data<float>();
			float* y			 = ptrs.template get_ffn_inp_data<float>();
			const void* w		 = ptrs.template get_attn_output_w_data<void>();
			if constexpr (processing_phase == processing_phases::eval_time && amd_detail::chains_decode<config_type>) {
				// left to mega_ffn of this block, whose launch starts with this projection
				auto& chain	   = amd_detail::decode_chain_state<config_type>::get();
				chain.attn_block = current_block;
				chain.w_o		 = w;
				chain.attn		 = attn;
				chain.layer_in	 = residual;
				chain.ffn_inp	 = y;
			} else if constexpr (processing_phase == processing_phases::eval_time) {
				amd_detail::check<config_type>(nh_q8_0_gemv_tiled_residual_f32(w, attn, residual, y, n_embd, n_embd, nullptr), "mega_attention_apply eval_time: attn_out mat-vec + residual");
			} else {
				const int64_t ws_bytes = nh_q8_0_mul_mat_workspace_bytes(rows, n_embd);
				void* ws			   = amd_detail::workspace<config_type>(amd_detail::slot_quantized, ws_bytes);
				amd_detail::check<config_type>(nh_q8_0_mul_mat_residual(w, attn, residual, y, rows, n_embd, n_embd, ws, ws_bytes, nullptr),
					"mega_attention_apply prompt_eval_time: attn_out mat-mat + residual");
			}
			amd_detail::after_launch<config_type>();
		}
	};

	// ---- mega_ffn -------------------------------------------------------------------------------------------------------

	template<typename config_type, typename core_traits_type, processing_phases processing_phase>
	struct kernel_dispatcher_impl<config_type, core_traits_type, device_types::gpu, gfx950_arch_index, core_types::mega_ffn, processing_phase> {
		static void impl(core_traits_type& params, int64_t current_block) {
			using mtt					   = typename core_traits_type::mtt;
			using cfg					   = typename core_traits_type::config_type;
			static constexpr int64_t n_embd = mtt::embedding_length;
			static constexpr int64_t n_ff   = mtt::feed_forward_length;
			static_assert(n_embd % 128 == 0 && n_ff % 128 == 0, "the tiled weight layout needs both lengths to be multiples of 128");

			auto& l_out_op		= params.values.template get_core<mega_ffn_types, mega_ffn_types::l_out>();
			auto& weights_core	= get_adjacent_value<cfg, core_types::weights>::impl(params);
			auto& attn_core		= get_adjacent_value<cfg, core_types::mega_attention_apply>::impl(params);
			auto& ffn_inp_op	= attn_core.values.template get_core<mega_attention_apply_types, mega_attention_apply_types::ffn_inp>();
			auto& ffn_norm_w_op = weights_core.values.template get_core<weight_types, weight_types::ffn_norm>();
			auto& ffn_gate_w_op = weights_core.values.template get_core<weight_types, weight_types::ffn_gate>();
			auto& ffn_up_w_op	= weights_core.values.template get_core<weight_types, weight_types::ffn_up>();
			auto& ffn_down_w_op = weights_core.values.template get_core<weight_types, weight_types::ffn_down>();

			const uint64_t sequence_length = l_out_op.get_seq_length_dim();
			params.data_ptrs.set_ptrs(l_out_op.get_data(), ffn_inp_op.get_data(), amd_detail::data_of(ffn_norm_w_op, current_block), amd_detail::data_of(ffn_gate_w_op, current_block),
				amd_detail::data_of(ffn_up_w_op, current_block), amd_detail::data_of(ffn_down_w_op, current_block));
			if (sequence_length == 0) {
				return;
			}
			auto ptrs			= params.data_ptrs;
			const float* x		= ptrs.template get_ffn_inp_data<float>();
			const float* norm_w = ptrs.template get_ffn_norm_w_data<float>();
			const void* w_gate	= ptrs.template get_ffn_gate_w_data<void>();
			const void* w_up	= ptrs.template get_ffn_up_w_data<void>();
			const void* w_down	= ptrs.template get_ffn_down_w_data<void>();
			float* y			= ptrs.template get_l_out_data<float>();
			if constexpr (processing_phase == processing_phases::eval_time) {
				auto& chain = amd_detail::decode_chain_state<config_type>::get();
				if (amd_detail::chains_decode<config_type> && chain.attn_block == current_block && chain.ffn_inp == x) {
					// attn_out + residual, this core, and what the next core starts with, as one launch
					static constexpr int64_t n_kv	   = mtt::n_embd_kv_gqa;
					static constexpr int64_t n_blocks  = mtt::block_count;
					const void* next_w[3]			   = {};
					float* next_y[3]				   = {};
					int64_t next_n[3]				   = {};
					int64_t next_count				   = 0;
					const float* next_norm			   = nullptr;
					if (current_block + 1 < n_blocks) {
						auto& qkv_core = get_adjacent_value<cfg, core_types::mega_qkv_prep_and_cache_publish>::impl(params);
						auto& q_out_op = qkv_core.values.template get_core<mega_qkv_prep_and_cache_publish_types, mega_qkv_prep_and_cache_publish_types::q_out>();
						next_w[0]	   = amd_detail::data_of(weights_core.values.template get_core<weight_types, weight_types::attn_q>(), current_block + 1);
						next_w[1]	   = amd_detail::data_of(weights_core.values.template get_core<weight_types, weight_types::attn_k>(), current_block + 1);
						next_w[2]	   = amd_detail::data_of(weights_core.values.template get_core<weight_types, weight_types::attn_v>(), current_block + 1);
						next_y[0]	   = q_out_op.template get_data<float>();
						next_y[1]	   = static_cast<float*>(amd_detail::workspace<config_type>(amd_detail::slot_k, n_kv * 4));
						next_y[2]	   = static_cast<float*>(amd_detail::workspace<config_type>(amd_detail::slot_v, n_kv * 4));
						next_n[0]	   = n_embd;
						next_n[1] = next_n[2] = n_kv;
						next_count			  = 3;
						next_norm = static_cast<const float*>(static_cast<const void*>(amd_detail::data_of(weights_core.values.template get_core<weight_types, weight_types::attn_norm>(), current_block + 1)));
					} else {
						next_w[0]  = weights_core.values.template get_core<weight_types, weight_types::output>().get_data();
						next_y[0]  = static_cast<float*>(amd_detail::workspace<config_type>(amd_detail::slot_logits, static_cast<int64_t>(mtt::vocab_size) * 4));
						next_n[0]  = mtt::vocab_size;
						next_count = 1;
						next_norm  = static_cast<const float*>(static_cast<const void*>(weights_core.values.template get_core<weight_types, weight_types::output_norm>().get_data()));
					}
					amd_detail::check<config_type>(nh_q8_0_decode_layer_f32(chain.w_o, chain.attn, chain.layer_in, chain.ffn_inp, w_gate, w_up, w_down, norm_w, y, next_w, next_y, next_n, next_count,
													   next_norm, mtt::layer_norm_rms_epsilon, n_embd, n_ff, nullptr),
						"mega_ffn eval_time: attn_out + ffn + next projections");
					chain.attn_block = -1;
					if (current_block + 1 < n_blocks) {
						chain.qkv_done_block = current_block + 1;
					} else {
						chain.logits_done = true;
					}
				} else {
					// norm, gate / up, SiLU * up, quantize, down and the residual add (residual = the FFN's own input) as one launch
					amd_detail::check<config_type>(nh_q8_0_ffn_f32(w_gate, w_up, w_down, x, norm_w, mtt::layer_norm_rms_epsilon, x, y, n_ff, n_embd, n_embd, nullptr), "mega_ffn eval_time");
				}
			} else {
				const int64_t rows = static_cast<int64_t>(sequence_length);
				// three launches: norm + quantize; gate and up mat-mats with SiLU * up and the quantizer behind them (one launch, no fp32
				// intermediates, where the shape takes the fused kernel: then gate_up_bytes is 0); down mat-mat with the residual in its store
				void* xq					= amd_detail::workspace<config_type>(amd_detail::slot_quantized, nh_q8_0_tiled_bytes(rows, n_embd));
				void* hq					= amd_detail::workspace<config_type>(amd_detail::slot_activation, nh_q8_0_tiled_bytes(rows, n_ff));
				const int64_t gate_up_bytes = nh_q8_0_gate_up_silu_workspace_bytes(rows, n_ff, n_embd);
				void* gate_up				= amd_detail::workspace<config_type>(amd_detail::slot_gate_up, gate_up_bytes);
				amd_detail::check<config_type>(nh_q8_0_rms_norm_quantize_tiled(x, norm_w, mtt::layer_norm_rms_epsilon, xq, rows, n_embd, nullptr), "mega_ffn prompt_eval_time: norm + quantize");
				amd_detail::check<config_type>(nh_q8_0_gemm_tiled_gate_up_silu(w_gate, w_up, xq, hq, gate_up, gate_up_bytes, rows, n_ff, n_embd, nullptr),
					"mega_ffn prompt_eval_time: gate / up mat-mats + SiLU * up + quantize");
				amd_detail::check<config_type>(nh_q8_0_gemm_tiled_residual(w_down, hq, x, y, rows, n_embd, n_ff, nullptr), "mega_ffn prompt_eval_time: down mat-mat + residual");
			}
			amd_detail::after_launch<config_type>();
		}
	};

	// ---- final_norm_and_sampling ----------------------------------------------------------------------------------------

	template<typename config_type, typename core_traits_type, processing_phases processing_phase>
	struct kernel_dispatcher_impl<config_type, core_traits_type, device_types::gpu, gfx950_arch_index, core_types::final_norm_and_sampling, processing_phase> {
		static void impl(core_traits_type& params) {
			using mtt					   = typename core_traits_type::mtt;
			using cfg					   = typename core_traits_type::config_type;
			static constexpr int64_t n_embd = mtt::embedding_length;
			static constexpr int64_t vocab  = mtt::vocab_size;

			auto& result_op		   = params.values.template get_core<final_norm_and_sampling_types, final_norm_and_sampling_types::result_token_id>();
			auto& weights_core	   = get_adjacent_value<cfg, core_types::weights>::impl(params);
			auto& inputs_core	   = get_adjacent_value<cfg, core_types::global_inputs>::impl(params);
			auto& ffn_core		   = get_adjacent_value<cfg, core_types::mega_ffn>::impl(params);
			auto& l_out_op		   = ffn_core.values.template get_core<mega_ffn_types, mega_ffn_types::l_out>();
			auto& output_norm_w_op = weights_core.values.template get_core<weight_types, weight_types::output_norm>();
			auto& output_w_op	   = weights_core.values.template get_core<weight_types, weight_types::output>();
			auto input			   = [&]<global_input_types which>() -> const void* {
				return inputs_core.values.template get_core<global_input_types, which>().get_data();
			};
			params.data_ptrs.set_ptrs(result_op.get_data(), l_out_op.get_data(), output_norm_w_op.get_data(), output_w_op.get_data(),
				input.template operator()<global_input_types::temperature>(), input.template operator()<global_input_types::top_k>(),
				input.template operator()<global_input_types::top_p>(), input.template operator()<global_input_types::repetition_penalty>(),
				input.template operator()<global_input_types::presence_penalty>(), input.template operator()<global_input_types::frequency_penalty>(),
				input.template operator()<global_input_types::rep_window>(), input.template operator()<global_input_types::token_history>(),
				inputs_core.values.template get_core<global_input_types, global_input_types::rng_state>().get_data(),
				input.template operator()<global_input_types::logits_bias>(), input.template operator()<global_input_types::allowed_vocab_mask>());

			// the last token's row of l_out (last_token_view, infra/core_traits.hpp:1184): one row in either phase
			const uint64_t sequence_length = processing_phase == processing_phases::eval_time ? 1 : l_out_op.get_seq_length_dim();
			if (sequence_length == 0) {
				return;
			}
			auto ptrs			= params.data_ptrs;
			const float* x		= ptrs.template get_l_out_data<float>() + (sequence_length - 1) * n_embd;
			const float* norm_w = ptrs.template get_output_norm_w_data<float>();
			const void* w		= ptrs.template get_output_w_data<void>();
			float* logits		= static_cast<float*>(amd_detail::workspace<config_type>(amd_detail::slot_logits, vocab * 4));
			const int64_t n		= vocab;
			auto& chain = amd_detail::decode_chain_state<config_type>::get();
			if (processing_phase == processing_phases::eval_time && amd_detail::chains_decode<config_type> && chain.logits_done) {
				// the last block's launch ended in this norm + mat-vec (same operands, same output): only the hook is left
			} else {
				amd_detail::check<config_type>(nh_q8_0_gemv_tiled_multi_norm_f32(&w, &logits, &n, 1, x, norm_w, mtt::layer_norm_rms_epsilon, n_embd, nullptr), "final_norm_and_sampling: norm + logits mat-vec");
			}
			chain.logits_done = false;
			amd_sampling<config_type>::impl(params, logits, nullptr);
			// the host reads the sampled token next (infra/model.hpp, the generation loop): this core always waits
			amd_detail::check<config_type>(nh_stream_sync(nullptr), "final_norm_and_sampling: stream sync");
		}
	};

} // namespace nihilus
