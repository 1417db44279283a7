// Test-local declarations standing where the reference's own headers would be when the dispatch headers are built inside
// the reference tree (NIHILUS_AMD_WITH_REFERENCE_HEADERS).  Each is written as the cited reference file declares it (names,
// template parameter lists, enumerator order); nothing here comes from reference_mirror.hpp, which that mode must not need.
// Paths relative to the reference's include/nihilus-incl/.
#pragma once

#include <array>
#include <cstdint>
#include <type_traits>

namespace nihilus {

	// common/data_types.hpp:28-44
	static constexpr uint64_t Q_SIZE{ 32 };
	using half = int16_t;
	template<typename half_type> struct block_q8_0 {
		half_type d;
		int8_t qs[Q_SIZE];
	};

	// common/config.hpp:173-177, :214-223, :225-251, :270-331, :372-376, :440-454
	enum class data_strategy_types : uint8_t { none, global, per_block };
	enum class core_types : uint8_t { weights, global_inputs, token_embeddings, mega_qkv_prep_and_cache_publish, mega_attention_apply, mega_ffn, final_norm_and_sampling, count };
	enum class kernel_types : uint8_t { weights, get_rows, rms_norm, mul, mul_mat, reshape, transpose, permute, view, rope, softmax, silu, copy, cont, add, sub, top_k_filter, top_p_filter,
		repetition_penalty, presence_penalty, temperature_scale, frequency_penalty, vocab_mask, sample_logits, count };
	enum class weight_types : uint8_t { attn_q, attn_k, attn_v, attn_output, attn_norm, ffn_gate, ffn_up, ffn_down, ffn_norm, token_embd, rope_freqs, output_norm, output, count };
	enum class global_input_types : uint8_t { inp_tokens, inp_pos, cache_k, cache_v, kq_mask, inp_out_ids, temperature, top_k, top_p, repetition_penalty, presence_penalty,
		frequency_penalty, rep_window, token_history, rng_state, logits_bias, allowed_vocab_mask, count };
	enum class token_embeddings_types : uint8_t { get_rows, count };
	enum class mega_qkv_prep_and_cache_publish_types : uint8_t { q_out, count };
	enum class mega_attention_apply_types { ffn_inp, count };
	enum class mega_ffn_types { l_out, count };
	enum class final_norm_and_sampling_types { result_token_id, count };
	enum class device_types : uint8_t { cpu, gpu, numa };
	enum class kernel_type_profiles : uint8_t { fp16_mha, fp16_moe, bf16_mha, bf16_gqa, q4_mha, q4_gqa, q4_moe, q8_mha, q8_gqa, q8_moe, mixed_fp16_fp32, mixed_bf16_fp32, count };

	// common/kernel_traits.hpp:114-117
	enum class processing_phases {
		prompt_eval_time,
		eval_time,
	};

	// common/kernel_traits.hpp:382-383, verbatim: the live specialisation point
	template<typename config_type, typename core_traits_type, device_types devive_type, uint64_t, core_types core_type, processing_phases processing_phase>
	struct kernel_dispatcher_impl;

	// common/concepts.hpp:251
	template<typename value_type>
	concept gpu_device_config_types = std::remove_cvref_t<value_type>::device_type == device_types::gpu;

	// infra/core_traits.hpp:34-74
	template<typename config_type_new, data_strategy_types data_strategy_type, typename output_type> struct data_mixin;
	template<typename config_type_new, typename output_type_new> struct data_mixin<config_type_new, data_strategy_types::global, output_type_new> {
		using output_type = output_type_new;
		static constexpr data_strategy_types data_strategy_type{ data_strategy_types::global };
		template<typename output_type_newer = output_type> output_type_newer* get_data() {
			return static_cast<output_type_newer*>(data);
		}
		void set_data(void* data_new) {
			data = data_new;
		}

	  protected:
		void* data{};
	};
	template<typename config_type_new, typename output_type_new> struct data_mixin<config_type_new, data_strategy_types::per_block, output_type_new> {
		using output_type = output_type_new;
		static constexpr data_strategy_types data_strategy_type{ data_strategy_types::per_block };
		template<typename output_type_newer = output_type> output_type_newer* get_data(uint64_t index) {
			return static_cast<output_type_newer*>(data[index]);
		}
		void set_data(void* data_new, uint64_t index) {
			data[index] = data_new;
		}

	  protected:
		std::array<void*, config_type_new::model_traits_type::block_count> data{};
	};

	// infra/core_traits.hpp:143 and :1528-1535 (the cathedral type comes from the thread pool there)
	template<typename config_type_new, core_types core_type> struct core_traits_old;
	template<typename config_type> struct nihilus_cathedral;
	template<typename config_type_new, auto kernel_type> struct get_adjacent_value {
		using derived_type = core_traits_old<config_type_new, kernel_type>;
		static auto& impl(auto& parse_core) {
			return *static_cast<derived_type*>(static_cast<nihilus_cathedral<config_type_new>*>(&parse_core));
		}
	};

	// infra/monolithic_dispatcher.hpp:30-39, :54-66, with the GPU properties of a gfx950 build (gpu_arch_index = 5)
	template<device_types device_type> constexpr uint64_t arch_index{ device_type == device_types::gpu ? 5 : 1 };
	template<typename config_type, processing_phases processing_phase, typename core_type> struct kernel_dispatcher;
	template<gpu_device_config_types config_type, processing_phases processing_phase, typename core_type> struct kernel_dispatcher<config_type, processing_phase, core_type> {
		static void impl(core_type& params, int64_t current_block) {
			kernel_dispatcher_impl<config_type, core_type, config_type::device_type, arch_index<config_type::device_type>, core_type::core_type, processing_phase>::impl(params,
				current_block);
		}
		static void impl(core_type& params) {
			kernel_dispatcher_impl<config_type, core_type, config_type::device_type, arch_index<config_type::device_type>, core_type::core_type, processing_phase>::impl(params);
		}
	};

}
