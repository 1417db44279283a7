// reference_mirror.hpp -- stand-alone declarations of the reference names that the gfx950 dispatch headers specialise
// or use, for builds WITHOUT the reference's own headers (this repository's tests and benchmark).
//
// Inside the reference tree this file is not included: define NIHILUS_AMD_WITH_REFERENCE_HEADERS, include the
// reference's headers first, and mega_dispatch.hpp / mul_mat_dispatch.hpp then attach to the reference's own
// declarations.  Everything here has the reference's name, template parameter list and enumerator order, so that code
// written against one compiles against the other (paths relative to include/nihilus-incl/):
//
//   device_types, core_types, kernel_types, kernel_type_profiles, data_strategy_types, weight_types, global_input_types,
//   token_embeddings_types, mega_*_types, final_norm_and_sampling_types      common/config.hpp:173-177, :214-251, :270-331, :372-376, :440-454
//   processing_phases                                                         common/kernel_traits.hpp:114-117
//   block_q8_0<half>, Q_SIZE                                                  common/data_types.hpp:28-44
//   core_trait_dims<d0, d1, d2, d3[, runtime_dim]>                            common/kernel_traits.hpp:121-213
//   kernel_traits_old<cfg, dims, kernel_types::{mul_mat, get_rows}, ...>      common/kernel_traits.hpp:393-417, :646-665
//   kernel_dispatcher_impl<cfg, core_traits, device, arch, core_types, phase> common/kernel_traits.hpp:382-383 (the live specialisation point)
//   kernel_dispatcher<cfg, phase, core_type> (GPU form)                       infra/monolithic_dispatcher.hpp:54-66
//   data_mixin<cfg, strategy, output_type>                                    infra/core_traits.hpp:34-74
//   core_traits_old<cfg, core_types>, get_adjacent_value<cfg, core_type>      infra/core_traits.hpp:143, :1528-1535
//
// What differs, by necessity: get_adjacent_value reaches a neighbouring core through nihilus_cathedral<config>, which a
// stand-alone user defines as the one object that derives from all its core_traits_old<config, ...> (the reference takes
// that type from its thread pool); model_traits_type<config> is whatever the user's config names as model_traits_type.
#pragma once

#include <array>
#include <cstdint>

namespace nihilus {

	inline constexpr uint64_t Q_SIZE{ 32 };
	using half = int16_t; // fp16 bit pattern, as the reference stores it

	template<typename half_type> struct block_q8_0 {
		using scale_type = half_type;
		using quant_type = int8_t;
		half_type d;
		int8_t qs[Q_SIZE];
	};
	static_assert(sizeof(block_q8_0<half>) == sizeof(half) + Q_SIZE, "Wrong q8_0 block size/padding.");

	enum class device_types : uint8_t { cpu, gpu, numa };
	enum class processing_phases { prompt_eval_time, eval_time };
	enum class kernel_type_profiles : uint8_t { fp16_mha, fp16_moe, bf16_mha, bf16_gqa, q4_mha, q4_gqa, q4_moe, q8_mha, q8_gqa, q8_moe, mixed_fp16_fp32, mixed_bf16_fp32, count };
	enum class data_strategy_types : uint8_t { none, global, per_block };
	enum class core_types : uint8_t { weights, global_inputs, token_embeddings, mega_qkv_prep_and_cache_publish, mega_attention_apply, mega_ffn, final_norm_and_sampling, count };
	enum class kernel_types : uint8_t {
		weights,
		get_rows,
		rms_norm,
		mul,
		mul_mat,
		reshape,
		transpose,
		permute,
		view,
		rope,
		softmax,
		silu,
		copy,
		cont,
		add,
		sub,
		top_k_filter,
		top_p_filter,
		repetition_penalty,
		presence_penalty,
		temperature_scale,
		frequency_penalty,
		vocab_mask,
		sample_logits,
		count,
	};
	enum class weight_types : uint8_t { attn_q, attn_k, attn_v, attn_output, attn_norm, ffn_gate, ffn_up, ffn_down, ffn_norm, token_embd, rope_freqs, output_norm, output, count };
	enum class global_input_types : uint8_t {
		inp_tokens,
		inp_pos,
		cache_k,
		cache_v,
		kq_mask,
		inp_out_ids,
		temperature,
		top_k,
		top_p,
		repetition_penalty,
		presence_penalty,
		frequency_penalty,
		rep_window,
		token_history,
		rng_state,
		logits_bias,
		allowed_vocab_mask,
		count,
	};
	enum class token_embeddings_types : uint8_t { get_rows, count };
	enum class mega_qkv_prep_and_cache_publish_types : uint8_t { q_out, count };
	enum class mega_attention_apply_types { ffn_inp, count };
	enum class mega_ffn_types { l_out, count };
	enum class final_norm_and_sampling_types { result_token_id, count };

	template<typename value_type>
	concept gpu_device_config_types = std::remove_cvref_t<value_type>::device_type == device_types::gpu;

	// Compile-time dims in ggml order (dim0 fastest); the optional fifth argument names the one runtime dim (5 = none).
	template<uint64_t... indices> struct core_trait_dims;

	template<uint64_t d0, uint64_t d1, uint64_t d2, uint64_t d3> struct core_trait_dims<d0, d1, d2, d3> {
		static constexpr uint64_t runtime_dim{ 5 };
		static constexpr std::array<uint64_t, 4> get_array() {
			return { d0, d1, d2, d3 };
		}
	};
	template<uint64_t d0, uint64_t d1, uint64_t d2, uint64_t d3> struct core_trait_dims<d0, d1, d2, d3, 1> {
		static constexpr uint64_t runtime_dim{ 1 };
		mutable uint64_t dim01{ d1 };
		static constexpr std::array<uint64_t, 4> get_array() {
			return { d0, d1, d2, d3 };
		}
		std::array<uint64_t, 4> get_array_rt() const {
			return { d0, dim01, d2, d3 };
		}
		uint64_t& get_seq_length_dim() const {
			return dim01;
		}
	};

	template<typename value_type>
	concept runtime_dims_t = requires(const value_type& v) { v.get_seq_length_dim(); };

	// Raw tensor storage of a graph node: one pointer, or one per transformer block for layer weights.
	template<typename config_type_new, data_strategy_types data_strategy_type, typename output_type> struct data_mixin;
	template<typename config_type_new, typename output_type_new> struct data_mixin<config_type_new, data_strategy_types::global, output_type_new> {
		using output_type = output_type_new;
		static constexpr data_strategy_types data_strategy_type{ data_strategy_types::global };
		template<typename value_type = output_type> value_type* get_data() {
			return static_cast<value_type*>(data);
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
		template<typename value_type = output_type> value_type* get_data(uint64_t index) {
			return static_cast<value_type*>(data[index]);
		}
		void set_data(void* data_new, uint64_t index) {
			data[index] = data_new;
		}

	  protected:
		std::array<void*, config_type_new::model_traits_type::block_count> data{};
	};

	template<typename config_type, typename dims_type, kernel_types kernel_type, typename output_type_new, typename... operand_types> struct kernel_traits_old;

	// mul_mat: out[ne0 = N, ne1 = M] = W[K, N] . act[K, M]; the shape rules of the reference, checked at compile time.
	template<typename config_type, typename dims_type_new, typename output_type_new, typename input_01_type_new, typename input_02_type_new>
	struct kernel_traits_old<config_type, dims_type_new, kernel_types::mul_mat, output_type_new, input_01_type_new, input_02_type_new> : public dims_type_new {
		using input_01_type					= input_01_type_new;
		using input_02_type					= input_02_type_new;
		using output_type					= output_type_new;
		using dims_type						= dims_type_new;
		static constexpr auto input_01_dims = input_01_type::get_array();
		static constexpr auto input_02_dims = input_02_type::get_array();
		static constexpr auto output_dims	= dims_type::get_array();
		static_assert(input_01_dims[0] == input_02_dims[0], "mul_mat: inner dimensions must match");
		static_assert(output_dims[0] == input_01_dims[1], "mul_mat: output rows must equal the first input's columns");
		static_assert(output_dims[1] == input_02_dims[1], "mul_mat: output columns must equal the second input's columns");
		static_assert(output_dims[2] == input_01_dims[2] || output_dims[2] == input_02_dims[2], "mul_mat: batch dim 2 must match an input");
		static_assert(output_dims[3] == input_01_dims[3] || output_dims[3] == input_02_dims[3], "mul_mat: batch dim 3 must match an input");
	};

	// get_rows: out[ne0 = K, ne1 = tokens] = rows of table[K, n_rows] picked by ids[tokens].
	template<typename config_type, typename dims_type_new, typename output_type_new, typename input_01_type_new, typename input_02_type_new>
	struct kernel_traits_old<config_type, dims_type_new, kernel_types::get_rows, output_type_new, input_01_type_new, input_02_type_new> : public dims_type_new {
		using input_01_type					= input_01_type_new;
		using input_02_type					= input_02_type_new;
		using output_type					= output_type_new;
		using dims_type						= dims_type_new;
		static constexpr auto input_01_dims = input_01_type::get_array();
		static constexpr auto input_02_dims = input_02_type::get_array();
		static constexpr auto output_dims	= dims_type::get_array();
		static_assert(input_02_dims[0] == output_dims[1], "get_rows: one index per output row");
		static_assert(input_02_dims[1] == 1 && input_02_dims[2] == 1 && input_02_dims[3] == 1, "get_rows: indices are one-dimensional");
		static_assert(output_dims[0] == input_01_dims[0], "get_rows: output row length must equal the embedding length");
		static_assert(output_dims[2] == 1 && output_dims[3] == 1, "get_rows: output is two-dimensional");
	};

	// The live specialisation point, declared exactly as common/kernel_traits.hpp:382-383 declares it.
	template<typename config_type, typename core_traits_type, device_types devive_type, uint64_t, core_types core_type, processing_phases processing_phase>
	struct kernel_dispatcher_impl;

	// One core of the model graph and the object that derives from all of them; a stand-alone user specialises both.
	template<typename config_type, core_types core_type> struct core_traits_old;
	template<typename config_type> struct nihilus_cathedral;

	template<typename config_type_new, auto kernel_type> struct get_adjacent_value {
		using derived_type = core_traits_old<config_type_new, kernel_type>;
		static auto& impl(auto& parse_core) {
			return *static_cast<derived_type*>(static_cast<nihilus_cathedral<config_type_new>*>(&parse_core));
		}
	};

	// 5 = gfx950; the reference's generated GPU properties header holds 1..4 for its CUDA targets (cuda/nihilus_gpu_properties.hpp:28-40).
	template<device_types device_type> inline constexpr uint64_t arch_index{ device_type == device_types::gpu ? 5 : 0 };

	// The caller's side of the live point for a GPU config: same two overloads as infra/monolithic_dispatcher.hpp:54-66.
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

} // namespace nihilus
