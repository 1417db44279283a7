// A small model graph in the shape the reference's dispatchers expect, for the tests of mega_dispatch.hpp: seven cores
// (weights, global_inputs, token_embeddings, the three mega cores, final_norm_and_sampling), each with `values`
// (get_core<enum_type, enum_value>()), the mega cores with `data_ptrs` packs whose set_ptrs argument order and getter names
// are those of the reference (infra/core_traits.hpp:408-504, :782-833, :1003-1048, :1234-1335), all reachable from one
// another through get_adjacent_value.  Test infrastructure; uses only names that either the reference's headers or
// reference_mirror.hpp declare, so the same file serves both build modes.
#pragma once

#include <cstdint>
#include <tuple>

namespace nihilus {

	// LLaMA-shaped, small enough for the CPU checker to follow in a blink; every length a multiple of 128
	struct tiny_llama_traits {
		static constexpr float layer_norm_rms_epsilon{ 1e-5f };
		static constexpr uint32_t vocab_size{ 4096 };
		static constexpr uint32_t embedding_length{ 1024 };
		static constexpr uint32_t block_count{ 2 };
		static constexpr uint32_t feed_forward_length{ 3584 };
		static constexpr uint32_t attention_head_count{ 8 };
		static constexpr uint32_t attention_head_count_kv{ 2 };
		static constexpr uint32_t rope_dimension_count{ embedding_length / attention_head_count };
		static constexpr uint64_t n_embd_kv_gqa{ rope_dimension_count * attention_head_count_kv };
	};

	// the shapes of the decode benchmark configuration (LLaMA-3-8B)
	struct llama3_8b_traits {
		static constexpr float layer_norm_rms_epsilon{ 1e-5f };
		static constexpr uint32_t vocab_size{ 128256 };
		static constexpr uint32_t embedding_length{ 4096 };
		static constexpr uint32_t block_count{ 32 };
		static constexpr uint32_t feed_forward_length{ 14336 };
		static constexpr uint32_t attention_head_count{ 32 };
		static constexpr uint32_t attention_head_count_kv{ 8 };
		static constexpr uint32_t rope_dimension_count{ embedding_length / attention_head_count };
		static constexpr uint64_t n_embd_kv_gqa{ rope_dimension_count * attention_head_count_kv };
	};

#ifndef NH_MOCK_MODEL_TRAITS
	#define NH_MOCK_MODEL_TRAITS tiny_llama_traits // a translation unit that wants the other set defines this before the include
#endif

	struct mock_config {
		static constexpr device_types device_type{ device_types::gpu };
		static constexpr kernel_type_profiles kernel_type_profile{ kernel_type_profiles::q8_gqa };
		static constexpr bool exceptions{ true };
		static constexpr bool dev{ false };
		static constexpr uint64_t max_sequence_length{ 64 };
		static constexpr bool amd_matmul_only{ true }; // the mat-mul path alone: the header's stand-in customisation points may be used
		using model_traits_type = NH_MOCK_MODEL_TRAITS;
	};

	// one graph node: raw storage (global or per block) + the runtime sequence length + its enumerator
	template<auto enum_value_new, data_strategy_types strategy> struct mock_op : data_mixin<mock_config, strategy, void> {
		static constexpr auto enum_value{ enum_value_new };
		mutable uint64_t sequence_length{ 1 };
		uint64_t& get_seq_length_dim() const {
			return sequence_length;
		}
	};

	template<typename... op_types> struct mock_ops {
		std::tuple<op_types...> ops{};
		template<typename enum_type, enum_type which> auto& get_core() {
			return pick<enum_type, which, 0>();
		}

	  private:
		template<typename enum_type, enum_type which, size_t index> auto& pick() {
			static_assert(index < sizeof...(op_types), "no such node in this core");
			using op_type = std::tuple_element_t<index, std::tuple<op_types...>>;
			if constexpr (op_type::enum_value == which) {
				return std::get<index>(ops);
			} else {
				return pick<enum_type, which, index + 1>();
			}
		}
	};

	template<weight_types w> using block_weight	 = mock_op<w, data_strategy_types::per_block>;
	template<weight_types w> using global_weight = mock_op<w, data_strategy_types::global>;
	template<global_input_types g> using input_op = mock_op<g, data_strategy_types::global>;

	template<> struct core_traits_old<mock_config, core_types::weights> {
		static constexpr core_types core_type{ core_types::weights };
		using config_type = mock_config;
		mock_ops<block_weight<weight_types::attn_q>, block_weight<weight_types::attn_k>, block_weight<weight_types::attn_v>, block_weight<weight_types::attn_output>,
			block_weight<weight_types::attn_norm>, block_weight<weight_types::ffn_gate>, block_weight<weight_types::ffn_up>, block_weight<weight_types::ffn_down>,
			block_weight<weight_types::ffn_norm>, global_weight<weight_types::token_embd>, global_weight<weight_types::rope_freqs>, global_weight<weight_types::output_norm>,
			global_weight<weight_types::output>>
			values{};
	};

	template<> struct core_traits_old<mock_config, core_types::global_inputs> {
		static constexpr core_types core_type{ core_types::global_inputs };
		using config_type = mock_config;
		mock_ops<input_op<global_input_types::inp_tokens>, input_op<global_input_types::inp_pos>, input_op<global_input_types::cache_k>, input_op<global_input_types::cache_v>,
			input_op<global_input_types::kq_mask>, input_op<global_input_types::inp_out_ids>, input_op<global_input_types::temperature>, input_op<global_input_types::top_k>,
			input_op<global_input_types::top_p>, input_op<global_input_types::repetition_penalty>, input_op<global_input_types::presence_penalty>,
			input_op<global_input_types::frequency_penalty>, input_op<global_input_types::rep_window>, input_op<global_input_types::token_history>,
			input_op<global_input_types::rng_state>, input_op<global_input_types::logits_bias>, input_op<global_input_types::allowed_vocab_mask>>
			values{};
	};

	template<> struct core_traits_old<mock_config, core_types::token_embeddings> {
		static constexpr core_types core_type{ core_types::token_embeddings };
		using config_type = mock_config;
		mock_ops<mock_op<token_embeddings_types::get_rows, data_strategy_types::global>> values{};
	};

#define NH_MOCK_GETTER(name, constness)                                               \
	template<typename value_type> constness value_type* get_##name() {                \
		return static_cast<constness value_type*>(name);                              \
	}

	template<> struct core_traits_old<mock_config, core_types::mega_qkv_prep_and_cache_publish> {
		static constexpr core_types core_type{ core_types::mega_qkv_prep_and_cache_publish };
		using config_type = mock_config;
		using mtt		  = NH_MOCK_MODEL_TRAITS;
		mock_ops<mock_op<mega_qkv_prep_and_cache_publish_types::q_out, data_strategy_types::global>> values{};
		struct kernel_data_ptrs_type {
			NH_MOCK_GETTER(inp_embd_data, const)
			NH_MOCK_GETTER(attn_norm_w_data, const)
			NH_MOCK_GETTER(attn_q_w_data, const)
			NH_MOCK_GETTER(attn_k_w_data, const)
			NH_MOCK_GETTER(attn_v_w_data, const)
			NH_MOCK_GETTER(inp_pos_data, const)
			NH_MOCK_GETTER(rope_freqs_data, const)
			NH_MOCK_GETTER(cache_k_data, )
			NH_MOCK_GETTER(cache_v_data, )
			NH_MOCK_GETTER(q_output_data, )
			void set_ptrs(void* q_output_data_new, const void* inp_embd_data_new, const void* attn_norm_w_data_new, const void* attn_q_w_data_new, const void* attn_k_w_data_new,
				const void* attn_v_w_data_new, const void* inp_pos_data_new, const void* rope_freqs_data_new, void* cache_k_data_new, void* cache_v_data_new) {
				q_output_data	 = q_output_data_new;
				inp_embd_data	 = inp_embd_data_new;
				attn_norm_w_data = attn_norm_w_data_new;
				attn_q_w_data	 = attn_q_w_data_new;
				attn_k_w_data	 = attn_k_w_data_new;
				attn_v_w_data	 = attn_v_w_data_new;
				inp_pos_data	 = inp_pos_data_new;
				rope_freqs_data	 = rope_freqs_data_new;
				cache_k_data	 = cache_k_data_new;
				cache_v_data	 = cache_v_data_new;
			}

		  protected:
			const void *inp_embd_data{}, *attn_norm_w_data{}, *attn_q_w_data{}, *attn_k_w_data{}, *attn_v_w_data{}, *inp_pos_data{}, *rope_freqs_data{};
			void *cache_k_data{}, *cache_v_data{}, *q_output_data{};
		};
		kernel_data_ptrs_type data_ptrs{};
	};

	template<> struct core_traits_old<mock_config, core_types::mega_attention_apply> {
		static constexpr core_types core_type{ core_types::mega_attention_apply };
		using config_type = mock_config;
		using mtt		  = NH_MOCK_MODEL_TRAITS;
		mock_ops<mock_op<mega_attention_apply_types::ffn_inp, data_strategy_types::global>> values{};
		struct kernel_data_ptrs {
			NH_MOCK_GETTER(q_input_data, const)
			NH_MOCK_GETTER(cache_k_data, const)
			NH_MOCK_GETTER(cache_v_data, const)
			NH_MOCK_GETTER(kq_mask_data, const)
			NH_MOCK_GETTER(attn_output_w_data, const)
			NH_MOCK_GETTER(inp_embd_data, const)
			NH_MOCK_GETTER(ffn_inp_data, )
			void set_ptrs(void* ffn_inp_data_new, const void* q_input_data_new, const void* cache_k_data_new, const void* cache_v_data_new, const void* kq_mask_data_new,
				const void* attn_output_w_data_new, const void* inp_embd_data_new) {
				ffn_inp_data	   = ffn_inp_data_new;
				q_input_data	   = q_input_data_new;
				cache_k_data	   = cache_k_data_new;
				cache_v_data	   = cache_v_data_new;
				kq_mask_data	   = kq_mask_data_new;
				attn_output_w_data = attn_output_w_data_new;
				inp_embd_data	   = inp_embd_data_new;
			}

		  protected:
			const void *q_input_data{}, *cache_k_data{}, *cache_v_data{}, *kq_mask_data{}, *attn_output_w_data{}, *inp_embd_data{};
			void* ffn_inp_data{};
		};
		kernel_data_ptrs data_ptrs{};
	};

	template<> struct core_traits_old<mock_config, core_types::mega_ffn> {
		static constexpr core_types core_type{ core_types::mega_ffn };
		using config_type = mock_config;
		using mtt		  = NH_MOCK_MODEL_TRAITS;
		mock_ops<mock_op<mega_ffn_types::l_out, data_strategy_types::global>> values{};
		struct kernel_data_ptrs {
			NH_MOCK_GETTER(ffn_inp_data, const)
			NH_MOCK_GETTER(ffn_norm_w_data, const)
			NH_MOCK_GETTER(ffn_gate_w_data, const)
			NH_MOCK_GETTER(ffn_up_w_data, const)
			NH_MOCK_GETTER(ffn_down_w_data, const)
			NH_MOCK_GETTER(l_out_data, )
			void set_ptrs(void* l_out_data_new, const void* ffn_inp_data_new, const void* ffn_norm_w_data_new, const void* ffn_gate_w_data_new, const void* ffn_up_w_data_new,
				const void* ffn_down_w_data_new) {
				l_out_data		= l_out_data_new;
				ffn_inp_data	= ffn_inp_data_new;
				ffn_norm_w_data = ffn_norm_w_data_new;
				ffn_gate_w_data = ffn_gate_w_data_new;
				ffn_up_w_data	= ffn_up_w_data_new;
				ffn_down_w_data = ffn_down_w_data_new;
			}

		  protected:
			const void *ffn_inp_data{}, *ffn_norm_w_data{}, *ffn_gate_w_data{}, *ffn_up_w_data{}, *ffn_down_w_data{};
			void* l_out_data{};
		};
		kernel_data_ptrs data_ptrs{};
	};

	template<> struct core_traits_old<mock_config, core_types::final_norm_and_sampling> {
		static constexpr core_types core_type{ core_types::final_norm_and_sampling };
		using config_type = mock_config;
		using mtt		  = NH_MOCK_MODEL_TRAITS;
		mock_ops<mock_op<final_norm_and_sampling_types::result_token_id, data_strategy_types::global>> values{};
		struct kernel_data_ptrs {
			NH_MOCK_GETTER(l_out_data, const)
			NH_MOCK_GETTER(output_norm_w_data, const)
			NH_MOCK_GETTER(output_w_data, const)
			NH_MOCK_GETTER(result_token_id_data, )
			void set_ptrs(void* result_token_id_data_new, const void* l_out_data_new, const void* output_norm_w_data_new, const void* output_w_data_new, const void*, const void*,
				const void*, const void*, const void*, const void*, const void*, const void*, void*, const void*, const void*) {
				result_token_id_data = result_token_id_data_new;
				l_out_data			 = l_out_data_new;
				output_norm_w_data	 = output_norm_w_data_new;
				output_w_data		 = output_w_data_new;
			}

		  protected:
			const void *l_out_data{}, *output_norm_w_data{}, *output_w_data{};
			void* result_token_id_data{};
		};
		kernel_data_ptrs data_ptrs{};
	};
#undef NH_MOCK_GETTER

	// the one object that is all cores at once (the reference's nihilus_cathedral, infra/nihilus_cathedral.hpp)
	template<> struct nihilus_cathedral<mock_config>
		: core_traits_old<mock_config, core_types::weights>,
		  core_traits_old<mock_config, core_types::global_inputs>,
		  core_traits_old<mock_config, core_types::token_embeddings>,
		  core_traits_old<mock_config, core_types::mega_qkv_prep_and_cache_publish>,
		  core_traits_old<mock_config, core_types::mega_attention_apply>,
		  core_traits_old<mock_config, core_types::mega_ffn>,
		  core_traits_old<mock_config, core_types::final_norm_and_sampling> {};

} // namespace nihilus
