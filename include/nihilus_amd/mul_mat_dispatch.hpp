// mul_mat_dispatch.hpp -- C++23 host side of the gfx950 Q8_0 mat-mul path.
//
// Keeps the reference's compile-time specialisation surface for this one path, so the GPU kernels sit where the
// CPU mul_mat kernel would:
//
//   reference (paths relative to include/nihilus-incl/)                    here
//   -------------------------------------------------------------------   ------------------------------------------
//   device_types, kernel_types, processing_phases, kernel_type_profiles    same names and enumerators
//     common/config.hpp:225-251, :372-376, :440-454; kernel_traits.hpp:114-117
//   block_q8_0<half>, Q_SIZE                    common/data_types.hpp:28-44 same layout, static_assert(sizeof == 34)
//   core_trait_dims<d0,d1,d2,d3[,runtime_dim]>  common/kernel_traits.hpp:121-213   get_array(), get_seq_length_dim()
//   kernel_traits_old<cfg, dims, kernel_types::mul_mat, out, in1, in2>     same shape static_asserts
//     common/kernel_traits.hpp:393-417
//   data_mixin<..., global / per_block>::get_data()  infra/core_traits.hpp:36-74    raw void* tensors, per-block arrays
//   arch_index<device_types::gpu>               infra/monolithic_dispatcher.hpp:30-39   5 (= gfx950; the reference uses 1..4 for CUDA)
//   kernel_dispatcher_impl<cfg, traits, device, arch, kernel_types::mul_mat, phase, traits, float,
//                          block_q8_0<half>, block_q8_0<half>>::impl      the per-op specialisation point, dead code in
//     cpu/avx_2.hpp:1296-1444 (placeholder bodies)                        the reference, implemented here for the GPU
//   nihilus_exception<exceptions, "msg", location>::impl(str)              throw, or log + std::exit(-1)
//     common/exception.hpp:65-107
//
// phase selects the kernel at compile time, as the reference's two specialisations per op do:
//   processing_phases::eval_time        -> fused quantize + streaming mat-vec (one token)
//   processing_phases::prompt_eval_time -> quantize (tiled) + int8-MFMA mat-mat (runtime sequence length)
//
// This header sees no HIP header: everything device-side is reached through the C ABI in q8_0_abi.h.
// Built against the reference's own headers, define NIHILUS_AMD_WITH_REFERENCE_HEADERS before including it and the
// mirrored declarations below are skipped in favour of the reference's.
#pragma once

#include "q8_0_abi.h"

#include <array>
#include <cstdint>
#include <cstdlib>
#include <iostream>
#include <source_location>
#include <stdexcept>
#include <string>
#include <string_view>

namespace nihilus {

#ifndef NIHILUS_AMD_WITH_REFERENCE_HEADERS

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
	enum class data_strategy_types : uint8_t { global, per_block };
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
	template<data_strategy_types strategy, uint64_t block_count> struct data_mixin;
	template<uint64_t block_count> struct data_mixin<data_strategy_types::global, block_count> {
		template<typename value_type = void> value_type* get_data() {
			return static_cast<value_type*>(data);
		}
		void set_data(void* data_new) {
			data = data_new;
		}

	  protected:
		void* data{};
	};
	template<uint64_t block_count> struct data_mixin<data_strategy_types::per_block, block_count> {
		template<typename value_type = void> value_type* get_data(uint64_t index) {
			return static_cast<value_type*>(data[index]);
		}
		void set_data(void* data_new, uint64_t index) {
			data[index] = data_new;
		}

	  protected:
		std::array<void*, block_count> data{};
	};

	template<typename config_type, typename dims_type, kernel_types kernel_type, typename output_type_new, typename... operand_types> struct kernel_traits_old;

	// mul_mat: out[ne0 = N, ne1 = M] = W[K, N] . act[K, M]; the three shape rules of the reference, checked at compile time.
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

	// get_rows: out[ne0 = K, ne1 = tokens] = rows of table[K, n_rows] picked by ids[tokens]; the reference's shape rules
	// (common/kernel_traits.hpp:646-665).
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

	// throw, or log and std::exit(-1), chosen by the config at compile time
	template<bool exceptions> struct nihilus_exception_impl {
		[[noreturn]] static void impl(std::string_view error_type, std::string_view detail, const std::source_location& where) {
			std::string text{ "Error: " };
			text.append(error_type).append(detail).append("\nIn File: ").append(where.file_name()).append("\nOn Line: ").append(std::to_string(where.line())).append("\n");
			std::cerr << text << std::endl;
			if constexpr (exceptions) {
				throw std::runtime_error{ text };
			} else {
				std::exit(-1);
			}
		}
	};

	template<device_types device_type> inline constexpr uint64_t arch_index{ device_type == device_types::gpu ? 5 : 0 }; // 5 = gfx950

	// The per-op specialisation point (ten template parameters in the reference's dead per-op form).
	template<typename config_type, typename core_traits_type, device_types device_type, uint64_t arch, kernel_types kernel_type, processing_phases processing_phase,
		typename... types>
	struct kernel_dispatcher_impl;

#endif // NIHILUS_AMD_WITH_REFERENCE_HEADERS

	namespace amd_detail {
		template<typename config_type> inline void check(int status, const char* what, const std::source_location where = std::source_location::current()) {
			if (status != NH_OK) {
				nihilus_exception_impl<config_type::exceptions>::impl("HIP Q8_0 mul_mat: ", std::string{ what } + ": " + nh_status_string(status), where);
			}
		}
	}

	// The weight operand of a GPU mul_mat holds the tiled copy made at load time (nh_q8_0_tile); the activation operand
	// holds fp32 values (the output of the rms_norm/mul or silu/mul step in front of it); the workspace operand is the
	// arena slice for the quantized activations of the prompt phase.
	//
	// eval_time: one token.  y[N] = W . quantize(x), quantize fused into the mat-vec kernel.
	template<typename config_type, typename core_traits_type>
	struct kernel_dispatcher_impl<config_type, core_traits_type, device_types::gpu, 5, kernel_types::mul_mat, processing_phases::eval_time, core_traits_type, float,
		block_q8_0<half>, block_q8_0<half>> {
		using input_type01			   = typename core_traits_type::input_01_type;
		using input_type02			   = typename core_traits_type::input_02_type;
		static constexpr uint64_t ne00 = input_type01::get_array()[0]; // K
		static constexpr uint64_t ne01 = input_type01::get_array()[1]; // N
		static_assert(ne00 % 128 == 0, "the tiled weight layout needs K to be a multiple of 128");

		// The same with the rms_norm and mul nodes that precede the projection folded in: activation is the un-normalised
		// row, norm_weight the fp32 [K] norm weight, eps the model's layer_norm_rms_epsilon (infra/core_traits.hpp:570-576).
		static void impl(core_traits_type& output, const void* weight_tiled, const float* activation, const float* norm_weight, float eps, void* stream = nullptr) {
			float* y		= output.template get_data<float>();
			const int64_t n = ne01;
			amd_detail::check<config_type>(nh_q8_0_gemv_tiled_multi_norm_f32(&weight_tiled, &y, &n, 1, activation, norm_weight, eps, ne00, stream), "eval_time norm + mat-vec");
			if constexpr (config_type::synchronous) {
				amd_detail::check<config_type>(nh_stream_sync(stream), "stream sync");
			}
		}

		// The same with the add node that follows the projection folded in (attn_out mul_mat -> residual add,
		// infra/core_traits.hpp:768-772): output = W . quantize(activation) + residual; residual may be the output buffer.
		static void impl_add(core_traits_type& output, const void* weight_tiled, const float* activation, const float* residual, void* stream = nullptr) {
			amd_detail::check<config_type>(nh_q8_0_gemv_tiled_residual_f32(weight_tiled, activation, residual, output.template get_data<float>(), ne01, ne00, stream),
				"eval_time mat-vec + residual");
			if constexpr (config_type::synchronous) {
				amd_detail::check<config_type>(nh_stream_sync(stream), "stream sync");
			}
		}

		// weight: device pointer to the tiled matrix; activation: fp32 [K]; output: fp32 [N]; stream may be null
		static void impl(core_traits_type& output, const void* weight_tiled, const float* activation, void* stream = nullptr) {
			amd_detail::check<config_type>(nh_q8_0_gemv_tiled_f32(weight_tiled, activation, output.template get_data<float>(), ne01, ne00, stream), "eval_time mat-vec");
			if constexpr (config_type::synchronous) {
				amd_detail::check<config_type>(nh_stream_sync(stream), "stream sync"); // the reference syncs after every launch (cuda/cuda_12.hpp:679)
			}
		}
	};

	// prompt_eval_time: M = runtime sequence length.  C[M][N] = quantize(A) . W^T on the int8 MFMA path.
	template<typename config_type, typename core_traits_type>
	struct kernel_dispatcher_impl<config_type, core_traits_type, device_types::gpu, 5, kernel_types::mul_mat, processing_phases::prompt_eval_time, core_traits_type, float,
		block_q8_0<half>, block_q8_0<half>> {
		using input_type01			   = typename core_traits_type::input_01_type;
		using input_type02			   = typename core_traits_type::input_02_type;
		static constexpr uint64_t ne00 = input_type01::get_array()[0]; // K
		static constexpr uint64_t ne01 = input_type01::get_array()[1]; // N
		static_assert(ne00 % 128 == 0, "the tiled weight layout needs K to be a multiple of 128");

		static int64_t workspace_bytes(uint64_t sequence_length) {
			return nh_q8_0_mul_mat_workspace_bytes(static_cast<int64_t>(sequence_length), ne00);
		}

		static void impl(core_traits_type& output, const void* weight_tiled, const float* activation, void* workspace, int64_t workspace_size, void* stream = nullptr) {
			const uint64_t sequence_length = output.get_seq_length_dim(); // the one runtime dim (ne1 of the output)
			if (sequence_length == 0) {
				return; // the reference launches nothing for an empty sequence (cuda/cuda_12.hpp:657)
			}
			amd_detail::check<config_type>(nh_q8_0_mul_mat(weight_tiled, activation, output.template get_data<float>(), static_cast<int64_t>(sequence_length), ne01, ne00,
											   workspace, workspace_size, stream),
				"prompt_eval_time mat-mat");
			if constexpr (config_type::synchronous) {
				amd_detail::check<config_type>(nh_stream_sync(stream), "stream sync");
			}
		}
			// The same with the add node behind the projection folded in (infra/core_traits.hpp:768-772, :988-992): output = mul_mat + residual,
		// residual fp32 [sequence_length][N], may be the output buffer.
		static void impl_add(core_traits_type& output, const void* weight_tiled, const float* activation, const float* residual, void* workspace, int64_t workspace_size,
			void* stream = nullptr) {
			const uint64_t sequence_length = output.get_seq_length_dim();
			if (sequence_length == 0) {
				return;
			}
			amd_detail::check<config_type>(nh_q8_0_mul_mat_residual(weight_tiled, activation, residual, output.template get_data<float>(), static_cast<int64_t>(sequence_length), ne01,
											   ne00, workspace, workspace_size, stream),
				"prompt_eval_time mat-mat + residual");
			if constexpr (config_type::synchronous) {
				amd_detail::check<config_type>(nh_stream_sync(stream), "stream sync");
			}
		}
	};

	// The key the reference implements on the CPU, <float, block_q8_0<half>, float> (cpu/avx_2.hpp:4854-5004): fp32 activations
	// against Q8_0 weights WITHOUT quantizing the activations, both phases (eval_time: one row; prompt_eval_time: the output's
	// runtime sequence length).  Not the path a model runs; a plain form that reads the weights once per activation row.
	template<typename config_type, typename core_traits_type, processing_phases processing_phase>
	struct kernel_dispatcher_impl<config_type, core_traits_type, device_types::gpu, 5, kernel_types::mul_mat, processing_phase, core_traits_type, float, block_q8_0<half>, float> {
		using input_type01			   = typename core_traits_type::input_01_type;
		static constexpr uint64_t ne00 = input_type01::get_array()[0]; // K
		static constexpr uint64_t ne01 = input_type01::get_array()[1]; // N
		static_assert(ne00 % 128 == 0, "the tiled weight layout needs K to be a multiple of 128");

		static void impl(core_traits_type& output, const void* weight_tiled, const float* activation, void* stream = nullptr) {
			const uint64_t rows = processing_phase == processing_phases::eval_time ? 1 : output.get_seq_length_dim();
			if (rows == 0) {
				return;
			}
			amd_detail::check<config_type>(nh_q8_0_mul_mat_f32_activations(weight_tiled, activation, output.template get_data<float>(), static_cast<int64_t>(rows), ne01, ne00, stream),
				"mul_mat with fp32 activations");
			if constexpr (config_type::synchronous) {
				amd_detail::check<config_type>(nh_stream_sync(stream), "stream sync");
			}
		}
	};

	// get_rows (token embeddings), both phases: out[t][:] = dequantized row ids[t] of the embedding table.  The table
	// operand holds the device copy of token_embd.weight, tiled (table_is_tiled) or as the packed blocks of the file.
	// eval_time looks up one token, prompt_eval_time the output's runtime sequence length; both index by the id (the
	// reference's CUDA eval-time kernel, cuda/cuda_12.hpp:691-722, dequantizes row 0 whatever the id).
	template<typename config_type, typename core_traits_type, processing_phases processing_phase>
	struct kernel_dispatcher_impl<config_type, core_traits_type, device_types::gpu, 5, kernel_types::get_rows, processing_phase, core_traits_type, float, block_q8_0<half>,
		int32_t> {
		using input_type01			   = typename core_traits_type::input_01_type;
		static constexpr uint64_t ne00 = input_type01::get_array()[0]; // embedding length
		static constexpr uint64_t ne01 = input_type01::get_array()[1]; // vocabulary size

		static void impl(core_traits_type& output, const void* table, bool table_is_tiled, const int32_t* token_ids, void* stream = nullptr) {
			uint64_t tokens = 1;
			if constexpr (processing_phase == processing_phases::prompt_eval_time) {
				tokens = output.get_seq_length_dim();
				if (tokens == 0) {
					return;
				}
			}
			const auto fn = table_is_tiled ? nh_q8_0_get_rows_tiled : nh_q8_0_get_rows;
			amd_detail::check<config_type>(fn(table, token_ids, output.template get_data<float>(), nullptr, static_cast<int64_t>(tokens), ne01, ne00, stream), "get_rows");
			if constexpr (config_type::synchronous) {
				amd_detail::check<config_type>(nh_stream_sync(stream), "stream sync");
			}
		}
	};

	// Caller-side helper: picks the specialisation from the config, as kernel_dispatcher does for the mega kernels
	// (infra/monolithic_dispatcher.hpp:41-63).
	template<typename config_type, processing_phases processing_phase, typename mul_mat_traits_type> struct mul_mat_dispatcher {
		using impl_type = kernel_dispatcher_impl<config_type, mul_mat_traits_type, config_type::device_type, arch_index<config_type::device_type>, kernel_types::mul_mat,
			processing_phase, mul_mat_traits_type, float, block_q8_0<half>, block_q8_0<half>>;
		template<typename... arg_types> static void impl(arg_types&&... args) {
			impl_type::impl(std::forward<arg_types>(args)...);
		}
		// the projection with the add node behind it folded in
		template<typename... arg_types> static void impl_add(arg_types&&... args) {
			impl_type::impl_add(std::forward<arg_types>(args)...);
		}
	};

	template<typename config_type, processing_phases processing_phase, typename get_rows_traits_type> struct get_rows_dispatcher {
		using impl_type = kernel_dispatcher_impl<config_type, get_rows_traits_type, config_type::device_type, arch_index<config_type::device_type>, kernel_types::get_rows,
			processing_phase, get_rows_traits_type, float, block_q8_0<half>, int32_t>;
		template<typename... arg_types> static void impl(arg_types&&... args) {
			impl_type::impl(std::forward<arg_types>(args)...);
		}
	};

} // namespace nihilus
