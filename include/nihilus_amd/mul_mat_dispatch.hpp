// mul_mat_dispatch.hpp -- C++23 host side of the gfx950 Q8_0 mat-mul path, per-op form.
//
// The reference selects kernels at compile time by specialising a class template.  Two such keys exist in its source
// (paths relative to include/nihilus-incl/):
//
//   * the LIVE one, keyed by core_types (one "mega" core of the model graph per specialisation):
//       kernel_dispatcher_impl<config, core_traits, device, arch, core_types, phase>::impl(params[, current_block])
//     common/kernel_traits.hpp:382-383, called from infra/monolithic_dispatcher.hpp:41-63.  The gfx950 specialisations
//     of that key are in mega_dispatch.hpp;
//   * an older per-op one, keyed by kernel_types plus the operand element types, which survives only inside a block
//     comment (cpu/avx_2.hpp:1296-1444, placeholder bodies for mul_mat).  It had the same template name with a different
//     parameter list, so the two cannot be declared in one translation unit; this header keeps the per-op key under the
//     name per_op_kernel_dispatcher_impl, with the old parameter list unchanged:
//       per_op_kernel_dispatcher_impl<config, core_traits, device, arch, kernel_types::mul_mat, phase, core_traits, float,
//                                     block_q8_0<half>, block_q8_0<half>>::impl
//
// phase selects the kernel at compile time, as the reference's two specialisations per op do:
//   processing_phases::eval_time        -> fused quantize + streaming mat-vec (one token)
//   processing_phases::prompt_eval_time -> quantize (tiled) + int8-MFMA mat-mat (runtime sequence length)
//
// This header sees no HIP header: everything device-side is reached through the C ABI in q8_0_abi.h.  The reference's
// names it uses (device_types, kernel_types, processing_phases, block_q8_0, half, core_trait_dims, kernel_traits_old)
// come from the reference's own headers when NIHILUS_AMD_WITH_REFERENCE_HEADERS is defined (include them first), and
// from reference_mirror.hpp otherwise.  Errors follow the reference's convention (common/exception.hpp:65-107): log,
// then throw or std::exit(-1) as config_type::exceptions says.
#pragma once

#include "q8_0_abi.h"

#ifndef NIHILUS_AMD_WITH_REFERENCE_HEADERS
	#include "reference_mirror.hpp"
#endif

#include <array>
#include <cstdint>
#include <cstdlib>
#include <iostream>
#include <source_location>
#include <stdexcept>
#include <string>
#include <string_view>
#include <utility>

namespace nihilus {

	// The arch index of this back end: the reference numbers its CUDA targets 1..4 (cuda/nihilus_gpu_properties.hpp:28-40).
	inline constexpr uint64_t gfx950_arch_index{ 5 };

	// The per-op specialisation point (the parameter list of the reference's dead per-op form, cpu/avx_2.hpp:1296).
	template<typename config_type, typename core_traits_type, device_types device_type, uint64_t arch, kernel_types kernel_type, processing_phases processing_phase,
		typename... types>
	struct per_op_kernel_dispatcher_impl;

	namespace amd_detail {
		// throw, or log and std::exit(-1), chosen by the config at compile time (the two forms of nihilus_exception,
		// common/exception.hpp:65-107; that template takes its message and location as template arguments, which a run-time
		// status text cannot be, hence this function of the same behaviour)
		template<bool exceptions> [[noreturn]] inline void raise(std::string_view error_type, std::string_view detail, const std::source_location& where) {
			std::string text{ "Error: " };
			text.append(error_type).append(detail).append("\nIn File: ").append(where.file_name()).append("\nOn Line: ").append(std::to_string(where.line())).append("\n");
			std::cerr << text << std::endl;
			if constexpr (exceptions) {
				throw std::runtime_error{ text };
			} else {
				std::exit(-1);
			}
		}
		template<typename config_type> inline void check(int status, const char* what, const std::source_location where = std::source_location::current()) {
			if (status != NH_OK) {
				raise<config_type::exceptions>("HIP Q8_0 mul_mat: ", std::string{ what } + ": " + nh_status_string(status), where);
			}
		}
	}

	// The weight operand of a GPU mul_mat holds the tiled copy made at load time (nh_q8_0_tile); the activation operand
	// holds fp32 values (the output of the rms_norm/mul or silu/mul step in front of it); the workspace operand is the
	// arena slice for the quantized activations of the prompt phase.
	//
	// eval_time: one token.  y[N] = W . quantize(x), quantize fused into the mat-vec kernel.
	template<typename config_type, typename core_traits_type>
	struct per_op_kernel_dispatcher_impl<config_type, core_traits_type, device_types::gpu, gfx950_arch_index, kernel_types::mul_mat, processing_phases::eval_time, core_traits_type, float,
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
	struct per_op_kernel_dispatcher_impl<config_type, core_traits_type, device_types::gpu, gfx950_arch_index, kernel_types::mul_mat, processing_phases::prompt_eval_time, core_traits_type, float,
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
	struct per_op_kernel_dispatcher_impl<config_type, core_traits_type, device_types::gpu, gfx950_arch_index, kernel_types::mul_mat, processing_phase, core_traits_type, float, block_q8_0<half>, float> {
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
	struct per_op_kernel_dispatcher_impl<config_type, core_traits_type, device_types::gpu, gfx950_arch_index, kernel_types::get_rows, processing_phase, core_traits_type, float, block_q8_0<half>,
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
		using impl_type = per_op_kernel_dispatcher_impl<config_type, mul_mat_traits_type, config_type::device_type, gfx950_arch_index, kernel_types::mul_mat,
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
		using impl_type = per_op_kernel_dispatcher_impl<config_type, get_rows_traits_type, config_type::device_type, gfx950_arch_index, kernel_types::get_rows,
			processing_phase, get_rows_traits_type, float, block_q8_0<half>, int32_t>;
		template<typename... arg_types> static void impl(arg_types&&... args) {
			impl_type::impl(std::forward<arg_types>(args)...);
		}
	};

} // namespace nihilus
