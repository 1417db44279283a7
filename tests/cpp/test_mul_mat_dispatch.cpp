// Exercises the C++23 dispatch surface (include/nihilus_amd/mul_mat_dispatch.hpp) end to end on the GPU:
// compile-time shape contract, phase -> kernel selection, runtime sequence length, error convention.
// Results are checked against the CPU checker (oracle/libq8_0_oracle.so); this file is a test, not product code.
// Exit status 0 = pass.  `--compile-only-check` returns after the static checks (no GPU needed).
#include <nihilus_amd/mul_mat_dispatch.hpp>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <vector>

extern "C" { // the CPU checker
void nho_fill_activations(uint64_t seed, float* x, int64_t count);
void nho_fill_weight_blocks(uint64_t seed, void* out, int64_t first_block, int64_t n_blocks);
void nho_quantize_rows_q8_0(const float* x, void* y, int64_t m, int64_t k);
void nho_gemm_q8_0(const void* w, const void* aq, float* c, int64_t m, int64_t n, int64_t k);
int64_t nho_get_rows_q8_0(const void* w, const int32_t* ids, float* out, int64_t n_tokens, int64_t n_rows, int64_t k);
void nho_mul_mat_q8_f32(const void* w, const float* x, float* y, int64_t m_rows, int64_t n_rows, int64_t k, int order);
}

using namespace nihilus;

struct test_config {
	static constexpr device_types device_type{ device_types::gpu };
	static constexpr kernel_type_profiles kernel_type_profile{ kernel_type_profiles::q8_gqa };
	static constexpr bool exceptions{ true };
	static constexpr bool synchronous{ true }; // sync after each launch, as the reference's GPU path does
	static constexpr uint64_t max_sequence_length{ 64 };
	struct model_traits_type {
		static constexpr uint32_t block_count{ 32 };
	};
};

// LLaMA-3-8B k-projection shape (infra/model_traits.hpp:49-65, infra/core_traits.hpp:583-584): W [K = 4096, N = 1024]
constexpr uint64_t K = 4096, N = 1024;
using weight_type	  = core_trait_dims<K, N, 1, 1>;
using activation_type = core_trait_dims<K, test_config::max_sequence_length, 1, 1, 1>; // dim1 = sequence length, runtime
using output_dims	  = core_trait_dims<N, test_config::max_sequence_length, 1, 1, 1>;

struct k_mul_mat_op : kernel_traits_old<test_config, output_dims, kernel_types::mul_mat, float, weight_type, activation_type>, data_mixin<test_config, data_strategy_types::global, float> {};

static_assert(k_mul_mat_op::input_01_dims[0] == K && k_mul_mat_op::output_dims[0] == N);
static_assert(arch_index<device_types::gpu> == 5 && gfx950_arch_index == 5);
static_assert(runtime_dims_t<k_mul_mat_op>);
static_assert(sizeof(block_q8_0<half>) == NH_Q8_0_BLOCK_BYTES && Q_SIZE == NH_Q8_0_QK);

// token embeddings: table [K, N rows] (the k-projection bytes stand in for an embedding table), ids [tokens], out [K, tokens]
using ids_type		= core_trait_dims<test_config::max_sequence_length, 1, 1, 1>;
using embd_out_dims = core_trait_dims<K, test_config::max_sequence_length, 1, 1, 1>;
struct get_rows_op : kernel_traits_old<test_config, embd_out_dims, kernel_types::get_rows, float, weight_type, ids_type>, data_mixin<test_config, data_strategy_types::global, float> {};
using embd_eval_dispatch   = get_rows_dispatcher<test_config, processing_phases::eval_time, get_rows_op>;
using embd_prompt_dispatch = get_rows_dispatcher<test_config, processing_phases::prompt_eval_time, get_rows_op>;

using eval_dispatch	  = mul_mat_dispatcher<test_config, processing_phases::eval_time, k_mul_mat_op>;
using prompt_dispatch = mul_mat_dispatcher<test_config, processing_phases::prompt_eval_time, k_mul_mat_op>;

static double rel_l2(const std::vector<float>& a, const std::vector<float>& b) {
	double num = 0, den = 0;
	for (size_t i = 0; i < a.size(); ++i) {
		num += (double(a[i]) - b[i]) * (double(a[i]) - b[i]);
		den += double(b[i]) * b[i];
	}
	return std::sqrt(num / den);
}

#define REQUIRE(cond)                                                  \
	do {                                                               \
		if (!(cond)) {                                                 \
			std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
			return 1;                                                  \
		}                                                              \
	} while (0)

int main(int argc, char** argv) {
	if (argc > 1 && std::strcmp(argv[1], "--compile-only-check") == 0) {
		std::printf("static checks ok\n");
		return 0;
	}
	const int64_t nb = K / 32, w_bytes = N * nb * 34;
	const int64_t M = 37; // a sequence length that is not a multiple of any tile

	// host data from the counter-based generator; CPU answers from the checker
	std::vector<uint8_t> w(w_bytes);
	nho_fill_weight_blocks(11, w.data(), 0, N * nb);
	std::vector<float> x(M * K);
	nho_fill_activations(11, x.data(), M * K);
	std::vector<uint8_t> aq(M * nb * 34);
	nho_quantize_rows_q8_0(x.data(), aq.data(), M, K);
	std::vector<float> want(M * N);
	nho_gemm_q8_0(w.data(), aq.data(), want.data(), M, N, K);

	// device arena
	void *d_blocks = nullptr, *d_tiled = nullptr, *d_x = nullptr, *d_y = nullptr, *d_ws = nullptr;
	const int64_t ws_bytes = prompt_dispatch::impl_type::workspace_bytes(test_config::max_sequence_length);
	REQUIRE(nh_malloc(&d_blocks, w_bytes) == NH_OK);
	REQUIRE(nh_malloc(&d_tiled, nh_q8_0_tiled_bytes(N, K)) == NH_OK);
	REQUIRE(nh_malloc(&d_x, M * K * 4) == NH_OK);
	REQUIRE(nh_malloc(&d_y, test_config::max_sequence_length * N * 4) == NH_OK);
	REQUIRE(nh_malloc(&d_ws, ws_bytes) == NH_OK);
	REQUIRE(nh_memcpy_h2d(d_blocks, w.data(), w_bytes, nullptr) == NH_OK);
	REQUIRE(nh_memcpy_h2d(d_x, x.data(), M * K * 4, nullptr) == NH_OK);
	REQUIRE(nh_q8_0_tile(d_blocks, d_tiled, N, K, nullptr) == NH_OK); // the load-time copy into the device layout
	REQUIRE(nh_stream_sync(nullptr) == NH_OK);

	k_mul_mat_op op;
	op.set_data(d_y);

	// eval_time: one token
	eval_dispatch::impl(op, d_tiled, static_cast<const float*>(d_x));
	std::vector<float> y(N);
	REQUIRE(nh_memcpy_d2h(y.data(), d_y, N * 4, nullptr) == NH_OK && nh_stream_sync(nullptr) == NH_OK);
	const double e1 = rel_l2(y, std::vector<float>(want.begin(), want.begin() + N));
	std::printf("eval_time        rel L2 %.3e\n", e1);
	REQUIRE(e1 <= 1e-4);

	// eval_time with the residual add folded in, in place: the buffer holds y, the same launch on top of it gives exactly 2 y
	eval_dispatch::impl_add(op, d_tiled, static_cast<const float*>(d_x), static_cast<const float*>(d_y));
	std::vector<float> y2(N);
	REQUIRE(nh_memcpy_d2h(y2.data(), d_y, N * 4, nullptr) == NH_OK && nh_stream_sync(nullptr) == NH_OK);
	for (uint64_t i = 0; i < N; ++i) {
		REQUIRE(y2[i] == 2.0f * y[i]);
	}

	// prompt_eval_time: runtime sequence length through the dims' runtime slot
	op.get_seq_length_dim() = M;
	prompt_dispatch::impl(op, d_tiled, static_cast<const float*>(d_x), d_ws, ws_bytes);
	std::vector<float> c(M * N);
	REQUIRE(nh_memcpy_d2h(c.data(), d_y, M * N * 4, nullptr) == NH_OK && nh_stream_sync(nullptr) == NH_OK);
	const double e2 = rel_l2(c, want);
	std::printf("prompt_eval_time rel L2 %.3e  (M = %lld)\n", e2, static_cast<long long>(M));
	REQUIRE(e2 <= 1e-4);

	// the same with the residual add folded in, in place on the buffer that holds C: exactly 2 C
	prompt_dispatch::impl_add(op, d_tiled, static_cast<const float*>(d_x), static_cast<const float*>(d_y), d_ws, ws_bytes);
	std::vector<float> c2(M * N);
	REQUIRE(nh_memcpy_d2h(c2.data(), d_y, M * N * 4, nullptr) == NH_OK && nh_stream_sync(nullptr) == NH_OK);
	for (uint64_t i = 0; i < M * N; ++i) {
		REQUIRE(c2[i] == 2.0f * c[i]);
	}

	// empty sequence: nothing is launched, nothing changes
	op.get_seq_length_dim() = 0;
	prompt_dispatch::impl(op, d_tiled, static_cast<const float*>(d_x), d_ws, ws_bytes);

	// error convention: a rejected argument becomes an exception when the config asks for exceptions
	bool thrown = false;
	try {
		eval_dispatch::impl(op, nullptr, static_cast<const float*>(d_x));
	} catch (const std::runtime_error& e) {
		thrown = std::strstr(e.what(), "null pointer") != nullptr;
	}
	REQUIRE(thrown);

	// the key the reference implements on the CPU, <float, block_q8_0<half>, float>: fp32 activations, no activation quantize
	{
		using f32_eval	 = per_op_kernel_dispatcher_impl<test_config, k_mul_mat_op, device_types::gpu, 5, kernel_types::mul_mat, processing_phases::eval_time, k_mul_mat_op, float, block_q8_0<half>, float>;
		using f32_prompt = per_op_kernel_dispatcher_impl<test_config, k_mul_mat_op, device_types::gpu, 5, kernel_types::mul_mat, processing_phases::prompt_eval_time, k_mul_mat_op, float, block_q8_0<half>,
			float>;
		std::vector<float> want_f(M * N), got_f(M * N);
		nho_mul_mat_q8_f32(w.data(), x.data(), want_f.data(), 1, N, K, 0); // the eval_time leaf's order
		f32_eval::impl(op, d_tiled, static_cast<const float*>(d_x));
		REQUIRE(nh_memcpy_d2h(got_f.data(), d_y, N * 4, nullptr) == NH_OK && nh_stream_sync(nullptr) == NH_OK);
		const double e3 = rel_l2(std::vector<float>(got_f.begin(), got_f.begin() + N), std::vector<float>(want_f.begin(), want_f.begin() + N));
		nho_mul_mat_q8_f32(w.data(), x.data(), want_f.data(), M, N, K, 1); // the prompt_eval_time leaf's
		op.get_seq_length_dim() = M;
		f32_prompt::impl(op, d_tiled, static_cast<const float*>(d_x));
		REQUIRE(nh_memcpy_d2h(got_f.data(), d_y, M * N * 4, nullptr) == NH_OK && nh_stream_sync(nullptr) == NH_OK);
		const double e4 = rel_l2(got_f, want_f);
		std::printf("fp32 activations rel L2 %.3e (eval) %.3e (prompt)\n", e3, e4);
		REQUIRE(e3 <= 1e-4 && e4 <= 1e-4);
		op.get_seq_length_dim() = 0;
	}

	// token embeddings: bit-exact, both phases, both table layouts; eval_time must honour the id
	{
		const int64_t T = 5;
		const int32_t ids[T] = { 1023, 0, 17, 17, 512 };
		std::vector<float> want_rows(T * K), got_rows(T * K);
		REQUIRE(nho_get_rows_q8_0(w.data(), ids, want_rows.data(), T, N, K) == 0);
		void *d_ids = nullptr, *d_e = nullptr;
		REQUIRE(nh_malloc(&d_ids, sizeof(ids)) == NH_OK && nh_malloc(&d_e, test_config::max_sequence_length * K * 4) == NH_OK);
		REQUIRE(nh_memcpy_h2d(d_ids, ids, sizeof(ids), nullptr) == NH_OK && nh_stream_sync(nullptr) == NH_OK);
		get_rows_op e;
		e.set_data(d_e);
		e.get_seq_length_dim() = T;
		for (const bool tiled : { false, true }) {
			embd_prompt_dispatch::impl(e, tiled ? d_tiled : d_blocks, tiled, static_cast<const int32_t*>(d_ids));
			REQUIRE(nh_memcpy_d2h(got_rows.data(), d_e, T * K * 4, nullptr) == NH_OK && nh_stream_sync(nullptr) == NH_OK);
			REQUIRE(std::memcmp(got_rows.data(), want_rows.data(), T * K * 4) == 0);
			embd_eval_dispatch::impl(e, tiled ? d_tiled : d_blocks, tiled, static_cast<const int32_t*>(d_ids) + 4); // id 512, not row 0
			REQUIRE(nh_memcpy_d2h(got_rows.data(), d_e, K * 4, nullptr) == NH_OK && nh_stream_sync(nullptr) == NH_OK);
			REQUIRE(std::memcmp(got_rows.data(), want_rows.data() + 4 * K, K * 4) == 0);
		}
		std::printf("get_rows         bit-exact (prompt and eval, blocks and tiled)\n");
		nh_free(d_ids);
		nh_free(d_e);
	}

	nh_free(d_blocks);
	nh_free(d_tiled);
	nh_free(d_x);
	nh_free(d_y);
	nh_free(d_ws);
	std::printf("mul_mat dispatch ok\n");
	return 0;
}
