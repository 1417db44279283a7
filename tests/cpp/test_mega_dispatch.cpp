// Runs the gfx950 specialisations of the reference's LIVE dispatch point (include/nihilus_amd/mega_dispatch.hpp) on the GPU
// through kernel_dispatcher<config, phase, core>::impl(params[, current_block]), exactly as the reference's scheduler calls
// them (infra/monolithic_dispatcher.hpp:54-66), on a two-block LLaMA-shaped graph, both phases, and checks every core's
// output against the CPU checker fed with the GPU's own inputs of that stage.  A test, not product code.
// Exit status 0 = pass.  `--compile-only-check` returns after the static checks (no GPU needed).
#include <nihilus_amd/mega_dispatch.hpp>

#include "mock_model.hpp"

#include <cmath>
#include <cstdio>
#include <cstring>
#include <type_traits>
#include <vector>

extern "C" { // the CPU checker
void nho_fill_activations(uint64_t seed, float* x, int64_t count);
void nho_fill_weight_blocks(uint64_t seed, void* out, int64_t first_block, int64_t n_blocks);
void nho_quantize_rows_q8_0(const float* x, void* y, int64_t m, int64_t k);
void nho_rms_norm_quantize_rows_q8_0(const float* x, const float* w, float eps, void* vy, int64_t m, int64_t k, float* scratch_row);
void nho_silu_mul_quantize_rows_q8_0(const float* gate, const float* up, void* vy, int64_t m, int64_t k);
void nho_gemm_q8_0(const void* w, const void* aq, float* c, int64_t m, int64_t n, int64_t k);
}

using namespace nihilus;

// what the hooks saw, for the checks below
static const float *seen_k = nullptr, *seen_v = nullptr, *seen_logits = nullptr;
static uint64_t seen_rows = 0;
template<> struct nihilus::amd_qkv_epilogue<mock_config> {
	template<typename core_traits_type> static void impl(core_traits_type&, int64_t, uint64_t rows, float*, const float* k, const float* v, void*) {
		seen_k	  = k;
		seen_v	  = v;
		seen_rows = rows;
	}
};
template<> struct nihilus::amd_sampling<mock_config> {
	template<typename core_traits_type> static void impl(core_traits_type&, const float* logits, void*) {
		seen_logits = logits;
	}
};

using mtt = tiny_llama_traits;
using qkv_core	 = core_traits_old<mock_config, core_types::mega_qkv_prep_and_cache_publish>;
using attn_core	 = core_traits_old<mock_config, core_types::mega_attention_apply>;
using ffn_core	 = core_traits_old<mock_config, core_types::mega_ffn>;
using final_core = core_traits_old<mock_config, core_types::final_norm_and_sampling>;

// the specialisations exist, are complete types and are the ones the caller-side template picks
static_assert(gfx950_arch_index == 5 && arch_index<device_types::gpu> == 5);
static_assert(sizeof(kernel_dispatcher_impl<mock_config, qkv_core, device_types::gpu, 5, core_types::mega_qkv_prep_and_cache_publish, processing_phases::eval_time>) > 0);
static_assert(sizeof(kernel_dispatcher_impl<mock_config, attn_core, device_types::gpu, 5, core_types::mega_attention_apply, processing_phases::prompt_eval_time>) > 0);
static_assert(sizeof(kernel_dispatcher_impl<mock_config, ffn_core, device_types::gpu, 5, core_types::mega_ffn, processing_phases::eval_time>) > 0);
static_assert(sizeof(kernel_dispatcher_impl<mock_config, final_core, device_types::gpu, 5, core_types::final_norm_and_sampling, processing_phases::prompt_eval_time>) > 0);

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

struct matrix {
	std::vector<uint8_t> blocks; // host copy, packed blocks (for the checker)
	void* tiled = nullptr; // device copy in the tiled layout (what the graph's weight nodes point at)
	int64_t n = 0, k = 0;
};

static int make_matrix(matrix& m, uint64_t seed, int64_t n, int64_t k) {
	m.n = n;
	m.k = k;
	m.blocks.resize(n * (k / 32) * 34);
	nho_fill_weight_blocks(seed, m.blocks.data(), 0, n * (k / 32));
	void* d_blocks = nullptr;
	REQUIRE(nh_malloc(&d_blocks, static_cast<int64_t>(m.blocks.size())) == NH_OK);
	REQUIRE(nh_malloc(&m.tiled, nh_q8_0_tiled_bytes(n, k)) == NH_OK);
	REQUIRE(nh_memcpy_h2d(d_blocks, m.blocks.data(), static_cast<int64_t>(m.blocks.size()), nullptr) == NH_OK);
	REQUIRE(nh_q8_0_tile(d_blocks, m.tiled, n, k, nullptr) == NH_OK); // the load-time copy into the device layout
	REQUIRE(nh_stream_sync(nullptr) == NH_OK);
	REQUIRE(nh_free(d_blocks) == NH_OK);
	return 0;
}

static int upload(void** dev, const std::vector<float>& host) {
	REQUIRE(nh_malloc(dev, static_cast<int64_t>(host.size() * 4)) == NH_OK);
	REQUIRE(nh_memcpy_h2d(*dev, host.data(), static_cast<int64_t>(host.size() * 4), nullptr) == NH_OK);
	return 0;
}

static int download(std::vector<float>& host, const void* dev, int64_t count) {
	host.resize(count);
	REQUIRE(nh_memcpy_d2h(host.data(), dev, count * 4, nullptr) == NH_OK && nh_stream_sync(nullptr) == NH_OK);
	return 0;
}

// C [m][n] = W . quantize(rows) on the CPU, with an optional norm in front and residual behind
static std::vector<float> cpu_mul_mat(const matrix& w, const std::vector<float>& x, int64_t m, const std::vector<float>* norm_w, const std::vector<float>* residual) {
	std::vector<uint8_t> xq(m * (w.k / 32) * 34);
	std::vector<float> row(w.k);
	if (norm_w) {
		nho_rms_norm_quantize_rows_q8_0(x.data(), norm_w->data(), mtt::layer_norm_rms_epsilon, xq.data(), m, w.k, row.data());
	} else {
		nho_quantize_rows_q8_0(x.data(), xq.data(), m, w.k);
	}
	std::vector<float> c(m * w.n);
	nho_gemm_q8_0(w.blocks.data(), xq.data(), c.data(), m, w.n, w.k);
	if (residual) {
		for (size_t i = 0; i < c.size(); ++i) {
			c[i] += (*residual)[i];
		}
	}
	return c;
}

// the mat-mul path alone, one launch per core in the decode phase too (every core's outputs complete when it returns)
struct per_core_config : mock_config {
	static constexpr bool amd_decode_per_core_launches{ true };
};
template<> struct nihilus::amd_qkv_epilogue<per_core_config> : nihilus::amd_qkv_epilogue<mock_config> {};
template<> struct nihilus::amd_sampling<per_core_config> : nihilus::amd_sampling<mock_config> {};

template<processing_phases phase, typename dispatch_config = mock_config> static int run_phase(nihilus_cathedral<mock_config>& model, const matrix (&wq)[2], const matrix (&wk)[2], const matrix (&wv)[2], const matrix (&wo)[2],
	const matrix (&wg)[2], const matrix (&wu)[2], const matrix (&wd)[2], const matrix& w_out, const std::vector<float> (&attn_norm)[2], const std::vector<float> (&ffn_norm)[2],
	const std::vector<float>& out_norm, const std::vector<float>& x0, int64_t rows, void* d_q, void* d_ffn_inp, void* d_l_out) {
	constexpr int64_t E = mtt::embedding_length, KV = mtt::n_embd_kv_gqa, F = mtt::feed_forward_length, V = mtt::vocab_size;
	// in the decode phase the cores chain (unless the config asks for one launch per core): mega_attention_apply leaves its projection
	// to mega_ffn, whose launch also does the next core's mat-vecs, so ffn_inp is complete after mega_ffn, not before
	constexpr bool chained = phase == processing_phases::eval_time && amd_detail::chains_decode<dispatch_config>;
	const char* name = phase == processing_phases::eval_time ? (chained ? "eval_time (chained)" : "eval_time (per core)") : "prompt_eval_time";
	auto dispatch = [&]<core_types core, typename core_type>(core_type& c, int64_t block) {
		kernel_dispatcher_impl<dispatch_config, core_type, device_types::gpu, gfx950_arch_index, core, phase>::impl(c, block);
	};
	auto& qkv		 = static_cast<qkv_core&>(model);
	auto& attn		 = static_cast<attn_core&>(model);
	auto& ffn		 = static_cast<ffn_core&>(model);
	auto& fin		 = static_cast<final_core&>(model);
	// the one runtime dim of every mega core's output node
	qkv.values.get_core<mega_qkv_prep_and_cache_publish_types, mega_qkv_prep_and_cache_publish_types::q_out>().get_seq_length_dim() = rows;
	attn.values.get_core<mega_attention_apply_types, mega_attention_apply_types::ffn_inp>().get_seq_length_dim()					= rows;
	ffn.values.get_core<mega_ffn_types, mega_ffn_types::l_out>().get_seq_length_dim()												= rows;

	std::vector<float> layer_in = x0, got, got_k, got_v;
	for (int64_t block = 0; block < 2; ++block) {
		if constexpr (std::is_same_v<dispatch_config, mock_config>) {
			kernel_dispatcher<mock_config, phase, qkv_core>::impl(qkv, block); // the reference's caller-side template picks the specialisation
		} else {
			dispatch.template operator()<core_types::mega_qkv_prep_and_cache_publish>(qkv, block);
		}
		REQUIRE(seen_rows == static_cast<uint64_t>(rows) && seen_k && seen_v);
		REQUIRE(download(got, d_q, rows * E) == 0 && download(got_k, seen_k, rows * KV) == 0 && download(got_v, seen_v, rows * KV) == 0);
		const double eq = rel_l2(got, cpu_mul_mat(wq[block], layer_in, rows, &attn_norm[block], nullptr));
		const double ek = rel_l2(got_k, cpu_mul_mat(wk[block], layer_in, rows, &attn_norm[block], nullptr));
		const double ev = rel_l2(got_v, cpu_mul_mat(wv[block], layer_in, rows, &attn_norm[block], nullptr));
		std::printf("%s block %lld mega_qkv        q %.2e  k %.2e  v %.2e\n", name, static_cast<long long>(block), eq, ek, ev);
		REQUIRE(eq <= 1e-4 && ek <= 1e-4 && ev <= 1e-4);

		const std::vector<float> q_gpu = got; // the stand-in attention output of the primary amd_attention
		dispatch.template operator()<core_types::mega_attention_apply>(attn, block);
		if constexpr (!chained) {
			REQUIRE(download(got, d_ffn_inp, rows * E) == 0);
		}
		dispatch.template operator()<core_types::mega_ffn>(ffn, block);
		if constexpr (chained) {
			REQUIRE(download(got, d_ffn_inp, rows * E) == 0);
		}
		const double eo = rel_l2(got, cpu_mul_mat(wo[block], q_gpu, rows, nullptr, &layer_in));
		std::printf("%s block %lld mega_attention  attn_out + residual %.2e\n", name, static_cast<long long>(block), eo);
		REQUIRE(eo <= 1e-4);

		const std::vector<float> ffn_in = got;
		REQUIRE(download(got, d_l_out, rows * E) == 0);
		const std::vector<float> g = cpu_mul_mat(wg[block], ffn_in, rows, &ffn_norm[block], nullptr), u = cpu_mul_mat(wu[block], ffn_in, rows, &ffn_norm[block], nullptr);
		std::vector<uint8_t> hq(rows * (F / 32) * 34);
		nho_silu_mul_quantize_rows_q8_0(g.data(), u.data(), hq.data(), rows, F);
		std::vector<float> want(rows * E);
		nho_gemm_q8_0(wd[block].blocks.data(), hq.data(), want.data(), rows, E, F);
		for (size_t i = 0; i < want.size(); ++i) {
			want[i] += ffn_in[i];
		}
		const double ef = rel_l2(got, want);
		std::printf("%s block %lld mega_ffn        l_out %.2e\n", name, static_cast<long long>(block), ef);
		// three dependent stages with a quantizer between them: a last-bit difference in gate / up can move a quant by one step, so
		// the end-to-end bound is looser than a single mat-mul's (the stages themselves are checked at 1e-4 by the Python suite)
		REQUIRE(ef <= 1e-3);
		layer_in = got;
	}
	seen_logits = nullptr;
	kernel_dispatcher_impl<dispatch_config, final_core, device_types::gpu, gfx950_arch_index, core_types::final_norm_and_sampling, phase>::impl(fin);
	REQUIRE(seen_logits);
	REQUIRE(download(got, seen_logits, V) == 0);
	const std::vector<float> last(layer_in.end() - E, layer_in.end());
	const double el = rel_l2(got, cpu_mul_mat(w_out, last, 1, &out_norm, nullptr));
	std::printf("%s final_norm_and_sampling    logits %.2e\n", name, el);
	REQUIRE(el <= 1e-4);
	return 0;
}

int main(int argc, char** argv) {
	if (argc > 1 && std::strcmp(argv[1], "--compile-only-check") == 0) {
		std::printf("static checks ok\n");
		return 0;
	}
	constexpr int64_t E = mtt::embedding_length, KV = mtt::n_embd_kv_gqa, F = mtt::feed_forward_length, V = mtt::vocab_size;
	constexpr int64_t MAX_ROWS = mock_config::max_sequence_length, ROWS = 37; // a sequence length that is not a multiple of any tile

	nihilus_cathedral<mock_config> model;
	auto& weights = static_cast<core_traits_old<mock_config, core_types::weights>&>(model);
	matrix wq[2], wk[2], wv[2], wo[2], wg[2], wu[2], wd[2], w_out;
	std::vector<float> attn_norm[2], ffn_norm[2], out_norm(E);
	auto norm_weight = [](uint64_t seed, std::vector<float>& w) {
		w.resize(E);
		nho_fill_activations(seed, w.data(), E);
		for (float& v : w) {
			v = 1.0f + 0.1f * v;
		}
	};
	for (int b = 0; b < 2; ++b) {
		REQUIRE(make_matrix(wq[b], 100 + b, E, E) == 0 && make_matrix(wk[b], 110 + b, KV, E) == 0 && make_matrix(wv[b], 120 + b, KV, E) == 0 && make_matrix(wo[b], 130 + b, E, E) == 0);
		REQUIRE(make_matrix(wg[b], 140 + b, F, E) == 0 && make_matrix(wu[b], 150 + b, F, E) == 0 && make_matrix(wd[b], 160 + b, E, F) == 0);
		norm_weight(170 + b, attn_norm[b]);
		norm_weight(180 + b, ffn_norm[b]);
		void *d_an = nullptr, *d_fn = nullptr;
		REQUIRE(upload(&d_an, attn_norm[b]) == 0 && upload(&d_fn, ffn_norm[b]) == 0);
		weights.values.get_core<weight_types, weight_types::attn_q>().set_data(wq[b].tiled, b);
		weights.values.get_core<weight_types, weight_types::attn_k>().set_data(wk[b].tiled, b);
		weights.values.get_core<weight_types, weight_types::attn_v>().set_data(wv[b].tiled, b);
		weights.values.get_core<weight_types, weight_types::attn_output>().set_data(wo[b].tiled, b);
		weights.values.get_core<weight_types, weight_types::attn_norm>().set_data(d_an, b);
		weights.values.get_core<weight_types, weight_types::ffn_gate>().set_data(wg[b].tiled, b);
		weights.values.get_core<weight_types, weight_types::ffn_up>().set_data(wu[b].tiled, b);
		weights.values.get_core<weight_types, weight_types::ffn_down>().set_data(wd[b].tiled, b);
		weights.values.get_core<weight_types, weight_types::ffn_norm>().set_data(d_fn, b);
	}
	REQUIRE(make_matrix(w_out, 190, V, E) == 0);
	norm_weight(191, out_norm);
	void* d_on = nullptr;
	REQUIRE(upload(&d_on, out_norm) == 0);
	weights.values.get_core<weight_types, weight_types::output>().set_data(w_out.tiled);
	weights.values.get_core<weight_types, weight_types::output_norm>().set_data(d_on);

	// activations: the token-embedding output (the first block's input) and the three mega cores' output tensors
	std::vector<float> x0(ROWS * E);
	nho_fill_activations(7, x0.data(), ROWS * E);
	void *d_x0 = nullptr, *d_q = nullptr, *d_ffn_inp = nullptr, *d_l_out = nullptr;
	REQUIRE(upload(&d_x0, x0) == 0);
	REQUIRE(nh_malloc(&d_q, MAX_ROWS * E * 4) == NH_OK && nh_malloc(&d_ffn_inp, MAX_ROWS * E * 4) == NH_OK && nh_malloc(&d_l_out, MAX_ROWS * E * 4) == NH_OK);
	static_cast<core_traits_old<mock_config, core_types::token_embeddings>&>(model).values.get_core<token_embeddings_types, token_embeddings_types::get_rows>().set_data(d_x0);
	static_cast<qkv_core&>(model).values.get_core<mega_qkv_prep_and_cache_publish_types, mega_qkv_prep_and_cache_publish_types::q_out>().set_data(d_q);
	static_cast<attn_core&>(model).values.get_core<mega_attention_apply_types, mega_attention_apply_types::ffn_inp>().set_data(d_ffn_inp);
	static_cast<ffn_core&>(model).values.get_core<mega_ffn_types, mega_ffn_types::l_out>().set_data(d_l_out);

	// every buffer the dispatchers need is sized once, up front; from here on no impl may allocate
	amd_prepare<mock_config, mtt>(MAX_ROWS);
	const int64_t allocations_after_prepare = amd_workspace_allocations<mock_config>();
	REQUIRE(allocations_after_prepare == 7);

	// eval_time: one token (the first row of x0); prompt_eval_time: 37 rows through the outputs' runtime dim
	const std::vector<float> x_one(x0.begin(), x0.begin() + E);
	REQUIRE(run_phase<processing_phases::eval_time>(model, wq, wk, wv, wo, wg, wu, wd, w_out, attn_norm, ffn_norm, out_norm, x_one, 1, d_q, d_ffn_inp, d_l_out) == 0);
	REQUIRE(run_phase<processing_phases::prompt_eval_time>(model, wq, wk, wv, wo, wg, wu, wd, w_out, attn_norm, ffn_norm, out_norm, x0, ROWS, d_q, d_ffn_inp, d_l_out) == 0);
	// a decode step right after a prompt pass (nothing of the prompt pass may be taken for a finished decode mat-vec), then the
	// same step with one launch per core
	REQUIRE(run_phase<processing_phases::eval_time>(model, wq, wk, wv, wo, wg, wu, wd, w_out, attn_norm, ffn_norm, out_norm, x_one, 1, d_q, d_ffn_inp, d_l_out) == 0);
	amd_prepare<per_core_config, mtt>(1);
	REQUIRE((run_phase<processing_phases::eval_time, per_core_config>(model, wq, wk, wv, wo, wg, wu, wd, w_out, attn_norm, ffn_norm, out_norm, x_one, 1, d_q, d_ffn_inp, d_l_out) == 0));

	// a long prompt after a short one, and nothing was allocated on the way; preparing again for the same length allocates nothing either
	REQUIRE(amd_workspace_allocations<mock_config>() == allocations_after_prepare);
	amd_prepare<mock_config, mtt>(MAX_ROWS);
	REQUIRE(amd_workspace_allocations<mock_config>() == allocations_after_prepare);

	// a sequence longer than prepared for is refused through the config's error convention, before anything is launched
	static_cast<ffn_core&>(model).values.get_core<mega_ffn_types, mega_ffn_types::l_out>().get_seq_length_dim() = MAX_ROWS + 1;
	bool refused = false;
	try {
		kernel_dispatcher<mock_config, processing_phases::prompt_eval_time, ffn_core>::impl(static_cast<ffn_core&>(model), 0);
	} catch (const std::runtime_error& e) {
		refused = std::strstr(e.what(), "amd_prepare") != nullptr;
	}
	REQUIRE(refused);
	REQUIRE(amd_workspace_allocations<mock_config>() == allocations_after_prepare);

	// an empty sequence launches nothing
	static_cast<ffn_core&>(model).values.get_core<mega_ffn_types, mega_ffn_types::l_out>().get_seq_length_dim() = 0;
	kernel_dispatcher<mock_config, processing_phases::prompt_eval_time, ffn_core>::impl(static_cast<ffn_core&>(model), 0);

	// error convention: a status from the C ABI becomes the config's exception
	static_cast<ffn_core&>(model).values.get_core<mega_ffn_types, mega_ffn_types::l_out>().get_seq_length_dim() = 1;
	weights.values.get_core<weight_types, weight_types::ffn_gate>().set_data(nullptr, 0);
	bool thrown = false;
	try {
		kernel_dispatcher<mock_config, processing_phases::eval_time, ffn_core>::impl(static_cast<ffn_core&>(model), 0);
	} catch (const std::runtime_error& e) {
		thrown = std::strstr(e.what(), "null pointer") != nullptr && std::strstr(e.what(), "mega_ffn eval_time") != nullptr;
	}
	REQUIRE(thrown);
	std::printf("mega dispatch ok\n");
	return 0;
}
