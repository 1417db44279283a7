// Times a decode token through the reference's dispatch point: kernel_dispatcher<config, eval_time, core>::impl(params[, block])
// for the three per-block mega cores of 32 blocks and the final core, at the LLaMA-3-8B shapes, with the gfx950 specialisations
// of include/nihilus_amd/mega_dispatch.hpp underneath (the call sequence of infra/monolithic_dispatcher.hpp:54-66).  Weights
// are made on the device by the library's generator; nothing here touches the CPU checker.  Prints one JSON object:
//   decode:   a whole token (32 x [norm -> q/k/v], [o + residual], [norm -> gate/up -> SiLU.up -> down + residual], norm -> lm_head;
//             the attention stand-in of the header's primary amd_attention: its output is q), the final core waits for the device
//             as the reference's does;
//   mega_ffn: the FFN core alone over the 32 blocks' weights (2.8 GB in rotation), one wait at the end.
// A measurement tool beside the tests; bench.py runs it when it has been built.
#define NH_MOCK_MODEL_TRAITS llama3_8b_traits
#include <nihilus_amd/mega_dispatch.hpp>

#include "mock_model.hpp"

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <vector>

using namespace nihilus;

using mtt		 = llama3_8b_traits;
using qkv_core	 = core_traits_old<mock_config, core_types::mega_qkv_prep_and_cache_publish>;
using attn_core	 = core_traits_old<mock_config, core_types::mega_attention_apply>;
using ffn_core	 = core_traits_old<mock_config, core_types::mega_ffn>;
using final_core = core_traits_old<mock_config, core_types::final_norm_and_sampling>;

#define REQUIRE(cond)                                                  \
	do {                                                               \
		if (!(cond)) {                                                 \
			std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
			return 1;                                                  \
		}                                                              \
	} while (0)

static int64_t weight_bytes = 0;

// a tiled Q8_0 weight [n][k] filled by the device generator
static int make_weight(void** tiled, uint64_t seed, int64_t n, int64_t k, void* staging) {
	const int64_t blocks = n * (k / 32);
	REQUIRE(nh_malloc(tiled, nh_q8_0_tiled_bytes(n, k)) == NH_OK);
	REQUIRE(nh_q8_0_fill_weight_blocks(staging, seed, 0, blocks, nullptr) == NH_OK);
	REQUIRE(nh_q8_0_tile(staging, *tiled, n, k, nullptr) == NH_OK);
	REQUIRE(nh_stream_sync(nullptr) == NH_OK);
	weight_bytes += blocks * 34;
	return 0;
}

static int make_norm(void** dev, uint64_t seed, int64_t count) {
	std::vector<float> host(count);
	REQUIRE(nh_malloc(dev, count * 4) == NH_OK);
	REQUIRE(nh_q8_0_fill_activations(static_cast<float*>(*dev), seed, count, nullptr) == NH_OK);
	REQUIRE(nh_memcpy_d2h(host.data(), *dev, count * 4, nullptr) == NH_OK && nh_stream_sync(nullptr) == NH_OK);
	for (float& v : host) {
		v = 1.0f + 0.1f * v;
	}
	REQUIRE(nh_memcpy_h2d(*dev, host.data(), count * 4, nullptr) == NH_OK && nh_stream_sync(nullptr) == NH_OK);
	return 0;
}

int main(int argc, char** argv) {
	const int tokens = argc > 1 ? std::atoi(argv[1]) : 30;
	const int warmup = argc > 2 ? std::atoi(argv[2]) : 3;
	constexpr int64_t E = mtt::embedding_length, KV = mtt::n_embd_kv_gqa, F = mtt::feed_forward_length, V = mtt::vocab_size, B = mtt::block_count;
	REQUIRE(tokens > 0 && warmup >= 0);

	static nihilus_cathedral<mock_config> model;
	auto& weights = static_cast<core_traits_old<mock_config, core_types::weights>&>(model);
	void* staging = nullptr;
	REQUIRE(nh_malloc(&staging, V * (E / 32) * 34) == NH_OK);
	for (int64_t b = 0; b < B; ++b) {
		void *wq, *wk, *wv, *wo, *wg, *wu, *wd, *an, *fn;
		REQUIRE(make_weight(&wq, 1000 + b, E, E, staging) == 0 && make_weight(&wk, 2000 + b, KV, E, staging) == 0 && make_weight(&wv, 3000 + b, KV, E, staging) == 0);
		REQUIRE(make_weight(&wo, 4000 + b, E, E, staging) == 0 && make_weight(&wg, 5000 + b, F, E, staging) == 0 && make_weight(&wu, 6000 + b, F, E, staging) == 0);
		REQUIRE(make_weight(&wd, 7000 + b, E, F, staging) == 0 && make_norm(&an, 8000 + b, E) == 0 && make_norm(&fn, 9000 + b, E) == 0);
		weights.values.get_core<weight_types, weight_types::attn_q>().set_data(wq, b);
		weights.values.get_core<weight_types, weight_types::attn_k>().set_data(wk, b);
		weights.values.get_core<weight_types, weight_types::attn_v>().set_data(wv, b);
		weights.values.get_core<weight_types, weight_types::attn_output>().set_data(wo, b);
		weights.values.get_core<weight_types, weight_types::attn_norm>().set_data(an, b);
		weights.values.get_core<weight_types, weight_types::ffn_gate>().set_data(wg, b);
		weights.values.get_core<weight_types, weight_types::ffn_up>().set_data(wu, b);
		weights.values.get_core<weight_types, weight_types::ffn_down>().set_data(wd, b);
		weights.values.get_core<weight_types, weight_types::ffn_norm>().set_data(fn, b);
	}
	const int64_t ffn_weight_bytes = 3 * F * (E / 32) * 34;
	void *w_out, *on;
	REQUIRE(make_weight(&w_out, 10000, V, E, staging) == 0 && make_norm(&on, 10001, E) == 0);
	weights.values.get_core<weight_types, weight_types::output>().set_data(w_out);
	weights.values.get_core<weight_types, weight_types::output_norm>().set_data(on);
	amd_prepare<mock_config, mtt>(1); // decode only: one row

	void *d_x0, *d_q, *d_ffn_inp, *d_l_out;
	REQUIRE(nh_malloc(&d_x0, E * 4) == NH_OK && nh_malloc(&d_q, E * 4) == NH_OK && nh_malloc(&d_ffn_inp, E * 4) == NH_OK && nh_malloc(&d_l_out, E * 4) == NH_OK);
	REQUIRE(nh_q8_0_fill_activations(static_cast<float*>(d_x0), 7, E, nullptr) == NH_OK);
	static_cast<core_traits_old<mock_config, core_types::token_embeddings>&>(model).values.get_core<token_embeddings_types, token_embeddings_types::get_rows>().set_data(d_x0);
	auto& qkv  = static_cast<qkv_core&>(model);
	auto& attn = static_cast<attn_core&>(model);
	auto& ffn  = static_cast<ffn_core&>(model);
	auto& fin  = static_cast<final_core&>(model);
	qkv.values.get_core<mega_qkv_prep_and_cache_publish_types, mega_qkv_prep_and_cache_publish_types::q_out>().set_data(d_q);
	attn.values.get_core<mega_attention_apply_types, mega_attention_apply_types::ffn_inp>().set_data(d_ffn_inp);
	ffn.values.get_core<mega_ffn_types, mega_ffn_types::l_out>().set_data(d_l_out);
	qkv.values.get_core<mega_qkv_prep_and_cache_publish_types, mega_qkv_prep_and_cache_publish_types::q_out>().get_seq_length_dim() = 1;
	attn.values.get_core<mega_attention_apply_types, mega_attention_apply_types::ffn_inp>().get_seq_length_dim()					= 1;
	ffn.values.get_core<mega_ffn_types, mega_ffn_types::l_out>().get_seq_length_dim()												= 1;
	REQUIRE(nh_q8_0_prepare() == NH_OK);

	constexpr auto phase = processing_phases::eval_time;
	auto token			 = [&] {
		  for (int64_t b = 0; b < B; ++b) {
			  kernel_dispatcher<mock_config, phase, qkv_core>::impl(qkv, b);
			  kernel_dispatcher<mock_config, phase, attn_core>::impl(attn, b);
			  kernel_dispatcher<mock_config, phase, ffn_core>::impl(ffn, b);
		  }
		  kernel_dispatcher<mock_config, phase, final_core>::impl(fin); // waits for the device
	};
	using clock = std::chrono::steady_clock;
	for (int i = 0; i < warmup; ++i) {
		token();
	}
	auto t0 = clock::now();
	for (int i = 0; i < tokens; ++i) {
		token();
	}
	const double token_s = std::chrono::duration<double>(clock::now() - t0).count() / tokens;

	const int ffn_steps = tokens * static_cast<int>(B);
	for (int i = 0; i < 2 * B; ++i) {
		kernel_dispatcher<mock_config, phase, ffn_core>::impl(ffn, i % B);
	}
	REQUIRE(nh_stream_sync(nullptr) == NH_OK);
	t0 = clock::now();
	for (int i = 0; i < ffn_steps; ++i) {
		kernel_dispatcher<mock_config, phase, ffn_core>::impl(ffn, i % B);
	}
	REQUIRE(nh_stream_sync(nullptr) == NH_OK);
	const double ffn_s = std::chrono::duration<double>(clock::now() - t0).count() / ffn_steps;
	REQUIRE(nh_q8_0_last_error() == NH_OK);

	const double ffn_bytes = static_cast<double>(ffn_weight_bytes) + 4.0 * E * 3; // weights once, the fp32 input row, the norm weights, the residual read = the output written
	std::printf("{\"entry\": \"nihilus::kernel_dispatcher<config, eval_time, core>::impl over kernel_dispatcher_impl<..., device_types::gpu, 5, core_types::mega_*, eval_time>\", "
				"\"decode\": {\"tokens\": %d, \"ms_per_token\": %.4f, \"tok_s\": %.1f, \"weight_bytes_per_token\": %lld, \"GBs\": %.1f}, "
				"\"mega_ffn\": {\"steps\": %d, \"us_per_step\": %.3f, \"bytes_per_step\": %.0f, \"GBs\": %.1f}}\n",
		tokens, token_s * 1e3, 1.0 / token_s, static_cast<long long>(weight_bytes), weight_bytes / token_s / 1e9, ffn_steps, ffn_s * 1e6, ffn_bytes, ffn_bytes / ffn_s / 1e9);
	return 0;
}
