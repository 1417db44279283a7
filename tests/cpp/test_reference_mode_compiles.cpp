// Compile-only: the dispatch headers in the mode a maintainer of the reference uses (NIHILUS_AMD_WITH_REFERENCE_HEADERS),
// where every reference name comes from elsewhere -- here from reference_decls.hpp, whose primary template is the reference's
// own declaration of the live specialisation point (common/kernel_traits.hpp:382-383) -- and reference_mirror.hpp is never
// seen.  Instantiates all eight specialisations (four cores x two phases) through the reference's caller-side template, so
// their bodies compile against that declaration; nothing runs on a GPU.
#define NIHILUS_AMD_WITH_REFERENCE_HEADERS
#include "reference_decls.hpp"

#include <nihilus_amd/mega_dispatch.hpp>

#include "mock_model.hpp"

#include <cstdio>

using namespace nihilus;

using qkv_core	 = core_traits_old<mock_config, core_types::mega_qkv_prep_and_cache_publish>;
using attn_core	 = core_traits_old<mock_config, core_types::mega_attention_apply>;
using ffn_core	 = core_traits_old<mock_config, core_types::mega_ffn>;
using final_core = core_traits_old<mock_config, core_types::final_norm_and_sampling>;

template<processing_phases phase> static const void* entry_points() {
	static void (*const per_block[])(qkv_core&, int64_t) = { &kernel_dispatcher<mock_config, phase, qkv_core>::impl };
	static void (*const attn)(attn_core&, int64_t)		 = &kernel_dispatcher<mock_config, phase, attn_core>::impl;
	static void (*const ffn)(ffn_core&, int64_t)		 = &kernel_dispatcher<mock_config, phase, ffn_core>::impl;
	static void (*const fin)(final_core&)				 = &kernel_dispatcher<mock_config, phase, final_core>::impl;
	return per_block[0] && attn && ffn && fin ? static_cast<const void*>(per_block) : nullptr;
}

int main() {
	const bool ok = entry_points<processing_phases::eval_time>() && entry_points<processing_phases::prompt_eval_time>();
	std::printf(ok ? "reference-mode build ok\n" : "missing entry point\n");
	return ok ? 0 : 1;
}
