// Must NOT compile: a config that neither specialises the three customisation points of mega_dispatch.hpp nor declares
// amd_matmul_only reaches the attention core.  The test suite compiles this file with -fsyntax-only and expects the
// header's static_assert (a model dropped onto the dispatch point without rope, cache write, attention and sampling would
// run and generate garbage).
#include <nihilus_amd/mega_dispatch.hpp>

#define mock_config full_model_config // the mock graph, under a config name of its own ...
#include "mock_model.hpp"
#undef mock_config

namespace nihilus {
	struct real_model_config : full_model_config {
		static constexpr bool amd_matmul_only{ false }; // ... that does not ask for the stand-ins
	};
}

using namespace nihilus;
using attn_core = core_traits_old<full_model_config, core_types::mega_attention_apply>;

void instantiate(attn_core& core) {
	kernel_dispatcher_impl<real_model_config, attn_core, device_types::gpu, gfx950_arch_index, core_types::mega_attention_apply, processing_phases::eval_time>::impl(core, 0);
}
