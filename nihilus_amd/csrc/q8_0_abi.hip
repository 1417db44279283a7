// extern "C" surface of the gfx950 Q8_0 library: argument checks, then the launch functions.
// Nothing here computes; every rejected argument returns a negative nh_status before any launch, so a
// malformed call can never reach a kernel with shapes the kernel does not expect.
#include "../../include/nihilus_amd/q8_0_abi.h"
#include "q8_0_plan.h"

#include <cstdlib>
#include <cstring>

namespace {

constexpr int64_t MAX_ROWS = int64_t{ 1 } << 30; // row and strip indices are 32-bit inside the kernels
constexpr int64_t MAX_BLOCKS = int64_t{ 1 } << 35; // blocks per matrix the element-wise kernels can index
constexpr int64_t MAX_K	   = int64_t{ 1 } << 24; // block and group indices along K are 32-bit
constexpr int64_t MAX_K_BLOCKS_GEMV = 49152; // the blocks-layout mat-vec keeps the whole activation row (K + K/8 bytes) in 64 KiB of LDS

inline bool aligned16(const void* p) {
	return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}
inline hipStream_t as_stream(void* s) {
	return static_cast<hipStream_t>(s);
}
inline int from_hip(hipError_t e) {
	if (e == hipErrorNotReady) {
		return NH_ERR_BUSY; // the only source: the per-device scratch is still in use by a launch on another stream
	}
	return e == hipSuccess ? NH_OK : static_cast<int>(e);
}

// Common shape checks: sizes non-negative, K a whole number of blocks (of groups for a tiled operand).
inline int check_shape(int64_t rows_a, int64_t rows_b, int64_t K, bool tiled) {
	if (rows_a < 0 || rows_b < 0 || K < 0) {
		return NH_ERR_SHAPE;
	}
	if (K % NH_Q8_0_QK != 0 || (tiled && K % nh::GROUP_K != 0)) {
		return NH_ERR_SHAPE;
	}
	if (rows_a > MAX_ROWS || rows_b > MAX_ROWS || K > MAX_K) {
		return NH_ERR_TOO_LARGE;
	}
	if (rows_a * (K / NH_Q8_0_QK) > MAX_BLOCKS || rows_b * (K / NH_Q8_0_QK) > MAX_BLOCKS) {
		return NH_ERR_TOO_LARGE; // one thread per four quants, 256 per workgroup, 2^31 workgroups at most
	}
	return NH_OK;
}

// First call on a thread: make sure a gfx950 device is current.  Returns NH_OK or NH_ERR_NO_DEVICE.
int require_device() {
	static thread_local int cached = 1; // 1 = not checked yet
	if (cached != 1) {
		return cached;
	}
	int count = 0;
	if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
		(void)hipGetLastError();
		return cached = NH_ERR_NO_DEVICE;
	}
	int dev = 0;
	hipDeviceProp_t prop;
	if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) {
		(void)hipGetLastError();
		return cached = NH_ERR_NO_DEVICE;
	}
	if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
		return cached = NH_ERR_NO_DEVICE; // the code object holds gfx950 ISA only
	}
	return cached = NH_OK;
}

} // namespace

#define NH_REQUIRE(cond, code) \
	do {                       \
		if (!(cond)) {         \
			return (code);     \
		}                      \
	} while (0)
#define NH_TRY(expr)        \
	do {                    \
		const int rc_ = (expr); \
		if (rc_ != NH_OK) { \
			return rc_;     \
		}                   \
	} while (0)

extern "C" {

const char* nh_status_string(int status) {
	switch (status) {
		case NH_OK:
			return "ok";
		case NH_ERR_NULL_POINTER:
			return "null pointer";
		case NH_ERR_ALIGNMENT:
			return "pointer not 16-byte aligned";
		case NH_ERR_SHAPE:
			return "bad shape (negative size, K not a multiple of 32, or of 128 for a tiled operand)";
		case NH_ERR_NO_DEVICE:
			return "no gfx950 device";
		case NH_ERR_TOO_LARGE:
			return "dimension too large";
		case NH_ERR_ARGUMENT:
			return "invalid argument";
		case NH_ERR_IO:
			return "file could not be opened or mapped";
		case NH_ERR_FORMAT:
			return "file format not accepted";
		case NH_ERR_NOT_FOUND:
			return "name not found";
		case NH_ERR_BUSY:
			return "the library's per-device scratch is still in use by a launch on another stream";
		case NH_ERR_DEVICE_TIMEOUT:
			return "a kernel gave up a bounded wait for data from another workgroup (its output holds NaN)";
		default:
			return status > 0 ? hipGetErrorString(static_cast<hipError_t>(status)) : "unknown status";
	}
}

int nh_abi_version(void) {
	return 1;
}

int nh_device_info(char* host_name, int64_t cap, int64_t* host_compute_units, int64_t* host_total_bytes) {
	NH_TRY(require_device());
	int dev = 0;
	hipDeviceProp_t prop;
	NH_TRY(from_hip(hipGetDevice(&dev)));
	NH_TRY(from_hip(hipGetDeviceProperties(&prop, dev)));
	if (host_name && cap > 0) {
		std::strncpy(host_name, prop.gcnArchName, static_cast<size_t>(cap - 1));
		host_name[cap - 1] = '\0';
	}
	if (host_compute_units) {
		*host_compute_units = prop.multiProcessorCount;
	}
	if (host_total_bytes) {
		*host_total_bytes = static_cast<int64_t>(prop.totalGlobalMem);
	}
	return NH_OK;
}

int nh_malloc(void** host_out_dev_ptr, int64_t bytes) {
	NH_REQUIRE(host_out_dev_ptr, NH_ERR_NULL_POINTER);
	NH_REQUIRE(bytes >= 0, NH_ERR_SHAPE);
	NH_TRY(require_device());
	*host_out_dev_ptr = nullptr;
	if (bytes == 0) {
		return NH_OK;
	}
	return from_hip(hipMalloc(host_out_dev_ptr, static_cast<size_t>(bytes)));
}

int nh_free(void* dev_ptr) {
	if (!dev_ptr) {
		return NH_OK;
	}
	return from_hip(hipFree(dev_ptr));
}

int nh_memcpy_h2d(void* dst_dev, const void* host_src, int64_t bytes, void* stream) {
	NH_REQUIRE(bytes >= 0, NH_ERR_SHAPE);
	if (bytes == 0) {
		return NH_OK;
	}
	NH_REQUIRE(dst_dev && host_src, NH_ERR_NULL_POINTER);
	NH_TRY(require_device());
	return from_hip(hipMemcpyAsync(dst_dev, host_src, static_cast<size_t>(bytes), hipMemcpyHostToDevice, as_stream(stream)));
}

int nh_memcpy_d2h(void* host_dst, const void* src_dev, int64_t bytes, void* stream) {
	NH_REQUIRE(bytes >= 0, NH_ERR_SHAPE);
	if (bytes == 0) {
		return NH_OK;
	}
	NH_REQUIRE(host_dst && src_dev, NH_ERR_NULL_POINTER);
	NH_TRY(require_device());
	return from_hip(hipMemcpyAsync(host_dst, src_dev, static_cast<size_t>(bytes), hipMemcpyDeviceToHost, as_stream(stream)));
}

int nh_memset(void* dst_dev, int value, int64_t bytes, void* stream) {
	NH_REQUIRE(bytes >= 0, NH_ERR_SHAPE);
	if (bytes == 0) {
		return NH_OK;
	}
	NH_REQUIRE(dst_dev, NH_ERR_NULL_POINTER);
	NH_TRY(require_device());
	return from_hip(hipMemsetAsync(dst_dev, value, static_cast<size_t>(bytes), as_stream(stream)));
}

int nh_stream_sync(void* stream) {
	NH_TRY(require_device());
	NH_TRY(from_hip(hipStreamSynchronize(as_stream(stream))));
	return nh::read_device_error(false) != nh::DEVICE_ERROR_NONE ? NH_ERR_DEVICE_TIMEOUT : NH_OK;
}

int nh_q8_0_last_error(void) {
	NH_TRY(require_device());
	return nh::read_device_error(false) != nh::DEVICE_ERROR_NONE ? NH_ERR_DEVICE_TIMEOUT : NH_OK;
}

int nh_q8_0_clear_error(void) {
	NH_TRY(require_device());
	return nh::read_device_error(true) != nh::DEVICE_ERROR_NONE ? NH_ERR_DEVICE_TIMEOUT : NH_OK;
}

int nh_q8_0_set_in_kernel_waits(int enabled) {
	return nh::set_in_kernel_waits(enabled != 0) ? 1 : 0;
}

int nh_q8_0_debug_set_spin_limit(int64_t polls) {
	// a test hook in a production library: it only works for a process that asked for it
	const char* hooks = std::getenv("NH_Q8_0_DEBUG_HOOKS");
	NH_REQUIRE(hooks && hooks[0] == '1' && hooks[1] == '\0', NH_ERR_ARGUMENT);
	NH_REQUIRE(polls >= 1, NH_ERR_ARGUMENT);
	nh::set_published_spin_limit(polls > nh::PUBLISHED_SPIN_LIMIT ? nh::PUBLISHED_SPIN_LIMIT : static_cast<int>(polls));
	return NH_OK;
}

int64_t nh_q8_0_blocks_bytes(int64_t rows, int64_t K) {
	if (rows < 0 || K < 0 || K % NH_Q8_0_QK != 0) {
		return NH_ERR_SHAPE;
	}
	return rows * (K / NH_Q8_0_QK) * NH_Q8_0_BLOCK_BYTES;
}

int64_t nh_q8_0_tiled_bytes(int64_t rows, int64_t K) {
	if (rows < 0 || K < 0 || K % nh::GROUP_K != 0) {
		return NH_ERR_SHAPE;
	}
	return (rows + nh::STRIP_ROWS - 1) / nh::STRIP_ROWS * (K / nh::GROUP_K) * nh::MACRO_BYTES;
}

int nh_q8_0_quantize(const float* x, void* xq_blocks, int64_t M, int64_t K, void* stream) {
	NH_TRY(check_shape(M, 0, K, false));
	if (M == 0 || K == 0) {
		return NH_OK;
	}
	NH_REQUIRE(x && xq_blocks, NH_ERR_NULL_POINTER);
	NH_REQUIRE(aligned16(x) && aligned16(xq_blocks), NH_ERR_ALIGNMENT);
	NH_TRY(require_device());
	return from_hip(nh::launch_quantize(x, xq_blocks, M, K, false, as_stream(stream)));
}

int nh_q8_0_quantize_tiled(const float* x, void* xq_tiled, int64_t M, int64_t K, void* stream) {
	NH_TRY(check_shape(M, 0, K, true));
	if (M == 0 || K == 0) {
		return NH_OK;
	}
	NH_REQUIRE(x && xq_tiled, NH_ERR_NULL_POINTER);
	NH_REQUIRE(aligned16(x) && aligned16(xq_tiled), NH_ERR_ALIGNMENT);
	NH_TRY(require_device());
	return from_hip(nh::launch_quantize(x, xq_tiled, M, K, true, as_stream(stream)));
}

static int silu_mul_quantize_common(const float* gate, const float* up, void* xq, int64_t M, int64_t K, bool tiled, void* stream) {
	NH_TRY(check_shape(M, 0, K, tiled));
	if (M == 0 || K == 0) {
		return NH_OK;
	}
	NH_REQUIRE(gate && up && xq, NH_ERR_NULL_POINTER);
	NH_REQUIRE(aligned16(gate) && aligned16(up) && aligned16(xq), NH_ERR_ALIGNMENT);
	NH_TRY(require_device());
	return from_hip(nh::launch_silu_mul_quantize(gate, up, xq, M, K, tiled, as_stream(stream)));
}

int nh_q8_0_silu_mul_quantize(const float* gate, const float* up, void* xq_blocks, int64_t M, int64_t K, void* stream) {
	return silu_mul_quantize_common(gate, up, xq_blocks, M, K, false, stream);
}

int nh_q8_0_silu_mul_quantize_tiled(const float* gate, const float* up, void* xq_tiled, int64_t M, int64_t K, void* stream) {
	return silu_mul_quantize_common(gate, up, xq_tiled, M, K, true, stream);
}

int nh_q8_0_tile(const void* blocks, void* tiled, int64_t rows, int64_t K, void* stream) {
	NH_TRY(check_shape(rows, 0, K, true));
	if (rows == 0 || K == 0) {
		return NH_OK;
	}
	NH_REQUIRE(blocks && tiled, NH_ERR_NULL_POINTER);
	NH_REQUIRE(aligned16(blocks) && aligned16(tiled), NH_ERR_ALIGNMENT);
	NH_REQUIRE(blocks != tiled, NH_ERR_ARGUMENT);
	NH_TRY(require_device());
	return from_hip(nh::launch_tile(blocks, tiled, rows, K, as_stream(stream)));
}

int nh_q8_0_untile(const void* tiled, void* blocks, int64_t rows, int64_t K, void* stream) {
	NH_TRY(check_shape(rows, 0, K, true));
	if (rows == 0 || K == 0) {
		return NH_OK;
	}
	NH_REQUIRE(blocks && tiled, NH_ERR_NULL_POINTER);
	NH_REQUIRE(aligned16(blocks) && aligned16(tiled), NH_ERR_ALIGNMENT);
	NH_REQUIRE(blocks != tiled, NH_ERR_ARGUMENT);
	NH_TRY(require_device());
	return from_hip(nh::launch_untile(tiled, blocks, rows, K, as_stream(stream)));
}

static int get_rows_common(const void* W, const int32_t* ids, float* out, int32_t* invalid_count, int64_t n_tokens, int64_t n_rows, int64_t K, bool tiled, void* stream) {
	NH_TRY(check_shape(n_rows, n_tokens, K, tiled));
	if (n_tokens == 0 || K == 0) {
		return NH_OK;
	}
	NH_REQUIRE(ids && out && (W || n_rows == 0), NH_ERR_NULL_POINTER);
	NH_REQUIRE(aligned16(W) && aligned16(out) && reinterpret_cast<uintptr_t>(ids) % 4 == 0 && reinterpret_cast<uintptr_t>(invalid_count) % 4 == 0, NH_ERR_ALIGNMENT);
	NH_TRY(require_device());
	return from_hip(nh::launch_get_rows(W, ids, out, invalid_count, n_tokens, n_rows, K, tiled, as_stream(stream)));
}

int nh_q8_0_get_rows(const void* W_blocks, const int32_t* ids, float* out, int32_t* invalid_count, int64_t n_tokens, int64_t n_rows, int64_t K, void* stream) {
	return get_rows_common(W_blocks, ids, out, invalid_count, n_tokens, n_rows, K, false, stream);
}

int nh_q8_0_get_rows_tiled(const void* W_tiled, const int32_t* ids, float* out, int32_t* invalid_count, int64_t n_tokens, int64_t n_rows, int64_t K, void* stream) {
	return get_rows_common(W_tiled, ids, out, invalid_count, n_tokens, n_rows, K, true, stream);
}

int nh_q8_0_ffn_f32(const void* W_gate_tiled, const void* W_up_tiled, const void* W_down_tiled, const float* x, const float* norm_weight, float eps, const float* residual, float* y,
	int64_t N_ff, int64_t K, int64_t N_out, void* stream) {
	NH_TRY(check_shape(N_ff, 0, K, true)); // gate, up: [N_ff x K]
	NH_TRY(check_shape(N_out, 0, N_ff, true)); // down: [N_out x N_ff]
	NH_REQUIRE(N_ff <= NH_Q8_0_FFN_MAX_HIDDEN, NH_ERR_TOO_LARGE);
	if (N_out == 0) {
		return NH_OK;
	}
	NH_REQUIRE(y, NH_ERR_NULL_POINTER);
	NH_REQUIRE(aligned16(y) && aligned16(residual) && aligned16(norm_weight), NH_ERR_ALIGNMENT);
	NH_REQUIRE(!norm_weight || (eps >= 0.0f && eps < 1.0f), NH_ERR_ARGUMENT);
	if (N_ff > 0 && K > 0) {
		NH_REQUIRE(W_gate_tiled && W_up_tiled && W_down_tiled && x, NH_ERR_NULL_POINTER);
		NH_REQUIRE(aligned16(W_gate_tiled) && aligned16(W_up_tiled) && aligned16(W_down_tiled) && aligned16(x), NH_ERR_ALIGNMENT);
	}
	NH_TRY(require_device());
	return from_hip(nh::launch_ffn_decode(W_gate_tiled, W_up_tiled, W_down_tiled, x, norm_weight, eps, residual, y, N_ff, K, N_out, as_stream(stream)));
}

int nh_q8_0_decode_layer_f32(const void* W_o_tiled, const float* attn, const float* layer_in, float* ffn_inp, const void* W_gate_tiled, const void* W_up_tiled, const void* W_down_tiled,
	const float* ffn_norm_weight, float* l_out, const void* const* host_W_next_tiled, float* const* host_y_next, const int64_t* host_N_next, int64_t count_next, const float* next_norm_weight,
	float eps, int64_t N_embd, int64_t N_ff, void* stream) {
	NH_TRY(check_shape(N_embd, 0, N_embd, true)); // attn_out: [N_embd x N_embd]; gate, up: [N_ff x N_embd]
	NH_TRY(check_shape(N_embd, 0, N_ff, true)); // down: [N_embd x N_ff]
	NH_REQUIRE(N_embd > 0 && N_ff > 0, NH_ERR_SHAPE);
	NH_REQUIRE(N_ff <= NH_Q8_0_FFN_MAX_HIDDEN, NH_ERR_TOO_LARGE);
	NH_REQUIRE(count_next >= 0 && count_next <= nh::GEMV_MAX_SEGMENTS, NH_ERR_ARGUMENT);
	NH_REQUIRE(W_o_tiled && attn && layer_in && ffn_inp && W_gate_tiled && W_up_tiled && W_down_tiled && ffn_norm_weight && l_out, NH_ERR_NULL_POINTER);
	NH_REQUIRE(aligned16(W_o_tiled) && aligned16(attn) && aligned16(layer_in) && aligned16(ffn_inp) && aligned16(W_gate_tiled) && aligned16(W_up_tiled) && aligned16(W_down_tiled) &&
				   aligned16(ffn_norm_weight) && aligned16(l_out),
		NH_ERR_ALIGNMENT);
	NH_REQUIRE(eps >= 0.0f && eps < 1.0f, NH_ERR_ARGUMENT);
	// ffn_inp and l_out are written by workgroups of different stages: as one buffer, which store lands last would be undefined
	NH_REQUIRE(ffn_inp != l_out && attn != ffn_inp && attn != l_out, NH_ERR_ARGUMENT);
	int64_t rows = 0;
	if (count_next > 0) {
		NH_REQUIRE(host_W_next_tiled && host_y_next && host_N_next && next_norm_weight, NH_ERR_NULL_POINTER);
		NH_REQUIRE(aligned16(next_norm_weight), NH_ERR_ALIGNMENT);
		for (int64_t i = 0; i < count_next; ++i) {
			NH_REQUIRE(host_N_next[i] >= 0, NH_ERR_SHAPE);
			if (host_N_next[i] > 0) {
				NH_REQUIRE(host_W_next_tiled[i] && host_y_next[i], NH_ERR_NULL_POINTER);
				NH_REQUIRE(aligned16(host_W_next_tiled[i]) && aligned16(host_y_next[i]), NH_ERR_ALIGNMENT);
				NH_REQUIRE(host_y_next[i] != ffn_inp && host_y_next[i] != l_out, NH_ERR_ARGUMENT);
			}
			rows += host_N_next[i];
		}
		NH_REQUIRE(rows <= MAX_ROWS, NH_ERR_TOO_LARGE);
	}
	NH_TRY(require_device());
	return from_hip(nh::launch_decode_layer(W_o_tiled, attn, layer_in, ffn_inp, W_gate_tiled, W_up_tiled, W_down_tiled, ffn_norm_weight, l_out, host_W_next_tiled, host_y_next, host_N_next,
		rows > 0 ? static_cast<int>(count_next) : 0, next_norm_weight, eps, N_embd, N_ff, as_stream(stream)));
}

int nh_q8_0_debug_ffn_gate_up(float* gate_out, float* up_out, int64_t N_ff, void* stream) {
	NH_REQUIRE(N_ff >= 0, NH_ERR_SHAPE);
	NH_REQUIRE(N_ff <= NH_Q8_0_FFN_MAX_HIDDEN, NH_ERR_TOO_LARGE);
	if (N_ff == 0) {
		return NH_OK;
	}
	NH_REQUIRE(gate_out && up_out, NH_ERR_NULL_POINTER);
	NH_TRY(require_device());
	return from_hip(nh::copy_ffn_gate_up(gate_out, up_out, N_ff, as_stream(stream)));
}

static int gemv_common(const void* W, const void* xq, float* y, int64_t N, int64_t K, bool tiled, void* stream) {
	NH_TRY(check_shape(N, 0, K, tiled));
	NH_REQUIRE(tiled || K <= MAX_K_BLOCKS_GEMV, NH_ERR_TOO_LARGE);
	if (N == 0) {
		return NH_OK;
	}
	NH_REQUIRE(y, NH_ERR_NULL_POINTER);
	NH_REQUIRE(aligned16(y), NH_ERR_ALIGNMENT);
	if (K > 0) {
		NH_REQUIRE(W && xq, NH_ERR_NULL_POINTER);
		NH_REQUIRE(aligned16(W) && aligned16(xq), NH_ERR_ALIGNMENT);
	}
	NH_TRY(require_device());
	return from_hip(nh::launch_gemv(W, xq, y, nullptr, N, K, tiled, as_stream(stream)));
}

int nh_q8_0_gemv(const void* W_blocks, const void* xq_blocks, float* y, int64_t N, int64_t K, void* stream) {
	return gemv_common(W_blocks, xq_blocks, y, N, K, false, stream);
}

int nh_q8_0_gemv_tiled(const void* W_tiled, const void* xq_blocks, float* y, int64_t N, int64_t K, void* stream) {
	return gemv_common(W_tiled, xq_blocks, y, N, K, true, stream);
}

static int gemv_multi_common(const void* const* host_W_tiled, float* const* host_y, const int64_t* host_N, int64_t count, const float* x, const float* norm_weight, float eps, int64_t K,
	void* stream, const float* const* host_residual = nullptr) {
	NH_REQUIRE(count >= 0 && count <= nh::GEMV_MAX_SEGMENTS, NH_ERR_ARGUMENT);
	if (count == 0) {
		return NH_OK;
	}
	NH_REQUIRE(host_W_tiled && host_y && host_N, NH_ERR_NULL_POINTER);
	int64_t rows = 0;
	for (int64_t i = 0; i < count; ++i) {
		NH_TRY(check_shape(host_N[i], 0, K, true));
		rows += host_N[i];
	}
	NH_REQUIRE(rows <= MAX_ROWS, NH_ERR_TOO_LARGE);
	if (rows == 0) {
		return NH_OK;
	}
	for (int64_t i = 0; i < count; ++i) {
		if (host_N[i] == 0) {
			continue;
		}
		NH_REQUIRE(host_y[i], NH_ERR_NULL_POINTER);
		NH_REQUIRE(aligned16(host_y[i]), NH_ERR_ALIGNMENT);
		NH_REQUIRE(!host_residual || aligned16(host_residual[i]), NH_ERR_ALIGNMENT);
		if (K > 0) {
			NH_REQUIRE(host_W_tiled[i], NH_ERR_NULL_POINTER);
			NH_REQUIRE(aligned16(host_W_tiled[i]), NH_ERR_ALIGNMENT);
		}
	}
	if (K > 0) {
		NH_REQUIRE(x, NH_ERR_NULL_POINTER);
		NH_REQUIRE(aligned16(x), NH_ERR_ALIGNMENT);
	}
	NH_REQUIRE(aligned16(norm_weight), NH_ERR_ALIGNMENT);
	NH_REQUIRE(!norm_weight || (eps >= 0.0f && eps < 1.0f), NH_ERR_ARGUMENT);
	NH_TRY(require_device());
	return from_hip(nh::launch_gemv_tiled_multi(host_W_tiled, host_y, host_N, static_cast<int>(count), x, true, K, as_stream(stream), norm_weight, eps, host_residual));
}

int nh_q8_0_gemv_tiled_multi_f32(const void* const* host_W_tiled, float* const* host_y, const int64_t* host_N, int64_t count, const float* x, int64_t K, void* stream) {
	return gemv_multi_common(host_W_tiled, host_y, host_N, count, x, nullptr, 0.0f, K, stream);
}

int nh_q8_0_gemv_tiled_multi_norm_f32(const void* const* host_W_tiled, float* const* host_y, const int64_t* host_N, int64_t count, const float* x, const float* norm_weight, float eps,
	int64_t K, void* stream) {
	NH_REQUIRE(norm_weight || K == 0 || count == 0, NH_ERR_NULL_POINTER);
	return gemv_multi_common(host_W_tiled, host_y, host_N, count, x, norm_weight, eps, K, stream);
}

int nh_q8_0_gemv_tiled_group_f32(const void* const* host_W_tiled, const float* const* host_x, float* const* host_y, const float* const* host_residual, const int64_t* host_N,
	const int64_t* host_K, int64_t count, void* stream) {
	NH_REQUIRE(count >= 0, NH_ERR_ARGUMENT);
	if (count == 0) {
		return NH_OK;
	}
	NH_REQUIRE(host_W_tiled && host_x && host_y && host_N && host_K, NH_ERR_NULL_POINTER);
	// everything is checked before the first launch, so a bad entry cannot leave half the list enqueued
	bool any = false;
	for (int64_t i = 0; i < count; ++i) {
		NH_TRY(check_shape(host_N[i], 0, host_K[i], true));
		if (host_N[i] == 0) {
			continue;
		}
		any = true;
		NH_REQUIRE(host_y[i], NH_ERR_NULL_POINTER);
		NH_REQUIRE(aligned16(host_y[i]) && (!host_residual || aligned16(host_residual[i])), NH_ERR_ALIGNMENT);
		if (host_K[i] > 0) {
			NH_REQUIRE(host_W_tiled[i] && host_x[i], NH_ERR_NULL_POINTER);
			NH_REQUIRE(aligned16(host_W_tiled[i]) && aligned16(host_x[i]), NH_ERR_ALIGNMENT);
		}
	}
	if (!any) {
		return NH_OK;
	}
	NH_TRY(require_device());
	constexpr int CHUNK = 64; // a multiple of the group size: chunk borders fall on group borders
	nh::gemv_group_op ops[CHUNK];
	int n = 0;
	for (int64_t i = 0; i < count; ++i) {
		if (host_N[i] > 0) {
			ops[n++] = { host_W_tiled[i], host_x[i], host_y[i], host_residual ? host_residual[i] : nullptr, host_N[i], host_K[i] };
		}
		if (n == CHUNK || (i + 1 == count && n > 0)) {
			NH_TRY(from_hip(nh::launch_gemv_independent(ops, n, as_stream(stream))));
			n = 0;
		}
	}
	return NH_OK;
}

int nh_q8_0_mul_mat_f32_activations(const void* W_tiled, const float* x, float* y, int64_t M, int64_t N, int64_t K, void* stream) {
	NH_TRY(check_shape(M, N, K, true));
	if (M == 0 || N == 0) {
		return NH_OK;
	}
	NH_REQUIRE(y && (K == 0 || (W_tiled && x)), NH_ERR_NULL_POINTER);
	NH_REQUIRE(aligned16(W_tiled) && aligned16(x) && aligned16(y), NH_ERR_ALIGNMENT);
	NH_REQUIRE(M * N <= MAX_BLOCKS, NH_ERR_TOO_LARGE);
	NH_TRY(require_device());
	return from_hip(nh::launch_mul_mat_f32act(W_tiled, x, y, M, N, K, as_stream(stream)));
}

int nh_q8_0_prepare(void) {
	NH_TRY(require_device());
	const hipError_t e = nh::prepare_gemv_scratch();
	return from_hip(e != hipSuccess ? e : nh::prepare_gemm_scratch());
}

int nh_q8_0_gemv_tiled_residual_f32(const void* W_tiled, const float* x, const float* residual, float* y, int64_t N, int64_t K, void* stream) {
	NH_REQUIRE(residual || N == 0, NH_ERR_NULL_POINTER);
	return gemv_multi_common(&W_tiled, &y, &N, 1, x, nullptr, 0.0f, K, stream, &residual);
}

int nh_q8_0_gemv_tiled_f32(const void* W_tiled, const float* x, float* y, int64_t N, int64_t K, void* stream) {
	return nh_q8_0_gemv_tiled_multi_f32(&W_tiled, &y, &N, 1, x, K, stream);
}

int nh_q8_0_gemv_tiled_f32_noalloc(const void* W_tiled, const float* x, float* y, int64_t N, int64_t K, void* stream) {
	NH_TRY(check_shape(N, 0, K, true));
	if (N == 0) {
		return NH_OK;
	}
	NH_REQUIRE(y, NH_ERR_NULL_POINTER);
	NH_REQUIRE(aligned16(y), NH_ERR_ALIGNMENT);
	if (K > 0) {
		NH_REQUIRE(W_tiled && x, NH_ERR_NULL_POINTER);
		NH_REQUIRE(aligned16(W_tiled) && aligned16(x), NH_ERR_ALIGNMENT);
		NH_REQUIRE(nh::gemv_noalloc_fits(N, K), NH_ERR_TOO_LARGE); // the K split's partial sums would not fit the built-in array
	}
	NH_TRY(require_device());
	return from_hip(nh::launch_gemv_tiled_f32_noalloc(W_tiled, x, y, N, K, as_stream(stream)));
}

int nh_q8_0_debug_fused_norm_quantize(const float* x, const float* norm_weight, float eps, void* xq_blocks_out, int64_t K, void* stream) {
	NH_TRY(check_shape(1, 0, K, true));
	if (K == 0) {
		return NH_OK;
	}
	NH_REQUIRE(x && xq_blocks_out, NH_ERR_NULL_POINTER);
	NH_REQUIRE(aligned16(x) && aligned16(xq_blocks_out) && aligned16(norm_weight), NH_ERR_ALIGNMENT);
	NH_TRY(require_device());
	return from_hip(nh::launch_gemv_dump_staged_x(x, xq_blocks_out, K, as_stream(stream), norm_weight, eps));
}

int nh_q8_0_debug_fused_quantize(const float* x, void* xq_blocks_out, int64_t K, void* stream) {
	return nh_q8_0_debug_fused_norm_quantize(x, nullptr, 0.0f, xq_blocks_out, K, stream);
}

static int rms_norm_quantize_common(const float* x, const float* norm_weight, float eps, void* xq, int64_t M, int64_t K, bool tiled, void* stream) {
	NH_TRY(check_shape(M, 0, K, true)); // the fixed order of the sum of squares is defined on 128-value groups, whatever the output layout
	if (M == 0 || K == 0) {
		return NH_OK;
	}
	NH_REQUIRE(x && norm_weight && xq, NH_ERR_NULL_POINTER);
	NH_REQUIRE(aligned16(x) && aligned16(norm_weight) && aligned16(xq), NH_ERR_ALIGNMENT);
	NH_REQUIRE(eps >= 0.0f && eps < 1.0f, NH_ERR_ARGUMENT);
	NH_TRY(require_device());
	return from_hip(nh::launch_rms_norm_quantize(x, norm_weight, eps, xq, M, K, tiled, as_stream(stream)));
}

int nh_q8_0_rms_norm_quantize(const float* x, const float* norm_weight, float eps, void* xq_blocks, int64_t M, int64_t K, void* stream) {
	return rms_norm_quantize_common(x, norm_weight, eps, xq_blocks, M, K, false, stream);
}

int nh_q8_0_rms_norm_quantize_tiled(const float* x, const float* norm_weight, float eps, void* xq_tiled, int64_t M, int64_t K, void* stream) {
	return rms_norm_quantize_common(x, norm_weight, eps, xq_tiled, M, K, true, stream);
}

static int gemm_common(const void* W, const void* A, float* C, int64_t M, int64_t N, int64_t K, bool tiled, void* stream, const float* residual = nullptr) {
	NH_TRY(check_shape(M, N, K, tiled));
	if (M == 0 || N == 0) {
		return NH_OK;
	}
	// grid.y of the kernel that will run: the MFMA tile kernel covers 64 rows per workgroup row (two 32-row strips), the streaming
	// kernel 32 or 64, the kernel on packed blocks 128
	NH_REQUIRE(M <= 65535 * (tiled ? 32 : 128), NH_ERR_TOO_LARGE);
	NH_REQUIRE(C, NH_ERR_NULL_POINTER);
	NH_REQUIRE(aligned16(C) && aligned16(residual), NH_ERR_ALIGNMENT);
	if (K > 0) {
		NH_REQUIRE(W && A, NH_ERR_NULL_POINTER);
		NH_REQUIRE(aligned16(W) && aligned16(A), NH_ERR_ALIGNMENT);
	}
	NH_TRY(require_device());
	return from_hip(nh::launch_gemm(W, A, C, nullptr, M, N, K, tiled, as_stream(stream), residual));
}

int nh_q8_0_gemm(const void* W_blocks, const void* Aq_blocks, float* C, int64_t M, int64_t N, int64_t K, void* stream) {
	return gemm_common(W_blocks, Aq_blocks, C, M, N, K, false, stream);
}

int nh_q8_0_gemm_tiled(const void* W_tiled, const void* Aq_tiled, float* C, int64_t M, int64_t N, int64_t K, void* stream) {
	return gemm_common(W_tiled, Aq_tiled, C, M, N, K, true, stream);
}

int nh_q8_0_gemm_tiled_residual(const void* W_tiled, const void* Aq_tiled, const float* residual, float* C, int64_t M, int64_t N, int64_t K, void* stream) {
	NH_REQUIRE(residual || M == 0 || N == 0, NH_ERR_NULL_POINTER);
	return gemm_common(W_tiled, Aq_tiled, C, M, N, K, true, stream, residual);
}

int64_t nh_q8_0_gate_up_silu_workspace_bytes(int64_t M, int64_t N_ff, int64_t K) {
	if (M < 0 || N_ff < 0 || K < 0 || K % nh::GROUP_K != 0 || N_ff % nh::GROUP_K != 0) {
		return NH_ERR_SHAPE;
	}
	if (M == 0 || N_ff == 0 || nh::plan_gate_up_fused(M, N_ff, K)) {
		return 0;
	}
	return 2 * M * N_ff * 4;
}

static int gate_up_silu_common(const void* W_gate, const void* W_up, const void* Aq, void* act_out, float* gate_out, float* up_out, void* workspace, int64_t workspace_bytes, int64_t M,
	int64_t N_ff, int64_t K, void* stream) {
	NH_TRY(check_shape(M, N_ff, K, true));
	NH_REQUIRE(N_ff % nh::GROUP_K == 0, NH_ERR_SHAPE); // the output is a tiled operand with N_ff as its inner dimension
	NH_REQUIRE(M <= 65535 * 32, NH_ERR_TOO_LARGE);
	if (M == 0 || N_ff == 0) {
		return NH_OK;
	}
	NH_REQUIRE(act_out, NH_ERR_NULL_POINTER);
	NH_REQUIRE(aligned16(act_out) && aligned16(gate_out) && aligned16(up_out) && aligned16(workspace), NH_ERR_ALIGNMENT);
	if (K > 0) {
		NH_REQUIRE(W_gate && W_up && Aq, NH_ERR_NULL_POINTER);
		NH_REQUIRE(aligned16(W_gate) && aligned16(W_up) && aligned16(Aq), NH_ERR_ALIGNMENT);
	}
	const int64_t need = (gate_out && up_out) ? 0 : nh_q8_0_gate_up_silu_workspace_bytes(M, N_ff, K);
	NH_REQUIRE(workspace_bytes >= need, NH_ERR_ARGUMENT);
	NH_REQUIRE(need == 0 || workspace, NH_ERR_NULL_POINTER);
	NH_TRY(require_device());
	return from_hip(nh::launch_gemm_gate_up_silu(W_gate, W_up, Aq, act_out, gate_out, up_out, static_cast<float*>(workspace), M, N_ff, K, as_stream(stream)));
}

int nh_q8_0_gemm_tiled_gate_up_silu(const void* W_gate_tiled, const void* W_up_tiled, const void* Aq_tiled, void* act_tiled_out, void* workspace, int64_t workspace_bytes, int64_t M, int64_t N_ff,
	int64_t K, void* stream) {
	return gate_up_silu_common(W_gate_tiled, W_up_tiled, Aq_tiled, act_tiled_out, nullptr, nullptr, workspace, workspace_bytes, M, N_ff, K, stream);
}

int nh_q8_0_debug_gemm_tiled_gate_up_silu(const void* W_gate_tiled, const void* W_up_tiled, const void* Aq_tiled, void* act_tiled_out, float* gate_out, float* up_out, int64_t M, int64_t N_ff,
	int64_t K, void* stream) {
	NH_REQUIRE((gate_out && up_out) || M == 0 || N_ff == 0, NH_ERR_NULL_POINTER);
	return gate_up_silu_common(W_gate_tiled, W_up_tiled, Aq_tiled, act_tiled_out, gate_out, up_out, nullptr, 0, M, N_ff, K, stream);
}

int64_t nh_q8_0_mul_mat_workspace_bytes(int64_t M, int64_t K) {
	if (M < 0 || K < 0 || K % nh::GROUP_K != 0) {
		return NH_ERR_SHAPE;
	}
	if (M <= nh::GEMV_ROWS_MAX) {
		return 0; // a few rows: the quantize happens inside the mat-vec kernel, nothing is staged in memory
	}
	return (nh_q8_0_tiled_bytes(M, K) + 255) / 256 * 256;
}

static int mul_mat_common(const void* W_tiled, const float* x, const float* residual, float* y, int64_t M, int64_t N, int64_t K, void* workspace, int64_t workspace_bytes, void* stream) {
	NH_TRY(check_shape(M, N, K, true));
	if (M == 0 || N == 0) {
		return NH_OK;
	}
	const int64_t need = nh_q8_0_mul_mat_workspace_bytes(M, K);
	NH_REQUIRE(workspace_bytes >= need, NH_ERR_ARGUMENT);
	if (K > 0) {
		NH_REQUIRE(x && (workspace || need == 0), NH_ERR_NULL_POINTER);
		NH_REQUIRE(aligned16(workspace) && aligned16(x), NH_ERR_ALIGNMENT);
	}
	const nh::mul_mat_plan plan = nh::plan_mul_mat(M, N, K); // which kernel: q8_0_plan.h
	if (M == 1) { // quantize fused into the mat-vec: the workspace stays unused
		return residual ? nh_q8_0_gemv_tiled_residual_f32(W_tiled, x, residual, y, N, K, stream) : nh_q8_0_gemv_tiled_f32(W_tiled, x, y, N, K, stream);
	}
	if (plan.kernel == nh::MM_GEMV_ROWS_MFMA) { // four to sixteen rows on small matrices: the streaming kernel with the rows as an MFMA operand
		NH_REQUIRE(W_tiled && y, NH_ERR_NULL_POINTER);
		NH_REQUIRE(aligned16(W_tiled) && aligned16(y) && aligned16(residual), NH_ERR_ALIGNMENT);
		NH_TRY(require_device());
		return from_hip(nh::launch_gemv_rows_mfma(W_tiled, x, y, M, N, K, as_stream(stream), residual));
	}
	if (plan.kernel == nh::MM_GEMV_ROWS) { // a few rows: the same streaming kernel with M dot products per weight tile
		NH_REQUIRE(W_tiled && y, NH_ERR_NULL_POINTER);
		NH_REQUIRE(aligned16(W_tiled) && aligned16(y) && aligned16(residual), NH_ERR_ALIGNMENT);
		NH_TRY(require_device());
		return from_hip(nh::launch_gemv_rows(W_tiled, x, y, M, N, K, as_stream(stream), residual));
	}
	NH_TRY(nh_q8_0_quantize_tiled(x, workspace, M, K, stream));
	return residual ? nh_q8_0_gemm_tiled_residual(W_tiled, workspace, residual, y, M, N, K, stream) : nh_q8_0_gemm_tiled(W_tiled, workspace, y, M, N, K, stream);
}

int nh_q8_0_debug_plan_mul_mat(int64_t M, int64_t N, int64_t K, int32_t* host_plan) {
	NH_TRY(check_shape(M, N, K, true));
	NH_REQUIRE(host_plan, NH_ERR_NULL_POINTER);
	const nh::mul_mat_plan p = nh::plan_mul_mat(M, N, K);
	for (int i = 0; i < 8; ++i) {
		host_plan[i] = 0;
	}
	host_plan[0] = p.kernel;
	host_plan[1] = p.quantize_launch;
	switch (p.kernel) {
		case nh::MM_GEMV:
		case nh::MM_GEMV_ROWS_MFMA:
			host_plan[2] = p.gemv.splits;
			host_plan[3] = p.gemv.tiles;
			host_plan[4] = p.gemv_row_parts;
			break;
		case nh::MM_GEMM_SKINNY:
			host_plan[2] = p.gemm.skinny.ms;
			host_plan[3] = p.gemm.skinny.splits;
			break;
		case nh::MM_GEMM_TILE_STREAM:
		case nh::MM_GEMM_TILE:
			host_plan[2] = p.gemm.tile.tm;
			host_plan[3] = p.gemm.tile.ks;
			host_plan[4] = p.gemm.tile.kz;
			host_plan[5] = static_cast<int32_t>(p.gemm.tile.grid_x);
			host_plan[6] = static_cast<int32_t>(p.gemm.tile.grid_y);
			break;
		default:
			break;
	}
	return NH_OK;
}

int nh_q8_0_mul_mat(const void* W_tiled, const float* x, float* y, int64_t M, int64_t N, int64_t K, void* workspace, int64_t workspace_bytes, void* stream) {
	return mul_mat_common(W_tiled, x, nullptr, y, M, N, K, workspace, workspace_bytes, stream);
}

int nh_q8_0_mul_mat_residual(const void* W_tiled, const float* x, const float* residual, float* y, int64_t M, int64_t N, int64_t K, void* workspace, int64_t workspace_bytes,
	void* stream) {
	NH_REQUIRE(residual || M == 0 || N == 0, NH_ERR_NULL_POINTER);
	return mul_mat_common(W_tiled, x, residual, y, M, N, K, workspace, workspace_bytes, stream);
}

int nh_q8_0_debug_block_sums(const void* W, const void* Aq, int32_t* sums, int64_t M, int64_t N, int64_t K, int path, void* stream) {
	NH_REQUIRE(path >= 0 && path <= 3, NH_ERR_ARGUMENT);
	const bool tiled = path >= 2;
	const bool mfma	 = (path & 1) != 0;
	NH_TRY(check_shape(M, N, K, tiled));
	NH_REQUIRE(mfma || M == 1, NH_ERR_ARGUMENT);
	NH_REQUIRE(mfma || tiled || K <= MAX_K_BLOCKS_GEMV, NH_ERR_TOO_LARGE);
	if (M == 0 || N == 0 || K == 0) {
		return NH_OK;
	}
	NH_REQUIRE(W && Aq && sums, NH_ERR_NULL_POINTER);
	NH_REQUIRE(aligned16(W) && aligned16(Aq) && aligned16(sums), NH_ERR_ALIGNMENT);
	NH_TRY(require_device());
	if (!mfma) {
		return from_hip(nh::launch_gemv(W, Aq, nullptr, sums, N, K, tiled, as_stream(stream)));
	}
	return from_hip(nh::launch_gemm(W, Aq, nullptr, sums, M, N, K, tiled, as_stream(stream)));
}

int nh_q8_0_fill_weight_blocks(void* blocks, uint64_t seed, int64_t first_block, int64_t n_blocks, void* stream) {
	NH_REQUIRE(n_blocks >= 0 && first_block >= 0, NH_ERR_SHAPE);
	if (n_blocks == 0) {
		return NH_OK;
	}
	NH_REQUIRE(n_blocks <= MAX_BLOCKS, NH_ERR_TOO_LARGE);
	NH_REQUIRE(blocks, NH_ERR_NULL_POINTER);
	NH_REQUIRE((reinterpret_cast<uintptr_t>(blocks) & 1u) == 0, NH_ERR_ALIGNMENT);
	NH_TRY(require_device());
	return from_hip(nh::launch_fill_weights(blocks, seed, first_block, n_blocks, as_stream(stream)));
}

int nh_q8_0_fill_activations(float* x, uint64_t seed, int64_t count, void* stream) {
	NH_REQUIRE(count >= 0, NH_ERR_SHAPE);
	if (count == 0) {
		return NH_OK;
	}
	NH_REQUIRE(x, NH_ERR_NULL_POINTER);
	NH_TRY(require_device());
	return from_hip(nh::launch_fill_activations(x, seed, count, as_stream(stream)));
}

} // extern "C"
