// Opt-in per-kernel timing and the native batch runner.
//
// Timing: while it is on for one kernel kind, each launch of that kind carries a start/stop event pair in its
// dispatch packet; nh_profile_end sums the elapsed times.  This measures the kernel alone (no launch gap), on the
// stream it runs on, inside the caller's own timed loop.  Off by default: a plain launch costs one branch.
//
// Batch runner: a list of mul_mat operations enqueued from native code in one call, so a decode step's
// launches (7 projections x 32 layers + lm_head at LLaMA-3-8B) are not paced by the caller's language runtime.
#include "../../include/nihilus_amd/q8_0_abi.h"
#include "q8_0_plan.h"

#include <atomic>
#include <mutex>
#include <vector>

namespace nh {

namespace {
	struct timer_state {
		std::mutex lock;
		std::atomic<int> kind{ -1 }; // kind being timed, -1 = off; read without the lock on every launch
		std::vector<hipEvent_t> events; // 2 per launch
		size_t used = 0; // events handed out
	};
	timer_state& timer() {
		static timer_state t;
		return t;
	}
} // namespace

bool profile_next(int kind, hipEvent_t* start, hipEvent_t* stop) {
	timer_state& t = timer();
	if (t.kind.load(std::memory_order_relaxed) != kind) { // fast path: one relaxed load per launch
		return false;
	}
	std::lock_guard<std::mutex> g(t.lock);
	if (t.kind.load(std::memory_order_relaxed) != kind || t.used + 2 > t.events.size()) {
		return false;
	}
	*start = t.events[t.used];
	*stop  = t.events[t.used + 1];
	t.used += 2;
	return true;
}

} // namespace nh

namespace nh {
// clock64 counts shader clocks, wall_clock64 a constant 100 MHz: one wave reads both, spins for `ticks` of the latter, reads both again
__global__ void shader_clock_kernel(long long* out, long long ticks) {
	const long long w0 = wall_clock64();
	const long long c0 = clock64();
	long long w1	   = w0;
	while (w1 - w0 < ticks) {
		__builtin_amdgcn_s_sleep(4);
		w1 = wall_clock64();
	}
	const long long c1 = clock64();
	if (threadIdx.x == 0) {
		out[0] = c1 - c0;
		out[1] = w1 - w0;
	}
}
} // namespace nh

extern "C" {

int nh_profile_shader_clock(double* host_mhz, int64_t spin_us) {
	if (!host_mhz || spin_us < 1 || spin_us > 100000) {
		return NH_ERR_ARGUMENT;
	}
	// a stream of its own (default priority, not synchronised with the NULL stream), so that the wave runs beside whatever
	// the caller has queued elsewhere: the clock read is the one the chip holds under that load
	hipStream_t s = nullptr;
	hipError_t e  = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);
	if (e != hipSuccess) {
		return static_cast<int>(e);
	}
	long long* dev = nullptr;
	long long host[2] = { 0, 0 };
	e = hipMalloc(&dev, sizeof(host));
	if (e == hipSuccess) {
		nh::shader_clock_kernel<<<dim3(1), dim3(64), 0, s>>>(dev, spin_us * 100);
		e = hipGetLastError();
	}
	if (e == hipSuccess) {
		e = hipMemcpyAsync(host, dev, sizeof(host), hipMemcpyDeviceToHost, s);
	}
	if (e == hipSuccess) {
		e = hipStreamSynchronize(s);
	}
	(void)hipFree(dev);
	(void)hipStreamDestroy(s);
	if (e != hipSuccess) {
		return static_cast<int>(e);
	}
	*host_mhz = host[1] > 0 ? static_cast<double>(host[0]) / static_cast<double>(host[1]) * 100.0 : 0.0;
	return NH_OK;
}

int nh_profile_begin(int kernel_kind, int64_t max_launches) {
	if (kernel_kind < 0 || kernel_kind >= nh::KIND_COUNT || max_launches <= 0 || max_launches > (1 << 20)) {
		return NH_ERR_ARGUMENT;
	}
	nh::timer_state& t = nh::timer();
	std::lock_guard<std::mutex> g(t.lock);
	if (t.kind.load(std::memory_order_relaxed) != -1) {
		return NH_ERR_ARGUMENT; // already timing
	}
	t.events.resize(static_cast<size_t>(max_launches) * 2);
	for (size_t i = 0; i < t.events.size(); ++i) {
		const hipError_t e = hipEventCreate(&t.events[i]);
		if (e != hipSuccess) {
			for (size_t j = 0; j < i; ++j) {
				(void)hipEventDestroy(t.events[j]);
			}
			t.events.clear();
			return static_cast<int>(e);
		}
	}
	t.used = 0;
	t.kind = kernel_kind;
	return NH_OK;
}

int nh_profile_end(double* host_total_ms, int64_t* host_launches, double* host_min_ms, double* host_max_ms) {
	nh::timer_state& t = nh::timer();
	std::lock_guard<std::mutex> g(t.lock);
	if (t.kind.load(std::memory_order_relaxed) == -1) {
		return NH_ERR_ARGUMENT;
	}
	t.kind		 = -1;
	int rc		 = NH_OK;
	double total = 0.0, mn = 0.0, mx = 0.0;
	int64_t n	 = 0;
	for (size_t i = 0; i + 1 < t.used; i += 2) {
		hipError_t e = hipEventSynchronize(t.events[i + 1]);
		float ms	 = 0.0f;
		if (e == hipSuccess) {
			e = hipEventElapsedTime(&ms, t.events[i], t.events[i + 1]);
		}
		if (e != hipSuccess) {
			rc = static_cast<int>(e);
			break;
		}
		total += ms;
		mn = (n == 0 || ms < mn) ? ms : mn;
		mx = (n == 0 || ms > mx) ? ms : mx;
		++n;
	}
	for (hipEvent_t ev : t.events) {
		(void)hipEventDestroy(ev);
	}
	t.events.clear();
	t.used = 0;
	if (host_total_ms) {
		*host_total_ms = total;
	}
	if (host_launches) {
		*host_launches = n;
	}
	if (host_min_ms) {
		*host_min_ms = mn;
	}
	if (host_max_ms) {
		*host_max_ms = mx;
	}
	return rc;
}

int nh_q8_0_mul_mat_batch(const nh_q8_0_mul_mat_op* host_ops, int64_t count, void* workspace, int64_t workspace_bytes, void* stream) {
	if (count < 0) {
		return NH_ERR_SHAPE;
	}
	if (count == 0) {
		return NH_OK;
	}
	if (!host_ops) {
		return NH_ERR_NULL_POINTER;
	}
	// validate everything before the first launch, so a bad entry cannot leave half a step enqueued
	for (int64_t i = 0; i < count; ++i) {
		const nh_q8_0_mul_mat_op& op = host_ops[i];
		if (op.M < 0 || op.N < 0 || op.K < 0 || op.K % nh::GROUP_K != 0) {
			return NH_ERR_SHAPE;
		}
		const int64_t need = nh_q8_0_mul_mat_workspace_bytes(op.M, op.K);
		if (need < 0 || need > workspace_bytes) {
			return NH_ERR_ARGUMENT;
		}
		if (op.M > 0 && op.N > 0 && (!op.y || (op.K > 0 && (!op.W_tiled || !op.x)))) {
			return NH_ERR_NULL_POINTER;
		}
		if (op.M > 0 && op.N > 0 && ((reinterpret_cast<uintptr_t>(op.W_tiled) | reinterpret_cast<uintptr_t>(op.x) | reinterpret_cast<uintptr_t>(op.y)) & 15u) != 0) {
			return NH_ERR_ALIGNMENT;
		}
	}
	constexpr int64_t MAX_RUN = 64; // M == 1 entries looked at together (a multiple of the group size)
	const float* quantized_x = nullptr; // activation currently held in the workspace (M > 1 only)
	int64_t quantized_m = -1, quantized_k = -1;
	for (int64_t i = 0; i < count;) {
		const nh_q8_0_mul_mat_op& op = host_ops[i];
		if (op.M == 0 || op.N == 0) {
			++i;
			continue;
		}
		if (op.M == 1) {
			// decode: the quantize lives inside the mat-vec kernel.  The longest run of M == 1 entries of which none reads or
			// overwrites what an earlier one of the run writes (seen from their x and y ranges) and none asks to be ordered
			// goes out together: the result is that of running them in list order, whatever runs side by side.
			auto overlap = [](const float* a, int64_t na, const float* b, int64_t nb) {
				const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
				return a0 < b0 + static_cast<uintptr_t>(nb) * 4 && b0 < a0 + static_cast<uintptr_t>(na) * 4;
			};
			int64_t g	= 1;
			bool shared = true; // every entry of the run has the first one's x and K
			while (i + g < count) {
				const nh_q8_0_mul_mat_op& o = host_ops[i + g];
				if (g >= MAX_RUN || o.M != 1 || o.N == 0 || o.ordered) { // MAX_RUN: the hazard check is quadratic in the run length
					break;
				}
				bool hazard = false;
				for (int64_t e = 0; e < g && !hazard; ++e) {
					const nh_q8_0_mul_mat_op& p = host_ops[i + e];
					hazard = overlap(o.y, o.N, p.y, p.N) || overlap(o.y, o.N, p.x, p.K) || overlap(o.x, o.K, p.y, p.N);
				}
				if (hazard) {
					break;
				}
				shared = shared && o.x == op.x && o.K == op.K;
				++g;
			}
			if (shared && g <= nh::GEMV_MAX_SEGMENTS) {
				// neighbours that share x and K (q/k/v, gate/up) and nothing else to go with them: segments of one mat-vec launch
				const void* w[nh::GEMV_MAX_SEGMENTS];
				float* y[nh::GEMV_MAX_SEGMENTS];
				int64_t n[nh::GEMV_MAX_SEGMENTS];
				for (int64_t e = 0; e < g; ++e) {
					w[e] = host_ops[i + e].W_tiled;
					y[e] = host_ops[i + e].y;
					n[e] = host_ops[i + e].N;
				}
				const int rc = nh_q8_0_gemv_tiled_multi_f32(w, y, n, g, op.x, op.K, stream);
				if (rc != NH_OK) {
					return rc;
				}
			} else {
				const void* w[MAX_RUN];
				const float* x[MAX_RUN];
				float* y[MAX_RUN];
				int64_t n[MAX_RUN], k[MAX_RUN];
				for (int64_t e = 0; e < g; ++e) {
					const nh_q8_0_mul_mat_op& o = host_ops[i + e];
					w[e] = o.W_tiled;
					x[e] = o.x;
					y[e] = o.y;
					n[e] = o.N;
					k[e] = o.K;
				}
				const int rc = nh_q8_0_gemv_tiled_group_f32(w, x, y, nullptr, n, k, g, stream);
				if (rc != NH_OK) {
					return rc;
				}
			}
			i += g;
			continue;
		}
		if (!nh::plan_mul_mat(op.M, op.N, op.K).quantize_launch) {
			// a few rows: still a mat-vec kernel (quantize inside), the workspace stays unused
			const int rc = nh_q8_0_mul_mat(op.W_tiled, op.x, op.y, op.M, op.N, op.K, workspace, workspace_bytes, stream);
			if (rc != NH_OK) {
				return rc;
			}
			++i;
			continue;
		}
		const bool reuse = op.reuse_quantized_x && quantized_x == op.x && quantized_m == op.M && quantized_k == op.K;
		if (!reuse) {
			const int rc = nh_q8_0_quantize_tiled(op.x, workspace, op.M, op.K, stream);
			if (rc != NH_OK) {
				return rc;
			}
			quantized_x = op.x;
			quantized_m = op.M;
			quantized_k = op.K;
		}
		const int rc = nh_q8_0_gemm_tiled(op.W_tiled, workspace, op.y, op.M, op.N, op.K, stream);
		if (rc != NH_OK) {
			return rc;
		}
		++i;
	}
	return NH_OK;
}

} // extern "C"
