// What a bare read of N bytes costs on this machine: the floor under a streaming mat-vec of a matrix of that size.
// A one-shot kernel at the mat-vec's geometry (1024-thread workgroups, every wave requests all of its bytes -- 4 KiB,
// non-temporal 16-byte loads -- before it waits), nothing computed but an xor that keeps the loads alive.  Buffers are
// rotated over more than 600 MB so that every launch comes from HBM, and timed with the dispatch packet's own
// start / stop timestamps (what a kernel trace calls the duration); the median of 60 launches is reported.
// Sizes: command-line arguments in bytes (default: the weight bytes of the LLaMA-3-8B decode shapes and of the FFN step).
// A measurement tool beside the tests; prints one JSON object.
#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <vector>

#define CK(x)                                                         \
	do {                                                              \
		hipError_t e_ = (x);                                          \
		if (e_ != hipSuccess) {                                       \
			std::printf("FAILED %s: %s\n", #x, hipGetErrorString(e_)); \
			return 1;                                                 \
		}                                                             \
	} while (0)

typedef int v4i __attribute__((ext_vector_type(4)));
constexpr int LOADS = 4; // 16-byte loads per lane: 4 KiB per wave, 64 KiB per workgroup

__global__ __launch_bounds__(1024) void read_kernel(const v4i* __restrict__ p, long long waves, int* sink) {
	const int lane	   = threadIdx.x & 63;
	const long long w = static_cast<long long>(blockIdx.x) * 16 + (threadIdx.x >> 6);
	if (w >= waves) {
		return;
	}
	v4i v[LOADS];
#pragma unroll
	for (int u = 0; u < LOADS; ++u) {
		v[u] = __builtin_nontemporal_load(p + w * (64 * LOADS) + u * 64 + lane);
	}
	int acc = 0;
#pragma unroll
	for (int u = 0; u < LOADS; ++u) {
		acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
	}
	if (acc == 0x12345678) { // never true for the filled buffer: the loads must still complete
		sink[w & 1023] = acc;
	}
}

int main(int argc, char** argv) {
	std::vector<long long> sizes;
	for (int i = 1; i < argc; ++i) {
		sizes.push_back(std::atoll(argv[i]));
	}
	if (sizes.empty()) {
		sizes = { 4456448, 17825792, 26738688, 62390272, 187170816, 558170112 };
	}
	const long long pool = 1200ll << 20;
	char* base = nullptr;
	int* sink  = nullptr;
	CK(hipMalloc(&base, pool));
	CK(hipMalloc(&sink, 4096));
	CK(hipMemset(base, 1, pool));
	CK(hipDeviceSynchronize());
	hipEvent_t e0, e1;
	CK(hipEventCreate(&e0));
	CK(hipEventCreate(&e1));
	std::printf("{\"workgroup_threads\": 1024, \"bytes_per_wave\": %d, \"reads\": [", LOADS * 1024);
	bool first = true;
	for (long long want : sizes) {
		const long long waves = want / (LOADS * 1024);
		const long long bytes = waves * LOADS * 1024;
		if (waves <= 0 || bytes > pool) {
			continue;
		}
		const int buffers = static_cast<int>(std::max(1ll, std::min(pool / bytes, (600ll << 20) / bytes + 2)));
		const unsigned grid = static_cast<unsigned>((waves + 15) / 16);
		std::vector<float> times;
		for (int r = 0; r < 80; ++r) {
			const v4i* src = reinterpret_cast<const v4i*>(base + static_cast<long long>(r % buffers) * bytes);
			hipExtLaunchKernelGGL(read_kernel, dim3(grid), dim3(1024), 0, 0, e0, e1, 0, src, waves, sink);
			CK(hipGetLastError());
			CK(hipEventSynchronize(e1));
			float ms = 0;
			CK(hipEventElapsedTime(&ms, e0, e1));
			if (r >= 20) {
				times.push_back(ms);
			}
		}
		std::sort(times.begin(), times.end());
		const double us = times[times.size() / 2] * 1e3;
		std::printf("%s{\"bytes\": %lld, \"workgroups\": %u, \"buffers_rotated\": %d, \"us\": %.3f, \"GBs\": %.1f}", first ? "" : ", ", bytes, grid, buffers, us, bytes / us / 1e3);
		first = false;
	}
	std::printf("]}\n");
	return 0;
}
