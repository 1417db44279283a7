// What one kernel dispatch costs on this machine before the kernel does anything: an empty kernel and a kernel with one
// dependent 16-byte load per lane, at the decode mat-vec's geometry (1024-thread workgroups), timed two ways:
//   queued:  2000 launches enqueued behind a kernel that holds the device for ~10 ms, so that the queue is full when it
//            drains: the device-side cost per dispatch (command processor, barrier between dependent dispatches, cache
//            maintenance), no host in the loop;
//   host:    2000 launches back to back from an idle queue: the host's submission rate, if it is the slower of the two.
// The figure bounds a chain of dependent launches from below (a decode token of L launches cannot take less than
// L x queued + bytes / bandwidth).  A measurement tool beside the tests; prints one JSON object.
#include <hip/hip_runtime.h>

#include <chrono>
#include <cstdio>

#define CK(x)                                                         \
	do {                                                              \
		hipError_t e_ = (x);                                          \
		if (e_ != hipSuccess) {                                       \
			std::printf("FAILED %s: %s\n", #x, hipGetErrorString(e_)); \
			return 1;                                                 \
		}                                                             \
	} while (0)

__global__ void hold_kernel(float* y, long long cycles) {
	const long long t0 = clock64();
	while (clock64() - t0 < cycles) {
	}
	if (cycles < 0) {
		y[0] = 1.0f;
	}
}
__global__ __launch_bounds__(1024) void empty_kernel(const uint4*, float*) {
}
__global__ __launch_bounds__(1024) void one_load_kernel(const uint4* w, float* y) {
	const uint4 v = w[static_cast<size_t>(blockIdx.x) * 1024 + threadIdx.x];
	if (v.x == 0x12345678u && v.y == 0x9abcdef0u) { // never true for the filled buffer: the load must still complete
		y[threadIdx.x] = 1.0f;
	}
}

template<typename K> static int measure(K kernel, int grid, const uint4* w, float* y, double* queued_us, double* host_us) {
	constexpr int N = 2000;
	hipEvent_t a, b;
	CK(hipEventCreate(&a));
	CK(hipEventCreate(&b));
	for (int i = 0; i < 20; ++i) {
		hipLaunchKernelGGL(kernel, dim3(grid), dim3(1024), 0, 0, w, y);
	}
	CK(hipDeviceSynchronize());
	hipLaunchKernelGGL(hold_kernel, dim3(1), dim3(64), 0, 0, y, 20000000LL);
	CK(hipEventRecord(a, 0));
	for (int i = 0; i < N; ++i) {
		hipLaunchKernelGGL(kernel, dim3(grid), dim3(1024), 0, 0, w, y);
	}
	CK(hipEventRecord(b, 0));
	CK(hipEventSynchronize(b));
	float ms = 0;
	CK(hipEventElapsedTime(&ms, a, b));
	*queued_us = ms / N * 1e3;
	CK(hipDeviceSynchronize());
	const auto t0 = std::chrono::steady_clock::now();
	for (int i = 0; i < N; ++i) {
		hipLaunchKernelGGL(kernel, dim3(grid), dim3(1024), 0, 0, w, y);
	}
	CK(hipDeviceSynchronize());
	*host_us = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() / N * 1e6;
	CK(hipEventDestroy(a));
	CK(hipEventDestroy(b));
	return 0;
}

int main() {
	uint4* w = nullptr;
	float* y = nullptr;
	CK(hipMalloc(&w, 512 * 1024 * sizeof(uint4)));
	CK(hipMalloc(&y, 4096));
	CK(hipMemset(w, 1, 512 * 1024 * sizeof(uint4)));
	double eq[2], eh[2], lq[2], lh[2];
	const int grids[2] = { 256, 448 };
	for (int i = 0; i < 2; ++i) {
		if (measure(empty_kernel, grids[i], w, y, &eq[i], &eh[i]) || measure(one_load_kernel, grids[i], w, y, &lq[i], &lh[i])) {
			return 1;
		}
	}
	std::printf("{\"workgroup_threads\": 1024, \"grids\": [256, 448], \"empty_kernel_queued_us\": [%.3f, %.3f], \"empty_kernel_host_us\": [%.3f, %.3f], "
				"\"one_load_kernel_queued_us\": [%.3f, %.3f], \"one_load_kernel_host_us\": [%.3f, %.3f]}\n",
		eq[0], eq[1], eh[0], eh[1], lq[0], lq[1], lh[0], lh[1]);
	return 0;
}
