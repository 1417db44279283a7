// Device-side helpers shared by the gfx950 Q8_0 kernels: layout constants, fp16 scale conversion,
// the packed int8 dot, and the launch functions each translation unit exports to the C ABI file.
#pragma once

#include <hip/hip_ext.h>
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nh {

constexpr int QK			= 32; // quants per block (Q_SIZE, common/data_types.hpp:28)
constexpr int BLOCK_BYTES	= 34; // fp16 d + 32 int8 (common/data_types.hpp:38-44)
constexpr int STRIP_ROWS	= 32; // rows per tiled strip = MFMA 32x32x32 operand rows
constexpr int GROUP_BLOCKS	= 4; // blocks per macro-tile along K
constexpr int GROUP_K		= GROUP_BLOCKS * QK; // 128
constexpr int TILE_BYTES	= 1024; // 32 rows x 32 quants, in MFMA operand order
constexpr int MACRO_BYTES	= GROUP_BLOCKS * TILE_BYTES + STRIP_ROWS * GROUP_BLOCKS * 2; // 4352 = 32 rows x 4 blocks x 34
constexpr int MACRO_D_OFFSET = GROUP_BLOCKS * TILE_BYTES; // 4096

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));

// fp16 bits -> fp32, exact (v_cvt_f32_f16; fp16 subnormals are honoured: the kernel's float mode keeps them).
__device__ __forceinline__ float half_bits_to_float(uint16_t h) {
	return __half2float(__ushort_as_half(h));
}
// fp32 -> fp16 bits, round to nearest even, subnormals kept, overflow to inf (v_cvt_f16_f32).
__device__ __forceinline__ uint16_t float_to_half_bits(float f) {
	return __half_as_ushort(__float2half_rn(f));
}
// c + sum of four int8 x int8 products, exact (v_dot4_i32_i8).
__device__ __forceinline__ int dot4(int a, int b, int c) {
	return __builtin_amdgcn_sdot4(a, b, c, false);
}
__device__ __forceinline__ int dot16(v4i a, v4i b) {
	int s = dot4(a.x, b.x, 0);
	s	  = dot4(a.y, b.y, s);
	s	  = dot4(a.z, b.z, s);
	return dot4(a.w, b.w, s);
}
// 16 bytes from an address that is only 2-byte aligned (the qs field of a packed 34-byte block).
__device__ __forceinline__ v4i load16_unaligned(const uint8_t* p) {
	v4i v;
	__builtin_memcpy(&v, p, 16);
	return v;
}
__device__ __forceinline__ uint16_t load_u16(const uint8_t* p) {
	return *reinterpret_cast<const uint16_t*>(p);
}

// q = int8(rne(fl32(f * id))): the last step of quantize_row_q8_0 for one value (reference cpu/avx_2.hpp:4465-4487).
__device__ __forceinline__ int quantize_value(float f, float id) {
	const float r = rintf(__fmul_rn(f, id)); // v_rndne_f32: ties to even
	// x86 cvtps_epi32 yields 0x80000000 for NaN and out-of-range values, which the reference's saturating packs
	// turn into -128.  Reachable only when 127/amax overflows to inf (amax below ~3.7e-37): inf, and 0*inf = NaN.
	const int q = (fabsf(r) < 2147483648.0f) ? static_cast<int>(r) : INT32_MIN;
	return max(-128, min(127, q));
}

// A value from another lane of the same row of 16 lanes, by a fixed pattern (data-parallel primitive: no LDS traffic, and it
// folds into the instruction that uses it).  All lanes involved must be active.
template<int CTRL> __device__ __forceinline__ float lane_pattern(float x) {
	return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, true));
}
constexpr int DPP_QUAD_SWAP_1	 = 0xB1; // quad_perm [1, 0, 3, 2]: lane ^ 1
constexpr int DPP_QUAD_SWAP_2	 = 0x4E; // quad_perm [2, 3, 0, 1]: lane ^ 2
constexpr int DPP_ROW_ROTATE_8	 = 0x128; // row_ror:8: lane (i + 8) % 16 of the same 16-lane row, i.e. lane ^ 8
constexpr int DPP_ROW_HALF_MIRROR = 0x141; // lane i <-> 7 - i within each group of eight: pairs the two quads of the group

// One lane's share of quantize_row_q8_0 (reference cpu/avx_2.hpp:4439-4489): eight consecutive lanes (a group aligned to eight)
// hold one 32-value block as eight float4.  Returns this lane's four quants packed little-endian; *dh = fp16 bits of d.
//   amax = max|x_i|; d = fp16_rne(amax / 127.f); id = amax != 0 ? 127.f / amax : 0; q_i = int8(rne(fl32(x_i * id)))
// Divide, multiply and rounding are separate correctly rounded fp32 operations; all eight lanes must be active.
// Two routes to the same bits.  The general one spells the operations out with every guard the corner cases need (NaN and
// infinity among the values, 127 / amax overflowing, quotients near the subnormal range).  The short one runs when no lane of the
// wave has such a block -- every value finite, amax zero or within [2^-60, 2^60]:
//   * amax / 127 as q = amax * c, r = fma(-127, q, amax), d = fma(r, c, q) with c = fl32(1 / 127): with the correctly rounded
//     reciprocal of the divisor and the exact remainder from the fma, one correction step gives the correctly rounded quotient;
//   * 127 / amax as the reciprocal estimate, one refinement of it and two of the quotient -- the steps of the general
//     division, without its rescaling and special-case handling, which are the identity in this range;
//   * |x_i * id| <= 127 (1 + 2^-23), so the rounded product converts to int8 without the NaN guard and the clamp.
__device__ __forceinline__ uint32_t quantize_block_lane(float4 v, uint16_t* dh) {
	float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
	amax	   = fmaxf(amax, lane_pattern<DPP_QUAD_SWAP_1>(amax));
	amax	   = fmaxf(amax, lane_pattern<DPP_QUAD_SWAP_2>(amax));
	amax	   = fmaxf(amax, lane_pattern<DPP_ROW_HALF_MIRROR>(amax));
	const float sum = (v.x + v.y) + (v.z + v.w); // NaN or infinity among the four makes this NaN or infinite
	const bool plain = (amax == 0.0f || (amax >= 0x1p-60f && amax <= 0x1p60f)) && fabsf(sum) <= 0x1p100f;
	if (__builtin_amdgcn_ballot_w64(!plain) == 0) {
		constexpr float c = 1.0f / 127.0f; // correctly rounded by the compiler
		const float q	  = __fmul_rn(amax, c);
		const float d	  = fmaf(fmaf(-127.0f, q, amax), c, q);
		const float y0	  = __builtin_amdgcn_rcpf(amax);
		const float y1	  = fmaf(fmaf(-amax, y0, 1.0f), y0, y0);
		const float q0	  = __fmul_rn(127.0f, y1);
		const float q1	  = fmaf(fmaf(-amax, q0, 127.0f), y1, q0);
		const float q2	  = fmaf(fmaf(-amax, q1, 127.0f), y1, q1);
		const float id	  = amax != 0.0f ? q2 : 0.0f;
		*dh				  = float_to_half_bits(d);
		const uint32_t a = static_cast<uint32_t>(static_cast<int>(rintf(__fmul_rn(v.x, id)))), b = static_cast<uint32_t>(static_cast<int>(rintf(__fmul_rn(v.y, id))));
		const uint32_t e = static_cast<uint32_t>(static_cast<int>(rintf(__fmul_rn(v.z, id)))), f = static_cast<uint32_t>(static_cast<int>(rintf(__fmul_rn(v.w, id))));
		// low bytes of a, b into bytes 0, 1; of e, f into bytes 2, 3 (selector: 0..3 = bytes of the second operand, 4..7 of the first, 0x0c = zero)
		return __builtin_amdgcn_perm(b, a, 0x0c0c0400u) | __builtin_amdgcn_perm(f, e, 0x04000c0cu);
	}
	const float d  = __fdiv_rn(amax, 127.0f);
	const float id = (amax != 0.0f) ? __fdiv_rn(127.0f, amax) : 0.0f;
	*dh			   = float_to_half_bits(d);
	auto q8 = [id](float f) -> uint32_t { return static_cast<uint32_t>(quantize_value(f, id)) & 0xFFu; };
	return q8(v.x) | (q8(v.y) << 8) | (q8(v.z) << 16) | (q8(v.w) << 24);
}

// exp(x) in fp32 as a fixed sequence of correctly rounded fp32 operations (multiply, fma, round-to-nearest-even,
// exponent insertion), so that a host restatement of the same sequence gives the same bits: the activation that
// feeds a quantizer must not depend on which math library evaluated it.  Range reduction by n = rne(x * log2 e) with
// a two-part ln 2, degree-5 polynomial (the classic Cephes single-precision coefficients) on |r| <= ln2 / 2; within
// 2 ulp of the true value.  The argument is clamped to [-87, 88] so that 2^n is a normal number.
__device__ __forceinline__ float exp_f32(float x) {
	x			  = fminf(fmaxf(x, -87.0f), 88.0f);
	const float n = rintf(__fmul_rn(x, 1.44269504088896341f));
	float r		  = fmaf(n, -0.693359375f, x);
	r			  = fmaf(n, 2.12194440e-4f, r);
	float p		  = 1.9875691500e-4f;
	p			  = fmaf(p, r, 1.3981999507e-3f);
	p			  = fmaf(p, r, 8.3334519073e-3f);
	p			  = fmaf(p, r, 4.1665795894e-2f);
	p			  = fmaf(p, r, 1.6666665459e-1f);
	p			  = fmaf(p, r, 5.0000001201e-1f);
	const float e = __fadd_rn(fmaf(p, __fmul_rn(r, r), r), 1.0f);
	return __fmul_rn(e, __uint_as_float(static_cast<uint32_t>(static_cast<int>(n) + 127) << 23));
}

// SiLU(g) * u, the activation in front of the FFN down projection (ffn_silu -> ffn_gate_par in the reference's graph,
// infra/core_traits.hpp:982-986; the reference's silu and mul kernels have no body, the formula is the model's:
// silu(g) = g / (1 + exp(-g))).  IEEE divide, separate multiply.
__device__ __forceinline__ float silu_mul(float g, float u) {
	return __fmul_rn(__fdiv_rn(g, __fadd_rn(1.0f, exp_f32(-g))), u);
}
__device__ __forceinline__ float4 silu_mul4(float4 g, float4 u) {
	return make_float4(silu_mul(g.x, u.x), silu_mul(g.y, u.y), silu_mul(g.z, u.z), silu_mul(g.w, u.w));
}

// RMS norm of a row, as a fixed order of fp32 operations over a 1024-thread workgroup (16 waves), restated by the CPU
// checker so that the normalised, quantized row is reproducible bit for bit:
//   runs:      the row's G = K / 128 groups are cut into 16 contiguous runs, run w = groups [w*q + min(w, r), ...) with
//              q = G / 16, r = G % 16 and the first r runs one group longer (the cut of an unsplit mat-vec launch);
//   lane l of wave w:  p = sum over the float4s l, l + 64, l + 128, ... of run w of x.x^2 + x.y^2 + x.z^2 + x.w^2,
//              each term folded in by fma, float4s in ascending order;
//   wave:      xor-butterfly over lane distances 32, 16, 8, 4, 2, 1 (every lane ends with the same value);
//   workgroup: the 16 wave sums added in wave order;
//   scale = 1 / sqrt(sum / K + eps) with IEEE divide and square root (the model's rms_norm; the reference's
//   sqrtf_fast, cpu/common.hpp:310/448, is an exact sqrt on one ISA and a bit trick on another, cpu/avx_2.hpp:5382-5384);
//   y_i = (x_i * scale) * w_i: the rms_norm node, then the mul node with the norm weight (infra/core_traits.hpp:570-573).
__device__ __forceinline__ float sumsq_fold(float p, float4 v) {
	p = fmaf(v.x, v.x, p);
	p = fmaf(v.y, v.y, p);
	p = fmaf(v.z, v.z, p);
	return fmaf(v.w, v.w, p);
}
// (distances 8, 2 and 1 by lane patterns -- a rotation of a 16-lane row by 8 and the two quad swaps reach exactly lane ^ 8, ^ 2, ^ 1 --
// the others through the LDS crossbar: same partners, same sums)
__device__ __forceinline__ float wave_sum_butterfly(float p) {
	p = __fadd_rn(p, __shfl_xor(p, 32));
	p = __fadd_rn(p, __shfl_xor(p, 16));
	p = __fadd_rn(p, lane_pattern<DPP_ROW_ROTATE_8>(p));
	p = __fadd_rn(p, __shfl_xor(p, 4));
	p = __fadd_rn(p, lane_pattern<DPP_QUAD_SWAP_2>(p));
	p = __fadd_rn(p, lane_pattern<DPP_QUAD_SWAP_1>(p));
	return p;
}
// lane's share of run `wave` of a row of `groups` 128-value groups (K % 128 == 0)
__device__ __forceinline__ float rms_run_sumsq(const float* x, int groups, int wave, int lane) {
	const int q	 = groups / 16, r = groups % 16;
	const int g0 = wave * q + min(wave, r);
	const int n4 = (q + (wave < r ? 1 : 0)) * 32; // float4s in the run
	const float4* x4 = reinterpret_cast<const float4*>(x) + g0 * 32;
	float p			 = 0.0f;
	for (int j = lane; j < n4; j += 64) {
		p = sumsq_fold(p, x4[j]);
	}
	return p;
}
// red: 16 floats of LDS.  Contains a workgroup barrier: every thread of the 1024 must call it.
__device__ __forceinline__ float rms_scale_workgroup(float p, float* red, int wave, int lane, int K, float eps) {
	p = wave_sum_butterfly(p);
	if (lane == 0) {
		red[wave] = p;
	}
	__syncthreads();
	float sum = red[0];
#pragma unroll
	for (int w = 1; w < 16; ++w) {
		sum = __fadd_rn(sum, red[w]);
	}
	return __fdiv_rn(1.0f, sqrtf(__fadd_rn(__fdiv_rn(sum, static_cast<float>(K)), eps))); // sqrtf is correctly rounded; __fsqrt_rn maps to the 1-ulp native one
}
__device__ __forceinline__ float4 norm_mul4(float4 x, float scale, float4 w) {
	return make_float4(__fmul_rn(__fmul_rn(x.x, scale), w.x), __fmul_rn(__fmul_rn(x.y, scale), w.y), __fmul_rn(__fmul_rn(x.z, scale), w.z), __fmul_rn(__fmul_rn(x.w, scale), w.w));
}

// 16 bytes per lane from global memory straight into LDS (lane l of the wave lands at lds_dst + 16 * l), no destination
// registers.  Written as inline assembly rather than through the compiler's builtin because the compiler, not able
// to tell which later LDS access such a transfer feeds, waits for ALL outstanding loads (the whole weight stream)
// at the next LDS access.  The caller orders its LDS reads behind the transfer itself: loads complete in issue order,
// so waiting for any register load issued after this one is enough.  lds_dst must be wave-uniform.
__device__ __forceinline__ void load_global_to_lds_b128(const void* src, void* lds_dst) {
	const uint32_t lds_addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) char*)(static_cast<char*>(lds_dst))));
	// the LDS address travels in M0, which the compiler may hold a value in: saved and put back around the transfer
	uint32_t saved_m0;
	asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b32 m0, %0" : "=&s"(saved_m0) : "v"(src), "s"(lds_addr) : "memory");
}

// Blocks the wave until every memory operation it has issued, stores included, has been acknowledged.  Placed
// between device-scope (write-through) stores of data and the device-scope store or atomic that tells another
// workgroup the data is there: a workgroup-scope release fence does not wait for the stores on this target, and an
// agent-scope one also writes back the L2 under the other workgroups' streaming loads.
__device__ __forceinline__ void wait_stores_acknowledged() {
	asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// Byte offset of macro-tile (strip, group) in a tiled matrix with `groups` = K/128 groups per strip.
__device__ __host__ __forceinline__ int64_t macro_offset(int64_t strip, int64_t group, int64_t groups) {
	return (strip * groups + group) * MACRO_BYTES;
}

// ---- per-kernel timing (opt-in instrumentation, see q8_0_profile.hip) ----

enum kernel_kind : int { KIND_QUANTIZE = 0, KIND_GEMV = 1, KIND_GEMM = 2, KIND_GET_ROWS = 3, KIND_COUNT = 4 };

// The K range (in 128-quant groups) of one wave when a strip's `groups` are cut over `1 << split_shift` workgroups of `waves`
// waves each: the groups go to the workgroups as evenly as they can (the first groups % splits take one more), then each
// workgroup's share to its waves the same way.  Workgroups of one launch must not differ by more than a group: the CUs
// that host the heavier ones finish last, and the launch with them (handing the remainder to the first waves of the
// first workgroups instead cost the LLaMA-3-8B down projection 4 % of its time).  With one workgroup this is the cut
// the fixed-order RMS-norm sum is defined on.  All operands are wave-uniform.
__device__ __forceinline__ void wave_k_range(int groups, int split_shift, int split, int waves, int wave, int& g0, int& g1) {
	const int splits  = 1 << split_shift;
	const int s_q	  = groups >> split_shift, s_r = groups & (splits - 1);
	const int s_start = split * s_q + min(split, s_r);
	const int s_cnt	  = s_q + (split < s_r ? 1 : 0);
	const int w_q = s_cnt / waves, w_r = s_cnt % waves;
	g0 = s_start + wave * w_q + min(wave, w_r);
	g1 = g0 + w_q + (wave < w_r ? 1 : 0);
}

// True while `s` is being captured into a HIP graph.  A captured launch is replayed with the arguments it was recorded with,
// so nothing a replay-unsafe protocol hands to the kernel per launch (the epoch of the K-split hand-off and of the one-launch
// FFN's published blocks) would change between replays: launchers pick forms without such state for a capturing stream.
inline bool stream_is_capturing(hipStream_t s) {
	hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
	if (hipStreamIsCapturing(s, &st) != hipSuccess) {
		(void)hipGetLastError();
		return false;
	}
	return st != hipStreamCaptureStatusNone;
}

// hipStreamQuery of a stream that is not itself capturing, safe to call while ANOTHER stream of this thread is being captured
// in the global mode (where a query would be refused and would invalidate that capture): the thread's capture mode is
// relaxed for the duration of the call.
inline hipError_t query_stream_any_capture_mode(hipStream_t s) {
	hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
	if (hipThreadExchangeStreamCaptureMode(&mode) != hipSuccess) {
		(void)hipGetLastError();
		return hipStreamQuery(s);
	}
	const hipError_t q = hipStreamQuery(s);
	(void)hipThreadExchangeStreamCaptureMode(&mode);
	return q;
}

// When timing is on for `kind` and the event pool has room, hands out an event pair for the next launch.
bool profile_next(int kind, hipEvent_t* start, hipEvent_t* stop);

// Every compute kernel goes through here: a plain launch, or, while timing is on, a launch whose dispatch
// packet records GPU timestamps at the kernel's own start and end (what a kernel trace reports as its duration).
template<typename Kernel, typename... Args>
inline hipError_t launch_kernel(int kind, Kernel kernel, dim3 grid, dim3 block, size_t shmem, hipStream_t s, Args... args) {
	hipEvent_t e0, e1;
	if (profile_next(kind, &e0, &e1)) {
		hipExtLaunchKernelGGL(kernel, grid, block, static_cast<uint32_t>(shmem), s, e0, e1, 0, args...);
	} else {
		kernel<<<grid, block, shmem, s>>>(args...);
	}
	return hipGetLastError();
}

// ---- launch functions (defined one per .hip file, called from q8_0_abi.hip after argument checks) ----

hipError_t launch_quantize(const float* x, void* out, int64_t M, int64_t K, bool tiled, hipStream_t s);
hipError_t launch_rms_norm_quantize(const float* x, const float* norm_w, float eps, void* out, int64_t M, int64_t K, bool tiled, hipStream_t s);
hipError_t launch_silu_mul_quantize(const float* gate, const float* up, void* out, int64_t M, int64_t K, bool tiled, hipStream_t s);
hipError_t launch_tile(const void* blocks, void* tiled, int64_t rows, int64_t K, hipStream_t s);
hipError_t launch_untile(const void* tiled, void* blocks, int64_t rows, int64_t K, hipStream_t s);
hipError_t launch_get_rows(const void* W, const int32_t* ids, float* out, int32_t* invalid, int64_t n_tokens, int64_t n_rows, int64_t K, bool tiled, hipStream_t s);
hipError_t launch_fill_weights(void* blocks, uint64_t seed, int64_t first_block, int64_t n_blocks, hipStream_t s);
hipError_t launch_fill_activations(float* x, uint64_t seed, int64_t count, hipStream_t s);
// sums == nullptr: production; otherwise the same kernel diverts the per-block int32 sums to `sums` and leaves y alone.
hipError_t launch_gemv(const void* W, const void* xq_blocks, float* y, int32_t* sums, int64_t N, int64_t K, bool tiled, hipStream_t s);
// Streaming mat-vec on tiled weights for up to GEMV_MAX_SEGMENTS matrices that share K and the activation row:
// one launch computes y[i] = W[i] . x for all of them.  x is either one row of packed blocks (x_is_f32 = false)
// or the fp32 activations themselves, quantized inside the kernel (x_is_f32 = true).
constexpr int GEMV_MAX_SEGMENTS = 3;
hipError_t launch_gemv_tiled_multi(const void* const* W, float* const* y, const int64_t* N, int count, const void* x, bool x_is_f32, int64_t K, hipStream_t s,
	const float* norm_w = nullptr, float norm_eps = 0.0f, const float* const* residual = nullptr);
// The fused quantize + mat-vec of one matrix with the K-split hand-off going through a device array that is part of the
// code object: nothing is allocated.  gemv_noalloc_fits says whether the shape's cut fits that array.
bool gemv_noalloc_fits(int64_t N, int64_t K);
hipError_t launch_gemv_tiled_f32_noalloc(const void* W, const float* x, float* y, int64_t N, int64_t K, hipStream_t s);
hipError_t launch_ffn_decode(const void* w_gate, const void* w_up, const void* w_down, const float* x, const float* norm_w, float norm_eps, const float* residual, float* y, int64_t n_ff,
	int64_t K, int64_t n_out, hipStream_t s);
hipError_t copy_ffn_gate_up(float* gate_out, float* up_out, int64_t n_ff, hipStream_t s);
// attn_out + residual -> norm -> gate/up -> SiLU * up -> down + residual -> norm -> up to GEMV_MAX_SEGMENTS projections, one launch where
// the shape allows it (decode_layer_chains), else the three launches it stands for (q8_0_decode_layer.hip).  ffn_inp != l_out.
bool decode_layer_chains(int64_t n_embd, int64_t n_ff, int64_t next_strips);
hipError_t launch_decode_layer(const void* w_o, const float* attn, const float* layer_in, float* ffn_inp, const void* w_gate, const void* w_up, const void* w_down, const float* ffn_norm_w,
	float* l_out, const void* const* w_next, float* const* y_next, const int64_t* n_next, int count_next, const float* next_norm_w, float eps, int64_t n_embd, int64_t n_ff, hipStream_t s);
// Runs only the activation staging of the fused kernel and writes what it staged as packed blocks (parity check).
hipError_t launch_gemv_dump_staged_x(const float* x, void* xq_blocks_out, int64_t K, hipStream_t s, const float* norm_w = nullptr, float norm_eps = 0.0f);
// fp32 activations [M][K] against tiled Q8_0 weights without quantizing the activations (the reference's <float, block_q8_0, float>
// mul_mat, cpu/avx_2.hpp:4782-5004): y [M][N].  K == 0 gives zeros.
hipError_t launch_mul_mat_f32act(const void* W_tiled, const float* x, float* y, int64_t M, int64_t N, int64_t K, hipStream_t s);

// Mat-vecs that share nothing (own activation row, K, N) as one launch, up to GEMV_GROUP_MAX of them; the caller vouches that
// none of them reads or overwrites another's output.  launch_gemv_group takes matrices whose waves own at most four groups
// (anything plan_gemv can cut that way); launch_gemv_independent takes any list and falls back to single launches for the rest.
constexpr int GEMV_GROUP_MAX = 8;
struct gemv_group_op {
	const void* W; // tiled
	const float* x; // fp32 [K]
	float* y; // fp32 [N]
	const float* residual; // fp32 [N] or null
	int64_t N, K;
};
hipError_t launch_gemv_group(const gemv_group_op* ops, int count, hipStream_t s);
hipError_t launch_gemv_independent(const gemv_group_op* ops, int64_t count, hipStream_t s);

// 2 <= M <= GEMV_ROWS_MAX fp32 activation rows against one tiled weight matrix: the streaming mat-vec with M dot products per
// weight tile, quantize included (q8_0_gemv_rows.hip).  y is [M][N].
constexpr int64_t GEMV_ROWS_MAX = 3;
inline bool gemv_rows_suits(int64_t M, int64_t /*N*/, int64_t /*K*/) {
	return M >= 2 && M <= GEMV_ROWS_MAX;
}
hipError_t launch_gemv_rows(const void* W, const float* x, float* y, int64_t M, int64_t N, int64_t K, hipStream_t s, const float* residual = nullptr);
// 1 <= M <= 8 rows on the matrix cores, quantize included, no workspace (q8_0_gemv_rows_mfma.hip).  y is [M][N].
hipError_t launch_gemv_rows_mfma(const void* W, const float* x, float* y, int64_t M, int64_t N, int64_t K, hipStream_t s, const float* residual = nullptr);
// residual (tiled operands only, or null): C = W . Aq + residual, one fp32 add per element after its sum; may be C itself
hipError_t launch_gemm(const void* W, const void* Aq, float* C, int32_t* sums, int64_t M, int64_t N, int64_t K, bool tiled, hipStream_t s, const float* residual = nullptr);
// The prefill FFN's first half: act_out (tiled [M x n_ff]) = quantize_row_q8_0(silu(W_gate . Aq) * (W_up . Aq)), one launch where the shape
// allows it (plan_gate_up_fused in q8_0_plan.h), else two mat-mats into `workspace` (2 * M * n_ff floats) and the SiLU * up quantizer.
hipError_t launch_gemm_gate_up_silu(const void* w_gate, const void* w_up, const void* aq, void* act_out, float* gate_dbg, float* up_dbg, float* workspace, int64_t M, int64_t n_ff, int64_t K,
	hipStream_t s);
// Tiled operands, M <= GEMM_SKINNY_MAX_M (or a tile-kernel grid of at most one workgroup per CU): the streaming MFMA kernel
// of batched decode (q8_0_gemm_skinny.hip), which walks larger M in groups of 64 rows.
constexpr int64_t GEMM_SKINNY_MAX_M = 64;
// Make this device's K-split scratch buffers now (otherwise: on the first launch that needs one).
hipError_t prepare_gemv_scratch();
hipError_t prepare_gemm_scratch();
constexpr int64_t GEMM_SPLIT_SCRATCH_FLOATS = 2048 * 2 * 16 * 64; // partial tiles of a K split over workgroups
constexpr int GEMM_SPLIT_MAX_UNITS			  = 512; // arrival counters
hipError_t acquire_gemm_split_scratch(float** partials, unsigned** counters, hipStream_t s);
hipError_t launch_gemm_skinny(const void* W, const void* Aq, float* C, int32_t* sums, int64_t M, int64_t N, int64_t K, hipStream_t s, const float* residual = nullptr);

} // namespace nh
