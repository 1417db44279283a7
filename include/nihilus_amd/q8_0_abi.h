/*
 * q8_0_abi.h -- C ABI of the MI355X (gfx950) Q8_0 mat-mul path.
 *
 * Plain C, no HIP or torch types: pointers, sizes, an opaque stream.  Every pointer is a DEVICE
 * pointer unless the parameter name starts with host_.  `stream` is a hipStream_t passed as void*
 * (NULL = the default stream).  Calls are asynchronous on that stream and return once the work is
 * enqueued; nothing here allocates or frees caller-visible memory except nh_malloc / nh_free.
 * Return value: 0 on success, a negative nh_status for a rejected argument, or a positive
 * hipError_t value when the HIP runtime reported one.  No exception crosses this boundary.
 *
 * What each entry point replaces in the reference (paths relative to include/nihilus-incl/):
 * the reference has no FFI for this path; its boundary is the class-template specialisation point
 * kernel_dispatcher_impl<config, core_traits, device, arch, ...>::impl (common/kernel_traits.hpp:382-383,
 * called from infra/monolithic_dispatcher.hpp:41-63).  The C++ header mul_mat_dispatch.hpp supplies
 * those specialisations for device_types::gpu and forwards to the functions below; mega_dispatch.hpp does the same
 * for the reference's live dispatch point (the core_types key).
 *
 * Streams
 *   Launches that hand data between workgroups do so through scratch memory that the library keeps per GPU (made on first
 *   use or by nh_q8_0_prepare): nh_q8_0_gemv_tiled*, nh_q8_0_gemv_tiled_group_f32, nh_q8_0_mul_mat*, nh_q8_0_mul_mat_batch,
 *   nh_q8_0_mul_mat_f32_activations (each when the shape makes them split K over workgroups), nh_q8_0_gemm_tiled* for M <= 64,
 *   and nh_q8_0_ffn_f32 and nh_q8_0_decode_layer_f32 always.  That scratch serves ONE stream at a time per GPU: enqueue such calls on one stream, or let
 *   the other stream drain first.  A call that would use the scratch while a launch from a different stream may still be
 *   running returns NH_ERR_BUSY and launches nothing (not detected: work on a capturing stream, work that followed a
 *   launch on the NULL stream, and replays of captured graphs, which the caller must keep from overlapping).
 *   The check queries the other stream; it does so in the relaxed capture mode, so it may run while a third stream of the
 *   calling thread is being captured in the global mode without disturbing that capture.
 *   A kernel that waits for another workgroup's data does so for a bounded time; if it gives up, the output holds NaN and
 *   every nh_stream_sync and nh_q8_0_last_error on that GPU returns NH_ERR_DEVICE_TIMEOUT from then on, whichever stream or
 *   thread asks, until nh_q8_0_clear_error resets it (one word per GPU: it says that some launch failed, not which).
 *
 * Data layouts
 *   "blocks"  the reference's wire layout: rows of packed 34-byte block_q8_0 { fp16 d; int8 qs[32] }
 *             (common/data_types.hpp:38-44), row stride (K/32)*34 bytes, row-major.
 *   "tiled"   this library's device layout for streaming and MFMA operands, same byte count per
 *             block.  Rows are padded to a multiple of 32, K must be a multiple of 128.  The matrix
 *             is a sequence of 4352-byte macro-tiles indexed [row strip s = r/32][k group g = k/128]:
 *               bytes [t*1024 + 16*l + i], t<4, l<64, i<16 : quant (16*(l/32) + i) of block 4g+t of
 *                                                          row 32s + (l%32)
 *               bytes [4096 + 8*r + 2*t]                  : fp16 d of block 4g+t of row 32s + r
 *             so one 64-lane wavefront fetches a 32-row x 32-quant tile with a single fully
 *             coalesced 16-byte-per-lane load that already is a v_mfma_i32_32x32x32_i8 operand.
 */
#ifndef NIHILUS_AMD_Q8_0_ABI_H
#define NIHILUS_AMD_Q8_0_ABI_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NH_Q8_0_QK 32 /* Q_SIZE, common/data_types.hpp:28 */
#define NH_Q8_0_BLOCK_BYTES 34 /* sizeof(block_q8_0<half>), common/data_types.hpp:44 */

typedef enum nh_status {
	NH_OK			   = 0,
	NH_ERR_NULL_POINTER = -1, /* a required pointer is NULL */
	NH_ERR_ALIGNMENT   = -2, /* a pointer is not 16-byte aligned (arena slices are 64-byte aligned, infra/core_traits.hpp:130) */
	NH_ERR_SHAPE	   = -3, /* negative size, K % 32 != 0, or K % 128 != 0 for a tiled operand */
	NH_ERR_NO_DEVICE   = -4, /* no gfx950 device visible */
	NH_ERR_TOO_LARGE   = -5, /* a dimension exceeds what the launch grid or 32-bit tile indices hold */
	NH_ERR_ARGUMENT	   = -6, /* any other invalid argument */
	NH_ERR_IO		   = -7, /* a file could not be opened or mapped */
	NH_ERR_FORMAT	   = -8, /* a file is not what its reader accepts */
	NH_ERR_NOT_FOUND   = -9, /* no tensor or metadata key of that name */
	NH_ERR_BUSY		   = -10, /* the per-device scratch is still in use by a launch on ANOTHER stream: nothing was launched (see "Streams" below) */
	NH_ERR_DEVICE_TIMEOUT = -11 /* reported by nh_stream_sync / nh_q8_0_last_error: a kernel gave up a bounded wait, its output holds NaN */
} nh_status;

/* Library / device ------------------------------------------------------------------------------ */

/* Human-readable text for a status returned by any function here (static storage). */
const char* nh_status_string(int status);
/* Version of this ABI; bumps when a signature changes. */
int nh_abi_version(void);
/* Fills name (NUL-terminated, up to cap bytes) with the device's gcnArchName and *compute_units with its
 * CU count.  Stands in for the generated nihilus_gpu_properties.hpp (cuda/nihilus_gpu_properties.hpp:28-40). */
int nh_device_info(char* host_name, int64_t cap, int64_t* host_compute_units, int64_t* host_total_bytes);

/* Arena plumbing for hosts that must not see HIP headers: cudaMalloc / cudaMemcpy wrappers of
 * cuda/memory_buffer.hpp:78-152.  host_* pointers are host memory. */
int nh_malloc(void** host_out_dev_ptr, int64_t bytes);
int nh_free(void* dev_ptr);
int nh_memcpy_h2d(void* dst_dev, const void* host_src, int64_t bytes, void* stream);
int nh_memcpy_d2h(void* host_dst, const void* src_dev, int64_t bytes, void* stream);
/* hipMemsetAsync: not for a stream that is being captured into a HIP graph (it would record a memset node; every launch entry
 * point of this library clears memory with fill kernels instead and can be captured). */
int nh_memset(void* dst_dev, int value, int64_t bytes, void* stream);
/* Blocks until the stream has drained: the cudaDeviceSynchronize after each launch in cuda/cuda_12.hpp:679.  Returns
 * NH_ERR_DEVICE_TIMEOUT if a kernel on this GPU has given up a bounded wait since the last nh_q8_0_clear_error. */
int nh_stream_sync(void* stream);
/* The GPU's sticky device-side error, read without waiting for anything and without resetting it: NH_OK or
 * NH_ERR_DEVICE_TIMEOUT.  The reference looks at the device's error state after a launch only in dev builds
 * (cuda/cuda_12.hpp:650-655). */
int nh_q8_0_last_error(void);
/* Resets that error and returns what it held (NH_OK or NH_ERR_DEVICE_TIMEOUT): for the owner of the failed launch, once it has
 * dealt with the NaN output.  A sync of an unrelated stream never resets it. */
int nh_q8_0_clear_error(void);
/* Whether a launch may contain workgroups that wait (for a bounded time) for other workgroups of the same launch: the decode FFN
 * as one launch, a block's mat-vecs as one launch, the normalised row that the first workgroups of a large mat-vec work out for the
 * rest.  Those forms rest on workgroups being dispatched in index order, which holds on this hardware and is nowhere promised.
 * enabled = 0 switches them off for the whole process: nh_q8_0_ffn_f32 and nh_q8_0_decode_layer_f32 then run as the launches they
 * stand for (what a capturing stream gets), each depending on the one before only through stream order -- the reference's own
 * model, one kernel per op back to back (cuda/thread_pool.hpp:46-67) -- and every workgroup of a mat-vec with a norm works the
 * row out itself.  Same results (the fp32 sums of the one-launch forms may be cut differently: 1e-6 relative).  Returns the
 * previous setting (1 or 0); 1 by default.  Takes effect for calls made afterwards; needs no GPU. */
int nh_q8_0_set_in_kernel_waits(int enabled);
/* Allocates, for the current device, the two internal scratch buffers that K-split launches hand partial sums through
 * (about 2.6 MiB and 16 MiB; otherwise made by the first launch that needs one).  After it no launch entry point of this library
 * allocates device memory: call it once per device before capturing launches into a HIP graph or entering a serving loop.
 * No counterpart in the reference, whose kernels never allocate (infra/model.hpp:241 owns the arena). */
int nh_q8_0_prepare(void);

/* Activation quantize -------------------------------------------------------------------------- */

/* quantize_row_q8_0 for M rows (cpu/avx_2.hpp:4439-4489): x fp32 [M][K] row-major -> blocks [M][K/32].
 * Per block: d = fp16_rne(amax/127), q = int8(round_half_even(x * (127/amax))), amax == 0 -> all zero.
 * Bit-exact with the reference arithmetic.  K % 32 == 0 (the reference ignores a ragged tail, :4440;
 * here a ragged K is rejected so no byte is silently dropped). */
int nh_q8_0_quantize(const float* x, void* xq_blocks, int64_t M, int64_t K, void* stream);
/* Same values written in the tiled layout (rows padded with zero blocks to a multiple of 32). K % 128 == 0. */
int nh_q8_0_quantize_tiled(const float* x, void* xq_tiled, int64_t M, int64_t K, void* stream);

/* FFN activation fused into the quantizer: xq = quantize_row_q8_0(silu(gate) * up), element-wise over [M][K],
 * silu(g) = g / (1 + exp(-g)).  Stands for the reference's ffn_silu -> ffn_gate_par (mul) -> activation operand of
 * ffn_down chain (infra/core_traits.hpp:982-989; the silu and mul kernels are empty in the reference,
 * cpu/avx_2.hpp:1946-2075, so the formula is the model's).  exp is evaluated as a fixed sequence of fp32 operations
 * (see the CPU checker's nho_expf for the same sequence), which makes the quantized bytes reproducible bit for bit. */
int nh_q8_0_silu_mul_quantize(const float* gate, const float* up, void* xq_blocks, int64_t M, int64_t K, void* stream);
int nh_q8_0_silu_mul_quantize_tiled(const float* gate, const float* up, void* xq_tiled, int64_t M, int64_t K, void* stream);

/* RMS norm * weight fused into the quantizer: xq[m] = quantize_row_q8_0((x[m] * scale_m) * norm_weight),
 * scale_m = 1 / sqrt(mean(x[m]^2) + eps).  Stands for the rms_norm -> mul -> activation operand chain in front of
 * the q/k/v, gate/up and output projections (infra/core_traits.hpp:570-576, :971-974, :1186-1190; dead fused attempt
 * cpu/avx_2.hpp:5331-5384, whose sqrtf_fast is an exact square root on one ISA and a bit trick on another,
 * cpu/common.hpp:310/448: here it is the IEEE square root and divide).  The sum of squares is taken in a fixed order
 * (see the CPU checker's nho_rms_norm_scale for the same order), so the quantized bytes are reproducible.
 * x: fp32 [M][K]; norm_weight: fp32 [K]; 0 <= eps < 1; K % 128 == 0 for both output layouts. */
int nh_q8_0_rms_norm_quantize(const float* x, const float* norm_weight, float eps, void* xq_blocks, int64_t M, int64_t K, void* stream);
int nh_q8_0_rms_norm_quantize_tiled(const float* x, const float* norm_weight, float eps, void* xq_tiled, int64_t M, int64_t K, void* stream);

/* Layout conversion ---------------------------------------------------------------------------- */

/* Bytes of a [rows x K] matrix: blocks = rows*(K/32)*34 (type_traits<block_q8_0>::total_byte_size,
 * common/type_traits.hpp:38-61, :185-193); tiled = ceil(rows/32)*(K/128)*4352.  Negative on bad shape. */
int64_t nh_q8_0_blocks_bytes(int64_t rows, int64_t K);
int64_t nh_q8_0_tiled_bytes(int64_t rows, int64_t K);
/* blocks -> tiled (done once per weight at load time, where the reference copies weights into its
 * device arena: infra/model_parser.hpp:151-154) and back.  Lossless byte permutation. */
int nh_q8_0_tile(const void* blocks, void* tiled, int64_t rows, int64_t K, void* stream);
int nh_q8_0_untile(const void* tiled, void* blocks, int64_t rows, int64_t K, void* stream);

/* Token-embedding lookup (get_rows) ------------------------------------------------------------- */

/* out[t][j] = f32(d[ids[t]][j/32]) * f32(qs[ids[t]][j]),  t < n_tokens, j < K: one fp32 multiply per element,
 * bit-exact against the CPU.  Replaces the reference's live token_embeddings kernels, both phases
 * (cpu/avx_2.hpp:40-66, :68-140; per-op form :1241-1294; cuda/cuda_12.hpp:560-601, and :691-722 whose missing
 * token index is not reproduced).  W: the [n_rows x K] embedding matrix, device, blocks or tiled layout;
 * ids: int32 [n_tokens], device (global_input_types::inp_tokens); out: fp32 [n_tokens][K], device.
 * The reference reads whatever row an id names; here an id outside [0, n_rows) yields a row of zeros and, if
 * invalid_count is not NULL, adds one to that device int32 (the caller zeroes it). K % 32 == 0 (tiled: % 128). */
int nh_q8_0_get_rows(const void* W_blocks, const int32_t* ids, float* out, int32_t* invalid_count, int64_t n_tokens, int64_t n_rows, int64_t K, void* stream);
int nh_q8_0_get_rows_tiled(const void* W_tiled, const int32_t* ids, float* out, int32_t* invalid_count, int64_t n_tokens, int64_t n_rows, int64_t K, void* stream);

/* Mat-vec (decode, eval_time) ------------------------------------------------------------------- */

/* y[n] = sum_b f32(dW[n][b]) * f32(dx[b]) * sum_{j<32} W.qs[n][b][j] * x.qs[b][j]
 * = vec_dot_q8_0_q8_0<K/32> per output row (cpu/avx_2.hpp:4534-4747), the body the eval_time mul_mat
 * dispatcher was meant to have (cpu/avx_2.hpp:1371-1444).  Integer block sums are exact; the fp32
 * accumulation order differs from the CPU's (<= 1e-4 relative L2 over y is the contract, ~1e-7 in practice).
 * W: N rows, xq: one row of K/32 blocks (always the blocks layout: it is 34*K/32 bytes), y: fp32 [N]. */
int nh_q8_0_gemv(const void* W_blocks, const void* xq_blocks, float* y, int64_t N, int64_t K, void* stream);
int nh_q8_0_gemv_tiled(const void* W_tiled, const void* xq_blocks, float* y, int64_t N, int64_t K, void* stream);

/* Fused decode step: y = W . quantize(x) with the quantize done inside the mat-vec kernel (no separate launch, the
 * quantized row never travels through memory).  x: fp32 [K].  Same values as nh_q8_0_quantize + nh_q8_0_gemv_tiled. */
int nh_q8_0_gemv_tiled_f32(const void* W_tiled, const float* x, float* y, int64_t N, int64_t K, void* stream);
/* The same with the residual add of the layer behind it (attn_out mul_mat -> residual add, infra/core_traits.hpp:768-772):
 * y = W . Q(x) + residual, one fp32 add after the row's sum.  residual may be y itself (in-place accumulate). */
int nh_q8_0_gemv_tiled_residual_f32(const void* W_tiled, const float* x, const float* residual, float* y, int64_t N, int64_t K, void* stream);
/* nh_q8_0_gemv_tiled_f32 for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): same kernels, same cut of the matrix, same bits in y, but the partial sums that a K split
 * hands between workgroups go through a 512 KiB array that is part of the library's code object (one copy per GPU, held until
 * the process ends) instead of a buffer allocated on first use.  The call allocates and frees nothing.  A shape whose cut
 * needs more than NH_Q8_0_NOALLOC_MAX_SPLIT_UNITS (32-row strip, K part) slots is rejected with NH_ERR_TOO_LARGE before
 * anything is launched ([4096 x 14336] uses 512, [8192 x 28672] 2048; shapes that need no K split always fit).  Every call on
 * a GPU shares that GPU's array: two such calls must not overlap on one GPU (run them on one stream; a call on another stream
 * while the previous user's stream still has work in flight returns NH_ERR_BUSY and launches nothing, as described under
 * "Streams").  No counterpart in the reference, whose kernels never allocate (infra/model.hpp:241 owns the arena). */
#define NH_Q8_0_NOALLOC_MAX_SPLIT_UNITS 2048
int nh_q8_0_gemv_tiled_f32_noalloc(const void* W_tiled, const float* x, float* y, int64_t N, int64_t K, void* stream);
/* The same for up to 3 weight matrices that share K and x (q/k/v, gate/up: infra/core_traits.hpp:575-594, :976-986)
 * as ONE launch: y[i] = W_tiled[i] . quantize(x), i < count.  host_* arrays are host memory, read before return. */
int nh_q8_0_gemv_tiled_multi_f32(const void* const* host_W_tiled, float* const* host_y, const int64_t* host_N, int64_t count, const float* x, int64_t K, void* stream);
/* The same with the RMS norm in front: y[i] = W_tiled[i] . quantize((x * scale) * norm_weight), scale = 1 / sqrt(mean(x^2) + eps),
 * all inside the one launch (the values of nh_q8_0_rms_norm_quantize + nh_q8_0_gemv_tiled).  This is the decode-time
 * rms_norm -> mul -> q/k/v (or gate/up, or output) group of the reference's mega cores (infra/core_traits.hpp:570-594). */
int nh_q8_0_gemv_tiled_multi_norm_f32(const void* const* host_W_tiled, float* const* host_y, const int64_t* host_N, int64_t count, const float* x, const float* norm_weight, float eps,
	int64_t K, void* stream);

/* The decode-time FFN as one launch:  y = W_down . Q(silu(W_gate . Q(n)) * (W_up . Q(n))) [+ residual],  Q = quantize_row_q8_0,
 * n = x, or with norm_weight != NULL n = (x * scale) * norm_weight (RMS norm as in nh_q8_0_rms_norm_quantize).
 * Stands for the eval_time body of the reference's mega_ffn core: ffn_gate and ffn_up mul_mat, silu, mul, ffn_down
 * mul_mat, residual add (infra/core_traits.hpp:971-995; the GPU dispatcher that would hold it is empty,
 * cuda/cuda_12.hpp:806-916).  Same arithmetic as nh_q8_0_gemv_tiled_multi_[norm_]f32 (gate, up) followed by
 * nh_q8_0_silu_mul_quantize and nh_q8_0_gemv_tiled (down), with K cut differently (last-bit differences in the fp32
 * sums): the down projection's workgroups ride in the same grid and start streaming their weights while gate/up are
 * still running.
 * W_gate, W_up: [N_ff x K] tiled; W_down: [N_out x N_ff] tiled; x: fp32 [K]; residual: fp32 [N_out] or NULL;
 * y: fp32 [N_out] (may alias residual).  K % 128 == 0, N_ff % 128 == 0, N_ff <= NH_Q8_0_FFN_MAX_HIDDEN.
 * Uses the library's per-device scratch: two such calls must not overlap on one GPU. */
#define NH_Q8_0_FFN_MAX_HIDDEN 65536
int nh_q8_0_ffn_f32(const void* W_gate_tiled, const void* W_up_tiled, const void* W_down_tiled, const float* x, const float* norm_weight, float eps, const float* residual, float* y,
	int64_t N_ff, int64_t K, int64_t N_out, void* stream);

/* A transformer block's decode-time mat-vecs from one attention to the next as ONE launch:
 *   ffn_inp = W_o . Q(attn) + layer_in                                      attn_out mul_mat -> residual add     (mega_attention_apply, infra/core_traits.hpp:768-772)
 *   l_out   = W_down . Q(silu(W_gate . Q(n1)) * (W_up . Q(n1))) + ffn_inp   n1 = rms_norm(ffn_inp) * ffn_norm_weight   (mega_ffn, :971-995)
 *   y_next[i] = W_next[i] . Q(n2),  i < count_next <= 3                     n2 = rms_norm(l_out) * next_norm_weight
 * the last line being the NEXT block's q / k / v projections (mega_qkv_prep_and_cache_publish, :570-594) or, behind the last block,
 * the logits (final_norm_and_sampling, :1186-1193); count_next == 0 leaves it out.  The reference runs these cores as separate
 * synchronous launches per block (cuda/thread_pool.hpp:46-67); here the stages are ranges of one grid, and a stage's workgroups have
 * their weight loads in flight while they wait for the stage before (see q8_0_decode_layer.hip).  Same arithmetic as
 * nh_q8_0_gemv_tiled_residual_f32, nh_q8_0_ffn_f32 (norm and residual) and nh_q8_0_gemv_tiled_multi_norm_f32 run one after the other.
 * W_o: [N_embd x N_embd] tiled; W_gate, W_up: [N_ff x N_embd]; W_down: [N_embd x N_ff]; W_next[i]: [N_next[i] x N_embd];
 * attn, layer_in, ffn_inp, l_out: fp32 [N_embd]; y_next[i]: fp32 [N_next[i]]; host_* arrays are host memory, read before return.
 * ffn_inp, l_out and every y_next must be distinct buffers (layer_in may be any of the inputs).  N_embd, N_ff multiples of 128.
 * Shapes the one launch does not take (N_embd > 8192) and streams under HIP graph capture run the three launches instead.
 * Uses the library's per-device scratch: two such calls must not overlap on one GPU (NH_ERR_BUSY, see "Streams"). */
int nh_q8_0_decode_layer_f32(const void* W_o_tiled, const float* attn, const float* layer_in, float* ffn_inp, const void* W_gate_tiled, const void* W_up_tiled, const void* W_down_tiled,
	const float* ffn_norm_weight, float* l_out, const void* const* host_W_next_tiled, float* const* host_y_next, const int64_t* host_N_next, int64_t count_next,
	const float* next_norm_weight, float eps, int64_t N_embd, int64_t N_ff, void* stream);

/* `count` INDEPENDENT mat-vecs, each with its own fp32 activation row, K and N (host arrays of device pointers and sizes;
 * host_residual or any entry of it may be NULL): y_i = W_i . quantize(x_i) [+ residual_i].  None of them may read or
 * overwrite what another one writes (a residual that is the op's own y is fine); given that, they run as one launch per up to
 * eight matrices instead of one each, so the ~3 us a launch spends filling and draining the chip are paid once per group.
 * Each matrix is cut as its own launch would cut it, so results equal those of separate nh_q8_0_gemv_tiled_f32 calls (bit for
 * bit unless the separate call would split a small matrix by rows, then to fp32 summation order).  No counterpart in the
 * reference, whose per-op dispatch (cpu/avx_2.hpp:1296-1444) runs one mul_mat per call; nh_q8_0_mul_mat_batch uses it for
 * neighbouring entries it can prove independent. */
int nh_q8_0_gemv_tiled_group_f32(const void* const* host_W_tiled, const float* const* host_x, float* const* host_y, const float* const* host_residual, const int64_t* host_N,
	const int64_t* host_K, int64_t count, void* stream);

/* Mat-mat (prefill, prompt_eval_time) ----------------------------------------------------------- */

/* C[m*N + n] (n fastest, ggml's dst[ir1*nr0 + ir0], cpu/avx_2.hpp:4934) = the same dot for activation
 * row m: output dims [ne0 = N, ne1 = M] of kernel_traits_old<..., mul_mat, ...> (common/kernel_traits.hpp:393-417),
 * the body the prompt_eval_time dispatcher was meant to have (cpu/avx_2.hpp:1296-1369).
 * int8 MFMA (v_mfma_i32_32x32x32_i8) per 32-quant block, fp32 scale application per block. */
int nh_q8_0_gemm(const void* W_blocks, const void* Aq_blocks, float* C, int64_t M, int64_t N, int64_t K, void* stream);
int nh_q8_0_gemm_tiled(const void* W_tiled, const void* Aq_tiled, float* C, int64_t M, int64_t N, int64_t K, void* stream);
/* The tiled mat-mat with the add node behind the projection folded into its store (attn_out mul_mat -> residual add,
 * infra/core_traits.hpp:768-772; down mul_mat -> add, :988-992): C = W . Aq + residual, one fp32 add per element after its
 * sum.  residual: fp32 [M][N], may be C itself (in-place accumulate). */
int nh_q8_0_gemm_tiled_residual(const void* W_tiled, const void* Aq_tiled, const float* residual, float* C, int64_t M, int64_t N, int64_t K, void* stream);

/* The prefill FFN's first half as one call: act = quantize_row_q8_0(silu(W_gate . Aq) * (W_up . Aq)), written in the tiled layout as the
 * activation operand of the down projection (rows padded with zero blocks to a multiple of 32).  Stands for the ffn_gate and ffn_up
 * mul_mat -> ffn_silu -> ffn_gate_par (mul) chain of the reference's mega_ffn core in the prompt phase (infra/core_traits.hpp:976-989).
 * Where each matrix alone would take the prefill MFMA kernel it is ONE launch: every workgroup computes the same tiles of both
 * mat-mats against one activation image and applies SiLU * up and the quantizer to them in registers, so the two fp32 [M x N_ff]
 * intermediates are never written and no separate quantize launch runs (nh_q8_0_gate_up_silu_workspace_bytes == 0 for such a
 * shape).  Other shapes run nh_q8_0_gemm_tiled twice into `workspace` and nh_q8_0_silu_mul_quantize_tiled.  Either way the bytes are
 * those of that three-call sequence.  W_gate, W_up: [N_ff x K] tiled; Aq: [M x K] tiled; act: [M x N_ff] tiled; N_ff, K % 128 == 0. */
int64_t nh_q8_0_gate_up_silu_workspace_bytes(int64_t M, int64_t N_ff, int64_t K);
int nh_q8_0_gemm_tiled_gate_up_silu(const void* W_gate_tiled, const void* W_up_tiled, const void* Aq_tiled, void* act_tiled_out, void* workspace, int64_t workspace_bytes, int64_t M, int64_t N_ff,
	int64_t K, void* stream);

/* Fused mul_mat: fp32 activations in, fp32 out -------------------------------------------------- */

/* Scratch the fused call needs for the quantized activations (device bytes, 256-byte aligned by the caller);
 * 0 for M <= 3, where the quantize happens inside the mat-vec kernel and workspace may be NULL. */
int64_t nh_q8_0_mul_mat_workspace_bytes(int64_t M, int64_t K);
/* quantize(x) then GEMV (M == 1; M = 2, 3: the same kernel with one dot product per row; M = 4 ... 16 on matrices up to 40 MB, M = 4 up to
 * 80 MB: the same kernel with the rows as an MFMA operand -- all of these quantize inside the kernel and leave the workspace
 * untouched) or GEMM (otherwise: a quantize launch into the workspace, then an MFMA kernel) against a tiled weight: the whole
 * rms_norm-output -> projection step of core_traits.hpp:575-594 / :976-989 as one call. */
int nh_q8_0_mul_mat(const void* W_tiled, const float* x, float* y, int64_t M, int64_t N, int64_t K, void* workspace, int64_t workspace_bytes, void* stream);
/* The same with the add node behind the projection folded in: y = mul_mat(W, x) + residual (fp32 [M][N], may be y itself),
 * for any M (the attn_out and down projections of core_traits.hpp:768-772, :988-992 in either phase). */
int nh_q8_0_mul_mat_residual(const void* W_tiled, const float* x, const float* residual, float* y, int64_t M, int64_t N, int64_t K, void* workspace, int64_t workspace_bytes,
	void* stream);

/* fp32 activations against Q8_0 weights WITHOUT quantizing the activations: y[m][n] = sum_b f32(d_w) * sum_i x[m][32b+i] * q_w[i],
 * all in fp32.  The mul_mat the reference implements for the key <float, block_q8_0<half>, float> (leaf vec_dot_q8_f32,
 * cpu/avx_2.hpp:4782-4852; eval_time dispatcher :4978-5004, prompt_eval_time :4854-4976); not the path a model runs (that one
 * quantizes the activations, above), kept as a plain form: the weights are read once per activation row.  One row of a long K
 * (M == 1, K split over workgroups as in the mat-vec) goes through the library's per-device scratch: two such calls must not overlap
 * on one GPU. */
int nh_q8_0_mul_mat_f32_activations(const void* W_tiled, const float* x, float* y, int64_t M, int64_t N, int64_t K, void* stream);

/* One entry of a batch: y[M][N] = mul_mat(W_tiled [N x K], x fp32 [M][K]).  reuse_quantized_x != 0 lets the runner
 * skip the quantize when the previous entry quantized the same x pointer with the same M and K (q/k/v share the
 * normed hidden state, gate/up share the FFN input: infra/core_traits.hpp:575-594, :976-986).
 * ordered != 0: the entry starts only after every earlier entry has finished, whatever its pointers say (set it when
 * the entry depends on earlier ones through memory other than their x and y ranges).  With ordered == 0 the runner may
 * put neighbouring M == 1 entries into one launch when it can see from their x and y ranges that none reads or
 * overwrites what another writes; entries whose ranges do overlap always run in list order. */
typedef struct nh_q8_0_mul_mat_op {
	const void* W_tiled;
	const float* x;
	float* y;
	int64_t M, N, K;
	int32_t reuse_quantized_x;
	int32_t ordered;
} nh_q8_0_mul_mat_op;
/* Enqueues `count` mul_mat operations in order on one stream from native code: one call per decode step instead
 * of one per projection (the per-block fold of cuda/thread_pool.hpp:46-67 over the three mega cores).  host_ops is
 * host memory, read before return.  workspace must hold the largest nh_q8_0_mul_mat_workspace_bytes(M, K) of the
 * list; entries that use it run in stream order, so sharing it is safe.  The result is that of running the entries one
 * after another in list order (independent neighbours may share a launch, see nh_q8_0_mul_mat_op).  All entries are
 * validated before the first launch. */
int nh_q8_0_mul_mat_batch(const nh_q8_0_mul_mat_op* host_ops, int64_t count, void* workspace, int64_t workspace_bytes, void* stream);

/* Per-kernel timing (instrumentation) ----------------------------------------------------------- */

/* kernel_kind: 0 = quantize, 1 = mat-vec, 2 = mat-mat, 3 = get_rows.  Between begin and end every launch of that kind (up to
 * max_launches) records GPU timestamps at the kernel's own start and end.  nh_profile_end waits for them and
 * returns the summed, smallest and largest kernel durations in milliseconds.  Process-wide; not for concurrent use. */
int nh_profile_begin(int kernel_kind, int64_t max_launches);
int nh_profile_end(double* host_total_ms, int64_t* host_launches, double* host_min_ms, double* host_max_ms);
/* The shader clock the GPU holds right now, in MHz: one wavefront on a stream of its own counts shader clocks against the
 * constant 100 MHz timer for spin_us microseconds (1 .. 100000) beside whatever the caller has queued on other streams, and
 * the call returns when it is done.  The int8-MFMA peak is quoted at 2.4 GHz; under a matrix-bound launch the chip holds
 * less, and a figure against that peak cannot be read without the clock.  Allocates 16 bytes for the duration of the call. */
int nh_profile_shader_clock(double* host_mhz, int64_t spin_us);

/* Parity instrumentation ------------------------------------------------------------------------ */

/* Per-(m, n, block) int32 sums as the production kernels compute them (same device code path, results
 * diverted before scaling): sums[(m*N + n)*(K/32) + b].
 *   path 0  mat-vec kernel on the blocks layout (v_dot4), M must be 1; W and Aq in the blocks layout
 *   path 1  mat-mat kernel on the blocks layout (MFMA);             W and Aq in the blocks layout
 *   path 2  streaming mat-vec kernel on the tiled layout, M must be 1; W tiled, Aq = one row of blocks
 *   path 3  mat-mat kernel on the tiled layout (MFMA);               W and Aq tiled */
int nh_q8_0_debug_block_sums(const void* W, const void* Aq, int32_t* sums, int64_t M, int64_t N, int64_t K, int path, void* stream);

/* What the fused mat-vec stages for x: runs the fused kernel's own quantize-and-stage code on fp32 x [K] and writes
 * the staged row back as K/32 packed blocks, to be compared byte for byte with nh_q8_0_quantize (or, with a norm
 * weight, with nh_q8_0_rms_norm_quantize). K % 128 == 0. */
int nh_q8_0_debug_fused_quantize(const float* x, void* xq_blocks_out, int64_t K, void* stream);
int nh_q8_0_debug_fused_norm_quantize(const float* x, const float* norm_weight, float eps, void* xq_blocks_out, int64_t K, void* stream);
/* The gate and up projections' fp32 outputs of the last nh_q8_0_ffn_f32 on this device (they never leave the
 * library otherwise), copied out for comparison. */
int nh_q8_0_debug_ffn_gate_up(float* gate_out, float* up_out, int64_t N_ff, void* stream);

/* Which kernel nh_q8_0_mul_mat(M, N, K) runs and how that kernel cuts the work: the launchers execute exactly this plan, so a
 * test can pin the route of a shape (and a parity test can assert that the variant it means to cover is the one that runs).
 * Needs no GPU.  host_plan receives eight int32:
 *   [0] kernel: 0 nothing (empty problem), 1 fused quantize + streaming mat-vec (M == 1), 2 the same kernel with one dot product
 *       per row (a few rows), 3 weight-streaming MFMA kernel, 4 MFMA tile kernel with non-temporal weights (batched decode on
 *       large matrices), 5 MFMA tile kernel (prefill), 6 the streaming mat-vec with four to sixteen rows as an MFMA operand, quantize
 *       inside (small matrices);
 *   [1] 1 when the activations are quantized by a launch of their own into the workspace (kernels 3, 4, 5);
 *   kernel 1, 6: [2] workgroups per 32-row strip along K, [3] 128-quant groups per wave, [4] row parts per strip;
 *   kernel 3:    [2] 32-row activation strips per workgroup, [3] workgroups per weight strip along K;
 *   kernel 4, 5: [2] activation strips per wave, [3] K sets of four waves per workgroup, [4] workgroups per tile along K,
 *                [5], [6] the grid (column blocks of 128 weight rows, groups of activation strips);
 *   the rest 0.  The same shape under HIP graph capture may take a form without state between launches (no K split). */
int nh_q8_0_debug_plan_mul_mat(int64_t M, int64_t N, int64_t K, int32_t* host_plan);

/* nh_q8_0_gemm_tiled_gate_up_silu with the fp32 outputs of the two mat-mats copied out as well (gate_out, up_out: [M][N_ff]), so that
 * the quantized activation can be compared with the CPU quantizer applied to exactly the sums the launch computed. */
int nh_q8_0_debug_gemm_tiled_gate_up_silu(const void* W_gate_tiled, const void* W_up_tiled, const void* Aq_tiled, void* act_tiled_out, float* gate_out, float* up_out, int64_t M, int64_t N_ff,
	int64_t K, void* stream);

/* How many polls a workgroup of nh_q8_0_ffn_f32 waits for another workgroup's data before it gives up (default and upper
 * limit 2^20, lower limit 1).  Test hook for the time-out report: with a limit of 1 the down projection's workgroups find
 * their activation missing and give up while every kernel still runs to its end.  Process-wide, and refused with
 * NH_ERR_ARGUMENT unless the process was started with NH_Q8_0_DEBUG_HOOKS=1 in its environment. */
int nh_q8_0_debug_set_spin_limit(int64_t polls);

/* Synthetic inputs (benchmark / test utility) --------------------------------------------------- */

/* Counter-based generator, identical by specification to the CPU checker's: weight blocks with quants uniform in
 * [-127,127] and d = fp16(|g|*0.01), activations g, g ~ Irwin-Hall(12) standardised.  first_block offsets the
 * counter so several matrices can be drawn from one seed. */
int nh_q8_0_fill_weight_blocks(void* blocks, uint64_t seed, int64_t first_block, int64_t n_blocks, void* stream);
int nh_q8_0_fill_activations(float* x, uint64_t seed, int64_t count, void* stream);

#ifdef __cplusplus
}
#endif
#endif
