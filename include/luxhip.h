/*
 * libluxhip -- C ABI of the MI355X (gfx950) backend for LuxLib's fused operators.
 *
 * The reference (LuxDL/Lux.jl, lib/LuxLib) has no C interface: a backend plugs in by adding
 * Julia methods on LuxLib.Impl's device-dispatch points.  Every entry point below names the
 * reference function(s) it stands behind (paths relative to lib/LuxLib/ of the reference).
 *
 * Conventions (modelled on the reference's vendor wrappers, ext/CUDAExt/cublaslt.jl:185-293
 * and ext/cuDNNExt/batchnorm.jl:81-118,221-241):
 *   - all tensors are dense, column-major (Julia order), passed as raw device pointers that
 *     the library only borrows for the duration of the call;
 *   - sizes are int64_t; leading dimensions are in elements;
 *   - every op is enqueued on the given stream and returns without synchronising the host;
 *   - return value: LUXHIP_OK, or a negative status.  LUXHIP_UNSUPPORTED (-1) means "this
 *     dtype / activation / shape is not handled" and the caller falls back to its generic
 *     path, exactly like cublaslt.jl:359-402; shape errors are expected to be raised by the
 *     host *before* the call (impl/matmul.jl:21-34, api/groupnorm.jl:40-64) and come back as
 *     LUXHIP_INVALID if they are not;
 *   - no exception crosses the ABI; luxhip_last_error() returns the message of the last
 *     failure on the calling thread;
 *   - optional tensors are passed as NULL (Julia `nothing`);
 *   - dtype selects the storage type of every tensor argument; arithmetic and reductions
 *     are carried in fp32 for both storage types.  Saved statistics are always fp32.
 */
#ifndef LUXHIP_H
#define LUXHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LUXHIP_OK 0
#define LUXHIP_UNSUPPORTED (-1)
#define LUXHIP_INVALID (-2)
#define LUXHIP_HIP_ERROR (-3)
#define LUXHIP_NOT_INITIALIZED (-4)

/* storage types */
#define LUXHIP_F32 0
#define LUXHIP_BF16 1
/* bf16 storage with one tensor of the call kept in fp32: accepted only where a function's comment
 * says which tensor that is (the products and the softmax passes of attention) */
#define LUXHIP_BF16_WIDE 2

/* activation ids.  tanh_fast / sigmoid_fast (NNlib.fast_act, src/layers/basic.jl:366-371 of
 * the reference) map to TANH / SIGMOID on the host side. */
#define LUXHIP_ACT_IDENTITY 0
#define LUXHIP_ACT_RELU 1
#define LUXHIP_ACT_TANH 2
#define LUXHIP_ACT_SIGMOID 3
#define LUXHIP_ACT_SWISH 4
#define LUXHIP_ACT_GELU 5 /* tanh approximation (NNlib.gelu) */
#define LUXHIP_ACT_SOFTPLUS 6
#define LUXHIP_ACT_LOGSIGMOID 7
#define LUXHIP_ACT_LISHT 8
#define LUXHIP_ACT_COUNT 9

typedef void* luxhip_stream_t; /* a hipStream_t; NULL is the null stream */
typedef void* luxhip_event_t;  /* a hipEvent_t */

/* ---------------------------------------------------------------- runtime ------------
 * The reference leaves device buffers and streams to CUDA.jl / AMDGPU.jl (task-local
 * handles, ext/CUDAExt/cublaslt.jl:80-82,156-178; CUDA.stream() :287).  This library owns
 * them instead.
 * One device per process: luxhip_init(device) binds the library to that device until
 * luxhip_shutdown; a second call with the same device is a no-op, with another device it returns
 * LUXHIP_INVALID ("already initialised on device N").  More than one GPU means one process per GPU. */
int luxhip_init(int device);
int luxhip_shutdown(void);
const char* luxhip_last_error(void);
int luxhip_device_info(char* name, size_t name_len, int* compute_units, int64_t* total_mem);

int luxhip_stream_create(luxhip_stream_t* out);
int luxhip_stream_synchronize(luxhip_stream_t s);
int luxhip_stream_destroy(luxhip_stream_t s);

/* Sizes the stream's scratch memory (reduction partials, operand copies of the contractions) to at
 * least `bytes` ahead of time.  Operators grow it on demand without making the host wait for the
 * device (the outgrown block is retired behind an event on the stream), but not while the stream
 * records a HIP graph: there a call that finds it too small returns LUXHIP_INVALID.  A caller that
 * records graphs runs each operator once eagerly before, or reserves here.  A recorded graph keeps
 * the address of the block that the stream had while it was recorded: if a later eager call on that
 * stream outgrows the block, the library keeps the old block allocated (it is never reused until
 * luxhip_shutdown, also when the stream is destroyed), so replays stay valid; they then use their
 * own scratch memory and must not overlap with each other, as before.  No counterpart in the
 * reference, whose vendor wrappers allocate their scratch arrays per call
 * (ext/cuDNNExt/batchnorm.jl:17-18). */
int luxhip_reserve(luxhip_stream_t s, size_t bytes);

int luxhip_event_create(luxhip_event_t* out);
int luxhip_event_record(luxhip_event_t e, luxhip_stream_t s);
int luxhip_event_elapsed_ms(float* ms, luxhip_event_t start, luxhip_event_t stop); /* waits for stop */
int luxhip_event_destroy(luxhip_event_t e);

/* Per-kernel timing (no counterpart in the reference, which has no tracing for its native GPU
 * path): while enabled, every kernel launch is timed with HIP events on its own stream.  The
 * streaming kernels (bias_activation, batchnorm, groupnorm, layernorm) hand two events to their
 * dispatch, which signals them at the begin and at the end of the kernel itself: the duration a
 * kernel trace reports.  The other launches are bracketed by events recorded around them (the
 * kernel plus the gap to the launch before it).  luxhip_profile_report synchronises, writes a JSON array of {kernel, count, total_ms, min_ms,
 * max_ms} into buf and clears the log. */
int luxhip_profile_enable(int on);
/* Tuning switches (no counterpart in LuxLib; tests use them to reach every code path):
 *   "bn_resident"   1 (default) / 0: single-pass batchnorm kernels that keep the tensor in registers
 *   "bn_spin_limit" polls after which a resident batchnorm workgroup stops waiting for its peer
 *                   workgroups and recomputes their share itself (default 2^22; 0 = never wait)
 *   "gemm_tile"     0 automatic (default), 82 | 42 | 22 | 11 force a GEMM tile shape
 *   "gemm_pretranspose" 1 (default) / 0: large bf16 matmul operands that are contiguous along m or n
 *                   are first copied into the k-contiguous layout the fastest kernel reads
 *   "workspace_epoch" (tests) the epoch from which the per-stream exchange words continue; the 32-bit
 *                   epoch wraps after 2^32 calls, at which point the library clears those words
 *   "conv_tile"     0 automatic (default); bf16 whole-tap convolution kernels: 82 = 256x256 tile on
 *                   8 waves, 84 / 83 = 512x128 on 8 waves with 4 / 3 LDS stages, 42 = 256x128 on 4 waves;
 *                   1 / 2: the 3x3 window kernel in tiles of 64 / 128 output channels whatever their number */
int luxhip_set_option(const char* name, int64_t value);
int luxhip_profile_report(char* buf, size_t len);

/* Achievable peaks of the device (no counterpart in the reference; the benchmark reports them next to
 * the published figures its roofline fractions divide by): a streaming copy of 512 MiB (GB/s of read +
 * written bytes), and register-only loops of v_mfma_f32_16x16x32_bf16 / v_mfma_f32_32x32x2_f32 on
 * pseudo-random operands, eight waves per compute unit, after a warm-up that lets the clocks settle
 * (TFLOP/s).  Any pointer may be NULL to skip that measurement.  Synchronises the stream; allocates and
 * frees 1 GiB of device memory. */
int luxhip_measure_peaks(luxhip_stream_t s, double* copy_GBps, double* mfma_bf16_TFLOPs, double* mfma_f32_TFLOPs);

/* Pooled device allocator, in place of the array package's pool that serves the reference's `similar`
 * calls (e.g. the outputs of src/impl/dense.jl:46-57, src/impl/conv.jl:62-72) (size-bucketed free lists; luxhip_free returns the block to the
 * pool, luxhip_trim releases the pool to the driver).  A freed block can be handed out again at
 * once: work that still uses it must have been enqueued on the stream on which the next owner will
 * enqueue (one stream: always true), or be finished - a caller with several streams synchronises
 * the stream that last used a block before freeing it. */
int luxhip_malloc(void** out, size_t bytes);
int luxhip_free(void* p);
int luxhip_trim(void);
int luxhip_memcpy_h2d(void* dst, const void* src, size_t bytes, luxhip_stream_t s); /* synchronous w.r.t. host */
int luxhip_memcpy_d2h(void* dst, const void* src, size_t bytes, luxhip_stream_t s); /* synchronous w.r.t. host */
int luxhip_memcpy_d2d(void* dst, const void* src, size_t bytes, luxhip_stream_t s); /* asynchronous */
int luxhip_fill_zero(void* dst, size_t bytes, luxhip_stream_t s);                   /* fill kernel, capturable */

/* out = convert(eltype_out, in) for n elements (bf16: round to nearest even).  The reference promotes
 * operands of mixed element types to the widest one before its fused dense and convolution kernels
 * (ext/CUDAExt/cublaslt.jl:46-63, src/impl/conv.jl:11-19); a host layer does the same with this and
 * takes the gradients back to each operand's own type. */
int luxhip_convert(luxhip_stream_t s, int dtype_in, int dtype_out, int64_t n, const void* in, void* out);

/* ---------------------------------------------------------------- bias_activation ----
 * x, y, pre, delta, out, dx: (I, C, N) column-major, I = product of the leading dims,
 * C = size(x, ndims-1), N = size(x, ndims).  bias, dbias: length C. */

/* y = act.(x .+ bias).  Stands behind Impl.bias_activation!(y, ::GPUBroadcastOp, act, x, bias)
 * (src/impl/bias_activation.jl:207-220) and Impl.activation! (src/impl/activation.jl:113-124)
 * when bias == NULL.  y may alias x (bias_activation!!, :143-152).  If pre != NULL it
 * receives x .+ bias (the `tmp` kept by the rrule, :86-95, and by bias_activation_cached!!,
 * :312-351). */
int luxhip_bias_activation_fwd(luxhip_stream_t s, int dtype, int act, int64_t I, int64_t C, int64_t N,
                               const void* x, const void* bias, void* y, void* pre);

/* dx = delta .* act'(out, pre);  dbias[c] = sum_{i,n} dx[i,c,n].  Stands behind
 * Impl.∇activation(::GPUBroadcastOp, Δ, out, act, x) (src/impl/activation.jl:139-141) fused
 * with Impl.∇bias_add / reduce_sum (src/impl/common_ops.jl:25-38), i.e. the pullbacks at
 * src/impl/bias_activation.jl:76-95.  out may be NULL for IDENTITY; pre may be NULL for
 * activations whose derivative needs only the output (identity, relu, tanh, sigmoid);
 * dbias may be NULL; dx may alias delta. */
int luxhip_bias_activation_bwd(luxhip_stream_t s, int dtype, int act, int64_t I, int64_t C, int64_t N,
                               const void* delta, const void* out, const void* pre, void* dx, void* dbias);

/* luxhip_bias_activation_bwd for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  Same arguments and results; the partial sums and arrival counters of the bias
 * gradient live in a fixed block of 2.25 MiB of device memory that the library holds per device from
 * luxhip_init to the end of the process, instead of the stream's workspace, and the call makes no
 * hipMalloc / hipFree and takes nothing from the library's pool (with luxhip_profile_enable off).
 * Limit: the partial sums (4 C S bytes with at most 256 slices S per
 * channel for I >= 64; 4 I C S bytes with S <= ceil(N / 8) batch slices otherwise) must fit 2 MiB:
 * larger shapes return LUXHIP_INVALID.  All calls on a device share the block, which keeps the last
 * call's contents (the counters are cleared on the stream by each call): calls that overlap in time
 * on one device, i.e. on different streams, race. */
int luxhip_bias_activation_bwd_noalloc(luxhip_stream_t s, int dtype, int act, int64_t I, int64_t C, int64_t N,
                                       const void* delta, const void* out, const void* pre, void* dx, void* dbias);

/* ---------------------------------------------------------------- batchnorm ----------
 * x, y, delta, dx: (I, C, N); gamma, beta, rmean, rvar, rmean_out, rvar_out, dgamma, dbeta:
 * length C in `dtype`; save_mean, save_invstd: length C, fp32. */

/* Whole-op override of Impl.batchnorm (src/impl/batchnorm.jl:29-49; precedent
 * ext/cuDNNExt/cuDNNExt.jl:26-54): statistics (compute_batch_statistics,
 * src/impl/normalization.jl:116-143), running-stat update (:20-110,
 * update_running_statistics_kernel! :78-93), and y = act(x*γ' + β')
 * (batchnorm_affine_normalize_internal_kernel!, src/impl/batchnorm.jl:333-403).
 * training != 0: batch statistics (biased variance); when rmean/rvar are given,
 *   rmean_out = (1-m) rmean + m μ and rvar_out = (1-m) rvar + m n/(n-1) σ² are written
 *   (new arrays; the inputs are not modified).
 * training == 0: rmean/rvar are the statistics (batch statistics if they are NULL).
 * gamma and beta are given together or both NULL.  save_mean / save_invstd (optional)
 * receive μ and 1/sqrt(σ²+eps) for the pullback. */
int luxhip_batchnorm_fwd(luxhip_stream_t s, int dtype, int act, int64_t I, int64_t C, int64_t N,
                         const void* x, const void* gamma, const void* beta, const void* rmean,
                         const void* rvar, int training, double momentum, double eps, void* y,
                         void* rmean_out, void* rvar_out, float* save_mean, float* save_invstd);

/* Complete pullback w.r.t. (x, γ, β): ∇activation, ∇batchnorm_affine_normalize
 * (src/impl/batchnorm.jl:445-663) and the mean_var rrule (src/impl/common_ops.jl:45-61)
 * in two passes over (delta, x).  The pre-activation is recomputed from x and the saved
 * statistics, so no activation intermediate is needed.  stats_from_batch == 0 treats the
 * statistics as constants (inference: only dx = ∂y γ').  dgamma / dbeta may be NULL. */
int luxhip_batchnorm_bwd(luxhip_stream_t s, int dtype, int act, int64_t I, int64_t C, int64_t N,
                         const void* delta, const void* x, const void* gamma, const void* beta,
                         const float* save_mean, const float* save_invstd, int stats_from_batch,
                         void* dx, void* dgamma, void* dbeta);

/* ---------------------------------------------------------------- groupnorm ----------
 * x viewed as (I, C/G, G, N) (src/impl/groupnorm.jl:13-15,76): channel c = j + (C/G) k.
 * gamma, beta, dgamma, dbeta: length C; save_mean, save_invstd: (G, N) fp32. */

/* Impl.groupnorm (src/impl/groupnorm.jl:5-22) = statistics per (group, sample) +
 * groupnorm_affine_normalize_kernel! (:315-347). */
int luxhip_groupnorm_fwd(luxhip_stream_t s, int dtype, int act, int64_t I, int64_t C, int64_t G, int64_t N,
                         const void* x, const void* gamma, const void* beta, double eps, void* y,
                         float* save_mean, float* save_invstd);

/* Pullback: ∇groupnorm_affine_normalize (src/impl/groupnorm.jl:383-598) + mean_var rrule. */
int luxhip_groupnorm_bwd(luxhip_stream_t s, int dtype, int act, int64_t I, int64_t C, int64_t G, int64_t N,
                         const void* delta, const void* x, const void* gamma, const void* beta,
                         const float* save_mean, const float* save_invstd, void* dx, void* dgamma,
                         void* dbeta);

/* instancenorm in training mode with running statistics in one launch: luxhip_groupnorm_fwd with G = C whose
 * workgroups also make the update that luxhip_instancenorm_running_stats describes (the workgroup of a
 * channel that finishes last averages the channel's N slice statistics, in sample order).  save_mean,
 * save_invstd: (C, N) fp32, required. */
int luxhip_instancenorm_fwd(luxhip_stream_t s, int dtype, int act, int64_t I, int64_t C, int64_t N, const void* x,
                            const void* gamma, const void* beta, double eps, void* y, float* save_mean, float* save_invstd,
                            double momentum, const void* rmean, const void* rvar, void* rmean_out, void* rvar_out);
/* instancenorm = the groupnorm kernels with G = C (statistics per channel and sample,
 * src/impl/normalization.jl:191-208) plus, in training with running statistics, this update
 * (update_normalization_statistics, src/impl/normalization.jl:91-110, reduce dims 1..N-2):
 *   rmean_out[c] = (1-m) rmean[c] + m mean_n(mu[c,n]),
 *   rvar_out[c]  = (1-m) rvar[c]  + m I/(I-1) mean_n(var[c,n]),   var = max(1/invstd^2 - eps, 0)
 * (luxhip_instancenorm_fwd uses the slice variances themselves, which stay exact where var << eps).
 * save_mean, save_invstd: (C, N) fp32 as written by luxhip_groupnorm_fwd with G = C and the same
 * eps; rmean, rvar, rmean_out, rvar_out: length C in the storage dtype. */
int luxhip_instancenorm_running_stats(luxhip_stream_t s, int dtype, int64_t I, int64_t C, int64_t N,
                                      const float* save_mean, const float* save_invstd, double eps,
                                      double momentum, const void* rmean, const void* rvar, void* rmean_out,
                                      void* rvar_out);

/* ---------------------------------------------------------------- attention ----------
 * scaled_dot_product_attention (src/impl/attention.jl:5-117) = batched_matmul(k, q .* scale) ->
 * apply_attention_mask_bias -> softmax over the key positions -> batched_matmul(v, probs).  The two
 * products are luxhip_batched_matmul_strided calls; these are the passes between them.
 * logits, probs, dprobs, dlogits: (S, L, H, B) column-major, S = key positions.
 * dtype LUXHIP_BF16_WIDE: bf16 storage, but the logits (forward) and dprobs (pullback) are fp32 as
 * luxhip_batched_matmul_strided writes them under the same dtype: a logit rounded to bf16 carries
 * an error of 2^-9 |logit|, which the exponential turns into a relative error of that size in the
 * weight; with the two tensors in fp32 the weights and gradients stay within the bf16 parity bar. */

/* probs[:, l, h, b] = softmax_s(scale * logits[s, l, h, b] + bias[s, l, h, b], -inf where masked)
 * (apply_attention_mask_bias, src/impl/attention.jl:119-128; NNlib.softmax(...; dims=1), :94-104).
 * The scale multiplies the logits here instead of q before the product (:98).  causal != 0: keep
 * s <= l (make_causal_mask, :130-134).  mask: bytes, non-zero = keep, or NULL; bias: storage dtype
 * or NULL; both (S, L, H or 1, B or 1): the strides (in elements) along h and b are 0 where the
 * extent is 1. */
int luxhip_attention_softmax_fwd(luxhip_stream_t s, int dtype, int64_t S, int64_t L, int64_t H, int64_t B,
                                 const void* logits, double scale, int causal, const uint8_t* mask,
                                 int64_t mask_stride_h, int64_t mask_stride_b, const void* bias,
                                 int64_t bias_stride_h, int64_t bias_stride_b, void* probs);

/* Pullback of the same (the softmax rule of NNlib, reached by AD in the reference):
 * dlogits = scale * probs .* (dprobs - sum_s dprobs .* probs); cols = L * H * B.  causal != 0:
 * 16-byte vectors of a column that lie wholly past s = l are neither read from dprobs / probs
 * (tiles of dprobs that structure 1 left untouched) nor computed: zeros are stored up to the end of
 * the block of 128 key positions that holds s = l, which is as far as the products with structure
 * 2 or 3 read; dlogits past that block is left untouched. */
int luxhip_attention_softmax_bwd(luxhip_stream_t s, int dtype, int64_t S, int64_t L, int64_t cols, int causal,
                                 const void* dprobs, const void* probs, double scale, void* dlogits);

/* The two steps above the pullback of the attention weights in one: the batched product
 * dprobs = v' d_out (the pullback of batched_matmul(v, probs), src/impl/batched_mul.jl:320-334) with the
 * softmax rule as its epilogue, dlogits = scale * probs .* (dprobs - sum_s dprobs .* probs).  The inner
 * sum equals sum_e d_out[e, l] out[e, l] (out = v probs), so it is taken from the forward result and the
 * cotangent of the weights never goes to memory (and stays fp32 in bf16 storage).  The identity holds for
 * the unrounded out: with dtype LUXHIP_BF16_WIDE `out` is the fp32 result of the forward product
 * (luxhip_batched_matmul_strided under the same dtype), which the caller keeps beside the bf16 array it
 * returns; an out rounded to bf16 shifts whole columns of dlogits by probs times the rounding error.
 * v: (Ev, S) per product with leading dimension ldv and batch strides strides_v; d_out, out: (Ev, L) with
 * ldo and strides_o (the same array layout); probs, dlogits: (S, L) with ldc and strides_c; batch_dims as
 * in luxhip_batched_matmul_strided.  structure 1: tiles with every s > l are left untouched (causal mask).
 * Not for calls with an fdrop (the weights that multiply v are then not the softmax result): those take
 * luxhip_batched_matmul_strided and luxhip_attention_softmax_bwd. */
int luxhip_attention_weights_pullback(luxhip_stream_t s, int dtype, int64_t S, int64_t L, int64_t Ev,
                                      const int64_t* batch_dims, const void* v, int64_t ldv,
                                      const int64_t* strides_v, const void* d_out, const void* out, int64_t ldo,
                                      const int64_t* strides_o, const void* probs, double scale, void* dlogits,
                                      int64_t ldc, const int64_t* strides_c, int structure);

/* ---------------------------------------------------------------- dropout ----------
 * The reference draws its noise with `rand!(rng, y)` from the array package's generator
 * (src/impl/dropout.jl:171-190); here a counter-based Philox4x32-10 stream stands in for it:
 * element e takes lane e % 4 of the block with counter offset + e / 4 under the 64-bit key `seed`.
 * A caller advances `offset` by ceil(n / 4) per call (the analogue of the replicated rng that the
 * reference returns).  Uniform values in [0, 1): (u >> 8) 2^-24 (fp32), (u >> 24) 2^-8 (bf16). */

/* rand!(rng, out) (src/impl/dropout.jl:173-176, 186-187). */
int luxhip_rand_uniform(luxhip_stream_t s, int dtype, int64_t n, uint64_t seed, uint64_t offset, void* out);

/* dropout with a full-size mask in one pass (src/impl/dropout.jl:3-6): mask = (noise > T(p)) T(invp)
 * (generate_dropout_mask!, :200-218), y = x .* mask (dropout_dot_mul, :220); the noise is never
 * stored.  x == y == NULL: only the mask (generate_dropout_mask, :179-190, for masks that are
 * broadcast over x).  mask == NULL: only y. */
int luxhip_dropout_fwd(luxhip_stream_t s, int dtype, int64_t n, uint64_t seed, uint64_t offset, double p,
                       double invp, const void* x, void* y, void* mask);

/* Impl.generate_dropout_mask!(y, opmode, p, invp) (src/impl/dropout.jl:200-218) on stored noise,
 * in place: y = (y > T(p)) T(invp). */
int luxhip_dropout_mask(luxhip_stream_t s, int dtype, int64_t n, double p, double invp, void* noise_to_mask);

/* dropout_dot_mul(x, mask) = x .* mask (src/impl/dropout.jl:220) and its pullback dx = delta .* mask
 * (:222-228).  mask_shape[d] is x_shape[d] or 1 (dropout_shape, :74-78); both column-major. */
int luxhip_dropout_mul(luxhip_stream_t s, int dtype, int ndim, const int64_t* x_shape, const int64_t* mask_shape,
                       const void* x, const void* mask, void* y);

/* alpha_dropout(opmode, noise, p, x, alpha, A, B) (src/impl/dropout.jl:84-89):
 * y = muladd(ifelse(noise > p, x, T(alpha)), T(A), T(B)); pullback (:137-150): dx = delta (noise > p) A. */
int luxhip_alpha_dropout_fwd(luxhip_stream_t s, int dtype, int64_t n, const void* noise, double p, const void* x,
                             double alpha, double A, double B, void* y);
int luxhip_alpha_dropout_bwd(luxhip_stream_t s, int dtype, int64_t n, const void* noise, double p,
                             const void* delta, double A, void* dx);

/* ---------------------------------------------------------------- layernorm ----------
 * x, y, delta, dx: (L, R): statistics over the L leading (contiguous) elements of each of
 * the R columns.  gamma, beta, dgamma, dbeta: length L (elementwise affine over the
 * normalised dims) or NULL; save_mean, save_invstd: length R, fp32.
 * The reference has no device hook for layernorm (src/impl/layernorm.jl:3-14 is generic
 * broadcasts); the host adds an Impl.layernorm method + rrule that call these. */
int luxhip_layernorm_fwd(luxhip_stream_t s, int dtype, int act, int64_t L, int64_t R, const void* x,
                         const void* gamma, const void* beta, double eps, void* y, float* save_mean,
                         float* save_invstd);
int luxhip_layernorm_bwd(luxhip_stream_t s, int dtype, int act, int64_t L, int64_t R, const void* delta,
                         const void* x, const void* gamma, const void* beta, const float* save_mean,
                         const float* save_invstd, void* dx, void* dgamma, void* dbeta);

/* ---------------------------------------------------------------- dense --------------*/

/* C (M x N) = op(A) * op(B) (+ bias broadcast down the columns).  Stands behind
 * Impl.matmul!(C, ::GPUBroadcastOp, A, B) and Impl.matmuladd!(C, ::GPUBroadcastOp, A, B, bias)
 * (src/impl/matmul.jl:85-94,120-125) including Adjoint/Transpose operands (transX != 0:
 * the stored matrix is the transpose of the operand, as unwrapped by prepare_transposed,
 * ext/CUDAExt/cublaslt.jl:15-33). */
int luxhip_matmul(luxhip_stream_t s, int dtype, int transA, int transB, int64_t M, int64_t N, int64_t K,
                  const void* A, int64_t lda, const void* B, int64_t ldb, const void* bias, void* C,
                  int64_t ldc);

/* Impl.batched_matmul!(z, opmode, x, y) (src/impl/batched_mul.jl:204-212; NNlib.batched_mul! on
 * 3-d arrays): C_b (M x N) = op(A_b) op(B_b) for b < batch, matrix b of an operand starting
 * b * stride elements after the first; a stride of 0 shares one matrix among all products
 * (batch dims of extent 1, :171-174, 255-268).  transA / transB as in luxhip_matmul: the pullback
 * multiplies by the batched adjoints (batched_mul.jl rrule: dx = dz y', dy = x' dz). */
int luxhip_batched_matmul(luxhip_stream_t s, int dtype, int transA, int transB, int64_t M, int64_t N, int64_t K,
                          int64_t batch, const void* A, int64_t lda, int64_t strideA, const void* B, int64_t ldb,
                          int64_t strideB, void* C, int64_t ldc, int64_t strideC);

/* The same over up to three nested batch dims (batch_dims[0] innermost) with one stride per dim and
 * operand: the products of permuted / repeated operands without copies, e.g. the (heads, batch)
 * dims of scaled_dot_product_attention's [E, H, L, B] tensors and the key/value groups that
 * repeat_inner_gqa (src/impl/attention.jl:1-3, 44-48) would materialise (stride 0 along the repeat).
 * The caller lays out C so that the products do not overlap.
 * structure: what a causal mask (keep key s for query l where s <= l, make_causal_mask,
 * src/impl/attention.jl:130-134) lets the products of attention skip; 0 for a plain product.
 *   1: the elements of C with m > n are not needed (logits[s, l], and their cotangent): tiles
 *      that hold only such elements are left untouched;
 *   2: op(B)[k, n] is zero for k > n (weights and their cotangent as the right operand, contracted
 *      over s): the contraction of a tile stops at its last column;
 *   3: op(B)[k, n] is zero for k < n (the same matrices transposed, contracted over l): it starts
 *      at the tile's first column.
 * dtype LUXHIP_BF16_WIDE: A and B bf16, C fp32 (the accumulators unrounded; ldc and stridesC in
 * elements as before). */
int luxhip_batched_matmul_strided(luxhip_stream_t s, int dtype, int transA, int transB, int64_t M, int64_t N,
                                  int64_t K, const int64_t* batch_dims, const void* A, int64_t lda,
                                  const int64_t* stridesA, const void* B, int64_t ldb, const int64_t* stridesB,
                                  void* C, int64_t ldc, const int64_t* stridesC, int structure);

/* `sum(tmp; dims=3)` of the batched_matmul pullback when an operand was shared among the
 * products (src/impl/batched_mul.jl:324-330): out[i] = sum_b in[i + b n], i < n, in batch order. */
int luxhip_batch_sum(luxhip_stream_t s, int dtype, int64_t n, int64_t batch, const void* in, void* out);

/* y (M x N) = act.(W (M x K) * x (K x N) .+ bias).  Stands behind
 * Impl.fused_dense!(y, ::GPUBroadcastOp, act, W, x, b) (src/impl/dense.jl:46-69; precedent
 * cublasLt_fused_dense!, ext/CUDAExt/cublaslt.jl:351-403).  If pre != NULL (M x N, ld =
 * ldy) it receives the pre-activation W*x .+ bias (the cuBLASLt AUX output used by the gelu
 * rrule, src/impl/dense.jl:116-134). */
int luxhip_fused_dense_fwd(luxhip_stream_t s, int dtype, int act, int64_t M, int64_t K, int64_t N,
                           const void* W, int64_t ldw, const void* x, int64_t ldx, const void* bias,
                           void* y, int64_t ldy, void* pre);

/* Pullback of fused_dense (src/impl/dense.jl:71-113, ∇matmul_bias :290-291):
 * dz = delta .* act'(y, pre); dbias = sum over the batch of dz; dW = dz * x'; dx = W' * dz.
 * delta, y, pre, dz: M x N contiguous; dW: M x K; dx: K x N contiguous.  dz is caller-
 * provided scratch of M*N elements (may alias delta when delta may be overwritten; may be
 * NULL for IDENTITY).  dbias, dW, dx may each be NULL to skip that output. */
int luxhip_fused_dense_bwd(luxhip_stream_t s, int dtype, int act, int64_t M, int64_t K, int64_t N,
                           const void* delta, const void* y, const void* pre, const void* W, int64_t ldw,
                           const void* x, int64_t ldx, void* dz, void* dW, void* dx, void* dbias);

/* ---------------------------------------------------------------- conv ---------------
 * The fields of NNlib.DenseConvDims the path consumes (2 spatial dims, WHCN tensors):
 * x (W, H, Cin, N); w (kW, kH, Cin/groups, Cout); y (OW, OH, Cout, N).
 * flipkernel == 0 is true convolution (the DenseConvDims default used by Lux.Conv,
 * src/layers/conv.jl:97-98 of the reference); != 0 is cross-correlation. */
typedef struct luxhip_conv_dims {
    int64_t W, H, Cin, N;
    int64_t kW, kH, Cout;
    int64_t stride_w, stride_h;
    int64_t pad_w_lo, pad_w_hi, pad_h_lo, pad_h_hi;
    int64_t dil_w, dil_h;
    int64_t groups;
    int64_t flipkernel;
} luxhip_conv_dims_t;

/* y = act.(conv(x, w) .+ bias[cout]).  Stands behind Impl.conv!(y, ::Type{Dev}, x, w, cdims)
 * (bias == NULL, act identity) and Impl.conv_bias_act(::Type{Dev}, x, w, cdims, bias, act)
 * (src/impl/conv.jl:29-60,138-166).  pre (optional) receives conv .+ bias.  xt_keep (optional, as
 * large as x): receives the channel-contiguous copy of x that the kernels read; an rrule keeps it
 * next to x and hands it to luxhip_fused_conv_bwd, which then does not make it again. */
int luxhip_conv_fwd(luxhip_stream_t s, int dtype, int act, const luxhip_conv_dims_t* d, const void* x,
                    const void* w, const void* bias, void* y, void* pre, void* xt_keep);
/* dx = ∇conv_data(dy, w, cdims) (src/impl/conv.jl:128-131). */
int luxhip_conv_bwd_data(luxhip_stream_t s, int dtype, const luxhip_conv_dims_t* d, const void* dy,
                         const void* w, void* dx);
/* dw = ∇conv_filter(x, dy, cdims) (src/impl/conv.jl:133-136). */
int luxhip_conv_bwd_filter(luxhip_stream_t s, int dtype, const luxhip_conv_dims_t* d, const void* x,
                           const void* dy, void* dw);
/* ∇fused_conv (src/impl/conv.jl:261-275): dz = delta .* act'(y, pre); dbias = sum_{w,h,n} dz;
 * dw = ∇conv_filter(x, dz); dx = ∇conv_data(dz, w).  dz: caller scratch like
 * luxhip_fused_dense_bwd.  xt_kept (optional): what luxhip_conv_fwd wrote to xt_keep for the same x. */
int luxhip_fused_conv_bwd(luxhip_stream_t s, int dtype, int act, const luxhip_conv_dims_t* d,
                          const void* delta, const void* y, const void* pre, const void* x, const void* w,
                          void* dz, void* dw, void* dx, void* dbias, const void* xt_kept);

/* out = permutedims(in, (p1, p2, p3, 4:N...)) for in of size (d1, d2, d3, outer) (p: a permutation of
 * 1:3).  scaled_dot_product_attention accepts the embedding (`head_dim`) and token dims in any of
 * the first three positions (src/impl/attention.jl:5-16,66-103); operands whose embedding dim is not
 * the first are brought to (E, H, L, B...) with this, and their gradients taken back. */
int luxhip_permute_leading3(luxhip_stream_t s, int dtype, int64_t d1, int64_t d2, int64_t d3, int64_t outer, int p1, int p2,
                            int p3, const void* in, void* out);

/* Convolutions with three spatial dims (x (W, H, D, C, N), w (kW, kH, kD, C/groups, Cout)): the
 * reference hands them to the same NNlib.conv / ∇conv_data / ∇conv_filter calls as the
 * two-dimensional ones (src/impl/conv.jl:29-60,128-136).  Here they run as the two-dimensional
 * problem on the depth-unfolded input: xu (W, H, kD*C, Dout*N), channel kd + kD*c of sample
 * od + Dout*n = depth slice od*stride_d + tap*dil_d - pad_d_lo of x (zeros outside), tap = kD-1-kd
 * for true convolution and kd with flipkernel; the weight read as (kW, kH, kD*C/groups, Cout) needs
 * no copy.  plane = W*H. */
int luxhip_conv_depth_unfold(luxhip_stream_t s, int dtype, int64_t plane, int64_t D, int64_t C, int64_t N, int64_t KD,
                             int64_t Dout, int64_t stride_d, int64_t pad_d_lo, int64_t dil_d, int flipkernel, const void* x,
                             void* xu);
/* The adjoint of luxhip_conv_depth_unfold (for NNlib.∇conv_data with three spatial dims, call site
 * src/impl/conv.jl:128-131): dx (plane, D, C, N) gathers, in a fixed order, the terms
 * of dxu (plane, kD*C, Dout, N) that the unfolding copied from it (∇conv_data of a three-dimensional
 * problem = this applied to the two-dimensional ∇conv_data). */
int luxhip_conv_depth_fold(luxhip_stream_t s, int dtype, int64_t plane, int64_t D, int64_t C, int64_t N, int64_t KD,
                           int64_t Dout, int64_t stride_d, int64_t pad_d_lo, int64_t dil_d, int flipkernel, const void* dxu,
                           void* dx);
/* No counterpart in the reference (NNlib writes (W, H, D, C, N) outputs directly).
 * out (inner, B, A, outer) = permutedims(in (inner, A, B, outer), (1, 3, 2, 4)): between the output
 * of the two-dimensional problem, (OW*OH, Cout, Dout, N), and the caller's (OW*OH, Dout, Cout, N). */
int luxhip_swap_middle_dims(luxhip_stream_t s, int dtype, int64_t inner, int64_t A, int64_t B, int64_t outer, const void* in,
                            void* out);

#ifdef __cplusplus
}
#endif
#endif /* LUXHIP_H */
