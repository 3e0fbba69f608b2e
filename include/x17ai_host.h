/*
 * x17ai_host.h -- flat C ABI of the host-side operator layer (libx17ai_host.so).
 *
 * The reference's operator layer is Rust (src/device/cuda/{gemm,attn,tensor_check,
 * kernel_build}.rs, src/tensor.rs, src/device/cuda.rs); its C++ mirror lives in
 * x17ai_amd/csrc/host/.  This header exposes that mirror to non-C++ callers (the Python
 * tests and bench drive it through ctypes).  Every function here ends in the C-ABI device
 * shim of include/x17ai_hip_shim.h; nothing in it computes on the CPU.
 *
 * Conventions: functions return 0 on success and non-zero on failure; after a failure
 * x17h_last_error() returns the message (thread-local, valid until the next call).
 * Handles are opaque and must be released with the matching *_free.
 */
#ifndef X17AI_HOST_H
#define X17AI_HOST_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct X17hDevice X17hDevice;       /* mirrors CudaDevice, src/device/cuda.rs:25-66 */
typedef struct X17hTensor X17hTensor;       /* mirrors Tensor, src/tensor.rs:23-256 */
typedef struct X17hTimer X17hTimer;         /* mirrors CudaTimer, src/device/cuda.rs:79-101 */
typedef struct X17hGemmKernel X17hGemmKernel;       /* mirrors GemmKernel<E>, src/device/cuda/gemm.rs:350-449 */
typedef struct X17hAttnKernel X17hAttnKernel;       /* mirrors AttnKernel, src/device/cuda/attn.rs:156-240 */
typedef struct X17hRmsNormKernel X17hRmsNormKernel; /* rms_norm.cu:55-113 as a kernel object */
typedef struct X17hDecodeKernel X17hDecodeKernel;   /* single-token decode; no reference counterpart */

/* DType, src/dtype.rs:1-15 */
enum { X17H_E4M3 = 0, X17H_INT8 = 1, X17H_BF16 = 2, X17H_F32 = 3 };
/* epilogues, src/device/cuda/gemm.rs:322-349 */
enum { X17H_EPI_SCALE = 0, X17H_EPI_GEGLU = 1, X17H_EPI_RESIDUAL = 2, X17H_EPI_RMSNORM = 3,
       /* no counterpart in gemm.rs: run-time per-row x per-column f32 scales, bf16 output */
       X17H_EPI_DEQUANT = 4,
       /* the older Q writer with a learned bf16 scale per column, cuda/qkvg_fwd_i8.cuh:145-219 (launch: extra =
        * q_norm_scales bf16 [b_rows]; head_dim, eps and out_scale as for RMSNorm, no V halves; inp_scale = the factor
        * applied after the learned scales, 1.0 or 0 for none -- the old writer's base class, which is gone from the
        * reference tree, was built with 1 / sqrt(MODEL_DIM), cuda/qkvg_fwd_i8.cuh:151-159) */
       X17H_EPI_QNORM = 5,
       /* no counterpart in gemm.rs: the q (Scale) and kv (RMSNorm) projections as one launch, x17h_gemm_kernel_launch_qkv */
       X17H_EPI_QKV = 6 };
enum { X17H_ACT_NONE = 0, X17H_ACT_GEGLU = 1 };

char const *x17h_last_error(void);
/* text of the warnings/errors collected by the last *_new call (kernel generation diagnostics) */
char const *x17h_last_diagnostics(void);
/* For callers of the raw shim that cannot implement the FfiBuffer callbacks themselves: hands `diag`
 * (a non-NULL X17DiagnosticBuffer* returned by an x17ai_hip_* function) to x17ai_move_diagnostic
 * through the operator layer's own growable buffer (the twin of src/util/ffi_buffer.rs:13-103) and
 * APPENDS the text to the NUL-terminated string in out[capacity].  Returns the new string length. */
size_t x17h_move_diagnostic_text(void *diag, char *out, size_t capacity);

/* CudaDevice::new, src/device/cuda.rs:31-38 */
int x17h_device_new(size_t device_id, X17hDevice **out);
void x17h_device_free(X17hDevice *dev);
int x17h_device_synchronize(X17hDevice *dev);
char const *x17h_device_name(X17hDevice *dev);

/* Tensor::new_empty + Device::upload_data / download_data, src/tensor.rs:36-112.
 * dev == NULL places the tensor on the CPU device (host memory), as Tensor::to_cpu does. */
int x17h_tensor_new_empty(X17hDevice *dev, size_t const *shape, size_t ndim, int dtype, X17hTensor **out);
void x17h_tensor_free(X17hTensor *t);
int x17h_tensor_upload(X17hTensor *t, void const *src, size_t bytes);      /* async on the device stream */
int x17h_tensor_download(X17hTensor *t, void *dst, size_t bytes);          /* async; synchronize before reading */
/* Tensor::from_safetensors_file, src/tensor.rs:155-179: exactly one tensor, dtype F8_E4M3 / I8 / BF16 / F32,
 * bytes uploaded unchanged.  dev == NULL loads onto the CPU.  shape must have room for 8 dimensions. */
int x17h_tensor_from_safetensors_file(X17hDevice *dev, char const *path, X17hTensor **out, int *dtype, size_t *shape, size_t *ndim);
/* Tensor::save_safetensors_file, src/tensor.rs:213-249: CPU tensors only, single entry "tensor" */
int x17h_tensor_save_safetensors_file(X17hTensor *t, char const *path);
void *x17h_tensor_device_ptr(X17hTensor *t);
size_t x17h_tensor_bytes(X17hTensor *t);
int x17h_tensor_reshape(X17hTensor *t, size_t const *shape, size_t ndim);  /* Tensor::reshape, in place */

/* CudaTimer, src/device/cuda.rs:79-101 (events on the device's stream) */
int x17h_timer_new(X17hDevice *dev, X17hTimer **out);
void x17h_timer_free(X17hTimer *t);
int x17h_timer_start(X17hTimer *t);
int x17h_timer_stop(X17hTimer *t);
int x17h_timer_elapsed_seconds(X17hTimer *t, double *seconds);

/* GemmConfig + epilogue configs, src/device/cuda/gemm.rs:28-76 */
typedef struct X17hGemmConfig {
	int a_dtype; size_t a_cols; size_t a_rows; /* 0 = runtime */ int a_trans;
	int b_dtype; size_t b_cols; size_t b_rows; /* 0 = runtime */ int b_trans;
	int c_dtype;
	int epilogue;            /* X17H_EPI_* */
	double inp_scale;
	double out_scale;
	double eps;              /* RMSNorm only */
	size_t head_dim;         /* RMSNorm only */
	size_t sep_dim;          /* RMSNorm only */
	int strict_math;         /* 1: deterministic transcendentals (parity build), 0: hardware ones */
	int activation;          /* Dequant only: X17H_ACT_* */
	/* X17H_EPI_QKV only: raw columns [0, q_cols) are the q projection (Scale writer with q_inp_scale * q_out_scale),
	 * the other b_rows - q_cols the kv projection (RMSNorm writer with inp_scale, out_scale, eps, head_dim, sep_dim) */
	size_t q_cols;
	double q_inp_scale;
	double q_out_scale;
} X17hGemmConfig;

/* GemmKernel::<E>::new, gemm.rs:368-437.  dev == NULL: generate and compile only. */
int x17h_gemm_kernel_new(X17hDevice *dev, char const *kernel_name, X17hGemmConfig const *config, X17hGemmKernel **out);
void x17h_gemm_kernel_free(X17hGemmKernel *k);
/* GemmKernel::launch, gemm.rs:439-443; extra = rrms (RMSNorm) / residual (Residual) / NULL */
int x17h_gemm_kernel_launch(X17hGemmKernel *k, X17hTensor *a, X17hTensor *b, X17hTensor *c, X17hTensor *extra);
/* Dequant epilogue: c[m, n] = bf16((acc * row_scale[m]) * col_scale[n]), or GeGLU over column pairs of that;
 * row_scale f32 [M], col_scale f32 [N_raw].  No counterpart in the reference (its scales are constants). */
int x17h_gemm_kernel_launch_dequant(X17hGemmKernel *k, X17hTensor *a, X17hTensor *b, X17hTensor *c,
                                    X17hTensor *row_scale, X17hTensor *col_scale);
/* X17H_EPI_QKV: the q projection (src/main.rs:387-438) and the kv projection (:440-493) as one launch that reads x
 * once.  x i8 [M, K]; q_weights i8 [q_cols, K]; kv_weights i8 [b_rows - q_cols, K]; q i8 [M, q_cols];
 * kv i8 [M, b_rows - q_cols]; rrms f32 [M, heads].  Outputs equal those of the two separate kernels bit for bit. */
int x17h_gemm_kernel_launch_qkv(X17hGemmKernel *k, X17hTensor *x, X17hTensor *q_weights, X17hTensor *kv_weights,
                                X17hTensor *q, X17hTensor *kv, X17hTensor *rrms);
/* GemmKernel::n_ops, gemm.rs:445-449 */
double x17h_gemm_kernel_n_ops(X17hGemmKernel *k, X17hTensor *a, X17hTensor *b);
/* launch geometry read back from meta.json: THREADS_PER_BLOCK, SMEM_BYTES, M_PER_BLOCK, N_PER_BLOCK */
int x17h_gemm_kernel_metadata(X17hGemmKernel *k, size_t out[4]);
/* resources of the loaded kernel: x17ai_hip_read_kernel_attrs (9 x int32) */
int x17h_gemm_kernel_attrs(X17hGemmKernel *k, int32_t out[9]);

/* AttnKernelConfig, attn.rs:45-152 */
typedef struct X17hAttnConfig {
	int dtype; size_t n_heads; size_t head_dim; size_t q_stride; size_t kv_stride; size_t o_stride;
	int strict_math;
	/* extension, no counterpart in the reference (its codes all share the scale 1/8): row_scales != 0 builds
	 * the kernel whose q/k/v codes carry one f32 scale per (row, head); out_dtype is then X17H_INT8
	 * (FixedI8 codes) or X17H_BF16 (real values), otherwise X17H_INT8 */
	int row_scales; int out_dtype;
	/* backward_q != 0 builds the backward-with-respect-to-q kernel of this configuration instead of the forward
	 * (launched with x17h_attn_kernel_launch_d_q).  The reference's attn_d_q.cuh:1-410 is its bf16 generation; the
	 * int8 generation has no backward there yet, so the operands are defined here: the forward's q, kv, sinks and
	 * temperatures, its FixedI8 output and log-sum-exp L, dO as bf16 -> dQ as bf16 (with respect to the real q) */
	int backward_q;
	/* backward_kv != 0 builds the backward-with-respect-to-k-and-v kernel instead (launched with
	 * x17h_attn_kernel_launch_d_kv; structure of attn_d_kv.cuh:1-431, likewise the reference's bf16 generation).  At most
	 * one of backward_q and backward_kv may be set. */
	int backward_kv;
} X17hAttnConfig;
/* AttnKernel::new, attn.rs:170-232 */
int x17h_attn_kernel_new(X17hDevice *dev, char const *kernel_name, X17hAttnConfig const *config, X17hAttnKernel **out);
void x17h_attn_kernel_free(X17hAttnKernel *k);
/* AttnKernel::launch, attn.rs:234-236 / 353-447.  l may be NULL.  batch > 1 is an extension:
 * the rows of q/kv/out are `batch` independent sequences of equal length. */
int x17h_attn_kernel_launch(X17hAttnKernel *k, X17hTensor *q, X17hTensor *kv, X17hTensor *sink_k,
                            X17hTensor *sink_v, X17hTensor *attn_temperature, X17hTensor *out,
                            X17hTensor *l, size_t window_size, size_t batch);
/* The same launch for a kernel built with row_scales (no counterpart in the reference; the closest
 * precedent is the per-head temperature vector of attn.rs:421-437).  q_scale, k_scale, v_weight: f32
 * [n_heads, rows] (head-major, like l); sink_v_weight, out_scale: f32 [n_heads].  Real q = code * q_scale, real k = code * k_scale,
 * real v = code * v_weight * v_ref[h]; sink_v_weight = (1/8) / v_ref, out_scale = v_ref (bf16 out) or 8 * v_ref. */
int x17h_attn_kernel_launch_row_scaled(X17hAttnKernel *k, X17hTensor *q, X17hTensor *kv, X17hTensor *sink_k,
                                       X17hTensor *sink_v, X17hTensor *attn_temperature, X17hTensor *out,
                                       X17hTensor *l, size_t window_size, size_t batch,
                                       X17hTensor *q_scale, X17hTensor *k_scale, X17hTensor *v_weight,
                                       X17hTensor *sink_v_weight, X17hTensor *out_scale);
/* Launch of a kernel built with backward_q (structure of attn_d_q.cuh:70-383: P from L, D = rowsum(dO * O) written to
 * `d` for a later dK/dV kernel, dS = P (dP - D), dQ = dS . K).  out: the forward's output i8 [rows, o_stride];
 * d_out: bf16 [rows, o_stride]; d_q: bf16 [rows, q_stride] (written); l: f32 [n_heads, rows]; d: f32 [n_heads, rows]
 * (written; may be NULL). */
int x17h_attn_kernel_launch_d_q(X17hAttnKernel *k, X17hTensor *q, X17hTensor *kv, X17hTensor *sink_k, X17hTensor *sink_v,
                                X17hTensor *attn_temperature, X17hTensor *out, X17hTensor *d_out, X17hTensor *d_q,
                                X17hTensor *l, X17hTensor *d, size_t window_size, size_t batch);
/* Launch of a kernel built with backward_kv (structure of attn_d_kv.cuh:200-400: a block of keys walks the queries that
 * see it; P from L, dV += P^T dO, dS = P (dP - D), dK += dS^T Q; like attn_d_kv.cuh it forms no gradient for the sink or
 * the temperatures).  d_out: bf16 [rows, o_stride]; l: f32 [n_heads, rows] of the forward; d: f32 [n_heads, rows] as
 * written by x17h_attn_kernel_launch_d_q; d_kv: bf16 [rows, kv_stride] (written), in the layout of kv: per head dK then
 * dV, gradients with respect to the real k and v. */
int x17h_attn_kernel_launch_d_kv(X17hAttnKernel *k, X17hTensor *q, X17hTensor *kv, X17hTensor *attn_temperature,
                                 X17hTensor *d_out, X17hTensor *l, X17hTensor *d, X17hTensor *d_kv,
                                 size_t window_size, size_t batch);
/* AttnKernelConfig::n_ops, attn.rs:72-84 */
double x17h_attn_kernel_n_ops(X17hAttnKernel *k, size_t seq_len, size_t window_size);
int x17h_attn_kernel_metadata(X17hAttnKernel *k, size_t out[3]);
int x17h_attn_kernel_attrs(X17hAttnKernel *k, int32_t out[9]);

/* rms_norm.cu:55-113: out[T, D] int8 = fixedi8(x * rsqrt(mean(x^2) + eps) * 8); in_dtype e4m3 or bf16 */
int x17h_rms_norm_kernel_new(X17hDevice *dev, char const *kernel_name, int in_dtype, size_t model_dim,
                             double eps, X17hRmsNormKernel **out);
void x17h_rms_norm_kernel_free(X17hRmsNormKernel *k);
int x17h_rms_norm_kernel_launch(X17hRmsNormKernel *k, X17hTensor *inp, X17hTensor *out);

/* Single-token decode against an int8 KV cache [S, capacity, 2*H*hd]: the attention recurrence
 * of attn_fwd_i8 for one query per sequence at position cache_len[s]. */
int x17h_decode_kernel_new(X17hDevice *dev, char const *kernel_name, size_t n_heads, size_t head_dim,
                           size_t cache_capacity, int strict_math, X17hDecodeKernel **out);
void x17h_decode_kernel_free(X17hDecodeKernel *k);
int x17h_decode_kernel_launch(X17hDecodeKernel *k, X17hTensor *q, X17hTensor *cache, X17hTensor *cache_len,
                              X17hTensor *sink_k, X17hTensor *sink_v, X17hTensor *attn_temperature,
                              X17hTensor *out, X17hTensor *l, size_t window_size);
/* The decode kernel over a row-scaled cache (as X17hAttnConfig.row_scales; no reference counterpart):
 * q_scale f32 [S, H]; k_scale, v_weight f32 [S, H, capacity]; sink_v_weight, out_scale f32 [H];
 * out_dtype X17H_INT8 or X17H_BF16.  Only the scales of visible rows are read. */
int x17h_decode_kernel_new_row_scaled(X17hDevice *dev, char const *kernel_name, size_t n_heads, size_t head_dim,
                                      size_t cache_capacity, int strict_math, int out_dtype, X17hDecodeKernel **out);
int x17h_decode_kernel_launch_row_scaled(X17hDecodeKernel *k, X17hTensor *q, X17hTensor *cache, X17hTensor *cache_len,
                                         X17hTensor *sink_k, X17hTensor *sink_v, X17hTensor *attn_temperature,
                                         X17hTensor *out, X17hTensor *l, size_t window_size,
                                         X17hTensor *q_scale, X17hTensor *k_scale, X17hTensor *v_weight,
                                         X17hTensor *sink_v_weight, X17hTensor *out_scale);

#ifdef __cplusplus
}
#endif
#endif /* X17AI_HOST_H */
