/*
 * af3_dpa.h -- C ABI of the MI355X (gfx950) biased dot-product-attention library.
 *
 * One shared library, libaf3_dpa.so, built from af3_kernels_amd/csrc/ by hipcc.  Every entry
 * point takes raw device pointers, sizes, element strides and a HIP stream; none of them
 * allocates, frees, synchronises or terminates the process.  All work is enqueued on the
 * stream that is passed in (NULL = the default stream).  Return value: AF3_OK (0) or a negative
 * af3_status; af3_status_string() turns it into text.
 *
 * The reference interface each entry point replaces is named beside it (paths are relative to
 * the reference repository).
 */
#ifndef AF3_DPA_H
#define AF3_DPA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum af3_status {
	AF3_OK                 = 0,
	AF3_ERR_NULL_POINTER   = -1, /* a required pointer is NULL */
	AF3_ERR_BAD_DTYPE      = -2, /* dtype combination not implemented */
	AF3_ERR_BAD_SHAPE      = -3, /* a dimension is <= 0 or exceeds the supported maximum */
	AF3_ERR_BAD_STRIDE     = -4, /* negative stride, or innermost stride != 1 */
	AF3_ERR_UNSUPPORTED_D  = -5, /* head_dim above the supported maximum */
	AF3_ERR_LAUNCH         = -6, /* hipGetLastError() reported a launch failure */
	AF3_ERR_BAD_ARGUMENT   = -7, /* any other invalid argument (e.g. N % BLK_SZ != 0) */
	AF3_ERR_NO_DEVICE_CODE = -8, /* the current device is not a gfx950 (host-side check before the launch, or the
	                                 runtime reporting that it has no code object for the device) */
	AF3_ERR_SCRATCH_LIMIT  = -9  /* af3_dpa_forward_static_scratch: the call needs more scratch than the library's
	                                 built-in AF3_STATIC_SCRATCH_BYTES */
} af3_status;

typedef enum af3_dtype {
	AF3_F32      = 0,
	AF3_BF16     = 1,
	AF3_FP8_E4M3 = 2, /* OCP e4m3fn: bias 7, max 448, no infinity */
	AF3_FP8_E5M2 = 3  /* OCP e5m2: bias 15, max 57344, infinities and NaN (af3_convert only) */
} af3_dtype;

#define AF3_DPA_MAX_HEAD_DIM 128

/*
 * Arguments of one attention call: out = softmax(q . k^T * softmax_scale + bias, key_mask) . v
 *
 *   q, k, v, out : [B, H, L, D], element strides given for the B, H and L axes, innermost
 *                  (D) stride is 1.  q_len == k_len == L, as the reference assumes
 *                  (src/csrc/dot_product_attention.cpp:50-52).
 *   bias         : [H, L, L] shared by every batch row, element strides for H and the query
 *                  axis, key axis stride 1.  A bias that is already padded to [H, M, M] is
 *                  passed with its padded strides (examples/self_attention.py:134-149).
 *                  NULL means no bias.
 *   key_mask     : bytes, non-zero = attend (the caller's mask BEFORE the reference wrapper
 *                  inverts it).  Laid out [B, L] with batch stride key_mask_stride_b; a stride
 *                  of 0 broadcasts one [L] mask over the batch.  NULL means attend to all.
 *                  A batch row whose keys are all dropped yields the mean of its V rows, as
 *                  masked_fill(-1e9) + softmax does in examples/dot_product_attention.py:37-39.
 *
 *   io_dtype     : element type of q, k, v.  AF3_F32, AF3_BF16, or AF3_FP8_E4M3 (then q, k
 *                  are e4m3 bytes [B,H,L,D] and v is e4m3 bytes laid out TRANSPOSED as
 *                  [B, H, D, L] -- v_stride then holds strides for B, H and D, innermost (L) 1 --
 *                  as written by af3_quantize_fp8_e4m3 with transpose_last2 = 1).  K rows are
 *                  fetched in 16-byte chunks through a range-checked buffer that ends at the last
 *                  valid byte of each (batch, head) slab: nothing behind it is read, so the
 *                  allocation needs no slack.
 *   bias_dtype   : AF3_F32 or AF3_BF16.          out_dtype : AF3_F32 or AF3_BF16.
 *   mma_dtype    : arithmetic of the two products: AF3_F32 (fp32 FMA), AF3_BF16 (bf16 MFMA,
 *                  fp32 accumulate) or AF3_FP8_E4M3 (e4m3 MFMA, fp32 accumulate).
 *   softmax_scale: D^-1/2 for the reference semantics.  For fp8 inputs the caller may fold it
 *                  into q before quantisation and pass 1.
 *   q_descale, k_descale, v_descale : real value = stored value * descale (fp8 only; must be
 *                  powers of two so that the bias can ride the matrix pipeline exactly).
 */
typedef struct af3_dpa_params {
	const void*    q;
	const void*    k;
	const void*    v;
	const void*    bias;
	const uint8_t* key_mask;
	void*          out;
	int64_t        B, H, L, D;
	int64_t        q_stride[3];
	int64_t        k_stride[3];
	int64_t        v_stride[3];
	int64_t        out_stride[3];
	int64_t        bias_stride[2];
	int64_t        key_mask_stride_b;
	int32_t        io_dtype;
	int32_t        bias_dtype;
	int32_t        out_dtype;
	int32_t        mma_dtype;
	float          softmax_scale;
	float          q_descale;
	float          k_descale;
	float          v_descale;
	int32_t        force_generic; /* non-zero: always take the fp32-FMA kernel (testing aid) */
	int32_t        reserved;      /* kernel hint for batched bf16 calls that the shared-bias kernel (two to four batch rows per
	                                 wavefront) can take (head_dim <= 32, B >= 2, L <= 4096): 0 = chosen by launch size, 1 = always,
	                                 2 = never (testing aids) */
	/* Optional: 3 device floats {q_descale, k_descale, v_descale} as written by
	 * af3_quantize_fp8_e4m3; when non-NULL they override the three host values above, so a
	 * quantise -> attend sequence needs no device-to-host copy. */
	const float*   device_descales;
	/* Optional scratch in device memory, at least af3_dpa_workspace_bytes() long and 256-byte
	 * aligned.  With it a bf16 call of two or more batch rows may first rewrite the bias once
	 * (scaled by log2 e and laid out in matrix-operand order, shared by all B batch rows) and
	 * then run its fastest variant; without it (NULL) the bias is read in place.  Contents are
	 * overwritten by every call.  What the rewritten bias holds depends on the kernel the call
	 * takes (af3_dpa_workspace_bytes() returns the size for that kernel):
	 *  - the shared-bias kernel (head_dim <= 32, batch rows that share the bias; the headline
	 *    path): fp32(bias * log2 e) in accumulator order, 4 bytes per logit, exact for bf16 and
	 *    fp32 biases alike; entries below -2^17 (log2 units), -inf and NaN become -2^17.
	 *  - the one-row kernel (head_dim 48/64, small launches): fp16(bias * log2 e), 2 bytes per
	 *    logit: each logit carries a rounding error of at most 2^-11 * |bias| * 1.4427 (0.4 % of
	 *    a softmax weight at |bias| = 8, 2 % at |bias| = 40; values beyond +-45400 saturate).
	 *    Callers whose biases are that large and who need them exact pass workspace = NULL.
	 * In place, a bf16 bias is added exactly; the shared-bias kernel clamps entries below -2^16
	 * (and -inf) to -2^16 first, the one-row kernel those below -2^126.  A clamped entry has
	 * weight exactly 0 beside any ordinary logit; a query row made of nothing but clamped entries
	 * comes out as the softmax of q.k alone over its live keys.  (Add-then-softmax in the
	 * reference differs only where a row mixes entries on both sides of the clamp that are all
	 * hugely negative, e.g. -1e9 beside -70000: there the reference lets the larger one win.) */
	void*          workspace;
	int64_t        workspace_bytes;
	/* Optional (fp8 only): residual tensors q_lo = e4m3(q*s - q8), k_lo = e4m3(k*s - k8) at the same
	 * scale and with the same strides as q and k (af3_quantize_fp8_e4m3 writes them).  When both
	 * are given the logits are q8.k8 + q8.k_lo + q_lo.k8: three e4m3 MFMAs per contraction chunk
	 * that recover about six mantissa bits for q and k.
	 * Accuracy of the e4m3 path against the formula on the un-quantised inputs (unit-variance q, k, v): with the
	 * residuals 6e-2 max-abs from about 1024 keys per row on (measured 4e-2 .. 6e-2 at L = 1536); without them
	 * about 0.10; on short rows (L <= 64) the e4m3 rounding of the softmax weights and of v alone reaches 0.15,
	 * whatever the logits' precision, because few keys average it out.  The reference has no e4m3 arithmetic to
	 * compare with (its converters are "not implemented" asserts, src/csrc/xsmm_functors.h:218-226). */
	const void*    q_lo;
	const void*    k_lo;
	/* Optional output gate (ABI version 2): out = sigmoid(gate) * (softmax(...) . v), the
	 * "weighted_avg *= sigmoid(gating_query(pair))" step of the reference's fused grid attention
	 * (src/csrc/dot_product_attention.cpp:335-349), applied in the kernel's epilogue so the
	 * un-gated result never goes to memory.  gate: [B, H, L, D] pre-activation values of io_dtype
	 * with element strides for B, H and L (innermost 1), 8-byte aligned rows.  NULL: no gate.
	 * Not available for fp8 inputs. */
	const void*    gate;
	int64_t        gate_stride[3];
} af3_dpa_params;

/*
 * The attention forward pass.
 * Replaces: at::Tensor dot_product_attention(q, k, v, mask, bias, use_flash_attention, BLK_SZ,
 * FLASH_SZ) -- src/csrc/dot_product_attention.h:25-32, implemented at
 * src/csrc/dot_product_attention.cpp:25-198 and :545-559, bound at src/csrc/init.cpp:349-351.
 * Differences: inputs are const (the reference scales q in place and returns it); the mask is
 * the un-inverted byte mask instead of a T-typed tensor of 0/1 later multiplied by -1e9; the
 * CPU blocking hints use_flash_attention / BLK_SZ / FLASH_SZ have no counterpart (the kernel is
 * always an online-softmax kernel and its tiling is fixed by the hardware).
 */
int af3_dpa_forward(const af3_dpa_params* params, void* hip_stream);

/* Bytes of workspace the call would use (0 when a workspace would not help, e.g. B == 1,
 * no bias, a bf16 bias with 16-byte aligned rows under too few batch rows for a rewrite to pay
 * off -- fewer than about 224 + 2.4e8 / (H L^2); it is then read in place, exactly -- or a kernel
 * that does not take one); negative = af3_status error.  Host only. */
int64_t af3_dpa_workspace_bytes(const af3_dpa_params* params);

/*
 * af3_dpa_forward for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments and results as
 * af3_dpa_forward called with a workspace of af3_dpa_workspace_bytes() bytes, except that params->workspace and
 * params->workspace_bytes are ignored: the scratch (the rewritten bias of the bf16 kernel) lives in a device array of
 * AF3_STATIC_SCRATCH_BYTES that is part of the library's code object, one copy per GPU for the life of the process.
 * The call allocates and frees nothing.  A call that needs more scratch than that returns AF3_ERR_SCRATCH_LIMIT and
 * enqueues nothing (H * ceil(L/32)^2 * 4 KiB must fit: e.g. 4 heads up to L = 1024, 16 heads up to L = 512); a call
 * that needs none (one batch row, no bias, float32 or fp8 arithmetic) is af3_dpa_forward.  The first call on a device
 * looks up the array's address and the device's properties and sets kernel attributes (host-side work that loads the
 * code object): make one call, of any size, on each device OUTSIDE stream capture before the first captured one.  The
 * array costs every GPU the process runs this library on 16 MiB of device memory, used or not.  Every call on one GPU shares
 * that GPU's array and overwrites all of it that it reads, so nothing needs clearing between calls, but calls that
 * overlap in time on one GPU (two streams, two threads) race on it: serialise them, or give af3_dpa_forward separate
 * workspaces instead.
 */
#define AF3_STATIC_SCRATCH_BYTES (16 * 1024 * 1024)
int af3_dpa_forward_static_scratch(const af3_dpa_params* params, void* hip_stream);

/* Which kernel af3_dpa_forward would run for these arguments: 0 = fp32 vector-FMA kernel,
 * 1 = bf16 MFMA kernel, 2 = fp8 MFMA kernel, 3 = fp32 MFMA kernel; negative = af3_status error.
 * Host only. */
int af3_dpa_select_kernel(const af3_dpa_params* params);

/*
 * Element-wise dtype conversion, n contiguous elements, round-to-nearest-even.
 * Replaces: tpp::ConvertTPP (src/csrc/xsmm_functors.h:838-885) and the AVX-512 helpers
 * _mm512_convert_bf_ps / _mm256_convert_ps_bf (src/csrc/xsmm_functors.h:139-145).
 * Supported pairs: f32->bf16, bf16->f32, fp8_e4m3->f32, fp8_e4m3->bf16, and the e5m2 pair of the reference's
 * _mm512_convert_bf8_ps / _mm_convert_ps_bf8 (src/csrc/xsmm_functors.h:211-217): fp8_e5m2->f32, fp8_e5m2->bf16 (exact),
 * f32->fp8_e5m2 and bf16->fp8_e5m2, rounded to nearest even in one step with overflow to infinity (torch.float8_e5m2's
 * rule; the reference's helper rounds to fp16 first and then truncates the low byte, which differs in the last bit for
 * about three values in eight).
 */
int af3_convert(const void* src, int32_t src_dtype, void* dst, int32_t dst_dtype, int64_t n, void* hip_stream);

/*
 * Per-tensor absolute maximum of n contiguous f32 or bf16 elements, accumulated into
 * *amax_out (a device float the caller has set to 0, or to a running maximum).
 * No reference counterpart: the reference's e4m3 converters are "not implemented" asserts
 * (src/csrc/xsmm_functors.h:218-226); this is the first half of per-tensor fp8 scaling.
 */
int af3_amax(const void* src, int32_t src_dtype, int64_t n, float* amax_out, void* hip_stream);

/*
 * Second half of per-tensor fp8 scaling.  Reads *amax (device), derives
 *     scale = 2^floor(log2(448 / (amax * pre_scale)))        (1 when amax == 0)
 * writes dst = e4m3(src * pre_scale * scale), saturating at +-448, and stores the descale
 * 1/scale to *descale_out (device float).  src is viewed as [rows, cols] row-major with
 * row stride src_row_stride; with transpose_last2 != 0, every consecutive block of
 * `rows_per_matrix` rows is written transposed: dst[matrix][col][row], row stride
 * dst_row_stride (>= rows_per_matrix, a multiple of 4), so V [B*H*L, D] becomes [B*H, D, L];
 * the padding bytes [rows_per_matrix, dst_row_stride) of every output row are written as zero.
 * dst_residual (optional, same layout as dst): e4m3(src * pre_scale * scale - dst), the rounding
 * error of dst at the same scale, for the compensated product of af3_dpa_forward.
 * No reference counterpart (see af3_amax).
 */
int af3_quantize_fp8_e4m3(const void* src, int32_t src_dtype, void* dst, int64_t rows, int64_t cols, int64_t src_row_stride,
						  int32_t transpose_last2, int64_t rows_per_matrix, int64_t dst_row_stride, float pre_scale, const float* amax,
						  float* descale_out, void* dst_residual, void* hip_stream);

/*
 * The whole per-tensor fp8 preparation of one attention call in two launches: amax of q, k and v,
 * then q8 = e4m3(q * q_pre_scale * sq), k8 = e4m3(k * sk) (both [B,H,L,D], with their residuals
 * q_lo, k_lo when those pointers are non-NULL) and v8t = e4m3(v * sv) transposed to
 * [B,H,D,v8t_row_stride] (padding written as zero), scales as in af3_quantize_fp8_e4m3.
 * q, k, v: contiguous [B,H,L,D] of src_dtype (AF3_F32 or AF3_BF16), D % 4 == 0.
 * descales: 3 device floats, written {1/sq, 1/sk, 1/sv} (pass them as device_descales).
 * scratch: AF3_QKV_SCRATCH_FLOATS device floats, overwritten; it need not be cleared.
 * No reference counterpart (see af3_amax).
 */
#define AF3_QKV_SCRATCH_FLOATS 768
int af3_quantize_qkv_fp8_e4m3(const void* q, const void* k, const void* v, int32_t src_dtype, int64_t B, int64_t H, int64_t L, int64_t D,
							  float q_pre_scale, void* q8, void* k8, void* v8t, int64_t v8t_row_stride, void* q_lo, void* k_lo,
							  float* descales, float* scratch, void* hip_stream);

/*
 * Grid (triangle) self-attention up to the sigmoid gate, in ONE kernel:
 *     q, k, v, g = pair . Wq, Wk, Wv, Wgate   (per head, C/head channels each)
 *     out[b, n, h*K : (h+1)*K] = softmax(q k^T / sqrt(K) + bias[h], key mask)[n, :] . v  *  sigmoid(g[n])
 * q, k, v and the gate never touch device memory: K and V of a (batch row, head) are projected into LDS once,
 * q and the gate per block of 32 query rows.
 * Replaces: _attention_impl<bfloat16> without its closing output projection -- src/csrc/dot_product_attention.cpp:
 * 200-362 (projections :286-345, logits / bias / mask / softmax :313-333, weighted average :346-352, sigmoid gate
 * :334-361), bound as `_attention` at src/csrc/init.cpp.  The output projection (:364-371) is a plain [B*N, C] x
 * [C, C] matrix product on the result: af3_linear below, or the caller's BLAS.
 * Supported (af3_grid_attention_supported() == 1): dtype AF3_BF16, C == 128, head == 4, N small enough for K and V
 * of one head to stay in LDS (N <= 1024); anything else returns AF3_ERR_BAD_ARGUMENT and the caller composes the
 * op from a projection product and af3_dpa_forward with its `gate` argument.
 */
typedef struct af3_grid_attention_params {
	const void* pair;            /* [B, N, C] normalised pair rows, innermost stride 1 */
	int64_t     pair_stride[2];  /* elements: batch row, token */
	/* weight^T of the four projections in the layout the reference's callers produce with
	 * vnni_repack_tensor(W.T, 2, C/head): [head][C/2][C/head][2] (src/af3_kernels/Attention.py:59-62) */
	const void* q_proj;
	const void* k_proj;
	const void* v_proj;
	const void* gating_query;
	const void* bias;            /* [head, N, N] (or NULL), AF3_BF16 or AF3_F32 */
	int64_t     bias_stride[2];  /* elements: head, query row */
	int32_t     bias_dtype;
	int32_t     dtype;           /* of pair, the weights and out */
	const uint8_t* key_mask;     /* [B, N] or [N] bytes, non-zero = attend; NULL = all */
	int64_t     key_mask_stride_b; /* 0 broadcasts one mask row over the batch */
	void*       out;             /* [B, N, C], innermost stride 1 */
	int64_t     out_stride[2];
	int64_t     B, N, C, head;
	void*       workspace;       /* af3_grid_attention_workspace_bytes() bytes, 256-byte aligned; required when bias != NULL */
	int64_t     workspace_bytes;
} af3_grid_attention_params;

int     af3_grid_attention_forward(const af3_grid_attention_params* params, void* hip_stream);
int64_t af3_grid_attention_workspace_bytes(const af3_grid_attention_params* params);
/* 1 when af3_grid_attention_forward handles these arguments, 0 when the caller must compose the op. Host only. */
int     af3_grid_attention_supported(const af3_grid_attention_params* params);

/*
 * The step in front of grid self-attention in one pass over the pair tensor: LayerNorm over the C channels of every
 * token (biased variance, eps inside the square root) and the projection of the normalised, bf16-rounded row to one
 * bias value per head, written as bias[h][i][j] -- the layout the attention entry points read.
 * Replaces the torch ops of src/af3_kernels/Attention.py:51-52 (act_norm, pair_bias_projection, permute(2, 0, 1));
 * the reference has no native code for this step.
 * pair [n_i, n_j, C] with element strides pair_stride[2] (innermost stride 1, multiples of 8), ln_weight / ln_bias [C],
 * proj_weight [head, C] (nn.Linear weight, contiguous), normed [n_i, n_j, C] contiguous, bias_stride = {head, row i}.
 * Supported: dtype AF3_BF16 or AF3_F32 (all tensors of that type), C <= 2048, head <= 64 with (2 + head) * C * 4 bytes
 * fitting in LDS, pointers aligned to their element size.  bf16 with C == 128, head == 4, 16-byte aligned pointers and
 * pair strides that are multiples of 8 takes a specialised kernel (four tokens per wave-wide load); everything else one
 * wavefront per token.  AF3_ERR_BAD_ARGUMENT for shapes beyond these.
 */
int af3_layernorm_pair_bias(const void* pair, const int64_t* pair_stride, const void* ln_weight, const void* ln_bias, float eps, const void* proj_weight,
							void* normed, void* bias, const int64_t* bias_stride, int64_t n_i, int64_t n_j, int64_t C, int64_t head, int32_t dtype, void* hip_stream);

/*
 * Gated linear unit: out[m][n] = silu(x[m] . Wa[:, n]) * (x[m] . Wb[:, n]) in one kernel (the [M, 2N] product is never
 * stored).  x [M, K] contiguous, out [M, N] contiguous, weight_t = [Wa | Wb]^T, i.e. [2N, K] row-major (the
 * nn.Linear layout [out_features, in_features]: rows 0..N-1 gate, rows N..2N-1 value).
 * Replaces: at::Tensor gated_linear_unit(input, weight, vnni_repacked, M_BLK, N_BLK) -- src/csrc/gated_linear_unit.h,
 * implemented at src/csrc/gated_linear_unit.cpp:20-80, :131-138 (the reference takes the weight as [K, 2N], plain or
 * VNNI-repacked; its CPU blocking arguments have no counterpart).
 * Supported: dtype AF3_BF16, K == 64 or 128, N % 32 == 0, 16-byte aligned x and weight_t; AF3_ERR_BAD_ARGUMENT otherwise.
 */
int af3_gated_linear_unit(const void* x, const void* weight_t, void* out, int64_t M, int64_t K, int64_t N, int32_t dtype, void* hip_stream);

/*
 * The gate of a gated linear unit on an already computed product: out[m][n] = silu(y[m][n]) * y[m][N + n] for y [M, 2N]
 * and out [M, N], both contiguous, AF3_BF16 or AF3_F32 (bf16: silu's result is rounded to bf16 before the product, as in
 * src/csrc/gated_linear_unit.cpp:56-61).  For shapes af3_gated_linear_unit does not take: the caller computes y = x . W
 * with a library GEMM and applies this.
 */
int af3_silu_mul(const void* y, void* out, int64_t M, int64_t N, int32_t dtype, void* hip_stream);

/*
 * Bias-free linear layer for narrow contractions: out[M, N] = x[M, K] . weight^T with weight in nn.Linear layout
 * [N, K] -- the same kernel as af3_gated_linear_unit without the gate (rows of x through LDS once, weight fragments in
 * registers, 16-byte stores).
 * Replaces: at::Tensor linear(input, weight, M_BLK, N_BLK) -- src/csrc/gated_linear_unit.cpp:82-129, :140-147 (the reference
 * takes the weight^T VNNI-repacked) -- and the closing output projection of _attention_impl (dot_product_attention.cpp:364-371).
 * Supported: dtype AF3_BF16, K == 64 or 128, N % 32 == 0, 16-byte aligned pointers; AF3_ERR_BAD_ARGUMENT otherwise.
 */
int af3_linear(const void* x, const void* weight, void* out, int64_t M, int64_t K, int64_t N, int32_t dtype, void* hip_stream);

/*
 * N-dimensional pad (ndim <= AF3_PAD_MAX_DIMS): copy src (shape src_shape, element strides
 * src_strides) into the low corner of a contiguous dst of shape dst_shape (>= src_shape in
 * every axis) and fill the rest with the 32-bit pattern `fill_bits` truncated to elem_size
 * (1, 2 or 4 bytes).  The shape / stride arrays are host memory, read before the call returns.
 * Replaces: pad_and_align_tensor / fast_memcpy -- src/csrc/tools.cpp:16-124.  The attention
 * kernels never need it (tails are predicated in the kernel); it exists for callers that used
 * the reference's helper directly.
 */
#define AF3_PAD_MAX_DIMS 6
int af3_pad_nd(const void* src, void* dst, int32_t ndim, const int64_t* src_shape, const int64_t* src_strides, const int64_t* dst_shape,
			   int32_t elem_size, uint32_t fill_bits, void* hip_stream);

/*
 * bf16 [M, N] -> per blk-wide column panel [N/blk][M/2][blk][2] (row pairs interleaved).
 * Replaces: vnni_repack_tensor with type = XFORM_N2V -- src/csrc/tools.cpp:151-176,
 * tpp::XformExtTPP::ref src/csrc/xsmm_functors.h:2100-2111.  The attention kernels do not
 * consume this layout (their matrix operands are packed in the load path); it is kept for
 * callers of the reference helper.  blk == 0 means blk = N.  M must be even, N % blk == 0.
 */
int af3_vnni_repack_bf16(const void* src, void* dst, int64_t M, int64_t N, int64_t blk, void* hip_stream);

const char* af3_status_string(int status);
/* ABI version of this header: bumped whenever a struct layout or signature changes. */
int af3_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* AF3_DPA_H */
