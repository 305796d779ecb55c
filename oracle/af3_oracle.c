/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the biased dot-product-attention path.
 *
 * This file is a plain-C restatement of the algorithm the reference runs on the CPU.  It is
 * the checker the GPU kernels are compared with; it is never linked into, imported by or
 * called from the shipped library.  Only the test-suite, the smoke check and the CPU-baseline
 * leg of the benchmark may load it.
 *
 * The reference's compiled path cannot be built here (its arithmetic lives in libxsmm, an
 * un-vendored submodule: /root/reference/.gitmodules:1-3, setup.py:39-43), so every primitive
 * below follows the readable ".ref()" twin the reference ships next to each JIT kernel and the
 * driver loop that strings them together.  Each function names the lines it follows.
 *
 * What pins this file (see tests/test_oracle_*.py): torch's scaled_dot_product_attention for
 * the bias-free case, an independent float64 numpy closed form, a pure-Python brute force on
 * tiny shapes, algebraic invariants (row-shift of the bias, key permutation, single live key,
 * uniform logits), flash == non-flash, torch's own bf16 / float8_e4m3fn casts for the
 * converters and a view/permute identity for the VNNI pack.  The callers around the core (af3o_fused_attention_*,
 * af3o_layernorm_pair_bias, af3o_gated_linear_unit) are pinned against torch library ops in float64 (linear,
 * scaled_dot_product_attention, sigmoid, layer_norm, silu), against independent numpy forms through the golden
 * vectors, and by special cases (zero gate weights, identity output projection, a q bias alone driving the logits,
 * constant rows under LayerNorm, a saturated GLU gate); their reference-arithmetic variants are checked against the
 * exact forms in fp32 (equal) and bf16 (within the bf16 budget).
 *
 * Parity unpinned: the bit pattern of the reference's bf16 pipeline (libxsmm's JIT exp
 * polynomial and BRGEMM summation order are not reproducible without libxsmm).  The oracle
 * uses expf and left-to-right fp32 sums; agreement with the reference binary is therefore
 * "to rounding", which is also all the reference's own harness measures
 * (examples/dot_product_attention.py:129-134 prints a relative L1, no threshold).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define AF3O_F32 0
#define AF3O_BF16 1

/* ---- scalar converters -------------------------------------------------------------- */

/* fp32 -> bf16 bits, round-to-nearest-even; xsmm_functors.h:142-145 (ROUNDNE then >>16). */
uint16_t af3o_f32_to_bf16_bits(float f) {
	uint32_t u;
	memcpy(&u, &f, 4);
	if((u & 0x7fffffffu) > 0x7f800000u) { /* NaN: keep quiet bit */
		return (uint16_t)((u >> 16) | 0x0040u);
	}
	u += 0x7fffu + ((u >> 16) & 1u);
	return (uint16_t)(u >> 16);
}

/* bf16 bits -> fp32; xsmm_functors.h:139-141 (shift left by 16). */
float af3o_bf16_bits_to_f32(uint16_t h) {
	uint32_t u = (uint32_t)h << 16;
	float    f;
	memcpy(&f, &u, 4);
	return f;
}

static inline float round_bf16(float f) {
	return af3o_bf16_bits_to_f32(af3o_f32_to_bf16_bits(f));
}

/* Storage rounding of the reference's template type T (float or at::BFloat16). */
static inline float round_T(float f, int dtype) {
	return dtype == AF3O_BF16 ? round_bf16(f) : f;
}

/*
 * fp32 -> OCP float8 e4m3fn bits (bias 7, max 448, no inf, NaN = S.1111.111), RNE, saturating.
 * The reference declares the type (xsmm_functors.h:35) but its converters are
 * "not implemented" asserts (xsmm_functors.h:218-226), so this follows the OCP 8-bit
 * floating point specification; it is pinned against torch.float8_e4m3fn for |x| <= 448.
 */
uint8_t af3o_f32_to_e4m3_bits(float f) {
	uint32_t u;
	memcpy(&u, &f, 4);
	uint8_t  sign = (uint8_t)((u >> 24) & 0x80u);
	uint32_t a    = u & 0x7fffffffu;
	if(a > 0x7f800000u) {
		return (uint8_t)(sign | 0x7fu);
	}
	float af;
	memcpy(&af, &a, 4);
	if(af >= 448.0f) {
		return (uint8_t)(sign | 0x7eu); /* saturate to 448 */
	}
	float q;
	if(af < 0.015625f) { /* below the smallest normal 2^-6: quantum 2^-9, RNE (a tie at 2^-10 goes to 0) */
		q = nearbyintf(af * 512.0f);
		return (uint8_t)(sign | (uint8_t)q); /* q == 8 is exactly the first normal's encoding 0x08 */
	}
	int   e;
	float m = frexpf(af, &e); /* af = m * 2^e, m in [0.5,1) */
	int   E = e - 1;          /* af = (2m) * 2^E, 2m in [1,2) */
	q = nearbyintf((2.0f * m - 1.0f) * 8.0f); /* 3 mantissa bits, RNE under default rounding mode */
	if(q >= 8.0f) {
		q = 0.0f;
		E += 1;
	}
	if(E > 8 || (E == 8 && q > 6.0f)) {
		return (uint8_t)(sign | 0x7eu);
	}
	return (uint8_t)(sign | (uint8_t)((E + 7) << 3) | (uint8_t)q);
}

float af3o_e4m3_bits_to_f32(uint8_t b) {
	int   s = b & 0x80;
	int   E = (b >> 3) & 0xf;
	int   m = b & 7;
	float v;
	if(E == 0xf && m == 7) {
		return NAN;
	}
	if(E == 0) {
		v = (float)m * 0.001953125f; /* m * 2^-9 */
	} else {
		v = ldexpf(1.0f + (float)m / 8.0f, E - 7);
	}
	return s ? -v : v;
}

/*
 * e5m2 ("bf8"): fp16's exponent range with two mantissa bits, infinities and NaN like IEEE.
 * af3o_e5m2_bits_to_f32: _mm512_convert_bf8_ps, xsmm_functors.h:211-213 -- the byte is the upper half of the fp16
 * pattern of the same value.
 * af3o_f32_to_e5m2_bits_reference: _mm_convert_ps_bf8, xsmm_functors.h:214-217 -- round to fp16 (nearest even), then
 * arithmetic shift right by 8, i.e. the low mantissa byte is dropped: two roundings, the second towards zero in magnitude
 * (the shift acts on the sign-magnitude pattern, so the sign bit is kept and the magnitude truncated).
 * af3o_f32_to_e5m2_bits: one rounding to nearest even from fp32, overflow to infinity -- the rule of the shipped
 * converter; pinned against torch.float8_e5m2.
 */
static uint16_t f32_to_f16_bits_rne(float f) {
	uint32_t u;
	memcpy(&u, &f, 4);
	uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
	uint32_t a    = u & 0x7fffffffu;
	if(a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
	if(a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* |x| >= 65536 (values that round up to it are caught below) */
	float af;
	memcpy(&af, &a, 4);
	if(af < 6.103515625e-05f) { /* below 2^-14: quantum 2^-24 */
		float q = nearbyintf(af * 16777216.0f);
		return (uint16_t)(sign | (uint16_t)q); /* q == 1024 is the first normal */
	}
	int   e;
	float m = frexpf(af, &e);
	int   E = e - 1;
	float q = nearbyintf((2.0f * m - 1.0f) * 1024.0f);
	if(q >= 1024.0f) {
		q = 0.0f;
		E += 1;
	}
	if(E > 15) return (uint16_t)(sign | 0x7c00u);
	return (uint16_t)(sign | (uint16_t)((E + 15) << 10) | (uint16_t)q);
}
uint8_t af3o_f32_to_e5m2_bits_reference(float f) {
	return (uint8_t)(f32_to_f16_bits_rne(f) >> 8);
}
uint8_t af3o_f32_to_e5m2_bits(float f) {
	uint32_t u;
	memcpy(&u, &f, 4);
	uint8_t  sign = (uint8_t)((u >> 24) & 0x80u);
	uint32_t a    = u & 0x7fffffffu;
	if(a > 0x7f800000u) return (uint8_t)(sign | 0x7fu);
	float af;
	memcpy(&af, &a, 4);
	if(af >= 65536.0f) return (uint8_t)(sign | 0x7cu);
	if(af < 6.103515625e-05f) { /* below 2^-14: quantum 2^-16 */
		float q = nearbyintf(af * 65536.0f);
		return (uint8_t)(sign | (uint8_t)q);
	}
	int   e;
	float m = frexpf(af, &e);
	int   E = e - 1;
	float q = nearbyintf((2.0f * m - 1.0f) * 4.0f);
	if(q >= 4.0f) {
		q = 0.0f;
		E += 1;
	}
	if(E > 15) return (uint8_t)(sign | 0x7cu);
	return (uint8_t)(sign | (uint8_t)((E + 15) << 2) | (uint8_t)q);
}
float af3o_e5m2_bits_to_f32(uint8_t b) {
	int   s = b & 0x80;
	int   E = (b >> 2) & 0x1f;
	int   m = b & 3;
	float v;
	if(E == 0x1f) {
		v = m ? NAN : INFINITY;
	} else if(E == 0) {
		v = (float)m * 1.52587890625e-05f; /* m * 2^-16 */
	} else {
		v = ldexpf(1.0f + (float)m / 4.0f, E - 15);
	}
	return s ? -v : v;
}
void af3o_convert_f32_to_e5m2(const float* in, uint8_t* out, int64_t n, int reference_rule) {
	for(int64_t i = 0; i < n; i++) {
		out[i] = reference_rule ? af3o_f32_to_e5m2_bits_reference(in[i]) : af3o_f32_to_e5m2_bits(in[i]);
	}
}
void af3o_convert_e5m2_to_f32(const uint8_t* in, float* out, int64_t n) {
	for(int64_t i = 0; i < n; i++) {
		out[i] = af3o_e5m2_bits_to_f32(in[i]);
	}
}

/* ConvertTPP::ref, xsmm_functors.h:867-873: out[i] = (Tout)in[i]. Array forms for the tests. */
void af3o_convert_f32_to_bf16(const float* in, uint16_t* out, int64_t n) {
	for(int64_t i = 0; i < n; i++) {
		out[i] = af3o_f32_to_bf16_bits(in[i]);
	}
}
void af3o_convert_bf16_to_f32(const uint16_t* in, float* out, int64_t n) {
	for(int64_t i = 0; i < n; i++) {
		out[i] = af3o_bf16_bits_to_f32(in[i]);
	}
}
/* Per-tensor scaled quantisation: scale = 448/amax (1 when amax == 0); q = e4m3(x*scale). */
float af3o_quantize_e4m3(const float* in, uint8_t* out, int64_t n) {
	float amax = 0.0f;
	for(int64_t i = 0; i < n; i++) {
		float a = fabsf(in[i]);
		if(a > amax) {
			amax = a;
		}
	}
	float scale = amax > 0.0f ? 448.0f / amax : 1.0f;
	for(int64_t i = 0; i < n; i++) {
		out[i] = af3o_f32_to_e4m3_bits(in[i] * scale);
	}
	return scale;
}
/* The shipped quantiser's variant: scale = 2^floor(log2(448 / (amax * |pre_scale|))) (1 when amax == 0),
 * q = e4m3(x * pre_scale * scale).  Power-of-two scales keep descale products exact. */
float af3o_quantize_e4m3_pow2(const float* in, uint8_t* out, int64_t n, float pre_scale) {
	float amax = 0.0f;
	for(int64_t i = 0; i < n; i++) {
		float a = fabsf(in[i]);
		if(a > amax) {
			amax = a;
		}
	}
	float a     = amax * fabsf(pre_scale);
	float scale = 1.0f;
	if(a > 0.0f && a < INFINITY) {
		int e;
		frexpf(448.0f / a, &e);
		scale = ldexpf(1.0f, e - 1);
	}
	for(int64_t i = 0; i < n; i++) {
		out[i] = af3o_f32_to_e4m3_bits(in[i] * pre_scale * scale);
	}
	return scale;
}
void af3o_dequantize_e4m3(const uint8_t* in, float* out, int64_t n, float inv_scale) {
	for(int64_t i = 0; i < n; i++) {
		out[i] = af3o_e4m3_bits_to_f32(in[i]) * inv_scale;
	}
}

/* ---- the TPP primitives on the path -------------------------------------------------- */

/* ScaleTPP::ref, xsmm_functors.h:1608-1613: alpha is rounded to T first, product stored as T. */
void af3o_scale(const float* in, float* out, int64_t n, float scale, int dtype) {
	float alpha = round_T(scale, dtype);
	for(int64_t i = 0; i < n; i++) {
		out[i] = round_T(in[i] * alpha, dtype);
	}
}

/*
 * BrgemmTPP::ref, xsmm_functors.h:2399-2444 (b_vnni == 0 branch, count == 1, beta == 0):
 * C[i][j] = sum_k A[i][k] * B[k][j], fp32 accumulate, one rounding to T on store.
 * b_trans != 0 means B is stored [N][K] (the logits GEMM, dot_product_attention.cpp:82).
 */
void af3o_brgemm(const float* A, const float* B, float* C, int M, int N, int K, int lda, int ldb, int ldc, int b_trans, int dtype) {
	for(int i = 0; i < M; i++) {
		for(int j = 0; j < N; j++) {
			float acc = 0.0f;
			if(b_trans) {
				for(int k = 0; k < K; k++) {
					acc += A[(int64_t)i * lda + k] * B[(int64_t)j * ldb + k];
				}
			} else {
				for(int k = 0; k < K; k++) {
					acc += A[(int64_t)i * lda + k] * B[(int64_t)k * ldb + j];
				}
			}
			C[(int64_t)i * ldc + j] = round_T(acc, dtype);
		}
	}
}

/* AddTPP::ref, xsmm_functors.h:1207-1227: out = in0 + in1 with three leading dimensions. */
void af3o_add(const float* in0, const float* in1, float* out, int rows, int cols, int ldi0, int ldi1, int ldo, int dtype) {
	for(int r = 0; r < rows; r++) {
		for(int c = 0; c < cols; c++) {
			out[(int64_t)r * ldo + c] = round_T(in0[(int64_t)r * ldi0 + c] + in1[(int64_t)r * ldi1 + c], dtype);
		}
	}
}

/* AddBiasTPP::ref, xsmm_functors.h:1079-1085: out[r][c] += in[c] (the key-mask add). */
void af3o_add_bias(const float* in, float* out, int rows, int cols, int ld, int dtype) {
	for(int r = 0; r < rows; r++) {
		for(int c = 0; c < cols; c++) {
			out[(int64_t)r * ld + c] = round_T(out[(int64_t)r * ld + c] + in[c], dtype);
		}
	}
}

/* SoftMaxFwdTPP::ref scalar branch, xsmm_functors.h:2920-2951 with S1 = 1: per row
 * max, exp(x - max) in fp32, multiply by 1/sum, store as T. */
void af3o_softmax_fwd(const float* in, float* out, int rows, int cols, int ld, int dtype) {
	float* tmp = (float*)malloc(sizeof(float) * (size_t)cols);
	for(int r = 0; r < rows; r++) {
		const float* x   = in + (int64_t)r * ld;
		float        max = x[0];
		float        sum = 0.0f;
		for(int c = 0; c < cols; c++) {
			if(max < x[c]) {
				max = x[c];
			}
		}
		for(int c = 0; c < cols; c++) {
			float z = expf(x[c] - max);
			tmp[c]  = z;
			sum += z;
		}
		sum = 1.0f / sum;
		for(int c = 0; c < cols; c++) {
			out[(int64_t)r * ld + c] = round_T(tmp[c] * sum, dtype);
		}
	}
	free(tmp);
}

/* VarSoftMaxFwdTPP::ref scalar branch with isFlash = true, xsmm_functors.h:3314-3361:
 * max starts from omax (when given), exp(x - max) stored un-normalised, max and sum returned. */
void af3o_var_softmax_flash(const float* in, float* out, int rows, int cols, int ld, float* max_buf, float* sum_buf, const float* omax_buf, int dtype) {
	for(int r = 0; r < rows; r++) {
		const float* x   = in + (int64_t)r * ld;
		float        max = omax_buf ? omax_buf[r] : x[0];
		float        sum = 0.0f;
		for(int c = 0; c < cols; c++) {
			if(max < x[c]) {
				max = x[c];
			}
		}
		for(int c = 0; c < cols; c++) {
			float z = expf(x[c] - max);
			sum += z;
			out[(int64_t)r * ld + c] = round_T(z, dtype);
		}
		max_buf[r] = max;
		sum_buf[r] = sum;
	}
}

/* SoftMaxFixUpTPP::ref with isFlash = true, xsmm_functors.h:3434-3462:
 * out = exp(omax - nmax) * out + cur; osum = csum + exp(omax - nmax) * osum; omax = nmax. */
void af3o_softmax_fixup_flash(const float* cur, float* out, int rows, int cols, const float* cmax, const float* csum, float* omax, float* osum, int dtype) {
	for(int r = 0; r < rows; r++) {
		float nmax = cmax[r] > omax[r] ? cmax[r] : omax[r];
		float oexp = expf(omax[r] - nmax);
		float nsum = csum[r] + oexp * osum[r];
		for(int c = 0; c < cols; c++) {
			out[(int64_t)r * cols + c] = round_T(oexp * out[(int64_t)r * cols + c] + cur[(int64_t)r * cols + c], dtype);
		}
		omax[r] = nmax;
		osum[r] = nsum;
	}
}

/* SoftMaxFlashScaleTPP::ref, xsmm_functors.h:3571-3581: buf[r][:] *= 1/osum[r]. */
void af3o_softmax_flash_scale(float* buf, const float* osum, int rows, int cols, int dtype) {
	for(int r = 0; r < rows; r++) {
		float isum = 1.0f / osum[r];
		for(int c = 0; c < cols; c++) {
			buf[(int64_t)r * cols + c] = round_T(buf[(int64_t)r * cols + c] * isum, dtype);
		}
	}
}

/*
 * pad_and_align_tensor restricted to what the path uses, tools.cpp:42-124: copy a
 * [rows][cols] block into the top-left corner of a [prows][pcols] block filled with `init`.
 * (Higher-rank tensors are padded by calling this once per leading index.)
 */
void af3o_pad_2d(const float* in, float* out, int64_t rows, int64_t cols, int64_t prows, int64_t pcols, float init) {
	for(int64_t r = 0; r < prows; r++) {
		for(int64_t c = 0; c < pcols; c++) {
			out[r * pcols + c] = (r < rows && c < cols) ? in[r * cols + c] : init;
		}
	}
}

/*
 * vnni_repack_tensor with type = XFORM_N2V, tools.cpp:151-176 + XformExtTPP::ref
 * xsmm_functors.h:2100-2111, for 16-bit elements (pack factor 2): per blk-wide column panel
 * starting at column p, out[p*M + i*blk*2 + j*2 + k] = in[(2i+k)*N + p + j].
 */
int af3o_vnni_repack(const uint16_t* in, uint16_t* out, int64_t M, int64_t N, int64_t blk) {
	if(blk == 0) {
		blk = N;
	}
	if(N % blk != 0 || (M & 1)) {
		return -1;
	}
	for(int64_t p = 0; p < N; p += blk) {
		uint16_t* o = out + p * M;
		for(int64_t i = 0; i < M / 2; i++) {
			for(int64_t j = 0; j < blk; j++) {
				for(int64_t k = 0; k < 2; k++) {
					o[i * blk * 2 + j * 2 + k] = in[(2 * i + k) * N + p + j];
				}
			}
		}
	}
	return 0;
}

/* ---- the driver ---------------------------------------------------------------------- */

/*
 * dot_product_attention_impl<T>, dot_product_attention.cpp:25-198, after the argument
 * preparation of src/af3_kernels/__init__.py:31-52 (mask lifted to [B,L], inverted, cast).
 *
 *   q,k,v : [B,H,L,D] fp32 values (already representable in T)
 *   bias  : [H,L,L]
 *   keep  : [B,L] bytes, non-zero = attend (the wrapper's un-inverted user mask)
 *   out   : [B,H,L,D]
 *
 * Steps, with the line each follows:
 *   :45-46   M = ceil(L/BLK)*BLK
 *   :50-54   zero-pad q,k,v,bias to M; pad the inverted mask with 1.0
 *   :63-74   mask *= T(-1e9)
 *   :88-122  non-flash core per (b,h,q-tile): scale, QK^T, +bias, +mask, softmax, PV
 *   :148-191 flash core: key axis in FLASH chunks (+ edge chunk), running max/sum, fix-up
 *   :194-197 narrow back to L
 * Every intermediate is rounded to T where the reference stores a T.
 * Returns 0, or -1 on allocation failure.
 */
int af3o_dpa_reference(const float* q, const float* k, const float* v, const float* bias, const uint8_t* keep, float* out, int64_t B, int64_t H, int64_t L, int64_t D, int dtype, int use_flash, int64_t BLK, int64_t FLASH) {
	const int64_t M  = (L + BLK - 1) / BLK * BLK;
	const int64_t Mb = M / BLK;
	float*        qp = (float*)calloc((size_t)(B * H * M * D), sizeof(float));
	float*        kp = (float*)calloc((size_t)(B * H * M * D), sizeof(float));
	float*        vp = (float*)calloc((size_t)(B * H * M * D), sizeof(float));
	float*        bp = (float*)calloc((size_t)(H * M * M), sizeof(float));
	float*        mp = (float*)malloc(sizeof(float) * (size_t)(B * M));
	if(!qp || !kp || !vp || !bp || !mp) {
		free(qp), free(kp), free(vp), free(bp), free(mp);
		return -1;
	}
	for(int64_t bh = 0; bh < B * H; bh++) {
		af3o_pad_2d(q + bh * L * D, qp + bh * M * D, L, D, M, D, 0.0f);
		af3o_pad_2d(k + bh * L * D, kp + bh * M * D, L, D, M, D, 0.0f);
		af3o_pad_2d(v + bh * L * D, vp + bh * M * D, L, D, M, D, 0.0f);
	}
	for(int64_t h = 0; h < H; h++) {
		af3o_pad_2d(bias + h * L * L, bp + h * M * M, L, L, M, M, 0.0f);
	}
	for(int64_t b = 0; b < B; b++) {
		for(int64_t c = 0; c < M; c++) {
			mp[b * M + c] = (c < L && keep[b * L + c]) ? 0.0f : 1.0f; /* ~mask, padded with 1.0 */
		}
		af3o_scale(mp + b * M, mp + b * M, M, -1e9f, dtype);
	}
	const float  scaling = 1.0f / sqrtf((float)D);
	const int    flash   = use_flash && M > FLASH;
	const int64_t ntask  = B * H * Mb;
	int           fail   = 0;
#pragma omp parallel for schedule(dynamic)
	for(int64_t t = 0; t < ntask; t++) {
		const int64_t i = t / (H * Mb), j = (t / Mb) % H, kb = t % Mb;
		float*        qt = qp + ((i * H + j) * M + kb * BLK) * D;
		const float*  kk = kp + (i * H + j) * M * D;
		const float*  vv = vp + (i * H + j) * M * D;
		const float*  bb = bp + (j * M + kb * BLK) * M;
		const float*  mm = mp + i * M;
		if(!flash) {
			float* tmp = (float*)malloc(sizeof(float) * (size_t)(BLK * M));
			if(!tmp) {
				fail = 1;
				continue;
			}
			af3o_scale(qt, qt, BLK * D, scaling, dtype);
			af3o_brgemm(qt, kk, tmp, (int)BLK, (int)M, (int)D, (int)D, (int)D, (int)M, 1, dtype);
			af3o_add(bb, tmp, tmp, 1, (int)(BLK * M), 0, 0, 0, dtype);
			af3o_add_bias(mm, tmp, (int)BLK, (int)M, (int)M, dtype);
			af3o_softmax_fwd(tmp, tmp, (int)BLK, (int)M, (int)M, dtype);
			af3o_brgemm(tmp, vv, qt, (int)BLK, (int)D, (int)M, (int)M, (int)D, (int)D, 0, dtype);
			free(tmp);
		} else {
			float* t1   = (float*)malloc(sizeof(float) * (size_t)(BLK * D));
			float* t2   = (float*)malloc(sizeof(float) * (size_t)(BLK * D));
			float* t3   = (float*)malloc(sizeof(float) * (size_t)(BLK * FLASH));
			float* st   = (float*)malloc(sizeof(float) * (size_t)(4 * BLK));
			if(!t1 || !t2 || !t3 || !st) {
				free(t1), free(t2), free(t3), free(st);
				fail = 1;
				continue;
			}
			float *omax = st, *osum = st + BLK, *cmax = st + 2 * BLK, *csum = st + 3 * BLK;
			af3o_scale(qt, qt, BLK * D, scaling, dtype);
			for(int64_t l = 0; l < M; l += FLASH) {
				const int64_t w = (M - l < FLASH) ? (M - l) : FLASH; /* edge chunk = M % FLASH, :138-146 */
				af3o_brgemm(qt, kk + l * D, t3, (int)BLK, (int)w, (int)D, (int)D, (int)D, (int)w, 1, dtype);
				af3o_add(bb + l, t3, t3, (int)BLK, (int)w, (int)M, (int)w, (int)w, dtype);
				af3o_add_bias(mm + l, t3, (int)BLK, (int)w, (int)w, dtype);
				if(l == 0) {
					af3o_var_softmax_flash(t3, t3, (int)BLK, (int)w, (int)w, omax, osum, NULL, dtype);
					af3o_brgemm(t3, vv + l * D, t2, (int)BLK, (int)D, (int)w, (int)w, (int)D, (int)D, 0, dtype);
				} else {
					af3o_var_softmax_flash(t3, t3, (int)BLK, (int)w, (int)w, cmax, csum, omax, dtype);
					af3o_brgemm(t3, vv + l * D, t1, (int)BLK, (int)D, (int)w, (int)w, (int)D, (int)D, 0, dtype);
					af3o_softmax_fixup_flash(t1, t2, (int)BLK, (int)D, cmax, csum, omax, osum, dtype);
				}
			}
			af3o_softmax_flash_scale(t2, osum, (int)BLK, (int)D, dtype);
			memcpy(qt, t2, sizeof(float) * (size_t)(BLK * D)); /* CpyTPP, :188 */
			free(t1), free(t2), free(t3), free(st);
		}
	}
	for(int64_t bh = 0; bh < B * H; bh++) {
		memcpy(out + bh * L * D, qp + bh * M * D, sizeof(float) * (size_t)(L * D)); /* narrow(2,0,L) */
	}
	free(qp), free(kp), free(vp), free(bp), free(mp);
	return fail ? -1 : 0;
}

/*
 * The reference harness's ground truth, examples/dot_product_attention.py:20-43:
 *   softmax(q*D^-1/2 . k^T + bias, masked_fill(~mask, -1e9)) . v
 * evaluated in double precision on the given fp32 values, result rounded once to fp32.
 * This is the comparator the stated tolerances (1e-4 / 2e-2 / 6e-2 max-abs) refer to.
 */
int af3o_dpa_formula(const float* q, const float* k, const float* v, const float* bias, const uint8_t* keep, float* out, int64_t B, int64_t H, int64_t L, int64_t D) {
	const double scaling = 1.0 / sqrt((double)D);
	int          fail    = 0;
#pragma omp parallel for schedule(dynamic)
	for(int64_t t = 0; t < B * H * L; t++) {
		const int64_t b = t / (H * L), h = (t / L) % H, r = t % L;
		double*       w = (double*)malloc(sizeof(double) * (size_t)L);
		if(!w) {
			fail = 1;
			continue;
		}
		const float* qr = q + ((b * H + h) * L + r) * D;
		double       mx = -INFINITY;
		for(int64_t c = 0; c < L; c++) {
			const float* kr = k + ((b * H + h) * L + c) * D;
			double       s  = 0.0;
			for(int64_t d = 0; d < D; d++) {
				s += (double)qr[d] * scaling * (double)kr[d];
			}
			s += bias ? (double)bias[(h * L + r) * L + c] : 0.0;
			if(keep && !keep[b * L + c]) {
				s = -1e9;
			}
			w[c] = s;
			if(s > mx) {
				mx = s;
			}
		}
		double sum = 0.0;
		for(int64_t c = 0; c < L; c++) {
			w[c] = exp(w[c] - mx);
			sum += w[c];
		}
		for(int64_t d = 0; d < D; d++) {
			double acc = 0.0;
			for(int64_t c = 0; c < L; c++) {
				acc += w[c] * (double)v[((b * H + h) * L + c) * D + d];
			}
			out[((b * H + h) * L + r) * D + d] = (float)(acc / sum);
		}
		free(w);
	}
	return fail ? -1 : 0;
}

/* ---- the two fused callers of the core ("next" rows) ------------------------------------ */

/* SigmoidFwdTPP::ref, xsmm_functors.h:2717-2723: out = 1 / (1 + exp(-in)), stored as T. */
void af3o_sigmoid(const float* in, float* out, int64_t n, int dtype) {
	for(int64_t i = 0; i < n; i++) {
		out[i] = round_T((float)(1. / (1. + exp(-(double)in[i]))), dtype);
	}
}

/* MulTPP::ref, xsmm_functors.h:1269-1275: out = in0 * in1, stored as T. */
void af3o_mul(const float* in0, const float* in1, float* out, int64_t n, int dtype) {
	for(int64_t i = 0; i < n; i++) {
		out[i] = round_T(in0[i] * in1[i], dtype);
	}
}

/*
 * Restatement of the two fused attention drivers:
 *   _attention_impl<T>      src/csrc/dot_product_attention.cpp:200-378  (wo != NULL, qbias == NULL)
 *   self_attention_impl<T>  src/csrc/dot_product_attention.cpp:380-543  (B == 1, wo == NULL, qbias optional)
 *
 *   x     : [B, L, C] input rows (the normalised pair rows / the single representation)
 *   keep  : [B, L] bytes, non-zero = attend
 *   bias  : [H, L, L]
 *   wq, wk, wv, wg : [C, C] = weight^T, natural row-major layout; head j uses columns j*K .. j*K+K-1,
 *           i.e. the [C, K] panel the reference addresses as q_a[j] (:241-244, :418-423) after its
 *           VNNI repack of the same matrix (the repack itself is af3o_vnni_repack)
 *   wo    : [C, C] = output_projection.weight^T or NULL
 *   qbias : [C] or NULL (added to q before the scaling, :490-492)
 *   out   : [B, L, C]
 *
 * Per (row i, head j), with every stored intermediate rounded to T as the reference stores a T:
 *   :290-303 / :461-476  k, v = x_i . Wk_j, x_i . Wv_j over the whole padded row
 *   :306-310 / :471-476  q = x_tile . Wq_j          (:490-492 q += q_bias)
 *   :311-314 / :493-496  q *= K^-1/2
 *   :315-319 / :497-501  logits = q . k^T
 *   :320-326 / :502-507  logits += bias ; logits += mask * -1e9
 *   :331-333 / :508-510  softmax over the padded row
 *   :334-338 / :511-515  weighted = P . v
 *   :339-349 / :516-527  gate = sigmoid(x_tile . Wg_j) ; out_a = weighted * gate
 *   :356-372             out = out_a . Wo   (_attention only)
 * M = ceil(L/BLK)*BLK; padded input rows are zero, padded mask entries dropped, padded bias 0.
 * Returns 0, or -1 on allocation failure.
 */
int af3o_fused_attention_reference(const float* x, const uint8_t* keep, const float* bias, const float* wq, const float* wk, const float* wv, const float* wg,
								   const float* wo, const float* qbias, float* out, int64_t B, int64_t L, int64_t C, int64_t H, int dtype, int64_t BLK) {
	const int64_t K = C / H, M = (L + BLK - 1) / BLK * BLK, Mb = M / BLK;
	float*        xp = (float*)calloc((size_t)(B * M * C), sizeof(float));
	float*        bp = (float*)calloc((size_t)(H * M * M), sizeof(float));
	float*        mp = (float*)malloc(sizeof(float) * (size_t)(B * M));
	float*        oa = (float*)calloc((size_t)(B * M * C), sizeof(float));
	if(!xp || !bp || !mp || !oa) {
		free(xp), free(bp), free(mp), free(oa);
		return -1;
	}
	for(int64_t i = 0; i < B; i++) af3o_pad_2d(x + i * L * C, xp + i * M * C, L, C, M, C, 0.0f);
	for(int64_t h = 0; h < H; h++) af3o_pad_2d(bias + h * L * L, bp + h * M * M, L, L, M, M, 0.0f);
	for(int64_t i = 0; i < B; i++) {
		for(int64_t c = 0; c < M; c++) mp[i * M + c] = (c < L && keep[i * L + c]) ? 0.0f : 1.0f;
		af3o_scale(mp + i * M, mp + i * M, M, -1e9f, dtype);
	}
	const float scaling = 1.0f / sqrtf((float)K);
	int         fail    = 0;
#pragma omp parallel for schedule(dynamic)
	for(int64_t t = 0; t < B * H; t++) {
		const int64_t i = t / H, j = t % H;
		float*        tk = (float*)malloc(sizeof(float) * (size_t)(M * K));
		float*        tv = (float*)malloc(sizeof(float) * (size_t)(M * K));
		float*        tq = (float*)malloc(sizeof(float) * (size_t)(BLK * K));
		float*        to = (float*)malloc(sizeof(float) * (size_t)(BLK * (M > K ? M : K)));
		if(!tk || !tv || !tq || !to) {
			free(tk), free(tv), free(tq), free(to);
			fail = 1;
			continue;
		}
		const float* xi = xp + i * M * C;
		af3o_brgemm(xi, wk + j * K, tk, (int)M, (int)K, (int)C, (int)C, (int)C, (int)K, 0, dtype);
		af3o_brgemm(xi, wv + j * K, tv, (int)M, (int)K, (int)C, (int)C, (int)C, (int)K, 0, dtype);
		for(int64_t kb = 0; kb < Mb; kb++) {
			const float* xt = xi + kb * BLK * C;
			af3o_brgemm(xt, wq + j * K, tq, (int)BLK, (int)K, (int)C, (int)C, (int)C, (int)K, 0, dtype);
			if(qbias) af3o_add_bias(qbias + j * K, tq, (int)BLK, (int)K, (int)K, dtype);
			af3o_scale(tq, tq, BLK * K, scaling, dtype);
			af3o_brgemm(tq, tk, to, (int)BLK, (int)M, (int)K, (int)K, (int)K, (int)M, 1, dtype);
			af3o_add(bp + (j * M + kb * BLK) * M, to, to, 1, (int)(BLK * M), 0, 0, 0, dtype);
			af3o_add_bias(mp + i * M, to, (int)BLK, (int)M, (int)M, dtype);
			af3o_softmax_fwd(to, to, (int)BLK, (int)M, (int)M, dtype);
			af3o_brgemm(to, tv, tq, (int)BLK, (int)K, (int)M, (int)M, (int)K, (int)K, 0, dtype);
			af3o_brgemm(xt, wg + j * K, to, (int)BLK, (int)K, (int)C, (int)C, (int)C, (int)K, 0, dtype);
			af3o_sigmoid(to, to, BLK * K, dtype);
			for(int64_t r = 0; r < BLK; r++) af3o_mul(to + r * K, tq + r * K, oa + (i * M + kb * BLK + r) * C + j * K, K, dtype);
		}
		free(tk), free(tv), free(tq), free(to);
	}
	if(!fail) {
		for(int64_t i = 0; i < B; i++) {
			if(wo) {
				float* row = (float*)malloc(sizeof(float) * (size_t)(M * C));
				if(!row) {
					fail = 1;
					break;
				}
				af3o_brgemm(oa + i * M * C, wo, row, (int)M, (int)C, (int)C, (int)C, (int)C, (int)C, 0, dtype);
				memcpy(out + i * L * C, row, sizeof(float) * (size_t)(L * C)); /* narrow(1, 0, Mp) */
				free(row);
			} else {
				memcpy(out + i * L * C, oa + i * M * C, sizeof(float) * (size_t)(L * C));
			}
		}
	}
	free(xp), free(bp), free(mp), free(oa);
	return fail ? -1 : 0;
}

/*
 * Ground truth of the two fused callers in double precision: the torch modules of the reference's
 * own harnesses (examples/grid_self_attention.py:46-94 without the LayerNorm / bias projection that
 * precede the op, examples/self_attention.py:64-96), evaluated on the given fp32 values and rounded
 * once to fp32.  Same arguments as af3o_fused_attention_reference.
 */
int af3o_fused_attention_formula(const float* x, const uint8_t* keep, const float* bias, const float* wq, const float* wk, const float* wv, const float* wg,
								 const float* wo, const float* qbias, float* out, int64_t B, int64_t L, int64_t C, int64_t H) {
	const int64_t K = C / H;
	double*       ga = (double*)malloc(sizeof(double) * (size_t)(B * L * C)); /* gated weighted average */
	if(!ga) return -1;
	int fail = 0;
#pragma omp parallel for schedule(dynamic)
	for(int64_t t = 0; t < B * H; t++) {
		const int64_t i = t / H, j = t % H;
		double*       q = (double*)malloc(sizeof(double) * (size_t)(L * K) * 4);
		double*       w = (double*)malloc(sizeof(double) * (size_t)L);
		if(!q || !w) {
			free(q), free(w);
			fail = 1;
			continue;
		}
		double *k = q + L * K, *v = k + L * K, *g = v + L * K;
		for(int64_t r = 0; r < L; r++) {
			for(int64_t d = 0; d < K; d++) {
				double sq = qbias ? (double)qbias[j * K + d] : 0.0, sk = 0.0, sv = 0.0, sg = 0.0;
				for(int64_t c = 0; c < C; c++) {
					const double xv = (double)x[(i * L + r) * C + c];
					sq += xv * (double)wq[c * C + j * K + d];
					sk += xv * (double)wk[c * C + j * K + d];
					sv += xv * (double)wv[c * C + j * K + d];
					sg += xv * (double)wg[c * C + j * K + d];
				}
				q[r * K + d] = sq / sqrt((double)K), k[r * K + d] = sk, v[r * K + d] = sv, g[r * K + d] = 1.0 / (1.0 + exp(-sg));
			}
		}
		for(int64_t r = 0; r < L; r++) {
			double mx = -INFINITY, sum = 0.0;
			for(int64_t c = 0; c < L; c++) {
				double sdot = 0.0;
				for(int64_t d = 0; d < K; d++) sdot += q[r * K + d] * k[c * K + d];
				sdot += (double)bias[(j * L + r) * L + c];
				if(!keep[i * L + c]) sdot = -1e9;
				w[c] = sdot;
				if(sdot > mx) mx = sdot;
			}
			for(int64_t c = 0; c < L; c++) {
				w[c] = exp(w[c] - mx);
				sum += w[c];
			}
			for(int64_t d = 0; d < K; d++) {
				double acc = 0.0;
				for(int64_t c = 0; c < L; c++) acc += w[c] * v[c * K + d];
				ga[(i * L + r) * C + j * K + d] = acc / sum * g[r * K + d];
			}
		}
		free(q), free(w);
	}
	if(!fail) {
#pragma omp parallel for schedule(static)
		for(int64_t r = 0; r < B * L; r++) {
			for(int64_t o = 0; o < C; o++) {
				if(wo) {
					double acc = 0.0;
					for(int64_t c = 0; c < C; c++) acc += ga[r * C + c] * (double)wo[c * C + o];
					out[r * C + o] = (float)acc;
				} else {
					out[r * C + o] = (float)ga[r * C + o];
				}
			}
		}
	}
	free(ga);
	return fail ? -1 : 0;
}

/* ---- the step in front of grid self-attention ("next" row) -------------------------------- */

/*
 * LayerNorm over the C channels of every token and the per-head bias projection of the normalised row, in
 * double precision: normed = (x - mean) / sqrt(var + eps) * gamma + beta (biased variance, torch.nn.LayerNorm),
 * bias[h][t] = normed[t] . wb[h]  (src/af3_kernels/Attention.py:51-52: act_norm, pair_bias_projection, permute(2,0,1);
 * examples/grid_self_attention.py:71-72).  x [T][C], wb [H][C] (nn.Linear weight), normed [T][C], bias [H][T].
 * round_bf16 != 0 rounds the normalised row to bf16 before it is stored and projected, and the bias after, which is what
 * the reference's bf16 module does between its torch ops.
 */
int af3o_layernorm_pair_bias(const float* x, const float* gamma, const float* beta, const float* wb, double eps, float* normed, float* bias, int64_t T, int64_t C, int64_t H,
							 int round_bf16) {
#pragma omp parallel for schedule(static)
	for(int64_t t = 0; t < T; t++) {
		const float* xr   = x + t * C;
		double       mean = 0.0, var = 0.0;
		for(int64_t c = 0; c < C; c++) mean += xr[c];
		mean /= (double)C;
		for(int64_t c = 0; c < C; c++) var += ((double)xr[c] - mean) * ((double)xr[c] - mean);
		var /= (double)C;
		const double rstd = 1.0 / sqrt(var + eps);
		for(int64_t c = 0; c < C; c++) {
			float y = (float)(((double)xr[c] - mean) * rstd * (double)gamma[c] + (double)beta[c]);
			if(round_bf16) y = af3o_bf16_bits_to_f32(af3o_f32_to_bf16_bits(y));
			normed[t * C + c] = y;
		}
		for(int64_t h = 0; h < H; h++) {
			double d = 0.0;
			for(int64_t c = 0; c < C; c++) d += (double)normed[t * C + c] * (double)wb[h * C + c];
			float b = (float)d;
			if(round_bf16) b = af3o_bf16_bits_to_f32(af3o_f32_to_bf16_bits(b));
			bias[h * T + t] = b;
		}
	}
	return 0;
}

/* ---- gated linear unit ("next" row) -------------------------------------------------------- */

/*
 * out[m][n] = silu(a) * b with a = x[m] . w[:, n], b = x[m] . w[:, N + n]  (examples/gated_linear_unit.py:18-22),
 * x [M][K], w [K][2N] row-major.  round_bf16 == 0: double precision throughout.  round_bf16 != 0: the reference's
 * bf16 pipeline (src/csrc/gated_linear_unit.cpp:56-61): both products accumulated in fp32 and rounded to bf16,
 * silu evaluated in fp32 on the rounded value and rounded, the product rounded.
 */
int af3o_gated_linear_unit(const float* x, const float* w, float* out, int64_t M, int64_t K, int64_t N, int round_bf16) {
#pragma omp parallel for schedule(static)
	for(int64_t m = 0; m < M; m++) {
		for(int64_t n = 0; n < N; n++) {
			if(!round_bf16) {
				double a = 0.0, b = 0.0;
				for(int64_t k = 0; k < K; k++) {
					a += (double)x[m * K + k] * (double)w[k * 2 * N + n];
					b += (double)x[m * K + k] * (double)w[k * 2 * N + N + n];
				}
				out[m * N + n] = (float)(a / (1.0 + exp(-a)) * b);
			} else {
				float a = 0.f, b = 0.f;
				for(int64_t k = 0; k < K; k++) {
					a += x[m * K + k] * w[k * 2 * N + n];
					b += x[m * K + k] * w[k * 2 * N + N + n];
				}
				a             = af3o_bf16_bits_to_f32(af3o_f32_to_bf16_bits(a));
				b             = af3o_bf16_bits_to_f32(af3o_f32_to_bf16_bits(b));
				const float s = af3o_bf16_bits_to_f32(af3o_f32_to_bf16_bits(a / (1.f + expf(-a))));
				out[m * N + n] = af3o_bf16_bits_to_f32(af3o_f32_to_bf16_bits(s * b));
			}
		}
	}
	return 0;
}
