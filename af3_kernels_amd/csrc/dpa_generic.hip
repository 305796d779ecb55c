// fp32-FMA attention kernel: any head_dim <= 128, any strides, fp32 or bf16 storage.
//
// This is the precision path (fp32 inputs, 1e-4 against the fp64 formula) and the fallback for
// shapes the matrix-core kernels do not take.  One 64-lane wavefront owns one query row and
// walks the key axis in chunks with a running max / sum (the recurrence of the reference's
// flash branch, src/csrc/dot_product_attention.cpp:148-191, kept in fp32 throughout):
//   phase 1  lanes over keys : s = scale * q.k + bias, dropped keys replaced by a constant
//   phase 2  lanes over keys : p = exp(s - m_new), chunk sum
//   phase 3  lanes over head : acc[d] = alpha * acc[d] + sum_j p[j] * v[j][d]
#include "common.hpp"

namespace af3 {

constexpr int GEN_WAVES = 4;    // query rows per workgroup
constexpr int GEN_CHUNK = 512;  // keys per chunk (LDS: 4 waves * (128 + 512) floats = 10 KB)

__device__ __forceinline__ float load_as_f32(const void* base, int64_t idx, int dtype) {
	if(dtype == AF3_F32) return static_cast<const float*>(base)[idx];
	return bf16_bits_to_f32(static_cast<const uint16_t*>(base)[idx]);
}

__device__ __forceinline__ float wave_max(float x) {
	for(int o = 32; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o));
	return x;
}
__device__ __forceinline__ float wave_sum(float x) {
	for(int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o);
	return x;
}

__global__ void __launch_bounds__(GEN_WAVES * 64) dpa_generic_kernel(af3_dpa_params p) {
	__shared__ float qs[GEN_WAVES][AF3_DPA_MAX_HEAD_DIM];
	__shared__ float pbuf[GEN_WAVES][GEN_CHUNK];
	const int     wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
	const int64_t rows_per_bh = (p.L + GEN_WAVES - 1) / GEN_WAVES;
	const int64_t bh  = blockIdx.x / rows_per_bh;
	const int64_t row = (blockIdx.x % rows_per_bh) * GEN_WAVES + wave;
	const int64_t b = bh / p.H, h = bh % p.H;
	if(row >= p.L) return;  // whole wave leaves; no workgroup barrier is used below
	const int D = (int)p.D;

	const int64_t qoff = b * p.q_stride[0] + h * p.q_stride[1] + row * p.q_stride[2];
	for(int d = lane; d < D; d += 64) qs[wave][d] = load_as_f32(p.q, qoff + d, p.io_dtype) * p.softmax_scale;
	__builtin_amdgcn_wave_barrier();
	__builtin_amdgcn_s_waitcnt(0);

	const int64_t  koff = b * p.k_stride[0] + h * p.k_stride[1];
	const int64_t  voff = b * p.v_stride[0] + h * p.v_stride[1];
	const int64_t  boff = h * p.bias_stride[0] + row * p.bias_stride[1];
	const uint8_t* keep = p.key_mask ? p.key_mask + b * p.key_mask_stride_b : nullptr;

	float m = -INFINITY, l = 0.f, acc0 = 0.f, acc1 = 0.f;
	for(int64_t c0 = 0; c0 < p.L; c0 += GEN_CHUNK) {
		const int n = (int)((p.L - c0 < GEN_CHUNK) ? (p.L - c0) : GEN_CHUNK);
		float cmax = -INFINITY;
		for(int j = lane; j < n; j += 64) {
			const int64_t key = c0 + j;
			const int64_t kr  = koff + key * p.k_stride[2];
			float s = 0.f;
			for(int d = 0; d < D; d++) s = fmaf(qs[wave][d], load_as_f32(p.k, kr + d, p.io_dtype), s);
			if(p.bias) s = fmaxf(s + load_as_f32(p.bias, boff + key, p.bias_dtype), -3.0e38f);  // (-inf in the bias: finite, so that a chunk of such keys leaves a finite maximum)
			if(keep && !keep[key]) s = MASK_DROPPED;  // masked_fill semantics: the logit is replaced
			pbuf[wave][j] = s;
			cmax = fmaxf(cmax, s);
		}
		cmax = wave_max(cmax);
		const float m_new = fmaxf(m, cmax);
		const float alpha = expf(m - m_new);  // exp(-inf) = 0 on the first chunk
		float csum = 0.f;
		for(int j = lane; j < n; j += 64) {
			const float e = expf(pbuf[wave][j] - m_new);
			pbuf[wave][j] = e;
			csum += e;
		}
		csum = wave_sum(csum);
		l = l * alpha + csum;
		m = m_new;
		__builtin_amdgcn_wave_barrier();
		__builtin_amdgcn_s_waitcnt(0);
		float s0 = 0.f, s1 = 0.f;
		const bool has0 = lane < D, has1 = lane + 64 < D;
		for(int j = 0; j < n; j++) {
			const float   e  = pbuf[wave][j];
			const int64_t vr = voff + (c0 + j) * p.v_stride[2];
			if(has0) s0 = fmaf(e, load_as_f32(p.v, vr + lane, p.io_dtype), s0);
			if(has1) s1 = fmaf(e, load_as_f32(p.v, vr + lane + 64, p.io_dtype), s1);
		}
		acc0 = acc0 * alpha + s0;
		acc1 = acc1 * alpha + s1;
		__builtin_amdgcn_wave_barrier();
	}
	const float   inv  = 1.f / l;
	const int64_t ooff = b * p.out_stride[0] + h * p.out_stride[1] + row * p.out_stride[2];
	for(int t = 0; t < 2; t++) {
		const int d = lane + 64 * t;
		if(d >= D) break;
		float o = (t == 0 ? acc0 : acc1) * inv;
		if(p.gate) o *= sigmoidf_fast(load_as_f32(p.gate, b * p.gate_stride[0] + h * p.gate_stride[1] + row * p.gate_stride[2] + d, p.io_dtype));
		if(p.out_dtype == AF3_F32) static_cast<float*>(p.out)[ooff + d] = o;
		else static_cast<uint16_t*>(p.out)[ooff + d] = (uint16_t)f32_to_bf16_bits(o);
	}
}

int launch_dpa_generic(const af3_dpa_params& p, hipStream_t s) {
	const int64_t rows_per_bh = (p.L + GEN_WAVES - 1) / GEN_WAVES;
	const int64_t blocks      = p.B * p.H * rows_per_bh;
	if(blocks <= 0 || blocks > 0x7fffffffLL) return AF3_ERR_BAD_SHAPE;
	hipLaunchKernelGGL(dpa_generic_kernel, dim3((unsigned)blocks), dim3(GEN_WAVES * 64), 0, s, p);
	return launch_status();
}

}  // namespace af3
