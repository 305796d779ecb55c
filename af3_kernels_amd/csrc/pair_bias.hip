// The step in front of grid self-attention, fused: LayerNorm over the 128 pair channels and the projection of
// the normalised row to one bias value per head,
//     normed[i][j][:] = (x[i][j][:] - mean) * rstd * gamma + beta          bias[h][i][j] = normed[i][j][:] . Wb[h][:]
// (torch ops in the reference: src/af3_kernels/Attention.py:51-52, examples/grid_self_attention.py:71-72).
// HBM-bound: x is read once, normed written once, and the [H, N, N] bias comes out in the layout the attention
// kernels stream (no permute pass over a [N, N, H] intermediate).
//
// Work split.  A token's 128 bf16 channels are 256 bytes = 16 lanes x 16 bytes, so one wave-wide load covers four
// consecutive tokens, fully coalesced; all reductions over channels stay inside a row of 16 lanes (DPP).  A
// wavefront handles 64 consecutive tokens j of one pair row i in 16 such steps and keeps the four bias values of
// step `it` in lane 16g + it of group g, so that after the last step every lane owns one token and each head's 64
// values leave as one 128-byte store.
#include "common.hpp"

namespace af3 {

namespace {

constexpr int PB_C     = 128;  // channels
constexpr int PB_H     = 4;    // heads
constexpr int PB_WAVES = 4;    // wavefronts per workgroup

// sum over the 16 lanes of a DPP row; every lane of the row receives the total
template <int CTRL>
__device__ __forceinline__ float dpp_add(float x) {
	return x + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float row16_sum(float x) {
	x = dpp_add<0xB1>(x);   // quad_perm [1,0,3,2]
	x = dpp_add<0x4E>(x);   // quad_perm [2,3,0,1]
	x = dpp_add<0x141>(x);  // row_half_mirror
	x = dpp_add<0x140>(x);  // row_mirror
	return x;
}

__device__ __forceinline__ void unpack8(const u32x4& raw, float (&f)[8]) {
#pragma unroll
	for(int j = 0; j < 4; j++) f[2 * j] = bf16_bits_to_f32(raw[j] & 0xffffu), f[2 * j + 1] = bf16_bits_to_f32(raw[j] >> 16);
}

__global__ void __launch_bounds__(PB_WAVES * 64) layernorm_pair_bias_kernel(const uint16_t* __restrict__ x, int64_t x_stride_i, int64_t x_stride_j, const uint16_t* __restrict__ gamma,
																			 const uint16_t* __restrict__ beta, const uint16_t* __restrict__ wb, float eps, uint16_t* __restrict__ normed,
																			 uint16_t* __restrict__ bias, int64_t n_i, int64_t n_j, int64_t bias_stride_h, int64_t bias_stride_i) {
	const int     lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
	const int     sub = lane & 15, grp = lane >> 4;  // channel chunk, token within a step
	const int64_t n_jblocks = (n_j + 63) / 64;
	const int64_t unit      = (int64_t)blockIdx.x * PB_WAVES + wave;
	if(unit >= n_i * n_jblocks) return;
	const int64_t i = unit / n_jblocks, j0 = (unit % n_jblocks) * 64;

	// per-lane constants for channels 8*sub .. 8*sub+7
	float g[8], bt[8], w[PB_H][8];
	unpack8(*reinterpret_cast<const u32x4*>(gamma + 8 * sub), g);
	unpack8(*reinterpret_cast<const u32x4*>(beta + 8 * sub), bt);
#pragma unroll
	for(int h = 0; h < PB_H; h++) unpack8(*reinterpret_cast<const u32x4*>(wb + h * PB_C + 8 * sub), w[h]);

	float mine[PB_H] = {0.f, 0.f, 0.f, 0.f};
	for(int it = 0; it < 16; it++) {
		const int64_t j  = j0 + 4 * it + grp;
		const bool    ok = j < n_j;
		u32x4         raw = {0u, 0u, 0u, 0u};
		if(ok) raw = *reinterpret_cast<const u32x4*>(x + i * x_stride_i + j * x_stride_j + 8 * sub);
		float v[8];
		unpack8(raw, v);
		float s = 0.f;
#pragma unroll
		for(int c = 0; c < 8; c++) s += v[c];
		const float mean = row16_sum(s) * (1.f / PB_C);
		float       ss   = 0.f;
#pragma unroll
		for(int c = 0; c < 8; c++) {
			v[c] -= mean;
			ss = __builtin_fmaf(v[c], v[c], ss);
		}
		const float rstd = __builtin_amdgcn_rsqf(row16_sum(ss) * (1.f / PB_C) + eps);
		// the normalised row, rounded to bf16: what is stored is also what is projected (as the reference's
		// Linear sees the LayerNorm's bf16 output)
		u32x4 o;
#pragma unroll
		for(int c = 0; c < 8; c += 2) {
			const float a = __builtin_fmaf(v[c] * rstd, g[c], bt[c]), b = __builtin_fmaf(v[c + 1] * rstd, g[c + 1], bt[c + 1]);
			o[c >> 1] = pack_bf16x2(a, b);
		}
		if(ok) *reinterpret_cast<u32x4*>(normed + ((i * n_j + j) * PB_C) + 8 * sub) = o;
		float y[8];
		unpack8(o, y);
#pragma unroll
		for(int h = 0; h < PB_H; h++) {
			float d = 0.f;
#pragma unroll
			for(int c = 0; c < 8; c++) d = __builtin_fmaf(y[c], w[h][c], d);
			d = row16_sum(d);
			if(sub == it) mine[h] = d;
		}
	}
	// lane (grp, sub) now owns token 4*sub + grp of this block of 64
	const int64_t j = j0 + 4 * sub + grp;
	if(j < n_j) {
#pragma unroll
		for(int h = 0; h < PB_H; h++) bias[h * bias_stride_h + i * bias_stride_i + j] = (uint16_t)f32_to_bf16_bits(mine[h]);
	}
}

}  // namespace

}  // namespace af3

using namespace af3;

extern "C" int af3_layernorm_pair_bias(const void* pair, const int64_t* pair_stride, const void* ln_weight, const void* ln_bias, float eps, const void* proj_weight,
									   void* normed, void* bias, const int64_t* bias_stride, int64_t n_i, int64_t n_j, int64_t C, int64_t head, int32_t dtype, void* stream) {
	if(!pair || !pair_stride || !ln_weight || !ln_bias || !proj_weight || !normed || !bias || !bias_stride) return AF3_ERR_NULL_POINTER;
	if(n_i <= 0 || n_j <= 0 || n_i > 0x3fffffff || n_j > 0x3fffffff) return AF3_ERR_BAD_SHAPE;
	if(dtype != AF3_BF16) return AF3_ERR_BAD_DTYPE;
	if(C != PB_C || head != PB_H) return AF3_ERR_BAD_ARGUMENT;
	if(!(eps >= 0.f)) return AF3_ERR_BAD_ARGUMENT;
	if(pair_stride[0] < 0 || pair_stride[1] < C || pair_stride[0] % 8 || pair_stride[1] % 8 || bias_stride[0] < 0 || bias_stride[1] < n_j) return AF3_ERR_BAD_STRIDE;
	for(const void* ptr : {pair, ln_weight, ln_bias, proj_weight, static_cast<const void*>(normed)})
		if(reinterpret_cast<uintptr_t>(ptr) & 15) return AF3_ERR_BAD_ARGUMENT;
	if(reinterpret_cast<uintptr_t>(bias) & 1) return AF3_ERR_BAD_ARGUMENT;
	const int64_t units  = n_i * ((n_j + 63) / 64);
	const int64_t blocks = (units + PB_WAVES - 1) / PB_WAVES;
	if(blocks > 0x7fffffffLL) return AF3_ERR_BAD_SHAPE;
	hipLaunchKernelGGL(layernorm_pair_bias_kernel, dim3((unsigned)blocks), dim3(PB_WAVES * 64), 0, static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(pair), pair_stride[0],
					   pair_stride[1], static_cast<const uint16_t*>(ln_weight), static_cast<const uint16_t*>(ln_bias), static_cast<const uint16_t*>(proj_weight), eps,
					   static_cast<uint16_t*>(normed), static_cast<uint16_t*>(bias), n_i, n_j, bias_stride[0], bias_stride[1]);
	return launch_status();
}
