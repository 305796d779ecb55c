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

// ---- any channel count, any head count, bfloat16 or float32 ---------------------------------------------------------------
// One wavefront per token, lane l on channels l, l + 64, ...: PER = ceil(C / 64) values per lane stay in registers for the
// three passes (mean, centred sum of squares, normalise + project), so the row is read once.  gamma, beta and the projection
// weights are staged in LDS as float32 once per workgroup.  Every reduction is a butterfly over the 64 lanes, one per head
// for the projection.  The specialised kernel above serves the pair tensor's own shape (128 channels, 4 heads, bfloat16).
constexpr int PBG_WAVES = 4;

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
	for(int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off);
	return x;
}

template <int PER, bool F32>
__global__ void __launch_bounds__(PBG_WAVES * 64) layernorm_pair_bias_any_kernel(const void* __restrict__ x, int64_t x_stride_i, int64_t x_stride_j, const void* __restrict__ gamma,
																				   const void* __restrict__ beta, const void* __restrict__ wb, float eps, void* __restrict__ normed,
																				   void* __restrict__ bias, int64_t n_i, int64_t n_j, int64_t bias_stride_h, int64_t bias_stride_i, int C, int H) {
	extern __shared__ float pbg_smem[];   // [gamma C][beta C][wb H x C]
	float* const s_g = pbg_smem;
	float* const s_b = pbg_smem + C;
	float* const s_w = pbg_smem + 2 * C;
	auto ld = [](const void* p, int64_t i) -> float { return F32 ? static_cast<const float*>(p)[i] : bf16_bits_to_f32(static_cast<const uint16_t*>(p)[i]); };
	for(int c = threadIdx.x; c < C; c += PBG_WAVES * 64) s_g[c] = ld(gamma, c), s_b[c] = ld(beta, c);
	for(int c = threadIdx.x; c < H * C; c += PBG_WAVES * 64) s_w[c] = ld(wb, c);
	__syncthreads();
	const int     lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
	const int64_t tokens = n_i * n_j;
	const float   inv_c  = 1.f / (float)C;
	for(int64_t t = (int64_t)blockIdx.x * PBG_WAVES + wave; t < tokens; t += (int64_t)gridDim.x * PBG_WAVES) {
		const int64_t i = t / n_j, j = t % n_j, base = i * x_stride_i + j * x_stride_j;
		float v[PER];
		float s = 0.f;
#pragma unroll
		for(int k = 0; k < PER; k++) {
			const int c = lane + 64 * k;
			v[k]        = c < C ? ld(x, base + c) : 0.f;
			s += v[k];
		}
		const float mean = wave_sum(s) * inv_c;
		float       ss   = 0.f;
#pragma unroll
		for(int k = 0; k < PER; k++) {
			const int c = lane + 64 * k;
			v[k]        = c < C ? v[k] - mean : 0.f;
			ss          = __builtin_fmaf(v[k], v[k], ss);
		}
		const float rstd = __builtin_amdgcn_rsqf(wave_sum(ss) * inv_c + eps);
		// the normalised row in the output's precision: what is stored is also what is projected
#pragma unroll
		for(int k = 0; k < PER; k++) {
			const int c = lane + 64 * k;
			if(c < C) {
				float y = __builtin_fmaf(v[k] * rstd, s_g[c], s_b[c]);
				if(F32) static_cast<float*>(normed)[t * C + c] = y;
				else {
					const uint32_t bits = f32_to_bf16_bits(y);
					static_cast<uint16_t*>(normed)[t * C + c] = (uint16_t)bits;
					y = bf16_bits_to_f32(bits);
				}
				v[k] = y;
			}
		}
		for(int h = 0; h < H; h++) {
			float d = 0.f;
#pragma unroll
			for(int k = 0; k < PER; k++) {
				const int c = lane + 64 * k;
				if(c < C) d = __builtin_fmaf(v[k], s_w[h * C + c], d);
			}
			d = wave_sum(d);
			if(lane == 0) {
				const int64_t o = h * bias_stride_h + i * bias_stride_i + j;
				if(F32) static_cast<float*>(bias)[o] = d;
				else static_cast<uint16_t*>(bias)[o] = (uint16_t)f32_to_bf16_bits(d);
			}
		}
	}
}

template <bool F32>
int launch_pair_bias_any(int per, dim3 grid, size_t smem, hipStream_t s, const void* x, int64_t si, int64_t sj, const void* g, const void* b, const void* w, float eps, void* normed,
						 void* bias, int64_t n_i, int64_t n_j, int64_t bsh, int64_t bsi, int C, int H) {
#define AF3_PBG(P)                                                                                                                                                          \
	{                                                                                                                                                                   \
		auto kern = layernorm_pair_bias_any_kernel<P, F32>;                                                                                                                \
		if(smem > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) return AF3_ERR_LAUNCH; \
		hipLaunchKernelGGL(kern, grid, dim3(PBG_WAVES * 64), smem, s, x, si, sj, g, b, w, eps, normed, bias, n_i, n_j, bsh, bsi, C, H);                                     \
	}
	if(per <= 1) AF3_PBG(1)
	else if(per <= 2) AF3_PBG(2)
	else if(per <= 4) AF3_PBG(4)
	else if(per <= 6) AF3_PBG(6)
	else if(per <= 8) AF3_PBG(8)
	else if(per <= 12) AF3_PBG(12)
	else if(per <= 16) AF3_PBG(16)
	else AF3_PBG(32)
#undef AF3_PBG
	return launch_status();
}

}  // namespace

}  // namespace af3

using namespace af3;

extern "C" int af3_layernorm_pair_bias(const void* pair, const int64_t* pair_stride, const void* ln_weight, const void* ln_bias, float eps, const void* proj_weight,
									   void* normed, void* bias, const int64_t* bias_stride, int64_t n_i, int64_t n_j, int64_t C, int64_t head, int32_t dtype, void* stream) {
	if(!pair || !pair_stride || !ln_weight || !ln_bias || !proj_weight || !normed || !bias || !bias_stride) return AF3_ERR_NULL_POINTER;
	if(n_i <= 0 || n_j <= 0 || n_i > 0x3fffffff || n_j > 0x3fffffff) return AF3_ERR_BAD_SHAPE;
	if(dtype != AF3_BF16 && dtype != AF3_F32) return AF3_ERR_BAD_DTYPE;
	if(C <= 0 || head <= 0) return AF3_ERR_BAD_SHAPE;
	if(!(eps >= 0.f)) return AF3_ERR_BAD_ARGUMENT;
	if(pair_stride[0] < 0 || pair_stride[1] < C || bias_stride[0] < 0 || bias_stride[1] < n_j) return AF3_ERR_BAD_STRIDE;
	const uintptr_t esz = dtype == AF3_F32 ? 4 : 2;
	for(const void* ptr : {pair, ln_weight, ln_bias, proj_weight, static_cast<const void*>(normed), static_cast<const void*>(bias)})
		if(reinterpret_cast<uintptr_t>(ptr) & (esz - 1)) return AF3_ERR_BAD_ARGUMENT;
	bool fast = dtype == AF3_BF16 && C == PB_C && head == PB_H && pair_stride[0] % 8 == 0 && pair_stride[1] % 8 == 0;
	for(const void* ptr : {pair, ln_weight, ln_bias, proj_weight, static_cast<const void*>(normed)}) fast = fast && (reinterpret_cast<uintptr_t>(ptr) & 15) == 0;
	if(!fast) {
		// any other shape: one wavefront per token (at most 2048 channels; gamma, beta and the weights as float32 in LDS)
		if(C > 2048 || head > 64 || (2 + head) * C * 4 > 160 * 1024 - 1024) return AF3_ERR_BAD_ARGUMENT;
		const int64_t tokens = n_i * n_j;
		const int64_t want   = (tokens + PBG_WAVES - 1) / PBG_WAVES;
		const dim3    grid((unsigned)(want > 256 * 16 ? 256 * 16 : want));
		const size_t  smem = (size_t)(2 + head) * C * 4;
		const int     per  = (int)((C + 63) / 64);
		hipStream_t   st   = static_cast<hipStream_t>(stream);
		return dtype == AF3_F32 ? launch_pair_bias_any<true>(per, grid, smem, st, pair, pair_stride[0], pair_stride[1], ln_weight, ln_bias, proj_weight, eps, normed, bias, n_i, n_j,
															 bias_stride[0], bias_stride[1], (int)C, (int)head)
								: launch_pair_bias_any<false>(per, grid, smem, st, pair, pair_stride[0], pair_stride[1], ln_weight, ln_bias, proj_weight, eps, normed, bias, n_i, n_j,
															  bias_stride[0], bias_stride[1], (int)C, (int)head);
	}
	const int64_t units  = n_i * ((n_j + 63) / 64);
	const int64_t blocks = (units + PB_WAVES - 1) / PB_WAVES;
	if(blocks > 0x7fffffffLL) return AF3_ERR_BAD_SHAPE;
	hipLaunchKernelGGL(layernorm_pair_bias_kernel, dim3((unsigned)blocks), dim3(PB_WAVES * 64), 0, static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(pair), pair_stride[0],
					   pair_stride[1], static_cast<const uint16_t*>(ln_weight), static_cast<const uint16_t*>(ln_bias), static_cast<const uint16_t*>(proj_weight), eps,
					   static_cast<uint16_t*>(normed), static_cast<uint16_t*>(bias), n_i, n_j, bias_stride[0], bias_stride[1]);
	return launch_status();
}
