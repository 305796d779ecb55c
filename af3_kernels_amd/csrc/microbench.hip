// Microbenchmarks behind the attention kernel's design notes (built into libaf3_microbench.so, not into the product
// library; run with `python -m af3_kernels_amd.microbench`).  They answer three questions about one gfx950 SIMD:
//   1. How well do the matrix pipe and the vector ALU overlap on the kernel's instruction mix?        (mix_kernel)
//   2. What does one stage of the bf16 attention kernel cost without any memory instruction, with its true
//      dependences -- and what do its LDS fragment reads, its bias-fragment loads, a second chain per wavefront and
//      random (instead of constant) operands add?                                                      (stage_kernel)
//   3. How fast do 16-byte loads stream a buffer that sits in L2, in MALL or in HBM?                   (stream_kernel)
// Timing is taken on the host (events around a launch of `iters` loop trips); results are meaningless numbers that
// only keep the compiler from dropping the work.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

#define FENCE() __builtin_amdgcn_sched_barrier(0)
#define AS_BF(x) __builtin_bit_cast(bf16x8, x)
#define AS_HF(x) __builtin_bit_cast(f16x8, x)

__device__ __forceinline__ uint32_t pack2(float a, float b) {
	bf16x2 p = {(__bf16)a, (__bf16)b};
	return __builtin_bit_cast(uint32_t, p);
}

// exp2 and pack of N of the 16 values of a 32x32 accumulator block, starting at I0
template <int I0, int N>
__device__ __forceinline__ void exp_pack(const f32x16& s, u32x4 (&p)[2]) {
#pragma unroll
	for(int i = I0; i < I0 + N; i += 2) p[i >> 3][(i & 7) >> 1] = pack2(__builtin_amdgcn_exp2f(s[i]), __builtin_amdgcn_exp2f(s[i + 1]));
}

// ---- 1. independent matrix and vector work ---------------------------------------------------------------------
// MODE 0: 8 MFMAs only; 1: 16 exp2 + 8 packs only; 2: MFMA, exp2, exp2, pack (x8); 3: 8 MFMAs, then 16 exp2, then 8 packs;
// 4: as 0 with operands taken from the buffer (random data) instead of constants
template <int MODE>
__global__ void __launch_bounds__(1024) mix_kernel(float* out, const u32x4* __restrict__ buf, int iters, float seed) {
	f32x16 acc[2];
	for(int j = 0; j < 2; j++)
		for(int i = 0; i < 16; i++) acc[j][i] = 0.f;
	bf16x8 a, b;
	for(int i = 0; i < 8; i++) a[i] = (__bf16)(seed + threadIdx.x), b[i] = (__bf16)(seed * 2 + i);
	if(MODE == 4) a = AS_BF(buf[threadIdx.x]), b = AS_BF(buf[1024 + threadIdx.x]);
	float t[16];
	for(int i = 0; i < 16; i++) t[i] = seed * (i + 1) - 3.f;
	uint32_t pk[8] = {0, 0, 0, 0, 0, 0, 0, 0};
	for(int it = 0; it < iters; it++) {
		if constexpr(MODE == 0 || MODE == 4) {
#pragma unroll
			for(int m = 0; m < 8; m++) {
				acc[m & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[m & 1], 0, 0, 0);
				FENCE();
			}
		} else if constexpr(MODE == 1) {
#pragma unroll
			for(int m = 0; m < 8; m++) {
				t[2 * m] = __builtin_amdgcn_exp2f(t[2 * m]), t[2 * m + 1] = __builtin_amdgcn_exp2f(t[2 * m + 1]);
				pk[(m + 7) & 7] ^= pack2(t[2 * ((m + 7) & 7)], t[2 * ((m + 7) & 7) + 1]);
				FENCE();
			}
		} else if constexpr(MODE == 2) {
#pragma unroll
			for(int m = 0; m < 8; m++) {
				acc[m & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[m & 1], 0, 0, 0);
				FENCE();
				t[2 * m] = __builtin_amdgcn_exp2f(t[2 * m]), t[2 * m + 1] = __builtin_amdgcn_exp2f(t[2 * m + 1]);
				pk[m] ^= pack2(t[2 * m], t[2 * m + 1]);
				FENCE();
			}
		} else {
#pragma unroll
			for(int m = 0; m < 8; m++) acc[m & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[m & 1], 0, 0, 0);
			FENCE();
#pragma unroll
			for(int x = 0; x < 16; x++) t[x] = __builtin_amdgcn_exp2f(t[x]);
			FENCE();
#pragma unroll
			for(int m = 0; m < 8; m++) pk[m] ^= pack2(t[2 * m], t[2 * m + 1]);
			FENCE();
		}
	}
	float r = 0.f;
	for(int j = 0; j < 2; j++)
		for(int i = 0; i < 16; i++) r += acc[j][i];
	for(int i = 0; i < 16; i++) r += t[i];
	for(int i = 0; i < 8; i++) r += (float)pk[i];
	out[blockIdx.x * blockDim.x + threadIdx.x] = r;
}

// ---- 2. one stage of the attention kernel, without its memory instructions ---------------------------------------
// State of one (32 query rows x keys) chain, as the kernel keeps it between stages.
struct chain_state {
	f32x16 oacc, s_a, s_b;  // O^T accumulator; S^T of the current and of the next sub-tile (ping-pong)
	f32x4  lacc;            // row sums
	u32x4  p_a[2], p_b[2];  // P^T fragments of the previous and of the current sub-tile (ping-pong)
	u32x4  qf[2];           // Q fragments
};

// FLAGS: 1 = bias fragments by two 16-byte buffer loads per stage (used one stage later); 2 = K/V fragments by LDS reads
// every stage; 4 = operands start from the buffer's (random) contents instead of constants; 8 = no row-sum check.
// CHAINS: 1 or 2 chains per wavefront (the second shares the K/V fragments and takes the vector work while the first
// takes the matrix work, and vice versa).
template <int FLAGS, int CHAINS>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(CHAINS == 1 ? 4 : 2)))
stage_kernel(float* out, const u32x4* __restrict__ buf, int n_vec, int iters, float seed) {
	constexpr bool LOADS = FLAGS & 1, LDSRD = FLAGS & 2, RANDOM = FLAGS & 4, CHECK = !(FLAGS & 8);
	__shared__ unsigned char lds[LDSRD ? 1280 * 16 : 16];
	const int lane = threadIdx.x & 63;
	chain_state c[CHAINS];
	u32x4       vf[2], kf[2], idf[2], bf_a[2], bf_b[2], mask_a, mask_b, ones;
	for(int x = 0; x < CHAINS; x++) {
		for(int i = 0; i < 16; i++) c[x].oacc[i] = 0.f, c[x].s_a[i] = -seed * i, c[x].s_b[i] = -seed * 2 * i;
		c[x].lacc = f32x4{0.f, 0.f, 0.f, 0.f};
		for(int j = 0; j < 2; j++)
			for(int i = 0; i < 4; i++) c[x].p_a[j][i] = c[x].p_b[j][i] = 0x3c003c00u, c[x].qf[j][i] = 0x3c003c00u + threadIdx.x + x;
	}
	for(int j = 0; j < 2; j++)
		for(int i = 0; i < 4; i++) {
			vf[j][i] = 0x3f803f80u + threadIdx.x, kf[j][i] = 0x3c003c00u + i, idf[j][i] = (i == (int)(threadIdx.x & 3)) ? 0x3c00u : 0u;
			bf_a[j][i] = bf_b[j][i] = 0x2c002c00u, mask_a[i] = 0u, mask_b[i] = 0x3f80u, ones[i] = 0x3f803f80u;
		}
	if(RANDOM) {
		for(int j = 0; j < 2; j++) {
			vf[j] = buf[threadIdx.x + 256 * j], kf[j] = buf[threadIdx.x + 512 + 256 * j], bf_a[j] = buf[threadIdx.x + 1024 + 256 * j], bf_b[j] = buf[threadIdx.x + 1536 + 256 * j];
			for(int x = 0; x < CHAINS; x++) c[x].p_a[j] = buf[threadIdx.x + 2048 + 512 * x + 256 * j], c[x].qf[j] = buf[threadIdx.x + 3072 + 512 * x + 256 * j];
		}
	}
	if(LDSRD) {
		for(int i = threadIdx.x; i < 1280 * 4; i += 256) reinterpret_cast<uint32_t*>(lds)[i] = RANDOM ? buf[i >> 2][i & 3] : 0x3c003c00u;
		__syncthreads();
	}
	int redo = 0, lpos = 0;
	int pos = __builtin_amdgcn_readfirstlane((int)(((long long)(blockIdx.x * 4 + (threadIdx.x >> 6)) * 7919) % (n_vec / 128)) * 128);
	const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<u32x4*>(buf), 0, n_vec * 16, 0x00020000);
	f32x16 zero;
	for(int i = 0; i < 16; i++) zero[i] = 0.f;

	// One stage: chain M runs the matrix side (PV of its previous sub-tile, S^T of its next one), chain V the vector side
	// (exp2 / pack / row sum of its current sub-tile).  With one chain per wavefront M == V, as in the kernel.
	auto stage = [&](chain_state& M, chain_state& V, f32x16& m_sn, const u32x4 (&m_pp)[2], const f32x16& v_sc, u32x4 (&v_pc)[2], const u32x4 (&bias_now)[2],
					 u32x4 (&bias_next)[2]) {
		asm volatile("" : "+v"(kf[0][0]));  // (keeps the loop-invariant S^T product inside the loop)
		if(LDSRD) {
			kf[0] = *reinterpret_cast<const u32x4*>(lds + ((lpos & 511) + lane) * 16);
			kf[1] = *reinterpret_cast<const u32x4*>(lds + ((lpos & 511) + 64 + lane) * 16);
			lpos += 128;
		}
		FENCE();
		M.oacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(AS_BF(vf[0]), AS_BF(m_pp[0]), M.oacc, 0, 0, 0);
		exp_pack<0, 2>(v_sc, v_pc);
		FENCE();
		M.oacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(AS_BF(vf[1]), AS_BF(m_pp[1]), M.oacc, 0, 0, 0);
		exp_pack<2, 2>(v_sc, v_pc);
		FENCE();
		m_sn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(AS_BF(kf[0]), AS_BF(M.qf[0]), zero, 0, 0, 0);
		if(LDSRD) {
			vf[0] = *reinterpret_cast<const u32x4*>(lds + (512 + (lpos & 511) + lane) * 16);
			vf[1] = *reinterpret_cast<const u32x4*>(lds + (512 + (lpos & 511) + 64 + lane) * 16);
		}
		exp_pack<4, 2>(v_sc, v_pc);
		FENCE();
		m_sn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(AS_BF(kf[1]), AS_BF(M.qf[1]), m_sn, 0, 0, 0);
		exp_pack<6, 2>(v_sc, v_pc);
		FENCE();
		m_sn   = __builtin_amdgcn_mfma_f32_32x32x16_f16(AS_HF(idf[0]), AS_HF(bias_now[0]), m_sn, 0, 0, 0);
		V.lacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(AS_BF(ones), AS_BF(v_pc[0]), V.lacc, 0, 0, 0);
		exp_pack<8, 2>(v_sc, v_pc);
		FENCE();
		m_sn = __builtin_amdgcn_mfma_f32_32x32x16_f16(AS_HF(idf[1]), AS_HF(bias_now[1]), m_sn, 0, 0, 0);
		exp_pack<10, 2>(v_sc, v_pc);
		FENCE();
		if(LOADS) {
			bias_next[0] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane * 16, pos * 16, 0));
			bias_next[1] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane * 16 + 1024, pos * 16, 0));
			pos += 128;
			if(pos >= n_vec) pos -= n_vec;
		}
		m_sn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(AS_BF(mask_a), AS_BF(mask_b), m_sn, 0, 0, 0);
		exp_pack<12, 4>(v_sc, v_pc);
		FENCE();
		V.lacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(AS_BF(ones), AS_BF(v_pc[1]), V.lacc, 0, 0, 0);
		FENCE();
		if(CHECK) {
			if(__ballot(!(V.lacc[0] < 1e30f))) redo++, V.lacc[0] = 0.f;
		}
	};

	if constexpr(CHAINS == 1) {
		for(int it = 0; it < iters; it += 2) {  // two stages per trip: the S^T and P^T blocks swap roles
			stage(c[0], c[0], c[0].s_b, c[0].p_a, c[0].s_a, c[0].p_b, bf_a, bf_b);
			stage(c[0], c[0], c[0].s_a, c[0].p_b, c[0].s_b, c[0].p_a, bf_b, bf_a);
		}
	} else {
		for(int it = 0; it < iters; it += 2) {  // four half-stages per trip = two stages of each chain
			stage(c[0], c[1], c[0].s_b, c[0].p_a, c[1].s_a, c[1].p_b, bf_a, bf_b);
			stage(c[1], c[0], c[1].s_a, c[1].p_b, c[0].s_b, c[0].p_a, bf_b, bf_a);
			stage(c[0], c[1], c[0].s_b, c[0].p_a, c[1].s_a, c[1].p_b, bf_a, bf_b);
			stage(c[1], c[0], c[1].s_a, c[1].p_b, c[0].s_b, c[0].p_a, bf_b, bf_a);
		}
	}
	float r = (float)redo;
	for(int x = 0; x < CHAINS; x++) {
		for(int i = 0; i < 16; i++) r += c[x].oacc[i] + c[x].s_a[i] + c[x].s_b[i];
		for(int i = 0; i < 4; i++) r += c[x].lacc[i];
	}
	out[blockIdx.x * blockDim.x + threadIdx.x] = r;
}

// ---- 3. streaming a buffer with 16-byte loads ----------------------------------------------------------------------
__global__ void __launch_bounds__(256) stream_kernel(const u32x4* __restrict__ buf, uint32_t* out, int n_vec, int iters) {
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
	u32x4     acc  = {0, 0, 0, 0};
	int       pos  = (int)(((long long)(blockIdx.x * 4 + wave) * 7919) % (n_vec / 64)) * 64;
	for(int it = 0; it < iters; it++) {
#pragma unroll
		for(int u = 0; u < 8; u++) {
			const u32x4 v = buf[pos + lane];
			acc[0] ^= v[0], acc[1] ^= v[1], acc[2] ^= v[2], acc[3] ^= v[3];
			pos += 64 * 13;
			if(pos >= n_vec) pos -= n_vec;
		}
	}
	if((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678u) out[0] = 1;
}

template <int FLAGS>
int launch_stage(int chains, int grid, float* out, const u32x4* buf, int n_vec, int iters, hipStream_t s) {
	if(chains == 1) hipLaunchKernelGGL((stage_kernel<FLAGS, 1>), dim3(grid), dim3(256), 0, s, out, buf, n_vec, iters, 0.001f);
	else hipLaunchKernelGGL((stage_kernel<FLAGS, 2>), dim3(grid), dim3(256), 0, s, out, buf, n_vec, iters, 0.001f);
	return 0;
}

}  // namespace

// which = 0: mix_kernel<variant> on `threads` threads per workgroup; 1: stage_kernel<flags = variant & 15, chains = 1 + (variant >> 4)> on 256 threads;
// 2: stream_kernel on 256 threads (8 KB per wavefront and trip).  out: at least grid * threads floats; buf: n_vec 16-byte vectors (n_vec a multiple
// of 128, at least 4096).  Returns 0, -1 for an unknown selector, -2 for a bad size, -3 when the launch failed.
extern "C" int af3_microbench_run(int which, int variant, int grid, int threads, void* out, const void* buf, int n_vec, int iters, void* stream) {
	hipStream_t s = static_cast<hipStream_t>(stream);
	if(grid <= 0 || iters <= 0 || !out) return -2;
	if(which == 0) {
		if(threads <= 0 || threads > 1024 || threads % 64 || !buf || n_vec < 4096) return -2;
		float*       o = static_cast<float*>(out);
		const u32x4* b = static_cast<const u32x4*>(buf);
		switch(variant) {
			case 0: hipLaunchKernelGGL(mix_kernel<0>, dim3(grid), dim3(threads), 0, s, o, b, iters, 0.001f); break;
			case 1: hipLaunchKernelGGL(mix_kernel<1>, dim3(grid), dim3(threads), 0, s, o, b, iters, 0.001f); break;
			case 2: hipLaunchKernelGGL(mix_kernel<2>, dim3(grid), dim3(threads), 0, s, o, b, iters, 0.001f); break;
			case 3: hipLaunchKernelGGL(mix_kernel<3>, dim3(grid), dim3(threads), 0, s, o, b, iters, 0.001f); break;
			case 4: hipLaunchKernelGGL(mix_kernel<4>, dim3(grid), dim3(threads), 0, s, o, b, iters, 0.001f); break;
			default: return -1;
		}
	} else if(which == 1) {
		if(!buf || n_vec < 4096 || n_vec % 128 || iters % 2) return -2;
		const int    chains = 1 + (variant >> 4);
		float*       o      = static_cast<float*>(out);
		const u32x4* b      = static_cast<const u32x4*>(buf);
		if(chains > 2) return -1;
		switch(variant & 15) {
			case 0: launch_stage<0>(chains, grid, o, b, n_vec, iters, s); break;
			case 1: launch_stage<1>(chains, grid, o, b, n_vec, iters, s); break;
			case 2: launch_stage<2>(chains, grid, o, b, n_vec, iters, s); break;
			case 3: launch_stage<3>(chains, grid, o, b, n_vec, iters, s); break;
			case 4: launch_stage<4>(chains, grid, o, b, n_vec, iters, s); break;
			case 7: launch_stage<7>(chains, grid, o, b, n_vec, iters, s); break;
			case 8: launch_stage<8>(chains, grid, o, b, n_vec, iters, s); break;
			default: return -1;
		}
	} else if(which == 2) {
		if(!buf || n_vec < 4096 || n_vec % 64) return -2;
		hipLaunchKernelGGL(stream_kernel, dim3(grid), dim3(256), 0, s, static_cast<const u32x4*>(buf), static_cast<uint32_t*>(out), n_vec, iters);
	} else {
		return -1;
	}
	return hipGetLastError() == hipSuccess ? 0 : -3;
}
