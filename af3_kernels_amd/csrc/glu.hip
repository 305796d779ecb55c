// Gated linear unit of the transition blocks in one kernel: out = silu(x . Wa) * (x . Wb), with W = [Wa | Wb] of shape
// [K, 2N], K = 64 or 128 input channels, N >= 32 output channels.  The product x . W (twice the size of the output)
// never exists in memory.
// Reference: gated_linear_unit_impl, src/csrc/gated_linear_unit.cpp:20-80 (per 128 x 128 block: BRGEMM, SiLU, BRGEMM,
// multiply); formula examples/gated_linear_unit.py:18-22.
//
// HBM-bound (rows in, rows out); the work split keeps every byte to one trip:
//   * a workgroup owns up to 512 output columns: wavefront w holds the weight fragments of gate columns
//     [32w, 32w+32) and of the matching value columns in registers for its whole life;
//   * it walks blocks of 32 rows (persistent, grid-strided); a block of x (32 x K bf16) is fetched once, 16 bytes per
//     thread, coalesced, into a double-buffered LDS tile from which all wavefronts read their MFMA operand;
//   * out^T[col][row] = W^T . x^T on v_mfma_f32_32x32x16_bf16: lane = row, registers = 4 x 4 consecutive columns, so
//     silu * value is in-lane and the result leaves as 8-byte stores.
#include "common.hpp"

namespace af3 {

namespace {

constexpr int GLU_MAX_WAVES = 16;

template <int KS>  // contraction steps of 16 channels: K = 16 * KS
__global__ void __launch_bounds__(GLU_MAX_WAVES * 64) glu_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ wt, uint16_t* __restrict__ out, int64_t M, int64_t N,
																  int n_waves) {
	constexpr int K          = 16 * KS;
	constexpr int ROW_BYTES  = K * 2;
	constexpr int CHUNKS     = 32 * ROW_BYTES / 16;  // 16-byte pieces of one block of x
	constexpr int TILE_BYTES = 32 * ROW_BYTES;
	__shared__ __attribute__((aligned(16))) unsigned char xs[2][TILE_BYTES];

	const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int n = lane & 31, half = lane >> 5;
	const int64_t col0   = ((int64_t)blockIdx.y * GLU_MAX_WAVES + wave) * 32;  // first gate column of this wavefront
	const bool    active = wave < n_waves && col0 < N;

	// weight fragments (A operand): lane (column n, g = half), step s: W^T[col][16s + 8g .. +7]; wt is [2N, K] row-major
	u32x4 wa[KS], wb[KS];
#pragma unroll
	for(int s = 0; s < KS; s++) {
		wa[s] = wb[s] = u32x4{0u, 0u, 0u, 0u};
		if(active) {
			wa[s] = *reinterpret_cast<const u32x4*>(wt + (col0 + n) * K + 16 * s + 8 * half);
			wb[s] = *reinterpret_cast<const u32x4*>(wt + (N + col0 + n) * K + 16 * s + 8 * half);
		}
	}

	const int64_t n_blocks = (M + 31) / 32;
	// x block loader: thread t < CHUNKS moves piece t (row t / (CHUNKS/32), 16-byte chunk t % (CHUNKS/32)); the chunk index is
	// XOR-swizzled with the row so that the operand reads below (same chunk, 8 consecutive rows per LDS cycle) spread over the banks
	constexpr int CPR  = ROW_BYTES / 16;
	const int     ld_r = tid / CPR, ld_c = tid % CPR;
	const int     ld_dst = ld_r * ROW_BYTES + ((ld_c ^ (ld_r & 7)) << 4);
	auto fetch = [&](int64_t blk) -> u32x4 {
		const int64_t row = blk * 32 + ld_r;
		if(tid < CHUNKS && row < M) return *reinterpret_cast<const u32x4*>(x + row * K + ld_c * 8);
		return u32x4{0u, 0u, 0u, 0u};
	};

	int64_t blk = blockIdx.x;
	if(blk >= n_blocks) return;  // (whole workgroup)
	u32x4 staged = fetch(blk);
	if(tid < CHUNKS) *reinterpret_cast<u32x4*>(xs[0] + ld_dst) = staged;
	__syncthreads();
	int buf = 0;
	for(; blk < n_blocks; blk += gridDim.x) {
		const int64_t next = blk + gridDim.x;
		if(next < n_blocks) staged = fetch(next);  // in flight during this block's matrix work
		if(active) {
			f32x16 ga, va;
#pragma unroll
			for(int i = 0; i < 16; i++) ga[i] = 0.f, va[i] = 0.f;
#pragma unroll
			for(int s = 0; s < KS; s++) {
				const u32x4 xf = *reinterpret_cast<const u32x4*>(xs[buf] + n * ROW_BYTES + (((2 * s + half) ^ (n & 7)) << 4));
				ga = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, wa[s]), __builtin_bit_cast(bf16x8, xf), ga, 0, 0, 0);
				va = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, wb[s]), __builtin_bit_cast(bf16x8, xf), va, 0, 0, 0);
			}
			const int64_t row = blk * 32 + n;
			if(row < M) {
				uint16_t* orow = out + row * N + col0 + 4 * half;
#pragma unroll
				for(int g4 = 0; g4 < 4; g4++) {
					float o[4];
#pragma unroll
					for(int r = 0; r < 4; r++) {
						const float a = ga[4 * g4 + r];
						o[r] = a * va[4 * g4 + r] * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-a * LOG2E));  // silu(a) * b
					}
					*reinterpret_cast<u32x2*>(orow + 8 * g4) = u32x2{pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3])};
				}
			}
		}
		if(next < n_blocks) {
			if(tid < CHUNKS) *reinterpret_cast<u32x4*>(xs[buf ^ 1] + ld_dst) = staged;  // (last read two barriers ago)
			__syncthreads();
			buf ^= 1;
		}
	}
}

}  // namespace

}  // namespace af3

using namespace af3;

extern "C" int af3_gated_linear_unit(const void* x, const void* weight_t, void* out, int64_t M, int64_t K, int64_t N, int32_t dtype, void* stream) {
	if(!x || !weight_t || !out) return AF3_ERR_NULL_POINTER;
	if(M <= 0 || N <= 0 || K <= 0 || M > ((int64_t)1 << 40)) return AF3_ERR_BAD_SHAPE;
	if(dtype != AF3_BF16) return AF3_ERR_BAD_DTYPE;
	if((K != 64 && K != 128) || N % 32 != 0) return AF3_ERR_BAD_ARGUMENT;
	if((reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(weight_t) & 15) || (reinterpret_cast<uintptr_t>(out) & 7)) return AF3_ERR_BAD_ARGUMENT;
	const int64_t col_tiles = N / 32;
	const int     n_waves   = (int)(col_tiles < GLU_MAX_WAVES ? col_tiles : GLU_MAX_WAVES);
	// the x loader needs one thread per 16-byte piece of a block: 32 * K / 8 threads
	const int     threads   = (n_waves * 64 < 4 * K ? 4 * (int)K : n_waves * 64);
	const int64_t n_blocks  = (M + 31) / 32;
	const dim3    grid((unsigned)(n_blocks < 512 ? n_blocks : 512), (unsigned)((col_tiles + GLU_MAX_WAVES - 1) / GLU_MAX_WAVES));
	const auto    s = static_cast<hipStream_t>(stream);
	const auto*   xp = static_cast<const uint16_t*>(x);
	const auto*   wp = static_cast<const uint16_t*>(weight_t);
	auto*         op = static_cast<uint16_t*>(out);
	if(K == 128)
		hipLaunchKernelGGL(glu_kernel<8>, grid, dim3(threads), 0, s, xp, wp, op, M, N, n_waves);
	else
		hipLaunchKernelGGL(glu_kernel<4>, grid, dim3(threads), 0, s, xp, wp, op, M, N, n_waves);
	return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}
