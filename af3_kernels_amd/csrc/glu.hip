// Gated linear unit of the transition blocks in one kernel: out = silu(x . Wa) * (x . Wb), with W = [Wa | Wb] of shape
// [K, 2N], K = 64 or 128 input channels, N >= 32 output channels.  The product x . W (twice the size of the output)
// never exists in memory.
// Reference: gated_linear_unit_impl, src/csrc/gated_linear_unit.cpp:20-80 (per 128 x 128 block: BRGEMM, SiLU, BRGEMM,
// multiply); formula examples/gated_linear_unit.py:18-22.
//
// HBM-bound (rows in, rows out).  Work split:
//   * a workgroup owns up to 512 output columns: wavefront w holds the weight fragments of gate columns
//     [32w, 32w+32) and of the matching value columns in registers for its whole life;
//   * it walks blocks of 32 rows (persistent, grid-strided); a block of x (32 x K bf16, one contiguous piece of memory) is
//     fetched once, every thread a few bytes, coalesced, into a double-buffered LDS tile from which all wavefronts read
//     their MFMA operand (reading the operand straight from memory in every wavefront -- 16 bytes per lane from 32 different
//     rows, sixteen wavefronts per block -- was tried: twice as slow);
//   * out^T[col][row] = W^T . x^T on v_mfma_f32_32x32x16_bf16: lane = row, registers = 4 x 4 consecutive columns, so
//     silu * value is in-lane;
//   * the 32 x 32 result tile is turned through a private LDS patch so that it leaves as 16-byte stores, four lanes per
//     64-byte row segment (8-byte stores straight from the accumulator layout made the memory system handle four times
//     as many write requests).
// Two details keep a wavefront from waiting for its own stores to be acknowledged in every block:
//   * loads and stores go through buffer descriptors of one block each (wave-uniform base, hardware range check), so rows
//     past M read zeros / store nothing without a branch around the instruction -- after a branch the compiler waits for
//     ALL outstanding memory operations where only the next block's rows are needed;
//   * the registers that feed the stores are kept out of circulation until the next block's stores (the compiler waits for
//     a store before it lets anything overwrite the store's data registers, and would otherwise hand them to the next
//     block's first matrix instruction).
// Also measured and not kept: four 16 x 16 sub-tiles on v_mfma_f32_16x16x32_bf16 with the silu of one sub-tile placed
// behind the next one's products (same instruction count, meant to overlap the two pipes inside a wavefront): 13-18 % slower.
#include <type_traits>

#include "common.hpp"

namespace af3 {

namespace {

constexpr int GLU_MAX_WAVES = 16;

// KS: contraction steps of 16 channels (K = 16 * KS).  WAVES: wavefronts per workgroup = 32-column tiles it owns.
// GATED: out = silu(x . Wa) * (x . Wb) with wt = [Wa | Wb]^T; otherwise the plain product out = x . W with wt = W^T.
template <int KS, int WAVES, bool GATED>
// (four wavefronts per SIMD whatever the workgroup size: 128 registers each)
__global__ void __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(4))) glu_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ wt, uint16_t* __restrict__ out, int64_t M, int64_t N) {
	constexpr int K          = 16 * KS;
	constexpr int ROW_BYTES  = K * 2;
	constexpr int TILE_BYTES = 32 * ROW_BYTES;
	constexpr int TPB        = TILE_BYTES / (WAVES * 64);  // bytes of a block per thread: 4 .. 32
	constexpr int PIECE      = TPB < 16 ? TPB : 16;         // moved in pieces of at most 16 bytes
	constexpr int PPT        = TPB / PIECE;
	constexpr int OUT_STRIDE = 80;  // bytes per row of the output patch: 64 of data, padded so that rows start in different banks
	static_assert(TILE_BYTES % (WAVES * 64) == 0 && TPB >= 4 && TPB % PIECE == 0, "every thread moves whole pieces of a block");
	__shared__ __attribute__((aligned(16))) unsigned char xs[2][TILE_BYTES];
	__shared__ __attribute__((aligned(16))) unsigned char os[WAVES][32 * OUT_STRIDE];

	const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int n = lane & 31, half = lane >> 5;
	const int64_t col0   = ((int64_t)blockIdx.y * WAVES + wave) * 32;  // first (gate) column of this wavefront
	const bool    active = col0 < N;  // wavefronts past the last column only help to move x

	// weight fragments (A operand): lane (column n, g = half), step s: W^T[col][16s + 8g .. +7]; wt is [2N, K] ([N, K]) row-major
	u32x4 wa[KS], wb[GATED ? KS : 1];
#pragma unroll
	for(int s = 0; s < KS; s++) {
		wa[s] = u32x4{0u, 0u, 0u, 0u};
		if(GATED) wb[s] = u32x4{0u, 0u, 0u, 0u};
		if(active) {
			wa[s] = *reinterpret_cast<const u32x4*>(wt + (col0 + n) * K + 16 * s + 8 * half);
			if(GATED) wb[s] = *reinterpret_cast<const u32x4*>(wt + (N + col0 + n) * K + 16 * s + 8 * half);
		}
	}

	const int64_t n_blocks = (M + 31) / 32;
	auto rows_in = [&](int64_t blk) -> int { return (int)(M - blk * 32 < 32 ? M - blk * 32 : 32); };
	// x block mover: thread t moves bytes [TPB*t, TPB*t + TPB) of the block, in pieces of at most 16 bytes.  In LDS the 16-byte
	// chunk index of a row is XOR-swizzled with the row so that the operand reads below (same chunk, consecutive rows) spread
	// over the banks.
	typedef typename std::conditional<PIECE == 16, u32x4, typename std::conditional<PIECE == 8, u32x2, uint32_t>::type>::type piece_t;
	struct staged_t {
		piece_t v[PPT];
	};
	auto lds_pos = [&](int off) -> int {
		const int r = off / ROW_BYTES, c = off % ROW_BYTES;
		return r * ROW_BYTES + (((c >> 4) ^ (r & 7)) << 4) + (c & 15);
	};
	auto fetch = [&](int64_t blk) -> staged_t {
		const __amdgpu_buffer_rsrc_t r =
			__builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(reinterpret_cast<const unsigned char*>(x)) + blk * TILE_BYTES, 0, rows_in(blk) * ROW_BYTES, 0x00020000);
		staged_t st;
#pragma unroll
		for(int i = 0; i < PPT; i++) {
			const int off = tid * TPB + i * PIECE;
			if constexpr(PIECE == 16) st.v[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0));
			else if constexpr(PIECE == 8) st.v[i] = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0));
			else st.v[i] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 0);
		}
		return st;
	};
	auto publish = [&](int buf, const staged_t& st) {
#pragma unroll
		for(int i = 0; i < PPT; i++) *reinterpret_cast<piece_t*>(xs[buf] + lds_pos(tid * TPB + i * PIECE)) = st.v[i];
	};
	// operand reads (lane = row n, chunk 2s + half, swizzled) and the output patch
	const int            x_rd  = n * ROW_BYTES;
	const int            sw    = n & 7;
	unsigned char* const patch = os[wave];
	const int            p_wr  = n * OUT_STRIDE + half * 8;
	const int            p_rd  = (lane >> 2) * OUT_STRIDE + (lane & 3) * 16;
	const int            o_off = (int)(((lane >> 2) * N + col0 + (lane & 3) * 8) * 2);  // bytes from the block's first row (N < 2^20 checked by the launcher)

	int64_t blk = blockIdx.x;
	if(blk >= n_blocks) return;  // (whole workgroup)
	staged_t staged = fetch(blk);
	publish(0, staged);
	__syncthreads();
	int   buf = 0;
	u32x4 sv[2] = {u32x4{0u, 0u, 0u, 0u}, u32x4{0u, 0u, 0u, 0u}};  // the data of the two stores of a block
	for(; blk < n_blocks; blk += gridDim.x) {
		const int64_t next     = blk + gridDim.x;
		const bool    has_next = next < n_blocks;  // (uniform)
		staged = fetch(has_next ? next : blk);       // in flight during this block's matrix work (the last block is fetched again: no branch)
		const unsigned char* const xb = xs[buf] + x_rd;
		f32x16 ga, va;
#pragma unroll
		for(int i = 0; i < 16; i++) ga[i] = 0.f, va[i] = 0.f;
#pragma unroll
		for(int s = 0; s < KS; s++) {
			const u32x4 xf = *reinterpret_cast<const u32x4*>(xb + (((2 * s + half) ^ sw) << 4));
			ga = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, wa[s]), __builtin_bit_cast(bf16x8, xf), ga, 0, 0, 0);
			if(GATED) va = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, wb[s]), __builtin_bit_cast(bf16x8, xf), va, 0, 0, 0);
		}
		// silu(a) * b, rounded to bf16, into this wavefront's patch: lane (row n, half) owns columns 8*g4 + 4*half .. +3
#pragma unroll
		for(int g4 = 0; g4 < 4; g4++) {
			float o[4];
#pragma unroll
			for(int r = 0; r < 4; r++) {
				const float a = ga[4 * g4 + r];
				o[r] = GATED ? a * va[4 * g4 + r] * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-a * LOG2E)) : a;
			}
			*reinterpret_cast<u32x2*>(patch + p_wr + g4 * 16) = u32x2{pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3])};
		}
		// (the same wavefront writes and reads the patch, and its LDS operations complete in order; the wave barriers
		// only keep the compiler from moving the reads above the writes, or the next block's writes above the reads)
		__builtin_amdgcn_wave_barrier();
		asm volatile("" : "+v"(sv[0]), "+v"(sv[1]));  // sv's registers stay reserved from the previous block's stores up to here
		sv[0] = *reinterpret_cast<const u32x4*>(patch + p_rd);
		sv[1] = *reinterpret_cast<const u32x4*>(patch + p_rd + 16 * OUT_STRIDE);
		__builtin_amdgcn_wave_barrier();
		const __amdgpu_buffer_rsrc_t orsrc = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<unsigned char*>(out) + blk * 32 * N * 2, 0, active ? (int)(rows_in(blk) * N * 2) : 0, 0x00020000);
		typedef __attribute__((ext_vector_type(4))) unsigned int store_t;
		__builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(store_t, sv[0]), orsrc, o_off, 0, 0);
		__builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(store_t, sv[1]), orsrc, o_off + (int)(16 * N * 2), 0, 0);
		// publish the next block (its LDS buffer was last read before the previous barrier)
		publish(buf ^ 1, staged);
		__syncthreads();
		buf ^= 1;
	}
}

}  // namespace

}  // namespace af3

using namespace af3;

namespace {

// out[M, N] = x[M, K] . wt^T (GATED: silu(x . Wa) * (x . Wb), wt = [Wa | Wb]^T) -- checks shared by both entry points
int launch_rows_times_weights(const void* x, const void* weight_t, void* out, int64_t M, int64_t K, int64_t N, int32_t dtype, bool gated, void* stream) {
	if(!x || !weight_t || !out) return AF3_ERR_NULL_POINTER;
	if(M <= 0 || N <= 0 || K <= 0 || M > ((int64_t)1 << 40)) return AF3_ERR_BAD_SHAPE;
	if(dtype != AF3_BF16) return AF3_ERR_BAD_DTYPE;
	if((K != 64 && K != 128) || N % 32 != 0 || N >= (1 << 20)) return AF3_ERR_BAD_ARGUMENT;
	if((reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(weight_t) & 15) || (reinterpret_cast<uintptr_t>(out) & 15)) return AF3_ERR_BAD_ARGUMENT;
	const int64_t col_tiles = N / 32;
	const int64_t n_blocks  = (M + 31) / 32;
	const auto    s  = static_cast<hipStream_t>(stream);
	const auto*   xp = static_cast<const uint16_t*>(x);
	const auto*   wp = static_cast<const uint16_t*>(weight_t);
	auto*         op = static_cast<uint16_t*>(out);
	// persistent workgroups: about sixteen resident wavefronts per compute unit
	auto go = [&](auto kern, int waves) {
		const unsigned gy   = (unsigned)((col_tiles + waves - 1) / waves);
		const int64_t  want = (int64_t)256 * (GLU_MAX_WAVES / waves) / gy > 0 ? (int64_t)256 * (GLU_MAX_WAVES / waves) / gy : 1;
		hipLaunchKernelGGL(kern, dim3((unsigned)(n_blocks < want ? n_blocks : want), gy), dim3(waves * 64), 0, s, xp, wp, op, M, N);
	};
	if(col_tiles <= 4 && !gated) {  // narrow plain products (the attention blocks' output projection): 4-wave workgroups, four per compute unit
		if(K == 128) go(glu_kernel<8, 4, false>, 4);
		else go(glu_kernel<4, 4, false>, 4);
	} else {
		if(K == 128) gated ? go(glu_kernel<8, GLU_MAX_WAVES, true>, GLU_MAX_WAVES) : go(glu_kernel<8, GLU_MAX_WAVES, false>, GLU_MAX_WAVES);
		else gated ? go(glu_kernel<4, GLU_MAX_WAVES, true>, GLU_MAX_WAVES) : go(glu_kernel<4, GLU_MAX_WAVES, false>, GLU_MAX_WAVES);
	}
	return launch_status();
}

}  // namespace

namespace {

// out[m][n] = silu(y[m][n]) * y[m][N + n]: the gate of a gated linear unit whose [M, 2N] product came from a library GEMM
// (the one-kernel form above takes the reference's own shapes; this closes every other shape without an elementwise
// pass of a second framework).  Arithmetic as in src/csrc/gated_linear_unit.cpp:56-61: silu in fp32 on the stored value.
template <bool F32>
__global__ void __launch_bounds__(256) silu_mul_kernel(const void* __restrict__ y, void* __restrict__ out, int64_t M, int64_t N) {
	const int64_t total = M * N, stride = (int64_t)gridDim.x * 256;
	for(int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
		const int64_t m = i / N, n = i - m * N;
		float         a, b;
		if(F32) a = static_cast<const float*>(y)[m * 2 * N + n], b = static_cast<const float*>(y)[m * 2 * N + N + n];
		else a = bf16_bits_to_f32(static_cast<const uint16_t*>(y)[m * 2 * N + n]), b = bf16_bits_to_f32(static_cast<const uint16_t*>(y)[m * 2 * N + N + n]);
		float g = a / (1.f + __expf(-a));
		if(!F32) g = bf16_bits_to_f32(f32_to_bf16_bits(g));   // (the reference rounds silu's result to the storage type before the product)
		const float o = g * b;
		if(F32) static_cast<float*>(out)[i] = o;
		else static_cast<uint16_t*>(out)[i] = (uint16_t)f32_to_bf16_bits(o);
	}
}

}  // namespace

extern "C" int af3_silu_mul(const void* y, void* out, int64_t M, int64_t N, int32_t dtype, void* stream) {
	if(!y || !out) return AF3_ERR_NULL_POINTER;
	if(M <= 0 || N <= 0 || M > ((int64_t)1 << 40) || N > ((int64_t)1 << 30)) return AF3_ERR_BAD_SHAPE;
	if(dtype != AF3_BF16 && dtype != AF3_F32) return AF3_ERR_BAD_DTYPE;
	const int64_t  blocks = (M * N + 255) / 256;
	const unsigned g      = (unsigned)(blocks > 256 * 32 ? 256 * 32 : blocks);
	if(dtype == AF3_F32) hipLaunchKernelGGL(silu_mul_kernel<true>, dim3(g), dim3(256), 0, static_cast<hipStream_t>(stream), y, out, M, N);
	else hipLaunchKernelGGL(silu_mul_kernel<false>, dim3(g), dim3(256), 0, static_cast<hipStream_t>(stream), y, out, M, N);
	return launch_status();
}

extern "C" int af3_gated_linear_unit(const void* x, const void* weight_t, void* out, int64_t M, int64_t K, int64_t N, int32_t dtype, void* stream) {
	return launch_rows_times_weights(x, weight_t, out, M, K, N, dtype, true, stream);
}

extern "C" int af3_linear(const void* x, const void* weight, void* out, int64_t M, int64_t K, int64_t N, int32_t dtype, void* stream) {
	return launch_rows_times_weights(x, weight, out, M, K, N, dtype, false, stream);
}
