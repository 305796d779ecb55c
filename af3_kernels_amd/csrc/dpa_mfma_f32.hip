// fp32 biased attention on the fp32 matrix cores of gfx950 (v_mfma_f32_32x32x2_f32): the full-precision
// path of dot_product_attention_impl<float> (reference src/csrc/dot_product_attention.cpp:25-198,
// dispatch :545-559), for float32 callers who want the 1e-4 tier at more than vector-FMA speed.
//
// Same transposed formulation as the bf16 kernel: S^T[key][q] = K.Q^T, so that in the 32x32
// accumulator layout a lane (q = lane%32, half = lane/32) holds 16 keys of ONE query row
// (register i <-> key 8*(i/4) + 4*half + i%4) and the softmax is an in-lane loop; O^T += V^T.P^T takes
// the probability registers directly as its B operand: step j of the contraction pairs the key of
// register j in each half-wave with the matching V row, so P needs no shuffle and no conversion.
//
// Workgroup = 4 wavefronts x 32 query rows of one (batch, head); keys in 32-key tiles, K and V tiles
// staged in LDS (double buffered: the next tile travels global -> registers during the matrix
// work and is written to the other buffer afterwards; one barrier per tile).  Exact running maximum
// (classic online softmax): with 32 fp32 MFMAs of 64 cycles per 32x32 block the matrix pipe is the
// bound by a wide margin and the vector work hides behind it.
//
// Semantics are the reference harness's (examples/dot_product_attention.py:20-43): a dropped key's
// logit is replaced by -1e9, so its weight is exactly 0 unless every key of the row is dropped, in
// which case the row is the mean of V; keys past L weigh 0.
#include "common.hpp"

namespace af3 {
namespace {

constexpr int F32_KT    = 32;     // keys per tile
constexpr int F32_NW    = 4;      // wavefronts per workgroup
constexpr int F32_MAX_L = 16384;  // key-state bytes and tile list live in LDS

__device__ __forceinline__ float other_half(float x) { return __shfl_xor(x, 32); }

template <int DP>
__global__ void __launch_bounds__(F32_NW * 64) dpa_mfma_f32_kernel(af3_dpa_params p, int n_qtiles, int64_t n_groups) {
	constexpr int NK  = DP / 2;   // QK^T contraction steps (2 head columns per MFMA)
	constexpr int NDB = DP / 32;  // 32-row blocks of O^T
	constexpr int RS  = DP + 4;   // LDS row stride in floats: 16-byte reads of 32 consecutive rows hit distinct banks
	constexpr int CH  = DP / 32;  // 16-byte chunks of a tile each thread moves, per tensor
	constexpr int TILE_FLOATS = F32_KT * RS;

	extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
	float* const   k_lds = reinterpret_cast<float*>(smem_raw);            // [2][32][RS]
	float* const   v_lds = k_lds + 2 * TILE_FLOATS;                       // [2][32][RS]
	const int      n_tiles = (int)((p.L + F32_KT - 1) / F32_KT);
	uint8_t* const state = reinterpret_cast<uint8_t*>(v_lds + 2 * TILE_FLOATS);  // per key: 1 live, 0 dropped, 2 past L
	int16_t* const live_list = reinterpret_cast<int16_t*>(state + n_tiles * F32_KT);
	__shared__ int s_nvalid, s_nlive;

	// workgroup -> (batch row, head, query tile); consecutive workgroups go round the 8 XCDs, so the
	// query tiles of one (b, h) are kept on one XCD and share its L2 copy of K and V
	// the kernel arguments that the start of a workgroup needs, requested in one batch (otherwise: the launch counts, a wait,
	// the early exit, and only then the fields of p -- memory latencies in a row that a small launch cannot hide)
	asm volatile("" ::"s"(n_qtiles), "s"(n_groups), "s"(p.q), "s"(p.k), "s"(p.v), "s"(p.bias), "s"(p.key_mask), "s"(p.H), "s"(p.L), "s"(p.D), "s"(p.key_mask_stride_b),
				 "s"(p.bias_stride[0]), "s"(p.bias_stride[1]));
	asm volatile("" ::"s"(p.q_stride[0]), "s"(p.q_stride[1]), "s"(p.q_stride[2]), "s"(p.k_stride[0]), "s"(p.k_stride[1]), "s"(p.k_stride[2]), "s"(p.v_stride[0]), "s"(p.v_stride[1]),
				 "s"(p.v_stride[2]));
	const int64_t wg    = blockIdx.x;
	const int     xcd   = (int)(wg & 7);
	const int64_t slot  = wg >> 3;
	const int64_t group = (slot / n_qtiles) * 8 + xcd;
	const int     qtile = (int)(slot % n_qtiles);
	if(group >= n_groups) return;
	const int64_t b = group / p.H, h = group % p.H;

	const int     tid = threadIdx.x, lane = tid & 63;
	const int     wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int     n = lane & 31, half = lane >> 5;
	const int64_t L = p.L;
	const int     D = (int)p.D;

	// ---- key states and the list of tiles with at least one live key ----
	if(tid == 0) s_nvalid = 0;
	__syncthreads();
	const uint8_t* keep = p.key_mask ? p.key_mask + b * p.key_mask_stride_b : nullptr;
	for(int kt = wave * 2 + half; kt < n_tiles; kt += 2 * F32_NW) {  // one half-wave per tile
		const int64_t key  = (int64_t)kt * F32_KT + n;
		const bool    in   = key < L;
		const bool    live = in && (keep ? keep[key] != 0 : true);
		state[key] = in ? (live ? 1 : 0) : 2;
		const unsigned long long bal  = __ballot(live);
		const unsigned           mine = half ? (unsigned)(bal >> 32) : (unsigned)bal;
		if(n == 0) {
			live_list[kt] = mine ? 1 : 0;
			if(mine) atomicAdd(&s_nvalid, 1);
		}
	}
	__syncthreads();
	if(wave == 0) {  // compact the flags into tile indices; a batch row without live keys keeps every tile
		const bool all = (s_nvalid == 0);
		int        cnt = 0;
		for(int base = 0; base < n_tiles; base += 64) {
			const int  kt     = base + lane;
			const bool keepit = kt < n_tiles && (all || live_list[kt] != 0);
			const unsigned long long bal = __ballot(keepit);
			const int rank = __builtin_amdgcn_mbcnt_hi((unsigned)(bal >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)bal, 0));
			__builtin_amdgcn_wave_barrier();  // every flag of this pass is read before an index is written (cnt + rank <= kt)
			if(keepit) live_list[cnt + rank] = (int16_t)kt;
			cnt += __builtin_popcountll(bal);
		}
		if(lane == 0) s_nlive = cnt;
	}
	__syncthreads();
	const int nlive = __builtin_amdgcn_readfirstlane(s_nlive);

	// ---- per-lane constants ----
	const int64_t qrow   = (int64_t)qtile * (F32_NW * 32) + wave * 32 + n;
	const bool    row_ok = qrow < L;
	// Q as the B operand: contraction step t pairs head columns t (half 0) and t + NK (half 1)
	float qreg[NK];
	{
		const float* qp = static_cast<const float*>(p.q) + b * p.q_stride[0] + h * p.q_stride[1] + qrow * p.q_stride[2] + half * NK;
#pragma unroll
		for(int t4 = 0; t4 < NK / 4; t4++) {
			float4 w = {0.f, 0.f, 0.f, 0.f};
			if(row_ok && half * NK + 4 * t4 < D) w = *reinterpret_cast<const float4*>(qp + 4 * t4);  // D % 4 == 0: a chunk is all in or all out
			qreg[4 * t4] = w.x * p.softmax_scale, qreg[4 * t4 + 1] = w.y * p.softmax_scale, qreg[4 * t4 + 2] = w.z * p.softmax_scale, qreg[4 * t4 + 3] = w.w * p.softmax_scale;
		}
	}
	const float* bias_row = p.bias ? static_cast<const float*>(p.bias) + h * p.bias_stride[0] + (row_ok ? qrow : 0) * p.bias_stride[1] : nullptr;

	// ---- tile mover: thread -> CH 16-byte chunks of the K tile and of the V tile ----
	const float* kbase = static_cast<const float*>(p.k) + b * p.k_stride[0] + h * p.k_stride[1];
	const float* vbase = static_cast<const float*>(p.v) + b * p.v_stride[0] + h * p.v_stride[1];
	float4       kstage[CH], vstage[CH];
	auto fetch_tile = [&](int kt) {
#pragma unroll
		for(int u = 0; u < CH; u++) {
			const int     c   = tid + 256 * u, row = c / (DP / 4), col = (c % (DP / 4)) * 4;
			const int64_t key = (int64_t)kt * F32_KT + row;
			const bool    ok  = key < L && col < D;
			kstage[u] = ok ? *reinterpret_cast<const float4*>(kbase + key * p.k_stride[2] + col) : float4{0.f, 0.f, 0.f, 0.f};
			vstage[u] = ok ? *reinterpret_cast<const float4*>(vbase + key * p.v_stride[2] + col) : float4{0.f, 0.f, 0.f, 0.f};
		}
	};
	auto store_tile = [&](int buf) {
#pragma unroll
		for(int u = 0; u < CH; u++) {
			const int c = tid + 256 * u, row = c / (DP / 4), col = (c % (DP / 4)) * 4;
			*reinterpret_cast<float4*>(k_lds + buf * TILE_FLOATS + row * RS + col) = kstage[u];
			*reinterpret_cast<float4*>(v_lds + buf * TILE_FLOATS + row * RS + col) = vstage[u];
		}
	};
	// bias of one tile in accumulator order: register i <-> key 8*(i/4) + 4*half + i%4 of this lane's query row
	const bool bias_vec = p.bias && ((reinterpret_cast<uintptr_t>(p.bias) & 15) == 0) && (p.bias_stride[0] % 4 == 0) && (p.bias_stride[1] % 4 == 0);
	auto fetch_bias = [&](int kt, float (&dst)[16]) {
#pragma unroll
		for(int r4 = 0; r4 < 4; r4++) {
			const int64_t key = (int64_t)kt * F32_KT + 8 * r4 + 4 * half;
			if(bias_row && row_ok && bias_vec && key + 3 < L) {
				const float4 w = *reinterpret_cast<const float4*>(bias_row + key);
				dst[4 * r4] = w.x, dst[4 * r4 + 1] = w.y, dst[4 * r4 + 2] = w.z, dst[4 * r4 + 3] = w.w;
			} else {
#pragma unroll
				for(int e = 0; e < 4; e++) dst[4 * r4 + e] = (bias_row && row_ok && key + e < L) ? bias_row[key + e] : 0.f;
			}
		}
	};

	// ---- online-softmax state ----
	float  m_run = -INFINITY, l_run = 0.f;  // natural units; l_run: this lane's half of the row sum
	f32x16 oacc[NDB];
#pragma unroll
	for(int db = 0; db < NDB; db++)
#pragma unroll
		for(int i = 0; i < 16; i++) oacc[db][i] = 0.f;

	float bcur[16], bnext[16];
	fetch_tile(live_list[0]);
	fetch_bias(live_list[0], bcur);
	store_tile(0);
	__syncthreads();

	for(int j = 0; j < nlive; j++) {
		const int  kt   = __builtin_amdgcn_readfirstlane((int)live_list[j]);
		const int  buf  = j & 1;
		const bool more = j + 1 < nlive;
		if(more) {
			const int ktn = __builtin_amdgcn_readfirstlane((int)live_list[j + 1]);
			fetch_tile(ktn);  // in flight during the matrix work below
			fetch_bias(ktn, bnext);
		}
		// S^T = K.Q^T: lane (key = n, half) supplies K[key][t + NK*half]
		f32x16       s;
		const float* krow = k_lds + buf * TILE_FLOATS + n * RS + half * NK;
#pragma unroll
		for(int i = 0; i < 16; i++) s[i] = 0.f;
#pragma unroll
		for(int t4 = 0; t4 < NK / 4; t4++) {
			const float4 w = *reinterpret_cast<const float4*>(krow + 4 * t4);
			s = __builtin_amdgcn_mfma_f32_32x32x2f32(w.x, qreg[4 * t4], s, 0, 0, 0);
			s = __builtin_amdgcn_mfma_f32_32x32x2f32(w.y, qreg[4 * t4 + 1], s, 0, 0, 0);
			s = __builtin_amdgcn_mfma_f32_32x32x2f32(w.z, qreg[4 * t4 + 2], s, 0, 0, 0);
			s = __builtin_amdgcn_mfma_f32_32x32x2f32(w.w, qreg[4 * t4 + 3], s, 0, 0, 0);
		}
		// The bias joins the finished products in one rounding, as an addition of two fp32 tensors would: products accumulated on
		// top of a bias of magnitude 10^3..10^4 (a row offset, a soft mask value) would be rounded at that magnitude D/2 times.
#pragma unroll
		for(int i = 0; i < 16; i++) s[i] += bcur[i];
		// key states of this lane's 16 keys: dropped -> -1e9 (as masked_fill does), past L -> -inf
		float mx = -INFINITY;
#pragma unroll
		for(int r4 = 0; r4 < 4; r4++) {
			const uint32_t st = *reinterpret_cast<const uint32_t*>(state + kt * F32_KT + 8 * r4 + 4 * half);
#pragma unroll
			for(int e = 0; e < 4; e++) {
				const uint32_t v = (st >> (8 * e)) & 0xffu;
				// (a live key whose bias is -inf keeps a finite logit, so that a tile of such keys leaves a finite maximum)
				const float    x = v == 1u ? fmaxf(s[4 * r4 + e], -3.0e38f) : (v == 0u ? -1.0e9f : -INFINITY);
				s[4 * r4 + e]    = x;
				mx               = fmaxf(mx, x);
			}
		}
		mx = fmaxf(mx, other_half(mx));
		const float m_new = fmaxf(m_run, mx);  // finite: every tile has a key below L, and a dropped key counts as -1e9
		const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * LOG2E);
		m_run = m_new;
		float psum = 0.f;
#pragma unroll
		for(int i = 0; i < 16; i++) {
			s[i] = __builtin_amdgcn_exp2f((s[i] - m_new) * LOG2E);  // (subtract first: the row maximum gets exactly 1)
			psum += s[i];
		}
		l_run = l_run * alpha + psum;
#pragma unroll
		for(int db = 0; db < NDB; db++)
#pragma unroll
			for(int i = 0; i < 16; i++) oacc[db][i] *= alpha;
		// O^T += V^T.P^T: step i pairs the key of register i in each half-wave: lane (d = n, half) supplies V[key_i(half)][d]
		const float* vcol = v_lds + buf * TILE_FLOATS + n;
#pragma unroll
		for(int i = 0; i < 16; i++) {
			const int key = 8 * (i / 4) + 4 * half + (i % 4);
#pragma unroll
			for(int db = 0; db < NDB; db++) oacc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(vcol[key * RS + 32 * db], s[i], oacc[db], 0, 0, 0);
		}
		if(more) {
			store_tile(buf ^ 1);  // that buffer was last read one iteration ago, before the barrier every wavefront has passed
#pragma unroll
			for(int i = 0; i < 16; i++) bcur[i] = bnext[i];
		}
		__syncthreads();
	}

	// ---- epilogue: O^T register i of block db is head column 32*db + 8*(i/4) + 4*half + i%4 ----
	const float l_tot = l_run + other_half(l_run);
	const float inv   = 1.f / l_tot;
	if(row_ok) {
		float* op = static_cast<float*>(p.out) + b * p.out_stride[0] + h * p.out_stride[1] + qrow * p.out_stride[2];
#pragma unroll
		for(int db = 0; db < NDB; db++)
#pragma unroll
			for(int r4 = 0; r4 < 4; r4++) {
				const int d0 = 32 * db + 8 * r4 + 4 * half;
				if(d0 < D) {
					float4 w = {oacc[db][4 * r4] * inv, oacc[db][4 * r4 + 1] * inv, oacc[db][4 * r4 + 2] * inv, oacc[db][4 * r4 + 3] * inv};
					if(p.gate) {  // out *= sigmoid(gate)
						const float4 g = *reinterpret_cast<const float4*>(static_cast<const float*>(p.gate) + b * p.gate_stride[0] + h * p.gate_stride[1] + qrow * p.gate_stride[2] + d0);
						w.x *= sigmoidf_fast(g.x), w.y *= sigmoidf_fast(g.y), w.z *= sigmoidf_fast(g.z), w.w *= sigmoidf_fast(g.w);
					}
					*reinterpret_cast<float4*>(op + d0) = w;
				}
			}
	}
}

template <int DP>
int launch(const af3_dpa_params& p, hipStream_t s) {
	const int     n_qtiles = (int)((p.L + F32_NW * 32 - 1) / (F32_NW * 32));
	const int     n_tiles  = (int)((p.L + F32_KT - 1) / F32_KT);
	const int64_t groups   = p.B * p.H;
	const int64_t grid     = ((groups + 7) / 8) * 8 * n_qtiles;
	if(grid > 0x7fffffff) return AF3_ERR_BAD_SHAPE;
	const size_t smem = (size_t)4 * F32_KT * (DP + 4) * 4 + (size_t)n_tiles * F32_KT + (size_t)n_tiles * 2 + 16;
	hipLaunchKernelGGL(dpa_mfma_f32_kernel<DP>, dim3((unsigned)grid), dim3(F32_NW * 64), smem, s, p, n_qtiles, groups);
	return launch_status();
}

}  // namespace

// fp32 tensors with 16-byte aligned rows and a head_dim the 32x32 tiles cover; everything else stays on
// the vector-FMA kernel.
bool mfma_f32_eligible(const af3_dpa_params& p) {
	if(p.io_dtype != AF3_F32 || p.mma_dtype != AF3_F32 || p.out_dtype != AF3_F32) return false;
	if(p.bias && p.bias_dtype != AF3_F32) return false;
	if(p.D > 64 || p.D % 4 != 0 || p.L > F32_MAX_L) return false;
	if(p.gate && ((reinterpret_cast<uintptr_t>(p.gate) & 15) || p.gate_stride[0] % 4 || p.gate_stride[1] % 4 || p.gate_stride[2] % 4)) return false;
	const void* ptrs[4] = {p.q, p.k, p.v, p.out};
	for(const void* ptr : ptrs)
		if(reinterpret_cast<uintptr_t>(ptr) & 15) return false;
	for(int i = 0; i < 3; i++)
		if(p.q_stride[i] % 4 || p.k_stride[i] % 4 || p.v_stride[i] % 4 || p.out_stride[i] % 4) return false;
	return true;
}

int launch_dpa_mfma_f32(const af3_dpa_params& p, hipStream_t s) { return p.D <= 32 ? launch<32>(p, s) : launch<64>(p, s); }

}  // namespace af3
