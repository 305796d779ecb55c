// bf16 matrix-core attention kernel for gfx950 (CDNA4): out = softmax(q.k^T*scale + bias, mask).v
//
// Work split.  One workgroup = 4 wavefronts = 128 query rows of one (batch, head); each
// wavefront owns 32 query rows and walks the key axis in tiles of 64 keys with an online
// softmax.  K and V tiles are staged once per workgroup in LDS (double buffered); the bias tile
// is not shared between wavefronts, so every lane loads its own 16-byte bias fragments straight
// from global memory (L2-resident: the bias is shared by all batch rows).
//
// Everything is computed "transposed" so that all per-query state is lane-local:
//   S^T[key][q]  = K . Q^T      v_mfma_f32_32x32x16_bf16, A = K tile (LDS), B = Q (registers)
//              += I . bias^T    same instruction with A = 0/1 identity fragment, B = bias
//                               fragment as loaded: bf16 * 1.0 accumulates exactly in fp32, so
//                               the bias add costs no vector-ALU work
//              += m . 1^T       one more MFMA whose A holds the additive key-mask value of each
//                               key in contraction slot 0 and whose B holds 1.0 in slot 0
//   In the 32x32 accumulator layout lane (q = lane%32, half = lane/32) holds 16 keys of one
//   query row, so row max / exp / row sum are in-lane loops plus one half-wave swap.
//   O^T[d][q]   += V^T . P^T    A = V^T fragment read with ds_read_b64_tr_b16 from the row-major
//                               V tile, B = P^T = the accumulator registers converted to bf16
//                               in place (the accumulator layout IS the B-operand layout).
// The pack of operands into MFMA layout therefore happens in the load path (global -> LDS ->
// register), which is this design's counterpart of the reference's VNNI repack
// (src/csrc/tools.cpp:151-176).
//
// Reference semantics followed: src/csrc/dot_product_attention.cpp:88-122 (what is computed) and
// :148-191 (the running max / sum recurrence); the harness formula
// examples/dot_product_attention.py:20-43 for masking (dropped keys get weight 0, an all-dropped
// row yields the mean of V).
#include "common.hpp"

namespace af3 {

constexpr int QT_WAVES = 4;              // wavefronts per workgroup
constexpr int QT       = QT_WAVES * 32;  // query rows per workgroup
constexpr int KT       = 64;             // keys per tile
constexpr int MAX_L_MFMA = 16384;        // mask table (2 B/key) and tile list live in LDS

// ---- LDS layout -----------------------------------------------------------------------------
// K tile: [KT rows][DP cols] bf16, 16-byte chunks XOR-swizzled so that the 8 lanes served in one
// LDS cycle of a ds_read_b128 (8 consecutive rows, same logical chunk) hit distinct banks.
template <int DP>
__device__ __forceinline__ int k_lds_offset(int row, int chunk) {  // in bf16 elements
	constexpr int CPR = DP / 8;
	const int     sw  = (CPR == 4) ? ((row >> 1) & 3) : (row & 7);
	return row * DP + ((chunk ^ sw) << 3);
}
// V tile: [KT rows][DP cols] bf16 row-major.  For DP = 64 the two 64-byte halves of a row are
// swapped on odd rows (keeps the transposed reads of 8 rows x 64 B spread over all banks).
template <int DP>
__device__ __forceinline__ int v_lds_offset(int row, int col) {
	if(DP == 64) return row * DP + (col ^ ((row & 1) << 5));
	return row * DP + col;
}

template <int DP>
struct SmemLayout {
	static constexpr int TILE_ELEMS = KT * DP;
	uint16_t k[2][TILE_ELEMS];
	uint16_t v[2][TILE_ELEMS];
};

// Load 8 consecutive bias values bias[row][key .. key+7] as 4 dwords (MFMA B fragment).
// Elements at key >= L read as zero.  `vec_ok` = the row base and key are 16-byte aligned.
template <bool BIAS_F32>
__device__ __forceinline__ u32x4 load_bias8(const void* bias_row, int64_t key, int64_t L, bool row_ok, bool vec_ok) {
	u32x4 r = {0u, 0u, 0u, 0u};
	if(!row_ok || key >= L) return r;
	if(BIAS_F32) {
		const float* b = static_cast<const float*>(bias_row) + key;
		float f[8];
#pragma unroll
		for(int j = 0; j < 8; j++) f[j] = (key + j < L) ? b[j] : 0.f;
#pragma unroll
		for(int j = 0; j < 4; j++) r[j] = pack_bf16x2(f[2 * j], f[2 * j + 1]);
		return r;
	}
	const uint16_t* b = static_cast<const uint16_t*>(bias_row) + key;
	if(vec_ok && key + 8 <= L) return *reinterpret_cast<const u32x4*>(b);
#pragma unroll
	for(int j = 0; j < 8; j++) {
		const uint32_t e = (key + j < L) ? (uint32_t)b[j] : 0u;
		r[j >> 1] |= e << ((j & 1) * 16);
	}
	return r;
}

__device__ __forceinline__ float half_swap_max(float x) {
	// lanes l and l^32 exchange; v_permlane32_swap swaps the upper half of one operand with the
	// lower half of the other, so (x, x) yields {low|low} and {high|high}.
	auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
	return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_swap_sum(float x) {
	auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
	return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// DP: head_dim padded to a multiple of 32 (32 or 64).  BIAS_F32: bias stored as fp32.
template <int DP, bool BIAS_F32>
__global__ void __launch_bounds__(QT_WAVES * 64, 2) dpa_mfma_bf16_kernel(af3_dpa_params p, int n_qtiles, int64_t n_groups) {
	constexpr int NC  = DP / 16;  // contraction chunks of QK^T
	constexpr int NDB = DP / 32;  // 32-row blocks of O^T
	constexpr int CPR = DP / 8;   // 16-byte chunks per K/V row
	constexpr int LOADS = KT * CPR / (QT_WAVES * 64);  // 16-byte chunks per thread per tile (1 or 2)

	extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
	SmemLayout<DP>& sm      = *reinterpret_cast<SmemLayout<DP>*>(smem_raw);
	uint16_t* mask_tab      = reinterpret_cast<uint16_t*>(smem_raw + sizeof(SmemLayout<DP>));  // [n_ktiles*KT]
	const int n_ktiles      = (int)((p.L + KT - 1) / KT);
	int16_t*  live_list     = reinterpret_cast<int16_t*>(mask_tab + n_ktiles * KT);            // [n_ktiles]
	__shared__ int s_nvalid;

	// ---- workgroup -> (batch, head, query tile).  Workgroups are handed to the 8 XCDs round
	// robin, so all query tiles of one (batch, head) are given ids that are congruent mod 8:
	// they share that XCD's L2 copy of K and V, and an XCD only ever sees heads h = xcd % H
	// (for H | 8), so its share of the bias stays L2-resident across the whole batch.
	const int64_t wg    = blockIdx.x;
	const int     xcd   = (int)(wg & 7);
	const int64_t slot  = wg >> 3;
	const int64_t group = (slot / n_qtiles) * 8 + xcd;
	const int     qtile = (int)(slot % n_qtiles);
	if(group >= n_groups) return;
	const int64_t b = group / p.H, h = group % p.H;

	const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
	const int n = lane & 31, half = lane >> 5;
	const int64_t L = p.L;
	const int     D = (int)p.D;

	// ---- key-mask table (bf16 additive values) and list of tiles with at least one live key ----
	if(tid == 0) s_nvalid = 0;
	__syncthreads();
	const uint8_t* keep = p.key_mask ? p.key_mask + b * p.key_mask_stride_b : nullptr;
	for(int kt = wave; kt < n_ktiles; kt += QT_WAVES) {
		const int64_t key  = (int64_t)kt * KT + lane;
		const bool    in   = key < L;
		const bool    live = in && (keep ? keep[key] != 0 : true);
		mask_tab[kt * KT + lane] = live ? (uint16_t)0 : (in ? MASK_DROPPED_BF16 : MASK_OUT_OF_RANGE_BF16);
		const unsigned long long bal = __ballot(live);
		if(lane == 0) {
			live_list[kt] = bal ? 1 : 0;
			if(bal) atomicAdd(&s_nvalid, 1);
		}
	}
	__syncthreads();
	// Compact the flags into a list (serial; at most a few hundred tiles).  If no key of this
	// batch row is live every tile is kept: the result is then the mean over all L keys.
	__shared__ int s_nlive;
	if(tid == 0) {
		const bool all = (s_nvalid == 0);
		int cnt = 0;
		for(int kt = 0; kt < n_ktiles; kt++)
			if(all || live_list[kt]) live_list[cnt++] = (int16_t)kt;
		s_nlive = cnt;
	}
	__syncthreads();
	const int nlive = s_nlive;

	// ---- per-lane constants ----
	const int64_t qrow   = (int64_t)qtile * QT + wave * 32 + n;
	const bool    row_ok = qrow < L;

	// Q fragments (B operand of S^T = K.Q^T): lane (q = n, g = half) holds q[q][16c + 8g .. +7]
	// scaled by softmax_scale and rounded to bf16 (the reference also rounds the scaled q,
	// src/csrc/dot_product_attention.cpp:95-98).
	bf16x8 qf[NC];
	{
		const uint16_t* qp = static_cast<const uint16_t*>(p.q) + b * p.q_stride[0] + h * p.q_stride[1] + qrow * p.q_stride[2];
#pragma unroll
		for(int c = 0; c < NC; c++) {
			const int d0 = 16 * c + 8 * half;
			u32x4     raw = {0u, 0u, 0u, 0u};
			if(row_ok && d0 < D) raw = *reinterpret_cast<const u32x4*>(qp + d0);
			u32x4 sc;
#pragma unroll
			for(int j = 0; j < 4; j++) {
				const float lo = bf16_bits_to_f32(raw[j] & 0xffffu) * p.softmax_scale;
				const float hi = bf16_bits_to_f32(raw[j] >> 16) * p.softmax_scale;
				sc[j] = pack_bf16x2(lo, hi);
			}
			qf[c] = __builtin_bit_cast(bf16x8, sc);
		}
	}
	// Identity fragments (A operand of the bias MFMA): lane (m = n, g = half), slot j of chunk c2
	// is 1.0 iff m == 16*c2 + 8*g + j.
	bf16x8 idf[2];
#pragma unroll
	for(int c2 = 0; c2 < 2; c2++) {
		u32x4     v = {0u, 0u, 0u, 0u};
		const int j = n - 16 * c2 - 8 * half;
		if(j >= 0 && j < 8) v[j >> 1] = 0x3F80u << ((j & 1) * 16);
		idf[c2] = __builtin_bit_cast(bf16x8, v);
	}
	// B operand of the mask MFMA: 1.0 in contraction slot 0.
	bf16x8 onef;
	{
		u32x4 v = {0u, 0u, 0u, 0u};
		if(half == 0) v[0] = 0x3F80u;
		onef = __builtin_bit_cast(bf16x8, v);
	}

	const unsigned char* bias_row = nullptr;
	bool                 bias_vec = false;
	if(p.bias) {
		const int64_t esz = BIAS_F32 ? 4 : 2;
		bias_row = static_cast<const unsigned char*>(p.bias) + (h * p.bias_stride[0] + (row_ok ? qrow : 0) * p.bias_stride[1]) * esz;
		bias_vec = ((reinterpret_cast<uintptr_t>(p.bias) & 15) == 0) && (p.bias_stride[0] % 8 == 0) && (p.bias_stride[1] % 8 == 0);
	}
	const bool has_bias = p.bias != nullptr;

	// ---- K/V tile loader: thread -> (row, chunk) of the tile ----
	const uint16_t* kbase = static_cast<const uint16_t*>(p.k) + b * p.k_stride[0] + h * p.k_stride[1];
	const uint16_t* vbase = static_cast<const uint16_t*>(p.v) + b * p.v_stride[0] + h * p.v_stride[1];
	u32x4 kreg[LOADS], vreg[LOADS];
	auto  load_tile = [&](int kt) {
#pragma unroll
		for(int i = 0; i < LOADS; i++) {
			const int     id  = tid + i * QT_WAVES * 64;
			const int     row = id / CPR, ch = id % CPR;
			const int64_t key = (int64_t)kt * KT + row;
			const bool    ok  = key < L && ch * 8 < D;
			u32x4         z   = {0u, 0u, 0u, 0u};
			kreg[i] = ok ? *reinterpret_cast<const u32x4*>(kbase + key * p.k_stride[2] + ch * 8) : z;
			vreg[i] = ok ? *reinterpret_cast<const u32x4*>(vbase + key * p.v_stride[2] + ch * 8) : z;
		}
	};
	auto store_tile = [&](int buf) {
#pragma unroll
		for(int i = 0; i < LOADS; i++) {
			const int id  = tid + i * QT_WAVES * 64;
			const int row = id / CPR, ch = id % CPR;
			*reinterpret_cast<u32x4*>(&sm.k[buf][k_lds_offset<DP>(row, ch)]) = kreg[i];
			*reinterpret_cast<u32x4*>(&sm.v[buf][v_lds_offset<DP>(row, ch * 8)]) = vreg[i];
		}
	};
	// bias fragments of one 64-key tile: [sub-tile][c2]
	u32x4 bnext[2][2];
	auto  load_bias_tile = [&](int kt) {
#pragma unroll
		for(int sub = 0; sub < 2; sub++)
#pragma unroll
			for(int c2 = 0; c2 < 2; c2++) {
				const int64_t key = (int64_t)kt * KT + 32 * sub + 16 * c2 + 8 * half;
				bnext[sub][c2] = load_bias8<BIAS_F32>(bias_row, key, L, row_ok && has_bias, bias_vec);
			}
	};

	// ---- online-softmax state (per lane: one query row; the two halves hold disjoint keys) ----
	const float c_log2 = LOG2E;  // logits are in natural units; exp(x) = exp2(x * log2 e)
	float       m_run  = -INFINITY;
	float       l_run  = 0.f;
	f32x16      oacc[NDB];
#pragma unroll
	for(int db = 0; db < NDB; db++)
#pragma unroll
		for(int i = 0; i < 16; i++) oacc[db][i] = 0.f;

	// prologue: first tile
	load_tile(live_list[0]);
	load_bias_tile(live_list[0]);
	store_tile(0);
	__syncthreads();

	for(int it = 0; it < nlive; it++) {
		const int  kt       = live_list[it];
		const int  buf      = it & 1;
		const bool has_next = it + 1 < nlive;
		u32x4      bcur[2][2];
#pragma unroll
		for(int sub = 0; sub < 2; sub++)
#pragma unroll
			for(int c2 = 0; c2 < 2; c2++) bcur[sub][c2] = bnext[sub][c2];
		if(has_next) {
			const int ktn = live_list[it + 1];
			load_tile(ktn);
			load_bias_tile(ktn);
		}

#pragma unroll
		for(int sub = 0; sub < 2; sub++) {
			// ---- S^T = K.Q^T + bias + mask for 32 keys x 32 queries ----
			f32x16 s;
#pragma unroll
			for(int i = 0; i < 16; i++) s[i] = 0.f;
#pragma unroll
			for(int c = 0; c < NC; c++) {
				const u32x4 kf = *reinterpret_cast<const u32x4*>(&sm.k[buf][k_lds_offset<DP>(32 * sub + n, 2 * c + half)]);
				s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kf), qf[c], s, 0, 0, 0);
			}
#pragma unroll
			for(int c2 = 0; c2 < 2; c2++)
				s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(idf[c2], __builtin_bit_cast(bf16x8, bcur[sub][c2]), s, 0, 0, 0);
			{
				u32x4 mv = {0u, 0u, 0u, 0u};
				const uint32_t mval = mask_tab[kt * KT + 32 * sub + n];
				mv[0] = half == 0 ? mval : 0u;
				s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, mv), onef, s, 0, 0, 0);
			}
			// ---- online softmax: accumulator register i of lane (q, half) is key 8*(i/4) + 4*half + i%4 ----
			float mx = s[0];
#pragma unroll
			for(int i = 1; i < 16; i++) mx = fmaxf(mx, s[i]);
			mx = half_swap_max(mx);
			const float m_new = fmaxf(m_run, mx);
			const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * c_log2);
			const float mc    = m_new * c_log2;
			m_run = m_new;
			float psum = 0.f;
			u32x4 pf[2];
#pragma unroll
			for(int i = 0; i < 16; i += 2) {
				const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i], c_log2, -mc));
				const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i + 1], c_log2, -mc));
				psum += p0 + p1;
				pf[i >> 3][(i & 7) >> 1] = pack_bf16x2(p0, p1);
			}
			l_run = l_run * alpha + psum;
#pragma unroll
			for(int db = 0; db < NDB; db++)
#pragma unroll
				for(int i = 0; i < 16; i++) oacc[db][i] *= alpha;
			// ---- O^T += V^T . P^T ; V^T fragments come from transposing LDS reads ----
#pragma unroll
			for(int cp = 0; cp < 2; cp++) {
#pragma unroll
				for(int db = 0; db < NDB; db++) {
					// lane l: i = l%16, G = l/16 ; supplies the 8-byte chunk at row keybase + i/4,
					// column 32*db + 16*(G%2) + 4*(i%4); receives 4 keys of head column 32*db + l%32.
					const int i16 = lane & 15, G = lane >> 4;
					const int col = 32 * db + 16 * (G & 1) + 4 * (i16 & 3);
					u32x4     vf;
#pragma unroll
					for(int t = 0; t < 2; t++) {
						const int   row = 32 * sub + 16 * cp + 8 * t + 4 * (G >> 1) + (i16 >> 2);
						const s16x4 r   = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
							(__attribute__((address_space(3))) s16x4*)(&sm.v[buf][v_lds_offset<DP>(row, col)]));
						const u32x2 rr = __builtin_bit_cast(u32x2, r);
						vf[2 * t]     = rr[0];
						vf[2 * t + 1] = rr[1];
					}
					oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vf), __builtin_bit_cast(bf16x8, pf[cp]), oacc[db], 0, 0, 0);
				}
			}
		}
		if(has_next) store_tile(buf ^ 1);
		__syncthreads();
	}

	// ---- epilogue: O^T register i of block db is head column 32*db + 8*(i/4) + 4*half + i%4 ----
	const float l_tot = half_swap_sum(l_run);
	const float inv   = 1.f / l_tot;
	if(row_ok) {
		const int64_t ooff = b * p.out_stride[0] + h * p.out_stride[1] + qrow * p.out_stride[2];
#pragma unroll
		for(int db = 0; db < NDB; db++)
#pragma unroll
			for(int g4 = 0; g4 < 4; g4++) {
				const int d0 = 32 * db + 8 * g4 + 4 * half;
				if(d0 >= D) continue;
				const float o0 = oacc[db][4 * g4] * inv, o1 = oacc[db][4 * g4 + 1] * inv;
				const float o2 = oacc[db][4 * g4 + 2] * inv, o3 = oacc[db][4 * g4 + 3] * inv;
				if(p.out_dtype == AF3_BF16) {
					u32x2 w = {pack_bf16x2(o0, o1), pack_bf16x2(o2, o3)};
					*reinterpret_cast<u32x2*>(static_cast<uint16_t*>(p.out) + ooff + d0) = w;
				} else {
					float4 w = {o0, o1, o2, o3};
					*reinterpret_cast<float4*>(static_cast<float*>(p.out) + ooff + d0) = w;
				}
			}
	}
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

bool mfma_bf16_eligible(const af3_dpa_params& p) {
	if(p.io_dtype != AF3_BF16 || p.mma_dtype != AF3_BF16) return false;
	if(p.D > 64 || p.D % 8 != 0 || p.L > MAX_L_MFMA) return false;
	if(!aligned16(p.q) || !aligned16(p.k) || !aligned16(p.v)) return false;
	for(int i = 0; i < 3; i++)
		if(p.q_stride[i] % 8 || p.k_stride[i] % 8 || p.v_stride[i] % 8) return false;
	if(p.out_dtype == AF3_BF16) {
		if((reinterpret_cast<uintptr_t>(p.out) & 7) || p.out_stride[0] % 4 || p.out_stride[1] % 4 || p.out_stride[2] % 4) return false;
	} else {
		if(!aligned16(p.out) || p.out_stride[0] % 4 || p.out_stride[1] % 4 || p.out_stride[2] % 4) return false;
	}
	return true;
}

template <int DP, bool BIAS_F32>
static int launch_one(const af3_dpa_params& p, hipStream_t s) {
	const int     n_qtiles = (int)((p.L + QT - 1) / QT);
	const int     n_ktiles = (int)((p.L + KT - 1) / KT);
	const int64_t n_groups = p.B * p.H;
	const int64_t blocks   = ((n_groups + 7) / 8) * 8 * n_qtiles;
	if(blocks <= 0 || blocks > 0x7fffffffLL) return AF3_ERR_BAD_SHAPE;
	const size_t smem = sizeof(SmemLayout<DP>) + (size_t)n_ktiles * KT * 2 + (size_t)n_ktiles * 2 + 16;
	auto         kern = dpa_mfma_bf16_kernel<DP, BIAS_F32>;
	hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(QT_WAVES * 64), smem, s, p, n_qtiles, n_groups);
	return hipGetLastError() == hipSuccess ? AF3_OK : AF3_ERR_LAUNCH;
}

int launch_dpa_mfma_bf16(const af3_dpa_params& p, hipStream_t s) {
	const bool bf32 = p.bias && p.bias_dtype == AF3_F32;
	if(p.D <= 32) return bf32 ? launch_one<32, true>(p, s) : launch_one<32, false>(p, s);
	return bf32 ? launch_one<64, true>(p, s) : launch_one<64, false>(p, s);
}

// The fp8 kernel is built in its own translation unit.
}  // namespace af3
