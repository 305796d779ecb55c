// fp8 (OCP e4m3) matrix-core attention kernel for gfx950: both products on
// v_mfma_f32_32x32x16_fp8_fp8 with fp32 accumulation, bf16 bias, bf16 or fp32 output.
//
// The reference has no fp8 path (its e4m3 converters are "not implemented" asserts,
// src/csrc/xsmm_functors.h:218-226); this kernel computes the same formula as
// src/csrc/dot_product_attention.cpp:88-122 on inputs quantised per tensor by
// af3_quantize_fp8_e4m3:
//     q8 = e4m3(q * softmax_scale * sq),  k8 = e4m3(k * sk),  v8t = e4m3(v * sv) transposed to [B,H,D,L]
// with power-of-two scales, so that with alpha = 1/(sq*sk)
//     logits = alpha * (q8 . k8^T) + bias            (natural units)
// Layout is the "transposed" one of the bf16 kernel (dpa_mfma.hip): S^T = K8 . Q8^T with lane
// (q = lane%32, half = lane/32) holding 16 keys of one query row; the bias rides an identity MFMA
// whose diagonal is 1/alpha (a power of two, exact in bf16), the key mask a third MFMA;
// P^T = exp(logit - m) * 2^8 is quantised to e4m3 in registers (values in (0, 256], e4m3 tops out at
// 448) and is the B operand of O^T += V8^T . P^T.  The row maximum m is the true running maximum
// (no slack: P must stay below the e4m3 range), the row sum is taken over the quantised P, on the matrix pipe.
// V arrives transposed, so V^T fragments are plain 4-byte LDS reads (no transposing loads exist for
// 8-bit data paired with this accumulator layout).
#include "common.hpp"

namespace af3 {

namespace {

constexpr int KT8   = 64;    // keys per tile
constexpr int NW8   = 4;     // wavefronts per workgroup (32 query rows each)
constexpr int MAX_L8 = 8192;
constexpr float P_SHIFT = 8.f;  // P is stored as p * 2^8

typedef __attribute__((ext_vector_type(2))) uint32_t u32v2;

__device__ __forceinline__ float hswap_max(float x) {
	auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
	return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// DP: head_dim padded to 32 or 64 (bytes per K row in LDS, rows of the V^T tile).
// COMP: compensated logits q8.k8 + q8.k_lo + q_lo.k8 (the residual tensors recover the e4m3 rounding of q and k).
template <int DP, bool COMP>
__global__ void __launch_bounds__(NW8 * 64) __attribute__((amdgpu_waves_per_eu(2))) dpa_mfma_fp8_kernel(af3_dpa_params p, int n_qtiles, int64_t n_groups) {
	constexpr int NC       = DP / 16;       // contraction chunks of QK^T
	constexpr int NDB      = DP / 32;       // 32-row blocks of O^T
	constexpr int K_TILE1  = KT8 * DP;      // bytes of one K tile
	constexpr int K_TILE   = K_TILE1 * (COMP ? 2 : 1);  // hi tile followed by the residual tile
	constexpr int V_TILE   = DP * KT8;      // bytes: [DP rows d][64 keys]
	constexpr int K_LOADS  = K_TILE1 / 1024; // 1 KB wave loads per K tile (2 or 4)
	constexpr int V_LOADS  = V_TILE / 1024;

	extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
	unsigned char* const k_lds     = smem;                  // [2][K_TILE]
	unsigned char* const v_lds     = smem + 2 * K_TILE;     // [2][V_TILE]
	uint32_t* const      mask_tab  = reinterpret_cast<uint32_t*>(smem + 2 * K_TILE + 2 * V_TILE);
	const int            n_ktiles  = (int)((p.L + KT8 - 1) / KT8);
	int16_t* const       live_list = reinterpret_cast<int16_t*>(mask_tab + n_ktiles * KT8 + 64);
	__shared__ int       s_nvalid, s_nlive;

	// workgroup -> (batch, head, query tile), all query tiles of one (batch, head) on one XCD
	// the kernel arguments that the start of a workgroup needs, requested in one batch (otherwise: the launch counts, a wait,
	// the early exit, and only then the fields of p -- memory latencies in a row that a small launch cannot hide)
	asm volatile("" ::"s"(n_qtiles), "s"(n_groups), "s"(p.q), "s"(p.k), "s"(p.v), "s"(p.bias), "s"(p.key_mask), "s"(p.H), "s"(p.L), "s"(p.D), "s"(p.key_mask_stride_b),
				 "s"(p.bias_stride[0]), "s"(p.bias_stride[1]), "s"(p.device_descales), "s"(p.k_lo));
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

	// zero both tile buffers (padded head columns and rows past L are never written; e4m3 zero is 0x00)
	for(int i = tid; i < (2 * K_TILE + 2 * V_TILE) / 16; i += NW8 * 64) reinterpret_cast<u32x4*>(smem)[i] = u32x4{0u, 0u, 0u, 0u};
	if(tid == 0) s_nvalid = 0;
	if(tid < 64) mask_tab[n_ktiles * KT8 + tid] = 0u;
	__syncthreads();
	const uint8_t* keep = p.key_mask ? p.key_mask + b * p.key_mask_stride_b : nullptr;
	for(int kt = wave; kt < n_ktiles; kt += NW8) {
		const int64_t key  = (int64_t)kt * KT8 + lane;
		const bool    in   = key < L;
		const bool    live = in && (keep ? keep[key] != 0 : true);
		mask_tab[kt * KT8 + lane] = live ? 0u : (in ? (uint32_t)MASK_DROPPED_BF16 : (uint32_t)MASK_OUT_OF_RANGE_BF16);
		const unsigned long long bal = __ballot(live);
		if(lane == 0) {
			live_list[kt] = bal ? 1 : 0;
			if(bal) atomicAdd(&s_nvalid, 1);
		}
	}
	__syncthreads();
	if(wave == 0) {
		const bool all = (s_nvalid == 0);
		int        cnt = 0;
		for(int base = 0; base < n_ktiles; base += 64) {
			const int  kt     = base + lane;
			const bool keepit = kt < n_ktiles && (all || live_list[kt] != 0);
			const unsigned long long bal = __ballot(keepit);
			const int rank = __builtin_amdgcn_mbcnt_hi((unsigned)(bal >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)bal, 0));
			__builtin_amdgcn_wave_barrier();
			if(keepit) live_list[cnt + rank] = (int16_t)kt;
			cnt += __builtin_popcountll(bal);
		}
		if(lane == 0) s_nlive = cnt;
	}
	__syncthreads();
	const int  nlive       = __builtin_amdgcn_readfirstlane(s_nlive);
	const bool all_dropped = __builtin_amdgcn_readfirstlane(s_nvalid) == 0;

	// scales: real = stored * descale
	float dq = p.q_descale, dk = p.k_descale, dv = p.v_descale;
	if(p.device_descales) dq = p.device_descales[0], dk = p.device_descales[1], dv = p.device_descales[2];
	const float alpha = dq * dk * p.softmax_scale;  // logits = alpha * (q8 . k8) + bias
	const float c_exp = alpha * LOG2E;              // exp(logit - m) = exp2(acc*c_exp - m_acc*c_exp), m_acc in accumulator units

	const int64_t qrow   = (int64_t)qtile * (NW8 * 32) + wave * 32 + n;
	const bool    row_ok = qrow < L;

	// Q fragments: lane (q, g = half) holds q8[q][16c + 8g .. +7] (8 bytes)
	long qf[NC];
	{
		const uint8_t* qp = static_cast<const uint8_t*>(p.q) + b * p.q_stride[0] + h * p.q_stride[1] + qrow * p.q_stride[2];
#pragma unroll
		for(int c = 0; c < NC; c++) {
			const int d0 = 16 * c + 8 * half;
			u32v2     w  = {0u, 0u};
			if(row_ok && d0 < D && !all_dropped) w = *reinterpret_cast<const u32v2*>(qp + d0);
			qf[c] = __builtin_bit_cast(long, w);
		}
	}
	long qlo[NC];
	if(COMP) {
		const uint8_t* qp = static_cast<const uint8_t*>(p.q_lo) + b * p.q_stride[0] + h * p.q_stride[1] + qrow * p.q_stride[2];
#pragma unroll
		for(int c = 0; c < NC; c++) {
			const int d0 = 16 * c + 8 * half;
			u32v2     w  = {0u, 0u};
			if(row_ok && d0 < D && !all_dropped) w = *reinterpret_cast<const u32v2*>(qp + d0);
			qlo[c] = __builtin_bit_cast(long, w);
		}
	}
	// identity fragments scaled by 1/alpha (power of two times 1/softmax_scale folded by the caller: exact in bf16
	// when alpha is a power of two)
	bf16x8 idf[2];
	{
		const uint32_t one_over_alpha = f32_to_bf16_bits(1.f / alpha);
#pragma unroll
		for(int c2 = 0; c2 < 2; c2++) {
			u32x4     v = {0u, 0u, 0u, 0u};
			const int j = n - 16 * c2 - 8 * half;
			if(j >= 0 && j < 8) v[j >> 1] = one_over_alpha << ((j & 1) * 16);
			idf[c2] = __builtin_bit_cast(bf16x8, v);
		}
	}
	u32x4 maskB = {0u, 0u, 0u, 0u};
	if(half == 0) maskB[0] = 0x3F80u;
	u32x4 maskA = {0u, 0u, 0u, 0u};

	const bool           has_bias = p.bias != nullptr && !all_dropped;
	const unsigned char* bias_row = nullptr;
	bool                 bias_vec = false;
	if(has_bias) {
		bias_row = static_cast<const unsigned char*>(p.bias) + (h * p.bias_stride[0] + (row_ok ? qrow : 0) * p.bias_stride[1]) * 2;
		bias_vec = ((reinterpret_cast<uintptr_t>(p.bias) & 15) == 0) && (p.bias_stride[0] % 8 == 0) && (p.bias_stride[1] % 8 == 0);
	}

	// ---- tile loaders (LDS-direct buffer loads, 1 KB per wave instruction) ----
	// K: lane i of load j -> tile row j*(1024/DP) + i/(DP/16), 16-byte chunk i%(DP/16)
	// V^T: lane i of load j -> row d = j*16 + i/4, 16-byte chunk i%4 of the 64-key row
	const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc(
		const_cast<uint8_t*>(static_cast<const uint8_t*>(p.k) + b * p.k_stride[0] + h * p.k_stride[1]), 0, (int)((L - 1) * p.k_stride[2] + D), 0x00020000);  // exact end of the slab: rows are fetched in 16-byte chunks, range-checked per dword, so the tail of the last chunk reads as zero
	const __amdgpu_buffer_rsrc_t klo_rsrc = __builtin_amdgcn_make_buffer_rsrc(
		const_cast<uint8_t*>(static_cast<const uint8_t*>(COMP ? p.k_lo : p.k) + b * p.k_stride[0] + h * p.k_stride[1]), 0, (int)((L - 1) * p.k_stride[2] + D), 0x00020000);
	const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc(
		const_cast<uint8_t*>(static_cast<const uint8_t*>(p.v) + b * p.v_stride[0] + h * p.v_stride[1]), 0, (int)((D - 1) * p.v_stride[2] + p.v_stride[2]), 0x00020000);
	constexpr int KCPR = DP / 16;       // 16-byte chunks per K row
	constexpr int KRPI = 1024 / DP;     // K rows per wave load
	const int  k_row = lane / KCPR, k_ch = lane % KCPR;
	const int  k_voff = (int)(k_row * p.k_stride[2]) + k_ch * 16;
	const bool k_act  = k_ch * 16 < D;
	const int  v_row = lane >> 2, v_ch = lane & 3;
	const int  v_voff = (int)(v_row * p.v_stride[2]) + v_ch * 16;
	auto load_tile = [&](int kt, int buf) {
#pragma unroll
		for(int t = 0; t < (K_LOADS + NW8 - 1) / NW8; t++) {
			const int j = wave + NW8 * t;
			if(j < K_LOADS && k_act) {
				__builtin_amdgcn_raw_ptr_buffer_load_lds(k_rsrc, (__attribute__((address_space(3))) void*)(k_lds + buf * K_TILE + j * 1024), 16, k_voff,
														 (int)((kt * KT8 + j * KRPI) * p.k_stride[2]), 0, 0);
				if(COMP)
					__builtin_amdgcn_raw_ptr_buffer_load_lds(klo_rsrc, (__attribute__((address_space(3))) void*)(k_lds + buf * K_TILE + K_TILE1 + j * 1024), 16, k_voff,
															 (int)((kt * KT8 + j * KRPI) * p.k_stride[2]), 0, 0);
			}
		}
#pragma unroll
		for(int t = 0; t < (V_LOADS + NW8 - 1) / NW8; t++) {
			const int j = wave + NW8 * t;
			if(j < V_LOADS && j * 16 + v_row < D)
				__builtin_amdgcn_raw_ptr_buffer_load_lds(v_rsrc, (__attribute__((address_space(3))) void*)(v_lds + buf * V_TILE + j * 1024), 16, v_voff,
														 (int)(j * 16 * p.v_stride[2]) + kt * KT8, 0, 0);
		}
	};
	u32x4 bfrag[4];
	auto  load_bias_tile = [&](int kt) {
		if(!has_bias) {
#pragma unroll
			for(int f = 0; f < 4; f++) bfrag[f] = u32x4{0u, 0u, 0u, 0u};
			return;
		}
		const int64_t   key0 = (int64_t)kt * KT8 + 8 * half;
		const uint16_t* bp   = reinterpret_cast<const uint16_t*>(bias_row);
		if(bias_vec && (int64_t)(kt + 1) * KT8 <= L) {
#pragma unroll
			for(int f = 0; f < 4; f++) bfrag[f] = row_ok ? *reinterpret_cast<const u32x4*>(bp + key0 + 16 * f) : u32x4{0u, 0u, 0u, 0u};
		} else {
#pragma unroll
			for(int f = 0; f < 4; f++) {
				u32x4 r = {0u, 0u, 0u, 0u};
#pragma unroll
				for(int j = 0; j < 8; j++) {
					const int64_t  key = key0 + 16 * f + j;
					const uint32_t e   = (row_ok && key < L) ? (uint32_t)bp[key] : 0u;
					r[j >> 1] |= e << ((j & 1) * 16);
				}
				bfrag[f] = r;
			}
		}
	};

	// per-lane LDS read offsets
	const int k_rd   = n * DP + 8 * half;                 // + 16*c, + sub*32*DP, + buf*K_TILE
	const int v_rd   = n * KT8 + 4 * half;                // row d = n (+32*db), + 32*sub + 16*cp (+8)
	const int mask_rd     = 2 * K_TILE + 2 * V_TILE + (half == 0 ? n * 4 : (n_ktiles * KT8 + n) * 4);
	const int mask_stride = half == 0 ? KT8 * 4 : 0;

	float  m_run = 0.f, mc = 0.f;  // m_run in accumulator units; mc = m_run*c_exp - P_SHIFT
	bool   first = true;
	// Row sums on the matrix pipe (as in dpa_mfma.hip): a 16x16x32 MFMA whose A operand is a 0/1 pattern adds the 16 quantised
	// probabilities that a query's two lanes hold of a fragment; register 0 of the result is, in every lane, the running sum of
	// that lane's own query row.  As a B operand of the 16x16x32 shape the P fragment's lane l is column l%16, contraction
	// group l/16, and holds query l%32: groups 0,2 belong to queries 0..15, groups 1,3 to queries 16..31; output register 0
	// of lane l is row 4*(l/16): rows 0 and 8 select the even groups, rows 4 and 12 the odd ones.  The normaliser is thus the
	// sum of exactly the e4m3 weights that enter P.V (the result is a convex combination of V rows), and 16 vector adds per
	// 32 x 32 block become two half-size matrix instructions.
	f32x4 lacc = {0.f, 0.f, 0.f, 0.f};
	long  ones_a;
	{
		const int  i16 = lane & 15, kg = lane >> 4;
		const bool on  = ((i16 == 0 || i16 == 8) && (kg & 1) == 0) || ((i16 == 4 || i16 == 12) && (kg & 1) == 1);
		const u32v2 w  = {on ? 0x38383838u : 0u, on ? 0x38383838u : 0u};  // e4m3 1.0
		ones_a = __builtin_bit_cast(long, w);
	}
	f32x16 oacc[NDB];
#pragma unroll
	for(int db = 0; db < NDB; db++)
#pragma unroll
		for(int i = 0; i < 16; i++) oacc[db][i] = 0.f;

	__syncthreads();
	const int kt0 = __builtin_amdgcn_readfirstlane((int)live_list[0]);
	load_tile(kt0, 0);
	load_bias_tile(kt0);
	asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
	__syncthreads();

	for(int it = 0; it < nlive; it++) {
		const int  kt       = __builtin_amdgcn_readfirstlane((int)live_list[it]);
		const int  buf      = it & 1;
		const bool has_next = it + 1 < nlive;
		const int  ktn      = has_next ? __builtin_amdgcn_readfirstlane((int)live_list[it + 1]) : kt;
		if(has_next) load_tile(ktn, buf ^ 1);
		u32x4 bcur[4];
#pragma unroll
		for(int f = 0; f < 4; f++) bcur[f] = bfrag[f];
		if(has_next) load_bias_tile(ktn);
		const int mask_addr = mask_rd + kt * mask_stride;
#pragma unroll
		for(int sub = 0; sub < 2; sub++) {
			f32x16 s;
#pragma unroll
			for(int i = 0; i < 16; i++) s[i] = 0.f;
#pragma unroll
			for(int c = 0; c < NC; c++) {
				const long kf = *reinterpret_cast<const long*>(k_lds + buf * K_TILE + k_rd + sub * 32 * DP + 16 * c);
				s = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(kf, qf[c], s, 0, 0, 0);
				if(COMP) {
					const long kl = *reinterpret_cast<const long*>(k_lds + buf * K_TILE + K_TILE1 + k_rd + sub * 32 * DP + 16 * c);
					s = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(kl, qf[c], s, 0, 0, 0);
					s = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(kf, qlo[c], s, 0, 0, 0);
				}
			}
#pragma unroll
			for(int c2 = 0; c2 < 2; c2++) s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(idf[c2], __builtin_bit_cast(bf16x8, bcur[2 * sub + c2]), s, 0, 0, 0);
			maskA[0] = *reinterpret_cast<const uint32_t*>(smem + mask_addr + sub * 32 * 4);
			s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, maskA), __builtin_bit_cast(bf16x8, maskB), s, 0, 0, 0);

			// online softmax with the true running maximum (in accumulator units)
			float mx = fmaxf(fmaxf(s[0], s[1]), s[2]);
#pragma unroll
			for(int i = 3; i < 15; i += 2) mx = fmaxf(fmaxf(mx, s[i]), s[i + 1]);
			mx = hswap_max(fmaxf(mx, s[15]));
			const float m_new = first ? mx : fmaxf(m_run, mx);
			if(__ballot(first || m_new > m_run)) {
				const float a = first ? 1.f : __builtin_amdgcn_exp2f((m_run - m_new) * c_exp);
#pragma unroll
				for(int i = 0; i < 4; i++) lacc[i] *= a;
#pragma unroll
				for(int db = 0; db < NDB; db++)
#pragma unroll
					for(int i = 0; i < 16; i++) oacc[db][i] *= a;
				m_run = m_new;
				mc    = m_new * c_exp - P_SHIFT;
				first = false;
			}
			u32v2 pf[2];
#pragma unroll
			for(int i = 0; i < 16; i += 4) {
				const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i], c_exp, -mc)), p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i + 1], c_exp, -mc));
				const float p2 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i + 2], c_exp, -mc)), p3 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i + 3], c_exp, -mc));
				uint32_t w = 0;
				w = __builtin_amdgcn_cvt_pk_fp8_f32(p0, p1, w, false);
				w = __builtin_amdgcn_cvt_pk_fp8_f32(p2, p3, w, true);
				pf[i >> 3][(i & 7) >> 2] = w;
			}
#pragma unroll
			for(int cp = 0; cp < 2; cp++) lacc = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(ones_a, __builtin_bit_cast(long, pf[cp]), lacc, 0, 0, 0);
			// O^T += V8^T . P^T: contraction slot j of chunk cp is key 16cp + 8(j/4) + 4half + j%4
#pragma unroll
			for(int cp = 0; cp < 2; cp++)
#pragma unroll
				for(int db = 0; db < NDB; db++) {
					const unsigned char* vp = v_lds + buf * V_TILE + v_rd + db * 32 * KT8 + 32 * sub + 16 * cp;
					u32v2 vf = {*reinterpret_cast<const uint32_t*>(vp), *reinterpret_cast<const uint32_t*>(vp + 8)};
					oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(__builtin_bit_cast(long, vf), __builtin_bit_cast(long, pf[cp]), oacc[db], 0, 0, 0);
				}
		}
		asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
		__syncthreads();
	}

	// epilogue: out = O * dv / l   (l was summed over p * 2^8, the same factor O carries; both half-waves are in it)
	const float inv = dv / lacc[0];
	if(row_ok) {
		const int64_t ooff = b * p.out_stride[0] + h * p.out_stride[1] + qrow * p.out_stride[2];
#pragma unroll
		for(int db = 0; db < NDB; db++)
#pragma unroll
			for(int g4 = 0; g4 < 4; g4++) {
				const int d0 = 32 * db + 8 * g4 + 4 * half;
				if(d0 >= D) continue;
				const float o0 = oacc[db][4 * g4] * inv, o1 = oacc[db][4 * g4 + 1] * inv, o2 = oacc[db][4 * g4 + 2] * inv, o3 = oacc[db][4 * g4 + 3] * inv;
				if(p.out_dtype == AF3_BF16) {
					u32v2 w = {pack_bf16x2(o0, o1), pack_bf16x2(o2, o3)};
					*reinterpret_cast<u32v2*>(static_cast<uint16_t*>(p.out) + ooff + d0) = w;
				} else {
					float4 w = {o0, o1, o2, o3};
					*reinterpret_cast<float4*>(static_cast<float*>(p.out) + ooff + d0) = w;
				}
			}
	}
}

template <int DP, bool COMP>
int launch8(const af3_dpa_params& p, hipStream_t s) {
	const int     n_qtiles = (int)((p.L + NW8 * 32 - 1) / (NW8 * 32));
	const int     n_ktiles = (int)((p.L + KT8 - 1) / KT8);
	const int64_t n_groups = p.B * p.H;
	const int64_t blocks   = ((n_groups + 7) / 8) * 8 * n_qtiles;
	if(blocks <= 0 || blocks > 0x7fffffffLL) return AF3_ERR_BAD_SHAPE;
	const size_t smem = (size_t)(COMP ? 6 : 4) * KT8 * DP + ((size_t)n_ktiles * KT8 + 64) * 4 + (size_t)n_ktiles * 2 + 16;
	hipLaunchKernelGGL((dpa_mfma_fp8_kernel<DP, COMP>), dim3((unsigned)blocks), dim3(NW8 * 64), smem, s, p, n_qtiles, n_groups);
	return launch_status();
}

}  // namespace

bool mfma_fp8_eligible(const af3_dpa_params& p) {
	if(p.io_dtype != AF3_FP8_E4M3 || p.mma_dtype != AF3_FP8_E4M3) return false;
	if(p.D > 64 || p.D % 8 != 0 || p.L > MAX_L8) return false;
	if(p.bias && p.bias_dtype != AF3_BF16) return false;
	// q rows are read 8 bytes at a time, K / V^T rows in 16-byte chunks at 4-byte aligned offsets
	if((reinterpret_cast<uintptr_t>(p.q) & 7) || (reinterpret_cast<uintptr_t>(p.k) & 3) || (reinterpret_cast<uintptr_t>(p.v) & 15)) return false;
	if((p.q_lo != nullptr) != (p.k_lo != nullptr)) return false;  // both residuals or none
	if((reinterpret_cast<uintptr_t>(p.q_lo) & 7) || (reinterpret_cast<uintptr_t>(p.k_lo) & 3)) return false;
	for(int i = 0; i < 3; i++)
		if(p.q_stride[i] % 8 || p.k_stride[i] % 4 || p.v_stride[i] % 16) return false;
	if(p.L * p.k_stride[2] >= 0x7fffffffLL || p.D * p.v_stride[2] >= 0x7fffffffLL) return false;
	if(p.out_dtype == AF3_BF16) {
		if((reinterpret_cast<uintptr_t>(p.out) & 7) || p.out_stride[0] % 4 || p.out_stride[1] % 4 || p.out_stride[2] % 4) return false;
	} else if((reinterpret_cast<uintptr_t>(p.out) & 15) || p.out_stride[0] % 4 || p.out_stride[1] % 4 || p.out_stride[2] % 4) {
		return false;
	}
	return true;
}

int launch_dpa_mfma_fp8(const af3_dpa_params& p, hipStream_t s) {
	const bool comp = p.q_lo != nullptr && p.k_lo != nullptr;
	if(p.D <= 32) return comp ? launch8<32, true>(p, s) : launch8<32, false>(p, s);
	return comp ? launch8<64, true>(p, s) : launch8<64, false>(p, s);
}

}  // namespace af3
