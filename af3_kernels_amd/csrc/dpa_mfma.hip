// bf16 matrix-core attention kernel for gfx950 (CDNA4): out = softmax(q.k^T*scale + bias, mask).v
//
// Work split.  One workgroup = NW wavefronts (4, 2 or 1, chosen so that the launch fills the
// chip) = NW*32 query rows of one (batch, head); each wavefront owns 32 query rows and walks the
// key axis in tiles of 64 keys with an online softmax.  K and V tiles are staged once per
// workgroup in LDS, triple buffered, by buffer loads that write LDS directly (no register
// staging, scalar tile offsets, hardware bounds check for rows past L).  The bias tile is not
// shared between wavefronts, so every lane loads its own 16-byte bias fragments straight from
// global memory (L2-resident: the bias is shared by all batch rows).
//
// Everything is computed "transposed" so that all per-query state is lane-local:
//   S^T[key][q]  = K . Q^T      v_mfma_f32_32x32x16_bf16, A = K tile (LDS), B = Q (registers)
//              += I . bias^T    same shape with A = 0/1 identity fragment, B = bias fragment as
//                               loaded: x * 1.0 accumulates exactly in fp32, so the bias add
//                               costs no vector-ALU work
//              += m . 1^T       one more MFMA whose A holds the additive key-mask value of each
//                               key in contraction slot 0 and whose B holds 1.0 in slot 0
//   In the 32x32 accumulator layout lane (q = lane%32, half = lane/32) holds 16 keys of one
//   query row, so exp / row sum are in-lane loops.
//   O^T[d][q]   += V^T . P^T    A = V^T fragment read with ds_read_b64_tr_b16 from the row-major
//                               V tile, B = P^T = the accumulator registers converted to bf16
//                               in place (the accumulator layout IS the B-operand layout).
// The pack of operands into MFMA layout therefore happens in the load path (global -> LDS ->
// register), which is this design's counterpart of the reference's VNNI repack
// (src/csrc/tools.cpp:151-176).
//
// Two variants of the inner loop:
//   natural  (no workspace)  logits in natural units, bias read in place through the identity
//                            MFMA (exact), p = exp2(fma(s, log2 e, -m*log2 e)).
//   log2     (workspace)     a prepass writes fp16(bias * log2 e) once per call in fragment order
//                            (every bias load is then one coalesced 1 KB wave access; fp16 keeps
//                            11 significant bits, 3 more than the bf16 bias itself), q is scaled
//                            by scale*log2 e, and the reference maximum m rides the mask MFMA
//                            (slot 1: A = 1.0, B = -m, m kept bf16-exact), so p = exp2(s) with no
//                            per-element subtract or multiply at all.
// Softmax bookkeeping is optimistic: only the very first sub-tile of a row computes a row
// maximum.  Afterwards p is computed against the current reference and the row sum (needed
// anyway) is checked; only if a sum is huge or not finite (a logit more than ~26 log2 units above
// the reference) does the wavefront take a rare path that finds the maximum, moves the reference
// and rescales the accumulators.  Probabilities may therefore exceed 1 (up to 2^30), which fp32
// accumulators and bf16 P carry without loss.
//
// Reference semantics followed: src/csrc/dot_product_attention.cpp:88-122 (what is computed) and
// :148-191 (the running max / sum recurrence); the harness formula
// examples/dot_product_attention.py:20-43 for masking (dropped keys get weight 0, an all-dropped
// row yields the mean of V).
#include "mfma_helpers.hpp"

namespace af3 {

// 8 consecutive bias values bias[row][key .. key+7], guarded: elements at key >= L read as zero.
template <bool BIAS_F32>
__device__ __forceinline__ void load_bias8_guarded(const void* bias_row, int64_t key, int64_t L, bool row_ok, float (&f)[8]) {
#pragma unroll
	for(int j = 0; j < 8; j++) {
		f[j] = 0.f;
		if(row_ok && key + j < L) f[j] = BIAS_F32 ? static_cast<const float*>(bias_row)[key + j] : bf16_bits_to_f32(static_cast<const uint16_t*>(bias_row)[key + j]);
	}
}

// A bias fragment that rides the identity MFMA meets 0 in every other contraction slot, and 0 * -inf is NaN: an
// additive -inf (a mask folded into the bias) is therefore replaced by -2^126 before the product (every bias below
// that, and the -NaN patterns, likewise), which gives that key weight exactly 0 like the reference's add-then-softmax;
// -2^126 rather than the most negative finite value so that the product with log2 e stays finite when a row's first
// keys all carry it and it becomes the softmax reference for a while.  +inf and +NaN pass through and yield NaN, as
// they do in the reference.  One packed unsigned minimum per dword.
typedef __attribute__((ext_vector_type(2))) unsigned short u16x2;
__device__ __forceinline__ u32x4 bias_frag_finite(u32x4 w) {
	const u16x2 lim = {(unsigned short)0xFE80, (unsigned short)0xFE80};
#pragma unroll
	for(int j = 0; j < 4; j++) {
		const uint32_t x = w[j];  // (a copy: __builtin_bit_cast applied to the vector element itself reads element 0 with this compiler)
		w[j] = __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(u16x2, x), lim));
	}
	return w;
}

// ---- bias prepass (log2 variant) ---------------------------------------------------------------
// Workspace layout: [H][query block of 32][key tile of 64][fragment 4][lane 64] x 16 bytes: exactly
// the B fragment lane (q = lane%32, g = lane/32) needs for the bias MFMA of fragment f = 2*sub+c2:
// fp16(bias[q][64*kt + 16*f + 8*g + 0..7] * log2 e), zero outside the L x L corner.
template <bool BIAS_F32>
__global__ void __launch_bounds__(256) bias_prepass_kernel(const void* __restrict__ bias, u32x4* __restrict__ ws, int64_t H, int64_t L, int64_t stride_h,
															 int64_t stride_q, int n_qblocks, int n_ktiles, bool vec_ok) {
	// one workgroup per (head, query block, key tile) and trip: the index arithmetic (divisions) is per workgroup, on the
	// scalar unit, not per thread; the launcher keeps the number of units below 2^31
	const uint32_t units = (uint32_t)(H * n_qblocks * (int64_t)n_ktiles);
	const int      lane = threadIdx.x & 63, frag = threadIdx.x >> 6;
	for(uint32_t u = blockIdx.x; u < units; u += gridDim.x) {
		const int64_t i    = (int64_t)u * 256 + threadIdx.x;
		const int     kt   = (int)(u % (uint32_t)n_ktiles);
		const uint32_t t2  = u / (uint32_t)n_ktiles;
		const int     qb   = (int)(t2 % (uint32_t)n_qblocks);
		const int64_t h    = t2 / (uint32_t)n_qblocks;
		const int64_t row  = (int64_t)qb * 32 + (lane & 31);
		const int64_t key  = (int64_t)kt * KT + 16 * frag + 8 * (lane >> 5);
		const int64_t esz  = BIAS_F32 ? 4 : 2;
		const unsigned char* rowp = static_cast<const unsigned char*>(bias) + (h * stride_h + (row < L ? row : 0) * stride_q) * esz;
		float f[8];
		if(!BIAS_F32 && vec_ok && row < L && key + 8 <= L) {
			const u32x4 raw = *reinterpret_cast<const u32x4*>(rowp + key * 2);
#pragma unroll
			for(int j = 0; j < 4; j++) f[2 * j] = bf16_bits_to_f32(raw[j] & 0xffffu), f[2 * j + 1] = bf16_bits_to_f32(raw[j] >> 16);
		} else {
			load_bias8_guarded<BIAS_F32>(rowp, key, L, row < L, f);
		}
		u32x4 o;
#pragma unroll
		for(int j = 0; j < 4; j++) {
			// clamp to the fp16 range: exp2 of anything below -65504 is zero anyway
			const float a = fminf(fmaxf(f[2 * j] * LOG2E, -65504.f), 65504.f), c = fminf(fmaxf(f[2 * j + 1] * LOG2E, -65504.f), 65504.f);
			f16x2       h2 = {(_Float16)a, (_Float16)c};
			o[j] = __builtin_bit_cast(uint32_t, h2);
		}
		ws[i] = o;
	}
}

// DP: head_dim padded to a multiple of 32 (32 or 64).  NW: wavefronts per workgroup.  L2DOM: log2
// variant (bias from the workspace, or no bias at all).  BIAS_F32: bias stored as fp32 (natural
// variant only).  SPLIT: for launches too small to fill the chip -- the NW wavefronts of a workgroup
// share ONE block of 32 query rows and split its key tiles round robin (each with private LDS
// buffers, no barrier in the loop); their partial (O, m, l) are merged through LDS at the end.
// KS2: the other cure for launches too small to fill the chip, for long rows: two wavefronts share each block of 32
// query rows AND the workgroup's K/V tiles -- wavefront 2q + s takes keys [32s, 32s + 32) of every 64-key tile for
// query block q, so a wavefront's dependent chain is half as long and no LDS is spent on private buffers; the two
// partial (O, m, l) are merged through LDS at the end.  The workgroup has NW + 4 wavefronts: the last four only issue the
// tile loads (a ring of five tiles, three tiles ahead: every tile is in LDS one barrier before its first use, so that a
// stage's LDS operands can be fetched at the end of the stage before), so that the NW computing ones never stand still behind a load that the
// compute unit's load path has not taken in yet.  Requires NW even, no SPLIT, not FUSED.  (KSL = 1.  KSL = 2: the four
// loading wavefronts and the ring of four tiles for workgroups of NW wavefronts with a query block each -- the form that
// single rows of head_dim 48 or 64 take.)
// FUSED: the grid-attention variant.  One workgroup = one (batch, head); q, k, v and the gate are not
// read from memory but projected in the kernel from the input rows x[b] (C channels) with the four
// weight matrices of this head, K and V of ALL keys stay in LDS for the whole workgroup, and each
// wavefront then walks query blocks qb = wave, wave + NW, ... on its own (no barrier after the
// projection of K and V).  Requires DP = 32, the log2 variant, no key split.
template <int DP, int NW, bool L2DOM, int BMODE, bool SPLIT, bool FUSED, int KSL>
// (at least 2 wavefronts per SIMD: keeps the register budget at 256 so that the compiler writes MFMA
// results to ordinary VGPRs instead of AGPRs, which every softmax operand would have to be copied out of;
// the key-split variants are limited to fewer than 2 wavefronts per SIMD by their LDS buffers anyway)
__global__ void __launch_bounds__((NW + (KSL ? 4 : 0)) * 64) __attribute__((amdgpu_waves_per_eu(FUSED ? (NW <= 4 ? 3 : (NW + 3) / 4) : KSL ? (NW + 7) / 4 : DP == 32 && !SPLIT ? (L2DOM ? 4 : 3) : 2))) dpa_mfma_bf16_kernel(af3_dpa_params p, int n_qtiles, int64_t n_groups, fused_grid_args fa) {
	constexpr int NC         = DP / 16;            // contraction chunks of QK^T
	constexpr int NDB        = DP / 32;            // 32-row blocks of O^T
	constexpr int CPR        = DP / 8;             // 16-byte chunks per K/V row
	constexpr int TILE_BYTES = KT * DP * 2;
	constexpr int NI         = TILE_BYTES / 1024;  // 1 KB wave loads per tile and tensor
	constexpr int RPI        = 512 / DP;           // tile rows covered by one wave load
	constexpr bool KS2       = KSL == 1;           // pairs of wavefronts on shared tiles (with loading wavefronts)
	constexpr bool LOADERS   = KSL != 0;           // four more wavefronts issue the tile loads (KSL == 2: one computing wavefront per query block)
	constexpr int QT         = SPLIT ? 32 : KS2 ? NW * 16 : NW * 32;
	constexpr int  LDS_SETS   = SPLIT ? NW : 1;  // private K/V buffer sets
	constexpr bool BIAS_F32   = BMODE == 1;      // natural variant, bias stored as fp32, read in place
	constexpr bool BRING      = BMODE == 2;      // natural variant, bf16 bias streamed through a per-wavefront LDS ring
	// tile buffers of the K/V ring and slots of a bias ring.  With loading wavefronts the loads run two tiles ahead; KS2 in
	// addition has every tile in LDS one barrier before its first use, so that a stage's LDS operands are fetched at the end of
	// the stage before it (AHEAD: the tile that has landed when iteration j passes its barrier is j + AHEAD).
	constexpr int  AHEAD      = KS2 ? 2 : 1;
	constexpr int  NBUF       = LOADERS ? AHEAD + 3 : 3;
	constexpr int  RING_BYTES = BRING ? (KS2 ? NW / 2 : NW) * NBUF * 4096 : 0;  // (KS2: one ring per pair of wavefronts)
	constexpr int  MASK_BASE  = LDS_SETS * 2 * NBUF * TILE_BYTES + RING_BYTES;
	static_assert(!(L2DOM && BMODE != 0), "the log2 variant reads its bias from the workspace");
	static_assert(FUSED || (LOADERS ? NI % 4 == 0 : NW <= NI), "every wavefront that loads fetches a whole number of 1 KB pieces of each tile");
	static_assert(!LOADERS || (!SPLIT && !FUSED), "loading wavefronts serve workgroups that share their tiles");
	static_assert(!KS2 || (!SPLIT && !FUSED && NW % 2 == 0), "the shared-tile key split pairs up the wavefronts of an unfused workgroup");
	static_assert(!FUSED || (DP == 32 && L2DOM && !SPLIT && NW % 2 == 0), "the fused variant exists for 32-channel heads in the log2 variant");

	extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
	// [K x NBUF][V x NBUF][bias ring: NBUF x 4 KB per wavefront (BRING)][mask table: (n_ktiles*64 + 64) dwords][live list]
	const int            tid_pre   = threadIdx.x;
	// FUSED: [K of all tiles][V of all tiles][Wq fragments][Wgate fragments][mask table][live list]
	const int            n_ktiles  = (int)((p.L + KT - 1) / KT);
	constexpr int        NS        = 8;  // FUSED: contraction steps of a projection (C = 128 input channels, 16 per MFMA)
	unsigned char* const k_lds     = smem + (SPLIT ? __builtin_amdgcn_readfirstlane(tid_pre >> 6) * 2 * NBUF * TILE_BYTES : 0);
	unsigned char* const v_lds     = k_lds + (FUSED ? n_ktiles : NBUF) * TILE_BYTES;
	unsigned char* const w_lds     = v_lds + n_ktiles * TILE_BYTES;  // FUSED only
	const int            mask_base = FUSED ? 2 * n_ktiles * TILE_BYTES + 2 * NS * 1024 : MASK_BASE;
	uint32_t* const      mask_tab  = reinterpret_cast<uint32_t*>(smem + mask_base);
	// unfused variants with an output gate: the gate rows of each wavefront's query block, [32][DP] bf16, behind the tile list
	const int            gate_base = (mask_base + (n_ktiles * KT + 64) * 4 + n_ktiles * 2 + 15) & ~15;
	int16_t* const       live_list = reinterpret_cast<int16_t*>(mask_tab + n_ktiles * KT + 64);
	__shared__ int       s_nvalid, s_nlive;

	// ---- workgroup -> (batch, head, query tile).  Workgroups are handed to the 8 XCDs round
	// robin, so all query tiles of one (batch, head) are given ids that are congruent mod 8:
	// they share that XCD's L2 copy of K and V, and an XCD only ever sees heads h = xcd % H
	// (for H | 8), so its share of the bias stays L2-resident across the whole batch.
	// The kernel arguments that the start of a workgroup needs, requested in one batch: left to itself the compiler fetches the
	// two launch counts, waits, tests the early exit below, and only then requests the fields of p -- two memory latencies
	// in a row, which every wavefront of a launch too small to hide them stands through.
	asm volatile("" ::"s"(n_qtiles), "s"(n_groups), "s"(p.q), "s"(p.k), "s"(p.v), "s"(p.bias), "s"(p.key_mask), "s"(p.H), "s"(p.L), "s"(p.D), "s"(p.key_mask_stride_b),
				 "s"(p.bias_stride[0]), "s"(p.bias_stride[1]));
	asm volatile("" ::"s"(p.q_stride[0]), "s"(p.q_stride[1]), "s"(p.q_stride[2]), "s"(p.k_stride[0]), "s"(p.k_stride[1]), "s"(p.k_stride[2]), "s"(p.v_stride[0]), "s"(p.v_stride[1]),
				 "s"(p.v_stride[2]));
	const int64_t wg    = blockIdx.x;
	const int     xcd   = (int)(wg & 7);
	const int64_t slot  = wg >> 3;
	const int64_t group = (slot / n_qtiles) * 8 + xcd;
	const int     qtile = (int)(slot % n_qtiles);
	if(!FUSED && group >= n_groups) return;
	// FUSED (4 heads): an XCD serves two heads -- their bias (2.4 MB) stays in its 4 MB L2 -- and the two
	// workgroups that read the same rows x[b] through that L2 are neighbours in dispatch order.
	const int64_t b = FUSED ? (slot >> 1) * 4 + (xcd >> 1) : group / p.H, h = FUSED ? 2 * (xcd & 1) + (slot & 1) : group % p.H;
	if(FUSED && b >= p.B) return;

	const int     tid = threadIdx.x, lane = tid & 63;
	const int     wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int     n = lane & 31, half = lane >> 5;
	const int64_t L = p.L;
	// KS2: the workgroup has four wavefronts more than the NW that compute (one per SIMD).  They issue the tile loads of the
	// workgroup, two or three tiles ahead, a quarter of every tile each, and otherwise only keep the barriers' count.  A wavefront that
	// issues a tile's loads itself stands still while the compute unit's load path (64 bytes per clock) takes them in -- with
	// one compute wavefront per SIMD nothing else runs in that time, and it was a quarter of the key loop.  (A single loader
	// is too few: one wavefront gets a load accepted every 45-64 clocks at best.)
	const bool    is_loader = LOADERS && wave >= NW;
	const int     ld        = wave - NW;  // which quarter (loader wavefronts)
	const int     D = (int)p.D;

	const int sub  = KS2 ? (wave & 1) : 0;                  // KS2: which 32 keys of every 64-key tile this wavefront takes
	const int wblk = SPLIT ? 0 : KS2 ? (wave >> 1) : wave;  // this wavefront's block of 32 query rows within the workgroup's QT rows

	// ---- K/V tile loader: buffer loads that write LDS directly ----
	// One wave load moves 1 KB: lane i -> LDS chunk i of the load's 1 KB window, i.e. tile row
	// j*RPI + i/CPR, physical chunk i%CPR.  The lane picks the global chunk that belongs there
	// under the swizzle; lanes of padded head columns (chunk*8 >= D) fetch the row's first chunk.
	const u32x4 k_rsrc = raw_rsrc(static_cast<const uint16_t*>(p.k) + b * p.k_stride[0] + h * p.k_stride[1], (uint32_t)(((L - 1) * p.k_stride[2] + D) * 2));
	const u32x4 v_rsrc = raw_rsrc(static_cast<const uint16_t*>(p.v) + b * p.v_stride[0] + h * p.v_stride[1], (uint32_t)(((L - 1) * p.v_stride[2] + D) * 2));
	const int  ld_row  = lane / CPR, ld_pc = lane % CPR;
	const int  k_chunk = ld_pc ^ k_swizzle<DP>(ld_row);
	const int  v_chunk = ld_pc ^ v_swizzle<DP>(ld_row);
	const int  k_voff  = (int)(ld_row * p.k_stride[2] * 2) + (k_chunk * 8 < D ? k_chunk * 16 : 0);   // (padded head columns: the first chunk again)
	const int  v_voff  = (int)(ld_row * p.v_stride[2] * 2) + (v_chunk * 8 < D ? v_chunk * 16 : 0);
	const int  k_row_bytes = (int)(p.k_stride[2] * 2), v_row_bytes = (int)(p.v_stride[2] * 2);
	const int  k_tile_stride = (int)(KT * p.k_stride[2] * 2), v_tile_stride = (int)(KT * p.v_stride[2] * 2);
	const int  k_ld_stride   = (int)(RPI * p.k_stride[2] * 2), v_ld_stride = (int)(RPI * p.v_stride[2] * 2);
	// byte offsets of piece j of tile kt for this lane; a piece that reaches past the last key (rare, wave-uniform test)
	// sends the lanes of rows >= L to row L - 1
	auto kv_offsets = [&](int kt, int j, int& ko, int& vo) {
		ko = k_voff + (kt * k_tile_stride + j * k_ld_stride), vo = v_voff + (kt * v_tile_stride + j * v_ld_stride);
		const int row0 = kt * KT + j * RPI;
		if(row0 + RPI > (int)L) {
			const int over = row0 + lane / CPR - ((int)L - 1);
			if(over > 0) ko -= over * k_row_bytes, vo -= over * v_row_bytes;
		}
	};
	const uint32_t k_lds_addr = lds_addr_of(k_lds), v_lds_addr = lds_addr_of(v_lds);
	auto load_tile = [&](int kt, int buf) {
		if(FUSED) return;  // K and V of every tile are already in LDS
		if constexpr(LOADERS) {  // pieces ld, ld + 4, ... of K and of V, by loader wavefront ld
			if(!is_loader) return;
#pragma unroll
			for(int t = 0; t < NI / 4; t++) {
				const int j = ld + 4 * t;
				int       ko, vo;
				kv_offsets(kt, j, ko, vo);
				lds_dma_b128(k_rsrc, k_lds_addr + buf * TILE_BYTES + j * 1024, ko);
				lds_dma_b128(v_rsrc, v_lds_addr + buf * TILE_BYTES + j * 1024, vo);
			}
			return;
		}
#pragma unroll
		for(int t = 0; t < (SPLIT ? NI : NI / NW); t++) {
			const int j = SPLIT ? t : wave + NW * t;  // split: this wavefront fetches whole tiles into its private buffers
			int ko, vo;
			kv_offsets(kt, j, ko, vo);
			lds_dma_b128(k_rsrc, k_lds_addr + buf * TILE_BYTES + j * 1024, ko);
			lds_dma_b128(v_rsrc, v_lds_addr + buf * TILE_BYTES + j * 1024, vo);
		}
	};

	// ---- bias ring (BRING): the 32 x 64 bias tile of this wavefront's query block, 4 KB, travels
	// HBM -> LDS by four LDS-direct loads of whole 128-byte row segments (eight lanes per row), two
	// tiles ahead of its use and without occupying registers.  Slot layout: [row 32][128 B], the
	// 16-byte chunk c of row r stored at chunk position c ^ (r & 7) so that the fragment reads (one
	// chunk per lane, 32 rows at once) spread over the banks.  Rows past L fetch row L - 1 and chunks of
	// keys past L (last tile) the row's last valid chunk, so padding behind a row's L valid entries is
	// never read and every byte of a slot is written with finite data by every load.
	const u32x4    b_rsrc    = raw_rsrc(BRING ? static_cast<const uint16_t*>(p.bias) + h * p.bias_stride[0] : nullptr,
										BRING ? (uint32_t)(((L - 1) * p.bias_stride[1] + L) * 2) : 0u);
	unsigned char* const bring = smem + LDS_SETS * 2 * NBUF * TILE_BYTES + (BRING ? (KS2 ? wblk : wave) * NBUF * 4096 : 0);  // (compute wavefronts)
	const uint32_t bring_addr = lds_addr_of(bring);
	const int      b_voff     = (int)((lane >> 3) * p.bias_stride[1] * 2) + (((lane & 7) ^ (lane >> 3)) << 4);
	const int      b_row0     = (int)((qtile * QT + wblk * 32) * p.bias_stride[1] * 2);
	const int      b_row8     = (int)(8 * p.bias_stride[1] * 2);
	const int      b_key      = ((lane & 7) ^ (lane >> 3)) * 8;  // first key of this lane's chunk within a tile
	auto load_bias_tile = [&](int kt, int slot_i) {
		if(!BRING) return;
		const int in_row   = kt * KT + b_key < (int)L ? b_voff + kt * (KT * 2) : b_voff - b_key * 2 + ((int)L - 8) * 2;
		if constexpr(LOADERS) {  // eight rows (piece ld) of the tiles of all the workgroup's query blocks, by loader wavefront ld
			if(!is_loader) return;
			const uint32_t rings = lds_addr_of(smem + LDS_SETS * 2 * NBUF * TILE_BYTES);
#pragma unroll
			for(int wb = 0; wb < (KS2 ? NW / 2 : NW); wb++) {
				const int blk_row0 = (int)(qtile * QT + wb * 32);
				int       off      = in_row + (int)(blk_row0 * p.bias_stride[1] * 2) + ld * b_row8;
				if(blk_row0 + 32 > (int)L) {  // (rare, wave-uniform: the matrix' last query block and blocks past it)
					const int over = blk_row0 + 8 * ld + (lane >> 3) - ((int)L - 1);
					if(over > 0) off -= over * (int)(p.bias_stride[1] * 2);
				}
				lds_dma_b128(b_rsrc, rings + (wb * NBUF + slot_i) * 4096 + ld * 1024, off);
			}
			return;
		}
		const int blk_row0 = (int)(qtile * QT + wblk * 32);
#pragma unroll
		for(int j = 0; j < 4; j++) {
			int off = in_row + (b_row0 + j * b_row8);
			if(blk_row0 + 32 > (int)L) {   // (rare, wave-uniform: the matrix' last query block)
				const int over = blk_row0 + 8 * j + (lane >> 3) - ((int)L - 1);
				if(over > 0) off -= over * (int)(p.bias_stride[1] * 2);
			}
			lds_dma_b128(b_rsrc, bring_addr + slot_i * 4096 + j * 1024, off);
		}
	};
	// ---- key-mask bytes: requested first.  With 4-byte aligned mask rows
	// a lane takes four keys per load (a chunk of 256 keys = four tiles per wavefront and load) and all of a wavefront's
	// loads -- up to eight per pass -- are in flight together: one memory latency, not one per tile (a single row's walk
	// is short enough for that to show). ----
	const uint8_t* keep     = p.key_mask ? p.key_mask + b * p.key_mask_stride_b : nullptr;
	const bool     mask_vec = !keep || (((reinterpret_cast<uintptr_t>(p.key_mask) | (uintptr_t)p.key_mask_stride_b | (uintptr_t)L) & 3) == 0);
	const int      n_chunks = (n_ktiles * KT + 255) / 256;
	uint32_t       mraw[8];
	auto request_mask = [&](int c0) {
#pragma unroll
		for(int i = 0; i < 8; i++) {
			const int64_t key0 = (int64_t)(c0 + i * NW) * 256 + 4 * lane;
			mraw[i]            = 0u;
			if(c0 + i * NW < n_chunks) mraw[i] = !keep ? 0x01010101u : (key0 < L ? *reinterpret_cast<const uint32_t*>(keep + key0) : 0u);
		}
	};
	if(mask_vec && !is_loader) request_mask(wave);
	[[maybe_unused]] u32x4 qraw[NC];
	if constexpr(!FUSED) {
		const int64_t   qrow0 = (int64_t)qtile * QT + wblk * 32 + n;
		const uint16_t* qp    = static_cast<const uint16_t*>(p.q) + b * p.q_stride[0] + h * p.q_stride[1] + qrow0 * p.q_stride[2];
#pragma unroll
		for(int c = 0; c < NC; c++) {
			const int d0 = 16 * c + 8 * half;
			qraw[c]      = u32x4{0u, 0u, 0u, 0u};
			if(qrow0 < L && d0 < D && !is_loader) qraw[c] = *reinterpret_cast<const u32x4*>(qp + d0);
		}
	}

	// ---- The other first requests go out now as well: the two tiles of K and V (and of the bias ring) that this wavefront
	// walks first if the leading tiles all hold a live key -- the tile list below tells; a wrong guess costs a second load
	// into the same buffer, and loads land in issue order.  One memory latency then covers the mask bytes, q and the first
	// tiles: a call too small to keep other workgroups on the compute unit has nothing else to hide them behind.  (These
	// loads are younger than the mask bytes, and the compiler does not count them: its wait for the mask bytes also waits
	// for most of them, which costs little since all were issued within a fraction of one latency.) ----
	const int  guess_kt0 = SPLIT ? wave : 0, guess_kt1 = SPLIT ? wave + NW : 1;
	const bool guessed0 = !FUSED && guess_kt0 < n_ktiles, guessed1 = !FUSED && guess_kt1 < n_ktiles;  // (wave-uniform)
	if(guessed0) {
		load_tile(guess_kt0, 0);
		load_bias_tile(guess_kt0, 0);
	}
	if(guessed1) {
		load_tile(guess_kt1, 1);
		load_bias_tile(guess_kt1, 1);
	}

	// (The K/V buffers and the bias ring are not cleared: every load of a tile writes every byte of its buffer with finite
	// data -- lanes of padded head columns fetch the row's first chunk again (q is zero there), rows and keys past L fetch the
	// last row / the row's last chunk again (their logits get the out-of-range mask value) -- so no stale LDS content is
	// ever read.  Clearing 72 KB with 128 threads cost a single-row call 3600 of its 24000 clocks.)
	// ---- key-mask table and list of tiles with at least one live key ----
	// entry = bf16 additive mask value in the low half (contraction slot 0) and, in the log2
	// variant, 1.0 in the high half (slot 1, multiplies -m_ref); the last 64 entries are zero
	// (read by the lanes of the upper half-wave, whose contraction slots are unused).
	// (No barrier in front of the table: each tile's flag has one writer, the count of live tiles is taken from the flags
	// below, and the zero entries are first read in the key loop.)
	if(tid < 64) mask_tab[n_ktiles * KT + tid] = 0u;
	if(is_loader) {
		// (the loader wavefront takes no part in the table)
	} else if(mask_vec) {
		for(int c0 = wave; c0 < n_chunks; c0 += 8 * NW) {
			if(c0 != wave) request_mask(c0);
#pragma unroll
			for(int i = 0; i < 8; i++) {
				const int c = c0 + i * NW;
				if(c >= n_chunks) break;
				const int64_t key0 = (int64_t)c * 256 + 4 * lane;
				u32x4         e;
				bool          any = false;
#pragma unroll
				for(int j = 0; j < 4; j++) {
					const bool in   = key0 + j < L;
					const bool live = in && ((mraw[i] >> (8 * j)) & 0xffu) != 0;
					any             = any || live;
					e[j]            = (live ? 0u : (in ? (uint32_t)MASK_DROPPED_BF16 : (uint32_t)MASK_OUT_OF_RANGE_BF16)) | (L2DOM ? 0x3F800000u : 0u);
				}
				if(key0 < (int64_t)n_ktiles * KT) *reinterpret_cast<u32x4*>(mask_tab + key0) = e;
				const unsigned long long bal = __ballot(any);   // 16 lanes per tile
				if(lane < 4 && 4 * c + lane < n_ktiles) {
					const bool tile_live = ((bal >> (16 * lane)) & 0xffffull) != 0;
					live_list[4 * c + lane] = tile_live ? 1 : 0;
				}
			}
		}
	} else {
		for(int kt = wave; kt < n_ktiles; kt += NW) {
			const int64_t  key  = (int64_t)kt * KT + lane;
			const bool     in   = key < L;
			const bool     live = in && keep[in ? key : 0] != 0;
			const uint32_t mv   = live ? 0u : (in ? (uint32_t)MASK_DROPPED_BF16 : (uint32_t)MASK_OUT_OF_RANGE_BF16);
			mask_tab[kt * KT + lane] = mv | (L2DOM ? 0x3F800000u : 0u);
			const unsigned long long bal = __ballot(live);
			if(lane == 0) {
				live_list[kt] = bal ? 1 : 0;
			}
		}
	}
	__syncthreads();
	// Compact the flags into a list of live tile indices (wavefront 0, 64 tiles per pass: rank =
	// number of live tiles below).  If no key of this batch row is live every tile is kept: the
	// result is then the mean over all L keys.
	if(wave == 0) {
		bool any_live = false;
		for(int base = 0; base < n_ktiles; base += 64) any_live = any_live || __ballot(base + lane < n_ktiles && live_list[base + lane] != 0) != 0;
		const bool all = !any_live;
		int        cnt = 0;
		for(int base = 0; base < n_ktiles; base += 64) {
			const int  kt   = base + lane;
			const bool keepit = kt < n_ktiles && (all || live_list[kt] != 0);
			const unsigned long long bal = __ballot(keepit);
			const int rank = __builtin_amdgcn_mbcnt_hi((unsigned)(bal >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)bal, 0));
			__builtin_amdgcn_wave_barrier();  // all flags of this pass are read before any index is written (cnt + rank <= kt)
			if(keepit) live_list[cnt + rank] = (int16_t)kt;
			cnt += __builtin_popcountll(bal);
		}
		if(lane == 0) s_nlive = cnt, s_nvalid = any_live ? 1 : 0;
	}
	__syncthreads();
	const int nlive = __builtin_amdgcn_readfirstlane(s_nlive);
	// A batch row without any live key: q and the bias are dropped so that every logit is exactly
	// the mask constant and the weights come out uniform whatever the accumulation order.
	const bool all_dropped = __builtin_amdgcn_readfirstlane(s_nvalid) == 0;

	if constexpr(LOADERS) {
		if(is_loader) {
			// ---- a loader wavefront: tile j of the walk goes to buffer j % NBUF and is requested AHEAD + 1 tiles before the compute
			// wavefronts fetch K fragments from it.  Its barriers mirror theirs one for one: one in front of the first S^T, one
			// per live tile, and (pairs) three in the merge. ----
			constexpr int PER_TILE = 2 * (NI / 4) + (BRING ? (KS2 ? NW / 2 : NW) : 0);  // this wavefront's loads per tile
			static_assert(PER_TILE <= 63, "the wait counter has six bits");
			auto walk = [&](int j) -> int { return __builtin_amdgcn_readfirstlane((int)live_list[j < nlive ? j : nlive - 1]); };
			const int kt0 = walk(0);
			if(!guessed0 || kt0 != guess_kt0) {
				load_tile(kt0, 0);
				load_bias_tile(kt0, 0);
			}
			if(nlive > 1) {
				const int kt1 = walk(1);
				if(!guessed1 || kt1 != guess_kt1) {
					load_tile(kt1, 1);
					load_bias_tile(kt1, 1);
				}
			}
			asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
			__syncthreads();  // (tiles 0 and 1 are in LDS)
#pragma unroll
			for(int j = 2; j <= AHEAD + 1; j++)
				if(j < nlive) {
					load_tile(walk(j), j);
					load_bias_tile(walk(j), j);
				}
			for(int it = 0; it < nlive; it++) {
				// tile it + AHEAD has landed (the tile behind it, if there is one, may still be on its way)
				if(it + AHEAD + 1 < nlive) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PER_TILE) : "memory");
				else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
				__syncthreads();  // (every wavefront is done with tile it - 1, whose buffer tile it + AHEAD + 2 takes)
				if(it + AHEAD + 2 < nlive) {
					load_tile(walk(it + AHEAD + 2), (it + AHEAD + 2) % NBUF);
					load_bias_tile(walk(it + AHEAD + 2), (it + AHEAD + 2) % NBUF);
				}
			}
			asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
			if constexpr(KS2) {
				__syncthreads();
				__syncthreads();
				__syncthreads();
			}
			return;
		}
	}

	// ---- FUSED: projections.  out^T[d][token] = sum_c W[c][d] * x[token][c], 32 tokens per matrix instruction chain:
	//   A operand (weights)    lane (d = lane%32, g = lane/32), step s: W[16s + 8g + 0..7][d]; in the panel layout
	//                          [C/2][32][2] of one head these are four dwords, 32 dwords apart;
	//   B operand (rows of x)  lane (token = lane%32, g), step s: x[token][16s + 8g + 0..7], one 16-byte load
	//                          (range-checked: rows past L read as zero);
	//   result                 lane = token, register i = output channel 8*(i/4) + 4*g + i%4.
	[[maybe_unused]] __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(static_cast<uint16_t*>(nullptr), 0, 0, 0x00020000);
	[[maybe_unused]] int x_row_bytes = 0;
	auto load_x_frags = [&](int token, u32x4 (&xf)[NS]) {
#pragma unroll
		for(int st = 0; st < NS; st++)
			xf[st] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, token * x_row_bytes + (16 * st + 8 * half) * 2, 0, 0));
	};
	// q fragments (B operand of S^T = K.Q^T) and, FUSED, the gate pre-activations of this lane's 16 output channels as
	// bf16 pairs: per query block; the fused variant prepares them one block ahead
	const float qmul = all_dropped ? 0.f : (L2DOM ? p.softmax_scale * LOG2E : p.softmax_scale);
	bf16x8      qf[NC];
	[[maybe_unused]] u32x4 gate_pk[2] = {u32x4{0u, 0u, 0u, 0u}, u32x4{0u, 0u, 0u, 0u}};
	// q and gate rows of a block from its rows of x (src/csrc/dot_product_attention.cpp:301-312, :334-345); q is scaled
	// in fp32 and rounded once, the gate is rounded to bf16 like the reference's tmp buffer
	auto project_q_gate = [&](const u32x4 (&xf)[NS]) {
		f32x16 aq, ag;
#pragma unroll
		for(int i = 0; i < 16; i++) aq[i] = 0.f, ag[i] = 0.f;
#pragma unroll
		for(int st = 0; st < NS; st++) {
			const u32x4 wqf = reinterpret_cast<const u32x4*>(w_lds)[st * 64 + lane], wgf = reinterpret_cast<const u32x4*>(w_lds)[(NS + st) * 64 + lane];
			aq = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, wqf), __builtin_bit_cast(bf16x8, xf[st]), aq, 0, 0, 0);
			ag = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, wgf), __builtin_bit_cast(bf16x8, xf[st]), ag, 0, 0, 0);
		}
#pragma unroll
		for(int c = 0; c < NC; c++) {
			u32x4 sc4;
#pragma unroll
			for(int j = 0; j < 4; j++) sc4[j] = pack_bf16x2(aq[8 * c + 2 * j] * qmul, aq[8 * c + 2 * j + 1] * qmul);
			qf[c] = __builtin_bit_cast(bf16x8, sc4);
		}
#pragma unroll
		for(int j = 0; j < 8; j++) gate_pk[j >> 2][j & 3] = pack_bf16x2(ag[2 * j], ag[2 * j + 1]);
	};
	const int n_qblocks_all = (int)((L + 31) / 32);
	int       qb_f          = 0;  // FUSED: the query block this wavefront works on
	// FUSED: q and gate of the block this wavefront takes second, projected while its rows of x were in registers for K and V
	[[maybe_unused]] bf16x8 q_next[NC];
	[[maybe_unused]] u32x4  gate_next[2] = {u32x4{0u, 0u, 0u, 0u}, u32x4{0u, 0u, 0u, 0u}};
	[[maybe_unused]] int    qb_next      = -1;  // which block q_next / gate_next belong to
	if constexpr(FUSED) {
		x_rsrc      = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(fa.x + b * fa.x_stride_b), 0, (int)(((L - 1) * fa.x_stride_n + 16 * NS) * 2), 0x00020000);
		x_row_bytes = (int)(fa.x_stride_n * 2);
		const int64_t head_dwords = h * (16 * NS * 32 / 2);
		// Wq and Wgate fragments -> LDS, [matrix][step][lane] x 16 bytes.  The rows of Wq are permuted so that the
		// registers of the q projection's result ARE the B operand of K.Q^T: register i of half-wave g must hold
		// channel 16*(i/8) + 8*g + i%8, and it holds result row 8*(i/4) + 4*g + i%4.
		for(int i = tid; i < 2 * NS * 64; i += NW * 64) {
			const int ln = i & 63, st = (i >> 6) % NS, m = i / (64 * NS);
			const int r = ln & 31, g = ln >> 5, a = r >> 3;
			const int d = m == 0 ? 16 * (a >> 1) + 8 * ((r >> 2) & 1) + 4 * (a & 1) + (r & 3) : r;
			const uint32_t* w32 = reinterpret_cast<const uint32_t*>(m == 0 ? fa.wq : fa.wg) + head_dwords + (8 * st + 4 * g) * 32 + d;
			reinterpret_cast<u32x4*>(w_lds)[i] = u32x4{w32[0], w32[32], w32[64], w32[96]};
		}
		__syncthreads();  // the fragments are read below
		// K and V of every key, 32 keys at a time (wavefront w takes blocks w, w + NW, ...), rounded to bf16 like the
		// reference's tmp_k / tmp_v (src/csrc/dot_product_attention.cpp:286-299) and stored where the tile loader of
		// the unfused kernel would have put them (K rows chunk-swizzled, V rows plain).  One load of the 32 rows
		// of x serves both products.
		const uint32_t* wk32 = reinterpret_cast<const uint32_t*>(fa.wk) + head_dwords + (4 * half) * 32 + n;
		const uint32_t* wv32 = reinterpret_cast<const uint32_t*>(fa.wv) + head_dwords + (4 * half) * 32 + n;
		u32x4           wkf[NS], wvf[NS];
#pragma unroll
		for(int st = 0; st < NS; st++) {
			wkf[st] = u32x4{wk32[(8 * st) * 32], wk32[(8 * st + 1) * 32], wk32[(8 * st + 2) * 32], wk32[(8 * st + 3) * 32]};
			wvf[st] = u32x4{wv32[(8 * st) * 32], wv32[(8 * st + 1) * 32], wv32[(8 * st + 2) * 32], wv32[(8 * st + 3) * 32]};
		}
		// This wavefront's query blocks are walked from the last one down: its rows of x are the ones used last here (unless
		// the last key block was padding past L), so q and the gate of that block come for free; those of the block before it
		// are projected when its rows pass by and kept in registers until its turn.
		const int qb_last = n_qblocks_all - 1 - (n_qblocks_all - 1 - wave + NW * 64) % NW;  // largest block index congruent to wave (negative: none)
		u32x4     xf[NS];
		int       sb_last = -1;
		for(int sb = wave; sb < 2 * n_ktiles; sb += NW) {
			const int key = sb * 32 + n;
			load_x_frags(key, xf);
			f32x16 ak, av;
#pragma unroll
			for(int i = 0; i < 16; i++) ak[i] = 0.f, av[i] = 0.f;
#pragma unroll
			for(int st = 0; st < NS; st++) {
				ak = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, wkf[st]), __builtin_bit_cast(bf16x8, xf[st]), ak, 0, 0, 0);
				av = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, wvf[st]), __builtin_bit_cast(bf16x8, xf[st]), av, 0, 0, 0);
			}
			unsigned char* const kdst = k_lds + key * (DP * 2) + half * 8;
			unsigned char* const vdst = v_lds + key * (DP * 2) + half * 8;
			const int            swz  = k_swizzle<DP>(n);
#pragma unroll
			for(int j = 0; j < 4; j++) {
				*reinterpret_cast<u32x2*>(kdst + ((j ^ swz) << 4)) = u32x2{pack_bf16x2(ak[4 * j], ak[4 * j + 1]), pack_bf16x2(ak[4 * j + 2], ak[4 * j + 3])};
				*reinterpret_cast<u32x2*>(vdst + (j << 4))         = u32x2{pack_bf16x2(av[4 * j], av[4 * j + 1]), pack_bf16x2(av[4 * j + 2], av[4 * j + 3])};
			}
			if(sb == qb_last - NW) {
				project_q_gate(xf);
#pragma unroll
				for(int c = 0; c < NC; c++) q_next[c] = qf[c];
				gate_next[0] = gate_pk[0], gate_next[1] = gate_pk[1];
				qb_next = sb;
			}
			sb_last = sb;
		}
		qb_f = qb_last;
		if(qb_f >= 0) {
			if(sb_last != qb_f) load_x_frags(qb_f * 32 + n, xf);
			project_q_gate(xf);
		}
		__syncthreads();  // K and V of every key are in LDS
	}

	// ---- one pass per block of 32 query rows: exactly one pass unless FUSED ----
	for(; qb_f >= 0; qb_f -= FUSED ? NW : 1) {
		// ---- per-lane constants ----
		const int64_t qrow   = FUSED ? (int64_t)qb_f * 32 + n : (int64_t)qtile * QT + wblk * 32 + n;
		const bool    row_ok = qrow < L;

		// Q fragments (B operand of S^T = K.Q^T): lane (q = n, g = half) holds q[q][16c + 8g .. +7]
		// scaled and rounded to bf16 (the reference also rounds the scaled q,
		// src/csrc/dot_product_attention.cpp:95-98).
		if constexpr(!FUSED) {
#pragma unroll
			for(int c = 0; c < NC; c++) {
				const u32x4 raw = qraw[c];
				u32x4       sc;
#pragma unroll
				for(int j = 0; j < 4; j++) sc[j] = pack_bf16x2(bf16_bits_to_f32(raw[j] & 0xffffu) * qmul, bf16_bits_to_f32(raw[j] >> 16) * qmul);
				qf[c] = __builtin_bit_cast(bf16x8, sc);
			}
		}
		// Identity fragments (A operand of the bias MFMA): lane (m = n, g = half), slot j of chunk c2
		// is 1.0 iff m == 16*c2 + 8*g + j.  bf16 1.0 for the natural variant, fp16 1.0 for the log2 one.
		u32x4 idf[2];
#pragma unroll
		for(int c2 = 0; c2 < 2; c2++) {
			u32x4     v = {0u, 0u, 0u, 0u};
			const int j = n - 16 * c2 - 8 * half;
			if(j >= 0 && j < 8) v[j >> 1] = (L2DOM ? 0x3C00u : 0x3F80u) << ((j & 1) * 16);
			idf[c2] = v;
		}
		// B operand of the mask MFMA: slot 0 = 1.0 (multiplies the key's mask value); log2 variant: slots 1
		// and 2 = the reference maximum as -(m_hi + m_lo), two bf16 terms (16 significant bits, so that a
		// reference of large magnitude -- a row whose biases are all hugely negative -- is still subtracted
		// to within a fraction of a unit), multiplying the 1.0 that every key carries in slots 1 and 2 of A.
		u32x4 maskB = {0u, 0u, 0u, 0u};
		if(half == 0) maskB[0] = 0x3F80u;
		u32x4 maskA = {0u, 0u, 0u, 0u};
		if(L2DOM && half == 0) maskA[1] = 0x3F80u;  // slot 2; slots 0 and 1 come from the mask table

		const bool has_bias = p.bias != nullptr && !all_dropped;
		// natural variant: direct bias access through per-lane row pointers
		const unsigned char* bias_row = nullptr;
		bool                 bias_vec = false;
		if(!L2DOM && has_bias) {
			const int64_t esz = BIAS_F32 ? 4 : 2;
			bias_row = static_cast<const unsigned char*>(p.bias) + (h * p.bias_stride[0] + (row_ok ? qrow : 0) * p.bias_stride[1]) * esz;
			bias_vec = !BIAS_F32 && ((reinterpret_cast<uintptr_t>(p.bias) & 15) == 0) && (p.bias_stride[0] % 8 == 0) && (p.bias_stride[1] % 8 == 0);
		}
		// log2 variant: fragment-ordered workspace; the tile base is wave-uniform
		const u32x4* ws_wave = nullptr;
		if(L2DOM && has_bias) {
			const int     n_qblocks = (int)((L + 31) / 32);
			const int64_t qb        = FUSED ? (int64_t)qb_f : SPLIT ? (int64_t)qtile : (int64_t)qtile * (QT / 32) + wblk;
			// query blocks beyond the last one only hold rows >= L; clamp so that loads stay in bounds
			const int64_t qbc = qb < n_qblocks ? qb : n_qblocks - 1;
			ws_wave = static_cast<const u32x4*>(p.workspace) + ((h * n_qblocks + qbc) * n_ktiles) * 256;
		}
		// (scalar base + per-lane 16-byte offset + scalar tile offset: no 64-bit pointer in vector registers)
		const __amdgpu_buffer_rsrc_t ws_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<u32x4*>(ws_wave), 0, ws_wave ? n_ktiles * 4096 : 0, 0x00020000);
		const int                    ws_voff = lane * 16 + sub * 2048;  // (KS2: fragments 2 and 3 of a tile belong to keys 32..63)

		// ---- output gate: fetched into LDS now, by loads that write LDS directly and hold no registers, and read in the
		// epilogue.  (Loading it in the epilogue exposed a full memory latency per workgroup: 8 % of the kernel's time.)
		// The first tile wait of the prologue below also covers these loads: they are older. ----
		unsigned char* const gate_lds = smem + gate_base + wblk * (32 * DP * 2);
		if(!FUSED && p.gate && (SPLIT ? wave == 0 : sub == 0)) {  // (the wavefronts that write results)
			const u32x4   g_rsrc = raw_rsrc(static_cast<const uint16_t*>(p.gate) + b * p.gate_stride[0] + h * p.gate_stride[1], (uint32_t)(((L - 1) * p.gate_stride[2] + D) * 2));
			constexpr int RPL    = 512 / DP;  // rows per 1 KB wave load
			const int     g_row  = lane / CPR, g_c = lane % CPR;
			const int64_t row0   = qrow - n;  // first row of this wavefront's block
#pragma unroll
			for(int t = 0; t < 32 / RPL; t++) {
				const int64_t row  = row0 + t * RPL + g_row;
				const int     voff = (g_c * 8 < D && row < L) ? (int)(row * p.gate_stride[2] * 2) + g_c * 16 : 0x7FFF0000;  // past the range: nothing is fetched
				lds_dma_b128(g_rsrc, lds_addr_of(gate_lds) + t * 1024, voff);
			}
		}

		// fragment read: lane (n, half) takes chunk 4*sub + 2*c2 + half of row n
		const int b_rd = (n * 128 + (((n & 7) ^ half) << 4)) ^ (sub << 6);  // (KS2: chunks 4..7 of a row hold keys 32..63)

		// Natural variant: four fragments in flight, each sub-tile's pair requested two stages before its
		// use.  Log2 variant (BIAS_LATE): one pair only -- the registers are the scarce resource at four
		// wavefronts per SIMD -- requested inside the previous stage, right after the matrix
		// instructions that consume the pair before it.
		constexpr bool BIAS_LATE = L2DOM || KS2;  // (KS2: one stage per tile, so one pair one stage ahead in every variant)
		u32x4 bfrag[4];
		auto  load_bias_frags = [&](int kt, auto sub_c) {
			constexpr int SUB = decltype(sub_c)::value;
			if(!has_bias || BRING) return;
			if(L2DOM) {
#pragma unroll
				for(int c2 = 0; c2 < 2; c2++)
					bfrag[c2] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(ws_rsrc, ws_voff + (2 * SUB + c2) * 1024, kt * 4096, 0));
				return;
			}
			const int64_t key0 = (int64_t)kt * KT + 8 * half + 32 * sub;
			if(bias_vec && (int64_t)(kt + 1) * KT <= L) {  // wave-uniform: whole tile in range, aligned rows
				const uint16_t* bp = reinterpret_cast<const uint16_t*>(bias_row) + key0;
				if(row_ok) {
#pragma unroll
					for(int f = 2 * SUB; f < 2 * SUB + 2; f++) bfrag[f] = bias_frag_finite(*reinterpret_cast<const u32x4*>(bp + 16 * f));
				} else {
#pragma unroll
					for(int f = 2 * SUB; f < 2 * SUB + 2; f++) bfrag[f] = u32x4{0u, 0u, 0u, 0u};
				}
			} else {
#pragma unroll
				for(int f = 2 * SUB; f < 2 * SUB + 2; f++) {
					float v8[8];
					load_bias8_guarded<BIAS_F32>(bias_row, key0 + 16 * f, L, row_ok, v8);
#pragma unroll
					for(int j = 0; j < 4; j++) bfrag[f][j] = pack_bf16x2(v8[2 * j], v8[2 * j + 1]);
					bfrag[f] = bias_frag_finite(bfrag[f]);
				}
			}
		};

		// ---- per-lane LDS read addresses (bytes, for buffer 0 / sub-tile 0; the rest are immediates) ----
		int k_rd[NC];
#pragma unroll
		for(int c = 0; c < NC; c++) k_rd[c] = (n + 32 * sub) * DP * 2 + (((2 * c + half) ^ k_swizzle<DP>(n)) << 4);  // (KS2: rows 32..63 of every tile)
		// V^T fragment reads: lane l: i = l%16, G = l/16 supplies the 8-byte chunk at tile row
		// base + 4*(G/2) + i/4, column 32*db + 16*(G%2) + 4*(i%4); it receives 4 keys of column 32*db + l%32.
		int v_rd[NDB];
		{
			const int i16 = lane & 15, G = lane >> 4;
			const int row = 4 * (G >> 1) + (i16 >> 2);
#pragma unroll
			for(int db = 0; db < NDB; db++) {
				const int col   = 32 * db + 16 * (G & 1) + 4 * (i16 & 3);
				const int chunk = (col >> 3) ^ v_swizzle<DP>(row);
				v_rd[db] = (row + 32 * sub) * DP * 2 + chunk * 16 + (col & 7) * 2;
			}
		}
		// mask table read address: lanes of the upper half-wave always read the zero entries
		const int mask_rd     = mask_base + (half == 0 ? (n + 32 * sub) * 4 : (n_ktiles * KT + n) * 4);
		const int mask_stride = half == 0 ? KT * 4 : 0;

		// ---- online-softmax state (per lane: one query row; the two halves hold disjoint keys) ----
		float  m_ref = 0.f;  // reference maximum: log2 units and bf16-exact (log2 variant), natural units (natural variant)
		float  mc    = 0.f;  // natural variant: m_ref * log2 e
		f32x4  lacc  = {0.f, 0.f, 0.f, 0.f};  // [0] = this lane's row sum (complete: the same value in both half-waves)
		f32x16 oacc[NDB];
#pragma unroll
		for(int db = 0; db < NDB; db++)
#pragma unroll
			for(int i = 0; i < 16; i++) oacc[db][i] = 0.f;

		// Move the reference of every row whose maximum is not within REF_SLACK of it (all rows when
		// `force`), rescale what has been accumulated, and re-express s (and a sub-tile that was
		// already issued against the old reference) relative to the new one.
		auto rereference = [&](f32x16& s, f32x16* pending, bool force) {
			float mx = fmaxf(fmaxf(s[0], s[1]), s[2]);
#pragma unroll
			for(int i = 3; i < 15; i += 2) mx = fmaxf(fmaxf(mx, s[i]), s[i + 1]);
			mx = half_swap_max(fmaxf(mx, s[15]));
			float alpha;
			if(L2DOM) {
				// s already has m_ref subtracted (by the mask MFMA)
				// A sub-tile whose keys are all dropped says nothing about the row: the reference stays at 0, its probabilities are
				// exactly 0, and the first live logits keep their own bits.  Until a row has a non-zero sum (`fresh`) its first
				// live logits fix the reference wherever they lie -- the largest then has probability exactly 1, so a row whose
				// biases are all hugely negative cannot end with a zero sum -- and nothing is accumulated that would need rescaling.
				const bool  fresh = force || lacc[0] == 0.f;
				const bool  need  = (fresh && (all_dropped || mx > -0x1p99f)) || mx > REF_SLACK;  // (a row without any live key keeps the mask constant as its reference)
				const float m_want = m_ref + mx;
				const float m_hi   = bf16_bits_to_f32(f32_to_bf16_bits(need ? m_want : m_ref));
				const float m_lo   = bf16_bits_to_f32(f32_to_bf16_bits((need ? m_want : m_ref) - m_hi));
				const float m_new  = m_hi + m_lo;  // exactly what the mask MFMA will subtract (unchanged when !need)
				const float delta  = m_new - m_ref;
				alpha = fresh ? 1.f : __builtin_amdgcn_exp2f(-delta);
#pragma unroll
				for(int i = 0; i < 16; i++) s[i] -= delta;
				if(pending) {
#pragma unroll
					for(int i = 0; i < 16; i++) (*pending)[i] -= delta;
				}
				m_ref = m_new;
				if(half == 0) {
					maskB[0] = 0x3F80u | (f32_to_bf16_bits(-m_hi) << 16);
					maskB[1] = f32_to_bf16_bits(-m_lo);
				}
			} else {
				const bool  need  = force || mx > m_ref + REF_SLACK * 0.6931472f;
				const float m_new = need ? mx : m_ref;
				alpha = force ? 1.f : __builtin_amdgcn_exp2f((m_ref - m_new) * LOG2E);
				m_ref = m_new;
				mc    = m_new * LOG2E;
			}
			lacc[0] *= alpha;
#pragma unroll
			for(int db = 0; db < NDB; db++)
#pragma unroll
				for(int i = 0; i < 16; i++) oacc[db][i] *= alpha;
		};

		// p = exp2(s - reference) for logits [I0, I0+N) of a sub-tile, packed to bf16 pairs.  (The row sum is
		// taken from the packed pairs on the matrix pipe, rowsum_mfma below: 16 vector adds per sub-tile
		// cost more, and v_dot2c_f32_bf16 on the pairs does not execute concurrently with MFMA.)
		auto exp_part = [&](const f32x16& s, u32x4 (&pf)[2], auto i0_c, auto n_c) {
			constexpr int I0 = decltype(i0_c)::value, N = decltype(n_c)::value;
#pragma unroll
			for(int i = I0; i < I0 + N; i += 2) {
				float p0, p1;
				if(L2DOM) {
					p0 = __builtin_amdgcn_exp2f(s[i]);
					p1 = __builtin_amdgcn_exp2f(s[i + 1]);
				} else {
					p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i], LOG2E, -mc));
					p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i + 1], LOG2E, -mc));
				}
				pf[i >> 3][(i & 7) >> 1] = pack_bf16x2(p0, p1);
			}
		};

		// One pipeline stage.  On entry `sc` holds the finished S^T of sub-tile j, `pprev`/`vprev` the
		// P^T and V^T fragments of sub-tile j-1.  The stage interleaves, one matrix instruction per
		// handful of vector instructions so that both pipes stay busy within this wavefront:
		//     matrix pipe                         vector ALU
		//     O^T += V^T . P^T   (sub-tile j-1)   exp2 / pack of sub-tile j
		//     S^T of sub-tile j+1 (K.Q^T, bias,   row sum of sub-tile j
		//                          mask)
		// and leaves S^T(j+1) in `sc`, P^T(j) in `pprev`, V^T(j) fragments in `vprev`.
		// k_off / v_off: byte offsets of the LDS buffers holding sub-tile j+1's K rows and sub-tile j's V rows;
		// SUBN / SUBC: which half of those tiles; FB: first bias fragment of sub-tile j+1.
		f32x16 sc;
		u32x4  pprev[2] = {u32x4{0u, 0u, 0u, 0u}, u32x4{0u, 0u, 0u, 0u}};
		u32x4  vprev[2][NDB];
#pragma unroll
		for(int cp = 0; cp < 2; cp++)
#pragma unroll
			for(int db = 0; db < NDB; db++) vprev[cp][db] = u32x4{0u, 0u, 0u, 0u};

		// Row sums on the matrix pipe: a 16x16x32 MFMA whose A operand is a 0/1 pattern adds the 16 packed
		// probabilities of a fragment (both half-waves) for every query; with this pattern register 0 of
		// the result holds, in every lane, the sum for that lane's own query row.  As a B operand of the
		// 16x16x32 shape the P fragment's lane l is column l%16, contraction group l/16, and holds query
		// l%32: groups 0,2 belong to queries 0..15, groups 1,3 to queries 16..31.  Output register 0 of
		// lane l is row 4*(l/16): rows 0 and 8 select the even groups, rows 4 and 12 the odd ones.
		u32x4 ones_a;
		{
			const int  i16 = lane & 15, kg = lane >> 4;
			const bool on  = ((i16 == 0 || i16 == 8) && (kg & 1) == 0) || ((i16 == 4 || i16 == 12) && (kg & 1) == 1);
			const uint32_t w = on ? 0x3F803F80u : 0u;
			ones_a = u32x4{w, w, w, w};
		}
		auto rowsum_mfma = [&](const u32x4& pf) {
			lacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, ones_a), __builtin_bit_cast(bf16x8, pf), lacc, 0, 0, 0);
		};
		auto read_kfrag = [&](int k_off, int sub, int c) -> u32x4 { return *reinterpret_cast<const u32x4*>(k_lds + k_rd[c] + k_off + sub * 32 * DP * 2); };
		auto read_vfrags = [&](int v_off, int sub) {
#pragma unroll
			for(int cp = 0; cp < 2; cp++)
#pragma unroll
				for(int db = 0; db < NDB; db++)
#pragma unroll
					for(int t = 0; t < 2; t++) {
						const int   off = v_off + (32 * sub + 16 * cp + 8 * t) * DP * 2;
						const s16x4 r   = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(v_lds + v_rd[db] + off));
						const u32x2 rr  = __builtin_bit_cast(u32x2, r);
						vprev[cp][db][2 * t]     = rr[0];
						vprev[cp][db][2 * t + 1] = rr[1];
					}
		};
		auto bias_mfma = [&](f32x16 s, int f) -> f32x16 {
			if(L2DOM) return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, idf[f & 1]), __builtin_bit_cast(f16x8, bfrag[f & 1]), s, 0, 0, 0);
			return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, idf[f & 1]), __builtin_bit_cast(bf16x8, bfrag[f]), s, 0, 0, 0);
		};
		// plain (not interleaved) S^T of one sub-tile; used once, for the very first sub-tile
		auto compute_s_plain = [&](int k_off, int sub, int mask_addr, int fb) -> f32x16 {
			f32x16 s;
#pragma unroll
			for(int i = 0; i < 16; i++) s[i] = 0.f;
#pragma unroll
			for(int c = 0; c < NC; c++) s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, read_kfrag(k_off, sub, c)), qf[c], s, 0, 0, 0);
			s = bias_mfma(s, fb);
			s = bias_mfma(s, fb + 1);
			maskA[0] = *reinterpret_cast<const uint32_t*>(smem + mask_addr + sub * 32 * 4);
			return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, maskA), __builtin_bit_cast(bf16x8, maskB), s, 0, 0, 0);
		};

		auto read_bias_ring = [&](int slot_off, auto sub_c) {
			constexpr int SUB = decltype(sub_c)::value;
#pragma unroll
			for(int c2 = 0; c2 < 2; c2++) bfrag[2 * SUB + c2] = bias_frag_finite(*reinterpret_cast<const u32x4*>(bring + slot_off + (b_rd ^ ((4 * SUB + 2 * c2) << 4))));
		};
		// ring_off (BRING): byte offset of the ring slot that holds the bias tile of sub-tile j+1
		// The LDS operands of S^T(j+1): K fragments, bias fragments (ring variants), mask entries.  KS2 fetches them at the end of
		// the stage before (every tile is in LDS one barrier early there), so that their latency hides behind that stage's
		// row-sum check instead of standing in front of this stage's first matrix instruction: a lone wavefront has nothing
		// else to run in that time.
		u32x4    kf[NC];
		uint32_t mask_next = 0;
		auto fetch_operands = [&](auto subn_c, int k_off, int mask_addr_next, int ring_off) {
			constexpr int SUBN = decltype(subn_c)::value;
			if(BRING) read_bias_ring(ring_off, subn_c);
#pragma unroll
			for(int c = 0; c < NC; c++) kf[c] = read_kfrag(k_off, SUBN, c);
			mask_next = *reinterpret_cast<const uint32_t*>(smem + mask_addr_next + SUBN * 32 * 4);
		};
		// k_next / mask_next_addr / ring_next (KS2): where the operands of the stage after this one are
		auto stage = [&](auto subn_c, int k_off, int mask_addr_next, int v_off, auto subc_c, int bias_kt, auto bias_sub_c, int ring_off, int k_next, int mask_next_addr, int ring_next) {
			constexpr int SUBN = decltype(subn_c)::value, SUBC = decltype(subc_c)::value, FB = 2 * SUBN;
			if constexpr(!KS2) fetch_operands(subn_c, k_off, mask_addr_next, ring_off);
			maskA[0] = mask_next;
			u32x4  pcur[2];
			f32x16 sn;
#pragma unroll
			for(int i = 0; i < 16; i++) sn[i] = 0.f;
			// One matrix instruction, then a handful of vector instructions, and so on: a dependent
			// MFMA chain would otherwise stall the wavefront for the full 32-cycle pass of each link.
			// The scheduling barriers keep the compiler from regrouping the chunks.
#define AF3_CHUNK_END() __builtin_amdgcn_sched_barrier(0)
			AF3_CHUNK_END();
			// O^T += V^T . P^T of the previous sub-tile, exp2 of this one
#pragma unroll
			for(int db = 0; db < NDB; db++)
				oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vprev[0][db]), __builtin_bit_cast(bf16x8, pprev[0]), oacc[db], 0, 0, 0);
			exp_part(sc, pcur, ic<0>{}, ic<2>{});
			AF3_CHUNK_END();
#pragma unroll
			for(int db = 0; db < NDB; db++)
				oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vprev[1][db]), __builtin_bit_cast(bf16x8, pprev[1]), oacc[db], 0, 0, 0);
			exp_part(sc, pcur, ic<2>{}, ic<2>{});
			AF3_CHUNK_END();
			// S^T of the next sub-tile
			sn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kf[0]), qf[0], sn, 0, 0, 0);
			// V^T fragments of this sub-tile for the next stage's PV product: issued as soon as the two PV
			// MFMAs above have consumed the previous fragments, a whole stage before their use
			read_vfrags(v_off, SUBC);
			exp_part(sc, pcur, ic<4>{}, ic<2>{});
			AF3_CHUNK_END();
			sn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kf[1]), qf[1], sn, 0, 0, 0);
			exp_part(sc, pcur, ic<6>{}, ic<2>{});
			AF3_CHUNK_END();
#pragma unroll
			for(int c = 2; c < NC; c++) sn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kf[c]), qf[c], sn, 0, 0, 0);
			// (the bias MFMAs run unconditionally -- on zero fragments when there is no bias -- so that the
			// whole stage stays one basic block)
			sn = bias_mfma(sn, FB);
			const float l_before = lacc[0];
			rowsum_mfma(pcur[0]);
			exp_part(sc, pcur, ic<8>{}, ic<2>{});
			AF3_CHUNK_END();
			sn = bias_mfma(sn, FB + 1);
			exp_part(sc, pcur, ic<10>{}, ic<2>{});
			AF3_CHUNK_END();
			if(BIAS_LATE) load_bias_frags(bias_kt, bias_sub_c);  // pair of the sub-tile after the next one
			sn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, maskA), __builtin_bit_cast(bf16x8, maskB), sn, 0, 0, 0);
			exp_part(sc, pcur, ic<12>{}, ic<4>{});
			AF3_CHUNK_END();
#undef AF3_CHUNK_END
			rowsum_mfma(pcur[1]);
			if constexpr(KS2) fetch_operands(subn_c, k_next, mask_next_addr, ring_next);  // (this stage's have been consumed)
			// The running sum stays below L * 2^REF_SLACK <= 2^25 while every probability respects the
			// reference, so this also catches a single probability near or beyond the limit (inf, NaN).  A sum that is still
			// zero (log2 variant: leading sub-tiles of dropped keys, or live logits so far below the initial reference that
			// their probabilities flush to zero) takes the same path, which then fixes the reference at the first live logits.
			if(__ballot(!(lacc[0] < PSUM_LIMIT) || (L2DOM && lacc[0] == 0.f))) {  // rare
				lacc[0] = l_before;
				rereference(sc, &sn, false);
				exp_part(sc, pcur, ic<0>{}, ic<16>{});
				rowsum_mfma(pcur[0]);
				rowsum_mfma(pcur[1]);
			}
			sc       = sn;
			pprev[0] = pcur[0];
			pprev[1] = pcur[1];
		};

		// ---- which live tiles this wavefront walks: all of them, or every NW-th one when splitting ----
		const int my_first = SPLIT ? wave : 0, my_step = SPLIT ? NW : 1;
		const int my_n     = SPLIT ? (nlive > wave ? (nlive - wave + NW - 1) / NW : 0) : nlive;
		auto live_at = [&](int j) -> int { return (int)live_list[my_first + (j < my_n ? j : my_n - 1) * my_step]; };

		if(my_n > 0) {
			// ---- prologue: first two tiles, first sub-tile's S^T and its row maximum ----
			const int kt0 = __builtin_amdgcn_readfirstlane(live_at(0));
			if(!guessed0 || kt0 != guess_kt0) {
				load_tile(kt0, 0);
				load_bias_tile(kt0, 0);
			}
			if(my_n > 1) {
				const int kt1_first = __builtin_amdgcn_readfirstlane(live_at(1));
				if(!guessed1 || kt1_first != guess_kt1) {
					load_tile(kt1_first, 1);
					load_bias_tile(kt1_first, 1);
				}
			}
#pragma unroll
			for(int f = 0; f < 4; f++) bfrag[f] = u32x4{0u, 0u, 0u, 0u};
			load_bias_frags(kt0, ic<0>{});
			if(!BIAS_LATE) load_bias_frags(kt0, ic<1>{});
			asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
			if(!SPLIT && !FUSED) __syncthreads();
			if(BRING) read_bias_ring(0, ic<0>{});
			sc = compute_s_plain(FUSED ? kt0 * TILE_BYTES : 0, 0, mask_rd + kt0 * mask_stride, 0);
			rereference(sc, nullptr, true);
			if constexpr(KS2) {
				const int kt1_first = __builtin_amdgcn_readfirstlane(live_at(1));
				load_bias_frags(kt1_first, ic<0>{});                                                // this wavefront's next sub-tile is in the next tile
				fetch_operands(ic<0>{}, TILE_BYTES, mask_rd + kt1_first * mask_stride, 4096);  // operands of the first stage: second tile of the walk, buffer 1
			} else if(BIAS_LATE) load_bias_frags(kt0, ic<1>{});
			else if(my_n > 1) load_bias_frags(__builtin_amdgcn_readfirstlane(live_at(1)), ic<0>{});

			int buf = 0;  // LDS buffer of tile `it` (it % NBUF)
			// tile indices of iterations it, it+1, it+2 are carried in scalar registers; the list entry for
			// it+3 is fetched at the top of an iteration and only consumed at its end
			int kt = kt0, kt1 = __builtin_amdgcn_readfirstlane(live_at(1)), kt2 = __builtin_amdgcn_readfirstlane(live_at(2));
			if constexpr(KS2) {
				// One stage per tile: this wavefront's 32 keys of tile `it` (exp, V fragments) and of tile it+1 (S^T).  Behind the
				// barrier tile it+2 is in LDS (the loading wavefronts have waited for it) and everyone is done with tile it-1,
				// whose buffer they now hand to tile it+4.
				auto tile_step = [&](int it) {
					const int bufn = buf == NBUF - 1 ? 0 : buf + 1, bufnn = bufn == NBUF - 1 ? 0 : bufn + 1;
					// The barrier hands the buffer of tile it-1 back to the loading wavefronts, so this wavefront's reads of that
					// tile must have returned; the operands fetched at the end of the stage before (the last OPERAND_READS LDS
					// reads issued, from the buffer of tile it+1) may stay in flight.  LDS reads return in issue order.  (The counter
					// also counts scalar memory loads, which do not: this relies on the loop holding none -- every kernel argument
					// is in registers before the loop, and the compiler has no reason to fetch one again while none is spilled.)
					constexpr int OPERAND_READS = NC + 1 + (BRING ? 2 : 0);
					asm volatile("s_waitcnt lgkmcnt(%0)\n\ts_barrier" ::"n"(OPERAND_READS) : "memory");
					const int kt3_v = live_at(it + 3);  // (behind the barrier, which would wait for this read)
					stage(ic<0>{}, bufn * TILE_BYTES, mask_rd + kt1 * mask_stride, buf * TILE_BYTES, ic<0>{}, kt2, ic<0>{}, bufn * 4096, bufnn * TILE_BYTES, mask_rd + kt2 * mask_stride,
						  bufnn * 4096);
					buf = bufn;
					kt  = kt1;
					kt1 = kt2;
					kt2 = __builtin_amdgcn_readfirstlane(kt3_v);
				};
				// two stages per trip, so that the score registers of consecutive stages swap roles instead of being copied
				int it = 0;
				for(; it + 1 < my_n; it += 2) {
					tile_step(it);
					tile_step(it + 1);
				}
				if(it < my_n) tile_step(it);
			} else
			for(int it = 0; it < my_n; it++) {
				const int kt3_v = live_at(it + 3);
				const int bufn = buf == NBUF - 1 ? 0 : buf + 1, bufnn = bufn == NBUF - 1 ? 0 : bufn + 1;
				// LDS offsets of tile it and of tile it+1: ring buffers, or the tiles' own places when all of K and V is resident
				const int off_cur = (FUSED ? kt : buf) * TILE_BYTES, off_next = (FUSED ? kt1 : bufn) * TILE_BYTES;
				// sub-tile (it, 0): next is (it, 1) in the same buffer
				stage(ic<1>{}, off_cur, mask_rd + kt * mask_stride, off_cur, ic<0>{}, kt1, ic<0>{}, buf * 4096, 0, 0, 0);
				if(!BIAS_LATE) load_bias_frags(kt1, ic<1>{});
				// Tile it+1 (issued one iteration ago) must have landed, and every wavefront must be done
				// with tile it-1, whose buffer tile it+2 is about to overwrite.  Loads complete in issue
				// order; the only loads this wavefront has issued since that tile are bias fragments: two in
				// the log2 variant (the pair requested inside the stage above), which may stay in flight.
				if(!FUSED) {
					if(L2DOM && has_bias) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
					else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
				}
				if(!SPLIT && !FUSED) __syncthreads();
				if(it + 2 < my_n) {
					load_tile(kt2, bufnn);
					load_bias_tile(kt2, bufnn);  // (its slot held tile it-1, last read in the stage above)
				}
				// sub-tile (it, 1): next is (it+1, 0) in the next buffer (harmless stale data after the last tile)
				stage(ic<0>{}, off_next, mask_rd + kt1 * mask_stride, off_cur, ic<1>{}, kt1, ic<1>{}, bufn * 4096, 0, 0, 0);
				if(!BIAS_LATE) load_bias_frags(kt2, ic<0>{});
				buf = bufn;
				kt  = kt1;
				kt1 = kt2;
				kt2 = __builtin_amdgcn_readfirstlane(kt3_v);
			}
		}
		// the last sub-tile's PV product
#pragma unroll
		for(int cp = 0; cp < 2; cp++)
#pragma unroll
			for(int db = 0; db < NDB; db++)
				oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vprev[cp][db]), __builtin_bit_cast(bf16x8, pprev[cp]), oacc[db], 0, 0, 0);

		if constexpr(KS2) {
			// ---- merge the two partial results of every pair of wavefronts (same 32 query rows, disjoint keys) ----
			asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
			__syncthreads();  // all K/V buffers are dead: reuse the front of LDS
			float* const mred = reinterpret_cast<float*>(smem);        // [NW][32] reference maxima
			float* const obuf = mred + NW * 32;                        // [NW / 2][16*NDB + 1][64]
			static_assert((NW * 32 + (NW / 2) * (16 * NDB + 1) * 64) * 4 <= 2 * NBUF * TILE_BYTES, "the merge area fits in the K/V buffers");
			// (a wavefront whose sum is zero has seen dropped keys only: its reference says nothing and must not enter the maximum)
			const bool started = lacc[0] > 0.f;
			if(half == 0) mred[wave * 32 + n] = started ? m_ref : -INFINITY;
			__syncthreads();
			const float mstar   = fmaxf(mred[(wave & ~1) * 32 + n], mred[(wave | 1) * 32 + n]);
			const float scale_w = started ? __builtin_amdgcn_exp2f((m_ref - mstar) * (L2DOM ? 1.f : LOG2E)) : 0.f;
			lacc[0] *= scale_w;
#pragma unroll
			for(int db = 0; db < NDB; db++)
#pragma unroll
				for(int i = 0; i < 16; i++) oacc[db][i] *= scale_w;
			float* const slot_p = obuf + wblk * (16 * NDB + 1) * 64 + lane;
			if(sub == 1) {
#pragma unroll
				for(int db = 0; db < NDB; db++)
#pragma unroll
					for(int i = 0; i < 16; i++) slot_p[(db * 16 + i) * 64] = oacc[db][i];
				slot_p[16 * NDB * 64] = lacc[0];
			}
			__syncthreads();
			if(sub == 1) return;
#pragma unroll
			for(int db = 0; db < NDB; db++)
#pragma unroll
				for(int i = 0; i < 16; i++) oacc[db][i] += slot_p[(db * 16 + i) * 64];
			lacc[0] += slot_p[16 * NDB * 64];
		}
		if(SPLIT) {
			// ---- merge the partial results of the NW wavefronts (same 32 query rows, disjoint keys) ----
			asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
			__syncthreads();  // all K/V buffers are dead: reuse the front of LDS
			float* const mred = reinterpret_cast<float*>(smem);        // [NW][32] reference maxima
			float* const obuf = mred + NW * 32;                        // [NW][16*NDB + 1][64]
			// (a wavefront without a tile, or whose sum is zero -- it has seen dropped keys only --, contributes nothing, and its
			// reference must not enter the maximum)
			const bool started = my_n > 0 && lacc[0] > 0.f;
			if(half == 0) mred[wave * 32 + n] = started ? m_ref : -INFINITY;
			__syncthreads();
			float mstar = mred[n];
#pragma unroll
			for(int w = 1; w < NW; w++) mstar = fmaxf(mstar, mred[w * 32 + n]);
			const float scale_w = started ? __builtin_amdgcn_exp2f((m_ref - mstar) * (L2DOM ? 1.f : LOG2E)) : 0.f;
			lacc[0] *= scale_w;
#pragma unroll
			for(int db = 0; db < NDB; db++)
#pragma unroll
				for(int i = 0; i < 16; i++) oacc[db][i] *= scale_w;
			if(wave > 0) {
				float* mine = obuf + wave * (16 * NDB + 1) * 64 + lane;
#pragma unroll
				for(int db = 0; db < NDB; db++)
#pragma unroll
					for(int i = 0; i < 16; i++) mine[(db * 16 + i) * 64] = oacc[db][i];
				mine[16 * NDB * 64] = lacc[0];
			}
			__syncthreads();
			if(wave > 0) return;
#pragma unroll
			for(int w = 1; w < NW; w++) {
				const float* theirs = obuf + w * (16 * NDB + 1) * 64 + lane;
#pragma unroll
				for(int db = 0; db < NDB; db++)
#pragma unroll
					for(int i = 0; i < 16; i++) oacc[db][i] += theirs[(db * 16 + i) * 64];
				lacc[0] += theirs[16 * NDB * 64];
			}
		}

		if(!FUSED && p.gate) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (the gate rows; long since landed unless there was no tile at all)
		// ---- epilogue: O^T register i of block db is head column 32*db + 8*(i/4) + 4*half + i%4 ----
		// (8-byte stores, 16 bytes per row and instruction.  Turning the tile through LDS for 16-byte stores of whole 64-byte
		// row segments was measured: 0.4 % faster in the fused variant, 1.5 % slower in the unfused ones, which spill at 128
		// registers; not kept.)
		const float l_tot = lacc[0];
		const float inv   = 1.f / l_tot;
		if(row_ok) {
			const int64_t ooff = b * p.out_stride[0] + h * p.out_stride[1] + qrow * p.out_stride[2];
#pragma unroll
			for(int db = 0; db < NDB; db++)
#pragma unroll
				for(int g4 = 0; g4 < 4; g4++) {
					const int d0 = 32 * db + 8 * g4 + 4 * half;
					if(d0 >= D) continue;
					float o0 = oacc[db][4 * g4] * inv, o1 = oacc[db][4 * g4 + 1] * inv;
					float o2 = oacc[db][4 * g4 + 2] * inv, o3 = oacc[db][4 * g4 + 3] * inv;
					if constexpr(FUSED) {
						const u32x2 gw = {gate_pk[g4 >> 1][2 * (g4 & 1)], gate_pk[g4 >> 1][2 * (g4 & 1) + 1]};
						o0 *= sigmoidf_fast(bf16_bits_to_f32(gw[0] & 0xffffu)), o1 *= sigmoidf_fast(bf16_bits_to_f32(gw[0] >> 16));
						o2 *= sigmoidf_fast(bf16_bits_to_f32(gw[1] & 0xffffu)), o3 *= sigmoidf_fast(bf16_bits_to_f32(gw[1] >> 16));
					} else if(p.gate) {  // out *= sigmoid(gate): this row's four consecutive head columns, fetched into LDS at the start
						const u32x2 gw = *reinterpret_cast<const u32x2*>(gate_lds + n * (DP * 2) + d0 * 2);
						o0 *= sigmoidf_fast(bf16_bits_to_f32(gw[0] & 0xffffu)), o1 *= sigmoidf_fast(bf16_bits_to_f32(gw[0] >> 16));
						o2 *= sigmoidf_fast(bf16_bits_to_f32(gw[1] & 0xffffu)), o3 *= sigmoidf_fast(bf16_bits_to_f32(gw[1] >> 16));
					}
					if(p.out_dtype == AF3_BF16) {
						u32x2 w = {pack_bf16x2(o0, o1), pack_bf16x2(o2, o3)};
						*reinterpret_cast<u32x2*>(static_cast<uint16_t*>(p.out) + ooff + d0) = w;
					} else {
						float4 w = {o0, o1, o2, o3};
						*reinterpret_cast<float4*>(static_cast<float*>(p.out) + ooff + d0) = w;
					}
				}
		}
		if constexpr(FUSED) {  // q and gate of this wavefront's next block
			if(qb_f - NW == qb_next) {  // (wave-uniform) already projected
#pragma unroll
				for(int c = 0; c < NC; c++) qf[c] = q_next[c];
				gate_pk[0] = gate_next[0], gate_pk[1] = gate_next[1];
			} else if(qb_f - NW >= 0) {
				u32x4 xf[NS];
				load_x_frags((qb_f - NW) * 32 + n, xf);
				project_q_gate(xf);
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
	// buffer addressing of one (batch, head) slab uses 32-bit byte offsets
	if(p.L * p.k_stride[2] * 2 >= 0x7fffffffLL || p.L * p.v_stride[2] * 2 >= 0x7fffffffLL) return false;
	if(p.gate && (!aligned16(p.gate) || p.gate_stride[0] % 8 || p.gate_stride[1] % 8 || p.gate_stride[2] % 8 || p.L * p.gate_stride[2] * 2 >= 0x7fffffffLL)) return false;
	if(p.out_dtype == AF3_BF16) {
		if((reinterpret_cast<uintptr_t>(p.out) & 7) || p.out_stride[0] % 4 || p.out_stride[1] % 4 || p.out_stride[2] % 4) return false;
	} else {
		if(!aligned16(p.out) || p.out_stride[0] % 4 || p.out_stride[1] % 4 || p.out_stride[2] % 4) return false;
	}
	return true;
}

static int64_t ws_bytes_needed(const af3_dpa_params& p) {
	const int64_t n_qblocks = (p.L + 31) / 32, n_ktiles = (p.L + KT - 1) / KT;
	return p.H * n_qblocks * n_ktiles * 256 * 16;
}

// Whether the call goes to the kernel of dpa_mfma_rows.hip (four batch rows per wavefront sharing each bias tile): its
// shape limits, enough workgroups of four-row groups to give every compute unit one (smaller launches through its workspace
// do better with this file's variants: 16 x 4 x 768 x 32 26 us here against 32 us there) or fewer than 128 batch rows whose
// bias it can stage in place, and the caller's hint (af3_dpa_params.reserved: 1 = take it whenever the shape allows, 2 = never).
static bool rows_kernel_wanted(const af3_dpa_params& p) {
	if(p.reserved == 2 || !mfma_rows_eligible(p)) return false;
	if(p.reserved == 1) return true;
	if((p.B / 4) * p.H * ((p.L + 127) / 128) >= 256) return true;  // (workgroups of the launch that takes the groups of four rows)
	return mfma_rows_suits_a_small_batch(p);
}

// The rewrite costs one extra pass over the bias; it pays off as soon as two batch rows share it.
int64_t mfma_bf16_workspace_bytes(const af3_dpa_params& p) {
	if(!mfma_bf16_eligible(p) || !p.bias || p.B < 2) return 0;
	if(rows_kernel_wanted(p)) return mfma_rows_workspace_bytes(p);
	return ws_bytes_needed(p);
}

// bias -> fp16(bias * log2 e) in fragment order, into p.workspace
static int launch_bias_prepass(const af3_dpa_params& p, hipStream_t s) {
	const bool     bf32      = p.bias_dtype == AF3_F32;
	const int      n_qblocks = (int)((p.L + 31) / 32), n_ktiles = (int)((p.L + KT - 1) / KT);
	const int64_t  total     = p.H * n_qblocks * (int64_t)n_ktiles * 256;
	if(total / 256 >= ((int64_t)1 << 31)) return AF3_ERR_BAD_SHAPE;  // (the prepass counts its units in 32 bits)
	const unsigned g         = (unsigned)((total + 255) / 256 > 65536 ? 65536 : (total + 255) / 256);
	const bool     vec_ok    = ((reinterpret_cast<uintptr_t>(p.bias) & 15) == 0) && (p.bias_stride[0] % 8 == 0) && (p.bias_stride[1] % 8 == 0);
	if(bf32)
		hipLaunchKernelGGL(bias_prepass_kernel<true>, dim3(g), dim3(256), 0, s, p.bias, static_cast<u32x4*>(p.workspace), p.H, p.L, p.bias_stride[0], p.bias_stride[1], n_qblocks,
						   n_ktiles, vec_ok);
	else
		hipLaunchKernelGGL(bias_prepass_kernel<false>, dim3(g), dim3(256), 0, s, p.bias, static_cast<u32x4*>(p.workspace), p.H, p.L, p.bias_stride[0], p.bias_stride[1], n_qblocks,
						   n_ktiles, vec_ok);
	return launch_status();
}

constexpr size_t LDS_LIMIT = 160 * 1024;  // per workgroup on gfx950

// dynamic LDS of one variant: K/V buffers, bias ring, mask table, tile list, gate rows of every wavefront that writes results
template <int DP, int NW, int BMODE, bool SPLIT, int KSL = 0>
static size_t lds_bytes(const af3_dpa_params& p) {
	const size_t n_ktiles = (size_t)((p.L + KT - 1) / KT);
	constexpr bool   KS2  = KSL == 1;
	const size_t writers  = SPLIT ? 1 : KS2 ? NW / 2 : NW;  // wavefronts that own a block of query rows
	constexpr size_t NBUF = KSL == 1 ? 5 : KSL ? 4 : 3;  // (as in the kernel)
	return (size_t)(SPLIT ? NW : 1) * 2 * NBUF * KT * DP * 2 + (BMODE == 2 ? (KS2 ? NW / 2 : NW) * NBUF * 4096 : 0) + (n_ktiles * KT + 64) * 4 + n_ktiles * 2 + 16 +
		   (p.gate ? writers * 32 * DP * 2 : 0);
}

template <int DP, int NW, bool L2DOM, int BMODE, bool SPLIT = false, int KSL = 0>
static int launch_one(const af3_dpa_params& p, hipStream_t s) {
	constexpr int QT       = SPLIT ? 32 : KSL == 1 ? NW * 16 : NW * 32;
	const int     n_qtiles = (int)((p.L + QT - 1) / QT);
	const int64_t n_groups = p.B * p.H;
	const int64_t blocks   = ((n_groups + 7) / 8) * 8 * n_qtiles;
	if(blocks <= 0 || blocks > 0x7fffffffLL) return AF3_ERR_BAD_SHAPE;
	const size_t smem = lds_bytes<DP, NW, BMODE, SPLIT, KSL>(p);
	if(smem > LDS_LIMIT) return AF3_ERR_BAD_SHAPE;  // (launch_nw only picks variants that fit)
	auto         kern = dpa_mfma_bf16_kernel<DP, NW, L2DOM, BMODE, SPLIT, false, KSL>;
	if(smem > 64 * 1024) {  // beyond the default dynamic-LDS limit: raise it for this kernel (idempotent, host side)
		if(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) return AF3_ERR_LAUNCH;
	}
	hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3((NW + (KSL ? 4 : 0)) * 64), smem, s, p, n_qtiles, n_groups, fused_grid_args{});  // (plus the four loader wavefronts)
	return launch_status();
}

// ---- fused grid attention: projections + attention + gate in one kernel ----
constexpr int64_t FUSED_LDS_LIMIT = 160 * 1024;
static size_t fused_lds_bytes(int64_t L) {
	const int64_t n_ktiles = (L + KT - 1) / KT;
	return (size_t)(2 * n_ktiles * KT * 32 * 2 + 2 * 8 * 1024 + (n_ktiles * KT + 64) * 4 + n_ktiles * 2 + 16);
}

bool grid_fused_eligible(const af3_grid_attention_params& g) {
	if(g.dtype != AF3_BF16 || g.C != 128 || g.head != 4) return false;  // AlphaFold 3's pair stack: 128 channels, 4 heads of 32
	if(g.N > MAX_L_MFMA || (int64_t)fused_lds_bytes(g.N) > FUSED_LDS_LIMIT) return false;
	if(!aligned16(g.pair) || g.pair_stride[0] % 8 || g.pair_stride[1] % 8 || g.pair_stride[1] < g.C) return false;
	if(g.N * g.pair_stride[1] * 2 >= 0x7fffffffLL) return false;
	for(const void* w : {g.q_proj, g.k_proj, g.v_proj, g.gating_query})
		if(!w || (reinterpret_cast<uintptr_t>(w) & 3)) return false;
	if((reinterpret_cast<uintptr_t>(g.out) & 7) || g.out_stride[0] % 4 || g.out_stride[1] % 4 || g.out_stride[1] < g.C) return false;
	if(g.bias && g.bias_dtype != AF3_BF16 && g.bias_dtype != AF3_F32) return false;
	return true;
}

static af3_dpa_params grid_as_dpa(const af3_grid_attention_params& g) {
	af3_dpa_params p{};
	p.B = g.B, p.H = g.head, p.L = g.N, p.D = g.C / g.head;
	p.bias = g.bias, p.bias_stride[0] = g.bias_stride[0], p.bias_stride[1] = g.bias_stride[1], p.bias_dtype = g.bias_dtype;
	p.key_mask = g.key_mask, p.key_mask_stride_b = g.key_mask_stride_b;
	p.out = g.out, p.out_stride[0] = g.out_stride[0], p.out_stride[1] = p.D, p.out_stride[2] = g.out_stride[1];
	p.io_dtype = p.out_dtype = p.mma_dtype = AF3_BF16;
	p.softmax_scale = 1.f / sqrtf((float)p.D);
	p.q_descale = p.k_descale = p.v_descale = 1.f;
	p.workspace = g.workspace, p.workspace_bytes = g.workspace_bytes;
	return p;
}

int64_t grid_fused_workspace_bytes(const af3_grid_attention_params& g) {
	if(!grid_fused_eligible(g) || !g.bias) return 0;
	return ws_bytes_needed(grid_as_dpa(g));
}

template <int NW>
static int launch_fused_nw(const af3_dpa_params& p, const fused_grid_args& fa, hipStream_t s) {
	const int64_t n_groups = p.B * p.H;
	const int64_t blocks   = 16 * ((p.B + 3) / 4);  // see the kernel's workgroup -> (batch row, head) map
	if(blocks <= 0 || blocks > 0x7fffffffLL) return AF3_ERR_BAD_SHAPE;
	const size_t smem = fused_lds_bytes(p.L);
	auto         kern = dpa_mfma_bf16_kernel<32, NW, true, 0, false, true, 0>;
	if(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) return AF3_ERR_LAUNCH;
	hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(NW * 64), smem, s, p, 1, n_groups, fa);
	return launch_status();
}

int launch_grid_fused(const af3_grid_attention_params& g, hipStream_t s) {
	af3_dpa_params p = grid_as_dpa(g);
	if(p.bias) {
		if(!p.workspace || p.workspace_bytes < ws_bytes_needed(p) || (reinterpret_cast<uintptr_t>(p.workspace) & 15)) return AF3_ERR_BAD_ARGUMENT;
		const int rc = launch_bias_prepass(p, s);
		if(rc != AF3_OK) return rc;
	}
	fused_grid_args fa{};
	fa.x = static_cast<const uint16_t*>(g.pair), fa.x_stride_b = g.pair_stride[0], fa.x_stride_n = g.pair_stride[1];
	fa.wq = g.q_proj, fa.wk = g.k_proj, fa.wv = g.v_proj, fa.wg = g.gating_query;
	// wavefronts per workgroup: 12 (three per SIMD) unless 8 leaves fewer of them idle in the last round of query blocks
	const int n_qblocks = (int)((p.L + 31) / 32);
	const int best      = ((n_qblocks + 7) / 8) * 8 < ((n_qblocks + 11) / 12) * 12 ? 8 : 12;
	// short rows: three 4-wave workgroups per compute unit instead of one large one, so that one workgroup's projection of
	// K and V overlaps the others' attention (measured at N = 256: 41.6 against 47.4 us)
	if(fused_lds_bytes(p.L) * 3 <= (size_t)FUSED_LDS_LIMIT && n_qblocks % 4 == 0) return launch_fused_nw<4>(p, fa, s);
	return best == 12 ? launch_fused_nw<12>(p, fa, s) : launch_fused_nw<8>(p, fa, s);
}

template <int DP, bool L2DOM, int BMODE>
static int launch_nw(const af3_dpa_params& p, hipStream_t s) {
	// the largest workgroup that still gives the 256 CUs a few workgroups each
	const int64_t groups = p.B * p.H;
	if(groups * ((p.L + 127) / 128) >= 768) return launch_one<DP, 4, L2DOM, BMODE>(p, s);
	if(L2DOM && groups * ((p.L + 63) / 64) >= 768) return launch_one<DP, 2, L2DOM, BMODE>(p, s);
	// Small launches: one 32-row block per workgroup, its key tiles split over 2 or 4 wavefronts so that
	// more of the 1024 SIMDs have work.  The private LDS buffers limit a compute unit to one 4-wave or
	// three 2-wave workgroups, so each split is only taken while the whole grid is resident at once
	// (measured: beyond that the second round of workgroups costs more than the split gains).
	const int64_t blocks1 = groups * ((p.L + 31) / 32), ktiles = (p.L + KT - 1) / KT;
	if(!L2DOM) {
		// In-place bias (one batch row): every single-wave workgroup would re-read the whole K and V of
		// its head from L2, which then outweighs the bias stream; from 512 query blocks on, four blocks
		// share each K/V tile instead (measured, B=1 H=16 D=24: L=1536 25.6 us against 32.7 us with
		// single-wave workgroups; L=768 14.0 us split in two against 14.3 / 17.8; L=384 8.5 us split in four).
		// Long rows with too few 128-row workgroups to fill the 256 compute units: pairs of wavefronts share a query block and
		// the workgroup's K/V tiles.  The work per SIMD is unchanged -- two wavefronts of half the length instead of one -- but
		// the two overlap their matrix and vector phases, and four more wavefronts issue the workgroup's loads (measured,
		// B=1 H=16 L=1536: 22.0 against 31.1 us at head_dim 24; at head_dim 48, padded to 64, the pairing gained nothing, so
		// that size keeps one wavefront per query block).  With 256..511 query blocks the same pairing in workgroups of
		// four compute wavefronts gives every compute unit at most one workgroup of uniform length, where 2-wave
		// workgroups with private tiles put two on half of the compute units and fetch every tile twice as often
		// (measured, B=1 H=16 L=768 D=24: 11.2 against 12.8 us; with 192 blocks, L=384, the four-way split of private
		// tiles stays ahead: 7.5 against 8.4 us, and with 768 blocks eight compute wavefronts per workgroup: 22.0 against 29.9).
		if constexpr(DP == 32) {
			if(blocks1 >= 512 && blocks1 <= 1024 && ktiles >= 8) return launch_one<DP, 8, L2DOM, BMODE, false, true>(p, s);
			if(blocks1 >= 256 && blocks1 < 512 && ktiles >= 8) return launch_one<DP, 4, L2DOM, BMODE, false, true>(p, s);
		}
		// One wavefront per query block, too few 128-row workgroups to give a compute unit more than one: the four loading
		// wavefronts again (measured, B=1 H=16 L=1536 D=48: 27.0 against 31.0 us).
		if(blocks1 >= 512 && blocks1 <= 1024 && lds_bytes<DP, 4, BMODE, false, 2>(p) <= LDS_LIMIT) return launch_one<DP, 4, L2DOM, BMODE, false, 2>(p, s);
		if(blocks1 >= 512) return launch_one<DP, 4, L2DOM, BMODE>(p, s);
		// (the split variants' private buffers plus a long row's mask table can exceed the LDS of a compute unit: then the next one)
		if(DP == 32 && ktiles >= 4 && blocks1 <= 256 && lds_bytes<DP, 4, BMODE, true>(p) <= LDS_LIMIT) return launch_one<DP, 4, L2DOM, BMODE, true>(p, s);
		if(ktiles >= 2 && lds_bytes<DP, 2, BMODE, true>(p) <= LDS_LIMIT) return launch_one<DP, 2, L2DOM, BMODE, true>(p, s);
		return launch_one<DP, 1, L2DOM, BMODE>(p, s);
	}
	if(DP == 32 && ktiles >= 4 && blocks1 <= 256 && lds_bytes<DP, 4, BMODE, true>(p) <= LDS_LIMIT) return launch_one<DP, 4, L2DOM, BMODE, true>(p, s);
	if(ktiles >= 2 && blocks1 <= 768 && lds_bytes<DP, 2, BMODE, true>(p) <= LDS_LIMIT) return launch_one<DP, 2, L2DOM, BMODE, true>(p, s);
	return launch_one<DP, 1, L2DOM, BMODE>(p, s);
}

int launch_dpa_mfma_bf16(const af3_dpa_params& p, hipStream_t s) {
	if(rows_kernel_wanted(p) && mfma_rows_can_serve(p)) return launch_dpa_mfma_rows(p, s);
	const bool bf32   = p.bias && p.bias_dtype == AF3_F32;
	const bool use_ws = p.bias && p.workspace && mfma_bf16_workspace_bytes(p) > 0 && p.workspace_bytes >= ws_bytes_needed(p) &&
						(reinterpret_cast<uintptr_t>(p.workspace) & 15) == 0;
	if(use_ws) {
		const int rc = launch_bias_prepass(p, s);
		if(rc != AF3_OK) return rc;
	}
	const bool l2dom = use_ws || !p.bias;
	// in-place bf16 bias: through the LDS ring when its rows can be fetched in aligned 16-byte chunks that
	// never straddle the end of a row's L valid entries, element-wise otherwise
	const bool ring = !l2dom && !bf32 && ((reinterpret_cast<uintptr_t>(p.bias) & 15) == 0) && (p.bias_stride[0] % 8 == 0) && (p.bias_stride[1] % 8 == 0) && (p.L % 8 == 0) &&
					  ((p.L - 1) * p.bias_stride[1] + p.L) * 2 < (int64_t)1 << 31;
	if(p.D <= 32) {
		if(l2dom) return launch_nw<32, true, 0>(p, s);
		return bf32 ? launch_nw<32, false, 1>(p, s) : ring ? launch_nw<32, false, 2>(p, s) : launch_nw<32, false, 0>(p, s);
	}
	if(l2dom) return launch_nw<64, true, 0>(p, s);
	return bf32 ? launch_nw<64, false, 1>(p, s) : ring ? launch_nw<64, false, 2>(p, s) : launch_nw<64, false, 0>(p, s);
}

}  // namespace af3
