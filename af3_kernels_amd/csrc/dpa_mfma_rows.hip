// bf16 matrix-core attention kernel for batched calls whose batch rows share one bias (triangle / grid attention):
// out[b] = softmax(q[b].k[b]^T*scale + bias, mask[b]).v[b] with bias [H, L, L] common to all b.
//
// The reference walks (batch, head, query tile) tasks and re-reads the bias tile for every batch row
// (src/csrc/dot_product_attention.cpp:88-110).  Here a wavefront owns one block of 32 query rows of one head for FOUR
// batch rows at once and walks the key axis once for all four: a 32 x 32 bias tile is loaded once, as fp32 already
// laid out like the matrix core's accumulator, and is the C operand of the first K.Q^T instruction of each of the
// four rows -- the bias add costs no instruction at all and a quarter of the loads.  The four rows are four
// independent dependence chains: while the vector ALU exponentiates the logits of one row, the matrix pipe computes
// the logits of the next row and the P.V product of the previous one.
//
// Per 32 x 32 block of logits: 2 MFMA K.Q^T (+ bias through C), 1 MFMA key mask and softmax reference, 2 MFMA
// V^T.P^T, 2 half-size MFMA row sums; 16 v_exp_f32 and 8 v_cvt_pk_bf16_f32 -- the arithmetic of dpa_mfma.hip's log2
// variant (same transposed layout, same optimistic softmax reference, same mask constants) without its two bias
// MFMAs.
//
// Work split.  Workgroup = NW wavefronts = NW blocks of 32 query rows of one (group of 4 batch rows, head).  K and V
// tiles (32 keys x 4 batch rows) are staged in LDS by loads that write LDS directly, four buffers deep, and shared
// by the NW wavefronts; one workgroup barrier per tile, i.e. per four blocks of logits of every wavefront.
#include "mfma_helpers.hpp"

namespace af3 {

namespace {

constexpr int KT_R   = 32;                 // keys per tile
constexpr int NBUF_R = 3;                  // tile buffers
constexpr int TILE_R = KT_R * 32 * 2;      // bytes of one tensor's tile of one batch row (head_dim padded to 32)
constexpr int MAX_L_ROWS = 4096;           // mask table: 8 bytes per key for the four rows
constexpr float BIAS_FLOOR = -0x1p17f;     // lowest value the rewritten bias holds (log2 units)

// ---- bias prepass ---------------------------------------------------------------------------------------------------
// Workspace layout: [H][query block of 32][key tile of 32][load 4][lane 64] x 16 bytes = the accumulator layout of
// v_mfma_f32_32x32x16: lane (q = lane%32, g = lane/32), register 4*ld + e  <->  key 32*t + 8*ld + 4*g + e.
// Values are fp32 bias * log2 e; zero outside the L x L corner; -inf, NaN and anything below -2^17 become -2^17: such an
// entry still gets weight exactly 0 beside any ordinary logit, a row made of nothing else still comes out uniform, and a
// softmax reference that starts there (a row whose first keys are all masked through the bias) leaves the logits that
// follow their fp32 precision to within 2^-6.
template <bool BIAS_F32>
__global__ void __launch_bounds__(256) bias_rows_prepass_kernel(const void* __restrict__ bias, f32x4* __restrict__ ws, int64_t H, int64_t L, int64_t stride_h, int64_t stride_q,
																  int n_qblocks, int n_tiles, bool vec_ok) {
	// one workgroup per (head, query block, key tile) and trip: the index arithmetic (divisions) is per workgroup, on the
	// scalar unit, not per thread; the launcher keeps the number of units below 2^31
	const uint32_t units = (uint32_t)(H * n_qblocks * (int64_t)n_tiles);
	const int      lane = threadIdx.x & 63, ld = threadIdx.x >> 6;
	for(uint32_t u = blockIdx.x; u < units; u += gridDim.x) {
		const int64_t  i  = (int64_t)u * 256 + threadIdx.x;
		const int      t  = (int)(u % (uint32_t)n_tiles);
		const uint32_t t2 = u / (uint32_t)n_tiles;
		const int      qb = (int)(t2 % (uint32_t)n_qblocks);
		const int64_t  h  = t2 / (uint32_t)n_qblocks;
		const int64_t row  = (int64_t)qb * 32 + (lane & 31);
		const int64_t key  = (int64_t)t * KT_R + 8 * ld + 4 * (lane >> 5);
		float         f[4] = {0.f, 0.f, 0.f, 0.f};
		if(row < L) {
			const int64_t off = h * stride_h + row * stride_q + key;
			if(BIAS_F32) {
				const float* bp = static_cast<const float*>(bias) + off;
				if(vec_ok && key + 4 <= L) {
					const f32x4 raw = *reinterpret_cast<const f32x4*>(bp);
					f[0] = raw[0], f[1] = raw[1], f[2] = raw[2], f[3] = raw[3];
				} else {
#pragma unroll
					for(int e = 0; e < 4; e++)
						if(key + e < L) f[e] = bp[e];
				}
			} else {
				const uint16_t* bp = static_cast<const uint16_t*>(bias) + off;
				if(vec_ok && key + 4 <= L) {
					const u32x2 raw = *reinterpret_cast<const u32x2*>(bp);
					f[0] = bf16_bits_to_f32(raw[0] & 0xffffu), f[1] = bf16_bits_to_f32(raw[0] >> 16);
					f[2] = bf16_bits_to_f32(raw[1] & 0xffffu), f[3] = bf16_bits_to_f32(raw[1] >> 16);
				} else {
#pragma unroll
					for(int e = 0; e < 4; e++)
						if(key + e < L) f[e] = bf16_bits_to_f32(bp[e]);
				}
			}
		}
		f32x4 o;
#pragma unroll
		for(int e = 0; e < 4; e++) o[e] = fmaxf(f[e] * LOG2E, BIAS_FLOOR);  // (fmaxf returns the other operand for NaN)
		ws[i] = o;
	}
}

// ROWS: batch rows per wavefront (2, 3 or 4); a workgroup is always four wavefronts = 128 query rows, and wavefront w < ROWS
// fetches the K and V tiles of batch row w.
// BMODE: 0 = no bias (C operand zero); 1 = bias from the rewritten fp32 workspace, one 4 KB fragment per tile through this
// wavefront's LDS slot; 2 = bf16 bias read in place (no workspace: for batches too small to pay for the rewrite), four
// 8-byte loads per lane and tile, converted to the accumulator layout in registers; 3 = bf16 bias read in place through LDS: the
// 32 x 32 tile of this wavefront's query block travels as two 1 KB loads of whole 64-byte row segments straight into one of
// two 2 KB halves of the wavefront's slot, a tile ahead of its conversion (needs 16-byte aligned rows; a quarter of mode
// 2's cache-line requests, whose lanes each fetch from a row of their own).
// The launch covers batch rows [b_first, b_first + b_count) in groups of ROWS.
template <int ROWS, int BMODE>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) dpa_rows_bf16_kernel(af3_dpa_params p, int n_qtiles, int64_t n_groups, int64_t b_first, int64_t b_count) {
	static_assert(ROWS >= 2 && ROWS <= 4, "two to four row chains per wavefront");
	constexpr int  NW       = 4;
	constexpr bool HAS_BIAS = BMODE != 0, SLOT = BMODE == 1, DIRECT = BMODE == 2, STAGED = BMODE == 3;
	constexpr int  BUF_R    = ROWS * 2 * TILE_R;                    // one buffer: [row][K tile | V tile]
	constexpr int  SLOT_BASE = NBUF_R * BUF_R;                      // per-wavefront bias slots (4 KB each)
	constexpr int  MASK_BASE = SLOT_BASE + (SLOT || STAGED ? NW * 4096 : 0);
	extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
	// [buffer 3][batch row 4][K tile 2 KB | V tile 2 KB] [bias slot 4 KB per wavefront] [mask table: (tiles + 1) x 4 rows x 32 keys, bf16 bits]
	const int64_t L        = p.L;
	const int     D        = (int)p.D;
	const int     n_t_all  = (int)((L + KT_R - 1) / KT_R);
	uint16_t* const mask_tab = reinterpret_cast<uint16_t*>(smem + MASK_BASE);
	__shared__ int  s_last[4];  // index of the last live key + 1 of each batch row (0: every key dropped)
	__shared__ int  s_first[4]; // index of the first key tile of each batch row that holds a live key

	// ---- workgroup -> (group of batch rows, head, query tile): all query tiles of one (group, head) get ids congruent
	// mod 8, i.e. the same XCD (they share that XCD's L2 copy of K and V), and an XCD only sees heads xcd % H (for H | 8),
	// so its share of the bias workspace stays L2-resident across the whole batch.
	// The kernel arguments that the start of a workgroup needs, requested in one batch (the compiler would fetch the launch
	// counts, wait, test the early exit, and only then request the fields of p, in two more batches: three memory latencies
	// in a row that the wavefronts of a small launch stand through).
	asm volatile("" ::"s"(n_qtiles), "s"(n_groups), "s"(b_first), "s"(b_count), "s"(p.q), "s"(p.k), "s"(p.v), "s"(p.bias), "s"(p.key_mask), "s"(p.workspace), "s"(p.H), "s"(p.L),
				 "s"(p.D), "s"(p.key_mask_stride_b), "s"(p.bias_stride[0]), "s"(p.bias_stride[1]));
	asm volatile("" ::"s"(p.q_stride[0]), "s"(p.q_stride[1]), "s"(p.q_stride[2]), "s"(p.k_stride[0]), "s"(p.k_stride[1]), "s"(p.k_stride[2]), "s"(p.v_stride[0]), "s"(p.v_stride[1]),
				 "s"(p.v_stride[2]));
	const int64_t wg    = blockIdx.x;
	const int     xcd   = (int)(wg & 7);
	const int64_t slot  = wg >> 3;
	const int64_t group = (slot / n_qtiles) * 8 + xcd;
	const int     qtile = (int)(slot % n_qtiles);
	if(group >= n_groups) return;
	const int64_t g = group / p.H, h = group % p.H;
	const int64_t b0 = b_first + g * ROWS, b_end = b_first + b_count;   // (rows past b_end repeat the last one and are not stored)

	const int tid = threadIdx.x, lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int n = lane & 31, half = lane >> 5;

	// ---- zero the tile buffers when a load can leave parts of them unwritten (padded head columns, rows past L):
	// stale LDS contents there must be finite ----
	if(D != 32 || L % KT_R != 0) {
		for(int i = tid; i < NBUF_R * BUF_R / 16; i += NW * 64) reinterpret_cast<u32x4*>(smem)[i] = u32x4{0u, 0u, 0u, 0u};
		__syncthreads();
	}

	if constexpr(STAGED) {  // (chunks past L are never fetched: what the slots hold there must be finite)
		for(int i = tid; i < NW * 4096 / 16; i += NW * 64) reinterpret_cast<u32x4*>(smem + SLOT_BASE)[i] = u32x4{0u, 0u, 0u, 0u};
		__syncthreads();
	}

	// ---- per-lane constants ----
	const int64_t qrow   = (int64_t)qtile * (NW * 32) + wave * 32 + n;
	const bool    row_ok = qrow < L;
	int n_t = 1;   // key tiles to walk: known once the key masks are read; the first tile is always walked

	// ---- tile and bias loaders: loads that write LDS directly (no registers, invisible to the compiler's wait counting;
	// every wait for them below is explicit).  This wavefront fetches K and V of batch row `wave`: four 1 KB pieces per
	// tile (K rows 0-15, 16-31, V rows 0-15, 16-31; lane i -> tile row i/4, 16-byte chunk i%4, K chunks swizzled), and
	// the four 1 KB pieces of its own bias fragment.  Lanes of padded head columns carry an offset beyond the buffer's
	// range: the hardware fetches nothing for them. ----
	const int64_t b_ld   = b0 + wave < b_end ? b0 + wave : b_end - 1;
	const bool    loader = wave < ROWS;  // (wave-uniform)
	const u32x4   k_rsrc = raw_rsrc(static_cast<const uint16_t*>(p.k) + b_ld * p.k_stride[0] + h * p.k_stride[1], (uint32_t)(((L - 1) * p.k_stride[2] + D) * 2));
	const u32x4   v_rsrc = raw_rsrc(static_cast<const uint16_t*>(p.v) + b_ld * p.v_stride[0] + h * p.v_stride[1], (uint32_t)(((L - 1) * p.v_stride[2] + D) * 2));
	const int     ld_row = lane >> 2, ld_pc = lane & 3;
	const int     k_chunk = ld_pc ^ k_swizzle<32>(ld_row);
	const int     k_voff  = k_chunk * 8 < D ? (int)(ld_row * p.k_stride[2] * 2) + k_chunk * 16 : 0x40000000;
	const int     v_voff  = ld_pc * 8 < D ? (int)(ld_row * p.v_stride[2] * 2) + ld_pc * 16 : 0x40000000;
	const int     k_tile_stride = (int)(KT_R * p.k_stride[2] * 2), v_tile_stride = (int)(KT_R * p.v_stride[2] * 2);
	const int     k_pc_stride = (int)(16 * p.k_stride[2] * 2), v_pc_stride = (int)(16 * p.v_stride[2] * 2);
	const uint32_t lds_tiles = lds_addr_of(smem) + wave * (2 * TILE_R);
	auto load_tile_piece = [&](int t, int buf_off, auto pc_c) {
		constexpr int PC = decltype(pc_c)::value;
		if(!loader || t >= n_t) return;   // (no request for a tile the walk stops short of: nothing is in flight when the kernel ends)
		if constexpr(PC == 0) lds_dma_b128(k_rsrc, lds_tiles + buf_off, k_voff + t * k_tile_stride);
		if constexpr(PC == 1) lds_dma_b128(k_rsrc, lds_tiles + buf_off + 1024, k_voff + (t * k_tile_stride + k_pc_stride));
		if constexpr(PC == 2) lds_dma_b128(v_rsrc, lds_tiles + buf_off + TILE_R, v_voff + t * v_tile_stride);
		if constexpr(PC == 3) lds_dma_b128(v_rsrc, lds_tiles + buf_off + TILE_R + 1024, v_voff + (t * v_tile_stride + v_pc_stride));
	};
	auto load_tile = [&](int t, int buf_off) {
		load_tile_piece(t, buf_off, ic<0>{}), load_tile_piece(t, buf_off, ic<1>{}), load_tile_piece(t, buf_off, ic<2>{}), load_tile_piece(t, buf_off, ic<3>{});
	};
	// bias fragment of key tile t: 4 KB of this (head, query block)'s slab of the workspace -> this wavefront's slot
	const int     n_qblocks = (int)((L + 31) / 32);
	const int64_t qb        = (int64_t)qtile * NW + wave;
	const int64_t qbc       = qb < n_qblocks ? qb : n_qblocks - 1;  // (blocks past the end only hold rows >= L)
	const u32x4   ws_rsrc   = raw_rsrc(SLOT ? static_cast<const unsigned char*>(p.workspace) + ((h * n_qblocks + qbc) * n_t_all) * 4096 : nullptr, SLOT ? (uint32_t)(n_t_all * 4096) : 0u);
	const int      ws_voff  = lane * 16;
	const uint32_t lds_slot = lds_addr_of(smem) + SLOT_BASE + wave * 4096;
	auto load_bias_piece = [&](int t, auto pc_c) {
		constexpr int PC = decltype(pc_c)::value;
		if(!SLOT || t >= n_t) return;
		lds_dma_b128(ws_rsrc, lds_slot + PC * 1024, ws_voff + (t * 4096 + PC * 1024));
	};
	auto load_bias = [&](int t) { load_bias_piece(t, ic<0>{}), load_bias_piece(t, ic<1>{}), load_bias_piece(t, ic<2>{}), load_bias_piece(t, ic<3>{}); };
	// direct mode: this lane's four 8-byte pieces of a tile's bias, bias[h][q][32 t + 8 ld + 4 half .. + 3] (bf16), through a
	// range-checked buffer over the head's slab; pieces whose keys lie at or beyond L are sent out of range and read as zero
	[[maybe_unused]] u32x2 braw[4] = {u32x2{0u, 0u}, u32x2{0u, 0u}, u32x2{0u, 0u}, u32x2{0u, 0u}};
	const int64_t qrow_b = qrow < L ? qrow : L - 1;
	const __amdgpu_buffer_rsrc_t bd_rsrc = __builtin_amdgcn_make_buffer_rsrc(
		DIRECT ? const_cast<uint16_t*>(static_cast<const uint16_t*>(p.bias)) + h * p.bias_stride[0] : nullptr, 0, DIRECT ? (int)(((L - 1) * p.bias_stride[1] + L) * 2) : 0, 0x00020000);
	const int bd_voff = (int)((qrow_b * p.bias_stride[1] + 4 * half) * 2);
	// staged mode: lane i of load j fetches 16 bytes of row 16 j + i / 4 of the tile; the chunk it fetches is the one that
	// belongs at its place under the swizzle (chunk c of row r sits at position c ^ ((r >> 2) & 3): the fragment reads of 32
	// rows then spread over the banks).  Rows past L fetch row L - 1; chunks whose keys lie at or beyond L are sent out of
	// range (nothing is fetched: the slot keeps finite data, and those keys carry the out-of-range mask value).
	const u32x4 st_rsrc = raw_rsrc(STAGED ? static_cast<const uint16_t*>(p.bias) + h * p.bias_stride[0] : nullptr, STAGED ? (uint32_t)(((L - 1) * p.bias_stride[1] + L) * 2) : 0u);
	int st_voff[2] = {0, 0};
	int st_key[2]  = {0, 0};  // first key (within a tile) of the chunk this lane fetches
	if constexpr(STAGED) {
#pragma unroll
		for(int j = 0; j < 2; j++) {
			const int     r   = 16 * j + (lane >> 2), c = (lane & 3) ^ ((r >> 2) & 3);
			const int64_t row = (int64_t)qtile * (NW * 32) + wave * 32 + r;
			st_voff[j] = (int)((row < L ? row : L - 1) * p.bias_stride[1] * 2) + c * 16;
			st_key[j]  = c * 8;
		}
	}
	auto load_bias_staged = [&](int t) {
		if(!STAGED || t >= n_t) return;
#pragma unroll
		for(int j = 0; j < 2; j++) lds_dma_b128(st_rsrc, lds_slot + (t & 1) * 2048 + j * 1024, t * KT_R + st_key[j] < L ? st_voff[j] + t * (KT_R * 2) : 0x40000000);
	};
	auto load_bias_direct = [&](int t) {
		if(!DIRECT || t >= n_t) return;
#pragma unroll
		for(int ld = 0; ld < 4; ld++) {
			const bool in = t * KT_R + 8 * ld + 4 * half < L;
			braw[ld] = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(bd_rsrc, in ? bd_voff + ld * 16 : 0x40000000, t * (KT_R * 2), 0));
		}
	};

	// ---- everything the walk needs before its first step is requested here in one go, so that the workgroup pays one
	// memory latency, not a chain of them: the first K and V tiles and the first bias fragment (straight into LDS), the raw
	// q rows, and the key-mask bytes ----
	load_tile(0, 0);
	load_bias(0);
	load_bias_direct(0);
	load_bias_staged(0);
	u32x4 qraw[ROWS][2];
#pragma unroll
	for(int r = 0; r < ROWS; r++) {
		const int64_t   br = b0 + r < b_end ? b0 + r : b_end - 1;
		const uint16_t* qp = static_cast<const uint16_t*>(p.q) + br * p.q_stride[0] + h * p.q_stride[1] + qrow * p.q_stride[2];
#pragma unroll
		for(int c = 0; c < 2; c++) {
			const int d0 = 16 * c + 8 * half;
			qraw[r][c]   = u32x4{0u, 0u, 0u, 0u};
			if(row_ok && d0 < D) qraw[r][c] = *reinterpret_cast<const u32x4*>(qp + d0);
		}
	}

	// ---- key-mask table: entry = additive mask value of (tile, batch row, key) as bf16 bits; wavefront w fills row w.
	// With 4-byte aligned mask rows a lane takes four keys per load and all loads of the row are in flight together. ----
	const int n_keys_tab = (n_t_all + 1) * KT_R;
	if(wave < ROWS) {
		const int      r    = wave;
		const int64_t  br   = b0 + r < b_end ? b0 + r : b_end - 1;
		const uint8_t* keep = p.key_mask ? p.key_mask + br * p.key_mask_stride_b : nullptr;
		int            last = 0, first = -1;   // (first: wave-uniform, from ballots)
		const bool     vec  = !keep || (((reinterpret_cast<uintptr_t>(p.key_mask) | (uintptr_t)p.key_mask_stride_b | (uintptr_t)L) & 3) == 0);
		if(vec) {
			constexpr int MAXC = MAX_L_ROWS / 256 + 1;   // chunks of 256 keys (4 per lane) that cover the table
			uint32_t      mraw[MAXC];
#pragma unroll
			for(int c = 0; c < MAXC; c++) {
				const int key0 = 256 * c + 4 * lane;
				mraw[c]        = 0u;
				if(256 * c < L) mraw[c] = !keep ? 0x01010101u : (key0 < L ? *reinterpret_cast<const uint32_t*>(keep + key0) : 0u);
			}
			auto write_chunks = [&](bool all_live) {
#pragma unroll
				for(int c = 0; c < MAXC; c++) {
					const int key0 = 256 * c + 4 * lane;
					if(256 * c >= n_keys_tab) break;
					uint32_t e[4];
#pragma unroll
					for(int j = 0; j < 4; j++) {
						const bool in   = key0 + j < L;
						const bool live = in && (all_live || ((mraw[c] >> (8 * j)) & 0xffu) != 0);
						e[j]            = live ? 0u : (in ? (uint32_t)MASK_DROPPED_BF16 : (uint32_t)MASK_OUT_OF_RANGE_BF16);
						if(live && !all_live) last = key0 + j + 1;
					}
					if(key0 < n_keys_tab) *reinterpret_cast<u32x2*>(mask_tab + ((key0 >> 5) * ROWS + r) * 32 + (key0 & 31)) = u32x2{e[0] | (e[1] << 16), e[2] | (e[3] << 16)};
				}
			};
#pragma unroll
			for(int c = MAXC - 1; c >= 0; c--) {   // a lane's four keys of chunk c lie in tile 8 c + lane / 8
				const unsigned long long bal = __ballot(mraw[c] != 0u);   // (chunks at or beyond L hold zeros)
				if(bal) first = 8 * c + (__builtin_ctzll(bal) >> 3);
			}
			write_chunks(false);
#pragma unroll
			for(int off = 32; off >= 1; off >>= 1) {
				const int o = __shfl_xor(last, off);
				last        = o > last ? o : last;
			}
			// A batch row without any live key yields the mean over all L keys (masked_fill(-1e9) + softmax in
			// examples/dot_product_attention.py:37-39): its keys count as live, and q and the bias are dropped for it
			// below, so that all its logits are exactly equal.
			if(last == 0) {
				write_chunks(true);
				last = 0;
			}
		} else {
			for(int base = 0; base < n_keys_tab; base += 64) {
				const int  key  = base + lane;
				const bool in   = key < L;
				const bool live = in && keep[in ? key : 0] != 0;
				if(key < n_keys_tab) mask_tab[((key >> 5) * ROWS + r) * 32 + (key & 31)] = live ? (uint16_t)0 : (in ? MASK_DROPPED_BF16 : MASK_OUT_OF_RANGE_BF16);
				const unsigned long long bal = __ballot(live);
				if(bal) last = base + 64 - __builtin_clzll(bal);
				if(bal && first < 0) first = (base + __builtin_ctzll(bal)) / KT_R;
			}
			if(last == 0)   // (as above)
				for(int key = lane; key < n_keys_tab; key += 64) mask_tab[((key >> 5) * ROWS + r) * 32 + (key & 31)] = key < L ? (uint16_t)0 : MASK_OUT_OF_RANGE_BF16;
		}
		if(lane == 0) s_last[r] = last, s_first[r] = first;
	}
	asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wavefront's pieces of the first tile and its bias fragment have landed
	__syncthreads();                                    // the mask table and the first tile are complete
	// keys behind the last live key of every row carry weight 0 and are not walked; a row without live keys needs them all
	// The softmax reference of a batch row is fixed by the first tile that holds a live key of that row (a tile of dropped
	// keys says nothing about the row's logits): tiles up to the last such tile over the group's rows (normally tile 0 alone)
	// run the variant of the tile code that can do so.
	int  l_eff = 0, t_force_max = 0;
	bool dropped[ROWS];
	uint32_t first_tiles = 0;   // byte r: the first tile of batch row r that holds a live key (at most 128 tiles)
#pragma unroll
	for(int r = 0; r < ROWS; r++) {
		const int last = __builtin_amdgcn_readfirstlane(s_last[r]);
		dropped[r]     = last == 0;
		const int need = dropped[r] ? (int)L : last;
		l_eff          = need > l_eff ? need : l_eff;
		const int ft   = dropped[r] ? 0 : __builtin_amdgcn_readfirstlane(s_first[r]);
		first_tiles |= (uint32_t)ft << (8 * r);
		t_force_max    = ft > t_force_max ? ft : t_force_max;
	}
	n_t = (l_eff + KT_R - 1) / KT_R;

	// Q fragments (B operand of S^T = K.Q^T): lane (q = n, g = half) holds q[q][16c + 8g .. +7], scaled by
	// softmax_scale * log2 e in fp32 and rounded once to bf16 (the reference rounds the scaled q too,
	// src/csrc/dot_product_attention.cpp:95-98).  A batch row without live keys gets q = 0.
	bf16x8 qf[ROWS][2];
#pragma unroll
	for(int r = 0; r < ROWS; r++) {
		const float qmul = dropped[r] ? 0.f : p.softmax_scale * LOG2E;
#pragma unroll
		for(int c = 0; c < 2; c++) {
			u32x4 sc4;
#pragma unroll
			for(int j = 0; j < 4; j++) {
				const uint32_t w = qraw[r][c][j];
				sc4[j] = pack_bf16x2(bf16_bits_to_f32(w & 0xffffu) * qmul, bf16_bits_to_f32(w >> 16) * qmul);
			}
			qf[r][c] = __builtin_bit_cast(bf16x8, sc4);
		}
	}
	// Operands of the mask MFMA (v_mfma_f32_32x32x8_bf16: four contraction slots per half-wave, two registers per operand).
	// A (per key): slot 0 = the key's mask value (from the table, zero-extended), slots 2 and 3 = 1.0.
	// B (per query): slot 0 = 1.0, slots 2 and 3 = -m_hi and -m_lo, the softmax reference of this lane's query row as two
	// bf16 terms (16 significant bits).  Lanes of the upper half-wave supply slots 4..7: their B is zero, so whatever
	// finite value their A holds contributes nothing.
	u32x2 maskA = {0u, 0x3F803F80u};
	u32x2 maskB[ROWS];
#pragma unroll
	for(int r = 0; r < ROWS; r++) maskB[r] = u32x2{half == 0 ? 0x3F80u : 0u, 0u};

	// ---- per-lane LDS read offsets inside a (buffer, batch row) block ----
	int k_rd[2];
#pragma unroll
	for(int c = 0; c < 2; c++) k_rd[c] = n * 64 + (((2 * c + half) ^ k_swizzle<32>(n)) << 4);
	// V^T fragment reads (ds_read_b64_tr_b16): lane l: i = l%16, G = l/16 supplies the 8-byte chunk at tile row
	// base + 4*(G/2) + i/4, column 16*(G%2) + 4*(i%4); it receives 4 keys of column l%32.
	int v_rd;
	{
		const int i16 = lane & 15, G = lane >> 4;
		const int row = 4 * (G >> 1) + (i16 >> 2), col = 16 * (G & 1) + 4 * (i16 & 3);
		v_rd = TILE_R + row * 64 + (col >> 3) * 16 + (col & 7) * 2;
	}
	const int mask_rd = MASK_BASE + n * 2;               // + ((tile * ROWS + row) * 32) * 2
	const int slot_rd = SLOT_BASE + wave * 4096 + lane * 16;  // + 1024 per group of four accumulator registers

	// ---- online-softmax state: one query row per lane and batch row (the two half-waves hold disjoint keys) ----
	float  m_ref[ROWS];   // reference maximum, log2 units, exactly m_hi + m_lo of two bf16 values
	float  lsum[ROWS];    // the row sum (complete: the same value in both half-waves)
	f32x16 oacc[ROWS];
#pragma unroll
	for(int r = 0; r < ROWS; r++) {
		m_ref[r] = 0.f;
		lsum[r]  = 0.f;
#pragma unroll
		for(int i = 0; i < 16; i++) oacc[r][i] = 0.f;
	}

	// Row sums on the matrix pipe (see dpa_mfma.hip): a 16x16x32 MFMA whose A operand is this 0/1 pattern leaves, in
	// register 0 of every lane, the sum of the 16 packed probabilities of that lane's own query row over both half-waves.
	u32x4 ones_a;
	{
		const int      i16 = lane & 15, kg = lane >> 4;
		const bool     on  = ((i16 == 0 || i16 == 8) && (kg & 1) == 0) || ((i16 == 4 || i16 == 12) && (kg & 1) == 1);
		const uint32_t w   = on ? 0x3F803F80u : 0u;
		ones_a = u32x4{w, w, w, w};
	}

	// Move the reference of batch row R for every query whose maximum is not within REF_SLACK of it (all queries when
	// `force`), rescale what has been accumulated and re-express s relative to the new reference.
	auto rereference = [&](auto r_c, f32x16& s, bool force) {
		constexpr int R = decltype(r_c)::value;
		float mx = fmaxf(fmaxf(s[0], s[1]), s[2]);
#pragma unroll
		for(int i = 3; i < 15; i += 2) mx = fmaxf(fmaxf(mx, s[i]), s[i + 1]);
		mx = half_swap_max(fmaxf(mx, s[15]));
		// s already has m_ref subtracted (by the mask MFMA)
		// (forced: the row's first tile with a live key.  Every query then has a logit above the mask constants, the new
		// reference is its maximum, and that key's probability is exactly 1: the row sum can no longer flush to zero however
		// negative the row's biases are.  Tiles in front of it hold dropped keys only: their probabilities are exactly 0
		// against the initial reference 0, and nothing has been accumulated when the reference moves.)
		const bool  need   = (force && mx > -0x1p99f) || mx > REF_SLACK;
		const float m_want = m_ref[R] + mx;
		const float m_hi   = bf16_bits_to_f32(f32_to_bf16_bits(need ? m_want : m_ref[R]));
		const float m_lo   = bf16_bits_to_f32(f32_to_bf16_bits((need ? m_want : m_ref[R]) - m_hi));
		const float m_new  = m_hi + m_lo;  // exactly what the mask MFMA will subtract (unchanged when !need)
		const float delta  = m_new - m_ref[R];
		const float alpha  = force ? 1.f : __builtin_amdgcn_exp2f(-delta);  // nothing is accumulated yet when forced
#pragma unroll
		for(int i = 0; i < 16; i++) s[i] -= delta;
		m_ref[R] = m_new;
		if(half == 0) maskB[R][1] = f32_to_bf16_bits(-m_hi) | (f32_to_bf16_bits(-m_lo) << 16);
		lsum[R] *= alpha;
#pragma unroll
		for(int i = 0; i < 16; i++) oacc[R][i] *= alpha;
	};
	auto exp_part = [&](const f32x16& s, u32x4 (&pf)[2], auto i0_c, auto n_c) {
		constexpr int I0 = decltype(i0_c)::value, N = decltype(n_c)::value;
#pragma unroll
		for(int i = I0; i < I0 + N; i += 2) pf[i >> 3][(i & 7) >> 1] = pack_bf16x2(__builtin_amdgcn_exp2f(s[i]), __builtin_amdgcn_exp2f(s[i + 1]));
	};
	auto read_kfrag = [&](int addr) -> u32x4 { return *reinterpret_cast<const u32x4*>(smem + addr); };
	auto rowsum     = [&](const f32x4& c, const u32x4& pf) -> f32x4 { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, ones_a), __builtin_bit_cast(bf16x8, pf), c, 0, 0, 0); };
	auto mask_mfma  = [&](const f32x16& c, const u32x2& b) -> f32x16 {
		return __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(__builtin_bit_cast(s16x4, maskA), __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
	};

	// Pipeline registers: S^T of the current step, P^T and V^T fragments of the previous one, K fragments of the next
	// one, and the bias fragment of the tile the next step belongs to (accumulator order: the C operand of that step's
	// first K.Q^T instruction).
	f32x16 sc, bias_frag;
	u32x4  kf[2];
	u32x4  pprev[2] = {u32x4{0u, 0u, 0u, 0u}, u32x4{0u, 0u, 0u, 0u}};
	u32x4  vprev[2] = {u32x4{0u, 0u, 0u, 0u}, u32x4{0u, 0u, 0u, 0u}};
#pragma unroll
	for(int i = 0; i < 16; i++) bias_frag[i] = 0.f;
	// the next tile's bias fragment -> registers: from the slot, or (direct mode) from the raw bf16 pieces loaded a tile ago:
	// clamped from below like the workspace's values (packed unsigned minimum: -2^16 and everything beyond it, -inf and
	// -NaN patterns included), widened to fp32 and scaled by log2 e
	auto next_bias_fragment = [&](int t_next) {  // t_next: the tile the fragment belongs to (staged mode: which half of the slot holds it)
		// (The old fragment is named once more behind its last reader: the registers it occupied then are the only free block of
		// 16 when the new one is defined, so the fragment keeps its place from tile to tile.  Without this the compiler lets
		// that reader's result overwrite the old fragment, puts the new one elsewhere and copies 16 registers per tile.)
		asm volatile("" ::"v"(bias_frag));
		if constexpr(SLOT) {
#pragma unroll
			for(int ld = 0; ld < 4; ld++) {
				const f32x4 v = *reinterpret_cast<const f32x4*>(smem + slot_rd + ld * 1024);
				bias_frag[4 * ld] = v[0], bias_frag[4 * ld + 1] = v[1], bias_frag[4 * ld + 2] = v[2], bias_frag[4 * ld + 3] = v[3];
			}
		} else if constexpr(DIRECT || STAGED) {
			typedef __attribute__((ext_vector_type(2))) unsigned short u16x2;
			const u16x2 lim = {(unsigned short)0xC780, (unsigned short)0xC780};
			if constexpr(STAGED) {  // this lane's four 8-byte pieces, keys 8 ld + 4 half .. + 3 of row n: chunk ld at its swizzled place
#pragma unroll
				for(int ld = 0; ld < 4; ld++)
					braw[ld] = *reinterpret_cast<const u32x2*>(smem + SLOT_BASE + wave * 4096 + (t_next & 1) * 2048 + n * 64 + ((ld ^ ((n >> 2) & 3)) << 4) + half * 8);
			}
#pragma unroll
			for(int ld = 0; ld < 4; ld++)
#pragma unroll
				for(int j = 0; j < 2; j++) {
					const uint32_t raw = braw[ld][j];
					const uint32_t w   = __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(u16x2, raw), lim));
					bias_frag[4 * ld + 2 * j]     = __uint_as_float(w << 16) * LOG2E;
					bias_frag[4 * ld + 2 * j + 1] = __uint_as_float(w & 0xffff0000u) * LOG2E;
				}
		}
	};

	// One step = one 32 x 32 block of logits of batch row R.  On entry `sc` holds its finished S^T, `pprev` / `vprev`
	// belong to the previous step (batch row R-1, or row 3 of the previous tile) and `kf` holds the K fragments of the
	// next step.  The step alternates matrix instructions of three independent chains with slices of its vector work
	//     matrix pipe                                            vector ALU
	//     O^T[R-1] += V^T . P^T (previous step, 2 instructions)   exp2 / pack of this step, two logits per slice
	//     S^T of the next step (K.Q^T + bias, mask: 3)
	//     row sum of this step (2 half-size instructions)
	// so that no instruction waits for the one issued just before it, and leaves S^T(next) in `sc`, P^T in `pprev`, this
	// step's V^T fragments in `vprev`, the K fragments of the step after the next in `kf`.
	// k_addr2: LDS byte address of the K tile of the step after the next; m_addr: (per lane) of the next step's mask
	// entries; v_addr: of this step's V tile; hook(i): run behind the i-th matrix instruction of the step (i = 0..4; 1 is the
	// first K.Q^T instruction of the next step).
	// FIRST: a leading tile, in which a row that meets its first live key (`force`, wave-uniform) fixes its softmax reference.  ANYDROP: some batch row of this group has no
	// live key (it then takes no bias: a wave-uniform branch the common instantiation does not carry).
	auto step = [&](auto r_c, auto first_c, auto anydrop_c, bool force, int k_addr2, int m_addr, int v_addr, auto&& hook) {
		constexpr int  R = decltype(r_c)::value, RN = (R + 1) % ROWS, RP = (R + ROWS - 1) % ROWS;
		constexpr bool FIRST = decltype(first_c)::value != 0, ANYDROP = decltype(anydrop_c)::value != 0;
		if constexpr(FIRST) rereference(r_c, sc, force);
		maskA[0] = *reinterpret_cast<const uint16_t*>(smem + m_addr);
		u32x4  pcur[2];
		f32x16 sn;
		f32x4  rs = {0.f, 0.f, 0.f, 0.f};
		// The order below is the order the instructions are meant to issue in: one matrix instruction, then a slice of the
		// vector work, so that consecutive matrix instructions belong to different chains.  Matrix intrinsics are pure
		// values to the compiler and would drift to wherever their consumers are; each slice therefore ends with an empty
		// asm statement that names what the slice produced and the operand the next slice's matrix instruction waits for
		// (asm statements keep their order, and so does everything that feeds or reads them), followed by a scheduling barrier.
#define AF3_PIN2(a, b)                                \
	{                                                 \
		auto pa_ = a;                                 \
		auto pb_ = b;                                 \
		asm volatile("" : "+v"(pa_), "+v"(pb_));      \
		a = pa_, b = pb_;                             \
	}                                                 \
	__builtin_amdgcn_sched_barrier(0)
#define AF3_PIN3(a, b, c)                                        \
	{                                                            \
		auto pa_ = a;                                            \
		auto pb_ = b;                                            \
		auto pc_ = c;                                            \
		asm volatile("" : "+v"(pa_), "+v"(pb_), "+v"(pc_));      \
		a = pa_, b = pb_, c = pc_;                               \
	}                                                            \
	__builtin_amdgcn_sched_barrier(0)
		__builtin_amdgcn_sched_barrier(0);
		oacc[RP] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vprev[0]), __builtin_bit_cast(bf16x8, pprev[0]), oacc[RP], 0, 0, 0);
		hook(ic<0>{});
		exp_part(sc, pcur, ic<0>{}, ic<2>{});
		AF3_PIN3(oacc[RP][0], pcur[0][0], kf[0][0]);
		{
			f32x16 z;
#pragma unroll
			for(int i = 0; i < 16; i++) z[i] = 0.f;
			bool with_bias = HAS_BIAS;
			if constexpr(ANYDROP) with_bias = HAS_BIAS && !dropped[RN];  // (wave-uniform)
			if(with_bias) sn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kf[0]), qf[RN][0], bias_frag, 0, 0, 0);
			else sn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kf[0]), qf[RN][0], z, 0, 0, 0);
		}
		hook(ic<1>{});
		exp_part(sc, pcur, ic<2>{}, ic<2>{});
		AF3_PIN3(sn[0], pcur[0][1], pprev[1][0]);
		oacc[RP] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vprev[1]), __builtin_bit_cast(bf16x8, pprev[1]), oacc[RP], 0, 0, 0);
		// V^T fragments of this step for the next step's P.V, now that the previous ones are consumed
#pragma unroll
		for(int cp = 0; cp < 2; cp++)
#pragma unroll
			for(int t = 0; t < 2; t++) {
				const s16x4 rr = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(smem + v_addr + v_rd + (16 * cp + 8 * t) * 64));
				const u32x2 r2 = __builtin_bit_cast(u32x2, rr);
				vprev[cp][2 * t] = r2[0], vprev[cp][2 * t + 1] = r2[1];
			}
		hook(ic<2>{});
		exp_part(sc, pcur, ic<4>{}, ic<2>{});
		AF3_PIN3(oacc[RP][0], pcur[0][2], kf[1][0]);
		sn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kf[1]), qf[RN][1], sn, 0, 0, 0);
		// K fragments of the step after the next, now that the next step's are consumed
		kf[0] = read_kfrag(k_addr2 + k_rd[0]);
		kf[1] = read_kfrag(k_addr2 + k_rd[1]);
		hook(ic<3>{});
		exp_part(sc, pcur, ic<6>{}, ic<2>{});
		AF3_PIN2(sn[0], pcur[0][3]);
		rs = rowsum(rs, pcur[0]);
		hook(ic<4>{});
		exp_part(sc, pcur, ic<8>{}, ic<4>{});
		AF3_PIN3(rs[0], pcur[1][0], pcur[1][1]);
		{
			uint32_t ma_ = maskA[0];
			asm volatile("" : "+v"(ma_));
			maskA[0] = ma_;
		}
		sn = mask_mfma(sn, maskB[RN]);
		exp_part(sc, pcur, ic<12>{}, ic<4>{});
		AF3_PIN3(sn[0], pcur[1][2], pcur[1][3]);
#undef AF3_PIN2
#undef AF3_PIN3
		rs = rowsum(rs, pcur[1]);
		// This step's sum stays below 32 * 2^REF_SLACK while every probability respects the reference, so the test also
		// catches a single probability near or beyond the limit (inf, NaN).
		if(__ballot(!(rs[0] < PSUM_LIMIT))) {  // rare
			rereference(r_c, sc, false);
			exp_part(sc, pcur, ic<0>{}, ic<16>{});
			rs = rowsum(f32x4{0.f, 0.f, 0.f, 0.f}, pcur[0]);
			rs = rowsum(rs, pcur[1]);
		}
		lsum[R] += rs[0];
		sc       = sn;
		pprev[0] = pcur[0];
		pprev[1] = pcur[1];
	};

	// One tile: ROWS steps.  Tile t sits in buffer t % 3.  In front of the last-but-one step the loads issued one tile
	// earlier (tile t + 1 and its bias fragment: the youngest loads this wavefront has in flight) are awaited and a barrier
	// publishes tile t + 1 -- that step fetches K fragments from it -- and tells that every wavefront is done with tile
	// t - 1, whose buffer tile t + 2 then overwrites.  That step's first matrix instruction is the last reader of bias
	// fragment t: behind it the fragment registers take fragment t + 1, and the slot (once those reads have returned: the
	// last step's first matrix instruction waits for them) or the raw-piece registers are refilled with fragment t + 2.
	auto tile = [&](auto first_c, auto anydrop_c, int t, int buf, int bufn, int bufnn) {
		const int m0 = mask_rd + t * (ROWS * 64);
		auto one = [&](auto r_c) {
			constexpr int R = decltype(r_c)::value;
			if constexpr(R < ROWS) {
				constexpr int R1 = R + 1, R2 = R + 2;                        // the next step and the one after it ...
				const int     k2 = (R2 >= ROWS ? bufn : buf) + (R2 % ROWS) * (2 * TILE_R);   // ... may belong to the next tile
				const int     m1 = m0 + R1 * 64;                             // (row ROWS of tile t is row 0 of tile t + 1)
				const int     vc = buf + R * (2 * TILE_R);
				const bool    fr = decltype(first_c)::value != 0 && t == (int)((first_tiles >> (8 * (R < ROWS ? R : 0))) & 0xffu);
				if constexpr(R == ROWS - 2) {
					asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
					step(r_c, first_c, anydrop_c, fr, k2, m1, vc, [&](auto s_c) {
						constexpr int S = decltype(s_c)::value;
						if constexpr(S == 1) {
							load_tile(t + 2, bufnn);
							next_bias_fragment(t + 1);
							load_bias_direct(t + 2);
							load_bias_staged(t + 2);   // (into the half that held fragment t, read a tile ago)
						}
					});
				} else if constexpr(R == ROWS - 1) {
					step(r_c, first_c, anydrop_c, fr, k2, m1, vc, [&](auto s_c) {
						constexpr int S = decltype(s_c)::value;
						if constexpr(S == 1) load_bias(t + 2);   // (behind this step's first K.Q^T instruction, which has waited for the slot's reads)
					});
				} else {
					step(r_c, first_c, anydrop_c, fr, k2, m1, vc, [](auto) {});
				}
			}
		};
		one(ic<0>{}), one(ic<1>{}), one(ic<2>{}), one(ic<3>{});
	};
	auto run = [&](auto anydrop_c) {
		constexpr bool ANYDROP = decltype(anydrop_c)::value != 0;
		// ---- prologue: the second tile and bias fragment, S^T of the first step, K fragments of the second ----
		// (tile 0 and bias fragment 0 were requested at the top of the kernel and are complete)
		next_bias_fragment(0);  // fragment 0 -> registers
		asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
		load_tile(1, BUF_R);
		load_bias(1);
		load_bias_direct(1);
		load_bias_staged(1);
		{
			f32x16 s0;
#pragma unroll
			for(int i = 0; i < 16; i++) s0[i] = (HAS_BIAS && !(ANYDROP && dropped[0])) ? bias_frag[i] : 0.f;
#pragma unroll
			for(int c = 0; c < 2; c++) s0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, read_kfrag(k_rd[c])), qf[0][c], s0, 0, 0, 0);
			maskA[0] = *reinterpret_cast<const uint16_t*>(smem + mask_rd);
			sc = mask_mfma(s0, maskB[0]);
			kf[0] = read_kfrag(2 * TILE_R + k_rd[0]);
			kf[1] = read_kfrag(2 * TILE_R + k_rd[1]);
		}
		int buf = 0, t = 0;
		for(; t <= t_force_max; t++) {   // (one trip unless some row's leading tiles hold dropped keys only)
			const int bufn = buf == (NBUF_R - 1) * BUF_R ? 0 : buf + BUF_R, bufnn = bufn == (NBUF_R - 1) * BUF_R ? 0 : bufn + BUF_R;
			tile(ic<1>{}, anydrop_c, t, buf, bufn, bufnn);
			buf = bufn;
		}
		for(; t < n_t; t++) {
			const int bufn = buf == (NBUF_R - 1) * BUF_R ? 0 : buf + BUF_R, bufnn = bufn == (NBUF_R - 1) * BUF_R ? 0 : bufn + BUF_R;
			tile(ic<0>{}, anydrop_c, t, buf, bufn, bufnn);
			buf = bufn;
		}
	};
	if(n_t > 0) {
		bool any_dropped = false;
#pragma unroll
		for(int r = 0; r < ROWS; r++) any_dropped = any_dropped || dropped[r];
		if(any_dropped) run(ic<1>{});
		else run(ic<0>{});
	}
	asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no load may still be writing LDS when the workgroup's allocation is released
	// the last step's P.V product (batch row 3)
	oacc[ROWS - 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vprev[0]), __builtin_bit_cast(bf16x8, pprev[0]), oacc[ROWS - 1], 0, 0, 0);
	oacc[ROWS - 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vprev[1]), __builtin_bit_cast(bf16x8, pprev[1]), oacc[ROWS - 1], 0, 0, 0);

	// ---- epilogue: O^T register i is head column 8*(i/4) + 4*half + i%4; optional output gate (out *= sigmoid(gate), the
	// reference's "weighted_avg *= sigmoid(gating_query(pair))", src/csrc/dot_product_attention.cpp:335-349) ----
	if(row_ok) {
#pragma unroll
		for(int r = 0; r < ROWS; r++) {
			if(b0 + r >= b_end) break;
			const float   inv  = 1.f / lsum[r];
			const int64_t ooff = (b0 + r) * p.out_stride[0] + h * p.out_stride[1] + qrow * p.out_stride[2];
			u32x2         gw[4] = {u32x2{0u, 0u}, u32x2{0u, 0u}, u32x2{0u, 0u}, u32x2{0u, 0u}};
			if(p.gate) {
				const uint16_t* gp = static_cast<const uint16_t*>(p.gate) + (b0 + r) * p.gate_stride[0] + h * p.gate_stride[1] + qrow * p.gate_stride[2];
#pragma unroll
				for(int g4 = 0; g4 < 4; g4++)
					if(8 * g4 + 4 * half < D) gw[g4] = *reinterpret_cast<const u32x2*>(gp + 8 * g4 + 4 * half);
			}
#pragma unroll
			for(int g4 = 0; g4 < 4; g4++) {
				const int d0 = 8 * g4 + 4 * half;
				if(d0 >= D) continue;
				float o0 = oacc[r][4 * g4] * inv, o1 = oacc[r][4 * g4 + 1] * inv, o2 = oacc[r][4 * g4 + 2] * inv, o3 = oacc[r][4 * g4 + 3] * inv;
				if(p.gate) {
					const uint32_t g0 = gw[g4][0], g1 = gw[g4][1];
					o0 *= sigmoidf_fast(bf16_bits_to_f32(g0 & 0xffffu)), o1 *= sigmoidf_fast(bf16_bits_to_f32(g0 >> 16));
					o2 *= sigmoidf_fast(bf16_bits_to_f32(g1 & 0xffffu)), o3 *= sigmoidf_fast(bf16_bits_to_f32(g1 >> 16));
				}
				if(p.out_dtype == AF3_BF16) {
					const u32x2 w = {pack_bf16x2(o0, o1), pack_bf16x2(o2, o3)};
					*reinterpret_cast<u32x2*>(static_cast<uint16_t*>(p.out) + ooff + d0) = w;
				} else {
					const float4 w = {o0, o1, o2, o3};
					*reinterpret_cast<float4*>(static_cast<float*>(p.out) + ooff + d0) = w;
				}
			}
		}
	}
}

int64_t rows_ws_bytes(const af3_dpa_params& p) {
	const int64_t n_qblocks = (p.L + 31) / 32, n_t_all = (p.L + KT_R - 1) / KT_R;
	return p.H * n_qblocks * n_t_all * 4096;
}

// The bf16 bias can be read in place when its rows start on 8-byte boundaries, keys come in whole groups of four and the
// slab of one head fits 32-bit byte offsets.
bool direct_bias_ok(const af3_dpa_params& p) {
	return p.bias && p.bias_dtype == AF3_BF16 && p.L % 4 == 0 && (reinterpret_cast<uintptr_t>(p.bias) & 7) == 0 && p.bias_stride[0] % 4 == 0 && p.bias_stride[1] % 4 == 0 &&
		   ((p.L - 1) * p.bias_stride[1] + p.L) * 2 < 0x40000000LL;
}

// ... and through LDS, in whole 16-byte chunks of whole rows, when rows start on 16-byte boundaries and keys come in groups of eight.
bool staged_bias_ok(const af3_dpa_params& p) {
	return direct_bias_ok(p) && p.L % 8 == 0 && (reinterpret_cast<uintptr_t>(p.bias) & 15) == 0 && p.bias_stride[0] % 8 == 0 && p.bias_stride[1] % 8 == 0;
}

// Staging the bf16 bias costs each step 8 vector instructions (widening it) that the fp32 workspace does not -- about 5 % of
// the kernel's time -- the workspace a prepass over the whole bias (about 3 us + 0.46 us per MB read and written) and twice
// the bytes per tile.  Staged / workspace, us, prepass included: 32 x 16 x 1536 x 24 245 / 299, 64 x 4 x 768 x 32 50 / 55,
// 128 x 4 x 768 x 32 90 / 91, 192 x 4 x 768 x 32 117 / 118, 384 x 4 x 384 x 32 60 / 62, 768 x 4 x 768 x 32 425 / 416.
// The prepass is worth its time from about 224 + 2.4e8 / (H L^2) batch rows on (the second term: its fixed cost against the
// time of one batch row).
constexpr int64_t STAGED_MAX_B_SMALL = 128;  // below this the kernel is taken for launches the one-row kernel would otherwise serve
static bool staged_preferred(const af3_dpa_params& p) {
	if(!staged_bias_ok(p)) return false;
	const double x = (double)p.H * (double)p.L * (double)p.L;
	return (double)p.B < 224.0 + 2.44e8 / x;
}

// 0 = no bias, 1 = through the rewritten workspace, 2 = read in place (3: through LDS), -1 = this kernel cannot serve the call.
int rows_bias_mode(const af3_dpa_params& p) {
	if(!p.bias) return 0;
	const bool ws_ok = p.workspace && p.workspace_bytes >= rows_ws_bytes(p) && (reinterpret_cast<uintptr_t>(p.workspace) & 15) == 0;
	if(staged_preferred(p)) return 3;
	if(p.B >= 16 && ws_ok) return 1;
	if(direct_bias_ok(p)) return staged_bias_ok(p) ? 3 : 2;
	return ws_ok ? 1 : -1;
}

template <int ROWS, int BMODE>
int launch_rows(const af3_dpa_params& p, int64_t b_first, int64_t b_count, hipStream_t s) {
	const int     n_qtiles = (int)((p.L + 127) / 128);
	const int64_t n_groups = ((b_count + ROWS - 1) / ROWS) * p.H;
	const int64_t blocks   = ((n_groups + 7) / 8) * 8 * n_qtiles;
	if(blocks <= 0 || blocks > 0x7fffffffLL) return AF3_ERR_BAD_SHAPE;
	const size_t n_t_all = (size_t)((p.L + KT_R - 1) / KT_R);
	const size_t smem    = (size_t)NBUF_R * ROWS * 2 * TILE_R + (BMODE == 1 || BMODE == 3 ? 4 * 4096 : 0) + (n_t_all + 1) * ROWS * 32 * 2;
	auto         kern    = dpa_rows_bf16_kernel<ROWS, BMODE>;
	if(smem > 64 * 1024) {
		if(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) return AF3_ERR_LAUNCH;
	}
	hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), smem, s, p, n_qtiles, n_groups, b_first, b_count);
	return launch_status();
}

template <int BMODE>
int launch_rows_n(int rows, const af3_dpa_params& p, int64_t b_first, int64_t b_count, hipStream_t s) {
	return rows == 4 ? launch_rows<4, BMODE>(p, b_first, b_count, s) : rows == 3 ? launch_rows<3, BMODE>(p, b_first, b_count, s) : launch_rows<2, BMODE>(p, b_first, b_count, s);
}

}  // namespace

// Shapes the kernel takes: what dpa_mfma.hip's kernel takes (mfma_bf16_eligible, checked by the caller), and in addition
// head_dim <= 32, at least two batch rows, a length whose mask table fits beside the tile buffers, 8-byte aligned gate rows.
bool mfma_rows_eligible(const af3_dpa_params& p) {
	if(p.D > 32 || p.B < 2 || p.L > MAX_L_ROWS) return false;
	if(p.gate && ((reinterpret_cast<uintptr_t>(p.gate) & 7) || p.gate_stride[0] % 4 || p.gate_stride[1] % 4 || p.gate_stride[2] % 4)) return false;
	return true;
}

// Workspace the call would use: none when the bias is better read in place (few batch rows).
int64_t mfma_rows_workspace_bytes(const af3_dpa_params& p) {
	if(!p.bias) return 0;
	if(staged_preferred(p) || (p.B < 16 && direct_bias_ok(p))) return 0;
	return rows_ws_bytes(p);
}

bool mfma_rows_can_serve(const af3_dpa_params& p) { return mfma_rows_eligible(p) && rows_bias_mode(p) >= 0; }

// Fewer than 128 batch rows whose bias this kernel can stage in place: the one-row kernel would first rewrite the whole bias
// into its workspace (a pass that so few rows do not amortise) and then stream the rewritten copy once per row; here each
// group of rows streams the original once.  Measured (one-row kernel with its rewrite / this kernel, us): 2 x 16 x 1536 x 24
// 61 / 38, 5 x 16 x 1536 x 24 79 / 67, 12 x 16 x 1536 x 24 139 / 109, 5 x 16 x 768 x 24 32 / 28, 8 x 4 x 2048 x 32 62 / 50,
// 12 x 4 x 384 x 32 21 / 17, 8 x 4 x 768 x 32 21 / 21, 16 x 4 x 768 x 32 26 / 22, 48 x 4 x 768 x 32 45 / 40,
// 16 x 16 x 1536 x 24 172 / 149, 40 x 4 x 384 x 32 22 / 18.  Not for long rows in so few workgroups that most compute units
// would stay empty (2 x 4 x 1536 x 32: 48 workgroups, 30 / 37 us: the one-row kernel splits the key axis of such rows).
bool mfma_rows_suits_a_small_batch(const af3_dpa_params& p) {
	if(!p.bias || p.B >= STAGED_MAX_B_SMALL || !staged_bias_ok(p)) return false;
	const int64_t wgs = ((p.B + 3) / 4) * p.H * ((p.L + 127) / 128);
	return wgs >= 64 || p.L < 1024;
}

int launch_dpa_mfma_rows(const af3_dpa_params& p, hipStream_t s) {
	const int mode = rows_bias_mode(p);
	if(mode < 0) return AF3_ERR_BAD_ARGUMENT;
	if(mode == 1) {
		const bool     bf32      = p.bias_dtype == AF3_F32;
		const int      n_qblocks = (int)((p.L + 31) / 32), n_t_all = (int)((p.L + KT_R - 1) / KT_R);
		const int64_t  total     = p.H * n_qblocks * (int64_t)n_t_all * 256;
		if(total / 256 >= ((int64_t)1 << 31)) return AF3_ERR_BAD_SHAPE;  // (the prepass counts its units in 32 bits)
		const unsigned g         = (unsigned)((total + 255) / 256 > 65536 ? 65536 : (total + 255) / 256);
		const int64_t  esz       = bf32 ? 4 : 2;
		const bool     vec_ok    = ((reinterpret_cast<uintptr_t>(p.bias) & (4 * esz - 1)) == 0) && (p.bias_stride[0] % 4 == 0) && (p.bias_stride[1] % 4 == 0);
		if(bf32)
			hipLaunchKernelGGL(bias_rows_prepass_kernel<true>, dim3(g), dim3(256), 0, s, p.bias, static_cast<f32x4*>(p.workspace), p.H, p.L, p.bias_stride[0], p.bias_stride[1],
							   n_qblocks, n_t_all, vec_ok);
		else
			hipLaunchKernelGGL(bias_rows_prepass_kernel<false>, dim3(g), dim3(256), 0, s, p.bias, static_cast<f32x4*>(p.workspace), p.H, p.L, p.bias_stride[0], p.bias_stride[1],
							   n_qblocks, n_t_all, vec_ok);
		const int rc = launch_status();
		if(rc != AF3_OK) return rc;
	}
	// The batch is cut into groups of `rows` batch rows per wavefront, the remainder into groups of two or three (a
	// remainder of one borrows from the last full group); every group of one launch has the same number of rows.  Four
	// rows share a bias tile best, but what counts is how evenly the workgroups fill the GPU's 512 slots (two per
	// compute unit): the launch time is about (rounds of 512 workgroups) x (rows per group) x (cost per row, which grows
	// as fewer rows share a tile: measured 1 : 1.075 : 1.09 for 4 : 3 : 2 rows), and the cheapest plan is taken.  For a
	// small batch the cheapest plan is often ONE launch whose last group is short (its missing rows repeat the last batch
	// row and are not stored): launches run one after the other, so 3 + 2 rows in two launches of half-empty rounds take
	// the time of five rows, the same five rows as 3 + (2 and a repeated one) in one launch the time of three.
	const int64_t B = p.B, per_row_wgs = p.H * ((p.L + 127) / 128);
	auto plan = [&](int rows, int64_t (&count)[3], int (&rows_of)[3]) -> double {
		static const double cost_per_row[5] = {0, 0, 1.09, 1.075, 1.0};
		int64_t full = B / rows, rem = B % rows;
		int     n    = 0;
		if(rem == 1 && rows > 2) {
			if(full >= 1) full -= 1, rem += rows;  // e.g. 4 + 1 -> 3 + 2
			else return 1e30;
		} else if(rem == 1) {
			return 1e30;  // (rows == 2 and an odd batch: another plan serves it)
		}
		if(full > 0) count[n] = full * rows, rows_of[n] = rows, n++;
		if(rem == 5) count[n] = 3, rows_of[n] = 3, n++, count[n] = 2, rows_of[n] = 2, n++;
		else if(rem == 4) count[n] = 2, rows_of[n] = 2, n++, count[n] = 2, rows_of[n] = 2, n++;   // (rows == 3: 3 + 1 -> 2 + 2)
		else if(rem > 0) count[n] = rem, rows_of[n] = (int)rem, n++;
		for(int i = n; i < 3; i++) count[i] = 0, rows_of[i] = 0;
		double t = 0;
		for(int i = 0; i < n; i++) {
			const int64_t wgs = ((count[i] + rows_of[i] - 1) / rows_of[i]) * per_row_wgs;
			t += (double)((wgs + 511) / 512) * rows_of[i] * cost_per_row[rows_of[i]];
		}
		return t;
	};
	int64_t count[3] = {0, 0, 0};
	int     rows_of[3] = {0, 0, 0};
	double  best = 1e30;
	for(int rows = 4; rows >= 2; rows--) {
		int64_t c[3];
		int     r[3];
		const double t = plan(rows, c, r);
		if(t < best * 0.999) {
			best = t;
			for(int i = 0; i < 3; i++) count[i] = c[i], rows_of[i] = r[i];
		}
		if(B % rows != 0) {   // one launch, last group short
			static const double cost_per_row[5] = {0, 0, 1.09, 1.075, 1.0};
			const int64_t wgs = ((B + rows - 1) / rows) * per_row_wgs;
			const double  t1  = (double)((wgs + 511) / 512) * rows * cost_per_row[rows];
			if(t1 < best * 0.999) {
				best = t1;
				count[0] = B, rows_of[0] = rows;
				count[1] = count[2] = 0, rows_of[1] = rows_of[2] = 0;
			}
		}
	}
	if(best >= 1e30) return AF3_ERR_BAD_SHAPE;  // (B == 1 is not eligible)
	int64_t done = 0;
	for(int i = 0; i < 3; i++) {
		if(count[i] == 0) continue;
		const int rc = mode == 0 ? launch_rows_n<0>(rows_of[i], p, done, count[i], s) : mode == 1 ? launch_rows_n<1>(rows_of[i], p, done, count[i], s) : mode == 2 ? launch_rows_n<2>(rows_of[i], p, done, count[i], s) : launch_rows_n<3>(rows_of[i], p, done, count[i], s);
		if(rc != AF3_OK) return rc;
		done += count[i];
	}
	return AF3_OK;
}

}  // namespace af3
