// Device helpers shared by the bf16 matrix-core attention kernels (dpa_mfma.hip, dpa_mfma_rows.hip).
#pragma once
#include <type_traits>

#include "common.hpp"

namespace af3 {

constexpr int   KT         = 64;       // keys per tile (dpa_mfma.hip)
constexpr int   MAX_L_MFMA = 8192;     // mask table (4 B/key) and tile list live in LDS
constexpr float REF_SLACK  = 12.f;     // log2 units: a moved reference sits this close to the row maximum
constexpr float PSUM_LIMIT = 0x1p30f;  // per-lane row-sum bound that triggers the rare path

typedef __attribute__((ext_vector_type(2))) __bf16   bf16x2;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
template <int V>
using ic = std::integral_constant<int, V>;

// ---- LDS layout -----------------------------------------------------------------------------
// K tile: [KT rows][DP cols] bf16; the 16-byte chunks of a row are XOR-swizzled so that the 8
// lanes served in one LDS cycle of a ds_read_b128 (8 consecutive rows, same logical chunk) hit
// distinct banks.  The swizzle only depends on row % 8.
template <int DP>
__device__ __forceinline__ int k_swizzle(int row) {
	return (DP == 32) ? ((row >> 1) & 3) : (row & 7);
}
// V tile: [KT rows][DP cols] bf16 row-major; for DP = 64 the two 64-byte halves of a row are
// swapped on odd rows (keeps the transposed reads of 8 rows x 64 B spread over all banks).
template <int DP>
__device__ __forceinline__ int v_swizzle(int row) {  // in 16-byte chunks
	return (DP == 64) ? ((row & 1) << 2) : 0;
}

__device__ __forceinline__ float half_swap_max(float x) {
	// lanes l and l^32 exchange; v_permlane32_swap swaps the upper half of one operand with the
	// lower half of the other, so (x, x) yields {low|low} and {high|high}.
	auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
	return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// 16 bytes per lane from a raw buffer straight into LDS (lane i lands at lds_addr + 16*i).  Written as
// inline assembly on purpose: the compiler makes every LDS read that follows an LDS-direct load it
// knows about wait for vmcnt(0), which exposes the whole latency of every tile load when only one or
// two wavefronts share a SIMD.  Loads issued here are invisible to it; the kernel orders them itself
// (explicit s_waitcnt vmcnt before the barrier that publishes a tile).  rsrc and lds_addr must be
// wave-uniform.  The whole byte offset travels in the vector operand, which the hardware range-checks
// against the buffer size: a lane whose offset is past the end fetches nothing from memory.
// M0 (the LDS base of the load) is written behind the compiler's back.  It cannot be declared: the compiler treats
// M0 as a reserved register and answers an "m0" clobber with a warning that it is ignored.  What keeps this safe is
// that nothing else in this file makes the compiler use M0 -- no LDS-direct builtins, no indirect register indexing,
// no message or GWS instructions -- and gfx950's LDS instructions do not read it.
__device__ __forceinline__ void lds_dma_b128(const u32x4& rsrc, uint32_t lds_addr, int voff) {
	asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(lds_addr), "v"(voff), "s"(rsrc) : "memory");
}
__device__ __forceinline__ u32x4 raw_rsrc(const void* base, uint32_t bytes) {
	const uint64_t a = reinterpret_cast<uint64_t>(base);
	return u32x4{(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a), (uint32_t)__builtin_amdgcn_readfirstlane((int)((uint32_t)(a >> 32) & 0xFFFFu)),
				 (uint32_t)__builtin_amdgcn_readfirstlane((int)bytes), 0x00020000u};
}
__device__ __forceinline__ uint32_t lds_addr_of(const void* ptr) {
	return (uint32_t)(uintptr_t)((__attribute__((address_space(3))) const void*)ptr);
}

}  // namespace af3
