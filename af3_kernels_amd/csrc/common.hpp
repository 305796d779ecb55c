// Shared declarations for the gfx950 attention library (internal; the public ABI is include/af3_dpa.h).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/af3_dpa.h"

namespace af3 {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;

// Additive key-mask values, exact in bf16 and powers of two so that multiplying them by any fp32
// constant is exact.  A dropped key adds MASK_DROPPED to its logit; a key beyond L adds
// MASK_OUT_OF_RANGE.  |logit| << 2^76, so logit + MASK_DROPPED == MASK_DROPPED in fp32: a row
// whose keys are all dropped sees equal logits on its L real keys and weight 0 on the padding,
// i.e. the mean of V, which is what masked_fill(-1e9) + softmax gives in the reference harness.
constexpr float    MASK_DROPPED            = -0x1p100f;
constexpr float    MASK_OUT_OF_RANGE       = -0x1p120f;
constexpr uint16_t MASK_DROPPED_BF16       = 0xF180;
constexpr uint16_t MASK_OUT_OF_RANGE_BF16  = 0xFB80;
constexpr float    LOG2E                   = 1.4426950408889634f;

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// fp32 -> bf16 bits, round-to-nearest-even (NaN stays NaN).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
	uint32_t u = __float_as_uint(f);
	if((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
	return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
	typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
	bf16x2 p = {(__bf16)lo, (__bf16)hi};  // v_cvt_pk_bf16_f32
	return __builtin_bit_cast(uint32_t, p);
}

// sigmoid for the optional output gate (reference: tpp::SigmoidFwdTPP, src/csrc/xsmm_functors.h:2694-2731)
__device__ __forceinline__ float sigmoidf_fast(float x) { return 1.f / (1.f + __builtin_amdgcn_exp2f(-x * LOG2E)); }

// Extra kernel arguments of the fused grid-attention variant of the bf16 kernel: the input rows and the four
// per-head projection matrices (weight^T in the reference's panel layout [head][C/2][32][2]).
struct fused_grid_args {
	const uint16_t* x;
	int64_t         x_stride_b, x_stride_n;  // elements
	const void *    wq, *wk, *wv, *wg;
};

// Status of the launch just enqueued.  A device this library carries no code for (anything but gfx950) shows up
// here as "no binary for this GPU" / "invalid device function" and is reported as such, not as a generic launch failure.
inline int launch_status() {
	const hipError_t e = hipGetLastError();
	if(e == hipSuccess) return AF3_OK;
	return (e == hipErrorNoBinaryForGpu || e == hipErrorInvalidDeviceFunction || e == hipErrorSharedObjectInitFailed || e == hipErrorNoDevice) ? AF3_ERR_NO_DEVICE_CODE : AF3_ERR_LAUNCH;
}
// AF3_OK when the calling thread's current device is a gfx950, AF3_ERR_NO_DEVICE_CODE otherwise (api.hip; one
// property query per device and process, then a table lookup).
int current_device_status();

// Launchers implemented in the .hip files; all validated by api.hip before the call.
int launch_dpa_generic(const af3_dpa_params& p, hipStream_t s);
int launch_dpa_mfma_bf16(const af3_dpa_params& p, hipStream_t s);
int launch_dpa_mfma_fp8(const af3_dpa_params& p, hipStream_t s);
// dpa_mfma_rows.hip: the bf16 kernel for batches that share a bias (four batch rows per wavefront); the caller has checked mfma_bf16_eligible
bool mfma_rows_eligible(const af3_dpa_params& p);
bool mfma_rows_can_serve(const af3_dpa_params& p);   // eligible, and its bias can be served (workspace given, or readable in place)
int64_t mfma_rows_workspace_bytes(const af3_dpa_params& p);
bool mfma_rows_suits_a_small_batch(const af3_dpa_params& p);  // fewer than 128 batch rows and a bias that this kernel stages in place
int launch_dpa_mfma_rows(const af3_dpa_params& p, hipStream_t s);
bool mfma_bf16_eligible(const af3_dpa_params& p);
int64_t mfma_bf16_workspace_bytes(const af3_dpa_params& p);
bool mfma_fp8_eligible(const af3_dpa_params& p);
int launch_dpa_mfma_f32(const af3_dpa_params& p, hipStream_t s);
bool mfma_f32_eligible(const af3_dpa_params& p);
bool grid_fused_eligible(const af3_grid_attention_params& g);
int64_t grid_fused_workspace_bytes(const af3_grid_attention_params& g);
int launch_grid_fused(const af3_grid_attention_params& g, hipStream_t s);

}  // namespace af3
