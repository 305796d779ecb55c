// C-ABI entry points for the attention forward pass: validation and kernel selection.
// Declared in include/af3_dpa.h.  Nothing here allocates, synchronises or exits.
#include "common.hpp"

#include <atomic>
#include <string.h>

using namespace af3;

int af3::current_device_status() {
	constexpr int       MAX_DEV = 64;
	static std::atomic<signed char> known[MAX_DEV];  // 0 = not asked yet, 1 = gfx950, -1 = anything else
	int dev = -1;
	if(hipGetDevice(&dev) != hipSuccess) {
		(void)hipGetLastError();
		return AF3_ERR_NO_DEVICE_CODE;  // no usable device at all
	}
	if(dev >= 0 && dev < MAX_DEV) {
		const signed char c = known[dev].load(std::memory_order_relaxed);
		if(c != 0) return c > 0 ? AF3_OK : AF3_ERR_NO_DEVICE_CODE;
	}
	hipDeviceProp_t prop;
	if(hipGetDeviceProperties(&prop, dev) != hipSuccess) {
		(void)hipGetLastError();
		return AF3_ERR_NO_DEVICE_CODE;
	}
	const bool ok = strncmp(prop.gcnArchName, "gfx950", 6) == 0;
	if(dev >= 0 && dev < MAX_DEV) known[dev].store(ok ? 1 : -1, std::memory_order_relaxed);
	return ok ? AF3_OK : AF3_ERR_NO_DEVICE_CODE;
}

namespace {

int validate(const af3_dpa_params* p) {
	if(!p) return AF3_ERR_NULL_POINTER;
	if(p->B <= 0 || p->H <= 0 || p->L <= 0 || p->D <= 0) return AF3_ERR_BAD_SHAPE;
	if(p->D > AF3_DPA_MAX_HEAD_DIM) return AF3_ERR_UNSUPPORTED_D;
	if(p->L > 0x3fffffff || p->B > 0x3fffffff || p->H > 0xffff) return AF3_ERR_BAD_SHAPE;
	if(!p->q || !p->k || !p->v || !p->out) return AF3_ERR_NULL_POINTER;
	for(int i = 0; i < 3; i++)
		if(p->q_stride[i] < 0 || p->k_stride[i] < 0 || p->v_stride[i] < 0 || p->out_stride[i] < 0) return AF3_ERR_BAD_STRIDE;
	// rows must not overlap: the innermost axis has stride 1 and D (or L for transposed fp8 V) elements
	if(p->q_stride[2] < p->D || p->k_stride[2] < p->D || p->out_stride[2] < p->D) return AF3_ERR_BAD_STRIDE;
	if(p->io_dtype == AF3_FP8_E4M3) {
		if(p->v_stride[2] < p->L) return AF3_ERR_BAD_STRIDE;
	} else if(p->v_stride[2] < p->D) {
		return AF3_ERR_BAD_STRIDE;
	}
	if(p->bias && (p->bias_stride[0] < 0 || p->bias_stride[1] < p->L)) return AF3_ERR_BAD_STRIDE;
	if(p->key_mask && p->key_mask_stride_b != 0 && p->key_mask_stride_b < p->L) return AF3_ERR_BAD_STRIDE;
	if(p->gate) {
		if(p->io_dtype == AF3_FP8_E4M3) return AF3_ERR_BAD_DTYPE;
		for(int i = 0; i < 3; i++)
			if(p->gate_stride[i] < 0) return AF3_ERR_BAD_STRIDE;
		if(p->gate_stride[2] < p->D) return AF3_ERR_BAD_STRIDE;
	}
	if(p->out_dtype != AF3_F32 && p->out_dtype != AF3_BF16) return AF3_ERR_BAD_DTYPE;
	if(p->bias && p->bias_dtype != AF3_F32 && p->bias_dtype != AF3_BF16) return AF3_ERR_BAD_DTYPE;
	if(!(p->softmax_scale > 0.f) || !(p->softmax_scale < INFINITY)) return AF3_ERR_BAD_ARGUMENT;
	switch(p->io_dtype) {
		case AF3_F32:
			if(p->mma_dtype != AF3_F32) return AF3_ERR_BAD_DTYPE;
			break;
		case AF3_BF16:
			if(p->mma_dtype != AF3_BF16 && p->mma_dtype != AF3_F32) return AF3_ERR_BAD_DTYPE;
			break;
		case AF3_FP8_E4M3:
			if(p->mma_dtype != AF3_FP8_E4M3) return AF3_ERR_BAD_DTYPE;
			break;
		default:
			return AF3_ERR_BAD_DTYPE;
	}
	return AF3_OK;
}

// 0 fp32 vector-FMA, 1 bf16 MFMA, 2 fp8 MFMA, 3 fp32 MFMA, or a negative status
int select_kernel(const af3_dpa_params& p) {
	if(p.io_dtype == AF3_FP8_E4M3) return mfma_fp8_eligible(p) ? 2 : AF3_ERR_BAD_ARGUMENT;
	if(p.force_generic) return 0;
	if(p.mma_dtype == AF3_F32) return mfma_f32_eligible(p) ? 3 : 0;
	return mfma_bf16_eligible(p) ? 1 : 0;
}

}  // namespace

extern "C" int64_t af3_dpa_workspace_bytes(const af3_dpa_params* params) {
	const int rc = validate(params);
	if(rc != AF3_OK) return rc;
	return select_kernel(*params) == 1 ? mfma_bf16_workspace_bytes(*params) : 0;
}

extern "C" int af3_dpa_select_kernel(const af3_dpa_params* params) {
	const int rc = validate(params);
	if(rc != AF3_OK) return rc;
	return select_kernel(*params);
}

// ---- the allocation-free entry point's scratch: a device array inside the code object, one copy per GPU ----
// In host code the array's name is only a handle for hipGetSymbolAddress; the address that kernels and copies may use
// is looked up once per device (with that device current) and kept here.
static __device__ __align__(256) unsigned char scratch[AF3_STATIC_SCRATCH_BYTES];

namespace {
constexpr int        SCRATCH_MAX_DEV = 64;
std::atomic<void*>   scratch_ptr[SCRATCH_MAX_DEV];

// device address of `scratch` on the current device, or nullptr with *status set
void* static_scratch_address(int* status) {
	int dev = -1;
	if(hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= SCRATCH_MAX_DEV) {
		(void)hipGetLastError();
		*status = AF3_ERR_NO_DEVICE_CODE;
		return nullptr;
	}
	void* ptr = scratch_ptr[dev].load(std::memory_order_acquire);
	if(ptr) return ptr;
	const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));  // (two threads may both ask: they get the same answer)
	if(e != hipSuccess || !ptr) {
		(void)hipGetLastError();
		*status = (e == hipErrorNoBinaryForGpu || e == hipErrorInvalidDeviceFunction || e == hipErrorSharedObjectInitFailed) ? AF3_ERR_NO_DEVICE_CODE : AF3_ERR_LAUNCH;
		return nullptr;
	}
	scratch_ptr[dev].store(ptr, std::memory_order_release);
	return ptr;
}
}  // namespace

extern "C" int af3_dpa_forward_static_scratch(const af3_dpa_params* params, void* hip_stream) {
	const int rc = validate(params);
	if(rc != AF3_OK) return rc;
	af3_dpa_params p = *params;
	p.workspace = nullptr, p.workspace_bytes = 0;
	const int64_t need = select_kernel(p) == 1 ? mfma_bf16_workspace_bytes(p) : 0;
	if(need > (int64_t)AF3_STATIC_SCRATCH_BYTES) return AF3_ERR_SCRATCH_LIMIT;
	if(const int dc = current_device_status(); dc != AF3_OK) return dc;
	if(need > 0) {
		int   st  = AF3_OK;
		void* ptr = static_scratch_address(&st);
		if(!ptr) return st;
		p.workspace = ptr, p.workspace_bytes = AF3_STATIC_SCRATCH_BYTES;
	}
	return af3_dpa_forward(&p, hip_stream);
}

extern "C" int af3_dpa_forward(const af3_dpa_params* params, void* hip_stream) {
	const int rc = validate(params);
	if(rc != AF3_OK) return rc;
	if(const int dc = current_device_status(); dc != AF3_OK) return dc;
	hipStream_t s = static_cast<hipStream_t>(hip_stream);
	switch(select_kernel(*params)) {
		case 0: return launch_dpa_generic(*params, s);
		case 1: return launch_dpa_mfma_bf16(*params, s);
		case 2: return launch_dpa_mfma_fp8(*params, s);
		case 3: return launch_dpa_mfma_f32(*params, s);
		default: return AF3_ERR_BAD_ARGUMENT;
	}
}

static int validate_grid(const af3_grid_attention_params* g) {
	if(!g || !g->pair || !g->out || !g->q_proj || !g->k_proj || !g->v_proj || !g->gating_query) return AF3_ERR_NULL_POINTER;
	if(g->B <= 0 || g->N <= 0 || g->C <= 0 || g->head <= 0 || g->C % g->head != 0 || g->B > 0x3fffffff) return AF3_ERR_BAD_SHAPE;
	if(g->pair_stride[0] < 0 || g->pair_stride[1] < g->C || g->out_stride[0] < 0 || g->out_stride[1] < g->C) return AF3_ERR_BAD_STRIDE;
	if(g->bias && (g->bias_stride[0] < 0 || g->bias_stride[1] < g->N)) return AF3_ERR_BAD_STRIDE;
	if(g->key_mask && g->key_mask_stride_b != 0 && g->key_mask_stride_b < g->N) return AF3_ERR_BAD_STRIDE;
	return AF3_OK;
}

extern "C" int af3_grid_attention_supported(const af3_grid_attention_params* g) { return validate_grid(g) == AF3_OK && grid_fused_eligible(*g) ? 1 : 0; }

extern "C" int64_t af3_grid_attention_workspace_bytes(const af3_grid_attention_params* g) {
	const int rc = validate_grid(g);
	return rc != AF3_OK ? rc : grid_fused_workspace_bytes(*g);
}

extern "C" int af3_grid_attention_forward(const af3_grid_attention_params* g, void* hip_stream) {
	const int rc = validate_grid(g);
	if(rc != AF3_OK) return rc;
	if(!grid_fused_eligible(*g)) return AF3_ERR_BAD_ARGUMENT;
	if(g->bias && (!g->workspace || g->workspace_bytes < grid_fused_workspace_bytes(*g) || (reinterpret_cast<uintptr_t>(g->workspace) & 15))) return AF3_ERR_BAD_ARGUMENT;
	if(const int dc = current_device_status(); dc != AF3_OK) return dc;
	return launch_grid_fused(*g, static_cast<hipStream_t>(hip_stream));
}

extern "C" const char* af3_status_string(int status) {
	switch(status) {
		case AF3_OK: return "ok";
		case AF3_ERR_NULL_POINTER: return "a required pointer is NULL";
		case AF3_ERR_BAD_DTYPE: return "dtype combination not implemented";
		case AF3_ERR_BAD_SHAPE: return "a dimension is not positive or exceeds the supported maximum";
		case AF3_ERR_BAD_STRIDE: return "negative stride, overlapping rows, or innermost stride != 1";
		case AF3_ERR_UNSUPPORTED_D: return "head_dim exceeds the supported maximum (128)";
		case AF3_ERR_LAUNCH: return "kernel launch failed";
		case AF3_ERR_BAD_ARGUMENT: return "invalid argument";
		case AF3_ERR_SCRATCH_LIMIT: return "the call needs more scratch than the library's static scratch array holds (use af3_dpa_forward with a workspace)";
		case AF3_ERR_NO_DEVICE_CODE: return "the current device is not a gfx950 (MI355X); this library carries code for nothing else";
		default: return "unknown status";
	}
}

extern "C" int af3_abi_version(void) { return 4; }
