// Torch-free check of the C ABI (include/af3_dpa.h): a plain HIP host program that allocates device
// buffers with hipMalloc, calls af3_dpa_forward on a stream of its own the way a C / C++ / cgo / JNI
// caller would, and compares the result with the CPU oracle's fp64 formula (af3o_dpa_formula).
//
//   abi_host_check            run every case on device 0; exit status 0 = all within tolerance
//   abi_host_check --list     print the cases, touch no GPU
//
// Built by tests/Makefile (hipcc, links libaf3_dpa.so and the oracle library); run by tests/test_abi_host.py.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "af3_dpa.h"

extern "C" int      af3o_dpa_formula(const float* q, const float* k, const float* v, const float* bias, const uint8_t* keep, float* out, int64_t B, int64_t H, int64_t L, int64_t D);
extern "C" int      af3o_fused_attention_formula(const float* x, const uint8_t* keep, const float* bias, const float* wq, const float* wk, const float* wv, const float* wg,
                                                 const float* wo, const float* qbias, float* out, int64_t B, int64_t L, int64_t C, int64_t H);
extern "C" int      af3o_vnni_repack(const uint16_t* in, uint16_t* out, int64_t M, int64_t N, int64_t blk);
extern "C" uint16_t af3o_f32_to_bf16_bits(float f);
extern "C" float    af3o_bf16_bits_to_f32(uint16_t h);

namespace {

struct Case {
	const char* name;
	int64_t     B, H, L, D;
	int         dtype;      // AF3_F32 or AF3_BF16
	int         workspace;  // 0: none; 1: hand the library its optional scratch buffer; 2: af3_dpa_forward_static_scratch (the library's own array)
	int         drop_tail;  // keys dropped at the end of every row of the last batch entry
	double      tol;
};

const Case CASES[] = {
	{"fp32 2x4x128x32 (fp32-FMA kernel)", 2, 4, 128, 32, AF3_F32, 0, 16, 1e-4},
	{"bf16 3x4x200x32 with workspace", 3, 4, 200, 32, AF3_BF16, 1, 20, 2e-2},
	{"bf16 3x4x200x32 without workspace", 3, 4, 200, 32, AF3_BF16, 0, 20, 2e-2},
	{"bf16 1x16x256x24 in-place bias", 1, 16, 256, 24, AF3_BF16, 0, 13, 2e-2},
	{"bf16 2x2x96x64", 2, 2, 96, 64, AF3_BF16, 1, 0, 2e-2},
	{"bf16 5x4x300x32 static scratch", 5, 4, 300, 32, AF3_BF16, 2, 9, 2e-2},
	{"bf16 3x4x200x32 static scratch (smaller call on the same array)", 3, 4, 200, 32, AF3_BF16, 2, 20, 2e-2},
};

// splitmix64 -> approximately normal values (sum of 4 uniforms), reproducible without <random>
struct Rng {
	uint64_t s;
	double   u() {
        uint64_t z = (s += 0x9E3779B97F4A7C15ull);
        z          = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z          = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return (double)((z ^ (z >> 31)) >> 11) / 9007199254740992.0;
	}
	float n() { return (float)((u() + u() + u() + u() - 2.0) * 1.7320508); }
};

#define HIP_OK(x)                                                                      \
	do {                                                                               \
		hipError_t e_ = (x);                                                           \
		if(e_ != hipSuccess) {                                                         \
			std::fprintf(stderr, "%s failed: %s\n", #x, hipGetErrorString(e_));        \
			return 2;                                                                  \
		}                                                                              \
	} while(0)

int run(const Case& c, hipStream_t stream) {
	const int64_t n = c.B * c.H * c.L * c.D, nb = c.H * c.L * c.L;
	Rng           rng{0x5eed0000ull + (uint64_t)(c.L * 131 + c.D)};
	std::vector<float> q(n), k(n), v(n), bias(nb), want(n);
	for(auto* t : {&q, &k, &v}) for(auto& x : *t) x = rng.n();
	for(auto& x : bias) x = rng.n();
	std::vector<uint8_t> keep(c.B * c.L, 1);
	for(int64_t j = c.L - c.drop_tail; j < c.L; j++) keep[(c.B - 1) * c.L + j] = 0;
	const bool bf = c.dtype == AF3_BF16;
	if(bf)  // the formula sees exactly what the kernel sees
		for(auto* t : {&q, &k, &v, &bias}) for(auto& x : *t) x = af3o_bf16_bits_to_f32(af3o_f32_to_bf16_bits(x));
	if(af3o_dpa_formula(q.data(), k.data(), v.data(), bias.data(), keep.data(), want.data(), c.B, c.H, c.L, c.D) != 0) return 2;

	const size_t         esz = bf ? 2 : 4;
	std::vector<uint8_t> hq(n * esz), hk(n * esz), hv(n * esz), hb(nb * esz), ho(n * esz);
	auto                 pack = [&](const std::vector<float>& src, std::vector<uint8_t>& dst) {
        for(size_t i = 0; i < src.size(); i++) {
            if(bf) {
                const uint16_t h = af3o_f32_to_bf16_bits(src[i]);
                std::memcpy(&dst[2 * i], &h, 2);
            } else {
                std::memcpy(&dst[4 * i], &src[i], 4);
            }
        }
	};
	pack(q, hq), pack(k, hk), pack(v, hv), pack(bias, hb);

	void *dq, *dk, *dv, *db, *dm, *dout, *dws = nullptr;
	HIP_OK(hipMalloc(&dq, hq.size()));
	HIP_OK(hipMalloc(&dk, hk.size()));
	HIP_OK(hipMalloc(&dv, hv.size()));
	HIP_OK(hipMalloc(&db, hb.size()));
	HIP_OK(hipMalloc(&dm, keep.size()));
	HIP_OK(hipMalloc(&dout, ho.size()));
	HIP_OK(hipMemcpy(dq, hq.data(), hq.size(), hipMemcpyHostToDevice));
	HIP_OK(hipMemcpy(dk, hk.data(), hk.size(), hipMemcpyHostToDevice));
	HIP_OK(hipMemcpy(dv, hv.data(), hv.size(), hipMemcpyHostToDevice));
	HIP_OK(hipMemcpy(db, hb.data(), hb.size(), hipMemcpyHostToDevice));
	HIP_OK(hipMemcpy(dm, keep.data(), keep.size(), hipMemcpyHostToDevice));

	af3_dpa_params p;
	std::memset(&p, 0, sizeof p);
	p.q = dq, p.k = dk, p.v = dv, p.bias = db, p.key_mask = static_cast<const uint8_t*>(dm), p.out = dout;
	p.B = c.B, p.H = c.H, p.L = c.L, p.D = c.D;
	const int64_t st[3] = {c.H * c.L * c.D, c.L * c.D, c.D};
	for(int i = 0; i < 3; i++) p.q_stride[i] = p.k_stride[i] = p.v_stride[i] = p.out_stride[i] = st[i];
	p.bias_stride[0] = c.L * c.L, p.bias_stride[1] = c.L;
	p.key_mask_stride_b = c.L;
	p.io_dtype = p.bias_dtype = p.out_dtype = p.mma_dtype = c.dtype;
	p.softmax_scale = 1.0f / std::sqrt((float)c.D);
	p.q_descale = p.k_descale = p.v_descale = 1.0f;
	const int64_t ws = af3_dpa_workspace_bytes(&p);
	if(c.workspace == 1 && ws > 0) {
		HIP_OK(hipMalloc(&dws, (size_t)ws));
		p.workspace = dws, p.workspace_bytes = ws;
	}
	const int kernel = af3_dpa_select_kernel(&p);
	const int rc     = c.workspace == 2 ? af3_dpa_forward_static_scratch(&p, stream) : af3_dpa_forward(&p, stream);
	if(rc != AF3_OK) {
		std::fprintf(stderr, "af3_dpa_forward: %s\n", af3_status_string(rc));
		return 1;
	}
	HIP_OK(hipStreamSynchronize(stream));
	HIP_OK(hipMemcpy(ho.data(), dout, ho.size(), hipMemcpyDeviceToHost));
	double err = 0.0;
	bool   finite = true;
	for(int64_t i = 0; i < n; i++) {
		float g;
		if(bf) {
			uint16_t h;
			std::memcpy(&h, &ho[2 * i], 2);
			g = af3o_bf16_bits_to_f32(h);
		} else {
			std::memcpy(&g, &ho[4 * i], 4);
		}
		finite = finite && std::isfinite(g);
		err    = std::fmax(err, std::fabs((double)g - (double)want[i]));
	}
	for(void* ptr : {dq, dk, dv, db, dm, dout, dws})
		if(ptr) HIP_OK(hipFree(ptr));
	const bool ok = finite && err <= c.tol;
	std::printf("%-40s kernel=%d workspace=%lld B  max_abs_err=%.3e (tol %.0e)  %s\n", c.name, kernel, (long long)(dws ? ws : 0), err, c.tol, ok ? "ok" : "FAIL");
	std::fflush(stdout);
	return ok ? 0 : 1;
}

// Grid self-attention up to the gate (af3_grid_attention_forward) on B batch rows of N tokens, 128 channels, 4 heads:
// weights handed over in the reference's VNNI panel layout, result against the fp64 formula without output projection.
int run_grid(int64_t B, int64_t N, hipStream_t stream) {
	const int64_t C = 128, H = 4;
	Rng           rng{0x9e1d0000ull + (uint64_t)N};
	auto          bf = [](float f) { return af3o_bf16_bits_to_f32(af3o_f32_to_bf16_bits(f)); };
	std::vector<float> x(B * N * C), bias(H * N * N), w[4], want(B * N * C);
	for(auto& v : x) v = bf(rng.n());
	for(auto& v : bias) v = bf(rng.n());
	for(auto& m : w) {
		m.resize(C * C);
		for(auto& v : m) v = bf(rng.n() / std::sqrt((float)C));
	}
	std::vector<uint8_t> keep(B * N, 1);
	for(int64_t j = N - N / 5; j < N; j++) keep[(B - 1) * N + j] = 0;
	if(af3o_fused_attention_formula(x.data(), keep.data(), bias.data(), w[0].data(), w[1].data(), w[2].data(), w[3].data(), nullptr, nullptr, want.data(), B, N, C, H) != 0) return 2;

	auto to_bits = [](const std::vector<float>& src) {
		std::vector<uint16_t> dst(src.size());
		for(size_t i = 0; i < src.size(); i++) dst[i] = af3o_f32_to_bf16_bits(src[i]);
		return dst;
	};
	const std::vector<uint16_t> hx = to_bits(x), hb = to_bits(bias);
	std::vector<uint16_t>       hw[4], ho(B * N * C);
	for(int i = 0; i < 4; i++) {
		const std::vector<uint16_t> nat = to_bits(w[i]);
		hw[i].resize(C * C);
		if(af3o_vnni_repack(nat.data(), hw[i].data(), C, C, C / H) != 0) return 2;
	}
	void *dx, *db, *dm, *dout, *dw[4], *dws = nullptr;
	HIP_OK(hipMalloc(&dx, hx.size() * 2));
	HIP_OK(hipMalloc(&db, hb.size() * 2));
	HIP_OK(hipMalloc(&dm, keep.size()));
	HIP_OK(hipMalloc(&dout, ho.size() * 2));
	HIP_OK(hipMemcpy(dx, hx.data(), hx.size() * 2, hipMemcpyHostToDevice));
	HIP_OK(hipMemcpy(db, hb.data(), hb.size() * 2, hipMemcpyHostToDevice));
	HIP_OK(hipMemcpy(dm, keep.data(), keep.size(), hipMemcpyHostToDevice));
	for(int i = 0; i < 4; i++) {
		HIP_OK(hipMalloc(&dw[i], C * C * 2));
		HIP_OK(hipMemcpy(dw[i], hw[i].data(), C * C * 2, hipMemcpyHostToDevice));
	}
	af3_grid_attention_params g;
	std::memset(&g, 0, sizeof g);
	g.pair = dx, g.pair_stride[0] = N * C, g.pair_stride[1] = C;
	g.q_proj = dw[0], g.k_proj = dw[1], g.v_proj = dw[2], g.gating_query = dw[3];
	g.bias = db, g.bias_stride[0] = N * N, g.bias_stride[1] = N, g.bias_dtype = AF3_BF16;
	g.key_mask = static_cast<const uint8_t*>(dm), g.key_mask_stride_b = N;
	g.out = dout, g.out_stride[0] = N * C, g.out_stride[1] = C;
	g.B = B, g.N = N, g.C = C, g.head = H, g.dtype = AF3_BF16;
	if(!af3_grid_attention_supported(&g)) {
		std::fprintf(stderr, "af3_grid_attention_supported: 0 for B=%lld N=%lld\n", (long long)B, (long long)N);
		return 1;
	}
	const int64_t ws = af3_grid_attention_workspace_bytes(&g);
	HIP_OK(hipMalloc(&dws, (size_t)ws));
	g.workspace = dws, g.workspace_bytes = ws;
	const int rc = af3_grid_attention_forward(&g, stream);
	if(rc != AF3_OK) {
		std::fprintf(stderr, "af3_grid_attention_forward: %s\n", af3_status_string(rc));
		return 1;
	}
	HIP_OK(hipStreamSynchronize(stream));
	HIP_OK(hipMemcpy(ho.data(), dout, ho.size() * 2, hipMemcpyDeviceToHost));
	double err = 0.0, top = 1.0;
	bool   finite = true;
	for(size_t i = 0; i < ho.size(); i++) {
		const float gv = af3o_bf16_bits_to_f32(ho[i]);
		finite = finite && std::isfinite(gv);
		err    = std::fmax(err, std::fabs((double)gv - (double)want[i]));
		top    = std::fmax(top, std::fabs((double)want[i]));
	}
	for(void* ptr : {dx, db, dm, dout, dw[0], dw[1], dw[2], dw[3], dws}) HIP_OK(hipFree(ptr));
	const double tol = 3e-2 * top;  // q, k, v and the gate are rounded to bf16 inside the op, like the reference's
	const bool   ok  = finite && err <= tol;
	std::printf("grid attention one kernel %lldx%lldx128, 4 heads  workspace=%lld B  max_abs_err=%.3e (tol %.1e)  %s\n", (long long)B, (long long)N, (long long)ws, err, tol,
				ok ? "ok" : "FAIL");
	std::fflush(stdout);
	return ok ? 0 : 1;
}

}  // namespace

int main(int argc, char** argv) {
	if(argc > 1 && std::strcmp(argv[1], "--list") == 0) {
		std::printf("abi version %d\n", af3_abi_version());
		for(const Case& c : CASES) std::printf("%s\n", c.name);
		std::printf("grid attention one kernel 3x100x128, 3x256x128\n");
		return 0;
	}
	HIP_OK(hipSetDevice(0));
	hipStream_t stream;
	HIP_OK(hipStreamCreate(&stream));
	int bad = 0;
	for(const Case& c : CASES) {
		const int r = run(c, stream);
		if(r == 2) return 2;
		bad += r;
	}
	for(const int64_t n : {int64_t{100}, int64_t{256}}) {
		const int r = run_grid(3, n, stream);
		if(r == 2) return 2;
		bad += r;
	}
	// error behaviour: a malformed call is refused with a status code, nothing is launched
	af3_dpa_params p;
	std::memset(&p, 0, sizeof p);
	const int rc = af3_dpa_forward(&p, stream);
	std::printf("empty params -> %d (%s)\n", rc, af3_status_string(rc));
	if(rc >= 0) bad++;
	HIP_OK(hipStreamDestroy(stream));
	return bad ? 1 : 0;
}
