"""Runs the microbenchmarks of csrc/microbench.hip on cuda:0 and prints one table:

    python -m af3_kernels_amd.microbench [--quick]

1. matrix / vector overlap on independent work, 2. the attention stage's instruction skeleton with and without its
memory instructions, a second chain per wavefront and random operands, 3. streaming bandwidth of 16-byte loads from
buffers that fit L2, MALL and HBM.  Times are per "round": the work of the four chains (32 query rows x 32 keys each)
that share one SIMD, i.e. 4 x (9 MFMAs + 16 exp2 + 8 packs); the bf16 attention kernel spends 1085 ns on it at cfg4.
"""
import ctypes
import os
import sys

import torch

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libaf3_microbench.so")


def _load():
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is missing: run `python -m af3_kernels_amd.build`")
    lib = ctypes.CDLL(LIB_PATH)
    lib.af3_microbench_run.restype = ctypes.c_int
    lib.af3_microbench_run.argtypes = [ctypes.c_int] * 4 + [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    return lib


class Runner:
    def __init__(self):
        if not torch.cuda.is_available():
            raise RuntimeError("the microbenchmarks need the GPU")
        self.lib = _load()
        self.out = torch.zeros(1 << 23, dtype=torch.float32, device="cuda")
        g = torch.Generator().manual_seed(0)
        self.n_vec = (1 << 20) // 16                                    # 1 MB: stays in every XCD's L2
        self.buf = (0.5 * torch.randn(self.n_vec * 8, generator=g)).to(torch.bfloat16).view(torch.int32).cuda()

    def ns_per_trip(self, which, variant, grid, threads, iters, buf=None, n_vec=None, reps=3):
        buf = self.buf if buf is None else buf
        n_vec = self.n_vec if n_vec is None else n_vec
        stream = torch.cuda.current_stream().cuda_stream

        def launch():
            rc = self.lib.af3_microbench_run(which, variant, grid, threads, self.out.data_ptr(), buf.data_ptr(), n_vec, iters, stream)
            if rc != 0:
                raise RuntimeError(f"af3_microbench_run({which}, {variant}) returned {rc}")
        launch()
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(reps):
            launch()
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) / reps * 1e6 / iters


def main(quick=False):
    r = Runner()
    n_cu = torch.cuda.get_device_properties(0).multi_processor_count
    it = 2000 if quick else 8000
    rows = []
    # 1: one workgroup of 1024 threads per CU = four wavefronts per SIMD; a trip is one stage of every wavefront
    for variant, name in ((0, "8 MFMA 32x32x16 bf16 only"), (4, "8 MFMA only, random operands"), (1, "16 exp2 + 8 packs only"), (2, "MFMA; exp2, exp2, pack (x8)"), (3, "8 MFMA; 16 exp2; 8 packs")):
        rows.append(("independent work, 4 wavefronts/SIMD: " + name, r.ns_per_trip(0, variant, n_cu, 1024, it)))
    # 2: 256-thread workgroups; 4 per CU with one chain per wavefront, 2 per CU with two: four chains per SIMD either way.
    #    A trip is one stage of every chain.
    for flags, name in ((8, "no memory instructions, no row-sum check"), (0, "no memory instructions"), (1, "+ two bias-fragment loads of random data"),
                        (2, "+ K/V fragment LDS reads"), (3, "+ both"), (4, "random operands, no memory instructions"), (7, "random operands, loads and LDS reads")):
        rows.append(("stage skeleton, 1 chain x 4 wavefronts/SIMD: " + name, r.ns_per_trip(1, flags, 4 * n_cu, 256, it)))
    zeros = torch.zeros_like(r.buf)
    rows.append(("stage skeleton, 1 chain x 4 wavefronts/SIMD: + two bias-fragment loads of zeros", r.ns_per_trip(1, 1, 4 * n_cu, 256, it, buf=zeros)))
    for flags, name in ((0, "no memory instructions"), (4, "random operands, no memory instructions")):
        rows.append(("stage skeleton, 2 chains x 2 wavefronts/SIMD: " + name, r.ns_per_trip(1, 16 + flags, 2 * n_cu, 256, it)))
    width = max(len(n) for n, _ in rows)
    print(f"{n_cu} CUs; ns per round (four chain-stages per SIMD)")
    for name, ns in rows:
        print(f"  {name:{width}s} {ns:8.1f}")
    # 3: 8 KB per wavefront and trip
    print("16-byte loads streaming a buffer, 4096 workgroups of 4 wavefronts:")
    for mb in ((1, 64) if quick else (1, 2, 3, 6, 16, 64, 512)):
        n_vec = mb * (1 << 20) // 16
        buf = torch.zeros(n_vec * 4, dtype=torch.int32, device="cuda")
        trips = 500 if quick else 2000
        ns = r.ns_per_trip(2, 0, 4096, 256, trips, buf=buf, n_vec=n_vec, reps=1)
        print(f"  {mb:4d} MB buffer {4096 * 4 * 8 * 1024 / ns / 1e3:8.2f} TB/s")
        del buf


if __name__ == "__main__":
    main(quick="--quick" in sys.argv)
