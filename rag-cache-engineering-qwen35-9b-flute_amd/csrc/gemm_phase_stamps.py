"""Reader of the GEMM kernel's phase stamps (a diagnostic of instrumented builds).

A library built with -DFLUTE_STAMPS writes, per wavefront of gemm_kernel, the wall time
(s_memrealtime, 10 ns units) at seven points of the kernel and the shader-clock count across the
K loop; the normal build holds none of this.  Build one beside the product library and read it:

    make -C <this directory> OUT=<package>/lib_stamps EXTRA=-DFLUTE_STAMPS -j8
    python3 gemm_phase_stamps.py <package>/lib_stamps/libflute_hip.so [N K M]

Prints, for whole flute_gemm calls on cold weights (twelve weights in rotation), the median and
the 10th/90th percentile over the wavefronts of every phase time since the first wavefront's
start, the cycle count of the K loop and the shader clock it implies (cycles / wall time of the
same interval of the same wavefront).
"""
import ctypes
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
from flute_extended import _lib as L  # noqa: E402

PHASES = ["start", "tables built, loop begins", "loop done", "all wavefronts past the loop",
          "K tree done", "totals tile written", "stored"]


def main(argv):
    if len(argv) < 2:
        raise SystemExit(__doc__)
    lib = ctypes.CDLL(os.path.abspath(argv[1]))
    if not hasattr(lib, "flute_debug_stamps"):
        raise SystemExit(f"{argv[1]} was not built with -DFLUTE_STAMPS")
    for name, (res, args) in L.SYMBOLS.items():
        if hasattr(lib, name):
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
    lib.flute_debug_stamps.argtypes = [ctypes.c_void_p]
    N, K, M = (int(v) for v in (argv[2:5] + ["12288", "4096", "256"][len(argv) - 2:]))
    dev = "cuda:0"
    gen = torch.Generator(device=dev).manual_seed(0)
    descs, keep = [], []
    for _ in range(12):
        blob = torch.randint(0, 256, (N * K // 2,), dtype=torch.uint8, device=dev, generator=gen)
        lut = (torch.randn(N // 128, 16, device=dev, generator=gen) * 0.02).sort(dim=1).values \
            .to(torch.bfloat16).contiguous()
        d = L.FluteLinear()
        d.q1, d.lut1, d.q1_bytes = blob.data_ptr(), lut.data_ptr(), blob.numel()
        d.N, d.K, d.b1, d.group_size, d.lut_rows, d.lut_dtype = N, K, 4, 128, N // 128, L.BF16
        descs.append(d)
        keep.append((blob, lut))
    A = torch.randn(M, K, device=dev, generator=gen).to(torch.bfloat16)
    C = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    stamps = torch.zeros(8192 * 8 * 8, dtype=torch.int64, device=dev)
    if lib.flute_debug_stamps(stamps.data_ptr()) != 0:
        raise SystemExit("flute_debug_stamps failed")
    stream = torch.cuda.current_stream().cuda_stream
    print(f"flute_gemm {K} -> {N}, M = {M}, bf16 LUT, bf16 activations, cold weights", flush=True)
    for rep in range(3):
        for d in descs:
            stamps.zero_()
            if lib.flute_gemm(ctypes.byref(d), A.data_ptr(), C.data_ptr(), M, K, N, L.BF16, stream) != 0:
                raise SystemExit(lib.flute_last_error())
        torch.cuda.synchronize()
        s = stamps.cpu().numpy().reshape(-1, 8)
        s = s[s[:, 0] != 0]                                  # the last call's wavefronts
        loop_ns = (s[:, 2] - s[:, 1]).astype(np.float64) * 10.0
        ghz = s[:, 7].astype(np.float64) / np.maximum(loop_ns, 1.0)
        t = s[:, 0:7].astype(np.float64) * 10.0
        t -= t[:, 0].min()
        print(f"call {rep}: {len(s)} wavefronts, last store at {t[:, 6].max():.0f} ns")
        for j, name in enumerate(PHASES):
            v = t[s[:, j] != 0, j]                           # (wavefronts that left before a point never stamp it)
            print(f"  {name:30s} p10 {np.percentile(v, 10):7.0f}  median {np.median(v):7.0f}  "
                  f"p90 {np.percentile(v, 90):7.0f} ns")
        print(f"  K loop: median {np.median(s[:, 7]):.0f} cycles in {np.median(loop_ns):.0f} ns; shader clock "
              f"median {np.median(ghz):.3f} GHz (p10 {np.percentile(ghz, 10):.3f}, p90 "
              f"{np.percentile(ghz, 90):.3f})", flush=True)


if __name__ == "__main__":
    main(sys.argv)
