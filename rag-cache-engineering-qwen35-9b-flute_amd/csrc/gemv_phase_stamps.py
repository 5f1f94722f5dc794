"""Reader of the lean GEMV kernel's phase stamps (a diagnostic of instrumented builds).

A library built with -DFLUTE_STAMPS writes, per wavefront of gemv4_kernel (single 4-bit stream,
LUT grouped along N, plain input), the wall time (s_memrealtime, 10 ns units) at eight points of
the kernel; the normal build holds none of this.  Build one beside the product library and read it:

    make -C <this directory> OUT=<some directory> EXTRA=-DFLUTE_STAMPS -j8
    python3 gemv_phase_stamps.py <some directory>/libflute_hip.so [N K ...]

Prints, for single flute_gemv calls on cold weights (launched eagerly, three in a row, the last
one's stamps kept), the median over the wavefronts of every phase time since the first wavefront's
start.  A stamp costs about 0.1 us (it waits for the scalar loads in flight and stores one value),
so the sum is longer than an uninstrumented launch; the proportions are what it is for.
"""
import ctypes
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
from flute_extended import _lib as L  # noqa: E402

PHASES = ["start", "LUT row in (kernel arguments, then the row)", "table written", "activations staged",
          "table barrier passed", "loop done", "row sums written", "last barrier passed"]


def run(lib, N, K, dtype):
    dev = "cuda:0"
    gen = torch.Generator(device=dev).manual_seed(0)
    count = min(64, max(4, int(3.1 * 256 * 2 ** 20 // (N * K // 2)) + 1))
    descs, keep = [], []
    for _ in range(count):
        blob = torch.randint(0, 256, (N * K // 2,), dtype=torch.uint8, device=dev, generator=gen)
        lut = (torch.randn(N // 128, 16, device=dev, generator=gen) * 0.02).sort(dim=1).values.half().contiguous()
        d = L.FluteLinear()
        d.q1, d.lut1, d.q1_bytes = blob.data_ptr(), lut.data_ptr(), blob.numel()
        d.N, d.K, d.b1, d.group_size, d.lut_rows, d.lut_dtype = N, K, 4, 128, N // 128, L.F16
        descs.append(d)
        keep.append((blob, lut))
    x = torch.randn(1, K, device=dev, generator=gen).to(dtype)
    y = torch.zeros(1, N, dtype=dtype, device=dev)
    act = L.BF16 if dtype == torch.bfloat16 else L.F16
    stamps = torch.zeros(4096 * 8 * 8, dtype=torch.int64, device=dev)
    if lib.flute_debug_gemv_stamps(stamps.data_ptr()) != 0:
        raise SystemExit("flute_debug_gemv_stamps failed")
    stream = torch.cuda.current_stream().cuda_stream
    rows = []
    for _ in range(3):
        for d in descs:
            stamps.zero_()
            for _ in range(3):
                if lib.flute_gemv(ctypes.byref(d), x.data_ptr(), y.data_ptr(), act, 0, stream) != 0:
                    raise SystemExit("flute_gemv failed")
            torch.cuda.synchronize()
            s = stamps.cpu().numpy().reshape(-1, 8)
            s = s[s[:, 0] != 0].astype(np.float64) * 10.0
            t0 = s[:, 0].min()
            rows.append([np.median(s[:, j] - t0) for j in range(8)] + [(s[:, 7] - t0).max(), len(s)])
    r = np.median(np.array(rows), axis=0)
    print(f"flute_gemv {K} -> {N}, {dtype}, cold weights: {int(r[9])} wavefronts, the last one through the "
          f"last barrier {r[8]:.0f} ns after the first one's start")
    for j, name in enumerate(PHASES):
        print(f"   {name:46s} median {r[j]:7.0f} ns")
    sys.stdout.flush()


def main(argv):
    if len(argv) < 2:
        raise SystemExit(__doc__)
    lib = ctypes.CDLL(os.path.abspath(argv[1]))
    if not hasattr(lib, "flute_debug_gemv_stamps"):
        raise SystemExit(f"{argv[1]} was not built with -DFLUTE_STAMPS")
    for name, (res, args) in L.SYMBOLS.items():
        if hasattr(lib, name):
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
    lib.flute_debug_gemv_stamps.argtypes = [ctypes.c_void_p]
    shapes = [(int(argv[i]), int(argv[i + 1])) for i in range(2, len(argv) - 1, 2)] or [(1024, 4096), (12288, 4096)]
    for N, K in shapes:
        run(lib, N, K, torch.bfloat16)


if __name__ == "__main__":
    main(sys.argv)
