#!/usr/bin/env python3
"""Benchmark of the idxN LUT-palettized linear layer on one MI355X.

Headline (`value`, `ms_per_step`, `roofline`): the M = 1 LUT GEMV of the MLP up-projection,
K = 4096 -> N = 12288, idx4 blob, group 128, fp16 LUT, bf16 activations.  One step = one
call of flute_gemv.  The weights live in HBM before the clock starts and consecutive steps
use different weights whose total size exceeds three times the 256 MB memory-side cache,
so every step streams its 24 MiB from HBM ("cold").  `value` = packed index + LUT bytes
per second (the numerator the target is stated on); `roofline.achieved` counts all
algorithmic bytes of the launch (indices, LUT, activations in, outputs).

Timing: the K steps are captured into one hipGraph; the graph is replayed 21 times with
events on the launch stream and the median replay is reported (time of exactly K steps).

Beside it, in the same JSON line: `mlp_block` (the fused MLP decode block of the second
configuration: merged gate+up with SiLU*mul, then down), `gemm` (the M > 1 LUT-GEMM, both
shapes, M = 16 / 64 / 256 / 1024), `other_m1_configs` (cache-resident, fused rotation,
lm_head, narrow shapes with the K splits swept) and `cpu_baseline` (the oracle's
restatement of the upstream torch path on the host cores, bounded samples).
Every row is parity-gated against the oracle; a row whose gate fails aborts the run.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path[:0] = [os.path.join(ROOT, "rag-cache-engineering-qwen35-9b-flute_amd")]

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E bandwidth
MFMA_PEAK_TFLOPS = 2500.0      # MI355X published dense bf16/fp16 MFMA rate
H, I, GS = 4096, 12288, 128
# HBM bytes one launch of the headline kernel moves come from FETCH_SIZE and WRITE_SIZE counter
# runs of this file under rocprofv3 (scaled by a copy of known size, --calibrate-copy); a
# counter cannot be read from inside the process, so the figure is read back from the summary
# those runs left in profiles/ (a line "traffic_bytes_per_launch: N"), null when it is absent.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "gemv4_4096x12288_hbm_traffic.txt")
REPLAYS = 21


GEMM_PROFILE = os.path.join(ROOT, "profiles", "gemm_m256_4096x12288_kernel_trace_and_counters.txt")


def _profile_value(path, key, cast=float):
    """A figure a profiler run left in profiles/ as a line "key: value" (None when absent)."""
    try:
        for line in open(path):
            if line.startswith(key + ":"):
                return cast(line.split(":", 1)[1].split()[0])
    except (OSError, ValueError, IndexError):
        pass
    return None


def _traffic_from_profile():
    return _profile_value(TRAFFIC_FILE, "traffic_bytes_per_launch", int)


def _weights(torch, N, K, gen, dev, lut_dtype):
    """A synthetic idx4 weight: uniform random blob bytes are uniform indices (the
    blob is a permutation of the logical nibbles); LUT ~ N(0, 0.02) sorted ascending."""
    blob = torch.randint(0, 256, (N * K // 2,), dtype=torch.uint8, device=dev, generator=gen)
    lut = (torch.randn(N // GS, 16, device=dev, generator=gen) * 0.02).sort(dim=1).values
    return blob, lut.to(lut_dtype).contiguous()


def _desc(_lib, blob, lut, N, K):
    d = _lib.FluteLinear()
    d.q1, d.lut1, d.q1_bytes = blob.data_ptr(), lut.data_ptr(), blob.numel()
    d.N, d.K, d.b1, d.group_size, d.lut_rows = N, K, 4, GS, lut.shape[0]
    d.lut_dtype = _lib.F16 if str(lut.dtype) == "torch.float16" else _lib.BF16
    return d


def _time_graph(torch, fn, reps=REPLAYS):
    """Capture fn() (a sequence of launches on the current stream) once, replay it `reps`
    times, return the median elapsed milliseconds of one replay."""
    fn()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fn()
    graph.replay()
    torch.cuda.synchronize()
    times = []
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1))
    times.sort()
    return times[len(times) // 2]


def _cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _cpu_baseline(torch):
    """The upstream reference path through the oracle, on the host cores, bounded samples:
    (i) as shipped: unpack the blob, gather the LUT, fp32 matmul on every call
        (scripts/palettized_modules.py:811-824, 1241-1251 upstream);
    (ii) cached logical indices: gather + matmul (:668-705);
    (iii) cached fp32 weight: the matmul alone, the best case.
    The headline workload (M = 1, 4096 -> 12288) gives `value`; the first configuration
    (4096 -> 4096, fp16) is listed with all three variants."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import flute_oracle as O
    import numpy as np

    def sample(fn, budget, at_least=3, at_most=40):
        fn()
        times, t_end = [], time.perf_counter() + budget
        while (time.perf_counter() < t_end or len(times) < at_least) and len(times) < at_most:
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
        times.sort()
        return times[len(times) // 2], len(times)

    def variants(N, K, dtype, budget):
        g = torch.Generator().manual_seed(N + K)
        blob = torch.randint(0, 256, (N * K // 2,), dtype=torch.uint8, generator=g).numpy()
        lut = (torch.randn(N // GS, 16, generator=g) * 0.02).sort(dim=1).values.half()
        x = torch.randn(1, K, generator=g).to(dtype)
        nbytes = N * K // 2 + lut.numel() * 2
        idx = torch.from_numpy(O.unpack_idxn(blob, N, K, 4).astype(np.int64))
        rows = torch.arange(N) // GS
        W = lut[rows].float().gather(1, idx)
        out = {}
        for name, fn in (
                ("as_shipped", lambda: O.linear_reference(x, blob, lut, N, K, GS, 4)),
                ("cached_indices", lambda: (x.float() @ lut[rows].float().gather(1, idx).t()).to(dtype)),
                ("cached_fp32_weight", lambda: (x.float() @ W.t()).to(dtype))):
            med, n = sample(fn, budget)
            out[name] = {"ms_per_call": round(med * 1e3, 3), "gbs_index_plus_lut": round(nbytes / med / 1e9, 4),
                         "calls": n}
        return out

    head = variants(I, H, torch.bfloat16, 4.0)
    first = variants(H, H, torch.float16, 2.0)
    return {"value": head["as_shipped"]["gbs_index_plus_lut"], "unit": "GB/s",
            "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"M=1 4096->12288 idx4 gs128, fp16 LUT, bf16 activations, upstream reference path as "
                      f"shipped (unpack + gather + fp32 matmul per call), median of "
                      f"{head['as_shipped']['calls']} calls, {head['as_shipped']['ms_per_call']} ms/call",
            "cpu_model": _cpu_model(), "os_cpu_count": os.cpu_count(),
            "torch_threads": torch.get_num_threads(),
            "variants_4096x12288_bf16": head, "variants_config0_4096x4096_fp16": first}


def _oracle_rows(O, blob, lut, K, tile, bits=4):
    """The 128 rows of one tile, dequantised by the oracle from the blob bytes (fp64)."""
    per = (K // 64) * 1024 * bits
    sub = blob[tile * per:(tile + 1) * per].cpu().numpy()
    return O.dequant(sub, lut[tile:tile + 1].cpu(), 128, K, GS, bits).double()


PARITY_GATE = 1e-3


def _parity(got, exact, act, what):
    """Two figures for a checked block of outputs: against the reference forward at the same
    rounding point (the fp32 sum rounded once to the output type: what upstream's forward
    returns, scripts/palettized_modules.py:1235-1251), gated at 1e-3, and against the
    unrounded fp64 value, beside what that one rounding costs by itself."""
    ref_same = exact.float().to(act).double()
    err = _rel(got, ref_same)
    if not err <= PARITY_GATE:
        raise SystemExit(f"bench.py: parity gate failed for {what}: {err:.2e} against the reference "
                         f"forward (gate {PARITY_GATE:g})")
    return {"parity_rel_l2": err, "vs_unrounded_fp64": _rel(got, exact),
            "output_rounding_alone": _rel(ref_same, exact)}


def _rel(got, ref):
    return float(((got - ref) ** 2).sum() / (ref ** 2).sum()) ** 0.5


class _Gemv:
    """flute_gemv over a rotation of weights of one shape, parity-gated against the oracle."""

    def __init__(self, torch, _lib, ctypes, O, dev):
        self.torch, self.lib, self.ct, self.O, self.dev = torch, _lib, ctypes, O, dev

    def run(self, name, descs, keep, N, K, x, xref=None, split=0, launches=None, keep2=None, bits2=0,
            rows_of=None, wbytes=None):
        """keep[i] = (blob, lut) of descs[i] (keep2: the second stream's); xref: the row the
        weights see (the rotated x for a fused rotation), default x.  rows_of(tile): the fp64
        rows of one 128-row tile of weight 0 where they are not the N-grouped dequantisation;
        wbytes: the bytes of one weight where they are not indices + N-grouped LUT."""
        torch, _lib, ctypes = self.torch, self.lib, self.ct
        act = x.dtype
        code = _lib.BF16 if act == torch.bfloat16 else _lib.F16
        y = torch.zeros(1, N, dtype=act, device=self.dev)

        def call(i):
            st = _lib.lib.flute_gemv(ctypes.byref(descs[i % len(descs)]), x.data_ptr(), y.data_ptr(),
                                     code, split, torch.cuda.current_stream().cuda_stream)
            if st != 0:
                raise RuntimeError(_lib.last_error())

        call(0)
        torch.cuda.synchronize()
        blob, lut = keep[0]
        xr = (x if xref is None else xref).cpu().double()
        tiles = sorted({0, (N // 128) // 2, N // 128 - 1})

        def rows(t):
            if rows_of is not None:
                return rows_of(t)
            w = _oracle_rows(self.O, blob, lut, K, t)
            if keep2 is not None:
                w = w + _oracle_rows(self.O, keep2[0][0], keep2[0][1], K, t, bits2)
            return w
        exact = torch.cat([xr @ rows(t).t() for t in tiles], 1)
        got = torch.cat([y[:, t * 128:(t + 1) * 128] for t in tiles], 1).cpu().double()
        res = _parity(got, exact, act, name)
        n = launches or max(96, len(descs))
        ms = _time_graph(torch, lambda: [call(i) for i in range(n)])
        us = ms / n * 1e3
        given = wbytes is not None
        wbytes = wbytes if given else N * K // 2 + (N // GS) * 32
        if keep2 is not None and not given:
            wbytes += N * K * bits2 // 8 + (N // GS) * (2 << bits2)
        res.update({"us_per_call": round(us, 3), "gbs_index_plus_lut": round(wbytes / us / 1e3, 1),
                    "frac_hbm_peak": round(wbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                    "launches_per_replay": n, "weights_in_rotation": len(descs),
                    "rotation_mib": len(descs) * wbytes >> 20})
        return res


def _read_probe(torch, _lib, dev, keep):
    """What one launch that only reads the 24 MiB of a weight's index blob reaches (same
    rotation of cold blobs, same graph timing as the headline): the level the GEMV's launch can
    be read against.  Grid size and loads in flight swept, best taken."""
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    nbytes = keep[0][0].numel()
    best = None
    for wgs in (768, 1536, 3072):
        for pf in (4, 8):
            def call(i, wgs=wgs, pf=pf):
                st = _lib.lib.flute_read_probe(keep[i % len(keep)][0].data_ptr(), nbytes, wgs, pf,
                                               sink.data_ptr(), torch.cuda.current_stream().cuda_stream)
                if st != 0:
                    raise RuntimeError(_lib.last_error())
            n = max(96, len(keep))
            us = _time_graph(torch, lambda: [call(i) for i in range(n)], reps=7) / n * 1e3
            if best is None or us < best[0]:
                best = (us, wgs, pf)
    us, wgs, pf = best
    return {"us_per_call": round(us, 3), "gbs": round(nbytes / us / 1e3, 1),
            "frac_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4), "bytes": nbytes,
            "workgroups": wgs, "loads_in_flight": pf, "parity_rel_l2": 0.0,
            "what": "flute_read_probe: 16-byte non-temporal loads only, no table, no arithmetic"}


def _copy_desc(_lib, ctypes, d):
    c = _lib.FluteLinear()
    ctypes.memmove(ctypes.byref(c), ctypes.byref(d), ctypes.sizeof(c))
    return c


def _other_m1(torch, _lib, ctypes, O, dev, gen, gv, gate, keep, down, keep_down, x):
    """The other M = 1 rows: the first configuration (4096 -> 4096, fp16 activations), the
    headline launch on one weight only (cache-resident), a (4, 1) two-stream weight (what
    upstream's deployed artifacts are), the Hadamard rotation fused into the prologue (blocks
    of 128 columns, and upstream's form over the descending power-of-two segments of K, on
    both MLP shapes), the lm_head shape, and the narrow shapes of the split-K configuration
    (the library's own choice and K splits 1/2/4/8)."""
    out = {}
    # configs[0]: M = 1, 4096 -> 4096, fp16 LUT, fp16 activations, cold (8 MiB each)
    count0 = int(3.1 * 256 * 2 ** 20 // (H * H // 2)) + 1
    ws = [_weights(torch, H, H, gen, dev, torch.float16) for _ in range(count0)]
    x16 = torch.randn(1, H, device=dev, generator=gen).to(torch.float16)
    out["gemv_config0_4096x4096_fp16"] = gv.run("config0", [_desc(_lib, b, l, H, H) for b, l in ws], ws,
                                                H, H, x16)
    del ws
    out["gemv_4096x12288_cache_resident"] = gv.run("cache_resident", gate[:1], keep[:1], I, H, x)
    out["read_probe_24MiB_cold"] = _read_probe(torch, _lib, dev, keep)
    # (4, 1) two streams: a 1-bit second stream with its own two-entry LUT
    two, keep2 = [], []
    for g_ in gate:
        q2 = torch.randint(0, 256, (I * H // 8,), dtype=torch.uint8, device=dev, generator=gen)
        l2 = (torch.randn(I // GS, 2, device=dev, generator=gen) * 0.005).sort(dim=1).values \
            .to(torch.float16).contiguous()
        d = _copy_desc(_lib, ctypes, g_)
        d.q2, d.lut2, d.q2_bytes, d.b2 = q2.data_ptr(), l2.data_ptr(), q2.numel(), 1
        two.append(d)
        keep2.append((q2, l2))
    out["gemv_4096x12288_two_streams_4_1"] = gv.run("two_streams", two, keep, I, H, x, keep2=keep2, bits2=1)
    # (1, 4): the same operands with the streams in the other order (upstream's most frequent pair)
    one_four = []
    for d4, (q1b, l1b) in zip(gate, keep2):
        d = _copy_desc(_lib, ctypes, d4)
        d.q2, d.lut2, d.q2_bytes, d.b2 = d4.q1, d4.lut1, d4.q1_bytes, 4
        d.q1, d.lut1, d.q1_bytes, d.b1 = q1b.data_ptr(), l1b.data_ptr(), q1b.numel(), 1
        one_four.append(d)
    both = lambda t: (_oracle_rows(O, keep[0][0], keep[0][1], H, t) +
                      _oracle_rows(O, keep2[0][0], keep2[0][1], H, t, 1))
    out["gemv_4096x12288_two_streams_1_4"] = gv.run(
        "two_streams_1_4", one_four, keep, I, H, x, rows_of=both,
        wbytes=I * H // 2 + (I // GS) * 32 + I * H // 8 + (I // GS) * 4)
    del two
    # LUT grouped along K: one row of 16 values per (output row, 128-wide K group), [N, K/128, 16]
    # (a form no upstream artifact has; bytes = indices + that LUT = 37,748,736 at 4096 -> 12288)
    def k_grouped(name, descs, blobs, N, K, xin):
        kluts = [(torch.randn(N, K // 128, 16, device=dev, generator=gen) * 0.02).sort(dim=2).values
                 .to(torch.float16).contiguous() for _ in descs]
        kds = []
        for g_, kl in zip(descs, kluts):
            d = _copy_desc(_lib, ctypes, g_)
            d.lut1, d.lut_rows, d.k_group, d.lut_dtype = kl.data_ptr(), N * (K // 128), 128, _lib.F16
            kds.append(d)

        def krows(t):
            per = (K // 64) * 1024 * 4
            idx = torch.from_numpy(O.unpack_idxn(blobs[0][0][t * per:(t + 1) * per].cpu().numpy(), 128, K, 4)).long()
            lk = kluts[0][t * 128:(t + 1) * 128].cpu().double()           # [128, K/128, 16]
            grp = (torch.arange(K) // 128)[None, :].expand(128, K)
            return lk[torch.arange(128)[:, None].expand(128, K), grp, idx]
        res = gv.run(name, kds, blobs, N, K, xin, rows_of=krows, wbytes=N * K // 2 + N * (K // 128) * 32)
        res["bytes_index_plus_lut"] = N * K // 2 + N * (K // 128) * 32
        return res
    out["gemv_4096x12288_lut_grouped_along_k"] = k_grouped("k_grouped_lut", gate, keep, I, H, x)
    out["gemv_12288x4096_lut_grouped_along_k"] = k_grouped(
        "k_grouped_lut_down", down, keep_down, H, I, torch.randn(1, I, device=dev, generator=gen).to(x.dtype))
    ws0 = [_weights(torch, H, H, gen, dev, torch.float16) for _ in range(count0)]
    out["gemv_config0_4096x4096_fp16_lut_grouped_along_k"] = k_grouped(
        "config0_k_grouped_lut", [_desc(_lib, b, l, H, H) for b, l in ws0], ws0, H, H, x16)
    del ws0
    # fused rotations
    signs = (torch.randint(0, 2, (H,), device=dev, generator=gen).float() * 2 - 1).contiguous()
    signs_d = (torch.randint(0, 2, (I,), device=dev, generator=gen).float() * 2 - 1).contiguous()
    xd_ = torch.randn(1, I, device=dev, generator=gen).to(x.dtype)

    def rotated(descs, sg, block):
        res = []
        for g_ in descs:
            d = _copy_desc(_lib, ctypes, g_)
            d.signs, d.rot_block = sg.data_ptr(), block
            res.append(d)
        return res
    out["gemv_4096x12288_fht128_fused"] = gv.run(
        "fht128", rotated(gate, signs, 128), keep, I, H, x,
        xref=O.block_fht_reference(x.cpu(), 128, signs.cpu()).to(x.dtype))
    out["gemv_4096x12288_fht_full_k_fused"] = gv.run(
        "fht_full_k_up", rotated(gate, signs, 0), keep, I, H, x, xref=O.fht_reference(x.cpu(), signs.cpu()))
    # what a deployed weight is: a (1, 4) pair behind upstream's full-K rotation
    out["gemv_4096x12288_two_streams_1_4_fht_full_k_fused"] = gv.run(
        "two_streams_1_4_fht_full_k", rotated(one_four, signs, 0), keep, I, H, x,
        xref=O.fht_reference(x.cpu(), signs.cpu()), rows_of=both,
        wbytes=I * H // 2 + (I // GS) * 32 + I * H // 8 + (I // GS) * 4)
    del keep2, one_four
    out["gemv_12288x4096_plain"] = gv.run("down_plain", down, keep_down, H, I, xd_)
    out["gemv_12288x4096_fht_full_k_fused"] = gv.run(
        "fht_full_k_down", rotated(down, signs_d, 0), keep_down, H, I, xd_,
        xref=O.fht_reference(xd_.cpu(), signs_d.cpu()))
    NV = 248320                                    # lm_head: 0.5 GB of indices, two in rotation
    ws = [_weights(torch, NV, H, gen, dev, torch.float16) for _ in range(2)]
    out["gemv_lm_head_4096x248320"] = gv.run("lm_head", [_desc(_lib, b, l, NV, H) for b, l in ws], ws,
                                             NV, H, x, launches=12)
    del ws
    for N in (1024, 512):
        count = int(3.1 * 256 * 2 ** 20 // (N * H // 2)) + 1
        ws = [_weights(torch, N, H, gen, dev, torch.float16) for _ in range(count)]
        ds = [_desc(_lib, b, l, N, H) for b, l in ws]
        res = gv.run(f"narrow{N}", ds, ws, N, H, x)
        res["split_chosen"] = int(_lib.lib.flute_pick_split(N, H))
        res["us_per_call_forced_split"] = {
            str(sp): gv.run(f"narrow{N}/split{sp}", ds, ws, N, H, x, split=sp)["us_per_call"]
            for sp in (1, 2, 4, 8)}
        out[f"gemv_narrow_4096x{N}"] = res
        del ws, ds
    return out


def _mlp_block(torch, _lib, ctypes, O, dev, gen, sets, x, act, steps):
    """Second configuration: one token through gate+up (one merged launch with SiLU*mul)
    and down; bytes = indices + LUTs + x, h written and read, y."""
    h = torch.zeros(1, I, dtype=act, device=dev)
    y = torch.zeros(1, H, dtype=act, device=dev)

    def block(s):
        st = _lib.lib.flute_mlp_block(ctypes.byref(s["g"]), ctypes.byref(s["u"]), ctypes.byref(s["d"]),
                                      x.data_ptr(), h.data_ptr(), y.data_ptr(), _lib.BF16,
                                      torch.cuda.current_stream().cuda_stream)
        if st != 0:
            raise RuntimeError(_lib.last_error())

    def gate_up(s):
        st = _lib.lib.flute_gemv_mlp(ctypes.byref(s["g"]), ctypes.byref(s["u"]), x.data_ptr(),
                                     h.data_ptr(), _lib.BF16, 0, torch.cuda.current_stream().cuda_stream)
        if st != 0:
            raise RuntimeError(_lib.last_error())

    block(sets[0])
    torch.cuda.synchronize()
    (gb, gl), (ub, ul), (db, dl) = sets[0]["t"]
    xd, hd = x.cpu().double(), h.cpu().double()
    ref_h = torch.cat([O.silu_mul_exact(xd @ _oracle_rows(O, gb, gl, H, t).t(),
                                        xd @ _oracle_rows(O, ub, ul, H, t).t()) for t in (0, 37, 95)], 1)
    got_h = torch.cat([hd[:, t * 128:(t + 1) * 128] for t in (0, 37, 95)], 1)
    ref_y = torch.cat([hd @ _oracle_rows(O, db, dl, I, t).t() for t in (0, 13, 31)], 1)
    got_y = torch.cat([y.cpu().double()[:, t * 128:(t + 1) * 128] for t in (0, 13, 31)], 1)
    par_h, par_y = _parity(got_h, ref_h, act, "MLP block h"), _parity(got_y, ref_y, act, "MLP block y")
    n = len(sets)
    ms_step = _time_graph(torch, lambda: [block(sets[i % n]) for i in range(steps)]) / steps
    ms_gu = _time_graph(torch, lambda: [gate_up(sets[i % n]) for i in range(steps)]) / steps
    lut_bytes = (I // GS) * 32
    bytes_gate_up = 2 * (I * H // 2 + lut_bytes) + H * 2 + I * 2
    bytes_down = H * I // 2 + (H // GS) * 32 + I * 2 + H * 2
    gbs = (bytes_gate_up + bytes_down) / (ms_step * 1e-3) / 1e9
    return {"workload": "fused MLP decode M=1: gate+up 4096->12288 (merged, SiLU*mul) + down "
                        "12288->4096, idx4, group 128, fp16 LUT, bf16 activations, cold weights",
            "us_per_block": round(ms_step * 1e3, 3), "gbs": round(gbs, 1),
            "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4), "bytes_per_block": bytes_gate_up + bytes_down,
            "gate_up_kernel": {"us_per_launch": round(ms_gu * 1e3, 3), "bytes": bytes_gate_up,
                               "gbs": round(bytes_gate_up / ms_gu / 1e6, 1),
                               "frac_hbm_peak": round(bytes_gate_up / ms_gu / 1e6 / HBM_PEAK_GBS, 4)},
            "parity": {"h": par_h, "y": par_y, "gate": PARITY_GATE},
            "weight_sets": n}


def _gemm_section(torch, _lib, ctypes, O, dev, gen, sets):
    """The second half of the metric: C[M, N] = A[M, K] @ W^T on idx4 blobs with a bf16 LUT,
    bf16 activations, bf16 MFMA with fp32 accumulate, for both shapes of the configuration
    (4096 -> 12288 and 12288 -> 4096) at M = 16 / 64 / 256 / 1024.  One call = flute_gemm as
    a caller sees it, its activation pre-pass included.  M >= 256 is priced against the
    matrix-core peak, M = 16 and 64 against HBM (index + LUT + A + C bytes): that is the
    roof that binds there."""
    shapes = {}
    for N, K, which in ((I, H, 0), (H, I, 2)):
        blobs = [s["t"][which][0] for s in sets]
        luts = [(torch.randn(N // GS, 16, device=dev, generator=gen) * 0.02).sort(dim=1).values
                .to(torch.bfloat16).contiguous() for _ in sets]
        descs = [_desc(_lib, b, l, N, K) for b, l in zip(blobs, luts)]
        rows = {}
        for M in (256, 16, 64, 1024):
            A = torch.randn(M, K, device=dev, generator=gen).to(torch.bfloat16)
            C = torch.empty(M, N, dtype=torch.bfloat16, device=dev)

            def call(i):
                st = _lib.lib.flute_gemm(ctypes.byref(descs[i % len(descs)]), A.data_ptr(), C.data_ptr(),
                                         M, K, N, _lib.BF16, torch.cuda.current_stream().cuda_stream)
                if st != 0:
                    raise RuntimeError(_lib.last_error())

            call(0)
            torch.cuda.synchronize()
            tiles = (0, (N // 128) // 2 - 1, N // 128 - 1)
            Ad = A.cpu().double()
            ref = torch.cat([Ad @ _oracle_rows(O, blobs[0], luts[0], K, t).t() for t in tiles], 1)
            got = torch.cat([C[:, t * 128:(t + 1) * 128] for t in tiles], 1).cpu().double()
            par = _parity(got, ref, torch.bfloat16, f"GEMM {K}->{N}, M={M}")
            n = 48
            us = _time_graph(torch, lambda: [call(i) for i in range(n)]) / n * 1e3
            tf = 2.0 * M * N * K / us / 1e6
            nbytes = N * K // 2 + (N // GS) * 32 + 2 * M * (K + N)
            rows[M] = {"us_per_call": round(us, 2), "tflops": round(tf, 1),
                       "frac_mfma": round(tf / MFMA_PEAK_TFLOPS, 4),
                       "gbs": round(nbytes / us / 1e3, 1), "frac_hbm": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                       "bound": "mfma" if M >= 256 else "hbm", **par}
        shapes[f"{K}x{N}"] = rows
    # the rotated-input configuration at M = 8: block-128 Hadamard rotation of the rows in
    # front of the 4096 -> 12288 GEMM, fp16 LUT, bf16 activations
    M, N, K = 8, I, H
    blob = sets[0]["t"][0][0]
    lut = sets[0]["t"][0][1]
    signs = (torch.randint(0, 2, (H,), device=dev, generator=gen).float() * 2 - 1).contiguous()
    rot = []
    for s_ in sets:
        r = _lib.FluteLinear()
        ctypes.memmove(ctypes.byref(r), ctypes.byref(s_["g"]), ctypes.sizeof(r))
        r.signs, r.rot_block = signs.data_ptr(), 128
        rot.append(r)
    A = torch.randn(M, K, device=dev, generator=gen).to(torch.bfloat16)
    C = torch.empty(M, N, dtype=torch.bfloat16, device=dev)

    def call_rot(i):
        st = _lib.lib.flute_gemm(ctypes.byref(rot[i % len(rot)]), A.data_ptr(), C.data_ptr(), M, K, N,
                                 _lib.BF16, torch.cuda.current_stream().cuda_stream)
        if st != 0:
            raise RuntimeError(_lib.last_error())

    call_rot(0)
    torch.cuda.synchronize()
    Ar = O.block_fht_reference(A.cpu(), 128, signs.cpu()).to(torch.bfloat16).double()
    tiles = (0, 41, 95)
    ref = torch.cat([Ar @ _oracle_rows(O, blob, lut, K, t).t() for t in tiles], 1)
    got = torch.cat([C[:, t * 128:(t + 1) * 128] for t in tiles], 1).cpu().double()
    par = _parity(got, ref, torch.bfloat16, "rotated GEMM M=8")
    us = _time_graph(torch, lambda: [call_rot(i) for i in range(48)]) / 48 * 1e3
    head = shapes[f"{H}x{I}"][256]
    return {"workload": "LUT-GEMM M=256: 4096->12288, idx4, group 128, bf16 LUT, bf16 activations, bf16 "
                        "MFMA fp32 accumulate; whole flute_gemm call (activation pre-pass + kernel)",
            "value": head["tflops"], "unit": "TFLOP/s", "peak": MFMA_PEAK_TFLOPS, "frac": head["frac_mfma"],
            "us_per_call": head["us_per_call"], "parity_rel_l2": head["parity_rel_l2"],
            "parity_gate": PARITY_GATE,
            "roofline": {"bound": "mfma", "achieved": head["tflops"], "peak": MFMA_PEAK_TFLOPS,
                         "unit": "TFLOP/s", "frac": head["frac_mfma"],
                         "flop_per_call": 2 * 256 * I * H,
                         "kernels": "gemm_prep_quad_kernel (activation image) + gemm_kernel<4, 4, 2, true, 4, "
                                    "true, false, true> (192 workgroups of eight wavefronts)",
                         "from_profiles": {
                             "source": "profiles/gemm_m256_4096x12288_kernel_trace_and_counters.txt (rocprofv3 "
                                       "runs of this command in an earlier process, not this run)",
                             "gemm_kernel_avg_ns": _profile_value(GEMM_PROFILE, "gemm_kernel_avg_ns"),
                             "prep_kernel_avg_ns": _profile_value(GEMM_PROFILE, "prep_kernel_avg_ns"),
                             "mfma_busy_frac_of_kernel_on_active_simds":
                                 _profile_value(GEMM_PROFILE, "mfma_busy_frac"),
                             "cus_occupied": _profile_value(GEMM_PROFILE, "cus_occupied", int),
                             "shader_clock_ghz_in_loop": _profile_value(GEMM_PROFILE, "shader_clock_ghz")}},
            "shapes": {k: {str(m): v[m] for m in (16, 64, 256, 1024)} for k, v in shapes.items()},
            "rotated_input_M8": {"us_per_call": round(us, 2), **par,
                                 "workload": "M=8, block-128 Hadamard rotation of the input + LUT-GEMM "
                                             "4096->12288, fp16 LUT, bf16 activations"}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=340)
    ap.add_argument("--warmup", type=int, default=34)
    ap.add_argument("--weights", type=int, default=34,
                    help="distinct 4096->12288 weights in rotation (24 MiB each; 34 = 850 MB)")
    ap.add_argument("--sets", type=int, default=12, help="MLP weight sets (72 MiB each)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-gemm", action="store_true", help="skip the M>1 LUT-GEMM section")
    ap.add_argument("--no-extra", action="store_true",
                    help="skip the MLP block and the other M=1 configurations")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch one plain 64 MiB device copy, so that a counter run of this "
                         "command holds a kernel of known traffic to scale FETCH_SIZE/WRITE_SIZE by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus must be 1 (the path shards along N "
              "without any exchange between devices)", file=sys.stderr)
        return 2

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    from flute_extended import _lib          # fails loudly if libflute_hip.so is missing
    import ctypes
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import flute_oracle as O                 # the checker of the parity gates only
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev).manual_seed(1234)
    act = torch.bfloat16

    # MLP weight sets: their gate and up projections are also the first 4096 -> 12288 weights
    # of the headline rotation
    sets = []
    for _ in range(args.sets):
        g, u, d = (_weights(torch, I, H, gen, dev, torch.float16),
                   _weights(torch, I, H, gen, dev, torch.float16),
                   _weights(torch, H, I, gen, dev, torch.float16))
        sets.append(dict(t=(g, u, d), g=_desc(_lib, *g, I, H), u=_desc(_lib, *u, I, H),
                         d=_desc(_lib, *d, H, I)))
    keep = [s["t"][0] for s in sets] + [s["t"][1] for s in sets]
    gate = [s["g"] for s in sets] + [s["u"] for s in sets]
    while len(gate) < args.weights:
        b, l = _weights(torch, I, H, gen, dev, torch.float16)
        keep.append((b, l))
        gate.append(_desc(_lib, b, l, I, H))
    gate, keep = gate[:max(args.weights, 1)], keep[:max(args.weights, 1)]
    x = torch.randn(1, H, device=dev, generator=gen).to(act)

    if args.calibrate_copy:
        src = torch.randint(0, 255, (64 << 20,), dtype=torch.uint8, device=dev, generator=gen)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()

    # ---- headline: the GEMV 4096 -> 12288, cold --------------------------------------
    gv = _Gemv(torch, _lib, ctypes, O, dev)
    y = torch.zeros(1, I, dtype=act, device=dev)
    for i in range(args.warmup):
        _lib.lib.flute_gemv(ctypes.byref(gate[i % len(gate)]), x.data_ptr(), y.data_ptr(), _lib.BF16, 0,
                            torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    head = gv.run("gemv_4096x12288", gate, keep, I, H, x, launches=args.steps)
    us = head["us_per_call"]
    wbytes = I * H // 2 + (I // GS) * 32
    alg_bytes = wbytes + H * 2 + I * 2
    value = wbytes / us / 1e3
    achieved = alg_bytes / us / 1e3
    touched = min(args.steps, len(gate))

    out = {
        "metric": "M=1 LUT-GEMV achieved HBM GB/s (% of peak); M=256 LUT-GEMM TFLOP/s (% MFMA)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(us * 1e-3, 6), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32 accumulate, f16 LUT, bf16 act",
        "data": "synthetic",
        "config": {"workload": "M=1 LUT-GEMV, MLP up-projection K=4096 -> N=12288, idx4, group 128, fp16 "
                               "LUT, bf16 activations, cold weights (the timed graph walks "
                               f"{touched} distinct weights = {touched * wbytes >> 20} MiB"
                               + ("" if touched * wbytes >= 3 * 256 * 2 ** 20 else
                                  ", less than three times the 256 MB memory-side cache: raise --steps "
                                  "to 32 or more for the full rotation") + ")",
                   "value_counts": "packed index + LUT bytes", "bytes_per_step": wbytes,
                   "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
                   "timing": f"hipGraph of {args.steps} launches, median of {REPLAYS} replays, events on "
                             "the launch stream",
                   "parity_rel_l2": head["parity_rel_l2"], "parity_gate": PARITY_GATE,
                   "parity_against": "the reference forward at the same rounding point (fp32 sum, one "
                                     "rounding to bf16), three 128-row tiles",
                   "vs_unrounded_fp64": head["vs_unrounded_fp64"],
                   "output_rounding_alone": head["output_rounding_alone"]},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": _traffic_from_profile(),
                     "traffic_source": "profiles/gemv4_4096x12288_hbm_traffic.txt: FETCH_SIZE + WRITE_SIZE "
                                       "counter runs of this command in an earlier process, not this run",
                     "kernel": "gemv4_kernel<5, 4, 4, false> (16 rows per workgroup, 768 workgroups)",
                     "us_per_launch": us, "algorithmic_bytes_per_launch": alg_bytes},
    }
    if not args.no_gemm:
        out["gemm"] = _gemm_section(torch, _lib, ctypes, O, dev, gen, sets)
    if not args.no_extra:
        out["mlp_block"] = _mlp_block(torch, _lib, ctypes, O, dev, gen, sets, x, act, 240)
        out["other_m1_configs"] = _other_m1(torch, _lib, ctypes, O, dev, gen, gv, gate, keep,
                                            [s_["d"] for s_ in sets], [s_["t"][2] for s_ in sets], x)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = _cpu_baseline(torch)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
