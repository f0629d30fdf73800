#!/usr/bin/env python3
"""Decode-step benchmark of the QVB8 dequantize-inside-the-matmul path on one MI355X.

A "step" is one token through the projections of a Qwen-9B-shape decoder (32 layers x q/k/v/o/gate/up/down, QVB8 at
tau = 1e-3, bf16 activations, M = 1) through the C-ABI entry point qvb8_mma, on packs that are resident in HBM before
the clock starts (5+ GB of distinct buffers, so nothing is served from cache).  Projections fed the same activation
(q+k+v, gate+up) are concatenated at load and run as one launch each (128 launches per step; --no-fuse: 224).  The step is captured once in a
HIP graph and replayed; `value` is the algorithmic bytes of a step (packed ids + row metadata + escapes + activations
in and out) divided by the measured time per step.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers 32] [--no-cpu] [--no-fuse] [--copy-probe]

Prints ONE JSON line.  `roofline` covers the dominant kernel (the tile kernel, every launch of the step):
algorithmic bytes per launch / average launch time, timed with HIP events on the launch stream over the timed region.
`cpu_baseline` is the CPU restatement of the reference's Python restore followed by a torch fp32 matmul, on a bounded
sample of the same workload (its first projections, about 12 s of CPU work), on the host cores of this machine.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
LAYER_9B = (("q", 4096, 4096), ("k", 1024, 4096), ("v", 1024, 4096), ("o", 4096, 4096),
            ("gate", 12288, 4096), ("up", 12288, 4096), ("down", 4096, 12288))
TAU = 1e-3
# HBM bytes per launch of the tile kernel from hardware counters (FETCH_SIZE scaled by 2.0 against a plain 1 GiB pass,
# plus WRITE_SIZE), as recorded in profiles/tile_kernel_9b_decode_step_hbm_traffic.md: {workgroups: bytes}
MEASURED_TRAFFIC = {256: (2 * 16078.3 + 39.8) * 1024, 64: (2 * 2014.4 + 4.9) * 1024}
MMA_FLAGS = int(os.environ.get("QVB8_BENCH_MMA_FLAGS", "1"))     # 1 = QVB8_MMA_SATURATE_X: the operator's default for bf16 x


def algorithmic_bytes(enc, M):
    """Bytes one product has to move: packed ids, 17 bytes of row metadata per row (min_s, tau_s, nbits, bit_off), 12
    per escape, the bf16 activations in and the bf16 results out."""
    ids = enc["ids"] if "ids" in enc else enc["ids_host"]
    return int(ids.numel() + 17 * enc["Q"] + 12 * enc["esc_idx"].numel() + 2 * M * enc["P"] + 2 * M * enc["Q"])


SAME_INPUT = (("q", "k", "v"), ("gate", "up"))          # projections fed the same activation: one launch each when fused


def build_layers(n_layers, dev, fuse):
    """Per layer: the encoded projections (kept for byte counts and the CPU leg) and the launch units made of them: one
    QVBandLinearV8 per projection, or one per same-input group when `fuse` (rows concatenated, results split as views)."""
    import torch
    from qvb8_amd.formats.qvb8 import pack as PK
    from qvb8_amd.formats.qvb8.fuse import concat_linears
    from qvb8_amd.formats.qvb8.module import QVBandLinearV8
    layers, units = [], []
    for li in range(n_layers):
        encs, mods = [], {}
        for pi, (name, Q, P) in enumerate(LAYER_9B):
            g = torch.Generator(device=dev).manual_seed(1000 * li + pi)
            W = (0.02 * torch.randn(Q, P, device=dev, generator=g)).to(torch.bfloat16)
            enc = PK.encode_tensor(W, TAU, restore="fp16")
            assert enc["max_err"] < TAU, (name, enc["max_err"])
            enc["name"] = name
            del W
            encs.append(enc)
            mods[name] = QVBandLinearV8.from_encoded(enc)
        layers.append(encs)
        done = set()
        for name, _, _ in LAYER_9B:
            if name in done:
                continue
            group = next((g for g in SAME_INPUT if name in g), (name,)) if fuse else (name,)
            lin = concat_linears([mods[n] for n in group])[0] if len(group) > 1 else mods[name]
            done.update(group)
            perm, rowinfo = lin._mma_order()
            units.append(dict(name="+".join(group), lin=lin, perm=perm, rowinfo=rowinfo, Q=lin.out_features,
                              P=lin.in_features, n_esc=lin.esc_idx.numel(),
                              Y=torch.empty((1, lin.out_features), dtype=torch.float32, device=dev),
                              bytes=sum(algorithmic_bytes(e, 1) for e in encs if e["name"] in group)))
        if fuse:
            for enc in encs:                          # the separate device copies are not needed any more
                if any(enc["name"] in g for g in SAME_INPUT):
                    enc["ids_host"] = enc["ids"].cpu()
                    del enc["ids"]
        mods.clear()
    return layers, units


def cpu_baseline(layers, x_by_p, budget_s=12.0):
    """Restore (CPU restatement of the reference's Python decode) + torch fp32 matmul, projection by projection in
    workload order, until about `budget_s` seconds of CPU work are done."""
    import numpy as np
    import torch
    from oracle import qvb8_oracle as O
    nbytes, done, dt = 0, [], 0.0
    for enc in (e for lay in layers for e in lay):
        d = {k: enc[k].cpu().numpy() for k in ("min_s", "tau_s", "nbits", "bit_off", "esc_idx", "esc_vals")}
        d["ids"] = (enc["ids_host"] if "ids_host" in enc else enc["ids"].cpu()).numpy()
        x = x_by_p[enc["P"]].float().cpu()
        t1 = time.perf_counter()
        ids = O.unpack_bits_rows(d["ids"], d["nbits"].astype(np.int64), d["bit_off"], enc["Q"], enc["P"])
        Wr = O.reconstruct(d["min_s"], d["tau_s"], ids, d["esc_idx"], d["esc_vals"])
        y = x @ torch.from_numpy(Wr).T
        assert y.shape == (1, enc["Q"])
        dt += time.perf_counter() - t1                   # restore + product only: the copies to host are not CPU work of the path
        nbytes += algorithmic_bytes(enc, 1)
        done.append(enc["name"])
        if dt >= budget_s:
            break
    return {"value": round(nbytes / dt / 1e9, 6), "unit": "GB/s", "cores": int(torch.get_num_threads()), "kind": "port",
            "sample": "numpy restore + torch fp32 matmul (M=1) of the first %d projections of the workload (%s; %.1f MB "
                      "packed) in %.1f s; the restore is single-threaded numpy, the matmul uses torch's threads"
                      % (len(done), ",".join(done), nbytes / 1e6, dt)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-fuse", action="store_true",
                    help="one launch per projection (7 per layer) instead of one per same-input group (q+k+v, gate+up: 4)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain elementwise pass over 1 GiB in and 1 GiB out (torch.add on 2^28 floats): the "
                         "known-size kernel that hardware byte counters of a profiler run are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path runs on ONE GPU (no collectives are part of it); run with --gpus 1", file=sys.stderr)
        return 2

    import torch
    from qvb8_amd import _lib
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    lib = _lib.load()                                       # raises when the HIP library is missing: no fallback
    layers, units = build_layers(args.layers, dev, fuse=not args.no_fuse)
    g = torch.Generator(device=dev).manual_seed(7)
    x_by_p = {P: torch.randn(1, P, device=dev, generator=g).to(torch.bfloat16) for P in (4096, 12288)}
    flat = [enc for lay in layers for enc in lay]
    step_bytes = sum(algorithmic_bytes(e, 1) for e in flat)
    assert step_bytes == sum(u["bytes"] for u in units)
    n_launch = len(units)

    def step():
        s = torch.cuda.current_stream().cuda_stream
        for u in units:
            x, lin = x_by_p[u["P"]], u["lin"]
            rc = lib.qvb8_mma(x.data_ptr(), _lib.dtype_code(x.dtype), 1, lin.ids.data_ptr(), lin.ids.numel(),
                              lin.min_s.data_ptr(), lin.tau_s.data_ptr(), lin.nbits.data_ptr(), lin.bit_off.data_ptr(),
                              u["Q"], u["P"], lin.esc_idx.data_ptr() if u["n_esc"] else None,
                              lin.esc_vals.data_ptr() if u["n_esc"] else None, u["n_esc"],
                              u["perm"].data_ptr(), u["rowinfo"].data_ptr(), MMA_FLAGS, u["Y"].data_ptr(), None, 0, s)
            if rc != 0:
                raise RuntimeError(lib.qvb8_last_error().decode())

    if args.copy_probe:
        src = torch.ones(1 << 28, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1.0, out=dst)
        torch.cuda.synchronize()
        del src, dst
    step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for _ in range(args.warmup):
        graph.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()                                             # the graph replays on this (the current) stream
    for _ in range(args.steps):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ev_ms = e0.elapsed_time(e1)
    ms_per_step = max(wall * 1e3, ev_ms) / args.steps
    gbs = step_bytes / (ms_per_step * 1e-3) / 1e9
    launch_us = ev_ms * 1e3 / (args.steps * n_launch)
    achieved = (step_bytes / n_launch) / (launch_us * 1e-6) / 1e9
    esc = sum(e["esc_idx"].numel() for e in flat)

    out = {
        "metric": "dequant-GEMV HBM GB/s (% of peak) + decode tokens/s, 9B-shape pack, 1 MI355X",
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 activations x fp32 band value, fp32 accumulate", "data": "synthetic",
        "tokens_per_s": round(1e3 / ms_per_step, 2), "pct_of_hbm_peak": round(100.0 * gbs / HBM_PEAK_GBS, 2),
        "config": {"workload": "Qwen-9B-shape decoder layer set (q/k/v/o 4096x4096 with k/v 1024, gate/up 12288, down "
                               "12288->4096), QVB8 tau=1e-3, bf16 activations, M=1, %d layers" % args.layers,
                   "launches_per_step": n_launch, "launch_units": "+".join(sorted({u["name"] for u in units}, key=len)),
                   "bytes_per_step": step_bytes, "escapes": esc,
                   "bits_per_weight": round(8.0 * sum(u["lin"].ids.numel() for u in units) / sum(e["Q"] * e["P"] for e in flat), 3)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": (round(sum(MEASURED_TRAFFIC[256 if e["Q"] >= 4096 else 64] for e in flat) / n_launch)
                                 if MMA_FLAGS == 1 and args.no_fuse else None),
                     "kernel": "qvb8::tile_kernel<1,4,false,true>", "bytes_per_launch": step_bytes // n_launch,
                     "launch_us": round(launch_us, 3)},
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(layers, x_by_p)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
