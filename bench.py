#!/usr/bin/env python3
"""Decode-step benchmark of the QVB8 dequantize-inside-the-matmul path on one MI355X.

A "step" is one token through the projections of a Qwen-9B-shape decoder (32 layers x q/k/v/o/gate/up/down, QVB8 at
tau = 1e-3, bf16 activations, M = 1) through the C-ABI entry point qvb8_mma, on packs that are resident in HBM before
the clock starts (5+ GB of distinct buffers, so nothing is served from cache).  Projections fed the same activation
(q+k+v, gate+up) are concatenated at load and run as one launch each (128 launches per step; --no-fuse: 224).  The step is captured once in a
HIP graph and replayed; `value` is the algorithmic bytes of a step (packed ids + row metadata + escapes + activations
in and out) divided by the measured time per step.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers N] [--no-cpu] [--no-fuse] [--no-sort] [--copy-probe]
                    [--workload decode9b|smallm|moe|qvb8r|lmhead|embed|attn|floor|mlp] [--tokens T]

Prints ONE JSON line.  `roofline` covers the dominant kernel (the tile kernel, every launch of the step):
algorithmic bytes per launch / average launch time, timed with HIP events on the launch stream over the timed region.
`cpu_baseline` is the CPU restatement of the reference's Python restore followed by a torch fp32 matmul, on a bounded
sample of the same workload (its first projections, about 12 s of CPU work), on the host cores of this machine.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
LAYER_9B = (("q", 4096, 4096), ("k", 1024, 4096), ("v", 1024, 4096), ("o", 4096, 4096),
            ("gate", 12288, 4096), ("up", 12288, 4096), ("down", 4096, 12288))
# 27B-class dense shapes (hidden 5120, FFN 17408; q/o 5120, k/v 1024 as in the 9B set): `--model 27b`, not the headline
LAYER_27B = (("q", 5120, 5120), ("k", 1024, 5120), ("v", 1024, 5120), ("o", 5120, 5120),
             ("gate", 17408, 5120), ("up", 17408, 5120), ("down", 5120, 17408))
TAU = 1e-3
def measured_figure(profile, key, kernel):
    """{class: value} of the `<key> <kernel> <class> <value>` lines of a summary under profiles/ ({} without the file)."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", profile)
    out = {}
    try:
        with open(path) as fh:
            for line in fh:
                f = line.split()
                if len(f) == 4 and f[0] == key and f[1] == kernel:
                    out[f[2]] = float(f[3])
    except OSError:
        pass
    return out


def measured_traffic(profile, kernel):
    """HBM bytes per launch by launch class: the `traffic_bytes_per_launch <kernel> <class> <bytes>` lines of a summary under
    profiles/ (hardware counters, recorded there with the commands that took them)."""
    return {k: int(v) for k, v in measured_figure(profile, "traffic_bytes_per_launch", kernel).items()}


SETTLE_MS = float(os.environ.get("QVB8_BENCH_SETTLE_MS", "120"))      # untimed replays before every timed region, see time_graph
MMA_FLAGS = int(os.environ.get("QVB8_BENCH_MMA_FLAGS", "1"))     # 1 = QVB8_MMA_SATURATE_X: the operator's default for bf16 x


def mma_flags(lin) -> int:
    """The flags the operator passes for this weight: 8 = QVB8_MMA_PLANES when its rows were stored in planes at load."""
    return MMA_FLAGS | (8 if lin._planes else 0)


def tile_traffic(units, n_launch, model="9b"):
    """Mean measured HBM bytes per launch of the step's launch mix (None when the counters' summary is not there)."""
    t = measured_traffic("tile_kernel_%s_decode_step_hbm_traffic.md" % model, "tile_kernel")
    if any(u["name"] not in t for u in units):
        return None
    return round(sum(t[u["name"]] for u in units) / n_launch)


def algorithmic_bytes(enc, M):
    """Bytes one product has to move: packed ids, 17 bytes of row metadata per row (min_s, tau_s, nbits, bit_off), 12
    per escape, the bf16 activations in and the results counted as bf16 (2 bytes each; the timed kernel writes them as
    fp32, 4 bytes each, which is more than is counted here -- 0.03 % of a projection's bytes)."""
    ids = enc["ids"] if "ids" in enc else enc["ids_host"]
    return int(ids.numel() + 17 * enc["Q"] + 12 * enc["esc_idx"].numel() + 2 * M * enc["P"] + 2 * M * enc["Q"])


def decode_metric_name(model):
    return "dequant-GEMV HBM GB/s (% of peak) + decode tokens/s, " + {"9b": "9B", "27b": "27B"}[model] + "-shape pack, 1 MI355X"


SAME_INPUT = (("q", "k", "v"), ("gate", "up"))          # projections fed the same activation: one launch each when fused


def build_layers(n_layers, dev, fuse, shapes=None):
    """Per layer: the encoded projections (kept for byte counts and the CPU leg) and the launch units made of them: one
    QVBandLinearV8 per projection, or one per same-input group when `fuse` (rows concatenated, results split as views)."""
    import torch
    from qvb8_amd.formats.qvb8 import pack as PK
    from qvb8_amd.formats.qvb8.fuse import concat_linears
    from qvb8_amd.formats.qvb8.module import QVBandLinearV8
    layers, units = [], []
    shapes = shapes or LAYER_9B
    for li in range(n_layers):
        encs, mods = [], {}
        for pi, (name, Q, P) in enumerate(shapes):
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
        for name, _, _ in shapes:
            if name in done:
                continue
            group = next((g for g in SAME_INPUT if name in g), (name,)) if fuse else (name,)
            lin = concat_linears([mods[n] for n in group])[0] if len(group) > 1 else mods[name]
            done.update(group)
            perm, rowinfo, layout = lin._mma_order()
            units.append(dict(name="+".join(group), lin=lin, perm=perm, rowinfo=rowinfo, layout=layout, Q=lin.out_features,
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


def time_graph(step, steps, warmup, spread=None):
    """Captures `step` (launches on torch's current stream) in a HIP graph, replays it `warmup` + `steps` times; returns
    (ms per step by HIP events on the replay stream, ms per step by the host clock).  With a dict as `spread`, every
    replay is bracketed by events of its own and the dict receives median / min / max of the replays in ms."""
    import torch
    step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for _ in range(warmup):
        graph.replay()
    torch.cuda.synchronize()
    # Untimed on top of the `warmup` replays asked for: replays until the GPU has been under this load for SETTLE_MS.  Right
    # after an idle stretch (pack building on the host) the first few dozen replays run 2-3 % slower than all later ones
    # (measured: three timed regions of 20 replays in a row 1.462, 1.458, 1.420 ms per step; 100 replays 1.423), which is the
    # machine settling, not the path under test.
    if SETTLE_MS > 0:
        t_settle = time.perf_counter()
        while (time.perf_counter() - t_settle) * 1e3 < SETTLE_MS:
            for _ in range(8):
                graph.replay()
            torch.cuda.synchronize()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1 if spread is not None else 2)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(steps):
        graph.replay()
        if spread is not None:
            marks[i + 1].record()
    if spread is None:
        marks[1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    if spread is not None:
        each = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(steps))
        spread.update(replays=steps, median_ms=round(each[len(each) // 2], 5), min_ms=round(each[0], 5), max_ms=round(each[-1], 5))
    return marks[0].elapsed_time(marks[-1]) / steps, wall * 1e3 / steps


def synthetic_routing(logits, k):
    """softmax -> top-k -> renormalise, the reference's router (run/run_inference.py:92-100): synthetic input of the MoE
    workload, built on the host before anything is timed."""
    import numpy as np
    z = np.asarray(logits, np.float64)
    z = z - z.max(-1, keepdims=True)
    p = np.exp(z)
    p /= p.sum(-1, keepdims=True)
    idx = np.argsort(-p, axis=-1, kind="stable")[:, :k]
    w = np.take_along_axis(p, idx, -1)
    return idx.astype(np.int64), (w / w.sum(-1, keepdims=True)).astype(np.float32)


def bench_moe(args, dev):
    """Config 4: Qwen-35B-A3B-shape MoE layer (hidden 2048, 128 experts of gate/up 2048->768 and down 768->2048, top-8
    routing from softmax of N(0,1) logits), QVB8 at tau = 2e-3, `--tokens` tokens.  A step = the expert stacks of
    `--layers` distinct layers through qvb8_moe_experts; bytes = packed ids + row metadata of the UNIQUE selected experts."""
    import numpy as np
    import torch
    from qvb8_amd import _lib
    from qvb8_amd.formats.qvb8 import pack as PK
    from qvb8_amd.formats.qvb8.backends_experts import QVBandExpertsV8
    from qvb8_amd.formats.qvb8.module import QVBandLinearV8
    lib = _lib.load()
    E, hidden, inter, k, T = 128, 2048, 768, 8, args.tokens
    stacks = []
    for l in range(args.layers):
        gu, dn = [], []
        for e in range(E):
            g = torch.Generator(device=dev).manual_seed(100000 * l + e)
            Wg = (0.02 * torch.randn(2 * inter, hidden, device=dev, generator=g)).to(torch.bfloat16)
            Wd = (0.02 * torch.randn(hidden, inter, device=dev, generator=g)).to(torch.bfloat16)
            gu.append(QVBandLinearV8.from_encoded(PK.encode_tensor(Wg, 2e-3)))
            dn.append(QVBandLinearV8.from_encoded(PK.encode_tensor(Wd, 2e-3)))
        if l == 0:                                    # an expert's bytes as encoded (the stack may store rows wider)
            encoded_bytes_per_expert = sum(int(lin.ids.numel()) for lin in gu + dn) // E
        m = QVBandExpertsV8(gu, dn, num_experts=E)
        assert m.build_stack()
        stacks.append(m._stk)
    rng = np.random.default_rng(7)
    x = torch.randn(T, hidden, device=dev, generator=torch.Generator(device=dev).manual_seed(7)).to(torch.bfloat16)
    out = torch.empty(T, hidden, dtype=torch.bfloat16, device=dev)
    ws = torch.empty(lib.qvb8_moe_workspace_bytes(T, k, E, 2 * inter, inter, hidden), dtype=torch.uint8, device=dev)
    # Every layer is called with several routings in turn (each its own random draw), until a step touches more than
    # 512 MB of distinct expert bytes: a replay then cannot be served from the 256 MB last-level cache.
    calls, step_bytes = [], 0
    per_expert = encoded_bytes_per_expert + 17 * (stacks[0][0]["Q"] + stacks[0][1]["Q"])
    rounds = 0
    while step_bytes < (512 << 20) and rounds < 16:
        for g_, d_ in stacks:
            idx, w = synthetic_routing(rng.normal(size=(T, E)), k)
            calls.append((g_, d_, torch.from_numpy(idx).to(dev), torch.from_numpy(w).to(dev)))
            step_bytes += len(np.unique(idx)) * per_expert + 2 * T * hidden * 2
        rounds += 1
    n_calls = len(calls)

    def step():
        s = torch.cuda.current_stream().cuda_stream
        for g_, d_, idx, w in calls:
            rc = lib.qvb8_moe_experts(x.data_ptr(), 2, T, idx.data_ptr(), w.data_ptr(), k, E,
                                      g_["ids"].data_ptr(), g_["ids"].numel(), g_["min_s"].data_ptr(), g_["tau_s"].data_ptr(),
                                      g_["nbits"].data_ptr(), g_["bit_off"].data_ptr(), g_["Q"], g_["P"],
                                      d_["ids"].data_ptr(), d_["ids"].numel(), d_["min_s"].data_ptr(), d_["tau_s"].data_ptr(),
                                      d_["nbits"].data_ptr(), d_["bit_off"].data_ptr(), d_["Q"], d_["P"],
                                      (0x100 if g_["regular"] else 0) | (0x200 if d_["regular"] else 0),   # what the operator passes
                                      out.data_ptr(), 2, ws.data_ptr(), ws.numel(), s)
            if rc != 0:
                raise RuntimeError(lib.qvb8_last_error().decode())
    spread = {}
    ev_ms, wall_ms = time_graph(step, args.steps, args.warmup, spread)
    ms = max(ev_ms, wall_ms)
    gbs = step_bytes / (ms * 1e-3) / 1e9
    per_layer_us = ev_ms * 1e3 / n_calls
    return {"metric": "expert-gathered fused decode-GEMV GB/s on the bytes of the unique selected experts, 35B-A3B-shape MoE "
                      "layer, 1 MI355X",
            "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(ms, 5), "spread": spread, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16 activations narrowed to fp16 x fp32 band value, fp32 accumulate", "data": "synthetic",
            "config": {"workload": "MoE layer: hidden 2048, 128 experts gate/up 2048->768 + down 768->2048, top-8, QVB8 "
                                   "tau=2e-3, %d token(s), %d layers x %d routings per step" % (T, args.layers, rounds),
                       "bytes_per_step": step_bytes, "us_per_layer": round(per_layer_us, 2)},
            "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(gbs / HBM_PEAK_GBS, 4),
                         # HBM bytes of one layer's launches from hardware counters, where the summary holds this token count
                         "traffic": measured_traffic("moe_kernels_35b_a3b_layer_kernel_trace.md", "moe_layer").get("tokens=%d" % T),
                         "kernel": ("qvb8::moe_one_kernel<4,false,..> + moe_one_kernel<6,true,..> (one layer = 2 launches)" if T <= 6 else
                                    "qvb8::moe_plan_kernel + moe_walk_kernel<4,false,..> + moe_walk_kernel<6,true,..> + "
                                    "moe_combine_kernel (one layer = 4 launches)" if T <= 16 else
                                    "qvb8::moe_plan_kernel + moe_gemv_kernel<0> + moe_gemv_kernel<1> + moe_combine_kernel "
                                    "(one layer = 4 launches)"),
                         "bytes_per_launch": step_bytes // n_calls, "launch_us": round(per_layer_us, 3)},
            "cpu_baseline": None}


QVB8R_SHAPES = {"27b": ("hidden 5120 / FFN 17408 (gate, up, down)", ((17408, 5120), (17408, 5120), (5120, 17408))),
                "65b": ("hidden 8192 / FFN 28672 (up 8192->28672, down 28672->8192)", ((28672, 8192), (8192, 28672)))}


def bench_qvb8r(args, dev, token_counts=None):
    """Config 5: large-dense shapes as QVB8R at tau = 2e-3, `--tokens` rows (1..48): `--model 65b` (default here) hidden 8192 /
    FFN 28672, `--model 27b` hidden 5120 / FFN 17408.  A step = the shapes' tensors of `--layers` layers through
    qvb8r_gemv; bytes = coded words + states + slot tables + row metadata.  With `token_counts` the packs are built once
    and one result per token count is returned."""
    import ctypes
    import torch
    from qvb8_amd import _lib, ext_qvb8r
    from qvb8_amd.formats.qvb8 import pack as PK
    from qvb8_amd.formats.qvb8r import pack as RP
    from qvb8_amd.formats.qvb8r.module import QVBandLinearV8R
    lib = _lib.load()
    shape_name, shapes = QVB8R_SHAPES[args.model if args.model in QVB8R_SHAPES else "65b"]
    units, coded_bytes, n_sym = [], 0, 0
    for l in range(args.layers):
        for pi, (Q, P) in enumerate(shapes):
            g = torch.Generator(device=dev).manual_seed(5000 + 10 * l + pi)
            W = (0.02 * torch.randn(Q, P, device=dev, generator=g)).to(torch.bfloat16)
            d = RP.transcode(PK.encode_tensor(W, 2e-3, keep_ids=True))
            del W
            lin = QVBandLinearV8R(d, device=dev)
            core, _, _ = ext_qvb8r._core(*lin._core(), P)
            units.append(dict(lin=lin, core=core, Q=Q, P=P, seed=5000 + 10 * l + pi))
            coded_bytes += 4 * len(d["words"]) + 8 * 32 * len(d["tiles"]) + 4 * 4096 * d["K"] + 12 * Q + 8 * Q
            n_sym += Q * P
            del d
    # the ceiling of this path, measured in the same run on the same packs: the launches of the one-row kernel with the
    # activations and the multiply-adds taken out (qvb8r_walk_probe), i.e. the entropy decode alone
    for u in units:
        u["Yp"] = torch.empty(1, u["Q"], dtype=torch.float32, device=dev)

    def walk_only():
        s = torch.cuda.current_stream().cuda_stream
        for u in units:
            if lib.qvb8r_walk_probe(ctypes.byref(u["core"]), u["lin"].T, u["Yp"].data_ptr(), s) != 0:
                raise RuntimeError(lib.qvb8_last_error().decode())
    walk_ms = max(time_graph(walk_only, args.steps, args.warmup))
    walk_tsym = n_sym / (walk_ms * 1e-3) / 1e12
    results = [_time_qvb8r(args, dev, lib, units, M, coded_bytes, n_sym, shape_name, walk_tsym) for M in (token_counts or [args.tokens])]
    return results if token_counts else results[0]


def _time_qvb8r(args, dev, lib, units, M, coded_bytes, n_sym, shape_name, walk_tsym):
    import ctypes
    import torch
    step_bytes = coded_bytes + sum(2 * M * (u["P"] + u["Q"]) for u in units)
    for u in units:
        g = torch.Generator(device=dev).manual_seed(u["seed"])
        u["x"] = torch.randn(M, u["P"], device=dev, generator=g).to(torch.bfloat16)
        u["Y"] = torch.empty(M, u["Q"], dtype=torch.float32, device=dev)
        u["ws"] = torch.empty(lib.qvb8r_gemv_workspace_bytes(M, u["P"]), dtype=torch.uint8, device=dev)

    def step():
        s = torch.cuda.current_stream().cuda_stream
        for u in units:
            rc = lib.qvb8r_gemv(u["x"].data_ptr(), 2, M, ctypes.byref(u["core"]), u["lin"].T, u["Y"].data_ptr(),
                                u["ws"].data_ptr(), u["ws"].numel(), s)
            if rc != 0:
                raise RuntimeError(lib.qvb8_last_error().decode())
    spread = {}
    ev_ms, wall_ms = time_graph(step, args.steps, args.warmup, spread)
    ms = max(ev_ms, wall_ms)
    gbs = step_bytes / (ms * 1e-3) / 1e9
    launch_us = ev_ms * 1e3 / len(units)
    # HBM bytes per launch of the one-row kernel from hardware counters (profiles/): the mean over the shapes' tensors
    key = "65b" if "8192" in shape_name else "27b"
    r_traffic = measured_traffic("r_gemv_kernel_65b_ffn_trace_and_counters.md" if key == "65b" else "r_gemv_kernel_27b_ffn_kernel_trace.md",
                                 "r_gemv_kernel").get(key) if M == 1 else None
    kernel = "qvb8::r_gemv_kernel<2>" if M == 1 else "qvb8::r_mma_kernel<%d, false> (+ r_pack_x_kernel)" % ((M + 15) // 16)
    return {"metric": "QVB8R fused entropy-decode + GEMV GB/s on coded bytes, large-dense FFN shapes, 1 MI355X",
            "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(ms, 5), "spread": spread, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16 activations x fp32 band value (M > 1: exact fp16 operands on the matrix cores), fp32 accumulate",
            "data": "synthetic",
            "config": {"workload": "QVB8R tau=2e-3, %s, M=%d, %d layers" % (shape_name, M, args.layers),
                       "bytes_per_step": step_bytes, "bits_per_weight": round(8.0 * step_bytes / n_sym, 3),
                       "symbols_per_s": round(n_sym / (ms * 1e-3), 1)},
            "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": r_traffic,
                         "kernel": kernel,
                         "bytes_per_launch": step_bytes // len(units), "launch_us": round(launch_us, 3),
                         "note": "the walk is bound by its instruction count (vector ALU 91 % busy), not by HBM"},
            "roofline_walk": {"bound": "the entropy decode alone: the same launches with the activations and the multiply-adds taken out "
                                       "(qvb8r_walk_probe), timed in this run on these packs",
                              "achieved": round(n_sym / (ms * 1e-3) / 1e12, 4), "peak": round(walk_tsym, 4), "unit": "T symbols/s",
                              "frac": round(n_sym / (ms * 1e-3) / 1e12 / walk_tsym, 4)},
            "cpu_baseline": None}


def build_vocab_table(dev):
    """248320 x 5120 at tau = 1e-3 (the 27B-class model's vocabulary table, output head and embedding alike), as one
    QVBandLinearV8: encoded in eight slices of rows, then concatenated."""
    import torch
    from qvb8_amd.formats.qvb8 import pack as PK
    from qvb8_amd.formats.qvb8.fuse import concat_linears
    from qvb8_amd.formats.qvb8.module import QVBandLinearV8
    Q, P = 248320, 5120
    parts = []
    for i in range(0, Q, 31040):
        g = torch.Generator(device=dev).manual_seed(9000 + i)
        W = (0.02 * torch.randn(31040, P, device=dev, generator=g)).to(torch.bfloat16)
        enc = PK.encode_tensor(W, TAU, restore="fp16")
        assert enc["max_err"] < TAU
        parts.append(QVBandLinearV8.from_encoded(enc))
        del W, enc
    return concat_linears(parts)[0]


def bench_embed(args, dev):
    """Embedding read of `--tokens` rows (default 4096, a prefill's worth) from the 248320 x 5120 table, bf16 out.  A
    step = 16 launches of qvb8_lookup_rows, each with its own random rows and its own output (one graph replay costs
    the host about 20 us, more than one launch takes).  Bytes: the looked-up rows' packed ids + 16 bytes of row
    metadata + the row numbers in, the bf16 rows out."""
    import torch
    lib = __import__("qvb8_amd._lib", fromlist=["load"]).load()
    from qvb8_amd import _lib
    lin = build_vocab_table(dev)
    Q, P = lin.out_features, lin.in_features
    T = args.tokens if args.tokens > 1 else 4096
    reps = 16
    g = torch.Generator(device=dev).manual_seed(11)
    toks = [torch.randint(0, Q, (T,), device=dev, generator=g) for _ in range(reps)]
    outs = [torch.empty((T, P), dtype=torch.bfloat16, device=dev) for _ in range(reps)]
    n_esc = lin.esc_idx.numel()
    nbytes = sum(int((lin.nbits[t].to(torch.int64) * P // 8).sum()) for t in toks) // reps + T * (16 + 8) + 2 * T * P

    def step():
        for tok, out in zip(toks, outs):
            rc = lib.qvb8_lookup_rows(tok.data_ptr(), T, lin.ids.data_ptr(), lin.ids.numel(), lin.min_s.data_ptr(),
                                      lin.tau_s.data_ptr(), lin.nbits.data_ptr(), lin.bit_off.data_ptr(), Q, P,
                                      lin.esc_idx.data_ptr() if n_esc else None, lin.esc_vals.data_ptr() if n_esc else None,
                                      n_esc, _lib.BF16, out.data_ptr(), torch.cuda.current_stream().cuda_stream)
            if rc != 0:
                raise RuntimeError(lib.qvb8_last_error().decode())
    ev_ms, wall_ms = time_graph(step, args.steps, args.warmup)
    ms = max(ev_ms, wall_ms)
    us = ms * 1e3 / reps
    gbs = nbytes / (us * 1e-6) / 1e9
    return {"metric": "embedding read HBM GB/s, 248320 x 5120 table, 1 MI355X",
            "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "fp32 band value, bf16 out", "data": "synthetic",
            "config": {"workload": "embedding read of %d random rows, 248320 x 5120, QVB8 tau=1e-3, bf16 out, %d launches per step" % (T, reps),
                       "bytes_per_launch": nbytes, "rows_per_s": round(T / (us * 1e-6)), "escapes": n_esc},
            "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None, "kernel": "qvb8::decode_kernel<2, true>",
                         "bytes_per_launch": nbytes, "launch_us": round(us, 3)},
            "cpu_baseline": None}


def bench_lmhead(args, dev):
    """The largest single GEMV of the 27B-class model: the output head, 248320 x 5120 at tau = 1e-3, M = `--tokens` (1 by
    default): one launch of qvb8_mma per step over 1.1 GB of packed ids (far beyond the 256 MB last-level cache, so
    every replay streams from HBM).  Shows what the kernel streams when the fixed cost of a launch no longer matters."""
    import torch
    lib = __import__("qvb8_amd._lib", fromlist=["load"]).load()
    from qvb8_amd import _lib
    Q, P, M = 248320, 5120, args.tokens
    lin = build_vocab_table(dev)
    perm, rowinfo, layout = lin._mma_order()
    x = torch.randn(M, P, device=dev, generator=torch.Generator(device=dev).manual_seed(3)).to(torch.bfloat16)
    Y = torch.empty((M, Q), dtype=torch.float32, device=dev)
    n_esc = lin.esc_idx.numel()
    nbytes = int(lin.ids.numel() + 17 * Q + 12 * n_esc + 2 * M * P + 2 * M * Q)

    def step():
        rc = lib.qvb8_mma(x.data_ptr(), _lib.dtype_code(x.dtype), M, lin.ids.data_ptr(), lin.ids.numel(),
                          lin.min_s.data_ptr(), lin.tau_s.data_ptr(), lin.nbits.data_ptr(), lin.bit_off.data_ptr(), Q, P,
                          lin.esc_idx.data_ptr() if n_esc else None, lin.esc_vals.data_ptr() if n_esc else None, n_esc,
                          perm.data_ptr(), rowinfo.data_ptr(), ctypes.addressof(layout) if layout is not None else None,
                          mma_flags(lin), Y.data_ptr(), None, 0, torch.cuda.current_stream().cuda_stream)
        if rc != 0:
            raise RuntimeError(lib.qvb8_last_error().decode())
    ev_ms, wall_ms = time_graph(step, args.steps, args.warmup)
    ms = max(ev_ms, wall_ms)
    gbs = nbytes / (ms * 1e-3) / 1e9
    return {"metric": "dequant-GEMV HBM GB/s (% of peak), output head 248320 x 5120, 1 MI355X",
            "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16 activations x fp32 band value, fp32 accumulate", "data": "synthetic",
            "config": {"workload": "output head 248320 x 5120, QVB8 tau=1e-3, bf16 activations, M=%d, one launch per step" % M,
                       "bytes_per_step": nbytes, "bits_per_weight": round(8.0 * lin.ids.numel() / (Q * P), 3)},
            "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                         "kernel": "qvb8::tile_kernel<1,5,false,true>", "bytes_per_launch": nbytes, "launch_us": round(ev_ms * 1e3, 2)},
            "cpu_baseline": None}


def bench_attn(args, dev):
    """Decode-step attention over a banded KV cache: `--layers` (default 16) distinct caches of `--context` keys (default
    32768; 4 kv heads x 256 channels, 6-bit ids in bytes, segments of 4096 keys), 24 query heads, `--tokens` query
    tokens at the end of the context.  A step = per layer one launch of qvb8_attn_fwd plus one of qvb8_attn_combine,
    all in one graph; the kernel alone is timed by a second graph for the roofline.  Bytes per launch: the
    ids of K and V once, the per-channel constants, q, and the per-split results written."""
    import torch
    from qvb8_amd.kv import codec as KC, fused_attn as FA
    n, hkv, G, D, seg, MQ = args.context, 4, 6, args.head_dim, 4096, args.tokens
    gen = torch.Generator(device=dev).manual_seed(5)
    lays = []
    for li in range(args.layers):
        segs_k, segs_v, seg_len = [], [], []
        for a in range(0, n, seg):
            sl = min(seg, n - a)
            k = (torch.randn(hkv, sl, D, device=dev, generator=gen) * (0.5 + 2 * torch.rand(hkv, 1, D, device=dev, generator=gen))).to(torch.bfloat16)
            v = torch.randn(hkv, sl, D, device=dev, generator=gen).to(torch.bfloat16)
            segs_k.append(KC.band_kv_heads(k, torch.bfloat16, 6, certify=False))
            segs_v.append(KC.band_kv_heads(v, torch.bfloat16, 6, certify=False))
            seg_len.append(sl)
        lay = FA.layout_from_segments(segs_k, segs_v, seg_len, dev)
        if args.head_major:                                  # the same ids, every kv head's keys contiguous in memory
            lay.ki = lay.ki.permute(1, 0, 2).contiguous().permute(1, 0, 2)
            lay.vi = lay.vi.permute(1, 0, 2).contiguous().permute(1, 0, 2)
        lays.append(lay)
    lay0 = lays[0]
    rows = MQ * G
    tps, n_splits = FA.plan_splits(lay0.n_tiles, hkv, rows, dev, d=D)
    scale = D ** -0.5
    q = torch.randn(MQ, hkv * G, D, device=dev, generator=gen).to(torch.bfloat16)
    q16 = (q.float() * scale).clamp_(-65504.0, 65504.0).to(torch.float16).contiguous()
    o = [torch.empty(n_splits, hkv, rows, D, device=dev) for _ in lays]
    m = [torch.empty(n_splits, hkv, rows, device=dev) for _ in lays]
    l = [torch.empty_like(x) for x in m]
    outs = [None] * len(lays)

    def kernels_only():
        for i, lay in enumerate(lays):
            FA.fwd(q16, lay.ki, lay.vi, lay.kmin, lay.kstep, lay.vmin, lay.vstep, lay.kc, lay.vc, lay.t_start, lay.t_len,
                   lay.t_seg, o[i], m[i], l[i], n - MQ, tps, 1.0, G)

    def step():
        for i, lay in enumerate(lays):
            FA.fwd(q16, lay.ki, lay.vi, lay.kmin, lay.kstep, lay.vmin, lay.vstep, lay.kc, lay.vc, lay.t_start, lay.t_len,
                   lay.t_seg, o[i], m[i], l[i], n - MQ, tps, 1.0, G)
            outs[i] = FA.combine_splits(o[i], m[i], l[i], G)
    k_ms, _ = time_graph(kernels_only, args.steps, args.warmup)
    ev_ms, wall_ms = time_graph(step, args.steps, args.warmup)
    ms = max(ev_ms, wall_ms)
    n_seg = len(lay0.kc)
    nbytes = int(2 * lay0.ki.numel() * lay0.ki.element_size() + 4 * 4 * n_seg * hkv * D + 2 * MQ * hkv * G * D
                 + 4 * n_splits * hkv * rows * (D + 2) + 12 * lay0.n_tiles)
    us = k_ms * 1e3 / len(lays)
    gbs_kernel = nbytes / (us * 1e-6) / 1e9
    gbs = nbytes * len(lays) / (ms * 1e-3) / 1e9
    return {"metric": "banded-KV attention HBM GB/s, decode step over %d keys, 1 MI355X" % n,
            "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "fp16 restored keys and values, fp32 accumulate", "data": "synthetic",
            "config": {"workload": "attention of %d query token(s), 24 heads over %d kv heads x %d channels, %d keys as 6-bit ids "
                                   "in bytes in segments of %d, %d layers with their own caches, %d splits of %d tiles%s"
                                   % (MQ, hkv, D, n, seg, len(lays), n_splits, tps, ", head-major ids" if args.head_major else ""),
                       "bytes_per_launch": nbytes, "us_per_layer": round(ms * 1e3 / len(lays), 2)},
            "roofline": {"bound": "hbm", "achieved": round(gbs_kernel, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(gbs_kernel / HBM_PEAK_GBS, 4),
                         # FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 of one launch over 32768 keys (profiles/attn_kernels_*.md)
                         "traffic": round((2 * 33133.0 + 4168.1) * 1024) if (n, MQ, D) == (32768, 1, 256) else None,
                         "kernel": "qvb8::attn_kernel<%d, unsigned char, %d>" % (D, 1 if MQ * G <= 16 else 2 if (MQ * G <= 32 or D == 256) else 4), "bytes_per_launch": nbytes, "launch_us": round(us, 3)},
            "cpu_baseline": None}


def bench_mlp(args, dev):
    """One decoder layer's MLP at decode, both ways: qvb8_mlp (gate+up, SiLU, down in ONE launch, the hand-over inside the
    grid) against the two separate qvb8_mma launches on the same bytes.  `--layers` distinct MLPs of the `--model` shapes
    (9b: hidden 4096, inter 12288; 27b: 5120 / 17408) per graph replay; `value` is the one-launch path's GB/s on the packed
    bytes, config carries microseconds per layer of both."""
    import torch
    from qvb8_amd import _lib
    from qvb8_amd.formats.qvb8 import pack as PK
    from qvb8_amd.formats.qvb8.mlp import QVBandMLPV8
    from qvb8_amd.formats.qvb8.module import QVBandLinearV8
    lib = _lib.load()
    hidden, inter = (5120, 17408) if args.model == "27b" else (4096, 12288)
    M = max(1, min(4, args.tokens))
    mlps = []
    for li in range(args.layers):
        mods = []
        for pi, (Q, P) in enumerate(((inter, hidden), (inter, hidden), (hidden, inter))):
            g = torch.Generator(device=dev).manual_seed(1000 * li + pi)
            W = (0.02 * torch.randn(Q, P, device=dev, generator=g)).to(torch.bfloat16)
            mods.append(QVBandLinearV8.from_encoded(PK.encode_tensor(W, TAU, restore="fp16")))
            del W
        m = QVBandMLPV8(*mods)
        if not m.fused_ready:
            raise RuntimeError("bench mlp: the one-launch kernel cannot read this pack")
        mlps.append(m)
    x = torch.randn(M, hidden, device=dev, generator=torch.Generator(device=dev).manual_seed(7)).to(torch.bfloat16)
    xh = torch.randn(M, inter, device=dev, generator=torch.Generator(device=dev).manual_seed(8)).to(torch.bfloat16)
    Y = torch.empty(M, hidden, dtype=torch.bfloat16, device=dev)
    Ygu = torch.empty(M, 2 * inter, dtype=torch.bfloat16, device=dev)
    nbytes = sum(m.gate_up.ids.numel() + m.down.ids.numel() + 17 * (2 * inter + hidden) + 2 * M * (2 * hidden + inter) for m in mlps)

    def one_launch():
        s = torch.cuda.current_stream().cuda_stream
        for m in mlps:
            rc = lib.qvb8_mlp(ctypes.addressof(m._plan), x.data_ptr(), _lib.BF16, M, 0, _lib.BF16, Y.data_ptr(), _lib.BF16, m._ws.data_ptr(), s)
            if rc != 0:
                raise RuntimeError(lib.qvb8_last_error().decode())

    def product(lin, xin, out):
        perm, rowinfo, layout = lin._mma_order()
        rc = lib.qvb8_mma(xin.data_ptr(), _lib.BF16, M, lin.ids.data_ptr(), lin.ids.numel(), lin.min_s.data_ptr(), lin.tau_s.data_ptr(),
                          lin.nbits.data_ptr(), lin.bit_off.data_ptr(), lin.out_features, lin.in_features, None, None, 0,
                          perm.data_ptr(), rowinfo.data_ptr(), ctypes.addressof(layout), 1 | 4 | 8, out.data_ptr(), None, 0,
                          torch.cuda.current_stream().cuda_stream)
        if rc != 0:
            raise RuntimeError(lib.qvb8_last_error().decode())

    def separate():
        for m in mlps:
            product(m.gate_up, x, Ygu)
            product(m.down, xh, Y)
    fused_ms = min(max(time_graph(one_launch, args.steps, args.warmup)) for _ in range(2))
    sep_ms = min(max(time_graph(separate, args.steps, args.warmup)) for _ in range(2))
    if any(m.error_raised() for m in mlps):
        raise RuntimeError("bench mlp: a wait for H ran out")
    gbs = nbytes / (fused_ms * 1e-3) / 1e9
    return {"metric": "decoder-layer MLP at decode in one launch (gate+up, SiLU, down): GB/s on packed bytes, 1 MI355X",
            "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(fused_ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16 activations narrowed to fp16, ids as exact fp16 operands, fp32 accumulate", "data": "synthetic",
            "config": {"workload": "MLP hidden %d / inter %d, QVB8 tau=1e-3, M=%d, %d layers per replay" % (hidden, inter, M, args.layers),
                       "bytes_per_step": nbytes, "one_launch_us_per_layer": round(fused_ms * 1e3 / args.layers, 2),
                       "two_launches_us_per_layer": round(sep_ms * 1e3 / args.layers, 2)},
            "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None, "kernel": "qvb8::mlp_kernel<4,3,1,true>",
                         "bytes_per_launch": nbytes // args.layers, "launch_us": round(fused_ms * 1e3 / args.layers, 3)},
            "cpu_baseline": None}


def bench_floor(args, dev):
    """What a launch costs on this machine.  (1) A graph of 128 launches of a kernel with the tile kernel's launch shape
    (256 workgroups x 512 threads, 40 KB of LDS, the same scalar arguments) that does nothing: microseconds per graph
    node.  (2) The tile kernel itself (qvb8_mma, M = 1, bf16 x) on 4096-column weights of 4096, 2048, 1024 and 512 rows,
    128 launches per graph over distinct packs: time per launch against bytes per launch; the straight line through
    those points gives the fixed cost per launch (its value at zero bytes) and the rate the bytes stream at beyond it."""
    import numpy as np
    import torch
    from qvb8_amd import _lib
    from qvb8_amd.formats.qvb8 import pack as PK
    from qvb8_amd.formats.qvb8.module import QVBandLinearV8
    lib = _lib.load()
    n = 128

    def probe_step():
        s = torch.cuda.current_stream().cuda_stream
        for _ in range(n):
            if lib.qvb8_launch_probe(256, 512, 40960, s) != 0:
                raise RuntimeError(lib.qvb8_last_error().decode())
    ev, wall = time_graph(probe_step, args.steps, args.warmup)
    empty_us = max(ev, wall) * 1e3 / n
    P, points = 4096, []
    x = torch.randn(1, P, device=dev, generator=torch.Generator(device=dev).manual_seed(1)).to(torch.bfloat16)
    for Q in (4096, 2048, 1024, 512):
        n_packs = max(2, min(n, (600 << 20) // (Q * P * 7 // 8)))          # distinct packs: 600 MB, beyond the last-level cache
        units = []
        for i in range(n_packs):
            g = torch.Generator(device=dev).manual_seed(77 * Q + i)
            W = (0.02 * torch.randn(Q, P, device=dev, generator=g)).to(torch.bfloat16)
            lin = QVBandLinearV8.from_encoded(PK.encode_tensor(W, TAU, restore="fp16"))
            perm, rowinfo, layout = lin._mma_order()
            units.append((lin, perm, rowinfo, layout, torch.empty((1, Q), dtype=torch.float32, device=dev)))
        nbytes = sum(int(u[0].ids.numel() + 17 * Q + 2 * P + 2 * Q) for u in units) / len(units)

        def step():
            s = torch.cuda.current_stream().cuda_stream
            for i in range(n):
                lin, perm, rowinfo, layout, Y = units[i % len(units)]
                ne = lin.esc_idx.numel()
                rc = lib.qvb8_mma(x.data_ptr(), _lib.dtype_code(x.dtype), 1, lin.ids.data_ptr(), lin.ids.numel(), lin.min_s.data_ptr(),
                                  lin.tau_s.data_ptr(), lin.nbits.data_ptr(), lin.bit_off.data_ptr(), Q, P,
                                  lin.esc_idx.data_ptr() if ne else None, lin.esc_vals.data_ptr() if ne else None, ne, perm.data_ptr(),
                                  rowinfo.data_ptr(), ctypes.addressof(layout) if layout is not None else None, mma_flags(lin),
                                  Y.data_ptr(), None, 0, s)
                if rc != 0:
                    raise RuntimeError(lib.qvb8_last_error().decode())
        ev, wall = time_graph(step, args.steps, args.warmup)
        points.append((nbytes, max(ev, wall) * 1e3 / n))
        del units
    b = np.array([p[0] for p in points])
    t = np.array([p[1] for p in points])
    slope, intercept = np.polyfit(b, t, 1)
    return {"metric": "cost of a launch: graph node of an empty kernel, and the tile kernel's time per launch against its bytes, 1 MI355X",
            "value": round(empty_us, 3), "unit": "us per empty launch", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(empty_us * n * 1e-3, 5), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
            "dtype": "u8", "data": "synthetic",
            "config": {"workload": "128-node graphs: an empty kernel of 256 x 512 threads with 40 KB of LDS; qvb8_mma M=1 on Q x 4096 weights, Q = 4096, 2048, 1024, 512",
                       "tile_kernel_points": [{"bytes_per_launch": int(p[0]), "us_per_launch": round(p[1], 3)} for p in points],
                       "fixed_us_per_launch": round(float(intercept), 3), "streaming_GBs_beyond_fixed": round(1e-3 / float(slope), 1)},
            "roofline": None, "cpu_baseline": None}


def bench_smallm(args, dev, prebuilt=None, tokens=None):
    """Config 3: the 9B projections with M = `--tokens` rows (draft-verify / prefill chunk), through QVBandLinearV8's own
    dispatch: M <= 48 the tile kernel (X in registers), 49..256 the workgroup-tiled decode + GEMM kernel (X staged in LDS,
    ids decoded in registers), above that dense restore to fp16 + library GEMM.  Reports GB/s on the packed bytes and TFLOP/s (2 M Q P per projection, decode ops not counted)."""
    import torch
    if prebuilt is None:
        layers, units = build_layers(args.layers, dev, fuse=not args.no_fuse)
    else:
        layers, units = prebuilt
    n_layers = len(layers)
    M = args.tokens if tokens is None else tokens
    g = torch.Generator(device=dev).manual_seed(7)
    x_by_p = {P: torch.randn(M, P, device=dev, generator=g).to(torch.bfloat16) for P in (4096, 12288)}
    flat = [enc for lay in layers for enc in lay]
    step_bytes = sum(algorithmic_bytes(e, M) for e in flat)
    flops = sum(2.0 * M * e["Q"] * e["P"] for e in flat)
    for u in units:
        u["lin"](x_by_p[u["P"]])                                    # builds the per-weight launch data outside the graph

    def step():
        for u in units:
            u["out"] = u["lin"](x_by_p[u["P"]])
    spread = {}
    ev_ms, wall_ms = time_graph(step, args.steps, args.warmup, spread)
    ms = max(ev_ms, wall_ms)
    gbs = step_bytes / (ms * 1e-3) / 1e9
    tflops = flops / (ms * 1e-3) / 1e12
    # HBM bytes per layer and the matrix pipes' busy share, from hardware counters (profiles/, with the commands that took
    # them): present for the row counts that were profiled
    prof = "gemm_kernel_9b_small_m_trace_and_counters.md"
    per_layer = measured_figure(prof, "traffic_bytes_per_layer", "qvb8_mma").get("M=%d" % M)
    busy_cycles = measured_figure(prof, "mfma_busy_cycles_per_layer", "qvb8_mma").get("M=%d" % M)
    # SQ_VALU_MFMA_BUSY_CYCLES summed over the chip's 1024 SIMDs, against this run's time per layer at 2.0 GHz
    mfma_busy = None if busy_cycles is None else round(100.0 * busy_cycles / 1024.0 / (ms * 1e-3 / n_layers * 2.0e9), 2)
    path = ("fused decode + MFMA, X in registers (qvb8_mma, tile kernel)" if M <= 48 else
            "fused decode + MFMA GEMM, X staged in LDS (qvb8_mma, workgroup-tiled kernel)" if M <= 256 else "fp16 restore + library GEMM")
    bound = "hbm" if M <= 64 else "mfma"
    return {"metric": "small-M fused decode + GEMM: GB/s on packed bytes and TFLOP/s, 9B projections, 1 MI355X",
            "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(ms, 5), "spread": spread, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16 activations narrowed to fp16, ids as exact fp16 operands, fp32 accumulate, bf16 out", "data": "synthetic",
            "tflops": round(tflops, 3), "mfma_busy_pct": mfma_busy,
            "config": {"workload": "9B-shape projections, QVB8 tau=1e-3, M=%d, %d layers, path: %s" % (M, n_layers, path),
                       "bytes_per_step": step_bytes, "flops_per_step": flops, "launch_units": len(units)},
            "roofline": ({"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None if per_layer is None else int(per_layer),
                          "bytes_per_layer": step_bytes // n_layers}
                         if bound == "hbm" else
                         {"bound": "mfma", "achieved": round(tflops, 3), "peak": 2500.0, "unit": "TFLOP/s",
                          "frac": round(tflops / 2500.0, 5), "traffic": None if per_layer is None else int(per_layer),
                          "bytes_per_layer": step_bytes // n_layers}),
            "cpu_baseline": None}


def run_legs(args, dev, lib, layers, units):
    """Short runs of the other configurations, each on its own synthetic packs, appended to the headline's line under
    `legs`: the 9B projections with 16 / 64 / 256 rows (the first 8 layers of the headline's packs), the decode step on 8
    layers of the 27B-class shapes, the 35B-A3B-shape MoE layer with 1 and 8 tokens, the QVB8R FFN pair of the 65B and of the
    27B shapes with 1 and 16 rows.  Every leg is a HIP graph replayed at least 100 times, each replay between events of
    its own: `ms_per_step` is the mean of the timed region, `spread` the median and the extremes of the replays."""
    import copy
    import gc
    import torch
    keep = ("metric", "value", "unit", "ms_per_step", "spread", "steps", "warmup", "tflops", "mfma_busy_pct", "dtype",
            "roofline", "roofline_walk", "config")
    legs = {}
    sub = copy.copy(args)
    sub.steps, sub.warmup = max(100, args.steps), 3
    sub.copy_probe = False
    n8 = min(8, len(layers))
    per_layer = len(units) // len(layers)
    for M in (16, 64, 256):
        r = bench_smallm(sub, dev, prebuilt=(layers[:n8], units[:n8 * per_layer]), tokens=M)
        legs["smallm_M%d" % M] = {k: r[k] for k in keep if k in r}
    layers.clear()
    units.clear()
    gc.collect()
    torch.cuda.empty_cache()
    l27, u27 = build_layers(8, dev, fuse=True, shapes=LAYER_27B)
    r = time_decode(sub, dev, lib, l27, u27, LAYER_27B, "27b")[0]
    legs["decode27b"] = {k: r[k] for k in keep if k in r}
    del l27, u27, r
    gc.collect()
    torch.cuda.empty_cache()
    sub.layers = 2
    for T in (1, 8):
        sub.tokens = T
        r = bench_moe(sub, dev)
        legs["moe_T%d" % T] = {k: r[k] for k in keep if k in r}
        gc.collect()
        torch.cuda.empty_cache()
    sub.layers = 1
    for model, tag in (("65b", "qvb8r"), ("27b", "qvb8r27b")):
        sub.model = model
        for M, r in zip((1, 16), bench_qvb8r(sub, dev, token_counts=[1, 16])):
            legs["%s_M%d" % (tag, M)] = {k: r[k] for k in keep if k in r}
        gc.collect()
        torch.cuda.empty_cache()
    return legs


def time_decode(args, dev, lib, layers, units, shapes, model):
    """Times the decode step (one row of X through every launch unit of `layers`) as a replayed HIP graph: `args.steps`
    replays between one pair of events give the line's value; a second pass of at least 100 replays, each between events of
    its own, gives `spread`.  Returns (line, the function that launches a list of units, the activations by width)."""
    import torch
    from qvb8_amd import _lib
    g = torch.Generator(device=dev).manual_seed(7)
    x_by_p = {P: torch.randn(1, P, device=dev, generator=g).to(torch.bfloat16) for P in sorted({p for _, _, p in shapes})}
    flat = [enc for lay in layers for enc in lay]
    step_bytes = sum(algorithmic_bytes(e, 1) for e in flat)
    assert step_bytes == sum(u["bytes"] for u in units)
    n_launch = len(units)

    def run_units(which):
        s = torch.cuda.current_stream().cuda_stream
        for u in which:
            x, lin = x_by_p[u["P"]], u["lin"]
            rc = lib.qvb8_mma(x.data_ptr(), _lib.dtype_code(x.dtype), 1, lin.ids.data_ptr(), lin.ids.numel(),
                              lin.min_s.data_ptr(), lin.tau_s.data_ptr(), lin.nbits.data_ptr(), lin.bit_off.data_ptr(),
                              u["Q"], u["P"], lin.esc_idx.data_ptr() if u["n_esc"] else None,
                              lin.esc_vals.data_ptr() if u["n_esc"] else None, u["n_esc"],
                              u["perm"].data_ptr(), u["rowinfo"].data_ptr(),
                              ctypes.addressof(u["layout"]) if u["layout"] is not None else None,
                              mma_flags(lin), u["Y"].data_ptr(), None, 0, s)
            if rc != 0:
                raise RuntimeError(lib.qvb8_last_error().decode())

    def step():
        run_units(units)

    if getattr(args, "copy_probe", False):
        src = torch.ones(1 << 28, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1.0, out=dst)
        torch.cuda.synchronize()
        del src, dst
    ev_per_step, wall_per_step = time_graph(step, args.steps, args.warmup)
    ev_ms, wall = ev_per_step * args.steps, wall_per_step * args.steps * 1e-3
    ms_per_step = max(wall * 1e3, ev_ms) / args.steps
    spread = {}
    time_graph(step, max(100, args.steps), 2, spread)
    gbs = step_bytes / (ms_per_step * 1e-3) / 1e9
    launch_us = ev_ms * 1e3 / (args.steps * n_launch)
    achieved = (step_bytes / n_launch) / (launch_us * 1e-6) / 1e9
    esc = sum(e["esc_idx"].numel() for e in flat)
    n_layers = len(layers)
    fused = len(units) < len(flat)

    out = {
        "metric": decode_metric_name(model),
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "spread": spread, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": ("bf16 activations narrowed to fp16 (saturating), ids as exact fp16 matrix-core operands, fp32 accumulate, "
                  "row scale and offset applied in double, fp32 out"), "data": "synthetic",
        "tokens_per_s": round(1e3 / ms_per_step, 2), "pct_of_hbm_peak": round(100.0 * gbs / HBM_PEAK_GBS, 2),
        "config": {"workload": ("Qwen-9B-shape decoder layer set (q/k/v/o 4096x4096 with k/v 1024, gate/up 12288, down "
                                "12288->4096), QVB8 tau=1e-3, bf16 activations, M=1, %d layers" % n_layers) if model == "9b" else
                               ("27B-class decoder layer set (q/o 5120x5120, k/v 1024x5120, gate/up 17408, down 17408->5120), "
                                "QVB8 tau=1e-3, bf16 activations, M=1, %d layers" % n_layers),
                   "settle_ms": SETTLE_MS, "launches_per_step": n_launch, "launch_units": "+".join(sorted({u["name"] for u in units}, key=len)),
                   "bytes_per_step": step_bytes, "escapes": esc,
                   "bits_per_weight": round(8.0 * sum(u["lin"].ids.numel() for u in units) / sum(e["Q"] * e["P"] for e in flat), 3)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": tile_traffic(units, n_launch, model) if (MMA_FLAGS == 1 and fused) else None,
                     "kernel": "qvb8::tile_kernel<1,4,false,true,XP,PL> (XP = 1 or 4 pieces of X per thread through LDS; PL: rows stored in planes)" + (" / <1,5,false,true,XP,PL> for 5120-column rows" if model == "27b" else ""),
                     "bytes_per_launch": step_bytes // n_launch,
                     "launch_us": round(launch_us, 3)},
    }
    return out, run_units, x_by_p


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--layers", type=int, default=None, help="layers of distinct packs (default 32; moe 4; qvb8r 2)")
    ap.add_argument("--workload", choices=("decode9b", "smallm", "moe", "qvb8r", "lmhead", "embed", "attn", "floor", "mlp"), default="decode9b",
                    help="decode9b (default, the headline metric): 9B-shape decode step; moe: 35B-A3B-shape expert stack; "
                         "qvb8r: entropy-coded 27B-class FFN shapes; smallm: the 9B projections with --tokens rows (16, 64, 256); "
                         "lmhead / embed: the 248320 x 5120 vocabulary table; attn: decode-step attention over a banded KV cache; "
                         "floor: what a launch costs (empty-kernel graph, tile kernel time against bytes); "
                         "mlp: a layer's MLP in one launch (qvb8_mlp) against its two separate launches")
    ap.add_argument("--context", type=int, default=32768, help="keys in the cache of the attn workload")
    ap.add_argument("--head-major", action="store_true",
                    help="attn workload: ids stored (kv heads, keys, channels) instead of the reference's (keys, kv heads, channels)")
    ap.add_argument("--head-dim", type=int, default=256, choices=(128, 256), help="channels per head of the attn workload")
    ap.add_argument("--tokens", type=int, default=1, help="token rows for the moe / qvb8r workloads")
    ap.add_argument("--model", choices=("9b", "27b", "65b"), default="9b",
                    help="decode9b workload: layer shapes (9b = the headline configuration; 27b = hidden 5120, FFN 17408); "
                         "qvb8r workload: 65b (default there: hidden 8192, FFN 28672) or 27b")
    ap.add_argument("--no-legs", action="store_true",
                    help="decode9b workload: skip the short legs of the other configurations (small-M, MoE, QVB8R) that the "
                         "default run appends under `legs`")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-sort", action="store_true",
                    help="keep the file's row order in memory (row addresses are then read from the row records instead of "
                         "being computed from the width-sorted layout)")
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
    if args.layers is None:
        args.layers = {"decode9b": 32, "smallm": 8, "moe": 4, "qvb8r": 1, "lmhead": 1, "embed": 1, "attn": 16, "floor": 1, "mlp": 16}[args.workload]
    if args.workload != "decode9b":
        fn = {"moe": bench_moe, "qvb8r": bench_qvb8r, "smallm": bench_smallm, "lmhead": bench_lmhead, "embed": bench_embed, "attn": bench_attn, "floor": bench_floor, "mlp": bench_mlp}[args.workload]
        print(json.dumps(fn(args, dev)))
        return 0
    if args.no_sort:
        from qvb8_amd.formats.qvb8.module import QVBandLinearV8
        QVBandLinearV8.sort_rows = False
    if args.model == "65b":
        print("bench.py: --model 65b names QVB8R shapes (--workload qvb8r); the decode step takes 9b or 27b", file=sys.stderr)
        return 2
    shapes = LAYER_27B if args.model == "27b" else LAYER_9B
    layers, units = build_layers(args.layers, dev, fuse=not args.no_fuse, shapes=shapes)
    out, run_units, x_by_p = time_decode(args, dev, lib, layers, units, shapes, args.model)
    # GB/s per projection group: the launches of one kind over all layers, replayed on their own (not part of `value`)
    per = {}
    for name in sorted({u["name"] for u in units}, key=len):
        mine = [u for u in units if u["name"] == name]
        ev_g, wall_g = time_graph(lambda: run_units(mine), max(5, args.steps // 2), 2)
        us = max(ev_g, wall_g) * 1e3 / len(mine)
        b = sum(u["bytes"] for u in mine) / len(mine)
        per[name] = {"us_per_launch": round(us, 2), "GB/s": round(b / (us * 1e-6) / 1e9, 1), "bytes_per_launch": int(b)}
    out["per_projection"] = per
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(layers, x_by_p)
    else:
        out["cpu_baseline"] = None
    if not args.no_legs and args.model == "9b" and not args.no_fuse:
        out["legs"] = run_legs(args, dev, lib, layers, units)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
