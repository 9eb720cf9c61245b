#!/usr/bin/env python3
"""Benchmark of the packed-weight decode path on one MI355X.

Headline workload (BASELINE.json configs[1]): Llama-3-8B-shaped Q8_0 projections at M=1,
all seven projections of a layer, 32 layers streamed back-to-back.  One "step" is one
token's pass over the 32 layers (224 packed matrices, 7 415 529 472 weight bytes, every one
read once).  `value` is weight-bytes-effective GB/s of the whole step with all inputs
resident in HBM; tokens/s of the same stream is in `config`.

The JSON line also carries
  roofline      achieved HBM GB/s of the dominant kernel (algorithmic bytes per launch over
                its average launch duration, from HIP events on the launch stream)
                and, beside it, the library's pure read kernel on the same number of bytes
                (hbm_read_probe_GBps): what a launch of that size can stream on this device
  cpu_baseline  the NumPy restatement of the reference's packed CPU path (dequantise on every
                call, fp32 matmul) timed on this box's host cores on bounded samples, with the
                library's scalar C++ host twin, configs[0] and one MoE decode token as legs
  extras        other configurations measured the same way: the layer launched in data-flow
                order, other formats and token counts, MoE decode (cold rotation, and hot), the
                grouped decode call, the layer half, MoE prefill, the vocabulary projection

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras]
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

# (name, N, K) of the seven projections of one Llama-3-8B layer
PROJECTIONS = [("q", 4096, 4096), ("k", 1024, 4096), ("v", 1024, 4096), ("o", 4096, 4096),
               ("gate", 14336, 4096), ("up", 14336, 4096), ("down", 4096, 14336)]
BLOCKS = {"Q8_0": (32, 34), "Q5_K": (256, 176), "Q4_K": (256, 144), "Q6_K": (256, 210), "BF16": (1, 2)}


def weight_bytes(fmt, n, k):
    e, b = BLOCKS[fmt]
    return n * k // e * b


def device_blocks(torch, fmt, n, k, gen, device):
    """Synthetic packed matrix [n, k] generated on the device with the distribution the
    workload names (see mylocal_llm_amd/synthetic.py for the host twin)."""
    e, b = BLOCKS[fmt]
    nb = n * k // e
    blk = torch.empty((nb, b), dtype=torch.uint8, device=device)

    def scale(count):
        return (torch.randn(count, device=device, generator=gen) * 1e-4 + 5e-4).abs().to(torch.float16).view(torch.uint8).reshape(count, 2)

    if fmt == "Q8_0":
        q = (torch.randn((nb, 32), device=device, generator=gen) * 40).round().clamp(-127, 127).to(torch.int8)
        blk[:, 0:2] = scale(nb)
        blk[:, 2:] = q.view(torch.uint8)
    elif fmt == "Q6_K":
        blk[:, 0:192] = torch.randint(0, 256, (nb, 192), device=device, generator=gen, dtype=torch.uint8)
        blk[:, 192:208] = torch.randint(-64, 64, (nb, 16), device=device, generator=gen, dtype=torch.int8).view(torch.uint8)
        blk[:, 208:210] = scale(nb)
    elif fmt in ("Q5_K", "Q4_K"):
        blk[:, 0:2] = scale(nb)
        blk[:, 2:4] = scale(nb)
        # any 12 bytes are a valid field of eight 6-bit (scale, min) pairs, uniform over 0..63
        blk[:, 4:] = torch.randint(0, 256, (nb, b - 4), device=device, generator=gen, dtype=torch.uint8)
    elif fmt == "BF16":
        v = (torch.randn(nb, device=device, generator=gen) * 0.02).to(torch.bfloat16)
        blk[:] = v.view(torch.uint8).reshape(nb, 2)
    else:
        raise ValueError(fmt)
    return blk.reshape(-1)


class LayerStream:
    """`layers` x 7 packed projections resident in HBM plus activation / output buffers."""

    # projections that may run together because none reads another's output
    GROUPS = ((0, 3), (3, 4), (4, 6), (6, 7))   # q k v | o | gate up | down

    def __init__(self, torch, lib, fmt, layers, tokens, device, seed=106, act="f32", by_dependency=False):
        from mylocal_llm_amd import _lib
        self.torch, self.lib, self.fmt, self.layers, self.tokens = torch, lib, fmt, layers, tokens
        gen = torch.Generator(device=device)
        gen.manual_seed(seed)
        self.weights = [[device_blocks(torch, fmt, n, k, gen, device) for _, n, k in PROJECTIONS] for _ in range(layers)]
        xgen = torch.Generator(device=device)
        xgen.manual_seed(103)
        # one activation buffer per data-flow group: (q, k, v) share the layer input, o reads the
        # attention output, (gate, up) the post-attention state, down the SwiGLU activation
        tdt, dt_id = {"f32": (torch.float32, 0), "f16": (torch.float16, 1), "bf16": (torch.bfloat16, 2)}[act]
        self.x = {name: torch.randn((tokens, k), device=device, generator=xgen).to(tdt)
                  for name, k in (("qkv", 4096), ("o", 4096), ("gateup", 4096), ("down", 14336))}
        group = {"q": "qkv", "k": "qkv", "v": "qkv", "o": "o", "gate": "gateup", "up": "gateup", "down": "down"}
        self.y = [torch.empty((tokens, n), device=device, dtype=tdt) for _, n, _ in PROJECTIONS]
        self.bytes_per_layer = sum(weight_bytes(fmt, n, k) for _, n, k in PROJECTIONS)
        fid = _lib.FORMAT_ID[fmt]
        self.batches = []
        for layer in range(layers):
            arr = (_lib.LinearProblem * len(PROJECTIONS))()
            for i, (name, n, k) in enumerate(PROJECTIONS):
                p = arr[i]
                p.w, p.x, p.y = self.weights[layer][i].data_ptr(), self.x[group[name]].data_ptr(), self.y[i].data_ptr()
                p.fmt, p.n, p.k, p.tokens, p.x_dtype, p.y_dtype = fid, n, k, tokens, dt_id, dt_id
            self.batches.append(arr)
        self.by_dependency = by_dependency
        self.launches_per_step = layers * (len(self.GROUPS) if by_dependency else 1)
        stride = ctypes.sizeof(_lib.LinearProblem)
        # (address of the first problem, count) of every ABI call of a step
        self.calls = [(ctypes.cast(ctypes.addressof(arr) + lo * stride, ctypes.POINTER(_lib.LinearProblem)), hi - lo)
                      for arr in self.batches for lo, hi in (self.GROUPS if by_dependency else ((0, len(PROJECTIONS)),))]

    def step(self, stream):
        lib = self.lib
        for first, count in self.calls:
            rc = lib.qmoe_linear_batch(first, count, stream)
            if rc:
                raise RuntimeError(lib.qmoe_last_error().decode())


def time_steps(torch, fn, steps, warmup):
    """(wall seconds, event milliseconds) for `steps` calls of fn after `warmup` untimed ones."""
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for _ in range(warmup):
        fn(stream)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn(stream)
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, start.elapsed_time(stop)


def cpu_baseline(budget_s=24.0):
    """The reference's packed CPU path on this box's host cores, on bounded samples of the
    benchmark's workloads.  `value` is the NumPy restatement (dequantise on every call + fp32
    matmul, the reference's default host branch) over ALL seven projections of one 8B layer at
    M = 1, each multiplied once; `legs` adds the same layer through the library's single-threaded
    scalar C++ host twin on a sample, the 2048x2048 single linear of configs[0], and one token of
    the 512-expert MoE decode step."""
    import numpy as np
    from mylocal_llm_amd import synthetic
    from mylocal_llm_amd.native_packed_cpu import packed_cpu_linear
    from oracle import reference_np as R
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
    except Exception:
        threads = os.cpu_count() or 1
    t_begin = time.perf_counter()
    shapes = [(n, k) for _, n, k in PROJECTIONS]
    distinct = {}
    for i, shape in enumerate(shapes):       # q/o and k/v, gate/up share a shape: one weight each is enough to time
        distinct.setdefault(shape, synthetic.packed_weight("Q8_0", shape, 106 + i))
    xs = {k: synthetic.activations((1, k), 103) for k in {k for _, k in shapes}}
    per_shape = {}
    for shape, w in distinct.items():
        R.linear(xs[shape[1]], w.data, w.shape, "Q8_0")   # untimed: the first call of a size pays for fresh pages
        t0 = time.perf_counter()
        R.linear(xs[shape[1]], w.data, w.shape, "Q8_0")
        per_shape[shape] = time.perf_counter() - t0
    layer_s = sum(per_shape[shape] for shape in shapes)
    layer_bytes = sum(weight_bytes("Q8_0", n, k) for n, k in shapes)
    legs = []
    # scalar C++ twin, one thread: the k projection and as many rows of the others as the budget allows
    w = distinct[(1024, 4096)]
    t0 = time.perf_counter()
    reps = 0
    while time.perf_counter() - t0 < 3.0:
        packed_cpu_linear(xs[4096], w)
        reps += 1
    native_s = (time.perf_counter() - t0) / reps
    legs.append({"workload": "Q8_0 M=1 k-proj 1024x4096, scalar C++ host twin (qmoe_linear_cpu)", "cores": 1, "kind": "own C++",
                 "GBps": round(w.nbytes / native_s / 1e9, 4), "ms": round(native_s * 1e3, 3), "repetitions": reps})
    # configs[0]: the single 2048 x 2048 Q8_0 linear at batch 1
    w0 = synthetic.packed_weight("Q8_0", (2048, 2048), 1)
    x0 = synthetic.activations((1, 2048), 2)
    t0 = time.perf_counter()
    reps = 0
    while time.perf_counter() - t0 < 2.0:
        R.linear(x0, w0.data, w0.shape, "Q8_0")
        reps += 1
    c0_s = (time.perf_counter() - t0) / reps
    legs.append({"workload": "configs[0]: Q8_0 2048x2048 M=1, NumPy", "cores": int(threads), "kind": "port",
                 "GBps": round(w0.nbytes / c0_s / 1e9, 4), "ms": round(c0_s * 1e3, 3), "repetitions": reps})
    # one token of the MoE decode step: router + 10 routed experts + shared expert (D=2048, F=512, shared 2048)
    e, d, f, fsh, k = 512, 2048, 512, 2048, 10
    experts = [tuple(synthetic.packed_weight("Q8_0", shape, 300 + 3 * i + j) for j, shape in enumerate(((f, d), (f, d), (d, f))))
               for i in range(k)]
    shared = tuple(synthetic.packed_weight("Q8_0", shape, 400 + j) for j, shape in enumerate(((fsh, d), (fsh, d), (d, fsh))))
    hidden = synthetic.activations((1, d), 7)
    logits = synthetic.router_logits(1, e, 9)
    gate_vec = np.random.default_rng(1).normal(0, .02, d).astype(np.float32)
    triple = lambda w: (w.data, w.shape, w.quant_type)
    t0 = time.perf_counter()
    _, ids = R.router_topk(logits, k, floor=2.0 ** -14)
    slot_of = {int(expert): i for i, expert in enumerate(ids[0])}
    R.moe_forward(hidden, logits, k, e, lambda i, rows: R.expert_ffn(rows, *(triple(w) for w in experts[slot_of[int(i)]])),
                  tuple(triple(w) for w in shared), gate_vec)
    moe_s = time.perf_counter() - t0
    moe_bytes = sum(w.nbytes for ex in experts for w in ex) + sum(w.nbytes for w in shared)
    legs.append({"workload": "MoE decode T=1 (512 experts, top-10, D=2048, F=512, shared 2048), NumPy", "cores": int(threads),
                 "kind": "port", "GBps": round(moe_bytes / moe_s / 1e9, 4), "ms": round(moe_s * 1e3, 2),
                 "tokens_per_s": round(1.0 / moe_s, 3), "repetitions": 1})
    # the reference's opt-in native backend (cpu_packed_backend="native"): its own native_packed_cpu.cpp,
    # compiled by oracle/Makefile with the flags the reference itself uses, where that build is present
    try:
        from oracle import native as oracle_native
        if oracle_native.load_ref() is not None:
            ref_s = {}
            for shape, w in distinct.items():
                oracle_native.ref_gemv(xs[shape[1]], w.data, w.shape, "Q8_0")   # untimed
                t0 = time.perf_counter()
                oracle_native.ref_gemv(xs[shape[1]], w.data, w.shape, "Q8_0")
                ref_s[shape] = time.perf_counter() - t0
            ref_layer_s = sum(ref_s[shape] for shape in shapes)
            legs.append({"workload": "one 8B layer, Q8_0, M=1, all seven projections: the reference's own native_packed_cpu.cpp "
                                     "(mylocal_packed_gemv, g++ -O3 as the reference builds it; oracle/_ref)",
                         "cores": 1, "kind": "reference", "GBps": round(layer_bytes / ref_layer_s / 1e9, 4),
                         "ms": round(ref_layer_s * 1e3, 2), "tokens_per_s_32_layers": round(1.0 / (32 * ref_layer_s), 4), "repetitions": 1})
    except Exception as exc:   # noqa: BLE001 - a missing or unloadable build only drops this leg
        legs.append({"workload": "the reference's native_packed_cpu.cpp (oracle/_ref)", "error": f"{type(exc).__name__}: {exc}"})
    return {"value": round(layer_bytes / layer_s / 1e9, 4), "unit": "GB/s", "cores": int(threads), "kind": "port",
            "sample": f"one 8B layer, Q8_0, M=1: all seven projections ({layer_bytes} weight bytes) multiplied once each "
                      f"(one warm-up and one timed call per distinct shape, {layer_s:.2f}s per layer), NumPy dequantise-every-call + fp32 matmul "
                      "(oracle/reference_np.linear)",
            "tokens_per_s_32_layers": round(1.0 / (32 * layer_s), 4), "legs": legs,
            "seconds_total": round(time.perf_counter() - t_begin, 1), "numpy": np.__version__, "host_cpus": os.cpu_count()}


TIMELINE_STAMPS = {
    0: ("route + gate/up kernel", ["wave enters", "row selected / summed, activations staged", "",
                                   "at the barrier", "past the barrier", "first item's rows arrived", "wave ends", "(first instruction)"]),
    1: ("down kernel", ["wave enters", "routing arrived, two rows requested", "activations arrived", "past the barrier",
                        "first row arrived", "wave ends", "(routing arrived)", "(row addresses ready)"]),
}


def read_timeline(lib, steps_fn, steps):
    """Per-phase timeline of the two MoE decode kernels from a library built with time stamps
    (python -m mylocal_llm_amd._build --timeline): one step at a time, stamps read back after each;
    microseconds after the first wave of the first kernel entered, min / mean / max over the waves
    that wrote the stamp, averaged over the steps."""
    import numpy as np
    if not hasattr(lib, "qmoe_timeline_read"):
        raise RuntimeError("this library was built without time stamps: build with `python -m mylocal_llm_amd._build --timeline` "
                           "and set QMOE_LIBRARY to mylocal_llm_amd/libqmoe_hip_timeline.so")
    lib.qmoe_timeline_read.argtypes = [ctypes.c_void_p]
    buf = np.zeros((2, 4096, 8), dtype=np.uint64)
    acc = {}
    for _ in range(steps):
        buf[:] = 0
        # clear the device copy by reading after a step only: stamps are rewritten by every wave of every launch
        steps_fn()
        if lib.qmoe_timeline_read(buf.ctypes.data):
            raise RuntimeError("qmoe_timeline_read failed")
        t0 = buf[0, :, 0][buf[0, :, 0] > 0].min()
        for kernel, (_, names) in TIMELINE_STAMPS.items():
            for i, name in enumerate(names):
                if not name:
                    continue
                col = buf[kernel, :, i]
                col = col[col >= t0].astype(np.float64)
                if col.size:
                    us = (col - float(t0)) / 100.0
                    acc.setdefault((kernel, i), []).append((us.min(), us.mean(), us.max(), col.size))
    out = []
    for kernel, (kname, names) in TIMELINE_STAMPS.items():
        for i, name in enumerate(names):
            rows = acc.get((kernel, i)) if name else None
            if rows:
                a = np.asarray(rows)
                out.append({"kernel": kname, "stamp": name, "waves": int(a[:, 3].mean()), "min_us": round(a[:, 0].mean(), 2),
                            "mean_us": round(a[:, 1].mean(), 2), "max_us": round(a[:, 2].mean(), 2)})
    return out


def moe_decode_extra(torch, lib, device, fmt, tokens, steps, warmup, layer_half=False, hot=False, timeline=False):
    """512-expert top-10 MoE decode step (D=2048, F=512, shared F=2048).

    Cold (the default, the figure a model with dozens of layers sees): steps rotate over four
    layers' banks, 48 different sets of router logits per bank and 48 different shared experts,
    so an expert's bytes come round again only after several GB of other weights (far beyond the
    4 MB L2 per XCD and the 256 MB memory-side cache).  ``hot`` repeats ONE bank, one set of
    logits and one shared expert: everything a step reads was read by the step before.
    With ``layer_half`` a step is the second half of a decoder layer: RMSNorm + router logits of the
    fp32 residual stream in one launch, the MoE step on the normalised rows, residual added in its
    last kernel (fp32 in, fp32 out)."""
    from mylocal_llm_amd import _lib
    from mylocal_llm_amd.moe import DevicePackedExpertBank, moe_step
    from mylocal_llm_amd.quantized_linear import DevicePackedGGUFWeight
    e, d, f, fsh, k = 512, 2048, 512, 2048, 10
    gen = torch.Generator(device=device)
    gen.manual_seed(7)
    n_banks, n_sets, n_shared = (1, 1, 1) if hot else (4, 48, 48)
    cycle = n_banks * n_sets
    banks, shareds = [], []
    for _ in range(n_banks):
        g = device_blocks(torch, fmt, e * f, d, gen, device)
        u = device_blocks(torch, fmt, e * f, d, gen, device)
        dn = device_blocks(torch, fmt, e * d, f, gen, device)
        banks.append(DevicePackedExpertBank((g, (e, f, d), fmt), (u, (e, f, d), fmt), (dn, (e, d, f), fmt)))
    for _ in range(n_shared):
        shareds.append(tuple(DevicePackedGGUFWeight(device_blocks(torch, fmt, n, kk, gen, device), (n, kk), fmt)
                             for n, kk in ((fsh, d), (fsh, d), (d, fsh))))
    hidden = torch.randn((tokens, d), device=device, generator=gen).to(torch.float32 if layer_half else torch.bfloat16)
    logits = torch.randn((cycle, tokens, e), device=device, generator=gen)
    gate_vec = torch.randn(d, device=device, generator=gen) * 0.02
    out = torch.empty((tokens, d), device=device, dtype=hidden.dtype)
    hdt = 0 if layer_half else 2
    if layer_half:
        residual = torch.randn((tokens, d), device=device, generator=gen)
        gamma = 1 + 0.1 * torch.randn(d, device=device, generator=gen)
        router_w = torch.randn((cycle, e, d), device=device, generator=gen) * 0.05
    nbytes_ws = lib.qmoe_moe_workspace_bytes(tokens, k, e, d, f, fsh)
    workspace = torch.empty(nbytes_ws, dtype=torch.uint8, device=device)
    # the C ABI is the boundary: argument structs are built once, a step is one call
    calls = []
    for i in range(cycle):       # step i: bank i % 4, its own logits (and router matrix), shared expert i % 48
        a = _lib.MoeArgs()
        a.hidden, a.hidden_dtype, a.tokens, a.top_k = hidden.data_ptr(), hdt, tokens, k
        a.logits, a.floor_value, a.renormalize = logits[i].data_ptr(), 2.0 ** -14, 1
        if layer_half:
            a.residual = residual.data_ptr()
        banks[i % n_banks].fill(a.bank)
        g, u, dn = shareds[i % n_shared]
        a.shared_gate_w, a.shared_up_w, a.shared_down_w = g.data.data_ptr(), u.data.data_ptr(), dn.data.data_ptr()
        a.shared_gate_fmt = a.shared_up_fmt = a.shared_down_fmt = _lib.FORMAT_ID[fmt]
        a.d_ff_shared, a.shared_gate = fsh, gate_vec.data_ptr()
        a.out, a.out_dtype = out.data_ptr(), hdt
        calls.append(a)
    state = {"i": 0}
    wsp = ctypes.c_void_p(workspace.data_ptr())

    def fn(stream):
        i = state["i"] % cycle
        a = calls[i]
        state["i"] += 1
        if layer_half:  # normalised rows -> `hidden`, logits -> this step's logits buffer
            rc = lib.qmoe_norm_router(residual.data_ptr(), tokens, d, gamma.data_ptr(), 1e-6, router_w[i].data_ptr(), None, e,
                                      hidden.data_ptr(), logits[i].data_ptr(), stream)
            if rc:
                raise RuntimeError(lib.qmoe_last_error().decode())
        rc = lib.qmoe_moe_forward(ctypes.byref(a), wsp, nbytes_ws, stream)
        if rc:
            raise RuntimeError(lib.qmoe_last_error().decode())

    if timeline:
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        for _ in range(warmup):
            fn(stream)
        torch.cuda.synchronize()
        return {"workload": f"moe_decode_{fmt}_T{tokens} timeline", "unit": "us after the first wave entered the first kernel",
                "stamps": read_timeline(lib, lambda: fn(stream), steps)}
    wall, ms = time_steps(torch, fn, steps, warmup)
    # algorithmic bytes: distinct selected experts (averaged over the steps actually run) + shared expert
    used = sorted({j % cycle for j in range(warmup, warmup + steps)})
    ids = torch.topk(logits[used], k, dim=-1).indices
    distinct = sum(len(torch.unique(ids[j])) for j in range(len(used))) / len(used)
    eb = 3 * weight_bytes(fmt, f, d)
    sb = 3 * weight_bytes(fmt, fsh, d)
    nbytes = distinct * eb + sb + (e * d * 4 if layer_half else 0)
    per_step = ms / steps * 1e-3
    return {"workload": f"moe_{'layer_half' if layer_half else 'decode'}_{fmt}_T{tokens}" + ("_hot" if hot else ""),
            "residency": "hot: one bank, one set of logits, every step re-reads the bytes of the step before" if hot else
                         "cold: 4 banks x 48 logits sets x 48 shared experts in rotation",
            "ms_per_step": round(ms / steps, 4),
            "weight_bytes": int(nbytes), "distinct_experts": distinct,
            "GBps": round(nbytes / per_step / 1e9, 1), "frac_hbm_peak": round(nbytes / per_step / 1e9 / HBM_PEAK_GBS, 4),
            "tokens_per_s": round(tokens / per_step, 1), "host_ms_per_step": round(wall / steps * 1e3, 4)}


def grouped_decode_extra(torch, lib, device, fmt, count, steps, warmup):
    """The reference's decode entry point (grouped_quantized_experts_forward): one token through
    `count` expert handles of the 512-expert layer's shape (2048 -> 512 -> 2048), no router and no
    shared expert; handles given as a host list per step (qmoe_grouped_decode_listed).  Cold: steps
    rotate over four banks and 48 different selections, as the MoE decode steps do."""
    e, d, f = 512, 2048, 512
    gen = torch.Generator(device=device)
    gen.manual_seed(11)
    banks = [tuple(device_blocks(torch, fmt, e * n, kk, gen, device) for n, kk in ((f, d), (f, d), (d, f))) for _ in range(4)]
    row = {"g": weight_bytes(fmt, f, d), "d": weight_bytes(fmt, d, f)}
    x = torch.randn((1, d), device=device, generator=gen)
    routes = torch.rand(count, device=device, generator=gen)
    out = torch.empty((1, d), device=device)
    workspace = torch.empty(count * (f + d + 8), device=device)
    import numpy as np
    cycle = 4 * 48
    rng = np.random.default_rng(5)
    tables = []
    for i in range(cycle):
        g, u, dn = banks[i % 4]
        chosen = np.sort(rng.choice(e, count, replace=False))
        ptrs = []
        for j in chosen:
            ptrs += [g.data_ptr() + int(j) * row["g"], u.data_ptr() + int(j) * row["g"], dn.data_ptr() + int(j) * row["d"]]
        tables.append((ctypes.c_void_p * (3 * count))(*ptrs))
    from mylocal_llm_amd import _lib
    state = {"i": 0}
    fid = _lib.FORMAT_ID[fmt]

    def fn(stream):
        table = tables[state["i"] % cycle]
        state["i"] += 1
        rc = lib.qmoe_grouped_decode_listed(x.data_ptr(), ctypes.cast(table, ctypes.c_void_p), count, fid, fid, fid, d, f,
                                            routes.data_ptr(), 1, None, out.data_ptr(), workspace.data_ptr(), stream)
        if rc:
            raise RuntimeError(lib.qmoe_last_error().decode())

    wall, ms = time_steps(torch, fn, steps, warmup)
    nbytes = count * 3 * row["g"]
    per_step = ms / steps * 1e-3
    return {"workload": f"grouped_decode_{fmt}_E{count}", "residency": "cold: 4 banks x 48 selections in rotation",
            "ms_per_step": round(ms / steps, 4), "weight_bytes": int(nbytes), "GBps": round(nbytes / per_step / 1e9, 1),
            "frac_hbm_peak": round(nbytes / per_step / 1e9 / HBM_PEAK_GBS, 4), "host_ms_per_step": round(wall / steps * 1e3, 4)}


def moe_prefill_extra(torch, lib, device, fmt, tokens, steps, warmup):
    """512-expert top-10 MoE step at prefill size: Zipf(1.1) expert popularity over a seeded
    permutation, routing from logits, token-tile MFMA GEMMs, fp32 output [T, 2048]."""
    import numpy as np
    from mylocal_llm_amd import _lib, synthetic
    from mylocal_llm_amd.moe import DevicePackedExpertBank
    from mylocal_llm_amd.quantized_linear import DevicePackedGGUFWeight
    e, d, f, fsh, k = 512, 2048, 512, 2048, 10
    gen = torch.Generator(device=device)
    gen.manual_seed(11)
    n_banks = 2
    banks, shareds = [], []
    for _ in range(n_banks):
        g = device_blocks(torch, fmt, e * f, d, gen, device)
        u = device_blocks(torch, fmt, e * f, d, gen, device)
        dn = device_blocks(torch, fmt, e * d, f, gen, device)
        banks.append(DevicePackedExpertBank((g, (e, f, d), fmt), (u, (e, f, d), fmt), (dn, (e, d, f), fmt)))
        shareds.append(tuple(DevicePackedGGUFWeight(device_blocks(torch, fmt, n, kk, gen, device), (n, kk), fmt)
                             for n, kk in ((fsh, d), (fsh, d), (d, fsh))))
    hidden = torch.randn((tokens, d), device=device, generator=gen).to(torch.bfloat16)
    logits_np = np.stack([synthetic.router_logits(tokens, e, 9 + i, zipf=1.1) for i in range(n_banks)])
    logits = torch.from_numpy(logits_np).to(device)
    gate_vec = torch.randn(d, device=device, generator=gen) * 0.02
    out = torch.empty((tokens, d), device=device, dtype=torch.float32)
    nbytes_ws = lib.qmoe_moe_workspace_bytes(tokens, k, e, d, f, fsh)
    workspace = torch.empty(nbytes_ws, dtype=torch.uint8, device=device)
    calls = []
    for i in range(n_banks):
        a = _lib.MoeArgs()
        a.hidden, a.hidden_dtype, a.tokens, a.top_k = hidden.data_ptr(), 2, tokens, k
        a.logits, a.floor_value, a.renormalize = logits[i].data_ptr(), 2.0 ** -14, 1
        banks[i].fill(a.bank)
        g, u, dn = shareds[i]
        a.shared_gate_w, a.shared_up_w, a.shared_down_w = g.data.data_ptr(), u.data.data_ptr(), dn.data.data_ptr()
        a.shared_gate_fmt = a.shared_up_fmt = a.shared_down_fmt = _lib.FORMAT_ID[fmt]
        a.d_ff_shared, a.shared_gate = fsh, gate_vec.data_ptr()
        a.out, a.out_dtype = out.data_ptr(), 0
        calls.append(a)
    state = {"i": 0}
    wsp = ctypes.c_void_p(workspace.data_ptr())

    def fn(stream):
        a = calls[state["i"] % n_banks]
        state["i"] += 1
        rc = lib.qmoe_moe_forward(ctypes.byref(a), wsp, nbytes_ws, stream)
        if rc:
            raise RuntimeError(lib.qmoe_last_error().decode())

    wall, ms = time_steps(torch, fn, steps, warmup)
    ids = np.argsort(-logits_np, axis=-1, kind="stable")[..., :k]
    counts = [np.bincount(ids[i].ravel(), minlength=e) for i in range(n_banks)]
    distinct = float(np.mean([(c > 0).sum() for c in counts]))
    # tokens are multiplied in tiles of 16 per expert: the MFMA work actually issued
    padded = float(np.mean([(np.ceil(c / 16) * 16).sum() for c in counts]))
    nbytes = distinct * 3 * weight_bytes(fmt, f, d) + 3 * weight_bytes(fmt, fsh, d)
    flops = 2.0 * (tokens * k) * 3 * f * d + 2.0 * tokens * 3 * fsh * d
    per_step = ms / steps * 1e-3
    return {"workload": f"moe_prefill_{fmt}_T{tokens}_zipf1.1", "ms_per_step": round(ms / steps, 4),
            "weight_bytes": int(nbytes), "distinct_experts": distinct, "max_tokens_per_expert": int(max(c.max() for c in counts)),
            "GBps": round(nbytes / per_step / 1e9, 1), "frac_hbm_peak": round(nbytes / per_step / 1e9 / HBM_PEAK_GBS, 4),
            "useful_TFLOPs": round(flops / per_step / 1e12, 2), "padded_assignments": padded,
            "tokens_per_s": round(tokens / per_step, 1), "host_ms_per_step": round(wall / steps * 1e3, 4)}


def read_probe_extra(torch, lib, device, nbytes, steps, warmup=3):
    """The library's pure read kernel over eight rotating buffers of `nbytes` each: the streaming
    ceiling of this device for launches the size of one layer."""
    nbytes = nbytes // 4096 * 4096
    buffers = [torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device=device) for _ in range(8)]
    sink = torch.zeros(4, dtype=torch.int32, device=device)
    state = {"i": 0}

    def fn(stream):
        buf = buffers[state["i"] % len(buffers)]
        state["i"] += 1
        rc = lib.qmoe_read_probe(buf.data_ptr(), nbytes, 0x12345678, sink.data_ptr(), stream)
        if rc:
            raise RuntimeError(lib.qmoe_last_error().decode())

    _, ms = time_steps(torch, fn, steps, warmup)
    per_launch = ms / steps * 1e-3
    return {"workload": f"hbm_read_probe {nbytes} bytes per launch (qmoe_read_probe, 8 rotating buffers)",
            "GBps": round(nbytes / per_launch / 1e9, 1), "frac_hbm_peak": round(nbytes / per_launch / 1e9 / HBM_PEAK_GBS, 4),
            "us_per_launch": round(per_launch * 1e6, 2)}


def layer_extra(torch, lib, device, fmt, tokens, act, steps, by_dependency=False):
    """Eight 8B-shape layers of one format at `tokens` tokens: time per layer and weight-effective rate.
    ``by_dependency`` launches what a decoder can launch: q k v | o | gate up | down, four calls per layer."""
    s = LayerStream(torch, lib, fmt, 8, tokens, device, act=act, by_dependency=by_dependency)
    _, m = time_steps(torch, s.step, steps, 2)
    per_layer = m / steps / 8 * 1e-3
    out = {"workload": f"8B projections {fmt} M={tokens} (8 layers)" + ("" if act == "f32" else f", {act} activations")
                       + (", four launches per layer in data-flow order (q k v | o | gate up | down)" if by_dependency else ""),
           "GBps": round(s.bytes_per_layer / per_layer / 1e9, 1),
           "frac_hbm_peak": round(s.bytes_per_layer / per_layer / 1e9 / HBM_PEAK_GBS, 4),
           "us_per_layer": round(per_layer * 1e6, 2),
           "tokens_per_s_32_layers": round(tokens / (per_layer * 32), 1)}
    del s
    torch.cuda.empty_cache()
    return out


def vocabulary_projection_extra(torch, lib, device, fmt, steps, copies=2):
    """The output projection of the reference's model at its real shape (151 936 x 2048,
    mini_llm/external/qwen3next_model.py:291-293), one token, one qmoe_linear call per step;
    steps alternate between `copies` matrices (each larger than the memory-side cache)."""
    from mylocal_llm_amd import _lib
    n, k = 151936, 2048
    gen = torch.Generator(device=device)
    gen.manual_seed(606)
    weights = [device_blocks(torch, fmt, n, k, gen, device) for _ in range(copies)]
    x = torch.randn((1, k), device=device, generator=gen)
    y = torch.empty((1, n), device=device, dtype=torch.float32)
    fid, turn = _lib.FORMAT_ID[fmt], [0]

    def step(stream):
        w = weights[turn[0] % copies]
        turn[0] += 1
        rc = lib.qmoe_linear(w.data_ptr(), fid, n, k, x.data_ptr(), 0, 1, y.data_ptr(), 0, stream)
        if rc:
            raise RuntimeError(lib.qmoe_last_error().decode())

    _, ms = time_steps(torch, step, steps, 2)
    per_call = ms / steps * 1e-3
    nbytes = weight_bytes(fmt, n, k)
    out = {"workload": f"vocabulary projection {fmt} 151936x2048 M=1", "weight_bytes": nbytes,
           "us_per_call": round(per_call * 1e6, 2), "GBps": round(nbytes / per_call / 1e9, 1),
           "frac_hbm_peak": round(nbytes / per_call / 1e9 / HBM_PEAK_GBS, 4)}
    del weights
    torch.cuda.empty_cache()
    return out


def guarded(fn, *args, **kwargs):
    """An extras entry, or the reason it could not be measured (the headline line is printed either way)."""
    try:
        return fn(*args, **kwargs)
    except Exception as exc:   # noqa: BLE001 - the message goes into the JSON line
        return {"workload": getattr(fn, "__name__", "extra"), "error": f"{type(exc).__name__}: {exc}"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--only", choices=["moe_prefill", "moe_decode", "moe_decode_hot", "moe_timeline", "moe_layer_half", "grouped_decode", "layer_few_tokens", "read_probe", "vocabulary_projection",
                                       "layer_q6_k", "layer_q5_k", "layer_q4_k", "layer_by_dependency"], default=None,
                    help="run one of the extra workloads alone and print its JSON (profiling runs)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 1 GiB device-to-device tensor copy (a kernel of known traffic, "
                         "used to scale FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on one GPU; --gpus {args.gpus} is not supported "
              "(no collectives or sharding in this path)", file=sys.stderr)
        sys.exit(2)
    import torch
    from mylocal_llm_amd import _lib
    if not torch.cuda.is_available():
        print("bench.py: no HIP device", file=sys.stderr)
        sys.exit(1)
    lib = _lib.load()
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)

    if args.only == "moe_prefill":
        print(json.dumps(moe_prefill_extra(torch, lib, device, "Q8_0", 512, max(4, args.steps), args.warmup)))
        return
    if args.only == "moe_decode":
        print(json.dumps([moe_decode_extra(torch, lib, device, "Q8_0", t, max(8, args.steps), args.warmup) for t in (1, 4, 16)]))
        return
    if args.only == "moe_timeline":
        print(json.dumps([moe_decode_extra(torch, lib, device, "Q8_0", t, max(8, args.steps), args.warmup, timeline=True) for t in (1, 4)], indent=1))
        return
    if args.only == "grouped_decode":
        print(json.dumps([grouped_decode_extra(torch, lib, device, fmt, 10, max(8, args.steps), args.warmup) for fmt in ("Q8_0", "Q6_K")]))
        return
    if args.only == "moe_decode_hot":
        print(json.dumps([moe_decode_extra(torch, lib, device, "Q8_0", t, max(8, args.steps), args.warmup, hot=True) for t in (1, 4, 16)]))
        return
    if args.only == "read_probe":
        layer_bytes = sum(weight_bytes("Q8_0", n, k) for _, n, k in PROJECTIONS)
        print(json.dumps([read_probe_extra(torch, lib, device, b, max(50, args.steps)) for b in (layer_bytes, 1 << 30)]))
        return
    if args.only in ("layer_q6_k", "layer_q5_k", "layer_q4_k"):
        print(json.dumps(layer_extra(torch, lib, device, args.only[6:].upper(), 1, "f32", max(10, args.steps))))
        return
    if args.only == "layer_by_dependency":
        print(json.dumps(layer_extra(torch, lib, device, "Q8_0", 1, "f32", max(10, args.steps), by_dependency=True)))
        return
    if args.only == "vocabulary_projection":
        print(json.dumps([vocabulary_projection_extra(torch, lib, device, fmt, max(10, args.steps)) for fmt in ("Q8_0", "Q6_K")]))
        return
    if args.only == "moe_layer_half":
        print(json.dumps([moe_decode_extra(torch, lib, device, "Q8_0", t, max(8, args.steps), args.warmup, layer_half=True) for t in (1, 4)]))
        return
    if args.only == "layer_few_tokens":
        print(json.dumps([layer_extra(torch, lib, device, "Q8_0", t, act, max(3, args.steps)) for t, act in ((2, "f32"), (4, "f32"), (4, "bf16"))]))
        return
    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=device)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    stream = LayerStream(torch, lib, "Q8_0", args.layers, 1, device)
    wall, ms = time_steps(torch, stream.step, args.steps, args.warmup)
    step_s = wall / args.steps
    total_bytes = stream.bytes_per_layer * args.layers
    value = total_bytes / step_s / 1e9
    launches = args.steps * stream.launches_per_step
    launch_ms = ms / launches
    achieved = stream.bytes_per_layer / (launch_ms * 1e-3) / 1e9
    traffic = traffic_source = None
    traffic_file = os.path.join(ROOT, "profiles", "stream_q8_0_layer_m1_hbm_traffic.json")
    if os.path.exists(traffic_file):  # from the two rocprofv3 --pmc runs described beside that file
        with open(traffic_file) as fh:
            traffic = json.load(fh).get("traffic_bytes_per_launch")
        traffic_source = "from profiles/stream_q8_0_layer_m1_hbm_traffic.json (two rocprofv3 --pmc runs of this command, not measured in this run)"
    result = {
        "metric": "effective weight GB/s (Q8_0 8B projections, M=1, 32 layers streamed)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"configs[1]: Llama-3-8B-shaped Q8_0 projections, M=1, {args.layers} layers x 7 "
                               "projections streamed back-to-back, one batched launch sequence per layer",
                   "weight_bytes_per_step": total_bytes, "tokens_per_s": round(1.0 / step_s, 1),
                   "tokens_per_s_is": "projection-only (no attention, norms or sampling), one launch per layer: the seven "
                                      "projections of a layer are multiplied together although o, gate/up and down depend on "
                                      "each other in a decoder; the data-flow-ordered figure is the first entry of extras",
                   "frac_hbm_peak": round(value / HBM_PEAK_GBS, 4), "activations": "fp32 N(0,1)"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": "linear (Q8_0, M=1), one layer = 7 projections per launch sequence",
                     "bytes_per_launch": stream.bytes_per_layer, "avg_launch_us": round(launch_ms * 1e3, 3)},
    }
    del stream
    torch.cuda.empty_cache()
    probe = read_probe_extra(torch, lib, device, result["roofline"]["bytes_per_launch"], 64)
    result["roofline"]["hbm_read_probe_GBps"] = probe["GBps"]
    result["roofline"]["frac_of_read_probe"] = round(achieved / probe["GBps"], 4)
    torch.cuda.empty_cache()
    if not args.no_extras:
        extras = [layer_extra(torch, lib, device, "Q8_0", 1, "f32", max(3, args.steps // 4), by_dependency=True)]
        for fmt, tokens, act in (("Q6_K", 1, "f32"), ("Q5_K", 1, "f32"), ("Q4_K", 1, "f32"), ("BF16", 1, "f32"), ("Q8_0", 2, "f32"),
                                 ("Q8_0", 4, "f32"),
                                 ("Q8_0", 16, "f32"), ("Q8_0", 64, "f32"), ("Q6_K", 16, "f32"), ("Q5_K", 16, "f32"), ("Q4_K", 16, "f32"),
                                 ("Q8_0", 4, "bf16"), ("Q8_0", 16, "bf16"), ("Q8_0", 64, "bf16"), ("Q5_K", 16, "bf16")):
            extras.append(layer_extra(torch, lib, device, fmt, tokens, act, max(3, args.steps // 4)))
        for fmt, tokens in (("Q8_0", 1), ("Q8_0", 4), ("Q8_0", 16), ("Q6_K", 1)):
            extras.append(moe_decode_extra(torch, lib, device, fmt, tokens, max(8, args.steps), 3))
            torch.cuda.empty_cache()
        extras.append(grouped_decode_extra(torch, lib, device, "Q8_0", 10, max(8, args.steps), 3))
        torch.cuda.empty_cache()
        extras.append(moe_decode_extra(torch, lib, device, "Q8_0", 1, max(8, args.steps), 3, hot=True))
        torch.cuda.empty_cache()
        for tokens in (1, 4):
            extras.append(moe_decode_extra(torch, lib, device, "Q8_0", tokens, max(8, args.steps), 3, layer_half=True))
            torch.cuda.empty_cache()
        for fmt in ("Q8_0", "Q6_K", "Q5_K"):
            extras.append(moe_prefill_extra(torch, lib, device, fmt, 512, 6, 2))
            torch.cuda.empty_cache()
        for fmt in ("Q8_0", "Q6_K"):
            extras.append(guarded(vocabulary_projection_extra, torch, lib, device, fmt, max(10, args.steps)))
        result["extras"] = extras
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
