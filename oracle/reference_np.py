"""CPU oracle (TEST INFRASTRUCTURE ONLY) for the packed-weight decode path.

This module is a NumPy restatement of the arithmetic the reference performs on
its host path.  It exists to *check* the HIP kernels; it is never the thing
measured or shipped.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import it.  The product package
``mylocal_llm_amd`` must not import anything from ``oracle/``.

Every function names the reference lines whose behaviour it restates.  How each
one is pinned (which known-answer vector, closed form or brute-force check would
catch a dropped term / wrong index) is listed in ``PINNING`` at the bottom and
exercised by ``tests/test_oracle_*.py``.

Reference files followed (relative to the reference checkout):
  mini_llm/ops/quantized_weight.py          block tables, dequantisation
  mini_llm/external/gguf_tensor.py:30-51    BF16 bit expansion
  mini_llm/ops/quantized_linear.py:292-305  host linear
  mini_llm/ops/quantized_linear.py:362-370  host SwiGLU
  mini_llm/ops/quantized_linear.py:403-424  packed expert FFN
  mini_llm/ops/router.py:21-43              softmax / top-k
  mini_llm/ops/router_inference.py:47-61    selected-mass renormalisation
  mini_llm/ops/router_decode.py:19-26       tie / NaN ordering of the selection
  mini_llm/ops/routing_plan.py:52-118       token -> expert plan
  mini_llm/ops/experts_inference.py:290-310 ordered dispatch + combine
  mini_llm/ops/grouped_quantized_experts.py:159-217  single-token grouped experts
  mini_llm/external/qwen3next_moe.py:129-147 routed + gated shared expert
"""

import numpy as np

# (elements per block, bytes per block) -- mini_llm/ops/quantized_weight.py:24-37.
# "BF16" is not a packed format in the reference (it is decoded as a dense
# tensor, gguf_tensor.py:30-51); it is listed here so that one table serves the
# linear operator for all four weight encodings on the path.
BLOCKS = {
    "Q8_0": (32, 34),
    "Q4_0": (32, 18),
    "Q4_K": (256, 144),
    "Q3_K": (256, 110),
    "Q5_K": (256, 176),
    "Q6_K": (256, 210),
    "BF16": (1, 2),
}


def packed_nbytes(shape, fmt):
    """Byte count of a packed tensor (quantized_weight.py:71-73)."""
    elems, nbytes = BLOCKS[fmt]
    if shape[-1] % elems:
        raise ValueError(f"GGUF {fmt}: innermost dimension must be a multiple of {elems}")
    total = 1
    for d in shape:
        total *= int(d)
    return total // elems * nbytes


def _half_field(blocks, offset):
    """Little-endian fp16 at ``offset`` of every block, widened to fp32.

    quantized_weight.py:40-41; subnormals, infinities and NaNs follow IEEE.
    """
    pair = np.ascontiguousarray(blocks[:, offset:offset + 2])
    return pair.view("<f2").astype(np.float32).reshape(-1)


def _k_scale_min(field):
    """Unpack the 12-byte K-quant scale field into 8 scales and 8 minima.

    quantized_weight.py:225-228.  ``field`` is [nblocks, 12] uint8.
    Groups 0..3 use the low six bits of bytes 0..3 (scale) and 4..7 (minimum);
    groups 4..7 use a nibble of bytes 8..11 plus the top two bits of bytes
    0..3 (scale) or 4..7 (minimum).
    """
    field = field.astype(np.uint8)
    sc = np.empty((field.shape[0], 8), np.uint8)
    mn = np.empty((field.shape[0], 8), np.uint8)
    for g in range(4):
        sc[:, g] = field[:, g] & 63
        mn[:, g] = field[:, 4 + g] & 63
        sc[:, 4 + g] = (field[:, 8 + g] & 15) | ((field[:, g] >> 6) << 4)
        mn[:, 4 + g] = (field[:, 8 + g] >> 4) | ((field[:, 4 + g] >> 6) << 4)
    return sc, mn


def dequantize(data, shape, fmt):
    """Dense fp32 tensor of ``shape`` from packed bytes.

    Restates PackedGGUFWeight.dequantize_reference (quantized_weight.py:151-250)
    for the formats on the path.  The float operation order of the reference is
    kept -- ``d*q`` (Q8_0 :208-211), ``(d*sc)*q - dmin*mn`` (Q4_K/Q5_K :217-237),
    ``(d*sc)*q`` (Q6_K :238-250, Q3_K :251-266) -- so the result is bit-identical, signed zeros
    included.
    """
    if fmt == "BF16":
        return bf16_expand(data).reshape(shape)
    elems, nbytes = BLOCKS[fmt]
    raw = np.asarray(data).view(np.uint8).reshape(-1)
    if raw.size != packed_nbytes(shape, fmt):
        raise ValueError(f"GGUF {fmt}: expected {packed_nbytes(shape, fmt)} bytes, got {raw.size}")
    blk = raw.reshape(-1, nbytes)
    nb = blk.shape[0]
    out = np.empty((nb, elems), np.float32)
    if fmt == "Q8_0":
        d = _half_field(blk, 0)
        q = np.ascontiguousarray(blk[:, 2:34]).view(np.int8)
        out[:] = d[:, None] * q.astype(np.float32)
    elif fmt == "Q4_0":
        # quantized_weight.py:212-216: low nibbles are elements 0..15, high 16..31.
        d = _half_field(blk, 0)
        qs = blk[:, 2:18]
        out[:, :16] = d[:, None] * ((qs & 15).astype(np.float32) - np.float32(8))
        out[:, 16:] = d[:, None] * ((qs >> 4).astype(np.float32) - np.float32(8))
    elif fmt in ("Q4_K", "Q5_K"):
        d = _half_field(blk, 0)
        dmin = _half_field(blk, 2)
        sc, mn = _k_scale_min(blk[:, 4:16])
        base = 48 if fmt == "Q5_K" else 16
        for g in range(8):
            # 32-byte chunk g//2 serves group g through its low (even g) or high nibble.
            chunk = blk[:, base + 32 * (g // 2): base + 32 * (g // 2) + 32]
            q = (chunk >> (4 * (g % 2))) & 15
            if fmt == "Q5_K":
                q = q | (((blk[:, 16:48] >> g) & 1) << 4)
            scale = d * sc[:, g].astype(np.float32)
            floor = dmin * mn[:, g].astype(np.float32)
            out[:, 32 * g:32 * g + 32] = scale[:, None] * q.astype(np.float32) - floor[:, None]
    elif fmt == "Q3_K":
        # quantized_weight.py:251-266: 2 low bits in qs, a "keep" bit in hmask (0 -> minus four),
        # sixteen 6-bit scales minus 32; w = (d * scale) * value.
        d = _half_field(blk, 108)
        sb = blk[:, 96:108]
        for g in range(16):
            low = (sb[:, g % 8] >> (4 * (g // 8))) & 15
            high = (sb[:, 8 + g % 4] >> (2 * (g // 4))) & 3
            scale = d * ((low | (high << 4)).astype(np.float32) - np.float32(32))
            first = 16 * g  # elements first..first+15: plane i // 32, byte lane i % 32
            lanes = np.arange(first, first + 16) % 32
            plane = first // 32
            two = (blk[:, 32 + (first // 128) * 32 + lanes] >> (2 * (plane % 4))) & 3
            keep = (blk[:, lanes] >> plane) & 1
            value = two.astype(np.int32) - 4 * (1 - keep.astype(np.int32))
            out[:, first:first + 16] = scale[:, None] * value.astype(np.float32)
    elif fmt == "Q6_K":
        d = _half_field(blk, 208)
        sub = np.ascontiguousarray(blk[:, 192:208]).view(np.int8).astype(np.float32)
        for half in range(2):
            ql = blk[:, 64 * half:64 * half + 64]
            qh = blk[:, 128 + 32 * half:128 + 32 * half + 32]
            for quarter in range(4):
                lo = (ql[:, 32 * (quarter % 2):32 * (quarter % 2) + 32] >> (4 * (quarter // 2))) & 15
                hi = (qh >> (2 * quarter)) & 3
                q = (lo | (hi << 4)).astype(np.float32) - np.float32(32)
                first = 128 * half + 32 * quarter
                for piece in range(2):
                    s = d * sub[:, first // 16 + piece]
                    out[:, first + 16 * piece:first + 16 * piece + 16] = (
                        s[:, None] * q[:, 16 * piece:16 * piece + 16])
    else:
        raise ValueError(f"Unsupported packed GGUF type: {fmt}")
    return out.reshape(shape)


def bf16_expand(data):
    """BF16 payload -> fp32 by integer bit expansion (gguf_tensor.py:38-51).

    Accepts uint8 little-endian bytes or 16-bit unsigned words of either byte
    order.  No floating-point cast occurs, so signs of zero and every NaN payload
    survive.
    """
    a = np.asarray(data)
    if a.dtype == np.uint8:
        words = np.ascontiguousarray(a).reshape(-1).view("<u2")
    elif a.dtype.kind == "u" and a.dtype.itemsize == 2:
        words = a.reshape(-1)
    else:
        raise ValueError("BF16 payload must be uint8 bytes or uint16 words")
    return (words.astype(np.uint32) << 16).view(np.float32)


def bf16_round(values):
    """fp32 -> nearest-even BF16 words (helper for generators and bf16 outputs)."""
    bits = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32)
    rounded = bits + np.uint32(0x7FFF) + ((bits >> 16) & 1)
    nan = (bits & 0x7FFFFFFF) > 0x7F800000
    out = (rounded >> 16).astype(np.uint16)
    out[nan] = ((bits[nan] >> 16) | 0x40).astype(np.uint16)
    return out


def linear(x, data, shape, fmt):
    """``x @ W.T`` with fp32 accumulation, cast back to ``x.dtype``.

    quantized_linear.py:300-305: the weight is dequantised on every call, the
    activations are widened to fp32, and the product is rounded once to the
    activation dtype.  x is [M,K] or [B,T,K].
    """
    x = np.asarray(x)
    if x.ndim not in (2, 3):
        raise ValueError("Expected x as [M, K] or [B, T, K]")
    n, k = shape
    if x.shape[-1] != k:
        raise ValueError("Input K does not match packed weight K")
    w = dequantize(data, shape, fmt)
    y = x.astype(np.float32).reshape(-1, k) @ w.T
    return y.astype(x.dtype).reshape(x.shape[:-1] + (n,))


def silu_mul(g, u):
    """``g / (1 + exp(-g)) * u`` in fp32 (quantized_linear.py:367-370)."""
    g = np.asarray(g, np.float32)
    with np.errstate(over="ignore"):
        return (g / (np.float32(1.0) + np.exp(-g))) * np.asarray(u, np.float32)


def swiglu(x, gate, up):
    """Host SwiGLU: two linears then the fp32 activation, cast to x.dtype.

    ``gate`` / ``up`` are (data, shape, fmt) triples (quantized_linear.py:362-370).
    """
    g = linear(x, *gate)
    u = linear(x, *up)
    return silu_mul(g, u).astype(np.asarray(x).dtype)


def expert_ffn(x, gate, up, down):
    """Packed SwiGLU expert: ``down(swiglu(x))`` (quantized_linear.py:414-424)."""
    return linear(np.ascontiguousarray(swiglu(x, gate, up)), *down)


def _selection_order(row):
    """Indices of ``row`` in descending value order, lower id first on ties, NaN last.

    router.py:35 takes ``argsort(-logits)``, whose order on exact ties is not
    defined by NumPy; the device kernel of the reference defines it
    (router_decode.py:19-26) and that definition is adopted here.
    """
    idx = np.arange(row.size)
    nan = np.isnan(row)
    # lexsort: last key is primary.  NaN flag ascending, then value descending, then id.
    key = np.where(nan, np.float32(0), row)
    return np.lexsort((idx, -key.astype(np.float64), nan.astype(np.int8)))


def router_topk(logits, k, *, renormalize=True, floor=2.0 ** -14):
    """Full softmax, exact top-k selection, optional selected-mass renormalisation.

    router.py:28-36 (max-centred fp32 softmax over all experts, ids by descending
    logit, weights gathered) and router_inference.py:56-60 (divide by
    ``max(sum(selected), floor)``).  Returns (weights fp32 [...,k], ids int64 [...,k]).
    """
    logits = np.asarray(logits)
    n = logits.shape[-1]
    if logits.ndim < 1 or not 1 <= int(k) <= n:
        raise ValueError("expert router expects 1 <= k <= n_experts")
    work = logits.astype(np.float32, copy=False)
    flat = work.reshape(-1, n)
    with np.errstate(invalid="ignore", over="ignore"):
        centred = flat - np.max(flat, axis=-1, keepdims=True)
        e = np.exp(centred)
        probs = e / np.sum(e, axis=-1, keepdims=True)
    ids = np.stack([_selection_order(r)[:k] for r in flat]).astype(np.int64)
    w = np.take_along_axis(probs, ids, axis=-1)
    if renormalize:
        total = np.sum(w, axis=-1, keepdims=True)
        with np.errstate(invalid="ignore"):
            w = w / np.maximum(total, np.float32(floor))
    out_shape = logits.shape[:-1] + (int(k),)
    return w.astype(np.float32).reshape(out_shape), ids.reshape(out_shape)


def routing_plan(ids, n_experts):
    """Group the T*k assignments by expert (routing_plan.py:52-118).

    Returns (token, slot, order, offsets): assignments sorted by expert id
    (stable, so ascending token inside an expert), ``token = order // k``,
    ``slot = order % k`` and the E+1 exclusive offsets from the per-expert counts.
    """
    ids = np.asarray(ids)
    k = ids.shape[-1]
    flat = ids.reshape(-1)
    order = np.argsort(flat, kind="stable")
    counts = np.bincount(flat, minlength=n_experts)
    offsets = np.concatenate(([0], np.cumsum(counts))).astype(np.int64)
    return order // k, order % k, order, offsets


def experts_forward(x, weights, ids, n_experts, expert_fn):
    """Sparse dispatch + ordered weighted combine (experts_inference.py:290-310).

    ``y = zeros``; for each active expert in ascending id:
    ``y[tokens] += w[:, None] * expert_fn(e, x[tokens])`` in ``x.dtype``.
    x is [T,D]; weights/ids are [T,k].
    """
    x = np.asarray(x)
    t, d = x.shape
    token, slot, _, offsets = routing_plan(np.asarray(ids).reshape(t, -1), n_experts)
    w = np.asarray(weights).reshape(t, -1)
    y = np.zeros((t, d), x.dtype)
    for e in range(n_experts):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if lo == hi:
            continue
        tok = token[lo:hi]
        out = expert_fn(e, x[tok])
        y[tok] += w[tok, slot[lo:hi]][:, None] * out
    return y


def grouped_decode(x, experts, routes, slots=None):
    """Single-token grouped experts with explicit fp32 storage boundaries.

    grouped_quantized_experts.py:161-177: fp32 gate/up GEMV -> stored fp32
    SwiGLU -> fp32 down GEMV -> stored fp32 product with the route -> sequential
    fp32 adds starting at zero, in handle order; no FMA or tree across experts.
    ``experts`` is a list of (gate, up, down) triples of (data, shape, fmt).
    """
    x = np.asarray(x, np.float32)
    routes = np.asarray(routes, np.float32)
    out = np.zeros_like(x)
    for i, (gate, up, down) in enumerate(experts):
        h = silu_mul(linear(x, *gate), linear(x, *up)).astype(np.float32)
        y = linear(h, *down).astype(np.float32)
        r = routes[i if slots is None else slots[i]]
        term = np.multiply(y, r, dtype=np.float32)
        out = np.add(out, term, dtype=np.float32)
    return out


def shared_gate_sigmoid(hidden, shared_gate):
    """``exp(-logaddexp(0, -hidden @ g))`` (qwen3next_moe.py:145-146)."""
    admission = np.asarray(hidden, np.float32) @ np.asarray(shared_gate, np.float32)
    return np.exp(-np.logaddexp(np.float32(0), -admission)).astype(np.float32)


def moe_forward(hidden, logits, k, n_experts, expert_fn, shared, shared_gate, *,
                floor=2.0 ** -14):
    """One MoE step for fp32 hidden [T,D] with router logits given [T,E].

    qwen3next_moe.py:138-147: renormalised top-k routing, routed experts through
    the ordered dispatcher, shared SwiGLU expert scaled by a sigmoid admission
    gate, ``routed + shared * sigmoid``.  ``shared`` is a (gate, up, down) triple.
    Returns (output, weights, ids).
    """
    hidden = np.asarray(hidden, np.float32)
    w, ids = router_topk(logits, k, renormalize=True, floor=floor)
    routed = experts_forward(hidden, w, ids, n_experts, expert_fn)
    gate, up, down = shared
    sh = silu_mul(linear(hidden, *gate), linear(hidden, *up)).astype(np.float32)
    sh = linear(sh, *down)
    sig = shared_gate_sigmoid(hidden, shared_gate)
    return routed + sh * sig[..., None], w, ids


def rmsnorm(x, gamma, eps):
    """``(x * inv_rms) * gamma`` with ``inv_rms = 1 / sqrt(mean(x*x) + eps)`` in fp32
    (mini_llm/ops/rmsnorm_inference.py:517-520; the fused kernel :109-118 has the same graph)."""
    x = np.asarray(x, np.float32)
    mean_sq = np.mean(x * x, axis=-1, keepdims=True, dtype=np.float32)
    inv_rms = np.float32(1.0) / np.sqrt(mean_sq + np.float32(eps))
    return (x * inv_rms) * np.asarray(gamma, np.float32)


def router_logits(x, router_weight, bias=None):
    """``x @ W_router + b`` with ``W_router = router_weight.T`` (router_weight is [E, D] as stored in
    ffn_gate_inp; mini_llm/ops/router_inference.py:40-46, qwen3next_moe.py:111-113), fp32."""
    out = np.asarray(x, np.float32) @ np.asarray(router_weight, np.float32).T
    return out if bias is None else out + np.asarray(bias, np.float32)


PINNING = {
    "dequantize/Q8_0": "closed form d*int8; large-output vector of tests/test_0106p (q=(row%15-7), d=.125)",
    "dequantize/Q4_0": "hand-packed vector of tests/test_0106a:18-25",
    "dequantize/Q4_K": "hand-packed vector of tests/test_0106a:28-33",
    "dequantize/Q3_K": "hand-packed mask / scale vectors of tests/test_0106a:36-43 (+2 / -2) + independent per-element scalar decode (oracle.c) + oracle/_ref where it builds",
    "dequantize/Q5_K": "hand-packed vectors of tests/test_0106g:23-45 (8.25 / 9.0) + independent per-lane scalar decode",
    "dequantize/Q6_K": "all-codes signed-extremes vector of tests/test_0106l_q6k:25-46 + independent per-lane scalar decode",
    "bf16_expand": "all 65536 patterns == word<<16 and the byte fixture of tests/test_0106l_gguf_bf16:47-57",
    "all formats": "cross-check against oracle/_ref (the reference's own C++ packed dot, identity rows) where it builds",
    "linear": "textbook fp32 GEMV; checked against an fp64 matmul of the dequantised matrix",
    "swiglu / expert_ffn": "closed form; fp64 matched-storage formula of diagnostics/quantized_numerics.py:42-59",
    "rmsnorm": "closed forms (constant rows -> gamma*c/sqrt(c*c+eps); eps=0 scale invariance) and an fp64 evaluation",
    "router_logits": "textbook fp32 GEMV against an fp64 matmul",
    "router_topk": "tie / inf / NaN fixtures of tests/test_0106v:44-62; sum(w)=1 when mass>=floor; ids unique",
    "experts_forward / grouped_decode": "ordered-sum cancellation fixtures (1e8,1,-1e8,3 -> 3) of tests/test_0106t:321-330; brute-force per-token loop",
    "moe_forward": "independent fp64 per-token loop after tests/test_0106o_qwen3next_decoder:103-127; zero gate -> x0.5",
}
