"""Seeded synthetic packed weights, activations and router logits.

Block contents follow the workload descriptions of the benchmark configurations:
  Q8_0  q = clip(rint(N(0,1)*40), -127, 127) int8,  d = |N(5e-4, 1e-4)| fp16
  Q6_K  6-bit codes uniform in [-32, 31] (4-bit low + 2-bit high planes), int8 sub-scales
        U[-64, 63], fp16 super-scale |N(5e-4, 1e-4)|
  Q5_K  5-bit codes uniform in [0, 31], eight 6-bit (scale, min) pairs U[0, 63], fp16 d and dmin
  Q4_K  as Q5_K without the high-bit plane;  Q4_0  nibbles uniform, fp16 d
  Q3_K  mask, 2-bit codes and 6-bit scales uniform, fp16 d
  BF16  N(0, 0.02) rounded to nearest-even bf16
All generators return a flat uint8 array in GGUF block layout for shape [..., K].
"""
import numpy as np

from .quantized_weight import BLOCK_FORMATS, PackedGGUFWeight


def _scale(rng, n):
    return np.abs(rng.normal(5e-4, 1e-4, n)).astype("<f2").view(np.uint8).reshape(n, 2)


def _pack_scale_min(sc, mn):
    """Eight 6-bit scales and minima -> the 12-byte K-quant field ([n, 12] uint8)."""
    sc = sc.astype(np.uint8)
    mn = mn.astype(np.uint8)
    field = np.zeros((sc.shape[0], 12), np.uint8)
    field[:, 0:4] = (sc[:, 0:4] & 63) | ((sc[:, 4:8] >> 4) << 6)
    field[:, 4:8] = (mn[:, 0:4] & 63) | ((mn[:, 4:8] >> 4) << 6)
    field[:, 8:12] = (sc[:, 4:8] & 15) | ((mn[:, 4:8] & 15) << 4)
    return field


def pack_blocks(fmt, rng, nblocks):
    """[nblocks, block_bytes] uint8 of freshly drawn blocks."""
    elems, nbytes = BLOCK_FORMATS[fmt]
    blk = np.zeros((nblocks, nbytes), np.uint8)
    if fmt == "Q8_0":
        q = np.clip(np.rint(rng.standard_normal((nblocks, 32), dtype=np.float32) * 40), -127, 127).astype(np.int8)
        blk[:, 0:2] = _scale(rng, nblocks)
        blk[:, 2:] = q.view(np.uint8)
    elif fmt == "Q4_0":
        blk[:, 0:2] = _scale(rng, nblocks)
        blk[:, 2:] = rng.integers(0, 256, (nblocks, 16), dtype=np.uint8)
    elif fmt in ("Q4_K", "Q5_K"):
        blk[:, 0:2] = _scale(rng, nblocks)
        blk[:, 2:4] = _scale(rng, nblocks)
        blk[:, 4:16] = _pack_scale_min(rng.integers(0, 64, (nblocks, 8)), rng.integers(0, 64, (nblocks, 8)))
        blk[:, 16:] = rng.integers(0, 256, (nblocks, nbytes - 16), dtype=np.uint8)
    elif fmt == "Q3_K":
        blk[:, 0:108] = rng.integers(0, 256, (nblocks, 108), dtype=np.uint8)
        blk[:, 108:110] = _scale(rng, nblocks)
    elif fmt == "Q6_K":
        blk[:, 0:192] = rng.integers(0, 256, (nblocks, 192), dtype=np.uint8)
        blk[:, 192:208] = rng.integers(-64, 64, (nblocks, 16)).astype(np.int8).view(np.uint8)
        blk[:, 208:210] = _scale(rng, nblocks)
    elif fmt == "BF16":
        v = rng.normal(0, 0.02, nblocks).astype(np.float32).view(np.uint32)
        words = ((v + 0x7FFF + ((v >> 16) & 1)) >> 16).astype("<u2")
        blk[:] = words.view(np.uint8).reshape(nblocks, 2)
    else:
        raise ValueError(f"Unsupported packed GGUF type: {fmt}")
    return blk


def packed_weight(fmt, shape, seed):
    """Seeded PackedGGUFWeight of canonical ``shape`` ([N, K] or [E, N, K])."""
    elems, nbytes = BLOCK_FORMATS[fmt]
    total = 1
    for d in shape:
        total *= int(d)
    rng = np.random.default_rng(seed)
    nblocks = total // elems
    out = np.empty((nblocks, nbytes), np.uint8)
    step = max(1, (1 << 25) // elems)  # bound the fp32 temporaries to ~128 MB
    for lo in range(0, nblocks, step):
        hi = min(nblocks, lo + step)
        out[lo:hi] = pack_blocks(fmt, rng, hi - lo)
    return PackedGGUFWeight(out.reshape(-1), tuple(shape), fmt)


def activations(shape, seed, dtype=np.float32):
    """N(0,1) activations; ``dtype='bf16'`` returns fp32 values that are exactly bf16."""
    x = np.random.default_rng(seed).standard_normal(shape, dtype=np.float32)
    if dtype == "bf16":
        b = x.view(np.uint32)
        b = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16) << 16
        return b.astype(np.uint32).view(np.float32)
    return x.astype(dtype)


def router_logits(tokens, n_experts, seed, *, zipf=None):
    """fp32 router logits.  ``zipf=s`` skews expert popularity: logit = log p_e + Gumbel with
    p_e proportional to rank^-s over a seeded permutation of the experts, so that top-k of a
    row is a Zipf-weighted sample without replacement."""
    rng = np.random.default_rng(seed)
    if zipf is None:
        return rng.standard_normal((tokens, n_experts), dtype=np.float32)
    ranks = rng.permutation(n_experts) + 1
    logp = -float(zipf) * np.log(ranks.astype(np.float64))
    gumbel = -np.log(-np.log(rng.random((tokens, n_experts))))
    return (logp[None, :] + gumbel).astype(np.float32)


def has_topk_ties(logits, k):
    """True if any row has equal values among its k+1 largest logits."""
    top = -np.sort(-np.asarray(logits), axis=-1)[..., :k + 1]
    return bool(np.any(top[..., :-1] == top[..., 1:]))
