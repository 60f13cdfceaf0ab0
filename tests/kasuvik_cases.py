"""Small Kasuvik configurations with random weights for the tests, none of them of a served model's sizes.
They differ from one another in every size and constant; between them they cover a delta-rule layer first and
last, a layer without a feed-forward, one query head, as many KV heads as query heads, a rotation of no, some
and all entries of a head, values wider and narrower than keys, convolutions of one to four taps, a block of
one token, a block longer than a page, a block that divides a page, and a window shorter than a block.
"""
import numpy as np
import torch


def _left(heads, kv, dim, vdim, conv, rot, base, scale, size, pool):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv, "rot": {"dims": rot, "base": base},
            "scale": scale, "mask": {"size": size, "pool": pool}}


def _right(inner, state, dt_rank, conv):
    return {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}


def _par(left, right, ff):
    return {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def _delta(heads, dim, rank, ff):
    return {"type": "general_delta", "mixer": {"heads": heads, "dim": dim, "rank": rank},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


CONFIGS = {
    # delta first; a parallel layer without a feed-forward; blocks of 5 in windows of 20 (pages of 16)
    "P": {"architecture": "Kasuvik", "vocab": 97, "width": 48, "embedding": {"scale": 2.0}, "norm": {"eps": 1e-5}, "layers": [
        _delta(3, 16, 8, 64),
        _par(_left(4, 2, 16, 24, 2, 8, 100.0, 0.3, 20, 5), _right(40, 6, 3, 3), 0),
        _par(_left(2, 2, 24, 8, 4, 24, 7000.0, 0.25, 33, 16), _right(56, 17, 5, 2), 80)]},
    # one head, no rotation, no convolution state, a block of one token, a block longer than a page, delta last
    "Q": {"architecture": "Kasuvik", "vocab": 64, "width": 32, "embedding": {"scale": 0.7}, "norm": {"eps": 3e-6}, "layers": [
        _par(_left(1, 1, 8, 40, 1, 0, 10.0, 0.5, 6, 1), _right(24, 3, 1, 1), 40),
        _par(_left(3, 1, 10, 10, 3, 4, 50000.0, 0.35, 9, 20), _right(36, 9, 2, 4), 0),
        _delta(1, 24, 5, 0)]},
    # head sizes that the wider loads of the kernels take (multiples of 8), a window shorter than a block
    "R": {"architecture": "Kasuvik", "vocab": 130, "width": 64, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6}, "layers": [
        _par(_left(4, 1, 32, 64, 3, 16, 250.0, 0.18, 7, 12), _right(96, 16, 4, 4), 96),
        _delta(2, 32, 16, 72),
        _par(_left(2, 2, 64, 32, 2, 64, 1000.0, 0.12, 48, 8), _right(72, 33, 6, 3), 56)]},
}
BLOCK_SIZE = {"P": 16, "Q": 8, "R": 16}


def tensors_for(raw, seed, sharpen=4.0):
    """Checkpoint names -> float32 tensors on the bfloat16 grid (so that both storage modes hold the same
    numbers).  Matrices N(0, 0.3 / sqrt(fan-in) * 3), norm weights 1 + 0.1 N; the q and k projections are
    scaled up so that attention is sharp enough for a wrong or missing key to show, and the decay parameters
    are spread so that the states neither die at once nor keep everything."""
    from kvcm_amd.config.kasuvik_config import KasuvikConfig
    from kvcm_amd.weights.random_init import expected_tensors
    cfg = KasuvikConfig.from_dict(raw)
    rng = np.random.default_rng(seed)
    out = {}
    for name, (shape, role) in sorted(expected_tensors("Kasuvik", cfg).items()):
        leaf = name.split(".", 1)[1] if name[0] == "l" and "." in name else name
        if len(shape) == 2 and not leaf.endswith(".conv") and not leaf.endswith("A_log"):
            a = rng.normal(size=shape) / np.sqrt(shape[1])
        else:
            a = rng.normal(size=shape) * 0.5
        if leaf.startswith("norm") or leaf in ("mix.left.out", "mix.right.out", "mix.norm") or name == "final.norm":
            a = 1.0 + 0.1 * rng.normal(size=shape)
        elif leaf in ("mix.left.q", "mix.left.k"):
            a = a * sharpen
        elif leaf == "mix.left.temp":
            a = 1.0 + 0.3 * rng.random(size=shape)
        elif leaf.endswith("A_log"):
            a = np.log(rng.uniform(0.3, 4.0, size=shape))
        elif leaf.endswith("dt.b"):
            a = rng.uniform(-3.0, 0.0, size=shape)
        elif leaf in ("embed",):
            a = rng.normal(size=shape)
        out[name] = torch.from_numpy(a).to(torch.bfloat16).to(torch.float32)
    return cfg, out


def as_numpy(tensors):
    return {k: v.double().numpy() for k, v in tensors.items()}


def requests_for(raw, lengths, seed):
    rng = np.random.default_rng(seed)
    return {f"r{i}": rng.integers(0, raw["vocab"], size=n).tolist() for i, n in enumerate(lengths)}
