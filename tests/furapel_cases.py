"""Small Furapel configurations with random weights for the tests, none of them of a served model's sizes.  They differ
from one another in every size and constant; between them they cover each mixer first and last, a layer without a
feed-forward, one head, as many KV heads as query heads and one for all, a rotation of no, some and all entries of a
head, with and without rescaling, values wider and narrower than keys, head shapes that the matrix-core kernels take and
shapes that they refuse, windows of one token, shorter and longer than a page, as many experts a row as there are, a
single expert, a stretch of layers that runs again (in the middle, at the start, a single layer, once only) and none.
"""
import numpy as np
import torch


def _attention(heads, kv, dim, vdim, scale, rot=0, base=10000.0, scaling=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if rot:
        m["rot"] = {"dims": rot, "base": base}
        if scaling:
            m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return "attention", m


def _latent(heads, dim, vdim, rank, scale, window):
    return "latent_attention", {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank, "scale": scale, "mask": {"size": window}}


def _memory(heads, dim, vdim, cap):
    return "mlstm", {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def _layer(mixer, experts=0, top=0, ff=0):
    kind, m = mixer
    return {"type": kind, "mixer": m, "mlp": {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}} if experts else None}


CONFIGS = {
    # a matrix memory first and without a feed-forward; odd head sizes everywhere; no stretch runs again
    "U": {"architecture": "Furapel", "vocab": 97, "width": 48, "embedding": {"scale": 3.0}, "norm": {"eps": 1e-5}, "logit_scale": 1.7,
          "layers": [_layer(_memory(3, 8, 12, 6.0)),
                     _layer(_attention(4, 2, 16, 24, 0.3, rot=8, base=100.0, scaling=(3.0, 40, 8.0, 1.0)), 5, 3, 20),
                     _layer(_latent(2, 12, 20, 24, 0.25, 7), 3, 1, 40)]},
    # head shapes of the matrix-core kernels (keys and values of 64; a latent size of 32), a rotation of the whole head without
    # rescaling, two layers in the middle that run twice, a window longer than a page and one shorter
    "V": {"architecture": "Furapel", "vocab": 130, "width": 64, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6}, "logit_scale": 0.5,
          "loop": {"start": 1, "stop": 3, "times": 2},
          "layers": [_layer(_attention(2, 2, 64, 64, 0.11, rot=64, base=5000.0), 4, 2, 24),
                     _layer(_latent(3, 16, 8, 32, 0.2, 20), 4, 2, 24),
                     _layer(_memory(2, 32, 16, 8.0), 6, 2, 16),
                     _layer(_latent(2, 8, 16, 16, 0.3, 33), 2, 2, 32)]},
    # one layer that runs three times at the start, one head, a window of one token, a single expert, as many experts a row as
    # there are, no rotation, a matrix memory last, no logit scale in the file
    "W": {"architecture": "Furapel", "vocab": 64, "width": 32, "embedding": {"scale": 0.7}, "norm": {"eps": 3e-6},
          "loop": {"start": 0, "stop": 1, "times": 3},
          "layers": [_layer(_memory(1, 24, 40, 15.0), 2, 2, 8),
                     _layer(_attention(3, 1, 10, 6, 0.35), 1, 1, 12),
                     _layer(_latent(1, 6, 10, 10, 0.5, 1)),
                     _layer(_memory(2, 16, 8, 4.0), 3, 2, 16)]},
    # a stretch that "runs again" once only (led in, no second pass), a rotation of part of a 128-wide head with rescaling,
    # three query heads per KV head, pages of 32
    "X": {"architecture": "Furapel", "vocab": 200, "width": 96, "embedding": {"scale": 2.0}, "norm": {"eps": 1e-5}, "logit_scale": 1.0,
          "loop": {"start": 1, "stop": 2, "times": 1},
          "layers": [_layer(_latent(4, 24, 24, 40, 0.2, 70), 8, 2, 48),
                     _layer(_attention(6, 2, 128, 128, 0.09, rot=32, base=25000.0, scaling=(4.0, 64, 16.0, 2.0)), 8, 3, 32)]},
}
BLOCK_SIZE = {"U": 16, "V": 16, "W": 8, "X": 32}


def tensors_for(raw, seed, sharpen=3.0):
    """Checkpoint names -> float32 tensors on the bfloat16 grid (so that both storage modes hold the same numbers).
    Matrices N(0, 1 / fan-in); the q and k projections are scaled up so that attention is sharp enough for a wrong or
    missing key to show; norm weights 1 + 0.1 N, their biases 0.1 N, their factors between 0.3 and 1; forget gates
    biased towards keeping, so that the memory neither dies at once nor drowns its input."""
    from kvcm_amd.config.furapel_config import FurapelConfig
    from kvcm_amd.weights.random_init import expected_tensors
    cfg = FurapelConfig.from_dict(raw)
    rng = np.random.default_rng(seed)
    out = {}
    for name, (shape, role) in sorted(expected_tensors("Furapel", cfg).items()):
        leaf = name.split(".", 1)[1] if name[0] == "l" and name[1].isdigit() else name
        if len(shape) == 2:
            a = rng.normal(size=shape) / np.sqrt(shape[1])
        else:
            a = rng.normal(size=shape) * 0.5
        if leaf.endswith(".alpha"):
            a = rng.uniform(0.3, 1.0, size=shape)
        elif leaf.endswith(".b") and "norm" in leaf:
            a = 0.1 * rng.normal(size=shape)
        elif leaf.startswith("norm") or leaf in ("mix.norm", "mix.dkv.norm") or name == "final.norm":
            a = 1.0 + 0.1 * rng.normal(size=shape)
        elif leaf in ("mix.q", "mix.k"):
            a = a * sharpen
        elif leaf == "mix.f.b":
            a = rng.uniform(1.0, 4.0, size=shape)
        elif leaf == "mix.i.b":
            a = rng.normal(size=shape)
        elif leaf in ("mix.i", "mix.f"):
            a = a * 2.0
        elif leaf == "mlp.router":
            a = a * 4.0
        elif name == "embed":
            a = rng.normal(size=shape)
        out[name] = torch.from_numpy(np.asarray(a, dtype=np.float64)).to(torch.bfloat16).to(torch.float32)
    return cfg, out


def as_numpy(tensors):
    return {k: v.double().numpy() for k, v in tensors.items()}


def requests_for(raw, lengths, seed):
    rng = np.random.default_rng(seed)
    return {f"r{i}": rng.integers(0, raw["vocab"], size=n).tolist() for i, n in enumerate(lengths)}
