"""Typed configuration of the Kasuvik decoder: a list of layers, each with one of two kinds of mixer and an
optional feed-forward, read from the nested keys of its config.json.

  architecture    "Kasuvik"
  vocab, width    sizes of the vocabulary and of the residual stream
  embedding.scale factor on the embedding
  norm.eps        epsilon of every RMS norm
  layers[i]       type: "parallel" | "general_delta"; mixer: that mixer's sizes; mlp: {kind: "dense", ff} or null

A "parallel" mixer has two halves: ``left`` (attention: heads, kv_heads, dim, vdim, conv taps, rot{dims, base},
scale, mask{size, pool}) and ``right`` (selective scan: inner, state, dt_rank, conv taps).  A "general_delta"
mixer has heads and dim.  Sizes that only a tensor's shape gives (the rank of the decay's two-step
projection) are read from the checkpoint by the loader, not from here.
"""
from dataclasses import dataclass
from typing import Optional, Tuple

from .model_config import ConfigError

NAME = "Kasuvik"


def _pos_int(problems, where, d, key, allow_zero=False):
    v = d.get(key) if isinstance(d, dict) else None
    if not isinstance(v, int) or isinstance(v, bool) or v < 0 or (v == 0 and not allow_zero):
        problems.append(f"{where}.{key} must be a {'non-negative' if allow_zero else 'positive'} integer (got {v!r})")
        return 1
    return v


def _number(problems, where, d, key, positive=True):
    v = d.get(key) if isinstance(d, dict) else None
    if not isinstance(v, (int, float)) or isinstance(v, bool) or (positive and v <= 0):
        problems.append(f"{where}.{key} must be a {'positive ' if positive else ''}number (got {v!r})")
        return 1.0
    return float(v)


@dataclass(frozen=True)
class ConvAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    rot_dims: int
    rot_base: float
    scale: float
    window: int
    pool: int

    def to_dict(self):
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv,
                "rot": {"dims": self.rot_dims, "base": self.rot_base}, "scale": self.scale,
                "mask": {"size": self.window, "pool": self.pool}}


@dataclass(frozen=True)
class ScanConfig:
    inner: int
    state: int
    dt_rank: int
    conv: int

    def to_dict(self):
        return {"inner": self.inner, "state": self.state, "dt_rank": self.dt_rank, "conv": self.conv}


@dataclass(frozen=True)
class DeltaConfig:
    heads: int
    dim: int
    rank: int = 0      # of the decay's two-step projection; 0: taken from the checkpoint (config.json does not carry it)

    def to_dict(self):
        d = {"heads": self.heads, "dim": self.dim}
        if self.rank:
            d["rank"] = self.rank
        return d


@dataclass(frozen=True)
class KasuvikLayer:
    type: str                                   # "parallel" | "general_delta"
    left: Optional[ConvAttentionConfig] = None
    right: Optional[ScanConfig] = None
    delta: Optional[DeltaConfig] = None
    ff: int = 0                                 # 0: the layer has no feed-forward

    def to_dict(self):
        mixer = {"left": self.left.to_dict(), "right": self.right.to_dict()} if self.type == "parallel" else self.delta.to_dict()
        return {"type": self.type, "mixer": mixer, "mlp": {"kind": "dense", "ff": self.ff} if self.ff else None}


@dataclass(frozen=True)
class KasuvikConfig:
    vocab: int
    width: int
    embedding_scale: float
    eps: float
    layers: Tuple[KasuvikLayer, ...]

    @classmethod
    def from_dict(cls, raw: dict) -> "KasuvikConfig":
        problems = []
        vocab, width = _pos_int(problems, "config", raw, "vocab"), _pos_int(problems, "config", raw, "width")
        scale = _number(problems, "embedding", raw.get("embedding"), "scale")
        eps = _number(problems, "norm", raw.get("norm"), "eps")
        layers = []
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            problems.append("'layers' must be a non-empty list")
            listed = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]"
            if not isinstance(entry, dict) or not isinstance(entry.get("mixer"), dict):
                problems.append(f"{where} must be an object with 'type' and 'mixer'")
                continue
            kind, mixer, mlp = entry.get("type"), entry["mixer"], entry.get("mlp")
            ff = 0
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                    problems.append(f"{where}.mlp.kind {mlp.get('kind') if isinstance(mlp, dict) else mlp!r} is not supported (dense, or null)")
                else:
                    ff = _pos_int(problems, where + ".mlp", mlp, "ff")
            if kind == "parallel":
                l, r = mixer.get("left"), mixer.get("right")
                if not isinstance(l, dict) or not isinstance(r, dict):
                    problems.append(f"{where}.mixer needs 'left' and 'right'")
                    continue
                w = where + ".mixer.left"
                rot, mask = l.get("rot") or {}, l.get("mask") or {}
                left = ConvAttentionConfig(
                    heads=_pos_int(problems, w, l, "heads"), kv_heads=_pos_int(problems, w, l, "kv_heads"),
                    dim=_pos_int(problems, w, l, "dim"), vdim=_pos_int(problems, w, l, "vdim"), conv=_pos_int(problems, w, l, "conv"),
                    rot_dims=_pos_int(problems, w + ".rot", rot, "dims", allow_zero=True),
                    rot_base=_number(problems, w + ".rot", rot, "base"), scale=_number(problems, w, l, "scale"),
                    window=_pos_int(problems, w + ".mask", mask, "size"), pool=_pos_int(problems, w + ".mask", mask, "pool"))
                if left.heads % left.kv_heads:
                    problems.append(f"{w}: heads {left.heads} is not a multiple of kv_heads {left.kv_heads}")
                if left.rot_dims % 2 or left.rot_dims > left.dim:
                    problems.append(f"{w}.rot.dims {left.rot_dims} must be even and at most dim {left.dim}")
                w = where + ".mixer.right"
                right = ScanConfig(inner=_pos_int(problems, w, r, "inner"), state=_pos_int(problems, w, r, "state"),
                                   dt_rank=_pos_int(problems, w, r, "dt_rank"), conv=_pos_int(problems, w, r, "conv"))
                layers.append(KasuvikLayer("parallel", left=left, right=right, ff=ff))
            elif kind == "general_delta":
                w = where + ".mixer"
                rank = mixer.get("rank", 0)
                layers.append(KasuvikLayer("general_delta", delta=DeltaConfig(
                    heads=_pos_int(problems, w, mixer, "heads"), dim=_pos_int(problems, w, mixer, "dim"),
                    rank=rank if isinstance(rank, int) and rank > 0 else 0), ff=ff))
            else:
                problems.append(f"{where}.type {kind!r} is not supported (parallel | general_delta)")
        if problems:
            raise ConfigError("config.json: " + "; ".join(problems))
        return cls(vocab=vocab, width=width, embedding_scale=scale, eps=eps, layers=tuple(layers))

    def to_dict(self) -> dict:
        return {"architecture": NAME, "vocab": self.vocab, "width": self.width, "embedding": {"scale": self.embedding_scale},
                "norm": {"eps": self.eps}, "layers": [l.to_dict() for l in self.layers]}
