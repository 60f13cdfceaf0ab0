"""Typed configuration of the Furapel decoder, read from the nested keys of its config.json.

  architecture    "Furapel"
  vocab, width    sizes of the vocabulary and of the residual stream
  embedding.scale factor on the embedding (default 1)
  norm.eps        epsilon of the root-mean-square divisions inside mixers (the layers' own norms use none)
  logit_scale     factor on the logits (default 1)
  layers[i]       type: "attention" | "latent_attention" | "mlstm"; mixer: that mixer's sizes;
                  mlp: {kind: "moe", expert: {ff}, router: {experts, top}} or null
  loop            {start, stop, times} or absent: layers start .. stop-1 run ``times`` times in a row, each pass with
                  caches of its own and led in by a product that mixes the stream with the embedding again

Mixers.  attention: heads, kv_heads, dim, vdim, scale, rot {dims, base, scaling {factor, original, fast, slow} or
absent} (rot absent or dims 0: no rotation; kv_heads defaults to heads, vdim to dim, rot.base to 10000).
latent_attention: heads, dim, vdim, kv_rank, scale, mask {size} (mask absent: every earlier token).
mlstm: heads, dim, vdim, gate_cap.
"""
from dataclasses import dataclass
from typing import Optional, Tuple

from .kasuvik_config import _number, _pos_int
from .model_config import ConfigError

NAME = "Furapel"
MIXERS = ("attention", "latent_attention", "mlstm")


@dataclass(frozen=True)
class RotaryScaling:
    factor: float
    original: float
    fast: float
    slow: float

    def to_dict(self):
        return {"factor": self.factor, "original": self.original, "fast": self.fast, "slow": self.slow}


@dataclass(frozen=True)
class GatedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int = 0
    rot_base: float = 10000.0
    scaling: Optional[RotaryScaling] = None

    def to_dict(self):
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.rot_dims:
            d["rot"] = {"dims": self.rot_dims, "base": self.rot_base}
            if self.scaling:
                d["rot"]["scaling"] = self.scaling.to_dict()
        return d


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int
    vdim: int
    kv_rank: int
    scale: float
    window: int

    def to_dict(self):
        d = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "kv_rank": self.kv_rank, "scale": self.scale}
        if self.window:
            d["mask"] = {"size": self.window}
        return d


@dataclass(frozen=True)
class MatrixMemoryConfig:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    def to_dict(self):
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


@dataclass(frozen=True)
class RoutedConfig:
    ff: int
    experts: int
    top: int

    def to_dict(self):
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}


@dataclass(frozen=True)
class FurapelLayer:
    type: str
    mixer: object
    mlp: Optional[RoutedConfig] = None

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None}


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int

    def to_dict(self):
        return {"start": self.start, "stop": self.stop, "times": self.times}


def _attention(problems, w, m):
    rot = m.get("rot")
    dims, base, scaling = 0, 10000.0, None
    if rot is not None:
        if not isinstance(rot, dict):
            problems.append(f"{w}.rot must be an object or absent")
            rot = {}
        dims = _pos_int(problems, w + ".rot", rot, "dims", allow_zero=True)
        if dims:
            base = _number(problems, w + ".rot", rot, "base") if "base" in rot else 10000.0
            sc = rot.get("scaling")
            if sc is not None:
                if not isinstance(sc, dict):
                    problems.append(f"{w}.rot.scaling must be an object or absent")
                    sc = {}
                ws = w + ".rot.scaling"
                scaling = RotaryScaling(_number(problems, ws, sc, "factor"), _number(problems, ws, sc, "original"),
                                        _number(problems, ws, sc, "fast"), _number(problems, ws, sc, "slow"))
                if base == 1.0:
                    problems.append(f"{w}.rot.base 1 cannot be rescaled")
    heads, dim = _pos_int(problems, w, m, "heads"), _pos_int(problems, w, m, "dim")
    cfg = GatedAttentionConfig(heads=heads, kv_heads=_pos_int(problems, w, m, "kv_heads") if "kv_heads" in m else heads,
                               dim=dim, vdim=_pos_int(problems, w, m, "vdim") if "vdim" in m else dim,
                               scale=_number(problems, w, m, "scale"), rot_dims=dims, rot_base=base, scaling=scaling)
    if cfg.heads % cfg.kv_heads:
        problems.append(f"{w}: heads {cfg.heads} is not a multiple of kv_heads {cfg.kv_heads}")
    if cfg.rot_dims % 2 or cfg.rot_dims > cfg.dim:
        problems.append(f"{w}.rot.dims {cfg.rot_dims} must be even and at most dim {cfg.dim}")
    return cfg


def _latent(problems, w, m):
    mask = m.get("mask")
    if mask is not None and not isinstance(mask, dict):
        problems.append(f"{w}.mask must be an object or absent")
        mask = None
    dim = _pos_int(problems, w, m, "dim")
    return LatentAttentionConfig(heads=_pos_int(problems, w, m, "heads"), dim=dim,
                                 vdim=_pos_int(problems, w, m, "vdim") if "vdim" in m else dim, kv_rank=_pos_int(problems, w, m, "kv_rank"),
                                 scale=_number(problems, w, m, "scale"),
                                 window=_pos_int(problems, w + ".mask", mask, "size") if mask is not None else 0)      # no mask: every earlier token


def _memory(problems, w, m):
    return MatrixMemoryConfig(heads=_pos_int(problems, w, m, "heads"), dim=_pos_int(problems, w, m, "dim"),
                              vdim=_pos_int(problems, w, m, "vdim"), gate_cap=_number(problems, w, m, "gate_cap"))


@dataclass(frozen=True)
class FurapelConfig:
    vocab: int
    width: int
    embedding_scale: float
    eps: float
    logit_scale: float
    layers: Tuple[FurapelLayer, ...]
    loop: Optional[LoopConfig] = None

    @classmethod
    def from_dict(cls, raw: dict) -> "FurapelConfig":
        problems = []
        vocab, width = _pos_int(problems, "config", raw, "vocab"), _pos_int(problems, "config", raw, "width")
        scale = _number(problems, "embedding", raw.get("embedding"), "scale") if isinstance(raw.get("embedding"), dict) and "scale" in raw["embedding"] else 1.0
        eps = _number(problems, "norm", raw.get("norm"), "eps")
        logit_scale = _number(problems, "config", raw, "logit_scale", positive=False) if "logit_scale" in raw else 1.0
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
            routed = None
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "moe":
                    problems.append(f"{where}.mlp.kind {mlp.get('kind') if isinstance(mlp, dict) else mlp!r} is not supported (moe, or null)")
                else:
                    w = where + ".mlp"
                    routed = RoutedConfig(ff=_pos_int(problems, w + ".expert", mlp.get("expert"), "ff"),
                                          experts=_pos_int(problems, w + ".router", mlp.get("router"), "experts"),
                                          top=_pos_int(problems, w + ".router", mlp.get("router"), "top"))
                    if routed.top > routed.experts:
                        problems.append(f"{w}.router.top {routed.top} exceeds its {routed.experts} experts")
            w = where + ".mixer"
            if kind == "attention":
                layers.append(FurapelLayer(kind, _attention(problems, w, mixer), routed))
            elif kind == "latent_attention":
                layers.append(FurapelLayer(kind, _latent(problems, w, mixer), routed))
            elif kind == "mlstm":
                layers.append(FurapelLayer(kind, _memory(problems, w, mixer), routed))
            else:
                problems.append(f"{where}.type {kind!r} is not supported ({' | '.join(MIXERS)})")
        loop = None
        if raw.get("loop") is not None:
            lp = raw["loop"]
            loop = LoopConfig(start=_pos_int(problems, "loop", lp, "start", allow_zero=True), stop=_pos_int(problems, "loop", lp, "stop"),
                              times=_pos_int(problems, "loop", lp, "times"))
            if not loop.start < loop.stop <= max(len(listed), 1):
                problems.append(f"loop: layers {loop.start} .. {loop.stop - 1} are not a stretch of the model's {len(listed)} layers")
        if problems:
            raise ConfigError("config.json: " + "; ".join(problems))
        return cls(vocab=vocab, width=width, embedding_scale=scale, eps=eps, logit_scale=logit_scale, layers=tuple(layers), loop=loop)

    def to_dict(self) -> dict:
        d = {"architecture": NAME, "vocab": self.vocab, "width": self.width, "embedding": {"scale": self.embedding_scale},
             "norm": {"eps": self.eps}, "logit_scale": self.logit_scale, "layers": [l.to_dict() for l in self.layers]}
        if self.loop:
            d["loop"] = self.loop.to_dict()
        return d
