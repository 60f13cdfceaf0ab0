"""The Furapel decoder as data: layers that run a mixer and a routed feed-forward side by side on one stream,
x += mixer(norm1(x)) + ff(norm2(x)), every norm a dynamic tanh.  Three kinds of mixer: ``attention`` (grouped queries,
a half-split rotation rescaled for long contexts, a gate per head), ``latent_attention`` (one cached latent vector per
token, a sliding window) and ``mlstm`` (a matrix memory with exponential gates).  A stretch of layers may run several
times in a row with the same weights: every pass is a layer of its own in the description (caches and states of its
own, the tensors shared by name), and the first layer of each pass mixes the stream with the embedding's output again.
Tensor names: ``l<i>.`` + norm1 | norm2 (+ ".b", ".alpha") | mix.* | mlp.*; ``embed``, ``loop.in``, ``final.norm``, ``head``.
"""
from ..config.furapel_config import NAME, FurapelConfig
from .. import parts  # noqa: F401  (registers the built-in part kinds)
from ..parts.base import LayerSpec, ModelSpec, PartSpec
from ..registry import ARCHITECTURES, Architecture


def _norm(cfg, name, ignore=()):
    return PartSpec("dynamic_tanh", {"size": cfg.width, "name": name, "ignore": tuple(ignore)})


def _mixer(cfg, layer, prefix):
    m = layer.mixer
    if layer.type == "attention":
        position = None
        if m.rot_dims:
            sc = m.scaling
            position = PartSpec("rotary_halves", {"dims": m.rot_dims, "base": m.rot_base,
                                                  "scaling": (sc.factor, sc.original, sc.fast, sc.slow) if sc else None})
        return PartSpec("gated_attention", {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim,
                                            "scale": m.scale, "window": 0, "position": position}, prefix)
    if layer.type == "latent_attention":
        return PartSpec("latent_attention", {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
                                             "scale": m.scale, "window": m.window, "eps": cfg.eps}, prefix)
    return PartSpec("matrix_memory", {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "gate_cap": m.gate_cap, "eps": cfg.eps}, prefix)


def layer_runs(cfg: FurapelConfig):
    """[(layer index, pass number, leads its pass?)] in the order the layers run."""
    n = len(cfg.layers)
    if cfg.loop is None:
        return [(i, 0, False) for i in range(n)]
    a, b = cfg.loop.start, cfg.loop.stop
    runs = [(i, 0, False) for i in range(a)]
    for t in range(cfg.loop.times):
        runs += [(i, t, i == a) for i in range(a, b)]
    return runs + [(i, 0, False) for i in range(b, n)]


def furapel_spec(cfg: FurapelConfig) -> ModelSpec:
    layers = []
    for i, t, leads in layer_runs(cfg):
        layer, p = cfg.layers[i], f"l{i}."
        second = (p + "norm2", p + "norm2.b", p + "norm2.alpha")
        parts_ = {"norm_mixer": _norm(cfg, p + "norm1", ignore=() if layer.mlp else second), "mixer": _mixer(cfg, layer, p + "mix.")}
        if layer.mlp:
            parts_["norm_ffn"] = _norm(cfg, p + "norm2")
            parts_["ffn"] = PartSpec("routed_experts", {"experts": layer.mlp.experts, "top": layer.mlp.top, "ff": layer.mlp.ff}, p + "mlp.")
        if leads:
            parts_["reentry"] = PartSpec("stream_reentry", {"name": "loop.in"})
        layers.append(LayerSpec(name=f"l{i}" if t == 0 else f"l{i}.pass{t}", block="side_by_side_residual", parts=parts_))
    return ModelSpec(
        architecture=NAME, hidden_size=cfg.width, vocab_size=cfg.vocab,
        embedding=PartSpec("scaled_token_embedding", {"vocab_size": cfg.vocab, "scale": cfg.embedding_scale, "name": "embed"}),
        layers=tuple(layers), schedule=tuple(range(len(layers))),
        final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "tied": False, "name": "head", "scale": cfg.logit_scale}),
        max_position=0, keep_embedding=cfg.loop is not None)


ARCHITECTURES.register(NAME, Architecture(NAME, FurapelConfig, furapel_spec))
