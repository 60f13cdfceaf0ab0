"""The Kasuvik decoder as data: a list of layers, each a mixer and (optionally) a dense gated feed-forward
between norms on both sides, x += norm_b(sublayer(norm(x))).  Two kinds of mixer: ``parallel`` (an attention
with short convolutions, a sliding window and pooled blocks, beside a selective scan, their normed outputs
averaged) and ``general_delta`` (the generalized delta rule).  Tensor names: ``l<i>.`` + norm1 | norm1b | norm2 |
norm2b | mix.* | mlp.*; ``embed``, ``final.norm``, ``head``.
"""
from ..config.kasuvik_config import NAME, KasuvikConfig
from .. import parts  # noqa: F401  (registers the built-in part kinds)
from ..parts.base import LayerSpec, ModelSpec, PartSpec
from ..registry import ARCHITECTURES, Architecture


def _norm(cfg, name):
    return PartSpec("rmsnorm_chain", {"size": cfg.width, "eps": cfg.eps, "name": name})


def kasuvik_spec(cfg: KasuvikConfig) -> ModelSpec:
    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        if layer.type == "parallel":
            l, r = layer.left, layer.right
            left = PartSpec("conv_window_pool_attention", {
                "heads": l.heads, "kv_heads": l.kv_heads, "dim": l.dim, "vdim": l.vdim, "conv": l.conv, "scale": l.scale,
                "window": l.window, "pool": l.pool,
                "position": PartSpec("rotary_pairs", {"dims": l.rot_dims, "base": l.rot_base})}, p + "mix.left.")
            right = PartSpec("selective_scan", {"inner": r.inner, "state": r.state, "dt_rank": r.dt_rank, "conv": r.conv},
                             p + "mix.right.")
            mixer = PartSpec("parallel_mixers", {"left": left, "right": right, "combine": 0.5}, p + "mix.")
        else:
            d = layer.delta
            mixer = PartSpec("general_delta", {"heads": d.heads, "dim": d.dim, "eps": cfg.eps, "rank": d.rank}, p + "mix.")
        parts_ = {"norm_mixer": _norm(cfg, p + "norm1"), "mixer": mixer, "norm_mixer_out": _norm(cfg, p + "norm1b")}
        if layer.ff:
            parts_.update({"norm_ffn": _norm(cfg, p + "norm2"),
                           "ffn": PartSpec("gated_mlp", {"intermediate_size": layer.ff, "activation": "relu"}, p + "mlp."),
                           "norm_ffn_out": _norm(cfg, p + "norm2b")})
        layers.append(LayerSpec(name=f"l{i}", block="sandwich_residual", parts=parts_))
    return ModelSpec(
        architecture=NAME, hidden_size=cfg.width, vocab_size=cfg.vocab,
        embedding=PartSpec("scaled_token_embedding", {"vocab_size": cfg.vocab, "scale": cfg.embedding_scale, "name": "embed"}),
        layers=tuple(layers), schedule=tuple(range(len(layers))),
        final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "tied": False, "name": "head"}),
        max_position=0)


ARCHITECTURES.register(NAME, Architecture(NAME, KasuvikConfig, kasuvik_spec))
