"""Parts for layers whose mixer and feed-forward run side by side on the same stream,
x += mixer(norm_mixer(x)) + ffn(norm_ffn(x)): a norm without statistics (dynamic tanh), the arrangement that
adds both outputs in the launch that norms the stream for the next layer, and a part that leads a stretch of
layers in by mixing the stream with the embedding's output again.  Every size, constant and tensor name is a
parameter.
"""

from ..registry import BLOCKS, NORMS, STREAM_PARTS
from .base import Block, Norm, ParamSpec, Part, as_tensor
from .chain_norm_parts import f32_params, linear32


class StreamAdditions:
    """Up to two 32-bit sublayer outputs [T, H] that are still to be added to the residual stream: what a
    side-by-side layer hands to whoever reads the stream next (``dynamic_tanh`` adds them in its own launch).  The first
    may be the un-added slices of a split product (ops.PartialSums)."""

    def __init__(self, a=None, b=None):
        self.a, self.b = (a, b) if a is not None else (b, None)

    def materialize(self):
        raise TypeError("stream additions are added by the stream's next norm (dynamic_tanh), not materialized")


@NORMS.register("dynamic_tanh")
class DynamicTanh(Norm):
    """out = tanh(alpha * x) * weight + bias in 32-bit, rounded once: no mean, no variance, so nothing crosses a row.
    params: size; name: the weight's checkpoint name (default prefix + "weight"), with the bias at name + ".b" and the
    scalar alpha at name + ".alpha"; ignore: checkpoint names that may be present unused."""

    capturable = True
    accepts_partial_sums = True      # ``add`` may be StreamAdditions

    def _name(self):
        return self.params.get("name", self.prefix + "weight")

    def param_specs(self):
        n, H = self._name(), self.params["size"]
        return [ParamSpec("weight", ((n, (H,)),), role="vector"), ParamSpec("bias", ((n + ".b", (H,)),), role="vector"),
                ParamSpec("alpha", ((n + ".alpha", ()),), role="vector")]

    def ignorable_tensors(self):
        return tuple(self.params.get("ignore", ()))

    def bind(self, tensors):
        super().bind(f32_params(tensors))
        # alpha is a constant of the model: read once, handed to the kernel as a number
        self.as_op = self.ctx.ops.DytNorm(self.w["weight"], self.w["bias"], float(self.w["alpha"].reshape(-1)[0].item())) \
            if self.ctx.ops is not None else None

    def bytes_read(self, rows):
        return 2 * self.params["size"] * 4

    @staticmethod
    def _additions(add):
        if add is None:
            return None, None
        if isinstance(add, StreamAdditions):
            return add.a, add.b
        return add, None

    def forward(self, x, out, add=None, rows=None):
        a, b = self._additions(add)
        self.ctx.ops.dyt_norm(x, self.as_op, out, add_a=a, add_b=b, rows=rows)
        return out

    def forward_with(self, other, x, out, other_out, add=None, replace=False):
        """This norm and ``other`` (or None) of the same stream in one launch, after x += add (``replace``: x = add)."""
        a, b = self._additions(add)
        self.ctx.ops.dyt_norm(x, self.as_op, out, other.as_op if other is not None else None, other_out, add_a=a, add_b=b,
                              replace=replace)


@STREAM_PARTS.register("stream_reentry")
class StreamReentry(Part):
    """x <- W [x ; x0]: the stream mixed with the embedding's output x0 (kept by the model, ModelSpec.keep_embedding)
    through one matrix [H, 2H], x first.  What is still to be added to x is added on the way in.  Returns the new
    stream as a 32-bit tensor; the arrangement's norm writes it over x.  params: name (the matrix's checkpoint name)."""

    capturable = True

    def param_specs(self):
        H = self.ctx.hidden_size
        return [ParamSpec("w", ((self.params["name"], (H, 2 * H)),))]

    def forward(self, step, x, add=None):
        x0 = step.shared.get("embedding_output")
        if x0 is None:
            raise RuntimeError("stream_reentry needs the embedding's output: the model's description must set keep_embedding")
        a, b = DynamicTanh._additions(add)
        a = as_tensor(a) if a is not None else None
        packed = step.ws("reentry_in", (step.rows, 2 * x.shape[1]))
        self.ctx.ops.stream_pack(x, x0, packed, a, b)
        return linear32(self.ctx, step, packed, self.w["w"], "reentry_out")


@BLOCKS.register("side_by_side_residual")
class SideBySideResidual(Block):
    """x += mixer(norm_mixer(x)) + ffn(norm_ffn(x)), both norms of the same x; ``ffn`` and ``norm_ffn`` may be absent.
    An optional part ``reentry`` replaces x before the norms.  The two outputs are handed on un-added
    (StreamAdditions): the next reader of the stream adds them in the launch that norms it."""

    capturable = True
    part_registries = {"reentry": "stream"}

    def forward(self, step, x, pending):
        p = self.parts
        if pending is not None and not isinstance(pending, StreamAdditions):
            pending = StreamAdditions(pending)      # a tensor, or the slices of a split product
        replace = False
        if "reentry" in p:
            pending, replace = StreamAdditions(p["reentry"].forward(step, x, pending)), True
        H = x.shape[1]
        h1 = step.ws("normed", (step.rows, H))
        ffn = p.get("ffn")
        h2 = step.ws("normed_ffn", (step.rows, H)) if ffn is not None else None
        p["norm_mixer"].forward_with(p["norm_ffn"] if ffn is not None else None, x, h1, h2, add=pending, replace=replace)
        a = p["mixer"].forward(step, h1)
        b = ffn.forward(step, h2) if ffn is not None else None
        return StreamAdditions(a, b)
