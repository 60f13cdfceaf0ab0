"""An attention whose q, k and v pass a short causal convolution, are rotated by interleaved pairs on a part
of each head, and which sees a sliding window of tokens plus one pooled key and value for every block of
tokens that lies wholly before the window; and the mixer that runs two mixers side by side on one input.
Every size, constant and tensor name is a parameter.
"""
import torch

from ..registry import MIXERS, POSITIONS
from .base import KVCacheNeed, Mixer, ParamSpec, PartSpec, PositionEncoding, StateNeed
from .chain_norm_parts import BranchPair, f32_params, linear32


@POSITIONS.register("rotary_pairs")
class InterleavedRotary(PositionEncoding):
    """Rotary positions by interleaved pairs: of every q and k head the entries (2i, 2i+1), i < dims/2, are turned
    by the angle position * base^(-2i/dims); entries from ``dims`` on pass.  params: dims, base."""

    capturable = True

    def pairs_table(self, step):
        """(cos, sin) of every row's angles, float32 [rows, dims/2, 2]; computed by the step's first layer that
        asks, read by the others with the same dims and base."""
        dims, base = self.params["dims"], float(self.params["base"])
        if dims == 0:
            return None
        key = ("rotary_pairs", base, dims)
        table = step.shared.get(key)
        if table is None:
            table = step.ws("rotary_pairs_%d_%s" % (dims, base.hex()), (step.rows, dims), torch.float32)
            self.ctx.ops.rotary_pairs_table(step.positions, table, dims, base, rows=step.rows)
            step.shared[key] = table
        return table

    def apply(self, step, qkv, num_heads, num_kv_heads, head_dim, cache=None, slots=None):
        raise NotImplementedError("rotary_pairs rotates inside ops.rotate_store (the mixer hands it pairs_table)")


@MIXERS.register("conv_window_pool_attention")
class ConvWindowPoolAttention(Mixer):
    """q, k, v = projections with biases; each channel then passes a causal convolution over time (``conv`` taps,
    no bias), q and k are rotated (``position``: a PartSpec), k and v go to the pages.  Query head h reads KV head
    h / (heads / kv_heads); score = (q . k) * scale * temp[h]; a row at position i sees the tokens j with
    0 <= i - j < window and one mean key and value for every block of ``pool`` tokens that ends at or before
    i - window (window 0: every token); one softmax; output projection.
    params: heads, kv_heads, dim, vdim, conv, scale, window, pool, position.
    Tensors under the prefix: q, k, v (+ ".b", + ".conv"), temp, o.  Keeps per request: pages of keys, values
    and pooled entries, and the convolution's last conv-1 inputs (32-bit)."""

    capturable = True
    sub_part_names = ("position",)

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        p = params
        self.nh, self.nkv, self.d, self.dv = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
        if self.nkv <= 0 or self.nh % self.nkv:
            raise ValueError(f"conv_window_pool_attention {prefix!r}: heads {self.nh} is not a multiple of kv_heads {self.nkv}")
        pos = p.get("position") or PartSpec("rotary_pairs", {"dims": 0, "base": 10000.0})
        self.position = POSITIONS.get(pos.kind)(pos.params, prefix, ctx)
        self.channels = (self.nh + self.nkv) * self.d + self.nkv * self.dv

    def sub_parts(self):
        return (self.position,)

    def param_specs(self):
        H, pre = self.ctx.hidden_size, self.prefix
        sizes = (("q", self.nh * self.d), ("k", self.nkv * self.d), ("v", self.nkv * self.dv))
        return [ParamSpec("w_qkv", tuple((pre + n, (c, H)) for n, c in sizes)),
                ParamSpec("bias", tuple((pre + n + ".b", (c,)) for n, c in sizes), role="vector"),
                ParamSpec("conv", tuple((pre + n + ".conv", (c, self.params["conv"])) for n, c in sizes)),
                ParamSpec("temp", ((pre + "temp", (self.nh,)),), role="vector"),
                ParamSpec("w_o", ((pre + "o", (H, self.nh * self.dv)),))]

    def bind(self, tensors):
        small = f32_params({k: tensors[k] for k in ("bias", "conv", "temp")})
        super().bind({**tensors, **small})

    def cache_needs(self):
        p = self.params
        needs = {"": KVCacheNeed(self.nkv, self.d, p["window"], value_dim=self.dv, pool=p["pool"] if p["window"] > 0 else 0)}
        if p["conv"] > 1:
            needs["conv"] = StateNeed((p["conv"] - 1, self.channels), torch.float32)
        return needs

    def flops(self, rows, attended=0):
        return super().flops(rows) + 2.0 * attended * (self.d + self.dv) * self.nh

    def forward(self, step, h):
        ops, p, w = self.ctx.ops, self.params, self.w
        g = self.cache.group
        kc, vc = self.cache.k(self.cache_index), self.cache.v(self.cache_index)
        pool = p["pool"] if p["window"] > 0 else 0
        pk, pv = (self.cache.pooled_k(self.cache_index), self.cache.pooled_v(self.cache_index)) if pool else (None, None)
        T, K = step.rows, p["conv"]
        proj = linear32(self.ctx, step, h, w["w_qkv"], "cwp_proj")
        mixed = step.ws("cwp_conv", (T, self.channels), torch.float32)
        conv_state = self.caches["conv"][0].slots(self.caches["conv"][1]) if K > 1 else None
        single = step.max_run == 1      # every sequence runs one row: the convolution leaves the new state itself
        ops.short_conv(proj, w["conv"], mixed, step, conv_state, bias_in=w["bias"], update_state=single)
        if not single:
            ops.short_conv_state(proj, conv_state, step, K, bias_in=w["bias"])
        q = step.ws("cwp_q", (T, self.nh * self.d))
        slots = step.slots(g) if self.cache_owner else None
        ops.rotate_store(mixed, q, self.nh, self.nkv, self.d, self.dv, cos_sin=self.position.pairs_table(step),
                         rot=self.position.params["dims"], slots=slots, kcache=kc, vcache=vc, rows=T)
        if pool and self.cache_owner:
            ops.pool_update(kc, vc, pk, pv, step.tables(g), step.table_stride(g), step.row_seq, step.positions, slots,
                            self.nkv, self.d, self.dv, pool, T)
        attn = step.ws("cwp_attn", (T, self.nh * self.dv))
        if step.max_run > 1 and ops.attention_window_pool_tiles_supported(self.d, self.dv, attn.dtype, kc.shape[2]):
            # runs of consecutive positions: 64 rows of a run share every staged key, on the matrix cores
            ops.attention_window_pool_tiles(q, attn, kc, vc, pk, pv, step.tables(g), step.table_stride(g), step.run_start,
                                            step.seq_start, step.seqs, step.max_run, self.nh, self.nkv, self.d, self.dv,
                                            p["scale"], p["window"], pool, head_scale=w["temp"])
            return linear32(self.ctx, step, attn, w["w_o"], "cwp_out")
        ops.attention_window_pool(q, attn, kc, vc, pk, pv, step.tables(g), step.table_stride(g), step.row_seq, step.ctx_lens,
                                  self.nh, self.nkv, self.d, self.dv, p["scale"], p["window"], pool, head_scale=w["temp"], rows=T)
        return linear32(self.ctx, step, attn, w["w_o"], "cwp_out")


@MIXERS.register("parallel_mixers")
class ParallelMixers(Mixer):
    """Two mixers side by side on the same input; the result is combine * (n(left) * w_left + n(right) * w_right),
    n: division by the root mean square over the model width (eps), the weights plain multipliers.  The two
    outputs are handed on as they are (BranchPair): the norm that adds the result to the stream combines them.
    The epsilon of these two norms is that of the norm which adds the result (one chain, one epsilon).
    params: left, right (PartSpecs of mixers), combine (default 0.5), left_weight, right_weight (checkpoint
    names after the prefix, defaults "left.out", "right.out")."""

    capturable = True
    sub_part_names = ("left", "right")

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.left, self.right = (MIXERS.get(s.kind)(s.params, s.prefix, ctx) for s in (params["left"], params["right"]))

    def sub_parts(self):
        return (self.left, self.right)

    def param_specs(self):
        H, pre, p = self.ctx.hidden_size, self.prefix, self.params
        return [ParamSpec("w_left", ((pre + p.get("left_weight", "left.out"), (H,)),), role="vector"),
                ParamSpec("w_right", ((pre + p.get("right_weight", "right.out"), (H,)),), role="vector")]

    def bind(self, tensors):
        super().bind(f32_params(tensors))

    def forward(self, step, h):
        a = self.left.forward(step, h)
        b = self.right.forward(step, h)
        return BranchPair(a, self.w["w_left"], b, self.w["w_right"], self.params.get("combine", 0.5))
