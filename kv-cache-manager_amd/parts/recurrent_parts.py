"""Mixers that carry a fixed-size 32-bit state per request instead of keys and values: the selective scan
(with the short convolution in front of it) and the generalized delta rule.  Their states live in the
cache manager's state slots; a request's portion that starts at position 0 starts from zero.  Every size,
constant and tensor name is a parameter.
"""
import torch

from ..registry import MIXERS
from .base import Mixer, ParamSpec, StateNeed
from .chain_norm_parts import f32_params, linear32
from .llama_parts import _linear

_SMALL = ("conv", "conv_bias", "dt_bias", "a_log", "d_skip", "a_bias", "w0", "w2", "norm")


class _StatefulMixer(Mixer):
    capturable = True

    def bind(self, tensors):
        small = f32_params({k: v for k, v in tensors.items() if k in _SMALL})
        super().bind({**tensors, **small})

    def state(self, name):
        storage, index, _ = self.caches[name]
        return storage.slots(index)


@MIXERS.register("selective_scan")
class SelectiveScanMixer(_StatefulMixer):
    """in -> [x | z]; x through a causal convolution (bias, silu); [dt | B | C] = W_x x; dt = softplus(W_dt dt + b);
    S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n with A = -exp(A_log); y = S C + D x; (y * silu(z)) -> out.
    params: inner, state, dt_rank, conv (taps).  Tensors under the prefix: in, conv, conv.b, x, dt, dt.b, A_log, D, o.
    Keeps per request: the convolution's last taps-1 inputs and S, both 32-bit."""

    def param_specs(self):
        H, p, pre = self.ctx.hidden_size, self.params, self.prefix
        C, N, R, K = p["inner"], p["state"], p["dt_rank"], p["conv"]
        return [ParamSpec("w_in", ((pre + "in", (2 * C, H)),)),
                ParamSpec("conv", ((pre + "conv", (C, K)),)),
                ParamSpec("conv_bias", ((pre + "conv.b", (C,)),), role="vector"),
                ParamSpec("w_x", ((pre + "x", (R + 2 * N, C)),)),
                ParamSpec("w_dt", ((pre + "dt", (C, R)),)),
                ParamSpec("dt_bias", ((pre + "dt.b", (C,)),), role="vector"),
                ParamSpec("a_log", ((pre + "A_log", (C, N)),)),
                ParamSpec("d_skip", ((pre + "D", (C,)),), role="vector"),
                ParamSpec("w_o", ((pre + "o", (H, C)),))]

    def cache_needs(self):
        p = self.params
        needs = {"scan": StateNeed((p["inner"], p["state"]), torch.float32)}
        if p["conv"] > 1:
            needs["conv"] = StateNeed((p["conv"] - 1, p["inner"]), torch.float32)
        return needs

    def flops(self, rows, attended=0):
        p = self.params
        return super().flops(rows) + rows * p["inner"] * (6.0 * p["state"] + 2.0 * p["conv"])

    def forward(self, step, h):
        ops, p, w = self.ctx.ops, self.params, self.w
        C, N, R, K = p["inner"], p["state"], p["dt_rank"], p["conv"]
        xz = linear32(self.ctx, step, h, w["w_in"], "scan_xz")
        conv_state = self.state("conv") if K > 1 else None
        x = step.ws("scan_x", (step.rows, C))
        single = step.max_run == 1      # every sequence runs one row: the convolution leaves the new state itself
        ops.short_conv(xz, w["conv"], x, step, conv_state, bias_out=w["conv_bias"], activation="silu", update_state=single)
        if not single:
            ops.short_conv_state(xz, conv_state, step, K)
        # the step size's low-rank input feeds a product (compute dtype); B and C enter the recurrence (32-bit)
        low = _linear(self.ctx, step, x, w["w_x"][:R], "scan_dt_low")
        bc = linear32(self.ctx, step, x, w["w_x"][R:], "scan_bc")
        dt = linear32(self.ctx, step, low, w["w_dt"], "scan_dt")
        y = step.ws("scan_y", (step.rows, C))
        # runs of some length: step sizes and gates made ahead; long runs: walked in pieces, all pieces at once
        carry = None
        if step.max_run >= 4 * ops.SCAN_PIECE:
            carry = step.flat("scan_carry", ops.selective_scan_carry_floats(max(step.rows, step.limits.max_tokens), step.limits.max_seqs, C, N))
        ops.selective_scan(x, dt, w["dt_bias"], bc, 0, N, w["a_log"], w["d_skip"], xz[:, C:], y, self.state("scan"), step,
                           prepare=step.max_run >= 16, carry=carry)
        return linear32(self.ctx, step, y, w["w_o"], "scan_out")


@MIXERS.register("general_delta")
class GeneralDeltaMixer(_StatefulMixer):
    """The generalized delta rule.  r, k, v, g, a (with a bias) and the first step of the decay's projection are
    one fused product; per head and key channel the decay is w = exp(-exp(-1/2) sigmoid(W_w2 tanh(W_w1 h) + w0)) and
    the removal rate a = sigmoid(W_a h + b); with u = k / sqrt(|k|^2 + 1e-6):
    S <- diag(w) S - (a u)(u^T S) + k v^T, o = S^T r; every head's o is divided by its root mean square, times a
    weight over all heads, times sigmoid(g), then the output projection.
    params: heads, dim, eps, rank (of the decay's projection; 0: as the checkpoint has it).
    Tensors under the prefix: r, k, v, g, a, a.b, w1, w2, w0, norm, o.  Keeps S [heads, dim, dim] per request."""

    def param_specs(self):
        H, p, pre = self.ctx.hidden_size, self.params, self.prefix
        D, R = p["heads"] * p["dim"], p.get("rank") or -1
        return [ParamSpec("w_proj", tuple((pre + n, (D, H)) for n in ("r", "k", "v", "g", "a")) + ((pre + "w1", (R, H)),)),
                ParamSpec("a_bias", ((pre + "a.b", (D,)),), role="vector"),
                ParamSpec("w2", ((pre + "w2", (D, R)),)),
                ParamSpec("w0", ((pre + "w0", (D,)),), role="vector"),
                ParamSpec("norm", ((pre + "norm", (D,)),), role="vector"),
                ParamSpec("w_o", ((pre + "o", (H, D)),))]

    def bind(self, tensors):
        super().bind(tensors)
        D = self.params["heads"] * self.params["dim"]
        self.rank = self.w["w2"].shape[1]
        self.w["w2"] = self.w["w2"].t().contiguous()      # [rank, heads*dim]: the kernel's lanes read neighbours
        if self.w["w_proj"].shape[0] != 5 * D + self.rank:
            raise ValueError(f"general_delta {self.prefix!r}: the two steps of the decay's projection do not agree on their rank "
                             f"({self.w['w_proj'].shape[0] - 5 * D} and {self.rank})")

    def cache_needs(self):
        p = self.params
        return {"delta": StateNeed((p["heads"], p["dim"], p["dim"]), torch.float32)}

    def flops(self, rows, attended=0):
        p = self.params
        return super().flops(rows) + rows * p["heads"] * 8.0 * p["dim"] * p["dim"]

    def forward(self, step, h):
        ops, p, w = self.ctx.ops, self.params, self.w
        heads, d = p["heads"], p["dim"]
        D, T = heads * d, step.rows
        proj = linear32(self.ctx, step, h, w["w_proj"], "delta_proj")
        r, k, v, g, a = (proj[:, i * D:(i + 1) * D] for i in range(5))
        low = proj[:, 5 * D:]
        decay, au, u = (step.ws(n, (T, D), torch.float32) for n in ("delta_w", "delta_au", "delta_u"))
        ops.delta_prepare(k, a, w["a_bias"], low, w["w2"], w["w0"], decay, au, u, heads, d, T)
        o = step.ws("delta_o", (T, D), torch.float32)
        ops.delta_scan(r, k, v, decay, au, u, o, self.state("delta"), step, heads, d, d)
        gated = step.ws("delta_gated", (T, D))
        ops.head_norm_gate(o, g, w["norm"], gated, heads, d, p["eps"])
        return linear32(self.ctx, step, gated, w["w_o"], "delta_out")


@MIXERS.register("matrix_memory")
class MatrixMemoryMixer(_StatefulMixer):
    """A matrix memory with exponential gates (the mLSTM cell).  q, k, v, the output gate g and one input and one forget
    gate per head are one fused product; q is scaled by dim^(-1/2); li = cap tanh((W_i h + b_i) / cap),
    lf = logsigmoid(cap tanh((W_f h + b_f) / cap)); m' = max(lf + m, li), S' = exp(lf + m - m') S + exp(li - m') k v^T, n'
    likewise with k alone, o = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6); every head's o is divided by its root mean
    square, times a weight over all heads, times sigmoid(g), then the output projection.  S, n and m start at 0.
    params: heads, dim, vdim, gate_cap, eps.  Tensors under the prefix: q, k, v, g, i, i.b, f, f.b, norm, o.
    Keeps S [heads, dim, vdim], n [heads, dim] and m [heads] per request, 32-bit."""

    def param_specs(self):
        H, p, pre = self.ctx.hidden_size, self.params, self.prefix
        heads, d, dv = p["heads"], p["dim"], p["vdim"]
        sizes = (("q", heads * d), ("k", heads * d), ("v", heads * dv), ("g", heads * dv), ("i", heads), ("f", heads))
        return [ParamSpec("w_proj", tuple((pre + n, (c, H)) for n, c in sizes)),
                ParamSpec("in_bias", ((pre + "i.b", (heads,)),), role="vector"),
                ParamSpec("keep_bias", ((pre + "f.b", (heads,)),), role="vector"),
                ParamSpec("norm", ((pre + "norm", (heads * dv,)),), role="vector"),
                ParamSpec("w_o", ((pre + "o", (H, heads * dv)),))]

    def bind(self, tensors):
        w = tensors["w_proj"]
        extra = -w.shape[0] % 16      # the few-row products take widths that are multiples of 16
        if extra:
            w = torch.cat([w, torch.zeros(extra, w.shape[1], dtype=w.dtype, device=w.device)], 0)
        small = f32_params({k: tensors[k] for k in ("in_bias", "keep_bias", "norm")})
        Mixer.bind(self, {**tensors, **small, "w_proj": w})

    def cache_needs(self):
        p = self.params
        return {"memory": StateNeed((p["heads"], p["dim"], p["vdim"]), torch.float32),
                "normalizer": StateNeed((p["heads"], p["dim"]), torch.float32),
                "maximum": StateNeed((p["heads"],), torch.float32)}

    def flops(self, rows, attended=0):
        p = self.params
        return super().flops(rows) + rows * p["heads"] * (4.0 * p["dim"] * p["vdim"] + 4.0 * p["dim"])

    def forward(self, step, h):
        ops, p, w = self.ctx.ops, self.params, self.w
        heads, d, dv = p["heads"], p["dim"], p["vdim"]
        T = step.rows
        proj = linear32(self.ctx, step, h, w["w_proj"], "memory_proj")
        at = [0, heads * d, 2 * heads * d, 2 * heads * d + heads * dv, 2 * heads * (d + dv), 2 * heads * (d + dv) + heads]
        q, k, v, g, gi, gf = (proj[:, lo:] for lo in at)
        coef = step.ws("memory_factors", (T, 4 * heads), torch.float32)
        seqs = max(step.seqs, step.limits.max_seqs if step.limits is not None else step.seqs)
        n_new = step.flat("memory_normalizer", seqs * heads * d)
        o = step.ws("memory_o", (T, heads * dv), torch.float32)
        ops.mlstm_scan(q, k, v, gi, gf, w["in_bias"], w["keep_bias"], p["gate_cap"], float(d) ** -0.5, coef, n_new, o,
                       self.state("memory"), self.state("normalizer"), self.state("maximum"), step, heads, d, dv)
        gated = step.ws("memory_gated", (T, heads * dv))
        ops.head_norm_gate(o, g, w["norm"], gated, heads, dv, p["eps"])
        return linear32(self.ctx, step, gated, w["w_o"], "memory_out", keep_partial=True)      # the stream's next norm adds the slices
