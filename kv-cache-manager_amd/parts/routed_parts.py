"""A routed feed-forward (mixture of experts): a router picks, for every row, a few of many small feed-forward
layers; the row's output is the sum of theirs, weighted by the router's scores.  Every size, constant and tensor
name is a parameter.
"""
import torch

from ..registry import FEED_FORWARDS
from .base import FeedForward, ParamSpec
from .chain_norm_parts import linear32


@FEED_FORWARDS.register("routed_experts")
class RoutedExperts(FeedForward):
    """Router logits z = W_router h in 32-bit, scores s = softmax(z) over all experts; the ``top`` experts with the
    largest scores each compute W_down act(W_up h), act = the square of relu, and the output is the sum of theirs times
    their scores as they are (not renormalized).  Experts have no biases.
    params: experts, top, ff; router (the router's checkpoint name after the prefix, default "router"); expert
    (a pattern for an expert's prefix, default "e{}."), up, down (names after it).  The result is 32-bit."""

    capturable = True
    # rows from which a bfloat16 step groups its (row, slot) pairs by expert; below, every pair streams its expert's rows itself
    GROUPED_MIN_ROWS = 16

    def param_specs(self):
        H, p, pre = self.ctx.hidden_size, self.params, self.prefix
        E, F = p["experts"], p["ff"]
        names = [pre + p.get("expert", "e{}.").format(e) for e in range(E)]
        return [ParamSpec("w_router", ((pre + p.get("router", "router"), (E, H)),)),
                ParamSpec("w_up", tuple((n + p.get("up", "up"), (F, H)) for n in names)),
                ParamSpec("w_down", tuple((n + p.get("down", "down"), (H, F)) for n in names))]

    def bind(self, tensors):
        E, F, H = self.params["experts"], self.params["ff"], self.ctx.hidden_size
        r = tensors["w_router"]
        extra = -r.shape[0] % 16      # the few-row products take widths that are multiples of 16; the route reads the first E
        if extra:
            r = torch.cat([r, torch.zeros(extra, r.shape[1], dtype=r.dtype, device=r.device)], 0)
        super().bind({"w_router": r, "w_up": tensors["w_up"].view(E, F, H), "w_down": tensors["w_down"].view(E, H, F)})

    def bytes_read(self, rows):
        """The router, and the experts that ``rows`` rows can reach at most."""
        p, w = self.params, self.w
        reached = min(p["experts"], rows * p["top"])
        per_expert = (w["w_up"][0].numel() + w["w_down"][0].numel()) * w["w_up"].element_size()
        return w["w_router"].numel() * w["w_router"].element_size() + reached * per_expert

    def flops(self, rows, attended=0):
        p, H = self.params, self.ctx.hidden_size
        return 2.0 * rows * (p["experts"] * H + p["top"] * 2 * p["ff"] * H)

    def forward(self, step, h):
        ops, p, w = self.ctx.ops, self.params, self.w
        E, top, F, T = p["experts"], p["top"], p["ff"], step.rows
        logits = linear32(self.ctx, step, h, w["w_router"], "routed_logits")
        chosen = step.ws("routed_chosen", (T, top), torch.int32)
        weight = step.ws("routed_weight", (T, top), torch.float32)
        ops.moe_route(logits, E, top, chosen, weight, rows=T)
        H = self.ctx.hidden_size
        act = step.ws("routed_act", (T, top * F)).view(T * top, F)
        out = step.ws("routed_out", (T, H), torch.float32)
        if T >= self.GROUPED_MIN_ROWS and ops.moe_grouped_supported(H, F, E, act.dtype) and h.stride(0) % 8 == 0:
            # many rows: the pairs grouped by expert, tiles on the matrix cores, every expert's weights read once per tile
            order = step.ws("routed_order", (T, top), torch.int32)
            tiles = step.flat("routed_tiles", ops.moe_grouped_tiles(max(T, step.limits.max_tokens if step.limits else T) * top, E), torch.int32)
            y = step.ws("routed_y", (T, top * H), torch.float32).view(T * top, H)
            return ops.moe_grouped(h, w["w_up"], w["w_down"], chosen, weight, order, tiles, act, y, out)
        return ops.moe_rows(h, w["w_up"], w["w_down"], chosen, weight, act, out)
