"""A routed feed-forward (mixture of experts): for every row a few of many small feed-forward layers are picked, by a
router's scores or by a table per token id; the row's output is the sum of theirs, weighted.  A shared feed-forward
may run for every row beside them.  Every size, constant and tensor name is a parameter.
"""
import torch

from ..registry import FEED_FORWARDS
from .base import FeedForward, ParamSpec
from .chain_norm_parts import linear32


def interleave_gate_up(gate, up):
    """[E, F, K] gate and up matrices of gated experts as the one matrix [E, 2F, K] the routed kernels read: rows
    interleaved sixteen at a time (gate 0..15, up 0..15, gate 16..31, ...).  F must be a multiple of 16."""
    E, F, K = gate.shape
    if F % 16 or tuple(up.shape) != (E, F, K):
        raise ValueError("interleave_gate_up: [E, F, K] twice, F a multiple of 16")
    return torch.stack([gate.reshape(E, F // 16, 16, K), up.reshape(E, F // 16, 16, K)], dim=2).reshape(E, 2 * F, K).contiguous()


@FEED_FORWARDS.register("routed_experts")
class RoutedExperts(FeedForward):
    """Which experts a row uses (``routing``):
      "softmax" (default)  router logits z = W_router h in 32-bit, scores s = softmax(z) over all experts; the ``top``
                           experts with the largest scores, weighted by their scores as they are (not renormalized)
      "softmax_chosen"     the ``top`` experts with the largest logits, weighted by the softmax over those logits alone
      "table"              an integer table [vocabulary, top] names the experts of every token id; each weighs 1 / top
    What an expert computes (``activation``):
      "relu2" (default)    W_down act(W_up h), act = the square of relu
      "silu_gated"         W_down (silu(W_gate h) * (W_up h))
    Experts have no biases.  ``shared``: a PartSpec of a feed-forward that runs for every row and is added (default none).
    params: experts, top, ff, routing, activation, shared, vocab_size (rows of the table; default: as stored); router / table (the checkpoint name after the prefix, defaults
    "router", "table"); expert (a pattern for an expert's prefix, default "e{}."), gate, up, down (names after it).
    The result is 32-bit."""

    capturable = True
    sub_part_names = ("shared",)
    # rows from which a bfloat16 step groups its (row, slot) pairs by expert; below, every pair streams its expert's rows itself
    GROUPED_MIN_ROWS = 16

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.routing, self.activation = params.get("routing", "softmax"), params.get("activation", "relu2")
        if self.routing not in ("softmax", "softmax_chosen", "table"):
            raise ValueError(f"routed_experts {prefix!r}: routing {self.routing!r} is not supported (softmax | softmax_chosen | table)")
        if self.activation not in ("relu2", "silu_gated"):
            raise ValueError(f"routed_experts {prefix!r}: activation {self.activation!r} is not supported (relu2 | silu_gated)")
        self.gated = self.activation == "silu_gated"
        sh = params.get("shared")
        self.shared = FEED_FORWARDS.get(sh.kind)(sh.params, sh.prefix, ctx) if sh is not None else None
        self.F = params["ff"]

    def sub_parts(self):
        return (self.shared,) if self.shared is not None else ()

    def param_specs(self):
        H, p, pre = self.ctx.hidden_size, self.params, self.prefix
        E, F = p["experts"], p["ff"]
        names = [pre + p.get("expert", "e{}.").format(e) for e in range(E)]
        specs = [ParamSpec("w_up", tuple((n + p.get("up", "up"), (F, H)) for n in names)),
                 ParamSpec("w_down", tuple((n + p.get("down", "down"), (H, F)) for n in names))]
        if self.gated:
            specs.append(ParamSpec("w_gate", tuple((n + p.get("gate", "gate"), (F, H)) for n in names)))
        if self.routing == "table":
            specs.append(ParamSpec("table", ((pre + p.get("table", "table"), (p.get("vocab_size", -1), p["top"])),), role="index", distinct_below=E))
        else:
            specs.append(ParamSpec("w_router", ((pre + p.get("router", "router"), (E, H)),)))
        return specs

    def bind(self, tensors):
        E, F, H = self.params["experts"], self.params["ff"], self.ctx.hidden_size
        bound = {}
        if self.routing == "table":
            bound["table"] = tensors["table"].contiguous()
        else:
            r = tensors["w_router"]
            extra = -r.shape[0] % 16      # the few-row products take widths that are multiples of 16; the route reads the first E
            if extra:
                r = torch.cat([r, torch.zeros(extra, r.shape[1], dtype=r.dtype, device=r.device)], 0)
            bound["w_router"] = r
        up, down = tensors["w_up"].view(E, F, H), tensors["w_down"].view(E, H, F)
        if self.gated:
            # gate and up as one matrix, rows interleaved sixteen at a time; columns that bring F to a multiple of 16 are zero
            # (silu(0) * 0 = 0, and the down matrix has zero columns there)
            gate, pad = tensors["w_gate"].view(E, F, H), -F % 16
            if pad:
                zeros = torch.zeros(E, pad, H, dtype=up.dtype, device=up.device)
                gate, up = torch.cat([gate, zeros], 1), torch.cat([up, zeros], 1)
                down = torch.cat([down, torch.zeros(E, H, pad, dtype=down.dtype, device=down.device)], 2).contiguous()
            up = interleave_gate_up(gate, up)
            self.F = F + pad
        bound["w_up"], bound["w_down"] = up, down
        super().bind(bound)

    def bytes_read(self, rows):
        """The router (or the rows' table entries), and the experts that ``rows`` rows can reach at most."""
        p, w = self.params, self.w
        reached = min(p["experts"], rows * p["top"])
        per_expert = (w["w_up"][0].numel() + w["w_down"][0].numel()) * w["w_up"].element_size()
        routing = rows * p["top"] * 4 if self.routing == "table" else w["w_router"].numel() * w["w_router"].element_size()
        return routing + reached * per_expert

    def flops(self, rows, attended=0):
        p, H = self.params, self.ctx.hidden_size
        router = 0 if self.routing == "table" else p["experts"] * H
        return 2.0 * rows * (router + p["top"] * (3 if self.gated else 2) * p["ff"] * H)

    def forward(self, step, h):
        ops, p, w = self.ctx.ops, self.params, self.w
        E, top, F, T = p["experts"], p["top"], self.F, step.rows
        chosen = step.ws("routed_chosen", (T, top), torch.int32)
        weight = step.ws("routed_weight", (T, top), torch.float32)
        if self.routing == "table":
            ops.moe_table_route(step.tokens, w["table"], top, chosen, weight, rows=T)
        else:
            logits = linear32(self.ctx, step, h, w["w_router"], "routed_logits", keep_partial=True)      # the route adds the slices
            ops.moe_route(logits, E, top, chosen, weight, rows=T, over_chosen=self.routing == "softmax_chosen")
        add = self.shared.forward(step, h) if self.shared is not None else None      # 32-bit [T, H]: the experts' sum starts from it
        H = self.ctx.hidden_size
        act = step.ws("routed_act", (T, top * F)).view(T * top, F)
        out = step.ws("routed_out", (T, H), torch.float32)
        if T >= self.GROUPED_MIN_ROWS and ops.moe_grouped_supported(H, F, E, act.dtype) and h.stride(0) % 8 == 0:
            # many rows: the pairs grouped by expert, tiles on the matrix cores, every expert's weights read once per tile
            order = step.ws("routed_order", (T, top), torch.int32)
            tiles = step.flat("routed_tiles", ops.moe_grouped_tiles(max(T, step.limits.max_tokens if step.limits else T) * top, E), torch.int32)
            y = step.ws("routed_y", (T, top * H), torch.float32).view(T * top, H)
            return ops.moe_grouped(h, w["w_up"], w["w_down"], chosen, weight, order, tiles, act, y, out, gated=self.gated, add=add)
        return ops.moe_rows(h, w["w_up"], w["w_down"], chosen, weight, act, out, gated=self.gated, add=add)
