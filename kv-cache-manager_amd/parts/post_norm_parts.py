"""Parts for layers that norm AFTER the sum: x <- ln(alpha * x + mixer(x)) * w1, then x <- ln(alpha * x + ff(x)) * w2,
with ln(v) = (v - mean(v)) / sqrt(mean((v - mean(v))^2) + eps): a layer norm with a weight and no bias, the stream scaled
by ``alpha`` before the sublayer's output is added.  The sublayers read the stream itself.  Every size, constant and
tensor name is a parameter.
"""
import torch

from ..registry import BLOCKS, NORMS
from .base import Block, Norm, ParamSpec
from .chain_norm_parts import f32_params


class StreamRows:
    """What an arrangement that leaves nothing to be added hands to the next one instead: the stream's rows as its
    sublayers read them (the compute dtype's rounding of x, made by the launch that wrote x), or None."""

    def __init__(self, rows):
        self.rows = rows

    def materialize(self):
        return None      # nothing is pending


@NORMS.register("layernorm_post")
class PostLayerNorm(Norm):
    """ln(v) * weight with every operation in 32-bit: the mean is taken off, the mean of the squared deviations (plus eps)
    is the variance, no bias.  ``add_norm`` does a layer's x <- ln(alpha * x + y) * weight in one launch and leaves the new
    rows for the next reader; ``forward`` norms gathered rows (the model's last norm).
    params: size, eps, alpha (the factor on the stream when a sublayer's output is added; default 1); name: the checkpoint
    name of the weight (default prefix + "weight")."""

    capturable = True
    accepts_partial_sums = True      # ``add`` is taken as it comes (StreamRows: nothing to add)

    def param_specs(self):
        name = self.params.get("name", self.prefix + "weight")
        return [ParamSpec("weight", ((name, (self.params["size"],)),), role="vector")]

    def bind(self, tensors):
        super().bind(f32_params(tensors))

    def add_norm(self, step, x, value):
        """x <- ln(alpha * x + value) * weight; ``value``: a sublayer's output (a 32-bit tensor, ops.PartialSums, or an
        ops.BiasedOutput of either).  Returns the new rows as the next sublayer reads them."""
        ops = self.ctx.ops
        out = None if self.ctx.dtype == torch.float32 else step.ws("stream_rows", (step.rows, x.shape[1]))
        ops.layernorm_post(x, self.w["weight"], self.params["eps"], alpha=self.params.get("alpha", 1.0), add=value, out=out)
        return x if out is None else out

    def forward(self, x, out, add=None, rows=None):
        if add is not None and not isinstance(add, StreamRows):
            raise TypeError("layernorm_post norms the stream as it is: a pending addition belongs to the arrangement before it")
        self.ctx.ops.layernorm_post(x, self.w["weight"], self.params["eps"], out=out, rows=rows)
        return out


@BLOCKS.register("postnorm_residual")
class PostNormResidual(Block):
    """x <- norm_mixer_out(alpha * x + mixer(x)); x <- norm_ffn_out(alpha * x + ffn(x)), the second half only where the
    layer has a feed-forward; alpha is the norms' parameter.  Each norm's launch adds, norms, writes the stream and
    leaves its rows in the compute dtype for the sublayer that reads them next."""

    capturable = True

    def forward(self, step, x, pending):
        p = self.parts
        if isinstance(pending, StreamRows) and pending.rows is not None:
            h = pending.rows
        elif pending is None or isinstance(pending, StreamRows):
            # the model's first layer: the embedding's rows, rounded for the products (32-bit: the stream itself)
            ctx = p["norm_mixer_out"].ctx
            h = x
            if ctx.dtype != torch.float32:
                h = step.ws("stream_rows", (step.rows, x.shape[1]))
                ctx.ops.rmsnorm_chain(x, 0.0, out=h, plain=True)      # the rows as they are, rounded once
        else:
            raise TypeError("postnorm_residual follows arrangements that leave nothing to be added")
        h = p["norm_mixer_out"].add_norm(step, x, p["mixer"].forward(step, h))
        if "ffn" in p:
            h = p["norm_ffn_out"].add_norm(step, x, p["ffn"].forward(step, h))
        return StreamRows(h)
