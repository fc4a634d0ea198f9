"""Parts for layers that norm a sublayer's output before adding it to the residual stream
(x += norm_out(sublayer(norm_in(x))), or x += norm_out(sublayer(x)) where the sublayers read the stream itself):
an RMS norm whose arithmetic is 32-bit throughout, the arrangements that chain such norms so that a layer boundary
is one launch, an embedding with a factor, and a gated feed-forward with a choice of activation.  Every size, constant and tensor name is a parameter.
"""
import torch

from ..registry import BLOCKS, EMBEDDINGS, FEED_FORWARDS, NORMS
from .base import Block, Embedding, FeedForward, Norm, ParamSpec
from .llama_parts import _linear


def f32_params(tensors):
    """Small tensors (norm weights, biases, per-head factors, convolution taps) as float32: widening what a
    checkpoint stores in 16 bits is exact, and the kernels that use them compute in 32-bit."""
    return {k: v.float().contiguous() for k, v in tensors.items()}


def linear32(ctx, step, x, w, name, keep_partial=False):
    """x @ w^T as 32-bit rows for a consumer that computes in 32-bit: the product's 32-bit sums as they are, from this
    package's kernels for few rows and from the vendor library's for many (``ops.gemm`` decides, as for every product);
    no path rounds the sums, so what enters a recurrence is as exact at one row as at thousands.  Few-row products stay
    split along K with a second launch that adds the slices up: run unsplit they were slower by more than that launch
    costs (a decode step at width 2048 0.71 -> 0.80 ms, at 4096 1.25 -> 1.49 ms).  ``keep_partial``: the product may come
    back as ops.PartialSums for a consumer that adds the slices itself.  The chained norm does: rows up to 8,192 wide
    stay in registers through all its stages, and the slices are added as they are loaded (5 us a launch at width 2048;
    the form that reads a row once per stage took 27 us with slices, more than the launch it saved).  Mixers' output
    projections use it; a feed-forward's does not where another part (a routed feed-forward's sum) starts from it."""
    return _linear(ctx, step, x, w, name, keep_partial=keep_partial, dtype=torch.float32)


class BranchPair:
    """Two sublayer outputs (32-bit tensors, or the un-added slices of their last products) side by side, still to be combined as combine * (n(a) * wa + n(b) * wb)
    (n: division by the root mean square): what a mixer of two halves hands to the arrangement, which
    passes it on to the norm that adds it to the stream (one launch for all of it)."""

    def __init__(self, a, wa, b, wb, combine):
        self.a, self.wa, self.b, self.wb, self.combine = a, wa, b, wb, combine


@NORMS.register("rmsnorm_chain")
class ChainedRMSNorm(Norm):
    """out = x / sqrt(mean(x^2) + eps) * weight with every operation in 32-bit and one rounding at the end.
    ``forward`` also takes the previous sublayer's output that is still to be normed and added (``add``: what
    ``pending`` of the norm after that sublayer made), so that addition and norm are one launch.
    params: size, eps; name: the checkpoint name of the weight (default prefix + "weight")."""

    capturable = True
    accepts_partial_sums = True      # ``add`` is taken as it comes (ops.NormedBranches)

    def param_specs(self):
        name = self.params.get("name", self.prefix + "weight")
        return [ParamSpec("weight", ((name, (self.params["size"],)),), role="vector")]

    def bind(self, tensors):
        super().bind(f32_params(tensors))

    def pending(self, value):
        """A sublayer's output (a 32-bit tensor, ops.PartialSums, or a BranchPair) as what the stream's next norm adds:
        x += n(value) * weight."""
        ops = self.ctx.ops
        if isinstance(value, BranchPair):
            return ops.NormedBranches(value.a, self.w["weight"], value.b, value.wa, value.wb, value.combine)
        return ops.NormedBranches(value, self.w["weight"])

    def forward(self, x, out, add=None, rows=None):
        ops = self.ctx.ops
        if add is not None and not isinstance(add, ops.NormedBranches):
            raise TypeError("rmsnorm_chain adds what a norm's pending() made (ops.NormedBranches)")
        ops.rmsnorm_chain(x, self.params["eps"], pending=add, weight=self.w["weight"], out=out, rows=rows)
        return out

    def read_stream(self, step, x, add=None):
        """x += what is still to be added (``add``: made by a norm's ``pending``), then the stream's rows as a sublayer
        reads them that takes the stream itself, not a normed copy: rounded to the compute dtype in the same launch, or,
        where the compute dtype is 32-bit, x itself."""
        ops = self.ctx.ops
        if add is not None and not isinstance(add, ops.NormedBranches):
            raise TypeError("rmsnorm_chain adds what a norm's pending() made (ops.NormedBranches)")
        if self.ctx.dtype == torch.float32:
            if add is not None:
                ops.rmsnorm_chain(x, self.params["eps"], pending=add)
            return x
        out = step.ws("stream_rows", (step.rows, x.shape[1]))
        ops.rmsnorm_chain(x, self.params["eps"], pending=add, out=out, plain=True)
        return out


@BLOCKS.register("sandwich_residual")
class SandwichResidual(Block):
    """x += norm_mixer_out(mixer(norm_mixer(x))); x += norm_ffn_out(ffn(norm_ffn(x))), the second half only
    where the layer has a feed-forward.  Each addition is done by the norm that reads the stream next."""

    capturable = True

    def forward(self, step, x, pending):
        p = self.parts
        buf = step.ws("normed", (step.rows, x.shape[1]))
        p["norm_mixer"].forward(x, buf, add=pending)
        pending = p["norm_mixer_out"].pending(p["mixer"].forward(step, buf))
        if "ffn" in p:
            p["norm_ffn"].forward(x, buf, add=pending)
            pending = p["norm_ffn_out"].pending(p["ffn"].forward(step, buf))
        return pending


@BLOCKS.register("output_norm_residual")
class OutputNormResidual(Block):
    """x += norm_mixer_out(mixer(x)); x += norm_ffn_out(ffn(x)), the second half only where the layer has a
    feed-forward.  No norm on the way in: the sublayers read the stream itself.  Each addition is done by the launch
    that hands the stream to its next reader."""

    capturable = True

    def forward(self, step, x, pending):
        p = self.parts
        h = p["norm_mixer_out"].read_stream(step, x, add=pending)
        pending = p["norm_mixer_out"].pending(p["mixer"].forward(step, h))
        if "ffn" in p:
            h = p["norm_ffn_out"].read_stream(step, x, add=pending)
            pending = p["norm_ffn_out"].pending(p["ffn"].forward(step, h))
        return pending


@EMBEDDINGS.register("scaled_token_embedding")
class ScaledTokenEmbedding(Embedding):
    """x = float(table[token]) * scale.  params: vocab_size, scale; name: the table's checkpoint name."""

    capturable = True

    def param_specs(self):
        name = self.params.get("name", self.prefix + "weight")
        return [ParamSpec("table", ((name, (self.params["vocab_size"], self.ctx.hidden_size)),), role="table")]

    def forward(self, step, out):
        self.ctx.ops.embed_scaled(step.tokens, self.w["table"], out, self.params.get("scale", 1.0))
        return out

    def bytes_read(self, rows):
        table = self.w["table"]
        return rows * table.shape[1] * table.element_size()

    def flops(self, rows, attended=0):
        return 0.0


@FEED_FORWARDS.register("gated_mlp")
class GatedFeedForward(FeedForward):
    """down(act(gate(h)) * up(h)), gate and up as one fused projection whose 32-bit sums go straight into the
    activation (steps of few rows in bfloat16 with silu: in the product's own epilogue).  params: intermediate_size, activation ("relu" | "silu" | "gelu_tanh"); gate, up, down: the
    checkpoint names after the prefix (defaults "gate", "up", "down").  The result is 32-bit: a norm reads it."""

    capturable = True

    def param_specs(self):
        H, I, pre, p = self.ctx.hidden_size, self.params["intermediate_size"], self.prefix, self.params
        return [ParamSpec("w_gate_up", ((pre + p.get("gate", "gate"), (I, H)), (pre + p.get("up", "up"), (I, H)))),
                ParamSpec("w_down", ((pre + p.get("down", "down"), (H, I)),))]

    def forward(self, step, h):
        I, ops = self.params["intermediate_size"], self.ctx.ops
        act = step.ws("gated_act", (step.rows, I))
        kind = self.params.get("activation", "silu")
        # few rows in bfloat16 with silu: the product that streams gate and up rows together and applies the activation
        # in its epilogue, one launch (the activation is rounded once more on the way, within the result's own rounding)
        if not (kind == "silu" and act.dtype == torch.bfloat16 and torch.is_tensor(h) and ops.gemm_swiglu(h, self.w["w_gate_up"], act)):
            gu = linear32(self.ctx, step, h, self.w["w_gate_up"], "gated_gate_up")
            ops.gated_act(gu, act, kind)
        return linear32(self.ctx, step, act, self.w["w_down"], "gated_out")


@FEED_FORWARDS.register("plain_mlp")
class PlainFeedForward(FeedForward):
    """down(act(up(h))): a feed-forward without a gate; the first product's 32-bit sums go straight into the activation.
    params: intermediate_size, activation ("relu" | "silu" | "gelu_tanh"); up, down: the checkpoint names after the
    prefix (defaults "up", "down").  The result is 32-bit: a norm reads it."""

    capturable = True

    def param_specs(self):
        H, I, pre, p = self.ctx.hidden_size, self.params["intermediate_size"], self.prefix, self.params
        return [ParamSpec("w_up", ((pre + p.get("up", "up"), (I, H)),)),
                ParamSpec("w_down", ((pre + p.get("down", "down"), (H, I)),))]

    def forward(self, step, h):
        I, ops = self.params["intermediate_size"], self.ctx.ops
        up = linear32(self.ctx, step, h, self.w["w_up"], "plain_up", keep_partial=True)      # slices are added by the activation's launch
        act = step.ws("plain_act", (step.rows, I))
        ops.act_rows(up, act, self.params.get("activation", "gelu_tanh"))
        return linear32(self.ctx, step, act, self.w["w_down"], "plain_out", keep_partial=True)      # the stream's next norm adds the slices
