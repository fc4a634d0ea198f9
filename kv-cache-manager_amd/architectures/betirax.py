"""The Betirax decoder as data: layers that norm AFTER the sum, x <- ln(alpha x + mixer(x)) * w1, then
x <- ln(alpha x + ff(x)) * w2 (a layer norm with a weight and no bias; the sublayers read x itself).  Two kinds of mixer:
``attention`` (grouped queries with biases, a norm per head, keys that double as values, a query temperature by position,
a bias by distance, a sliding window and a gate per element) and ``latent_attention`` (queries through a latent of their
own; one cached latent and one rotated key part per token from which every head's keys and values are made; rotary
positions rescaled pair by pair; a gate per element; a layer may read an earlier layer's pages).  The feed-forward is a
dense one with the tanh form of gelu, or a mixture of gated experts weighted by the softmax over the chosen logits beside a
shared expert.  The output head is the embedding table itself.
Tensor names: ``l<i>.`` + norm1 | norm2 | mix.* | mlp.*; ``embed``, ``final.norm``.
"""
from ..config.betirax_config import NAME, BetiraxConfig
from .. import parts  # noqa: F401  (registers the built-in part kinds)
from ..parts.base import LayerSpec, ModelSpec, PartSpec
from ..registry import ARCHITECTURES, Architecture

SLOPE_EXPONENT = 8.0      # head h's distance slope is 2^(-8 (h + 1) / heads)


def _norm(cfg, name, alpha=1.0):
    return PartSpec("layernorm_post", {"size": cfg.width, "eps": cfg.eps, "alpha": alpha, "name": name})


def _mixer(cfg, layer, prefix):
    m = layer.mixer
    if layer.type == "attention":
        return PartSpec("headnorm_window_attention", {
            "heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale, "window": m.window,
            "eps": cfg.eps, "bias": True, "values": "keys", "q_temp": (m.temp_coef, m.temp_every) if m.temp_every else None,
            "distance_bias": True, "slope_exponent": SLOPE_EXPONENT, "gate": True}, prefix)
    position = None
    if m.rot_dims:
        sc = m.scaling
        position = PartSpec("rotary_halves", {"dims": m.rot_dims, "base": m.rot_base,
                                              "scaling": (sc.factor, sc.original, sc.fast, sc.slow) if sc else None})
    return PartSpec("latent_attention", {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale,
                                         "window": 0, "eps": cfg.eps, "rot_dim": m.rot_dim, "position": position,
                                         "q_rank": m.q_rank, "gate": True, "shares_kv": m.kv_from is not None}, prefix)


def _feed_forward(cfg, ff, prefix):
    if ff.kind == "dense":
        return PartSpec("plain_mlp", {"intermediate_size": ff.ff, "activation": "gelu_tanh"}, prefix)
    shared = PartSpec("gated_mlp", {"intermediate_size": ff.shared_ff, "activation": "silu"}, prefix + "shared.") if ff.shared_ff else None
    return PartSpec("routed_experts", {"experts": ff.experts, "top": ff.top, "ff": ff.ff, "routing": "softmax_chosen",
                                       "activation": "silu_gated", "shared": shared}, prefix)


def betirax_spec(cfg: BetiraxConfig) -> ModelSpec:
    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        parts_ = {"mixer": _mixer(cfg, layer, p + "mix."), "norm_mixer_out": _norm(cfg, p + "norm1", cfg.alpha)}
        if layer.mlp:
            parts_.update({"ffn": _feed_forward(cfg, layer.mlp, p + "mlp."), "norm_ffn_out": _norm(cfg, p + "norm2", cfg.alpha)})
        source = layer.mixer.kv_from if layer.type == "latent_attention" else None
        layers.append(LayerSpec(name=f"l{i}", block="postnorm_residual", parts=parts_,
                                cache_from=None if source is None else {"mixer": f"l{source}"}))
    return ModelSpec(
        architecture=NAME, hidden_size=cfg.width, vocab_size=cfg.vocab,
        embedding=PartSpec("scaled_token_embedding", {"vocab_size": cfg.vocab, "scale": cfg.embedding_scale, "name": "embed"}),
        layers=tuple(layers), schedule=tuple(range(len(layers))),
        final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "tied": True, "name": "head"}),
        max_position=0)


ARCHITECTURES.register(NAME, Architecture(NAME, BetiraxConfig, betirax_spec))
