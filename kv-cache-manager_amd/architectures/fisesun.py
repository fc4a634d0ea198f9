"""The Fisesun decoder as data: layers that norm a sublayer's OUTPUT before adding it to the stream,
x += rms(mixer(x)) * w1, then x += rms(ff(x)) * w2, the sublayers reading the stream itself.  Two kinds of mixer:
``attention`` (grouped queries; q and k normed over their whole projection, a half-split rotation rescaled by
wavelength, capped scores, a sliding window that keeps the sequence's first tokens in sight, values blended with those
of the first such layer) and ``mlstm`` (a matrix memory with exponential gates).  The feed-forward is a dense gated one
or a mixture of gated experts that a table names per token id, beside a shared expert.  The logits are capped.
Tensor names: ``l<i>.`` + norm1 | norm2 | mix.* | mlp.*; ``embed``, ``final.norm``, ``head``.
"""
from ..config.fisesun_config import NAME, FisesunConfig
from .. import parts  # noqa: F401  (registers the built-in part kinds)
from ..parts.base import LayerSpec, ModelSpec, PartSpec
from ..registry import ARCHITECTURES, Architecture


def _norm(cfg, name):
    return PartSpec("rmsnorm_chain", {"size": cfg.width, "eps": cfg.eps, "name": name})


def _mixer(cfg, layer, prefix, value_mix):
    m = layer.mixer
    if layer.type == "attention":
        position = None
        if m.rot_dims:
            sc = m.scaling
            position = PartSpec("rotary_halves", {"dims": m.rot_dims, "base": m.rot_base, "scaling_kind": "wavelength",
                                                  "scaling": (sc.factor, sc.low, sc.high, sc.original) if sc else None})
        return PartSpec("capped_window_attention", {
            "heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale, "softcap": m.softcap,
            "window": m.window, "keep_first": m.keep_first, "qk_norm_eps": cfg.eps, "value_mix": value_mix,
            "position": position}, prefix)
    return PartSpec("matrix_memory", {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "gate_cap": m.gate_cap, "eps": cfg.eps}, prefix)


def _feed_forward(cfg, ff, prefix):
    if ff.kind == "dense":
        return PartSpec("gated_mlp", {"intermediate_size": ff.ff, "activation": "silu"}, prefix)
    shared = PartSpec("gated_mlp", {"intermediate_size": ff.shared_ff, "activation": "silu"}, prefix + "shared.") if ff.shared_ff else None
    return PartSpec("routed_experts", {"experts": ff.experts, "top": ff.top, "ff": ff.ff, "routing": "table", "vocab_size": cfg.vocab,
                                       "activation": "silu_gated", "shared": shared}, prefix)


def fisesun_spec(cfg: FisesunConfig) -> ModelSpec:
    layers, source_seen = [], False
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        value_mix = None
        if layer.type == "attention" and layer.mixer.v_mix:      # the first such layer lends its values to the later ones
            value_mix = "blend" if source_seen else "source"
            source_seen = True
        parts_ = {"mixer": _mixer(cfg, layer, p + "mix.", value_mix), "norm_mixer_out": _norm(cfg, p + "norm1")}
        if layer.mlp:
            parts_.update({"ffn": _feed_forward(cfg, layer.mlp, p + "mlp."), "norm_ffn_out": _norm(cfg, p + "norm2")})
        layers.append(LayerSpec(name=f"l{i}", block="output_norm_residual", parts=parts_))
    return ModelSpec(
        architecture=NAME, hidden_size=cfg.width, vocab_size=cfg.vocab,
        embedding=PartSpec("scaled_token_embedding", {"vocab_size": cfg.vocab, "scale": cfg.embedding_scale, "name": "embed"}),
        layers=tuple(layers), schedule=tuple(range(len(layers))),
        final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "tied": False, "name": "head", "softcap": cfg.logit_softcap}),
        max_position=0)


ARCHITECTURES.register(NAME, Architecture(NAME, FisesunConfig, fisesun_spec))
