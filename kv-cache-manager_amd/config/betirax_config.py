"""Typed configuration of the Betirax decoder, read from the nested keys of its config.json.

  architecture    "Betirax"
  vocab, width    sizes of the vocabulary and of the residual stream
  embedding.scale factor on the embedding (default 1)
  norm.eps        epsilon of every norm (the layers' layer norms and the root-mean-square divisions inside the mixers)
  postln_alpha    factor on the stream when a sublayer's output is added, x <- ln(alpha x + sublayer(x)) (default 1)
  layers[i]       type: "attention" | "latent_attention"; mixer: that mixer's sizes; mlp: null, {kind: "dense", ff} or
                  {kind: "moe", expert: {ff}, router: {experts, top}, shared: {ff} or absent}

Mixers.  attention: heads, kv_heads (default heads), dim, vdim (default dim; the values are the keys, so it must equal dim),
scale, mask {size} (absent: every earlier token), q_temp {coef, every} (absent: none).  latent_attention: heads, dim,
rot_dim, vdim, kv_rank, q_rank, scale, rot {dims (default rot_dim), base (default 10000), scaling {factor, original, fast,
slow} or absent}, kv_from (absent or a layer's number: that layer's cached latents and rotated key parts are read and this
layer has no down-projection for keys and values of its own).
"""
from dataclasses import dataclass
from typing import Optional, Tuple

from .fisesun_config import _object
from .kasuvik_config import _number, _pos_int
from .model_config import ConfigError

NAME = "Betirax"
MIXERS = ("attention", "latent_attention")


@dataclass(frozen=True)
class RampScaling:
    """Pairs below a first index keep their frequency, pairs above a last one turn ``factor`` times slower, those between
    are blended; the two indices are where a pair makes ``fast`` and ``slow`` turns over ``original`` positions."""
    factor: float
    original: float
    fast: float
    slow: float

    def to_dict(self):
        original = int(self.original) if float(self.original).is_integer() else self.original
        return {"factor": self.factor, "original": original, "fast": self.fast, "slow": self.slow}


@dataclass(frozen=True)
class WindowAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = 0
    temp_coef: float = 0.0
    temp_every: int = 0

    def to_dict(self):
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.window:
            d["mask"] = {"size": self.window}
        if self.temp_every:
            d["q_temp"] = {"coef": self.temp_coef, "every": self.temp_every}
        return d


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot_dims: int = 0
    rot_base: float = 10000.0
    scaling: Optional[RampScaling] = None
    kv_from: Optional[int] = None

    def to_dict(self):
        d = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
             "q_rank": self.q_rank, "scale": self.scale}
        if self.rot_dim:
            d["rot"] = {"dims": self.rot_dims, "base": self.rot_base}
            if self.scaling:
                d["rot"]["scaling"] = self.scaling.to_dict()
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d

    def cache_shape(self):
        """What two layers must agree in for one to read the other's pages."""
        return (self.kv_rank, self.rot_dim, self.rot_dims, self.rot_base, self.scaling)


@dataclass(frozen=True)
class FeedForwardConfig:
    """kind "dense": W_down act(W_up h) with ``ff`` columns.  kind "moe": ``experts`` gated experts of ``ff`` columns of which
    a token uses ``top``, chosen by a router, and a shared expert of ``shared_ff`` columns (0: none)."""
    kind: str
    ff: int
    experts: int = 0
    top: int = 0
    shared_ff: int = 0

    def to_dict(self):
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        d = {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff:
            d["shared"] = {"ff": self.shared_ff}
        return d


@dataclass(frozen=True)
class BetiraxLayer:
    type: str
    mixer: object
    mlp: Optional[FeedForwardConfig] = None

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None}


def _attention(problems, w, m):
    heads, dim = _pos_int(problems, w, m, "heads"), _pos_int(problems, w, m, "dim")
    mask, window = _object(problems, w, m, "mask"), 0
    if mask is not None:
        window = _pos_int(problems, w + ".mask", mask, "size")
    temp, coef, every = _object(problems, w, m, "q_temp"), 0.0, 0
    if temp is not None:
        coef = _number(problems, w + ".q_temp", temp, "coef", positive=False)
        every = _pos_int(problems, w + ".q_temp", temp, "every")
    cfg = WindowAttentionConfig(heads=heads, kv_heads=_pos_int(problems, w, m, "kv_heads") if "kv_heads" in m else heads, dim=dim,
                                vdim=_pos_int(problems, w, m, "vdim") if "vdim" in m else dim, scale=_number(problems, w, m, "scale"),
                                window=window, temp_coef=coef, temp_every=every)
    if cfg.heads % cfg.kv_heads:
        problems.append(f"{w}: heads {cfg.heads} is not a multiple of kv_heads {cfg.kv_heads}")
    if cfg.vdim != cfg.dim:
        problems.append(f"{w}: the values are the keys, so vdim {cfg.vdim} must equal dim {cfg.dim}")
    return cfg


def _latent(problems, w, m):
    rot_dim = _pos_int(problems, w, m, "rot_dim", allow_zero=True) if "rot_dim" in m else 0
    rot, dims, base, scaling = _object(problems, w, m, "rot"), rot_dim, 10000.0, None
    if rot is not None and rot_dim:
        dims = _pos_int(problems, w + ".rot", rot, "dims", allow_zero=True) if "dims" in rot else rot_dim
        base = _number(problems, w + ".rot", rot, "base") if "base" in rot else 10000.0
        sc = _object(problems, w + ".rot", rot, "scaling")
        if sc is not None:
            ws = w + ".rot.scaling"
            scaling = RampScaling(*(_number(problems, ws, sc, k) for k in ("factor", "original", "fast", "slow")))
    source = m.get("kv_from")
    if source is not None and (not isinstance(source, int) or isinstance(source, bool) or source < 0):
        problems.append(f"{w}.kv_from must be a layer's number (got {source!r})")
        source = None
    cfg = LatentAttentionConfig(heads=_pos_int(problems, w, m, "heads"), dim=_pos_int(problems, w, m, "dim"), rot_dim=rot_dim,
                                vdim=_pos_int(problems, w, m, "vdim") if "vdim" in m else _pos_int(problems, w, m, "dim"),
                                kv_rank=_pos_int(problems, w, m, "kv_rank"), q_rank=_pos_int(problems, w, m, "q_rank"),
                                scale=_number(problems, w, m, "scale"), rot_dims=dims if rot_dim else 0, rot_base=base,
                                scaling=scaling, kv_from=source)
    if cfg.rot_dims % 2 or cfg.rot_dims > cfg.rot_dim:
        problems.append(f"{w}.rot.dims {cfg.rot_dims} must be even and at most rot_dim {cfg.rot_dim}")
    return cfg


def _feed_forward(problems, w, mlp):
    kind = mlp.get("kind")
    if kind == "dense":
        return FeedForwardConfig("dense", _pos_int(problems, w, mlp, "ff"))
    if kind == "moe":
        router = mlp.get("router")
        shared = _object(problems, w, mlp, "shared")
        cfg = FeedForwardConfig("moe", _pos_int(problems, w + ".expert", mlp.get("expert"), "ff"),
                                experts=_pos_int(problems, w + ".router", router, "experts"),
                                top=_pos_int(problems, w + ".router", router, "top"),
                                shared_ff=_pos_int(problems, w + ".shared", shared, "ff") if shared is not None else 0)
        if cfg.top > cfg.experts:
            problems.append(f"{w}.router.top {cfg.top} exceeds its {cfg.experts} experts")
        return cfg
    problems.append(f"{w}.kind {kind!r} is not supported (dense | moe, or a null mlp)")
    return None


@dataclass(frozen=True)
class BetiraxConfig:
    vocab: int
    width: int
    embedding_scale: float
    eps: float
    alpha: float
    layers: Tuple[BetiraxLayer, ...]

    @classmethod
    def from_dict(cls, raw: dict) -> "BetiraxConfig":
        problems = []
        vocab, width = _pos_int(problems, "config", raw, "vocab"), _pos_int(problems, "config", raw, "width")
        emb = raw.get("embedding")
        scale = _number(problems, "embedding", emb, "scale", positive=False) if isinstance(emb, dict) and "scale" in emb else 1.0
        eps = _number(problems, "norm", raw.get("norm"), "eps")
        alpha = _number(problems, "config", raw, "postln_alpha", positive=False) if "postln_alpha" in raw else 1.0
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            problems.append("'layers' must be a non-empty list")
            listed = []
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]"
            if not isinstance(entry, dict) or not isinstance(entry.get("mixer"), dict):
                problems.append(f"{where} must be an object with 'type' and 'mixer'")
                continue
            kind, mixer, mlp = entry.get("type"), entry["mixer"], entry.get("mlp")
            ff = None
            if mlp is not None:
                if not isinstance(mlp, dict):
                    problems.append(f"{where}.mlp must be an object or null")
                else:
                    ff = _feed_forward(problems, where + ".mlp", mlp)
            if kind == "attention":
                layers.append(BetiraxLayer(kind, _attention(problems, where + ".mixer", mixer), ff))
            elif kind == "latent_attention":
                layers.append(BetiraxLayer(kind, _latent(problems, where + ".mixer", mixer), ff))
            else:
                problems.append(f"{where}.type {kind!r} is not supported ({' | '.join(MIXERS)})")
        if len(layers) == len(listed):      # kv_from: an earlier latent layer with pages of its own and of the same shape
            for i, layer in enumerate(layers):
                j = layer.mixer.kv_from if layer.type == "latent_attention" else None
                if j is None:
                    continue
                where = f"layers[{i}].mixer.kv_from"
                if j >= i or layers[j].type != "latent_attention":
                    problems.append(f"{where} {j} must name an earlier latent_attention layer")
                elif layers[j].mixer.kv_from is not None:
                    problems.append(f"{where} {j} names a layer that has no keys and values of its own")
                elif layers[j].mixer.cache_shape() != layer.mixer.cache_shape():
                    problems.append(f"{where} {j}: kv_rank, rot_dim and rot must equal that layer's")
        if problems:
            raise ConfigError("config.json: " + "; ".join(problems))
        return cls(vocab=vocab, width=width, embedding_scale=scale, eps=eps, alpha=alpha, layers=tuple(layers))

    def to_dict(self) -> dict:
        return {"architecture": NAME, "vocab": self.vocab, "width": self.width, "embedding": {"scale": self.embedding_scale},
                "norm": {"eps": self.eps}, "postln_alpha": self.alpha, "layers": [l.to_dict() for l in self.layers]}
