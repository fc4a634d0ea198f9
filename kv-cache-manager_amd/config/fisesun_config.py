"""Typed configuration of the Fisesun decoder, read from the nested keys of its config.json.

  architecture    "Fisesun"
  vocab, width    sizes of the vocabulary and of the residual stream
  embedding.scale factor on the embedding (default 1)
  norm.eps        epsilon of every root-mean-square division
  logit_softcap   c > 0: logits <- c tanh(logits / c) (absent or 0: none)
  layers[i]       type: "attention" | "mlstm"; mixer: that mixer's sizes; mlp: null, {kind: "dense", ff} or
                  {kind: "moe", expert: {ff}, router: {experts, top}, shared: {ff} or absent}

Mixers.  attention: heads, kv_heads, dim, vdim, scale, softcap (absent or 0: none), mask {size, keep_first} (absent:
every earlier token; keep_first defaults to 0), rot {dims, base, scaling {factor, low, high, original} or absent}
(rot absent or dims 0: no rotation), v_mix (default false).  kv_heads defaults to heads, vdim to dim, rot.base to 10000.
mlstm: heads, dim, vdim, gate_cap.
"""
from dataclasses import dataclass
from typing import Optional, Tuple

from .kasuvik_config import _number, _pos_int
from .model_config import ConfigError

NAME = "Fisesun"
MIXERS = ("attention", "mlstm")


@dataclass(frozen=True)
class WavelengthScaling:
    """Pairs whose wavelength is shorter than original/high keep their frequency, those longer than original/low turn
    ``factor`` times slower, those between are blended."""
    factor: float
    low: float
    high: float
    original: float

    def to_dict(self):
        return {"factor": self.factor, "low": self.low, "high": self.high, "original": self.original}


@dataclass(frozen=True)
class CappedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float = 0.0
    window: int = 0
    keep_first: int = 0
    rot_dims: int = 0
    rot_base: float = 10000.0
    scaling: Optional[WavelengthScaling] = None
    v_mix: bool = False

    def to_dict(self):
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
             "v_mix": self.v_mix}
        if self.softcap:
            d["softcap"] = self.softcap
        if self.window:
            d["mask"] = {"size": self.window, "keep_first": self.keep_first}
        if self.rot_dims:
            d["rot"] = {"dims": self.rot_dims, "base": self.rot_base}
            if self.scaling:
                d["rot"]["scaling"] = self.scaling.to_dict()
        return d


@dataclass(frozen=True)
class MemoryConfig:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    def to_dict(self):
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


@dataclass(frozen=True)
class FeedForwardConfig:
    """kind "dense": one gated feed-forward of ``ff`` columns.  kind "moe": ``experts`` gated experts of ``ff`` columns of
    which a token uses ``top``, named by a table per token id, and a shared expert of ``shared_ff`` columns (0: none)."""
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
class FisesunLayer:
    type: str
    mixer: object
    mlp: Optional[FeedForwardConfig] = None

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None}


def _object(problems, where, d, key):
    """d[key] when it is an object, None when it is absent or null; anything else is a problem."""
    v = d.get(key)
    if v is None or isinstance(v, dict):
        return v
    problems.append(f"{where}.{key} must be an object or absent")
    return None


def _attention(problems, w, m):
    heads, dim = _pos_int(problems, w, m, "heads"), _pos_int(problems, w, m, "dim")
    rot, dims, base, scaling = _object(problems, w, m, "rot"), 0, 10000.0, None
    if rot is not None:
        dims = _pos_int(problems, w + ".rot", rot, "dims", allow_zero=True)
        if dims:
            base = _number(problems, w + ".rot", rot, "base") if "base" in rot else 10000.0
            sc = _object(problems, w + ".rot", rot, "scaling")
            if sc is not None:
                ws = w + ".rot.scaling"
                scaling = WavelengthScaling(*(_number(problems, ws, sc, k) for k in ("factor", "low", "high", "original")))
                if scaling.high == scaling.low:
                    problems.append(f"{ws}: low and high must differ")
    mask, window, keep = _object(problems, w, m, "mask"), 0, 0
    if mask is not None:
        window = _pos_int(problems, w + ".mask", mask, "size")
        keep = _pos_int(problems, w + ".mask", mask, "keep_first", allow_zero=True) if "keep_first" in mask else 0
    v_mix = m.get("v_mix", False)
    if not isinstance(v_mix, bool):
        problems.append(f"{w}.v_mix must be true or false")
        v_mix = False
    cfg = CappedAttentionConfig(
        heads=heads, kv_heads=_pos_int(problems, w, m, "kv_heads") if "kv_heads" in m else heads, dim=dim,
        vdim=_pos_int(problems, w, m, "vdim") if "vdim" in m else dim, scale=_number(problems, w, m, "scale"),
        softcap=_number(problems, w, m, "softcap", positive=False) if m.get("softcap") is not None else 0.0,
        window=window, keep_first=keep, rot_dims=dims, rot_base=base, scaling=scaling, v_mix=v_mix)
    if cfg.heads % cfg.kv_heads:
        problems.append(f"{w}: heads {cfg.heads} is not a multiple of kv_heads {cfg.kv_heads}")
    if cfg.rot_dims % 2 or cfg.rot_dims > cfg.dim:
        problems.append(f"{w}.rot.dims {cfg.rot_dims} must be even and at most dim {cfg.dim}")
    if cfg.softcap < 0:
        problems.append(f"{w}.softcap must not be negative")
    return cfg


def _memory(problems, w, m):
    return MemoryConfig(heads=_pos_int(problems, w, m, "heads"), dim=_pos_int(problems, w, m, "dim"),
                        vdim=_pos_int(problems, w, m, "vdim") if "vdim" in m else _pos_int(problems, w, m, "dim"),
                        gate_cap=_number(problems, w, m, "gate_cap"))


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
class FisesunConfig:
    vocab: int
    width: int
    embedding_scale: float
    eps: float
    logit_softcap: float
    layers: Tuple[FisesunLayer, ...]

    @classmethod
    def from_dict(cls, raw: dict) -> "FisesunConfig":
        problems = []
        vocab, width = _pos_int(problems, "config", raw, "vocab"), _pos_int(problems, "config", raw, "width")
        emb = raw.get("embedding")
        scale = _number(problems, "embedding", emb, "scale", positive=False) if isinstance(emb, dict) and "scale" in emb else 1.0
        eps = _number(problems, "norm", raw.get("norm"), "eps")
        cap = _number(problems, "config", raw, "logit_softcap", positive=False) if raw.get("logit_softcap") is not None else 0.0
        if cap < 0:
            problems.append("config.logit_softcap must not be negative")
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
                layers.append(FisesunLayer(kind, _attention(problems, where + ".mixer", mixer), ff))
            elif kind == "mlstm":
                layers.append(FisesunLayer(kind, _memory(problems, where + ".mixer", mixer), ff))
            else:
                problems.append(f"{where}.type {kind!r} is not supported ({' | '.join(MIXERS)})")
        # layers that blend their values with the first such layer's need values of that layer's size
        mixing = [(i, l.mixer) for i, l in enumerate(layers) if l.type == "attention" and l.mixer.v_mix]
        for i, m in mixing[1:]:
            first = mixing[0][1]
            if (m.kv_heads, m.vdim) != (first.kv_heads, first.vdim):
                problems.append(f"layers[{i}].mixer: v_mix needs the values of layers[{mixing[0][0]}] ({first.kv_heads} x {first.vdim}), "
                                f"this layer has {m.kv_heads} x {m.vdim}")
        if problems:
            raise ConfigError("config.json: " + "; ".join(problems))
        return cls(vocab=vocab, width=width, embedding_scale=scale, eps=eps, logit_softcap=cap, layers=tuple(layers))

    def to_dict(self) -> dict:
        d = {"architecture": NAME, "vocab": self.vocab, "width": self.width, "embedding": {"scale": self.embedding_scale},
             "norm": {"eps": self.eps}, "layers": [l.to_dict() for l in self.layers]}
        if self.logit_softcap:
            d["logit_softcap"] = self.logit_softcap
        return d
