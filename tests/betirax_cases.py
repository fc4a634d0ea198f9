"""Small Betirax configurations with random weights for the tests, none of them of a served model's sizes.  They differ
from one another in every size and constant; between them they cover each mixer first and last, a layer without a
feed-forward, dense and routed feed-forwards with and without a shared expert, expert sizes that are and are not
multiples of 16, one expert, as many experts a token as there are, one head, as many KV heads as query heads and one
for all, a rotated key part that is absent, partly and wholly rotated, with and without rescaling, latent sizes that the
matrix-core kernels take and sizes that they refuse, windows of one token, shorter and longer than a page and none,
query temperatures whose steps are shorter and longer than a page and none, a stream factor of one (left out of the
file) and others, and layers that read an earlier layer's pages right after it and several layers later, two of them the
same layer's, and sizes of which none is a multiple of 8.
"""
import numpy as np
import torch


def _attention(heads, kv, dim, scale, window=0, temp=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    if temp:
        m["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return "attention", m


def _latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, dims=None, base=10000.0, scaling=None, kv_from=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale}
    if rot_dim:
        m["rot_dim"] = rot_dim
        m["rot"] = {"dims": rot_dim if dims is None else dims, "base": base}
        if scaling:
            m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    if kv_from is not None:
        m["kv_from"] = kv_from
    return "latent_attention", m


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, ff, shared=0):
    d = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        d["shared"] = {"ff": shared}
    return d


def _layer(mixer, mlp=None):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


_ROT_P = dict(dims=4, base=100.0, scaling=(3.0, 40, 4.0, 1.0))
_ROT_Q = dict(dims=32, base=5000.0, scaling=(8.0, 256, 16.0, 2.0))
_ROT_T = dict(dims=12, base=30000.0, scaling=(6.0, 512, 20.0, 1.5))
CONFIGS = {
    # a latent attention first whose pages the third layer reads; odd head sizes off the multiples of 8; a layer without a
    # feed-forward; expert sizes off the multiples of 16; temperature steps shorter than a page
    "P": {"architecture": "Betirax", "vocab": 97, "width": 48, "embedding": {"scale": 3.0}, "norm": {"eps": 1e-5}, "postln_alpha": 1.7,
          "layers": [_layer(_latent(3, 8, 4, 12, 20, 24, 0.3, **_ROT_P), _moe(5, 3, 20, shared=24)),
                     _layer(_attention(4, 2, 16, 0.3, window=20, temp=(0.3, 5)), _dense(40)),
                     _layer(_latent(2, 12, 4, 8, 20, 10, 0.25, kv_from=0, **_ROT_P)),
                     _layer(_attention(6, 2, 8, 0.4, window=7, temp=(0.5, 16)), _moe(3, 1, 7))]},
    # sizes of the matrix-core kernels (keys 64; cached latent keys of 128 with values of 64), a rotated part of which half is
    # rotated, rescaled through every band, a window longer than a page, an attention that sees everything and has no
    # temperature, the reading layer two layers after the one that writes
    "Q": {"architecture": "Betirax", "vocab": 130, "width": 64, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6}, "postln_alpha": 0.8,
          "layers": [_layer(_attention(2, 1, 64, 0.11, window=33, temp=(0.4, 32)), _moe(4, 2, 32, shared=16)),
                     _layer(_latent(4, 32, 64, 40, 64, 48, 0.13, **_ROT_Q), _dense(96)),
                     _layer(_attention(4, 4, 32, 0.2), _dense(72)),
                     _layer(_latent(2, 16, 64, 24, 64, 32, 0.2, kv_from=1, **_ROT_Q), _moe(2, 2, 48, shared=32))]},
    # one head, one expert, as many experts a token as there are, no rotated key part, no embedding factor and no stream
    # factor in the file, a window of one token, pages of 8
    "R": {"architecture": "Betirax", "vocab": 64, "width": 32, "norm": {"eps": 3e-6},
          "layers": [_layer(_attention(1, 1, 10, 0.35, window=1), _moe(1, 1, 12)),
                     _layer(_latent(1, 6, 0, 10, 7, 5, 0.4), _moe(2, 2, 8, shared=8)),
                     _layer(_attention(3, 3, 16, 0.3, window=40, temp=(1.0, 1)), None),
                     _layer(_latent(2, 16, 0, 8, 7, 9, 0.3, kv_from=1), _dense(24)),
                     _layer(_latent(3, 4, 0, 12, 7, 11, 0.5, kv_from=1), _moe(3, 2, 16))]},
    # pages of 32, 128-wide heads with three query heads per KV head, a long window, a wholly rotated key part without rescaling
    "S": {"architecture": "Betirax", "vocab": 200, "width": 96, "embedding": {"scale": 0.5}, "norm": {"eps": 1e-5}, "postln_alpha": 3.0,
          "layers": [_layer(_attention(6, 2, 128, 0.09, window=70, temp=(0.25, 64)), _moe(8, 3, 48, shared=64)),
                     _layer(_latent(2, 48, 16, 24, 40, 56, 0.15, base=25000.0), _dense(64))]},
    # nothing a multiple of 8: a width of 100, an odd vocabulary, five heads of 20, latents of 36 beside a rotated part of 12
    "T": {"architecture": "Betirax", "vocab": 451, "width": 100, "embedding": {"scale": 7.0}, "norm": {"eps": 1e-5}, "postln_alpha": 2.2,
          "layers": [_layer(_attention(5, 5, 20, 0.2, window=23, temp=(0.7, 30)), _dense(150)),
                     _layer(_latent(3, 20, 12, 28, 36, 44, 0.17, **_ROT_T), _moe(6, 3, 50, shared=70)),
                     _layer(_attention(6, 3, 12, 0.25, window=64, temp=(0.2, 7)), _moe(3, 2, 33)),
                     _layer(_latent(5, 10, 12, 14, 36, 21, 0.2, kv_from=1, **_ROT_T), _dense(77))]},
}
BLOCK_SIZE = {"P": 16, "Q": 16, "R": 8, "S": 32, "T": 16}


def tensors_for(raw, seed, sharpen=3.0):
    """Checkpoint names -> tensors (float32 on the bfloat16 grid, so that both storage modes hold the same numbers).
    Matrices N(0, 1 / fan-in); the projections that make queries and keys are scaled up so that attention is sharp
    enough for a wrong or missing key to show; norm weights 1 + 0.1 N; biases 0.3 N."""
    from kvcm_amd.config.betirax_config import BetiraxConfig
    from kvcm_amd.weights.random_init import expected_tensors
    cfg = BetiraxConfig.from_dict(raw)
    rng = np.random.default_rng(seed)
    out = {}
    for name, (shape, role) in sorted(expected_tensors("Betirax", cfg).items()):
        leaf = name.split(".", 1)[1] if name[0] == "l" and name[1].isdigit() else name
        if len(shape) == 2:
            a = rng.normal(size=shape) / np.sqrt(shape[1])
        else:
            a = rng.normal(size=shape) * 0.3
        if role == "vector":
            a = 1.0 + 0.1 * rng.normal(size=shape)
        elif leaf in ("mix.q", "mix.k", "mix.uq", "mix.dkv"):
            a = a * sharpen
        elif name == "embed":
            a = rng.normal(size=shape) * 0.5
        out[name] = torch.from_numpy(np.asarray(a, dtype=np.float64)).to(torch.bfloat16).to(torch.float32)
    return cfg, out


def as_numpy(tensors):
    return {k: v.double().numpy() for k, v in tensors.items()}


def requests_for(raw, lengths, seed):
    rng = np.random.default_rng(seed)
    return {f"r{i}": rng.integers(0, raw["vocab"], size=n).tolist() for i, n in enumerate(lengths)}


def with_every_expert_chosen(raw):
    """The configuration with ``top`` raised to the number of experts in every routed layer: nothing is chosen, so no choice
    hangs on rounding.  (Where 8-bit rounding decides between two experts of nearly equal logits, the other expert's output
    enters that token's keys and stays in the pages for every later token: a test of long decoding should not rest on it.)"""
    import copy
    out = copy.deepcopy(raw)
    for layer in out["layers"]:
        if layer["mlp"] and layer["mlp"]["kind"] == "moe":
            layer["mlp"]["router"]["top"] = layer["mlp"]["router"]["experts"]
    return out
