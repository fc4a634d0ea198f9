"""Small Fisesun configurations with random weights for the tests, none of them of a served model's sizes.  They differ
from one another in every size and constant; between them they cover each mixer first and last, a layer without a
feed-forward, dense and routed feed-forwards with and without a shared expert, expert sizes that are and are not
multiples of 16, one expert, as many experts a token as there are, one head, as many KV heads as query heads and one
for all, a rotation of no, some and all entries of a head, with and without rescaling, values wider and narrower than
keys, head shapes that the matrix-core kernels take and shapes that they refuse, windows shorter and longer than a
page with none, few and many kept first tokens (more than a page, more than the window), no window at all, scores
with and without a cap, no, one, and several layers that blend values, logits with and without a cap.
"""
import numpy as np
import torch


def _attention(heads, kv, dim, vdim, scale, cap=None, window=0, keep=0, rot=0, base=10000.0, scaling=None, v_mix=False):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "v_mix": v_mix}
    if cap:
        m["softcap"] = cap
    if window:
        m["mask"] = {"size": window, "keep_first": keep}
    if rot:
        m["rot"] = {"dims": rot, "base": base}
        if scaling:
            m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return "attention", m


def _memory(heads, dim, vdim, cap):
    return "mlstm", {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, ff, shared=0):
    d = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        d["shared"] = {"ff": shared}
    return d


def _layer(mixer, mlp=None):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


CONFIGS = {
    # a matrix memory first and without a feed-forward; odd head sizes; three blending layers of which the middle one
    # sees everything; kept tokens within the first page; expert sizes off the multiples of 16
    "P": {"architecture": "Fisesun", "vocab": 97, "width": 48, "embedding": {"scale": 3.0}, "norm": {"eps": 1e-5}, "logit_softcap": 9.0,
          "layers": [_layer(_memory(3, 8, 12, 6.0)),
                     _layer(_attention(4, 2, 16, 24, 0.3, cap=5.0, window=20, keep=3, rot=8, base=100.0, scaling=(3.0, 1.0, 4.0, 40), v_mix=True), _moe(5, 3, 20, shared=24)),
                     _layer(_attention(2, 2, 12, 24, 0.25, cap=50.0, rot=12, base=50.0, v_mix=True), _dense(40)),
                     _layer(_attention(6, 2, 8, 24, 0.4, window=7, keep=0, v_mix=True), _moe(3, 1, 7))]},
    # head shapes of the matrix-core kernels (keys 64, values 40 and 64), a rotation of the whole head with rescaling that
    # touches every band, more kept tokens than a page holds and more than the window, a window longer than a page
    "Q": {"architecture": "Fisesun", "vocab": 130, "width": 64, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6}, "logit_softcap": 30.0,
          "layers": [_layer(_attention(2, 1, 64, 40, 0.11, cap=20.0, window=33, keep=21, rot=64, base=5000.0, scaling=(8.0, 1.0, 4.0, 256), v_mix=True), _moe(4, 2, 32, shared=16)),
                     _layer(_memory(2, 32, 16, 8.0), _moe(6, 2, 16)),
                     _layer(_attention(4, 1, 64, 40, 0.13, cap=20.0, window=10, keep=40, rot=32, base=300.0, v_mix=True), _dense(96)),
                     _layer(_attention(2, 2, 32, 64, 0.2, window=40, keep=5), _moe(2, 2, 48, shared=32))]},
    # one head, one expert, as many experts a token as there are, no rotation, no cap anywhere, no logit cap and no
    # embedding factor in the file, a single blending layer (nobody to blend with), a window of one token that keeps two
    "R": {"architecture": "Fisesun", "vocab": 64, "width": 32, "norm": {"eps": 3e-6},
          "layers": [_layer(_attention(1, 1, 10, 6, 0.35, window=1, keep=2, v_mix=True), _moe(1, 1, 12)),
                     _layer(_memory(1, 24, 40, 15.0), _moe(2, 2, 8, shared=8)),
                     _layer(_attention(3, 3, 16, 16, 0.3), None),
                     _layer(_memory(2, 16, 8, 4.0), _dense(24))]},
    # pages of 32, 128-wide heads with a partial rescaled rotation, three query heads per KV head, a long window with
    # kept tokens that end inside the second page
    "S": {"architecture": "Fisesun", "vocab": 200, "width": 96, "embedding": {"scale": 0.5}, "norm": {"eps": 1e-5}, "logit_softcap": 15.0,
          "layers": [_layer(_attention(6, 2, 128, 128, 0.09, cap=30.0, window=70, keep=37, rot=32, base=25000.0, scaling=(4.0, 2.0, 16.0, 64)), _moe(8, 3, 48, shared=64)),
                     _layer(_memory(2, 48, 24, 12.0), _dense(64))]},
}
BLOCK_SIZE = {"P": 16, "Q": 16, "R": 8, "S": 32}


def tensors_for(raw, seed, sharpen=3.0):
    """Checkpoint names -> tensors (float32 on the bfloat16 grid, so that both storage modes hold the same numbers; the
    experts' tables int32).  Matrices N(0, 1 / fan-in); the q and k projections are scaled up so that attention is sharp
    enough for a wrong or missing key to show; norm weights 1 + 0.1 N; the blending factors between 0.2 and 0.8; forget
    gates biased towards keeping; every row of a table names distinct experts."""
    from kvcm_amd.config.fisesun_config import FisesunConfig
    from kvcm_amd.weights.random_init import expected_tensors
    cfg = FisesunConfig.from_dict(raw)
    rng = np.random.default_rng(seed)
    out = {}
    for name, (shape, role) in sorted(expected_tensors("Fisesun", cfg).items()):
        leaf = name.split(".", 1)[1] if name[0] == "l" and name[1].isdigit() else name
        if role == "index":
            experts = raw["layers"][int(name[1:name.index(".")])]["mlp"]["router"]["experts"]
            out[name] = torch.from_numpy(np.stack([rng.permutation(experts)[:shape[1]] for _ in range(shape[0])]).astype(np.int32))
            continue
        if len(shape) == 2:
            a = rng.normal(size=shape) / np.sqrt(shape[1])
        else:
            a = rng.normal(size=shape) * 0.5
        if leaf == "mix.vmix":
            a = rng.uniform(0.2, 0.8, size=shape)
        elif leaf.startswith("norm") or leaf in ("mix.norm", "mix.q.norm", "mix.k.norm") or name == "final.norm":
            a = 1.0 + 0.1 * rng.normal(size=shape)
        elif leaf in ("mix.q", "mix.k"):
            a = a * sharpen
        elif leaf == "mix.f.b":
            a = rng.uniform(1.0, 4.0, size=shape)
        elif leaf == "mix.i.b":
            a = rng.normal(size=shape)
        elif leaf in ("mix.i", "mix.f"):
            a = a * 2.0
        elif name == "embed":
            a = rng.normal(size=shape)
        out[name] = torch.from_numpy(np.asarray(a, dtype=np.float64)).to(torch.bfloat16).to(torch.float32)
    return cfg, out


def as_numpy(tensors):
    return {k: (v.double().numpy() if v.is_floating_point() else v.numpy().astype(np.int64)) for k, v in tensors.items()}


def requests_for(raw, lengths, seed):
    rng = np.random.default_rng(seed)
    return {f"r{i}": rng.integers(0, raw["vocab"], size=n).tolist() for i, n in enumerate(lengths)}
