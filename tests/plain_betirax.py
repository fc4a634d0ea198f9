"""A plain, slow implementation of the Betirax decoder in NumPy float64, one function per mechanism, written
from the design's equations and sharing no code with the package.  Tests compare the engine with it; it reads a
configuration as the dictionary config.json holds and tensors by their checkpoint names.

Notation: T tokens of one sequence at positions 0 .. T-1; a stored matrix W is [out, in] and "W x" is
``x @ W.T``.  A layer norms after the sum: x <- ln(alpha x + mixer(x)) * w1, then x <- ln(alpha x + ff(x)) * w2,
ln(v) = (v - mean(v)) / sqrt(var(v) + eps); the sublayers read x itself.
"""
import json
import struct

import numpy as np


# ----------------------------------------------------------------------------------- files
def read_tensors(path):
    """name -> float64 (or int64) array of a safetensors file; bfloat16 is widened exactly."""
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        blob = f.read()
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        lo, hi = info["data_offsets"]
        kind = info["dtype"]
        if kind == "BF16":
            a = (np.frombuffer(blob[lo:hi], dtype="<u2").astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        elif kind == "F32":
            a = np.frombuffer(blob[lo:hi], dtype="<f4").astype(np.float64)
        elif kind == "I32":
            a = np.frombuffer(blob[lo:hi], dtype="<i4").astype(np.int64)
        else:
            raise ValueError(f"{name}: dtype {kind}")
        out[name] = a.reshape(info["shape"])
    return out


# ------------------------------------------------------------------------------ elementwise
def logistic(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * logistic(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (z + 0.044715 * z ** 3)))


def rms(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def layer_norm(x, weight, eps):
    """(x - mean) / sqrt(mean of squared deviations + eps) * weight; no bias."""
    c = x - np.mean(x, axis=-1, keepdims=True)
    return c / np.sqrt(np.mean(c * c, axis=-1, keepdims=True) + eps) * weight


def softmax(z):
    z = z - np.max(z, axis=-1, keepdims=True)
    e = np.exp(z)
    return e / np.sum(e, axis=-1, keepdims=True)


# ---------------------------------------------------------------------------------- rotation
def ramp_frequencies(dims, base, scaling=None):
    """-> (frequencies of the dims/2 pairs, factor on cos and sin).  Plain: f_i = base^(-2i/dims), factor 1.  With
    scaling {factor s, original L, fast, slow}: pair(t) = dims ln(L / (2 pi t)) / (2 ln base); lo = max(floor(pair(fast)), 0),
    hi = min(ceil(pair(slow)), dims - 1); r_i = clip((i - lo) / max(hi - lo, 0.001), 0, 1); the pair turns at
    f_i / s * r_i + f_i (1 - r_i), and cos and sin grow by 0.1 ln s + 1."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = float(base) ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    s, L = float(scaling["factor"]), float(scaling["original"])

    def pair(turns):
        return dims * np.log(L / (2.0 * np.pi * turns)) / (2.0 * np.log(base))

    lo = max(np.floor(pair(float(scaling["fast"]))), 0.0)
    hi = min(np.ceil(pair(float(scaling["slow"]))), dims - 1.0)
    r = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / s * r + f * (1.0 - r), 0.1 * np.log(s) + 1.0


def rotate_halves(x, positions, dims, freqs, factor=1.0):
    """x [T, ..., n]: entry i of the first ``dims`` is paired with entry i + dims/2 and the pair turned by position * f_i;
    cos and sin carry ``factor``.  The other entries pass."""
    out = np.array(x, dtype=np.float64, copy=True)
    half = dims // 2
    a = np.asarray(positions, dtype=np.float64)[:, None] * freqs[None, :]
    shape = (len(positions),) + (1,) * (x.ndim - 2) + (half,)
    c, s = (np.cos(a) * factor).reshape(shape), (np.sin(a) * factor).reshape(shape)
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


# --------------------------------------------------------------------------------- attention
def distance_slopes(heads):
    """slope of head h = 2^(-8 (h + 1) / heads)."""
    return 2.0 ** (-8.0 * (np.arange(heads) + 1.0) / heads)


def query_temperature(positions, coef, every):
    """1 + coef * ln(floor((p + 1) / every) + 1)."""
    p = np.asarray(positions, dtype=np.int64)
    return 1.0 + coef * np.log((p + 1) // every + 1.0)


def softmax_attention(q, k, v, scale, qpos, kpos, window=0, slopes=None):
    """q [Tq, H, d], k [Tk, G, d], v [Tk, G, dv]; head h reads key/value head h // (H / G).  A query at position i sees
    the keys at j <= i, with a window only those with i - j < window.  score = (q . k) * scale - slope_h (i - j)."""
    Tq, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((Tq, H, v.shape[2]))
    qpos, kpos = np.asarray(qpos), np.asarray(kpos)
    dist = qpos[:, None] - kpos[None, :]
    seen = dist >= 0
    if window:
        seen &= dist < window
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h, :] @ k[:, g, :].T) * scale
        if slopes is not None:
            s = s - slopes[h] * dist
        s = np.where(seen, s, -np.inf)
        out[:, h, :] = softmax(s) @ v[:, g, :]
    return out


def window_attention(h, w, pre, m, eps, positions=None):
    """The mixer 'attention': biased q and k projections, the values are the keys as projected; q and k normed per head
    with one weight of the head's size; q times a temperature of its position; a distance bias and a sliding window;
    the heads' outputs times sigmoid(W_g h) element by element; biased output projection."""
    T = h.shape[0]
    positions = np.arange(T) if positions is None else positions
    H, G, d = m["heads"], m.get("kv_heads", m["heads"]), m["dim"]
    q = (h @ w[pre + "q"].T + w[pre + "q.b"]).reshape(T, H, d)
    k = (h @ w[pre + "k"].T + w[pre + "k.b"]).reshape(T, G, d)
    v = k
    q = rms(q, eps) * w[pre + "q.norm"]
    k = rms(k, eps) * w[pre + "k.norm"]
    temp = m.get("q_temp")
    if temp:
        q = q * query_temperature(positions, temp["coef"], temp["every"])[:, None, None]
    window = (m.get("mask") or {}).get("size", 0)
    o = softmax_attention(q, k, v, m["scale"], positions, positions, window, distance_slopes(H)).reshape(T, -1)
    o = o * logistic(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T + w[pre + "o.b"]


def latent_kv(h, w, pre, m, eps, positions):
    """-> (latent c [T, kv_rank], the rotated key part shared by all heads [T, rot_dim]): what a request keeps."""
    r, rd = m["kv_rank"], m.get("rot_dim", 0)
    dkv = h @ w[pre + "dkv"].T
    c = rms(dkv[:, :r], eps) * w[pre + "dkv.norm"]
    rot = m.get("rot") or {}
    dims = rot.get("dims", rd)
    freqs, factor = ramp_frequencies(dims, rot.get("base", 10000.0), rot.get("scaling")) if dims else (np.zeros(0), 1.0)
    kr = rotate_halves(dkv[:, r:r + rd], positions, dims, freqs, factor) if dims else dkv[:, r:r + rd]
    return c, kr


def latent_attention(h, w, pre, m, eps, kv=None, positions=None):
    """The mixer 'latent_attention'.  ``kv``: another layer's (c, rotated key part), for a layer without W_dkv."""
    T = h.shape[0]
    positions = np.arange(T) if positions is None else positions
    H, d, rd, dv = m["heads"], m["dim"], m.get("rot_dim", 0), m.get("vdim", m["dim"])
    cq = rms(h @ w[pre + "dq"].T, eps) * w[pre + "dq.norm"]
    q = (cq @ w[pre + "uq"].T).reshape(T, H, d + rd)
    c, kr = latent_kv(h, w, pre, m, eps, positions) if kv is None else kv
    rot = m.get("rot") or {}
    dims = rot.get("dims", rd)
    if dims:
        freqs, factor = ramp_frequencies(dims, rot.get("base", 10000.0), rot.get("scaling"))
        q = np.concatenate([q[..., :d], rotate_halves(q[..., d:], positions, dims, freqs, factor)], axis=-1)
    ku = (c @ w[pre + "uk"].T).reshape(T, H, d)
    v = (c @ w[pre + "uv"].T).reshape(T, H, dv)
    k = np.concatenate([ku, np.broadcast_to(kr[:, None, :], (T, H, rd))], axis=-1)
    o = softmax_attention(q, k, v, m["scale"], positions, positions).reshape(T, -1)
    o = o * logistic(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T, (c, kr)


# ------------------------------------------------------------------------------ feed-forward
def dense_ff(h, w, pre):
    return gelu_tanh(h @ w[pre + "up"].T) @ w[pre + "down"].T


def gated_expert(h, w, pre):
    return (silu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def choose_experts(logits, top):
    """-> (indices [T, top] of the largest logits, their weights: the softmax over the chosen logits only)."""
    order = np.argsort(-logits, axis=-1, kind="stable")[:, :top]
    return order, softmax(np.take_along_axis(logits, order, axis=-1))


def mixture(h, w, pre, mlp):
    z = h @ w[pre + "router"].T
    chosen, weight = choose_experts(z, mlp["router"]["top"])
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t], weight[t]):
            out[t] += a * gated_expert(h[t:t + 1], w, f"{pre}e{e}.")[0]
    if mlp.get("shared"):
        out = out + gated_expert(h, w, pre + "shared.")
    return out


def feed_forward(h, w, pre, mlp):
    if mlp["kind"] == "dense":
        return dense_ff(h, w, pre)
    if mlp["kind"] == "moe":
        return mixture(h, w, pre, mlp)
    raise ValueError(mlp["kind"])


# ------------------------------------------------------------------------------------ model
def forward(raw, w, tokens, trace=None):
    """Logits [T, vocab] of one sequence.  ``trace``: a list that receives the stream after every layer."""
    eps, alpha = raw["norm"]["eps"], raw.get("postln_alpha", 1.0)
    tokens = np.asarray(tokens)
    x = w["embed"][tokens] * (raw.get("embedding") or {}).get("scale", 1.0)
    kept = {}
    for i, layer in enumerate(raw["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        if layer["type"] == "attention":
            y = window_attention(x, w, p + "mix.", m, eps)
        elif layer["type"] == "latent_attention":
            src = m.get("kv_from")
            y, kept[i] = latent_attention(x, w, p + "mix.", m, eps, kv=None if src is None else kept[src])
        else:
            raise ValueError(layer["type"])
        x = layer_norm(alpha * x + y, w[p + "norm1"], eps)
        if layer.get("mlp"):
            x = layer_norm(alpha * x + feed_forward(x, w, p + "mlp.", layer["mlp"]), w[p + "norm2"], eps)
        if trace is not None:
            trace.append(x.copy())
    return layer_norm(x, w["final.norm"], eps) @ w["embed"].T
