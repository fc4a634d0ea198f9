"""A plain, slow implementation of the Fisesun decoder in NumPy float64, one function per mechanism, written
from the design's equations and sharing no code with the package.  Tests compare the engine with it; it reads a
configuration as the dictionary config.json holds and tensors by their checkpoint names.

Notation: T tokens of one sequence at positions 0 .. T-1; a stored matrix W is [out, in] and "W x" is
``x @ W.T``; rms(x) = x / sqrt(mean(x^2) + eps).  A layer is x <- x + rms(mixer(x)) * w1, then
x <- x + rms(ff(x)) * w2 (no norm on the way in: the sublayers read x itself).
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


def log_logistic(z):
    return -np.logaddexp(0.0, -z)


def silu(z):
    return z * logistic(z)


def rms(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def tanh_cap(z, cap):
    return cap * np.tanh(z / cap)


# ---------------------------------------------------------------------------------- rotation
def pair_frequencies(dims, base, scaling=None):
    """Frequencies of the dims/2 pairs.  Plain: f_i = base^(-2i/dims).  With scaling (factor, low, high, original):
    a pair whose wavelength 2 pi / f is shorter than original/high keeps f; longer than original/low it turns at
    f / factor; between the two it is blended, (1 - s) f / factor + s f with s = (original/wavelength - low) / (high - low)."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = float(base) ** (-2.0 * i / dims)
    if not scaling:
        return f
    factor, low, high, L = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    out = np.empty_like(f)
    for n, fi in enumerate(f):
        wavelength = 2.0 * np.pi / fi
        if wavelength < L / high:
            out[n] = fi
        elif wavelength > L / low:
            out[n] = fi / factor
        else:
            s = (L / wavelength - low) / (high - low)
            out[n] = (1.0 - s) * fi / factor + s * fi
    return out


def rotate_halves(x, positions, dims, freqs):
    """x [T, heads, dim]: entry i < dims/2 and entry i + dims/2 are one pair (u, v), turned by a = position * freqs[i]
    into (u cos a - v sin a, v cos a + u sin a); entries from ``dims`` on pass."""
    if not dims:
        return x.copy()
    half = dims // 2
    a = np.asarray(positions, dtype=np.float64)[:, None] * freqs[None, :]
    c, s = np.cos(a)[:, None, :], np.sin(a)[:, None, :]
    out = x.copy()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


# --------------------------------------------------------------------------------- attention
def sees(qpos, kpos, window, keep_first):
    """[Q, K] bool: the query at position i sees the key at j when j <= i and (i - j < window or j < keep_first);
    window 0: every earlier token."""
    i, j = np.asarray(qpos)[:, None], np.asarray(kpos)[None, :]
    ok = j <= i
    if window:
        ok &= (i - j < window) | (j < keep_first)
    return ok


def capped_softmax_attention(q, k, v, scale, cap, mask):
    """q [Q, H, d], k [K, G, d], v [K, G, dv], mask [Q, K] -> [Q, H, dv]; query head h reads key head h // (H / G);
    score = cap tanh((q . k) scale / cap) (cap 0 or None: none), one ordinary softmax over the visible keys."""
    Q, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((Q, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        z = (q[:, h] @ k[:, g].T) * scale
        if cap:
            z = tanh_cap(z, cap)
        z = np.where(mask, z, -np.inf)
        e = np.exp(z - z.max(axis=-1, keepdims=True))
        out[:, h] = (e / e.sum(axis=-1, keepdims=True)) @ v[:, g]
    return out


def attention_qkv(h, w, pre, m, eps, positions, v_first=None):
    """q, k (normed over the whole projection, then rotated) and v (mixed with ``v_first`` when given) of the rows h."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    q = rms(h @ w[pre + "q"].T, eps) * w[pre + "q.norm"]
    k = rms(h @ w[pre + "k"].T, eps) * w[pre + "k.norm"]
    v = h @ w[pre + "v"].T
    if v_first is not None:
        lam = float(w[pre + "vmix"])
        v = (1.0 - lam) * v + lam * v_first
    q, k = q.reshape(T, H, d), k.reshape(T, G, d)
    rot = m.get("rot") or {}
    dims = rot.get("dims", 0)
    if dims:
        f = pair_frequencies(dims, rot.get("base", 10000.0), rot.get("scaling"))
        q, k = rotate_halves(q, positions, dims, f), rotate_halves(k, positions, dims, f)
    return q, k, v.reshape(T, G, dv)


def attention(h, w, pre, m, eps, v_first=None):
    """The whole mixer on one sequence from position 0.  -> (output [T, width], the values before mixing [T, G*dv])."""
    T = h.shape[0]
    pos = np.arange(T)
    q, k, v = attention_qkv(h, w, pre, m, eps, pos, v_first)
    mask_cfg = m.get("mask") or {}
    mask = sees(pos, pos, mask_cfg.get("size", 0), mask_cfg.get("keep_first", 0))
    o = capped_softmax_attention(q, k, v, m["scale"], m.get("softcap"), mask)
    return o.reshape(T, -1) @ w[pre + "o"].T, h @ w[pre + "v"].T


# --------------------------------------------------------------------------- matrix memory
def memory_walk(q, k, v, log_in, log_keep, state=None):
    """One head, token by token.  q, k [T, d] (q already scaled), v [T, dv], log_in, log_keep [T].
    state = (S [d, dv], n [d], m) or None for zeros (m too starts at 0).  Returns (o [T, dv], state)."""
    T, d = k.shape
    S, n, m = (np.zeros((d, v.shape[1])), np.zeros(d), 0.0) if state is None else state
    out = np.zeros((T, v.shape[1]))
    for t in range(T):
        m_next = max(log_keep[t] + m, log_in[t])
        keep, take = np.exp(log_keep[t] + m - m_next), np.exp(log_in[t] - m_next)
        S = keep * S + take * np.outer(k[t], v[t])
        n = keep * n + take * k[t]
        m = m_next
        out[t] = (S.T @ q[t]) / (max(abs(n @ q[t]), np.exp(-m)) + 1e-6)
    return out, (S, n, m)


def mlstm(h, w, pre, m, eps):
    T = h.shape[0]
    H, d, dv, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    q = (h @ w[pre + "q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ w[pre + "k"].T).reshape(T, H, d)
    v = (h @ w[pre + "v"].T).reshape(T, H, dv)
    log_in = tanh_cap(h @ w[pre + "i"].T + w[pre + "i.b"], cap)
    log_keep = log_logistic(tanh_cap(h @ w[pre + "f"].T + w[pre + "f.b"], cap))
    o = np.zeros((T, H, dv))
    for a in range(H):
        o[:, a], _ = memory_walk(q[:, a], k[:, a], v[:, a], log_in[:, a], log_keep[:, a])
    o = rms(o, eps).reshape(T, H * dv) * w[pre + "norm"]
    return (o * logistic(h @ w[pre + "g"].T)) @ w[pre + "o"].T


# ------------------------------------------------------------------------------ feed-forward
def gated_ff(h, w, pre):
    return (silu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def table_mixture(h, tokens, w, pre, mlp):
    """Every token id has its experts in a table [vocab, top]; each counts 1/top; a shared expert is added."""
    top = mlp["router"]["top"]
    table = w[pre + "table"]
    out = np.zeros((h.shape[0], w[pre + "e0.down"].shape[0]))
    for t, tok in enumerate(tokens):
        for e in table[int(tok)][:top]:
            out[t] += gated_ff(h[t:t + 1], w, pre + f"e{int(e)}.")[0] / top
    if mlp.get("shared"):
        out += gated_ff(h, w, pre + "shared.")
    return out


def feed_forward(h, tokens, w, pre, mlp):
    if mlp["kind"] == "dense":
        return gated_ff(h, w, pre)
    if mlp["kind"] == "moe":
        return table_mixture(h, tokens, w, pre, mlp)
    raise ValueError(mlp["kind"])


# ----------------------------------------------------------------------------------- model
def forward(raw, w, tokens, trace=None):
    """Logits [T, vocab] of one sequence; ``trace``: a list that receives the stream after every layer."""
    eps = raw["norm"]["eps"]
    tokens = np.asarray(tokens)
    x = w["embed"][tokens] * raw.get("embedding", {}).get("scale", 1.0)
    v_first = None
    for i, L in enumerate(raw["layers"]):
        p, m = f"l{i}.", L["mixer"]
        if L["type"] == "attention":
            mixes = bool(m.get("v_mix"))
            y, v_own = attention(x, w, p + "mix.", m, eps, v_first if mixes else None)
            if mixes and v_first is None:
                v_first = v_own
        elif L["type"] == "mlstm":
            y = mlstm(x, w, p + "mix.", m, eps)
        else:
            raise ValueError(L["type"])
        x = x + rms(y, eps) * w[p + "norm1"]
        if L.get("mlp"):
            x = x + rms(feed_forward(x, tokens, w, p + "mlp.", L["mlp"]), eps) * w[p + "norm2"]
        if trace is not None:
            trace.append(x.copy())
    z = (rms(x, eps) * w["final.norm"]) @ w["head"].T
    cap = raw.get("logit_softcap")
    return tanh_cap(z, cap) if cap else z
