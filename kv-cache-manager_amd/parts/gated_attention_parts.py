"""Three attentions over the paged cache that share the kernels of the window attention (ops.attention_window_pool,
its matrix-core form for runs of positions, ops.rotate_store): grouped-query attention with a half-split rotation on
part of each head, rescaled pair by pair for longer contexts, and one sigmoid gate per head; a latent attention
that caches one small normed vector per token from which every head's keys and values are made; and a grouped-query
attention with queries and keys normed over their whole projection, capped scores, a window that keeps a sequence's
first tokens in sight, and values blended with an earlier layer's.  Every size, constant and tensor name is a parameter.
"""
import math

import torch

from ..registry import MIXERS, POSITIONS
from . import paged_attention
from .base import KVCacheNeed, Mixer, ParamSpec, PartSpec, PositionEncoding
from .chain_norm_parts import f32_params, linear32


def rescaled_frequencies(dims, base, scaling=None):
    """-> (frequencies of the dims/2 pairs as a list of Python floats, factor on cos and sin).  Plain:
    f_i = base^(-2i/dims), factor 1.  ``scaling`` = (factor s, original length L, fast, slow): with
    pair(t) = dims ln(L / (2 pi t)) / (2 ln base), lo = max(floor(pair(fast)), 0), hi = min(ceil(pair(slow)), dims - 1)
    and ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), pair i turns at f_i / s * ramp_i + f_i (1 - ramp_i), and
    cos and sin are multiplied by 0.1 ln s + 1."""
    freqs = [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return freqs, 1.0
    s, L, fast, slow = (float(v) for v in scaling)

    def pair(turns):
        return dims * math.log(L / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo, hi = max(math.floor(pair(fast)), 0), min(math.ceil(pair(slow)), dims - 1)
    out = []
    for i, f in enumerate(freqs):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / s * ramp + f * (1.0 - ramp))
    return out, 0.1 * math.log(s) + 1.0


def wavelength_scaled_frequencies(dims, base, scaling=None):
    """-> frequencies of the dims/2 pairs as a list of Python floats.  Plain: f_i = base^(-2i/dims).  ``scaling`` =
    (factor s, low, high, original length L): with the wavelength l_i = 2 pi / f_i, a pair keeps f_i where l_i < L / high,
    turns at f_i / s where l_i > L / low, and between the two at (1 - t) f_i / s + t f_i with t = (L / l_i - low) / (high - low)."""
    freqs = [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return freqs
    s, low, high, L = (float(v) for v in scaling)
    out = []
    for f in freqs:
        wavelength = 2.0 * math.pi / f
        if wavelength < L / high:
            out.append(f)
        elif wavelength > L / low:
            out.append(f / s)
        else:
            t = (L / wavelength - low) / (high - low)
            out.append((1.0 - t) * f / s + t * f)
    return out


@POSITIONS.register("rotary_halves")
class HalfSplitRotary(PositionEncoding):
    """Rotary positions on the first ``dims`` entries of every q and k head, entry i paired with entry i + dims/2,
    with frequencies that may be rescaled for longer contexts.  params: dims, base, scaling (None or four numbers),
    scaling_kind: "ramp" (default; ``rescaled_frequencies``: (factor, original, fast, slow), cos and sin grow with
    the factor) or "wavelength" (``wavelength_scaled_frequencies``: (factor, low, high, original))."""

    capturable = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.dims = params["dims"]
        kind = params.get("scaling_kind", "ramp")
        if kind not in ("ramp", "wavelength"):
            raise ValueError(f"rotary_halves {prefix!r}: scaling_kind {kind!r} is not supported (ramp | wavelength)")
        if not self.dims:
            self.freqs, self.factor = [], 1.0
        elif kind == "wavelength":
            self.freqs, self.factor = wavelength_scaled_frequencies(self.dims, params["base"], params.get("scaling")), 1.0
        else:
            self.freqs, self.factor = rescaled_frequencies(self.dims, params["base"], params.get("scaling"))
        self._device_freqs = None

    def bind(self, tensors):
        super().bind(tensors)
        if self.dims and self.ctx.device.type == "cuda":      # made once, here: a step allocates nothing
            self._device_freqs = torch.tensor(self.freqs, dtype=torch.float64, device=self.ctx.device)

    def pairs_table(self, step):
        """factor * (cos, sin) of every row's angles, float32 [rows, dims/2, 2]; made by the step's first layer that asks,
        read by the others with the same frequencies."""
        if not self.dims:
            return None
        key = ("rotary_halves", self.dims, tuple(self.freqs), self.factor)
        table = step.shared.get(key)
        if table is None:
            if self._device_freqs is None:
                self._device_freqs = torch.tensor(self.freqs, dtype=torch.float64, device=self.ctx.device)
            name = "rotary_halves_%d_%s" % (self.dims, float(sum(self.freqs)).hex())
            table = step.ws(name, (step.rows, self.dims), torch.float32)
            self.ctx.ops.rotary_freq_table(step.positions, self._device_freqs, table, self.dims, self.factor, rows=step.rows)
            step.shared[key] = table
        return table

    def apply(self, step, qkv, num_heads, num_kv_heads, head_dim, cache=None, slots=None):
        raise NotImplementedError("rotary_halves rotates inside ops.rotate_store (the mixer hands it pairs_table)")


def _pad_rows(t, multiple=16):
    """A matrix with zero rows appended up to a multiple (the few-row products take such widths)."""
    extra = -t.shape[0] % multiple
    if not extra:
        return t
    return torch.cat([t, torch.zeros(extra, t.shape[1], dtype=t.dtype, device=t.device)], 0)


def _attend(mixer, step, q, attn, kc, vc, g, nh, nkv, d, dv, scale, window, keep_first=0, softcap=0.0):
    """Keys and values of one size, no window, no cap on the scores, bfloat16: the kernels every attention over paged
    keys and values takes (parts/paged_attention.py: partitioned for single rows, tiled for runs of positions).
    Otherwise the window attention's: steps with runs of positions take its matrix-core kernel where it has the head
    shape, others one (row, head) per workgroup."""
    ops = mixer.ctx.ops
    if d == dv and window == 0 and not softcap and attn.dtype == torch.bfloat16 and d % 8 == 0 and d <= 256:
        return paged_attention.attend(step, ops, q, attn, kc, vc, g, nh, nkv, d, scale, 0)
    if step.max_run > 1 and ops.attention_window_pool_tiles_supported(d, dv, attn.dtype, kc.shape[2]):
        ops.attention_window_pool_tiles(q, attn, kc, vc, None, None, step.tables(g), step.table_stride(g), step.run_start,
                                        step.seq_start, step.seqs, step.max_run, nh, nkv, d, dv, scale, window, 0,
                                        keep_first=keep_first, softcap=softcap)
    else:
        ops.attention_window_pool(q, attn, kc, vc, None, None, step.tables(g), step.table_stride(g), step.row_seq, step.ctx_lens,
                                  nh, nkv, d, dv, scale, window, 0, rows=step.rows, keep_first=keep_first, softcap=softcap)


@MIXERS.register("gated_attention")
class GatedAttention(Mixer):
    """q, k, v and one gate logit per query head come from one fused projection without biases; q and k are rotated
    (``position``: a PartSpec, default none); query head h reads KV head h / (heads / kv_heads); score = (q . k) * scale;
    a row sees every earlier token and itself (window 0) or the last ``window``; head h's output is multiplied by
    sigmoid(gate_h) before the output projection.
    params: heads, kv_heads, dim, vdim, scale, window, position.  Tensors under the prefix: q, k, v, g, o."""

    capturable = True
    sub_part_names = ("position",)

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        p = params
        self.nh, self.nkv, self.d, self.dv = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
        if self.nkv <= 0 or self.nh % self.nkv:
            raise ValueError(f"gated_attention {prefix!r}: heads {self.nh} is not a multiple of kv_heads {self.nkv}")
        pos = p.get("position") or PartSpec("rotary_halves", {"dims": 0, "base": 10000.0})
        self.position = POSITIONS.get(pos.kind)(pos.params, prefix, ctx)
        self.gate_at = (self.nh + self.nkv) * self.d + self.nkv * self.dv

    def sub_parts(self):
        return (self.position,)

    def param_specs(self):
        H, pre = self.ctx.hidden_size, self.prefix
        sizes = (("q", self.nh * self.d), ("k", self.nkv * self.d), ("v", self.nkv * self.dv), ("g", self.nh))
        return [ParamSpec("w_proj", tuple((pre + n, (c, H)) for n, c in sizes)),
                ParamSpec("w_o", ((pre + "o", (H, self.nh * self.dv)),))]

    def bind(self, tensors):
        super().bind({**tensors, "w_proj": _pad_rows(tensors["w_proj"])})

    def cache_need(self):
        return KVCacheNeed(self.nkv, self.d, self.params.get("window", 0), value_dim=self.dv)

    def flops(self, rows, attended=0):
        return super().flops(rows) + 2.0 * attended * (self.d + self.dv) * self.nh

    def forward(self, step, h):
        ops, p, w = self.ctx.ops, self.params, self.w
        g = self.cache.group
        kc, vc = self.cache.k(self.cache_index), self.cache.v(self.cache_index)
        T = step.rows
        proj = linear32(self.ctx, step, h, w["w_proj"], "ga_proj")
        q = step.ws("ga_q", (T, self.nh * self.d))
        slots = step.slots(g) if self.cache_owner else None
        ops.rotate_store(proj, q, self.nh, self.nkv, self.d, self.dv, cos_sin=self.position.pairs_table(step),
                         rot=self.position.params["dims"], slots=slots, kcache=kc, vcache=vc, rows=T, halves=True)
        attn = step.ws("ga_attn", (T, self.nh * self.dv))
        _attend(self, step, q, attn, kc, vc, g, self.nh, self.nkv, self.d, self.dv, p["scale"], p.get("window", 0))
        ops.head_gate(attn, proj[:, self.gate_at:], self.nh, self.dv, rows=T)
        return linear32(self.ctx, step, attn, w["w_o"], "ga_out", keep_partial=True)      # the stream's next norm adds the slices


@MIXERS.register("latent_attention")
class LatentAttention(Mixer):
    """Attention without positions whose keys and values are made from one latent vector per token:
    c = n(W_dkv h) * w_norm (n: division by the root mean square, eps), k_h = W_uk,h c, v_h = W_uv,h c, q_h = W_q,h h,
    score = (q_h . k_h) * scale over the last ``window`` tokens (0: all).  Only c is cached.  The products with W_uk and
    W_uv are moved to the query's and the output's side when the weights are bound (q_h . W_uk,h c = (W_uk,h^T q_h) . c,
    and sum_j p_j W_uv,h c_j = W_uv,h sum_j p_j c_j): the step computes q' = (W_uk^T W_q) h per head, attends over the
    cached c as the one key and value head of size kv_rank, and projects with W_o W_uv.
    params: heads, dim, vdim, kv_rank, scale, window, eps.  Tensors under the prefix: q, dkv, dkv.norm, uk, uv, o."""

    capturable = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        p = params
        self.nh, self.d, self.dv, self.r = p["heads"], p["dim"], p["vdim"], p["kv_rank"]

    def param_specs(self):
        H, pre = self.ctx.hidden_size, self.prefix
        return [ParamSpec("w_q", ((pre + "q", (self.nh * self.d, H)),)),
                ParamSpec("w_dkv", ((pre + "dkv", (self.r, H)),)),
                ParamSpec("c_norm", ((pre + "dkv.norm", (self.r,)),), role="vector"),
                ParamSpec("w_uk", ((pre + "uk", (self.nh * self.d, self.r)),)),
                ParamSpec("w_uv", ((pre + "uv", (self.nh * self.dv, self.r)),)),
                ParamSpec("w_o", ((pre + "o", (H, self.nh * self.dv)),))]

    def bind(self, tensors):
        nh, d, dv, r = self.nh, self.d, self.dv, self.r
        t = tensors
        H = t["w_q"].shape[1]
        dt = t["w_q"].dtype
        # the two small products folded into their neighbours, formed in double precision and rounded once
        q_abs = torch.einsum("hdr,hdw->hrw", t["w_uk"].double().view(nh, d, r), t["w_q"].double().view(nh, d, H)).reshape(nh * r, H)
        o_abs = torch.einsum("whv,hvr->whr", t["w_o"].double().view(H, nh, dv), t["w_uv"].double().view(nh, dv, r)).reshape(H, nh * r)
        w_proj = torch.cat([q_abs.to(dt), t["w_dkv"], t["w_dkv"]], 0)      # [q' | c | c]: c goes to the pages as key and as value
        super().bind({"w_proj": _pad_rows(w_proj.contiguous()), "w_o": o_abs.to(dt).contiguous(), **f32_params({"c_norm": t["c_norm"]})})

    def cache_need(self):
        return KVCacheNeed(1, self.r, self.params.get("window", 0), value_dim=self.r)

    def flops(self, rows, attended=0):
        window = self.params.get("window", 0)
        seen = min(attended, rows * window) if window else attended      # a row sees at most its window
        return super().flops(rows) + 4.0 * seen * self.r * self.nh

    def forward(self, step, h):
        ops, p, w = self.ctx.ops, self.params, self.w
        g = self.cache.group
        kc, vc = self.cache.k(self.cache_index), self.cache.v(self.cache_index)
        T, nh, r = step.rows, self.nh, self.r
        proj = linear32(self.ctx, step, h, w["w_proj"], "la_proj")
        ops.rms_groups(proj, nh * r, r, 2, w["c_norm"], p["eps"], rows=T)
        q = step.ws("la_q", (T, nh * r))
        slots = step.slots(g) if self.cache_owner else None
        ops.rotate_store(proj, q, nh, 1, r, r, rot=0, slots=slots, kcache=kc, vcache=vc, rows=T)
        attn = step.ws("la_attn", (T, nh * r))
        _attend(self, step, q, attn, kc, vc, g, nh, 1, r, r, p["scale"], p.get("window", 0))
        return linear32(self.ctx, step, attn, w["w_o"], "la_out", keep_partial=True)


@MIXERS.register("capped_window_attention")
class CappedWindowAttention(Mixer):
    """Grouped-query attention without biases.  q and k may each be divided by the root mean square over their whole
    projection (all heads at once, before the split into heads) and multiplied by a weight of that size (``qk_norm_eps``),
    then rotated (``position``: a PartSpec, default none).  score = (q . k) * scale, capped as softcap * tanh(score /
    softcap) where ``softcap`` > 0; a row at position i sees j <= i with i - j < window or j < keep_first (window 0: every
    earlier token); an ordinary softmax.  ``value_mix``: "source" keeps the values this layer's projection made at hand
    for later layers of the step; "blend" replaces this layer's values by (1 - lambda) v + lambda v_source, v_source the
    "source" layer's values of the same token and lambda the scalar tensor ``vmix``; the blended values are what the pages
    hold.  params: heads, kv_heads, dim, vdim, scale, softcap, window, keep_first, qk_norm_eps, value_mix, position.
    Tensors under the prefix: q, k, v, o, q.norm, k.norm (with qk_norm_eps), vmix (with value_mix)."""

    capturable = True
    sub_part_names = ("position",)

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        p = params
        self.nh, self.nkv, self.d, self.dv = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
        if self.nkv <= 0 or self.nh % self.nkv:
            raise ValueError(f"capped_window_attention {prefix!r}: heads {self.nh} is not a multiple of kv_heads {self.nkv}")
        self.value_mix = p.get("value_mix")
        if self.value_mix not in (None, "source", "blend"):
            raise ValueError(f"capped_window_attention {prefix!r}: value_mix {self.value_mix!r} is not supported (source | blend)")
        self.window = p.get("window", 0)
        self.keep_first = p.get("keep_first", 0) if self.window else 0
        pos = p.get("position") or PartSpec("rotary_halves", {"dims": 0, "base": 10000.0})
        self.position = POSITIONS.get(pos.kind)(pos.params, prefix, ctx)
        self.mix = 0.0

    def sub_parts(self):
        return (self.position,)

    def param_specs(self):
        H, pre = self.ctx.hidden_size, self.prefix
        sizes = (("q", self.nh * self.d), ("k", self.nkv * self.d), ("v", self.nkv * self.dv))
        specs = [ParamSpec("w_proj", tuple((pre + n, (c, H)) for n, c in sizes)),
                 ParamSpec("w_o", ((pre + "o", (H, self.nh * self.dv)),))]
        if self.params.get("qk_norm_eps") is not None:
            specs += [ParamSpec("q_norm", ((pre + "q.norm", (self.nh * self.d,)),), role="vector"),
                      ParamSpec("k_norm", ((pre + "k.norm", (self.nkv * self.d,)),), role="vector")]
        if self.value_mix == "blend":
            specs.append(ParamSpec("mix", ((pre + "vmix", ()),), role="vector"))
        return specs

    def ignorable_tensors(self):
        return () if self.value_mix == "blend" else (self.prefix + "vmix",)      # a layer that does not blend may still carry one

    def bind(self, tensors):
        small = f32_params({k: tensors[k] for k in ("q_norm", "k_norm") if k in tensors})
        if "mix" in tensors:      # a constant of the model: read once, handed to the kernel as a number
            self.mix = float(tensors["mix"].float().reshape(-1)[0].item())
        super().bind({"w_proj": _pad_rows(tensors["w_proj"]), "w_o": tensors["w_o"], **small})

    def cache_need(self):
        return KVCacheNeed(self.nkv, self.d, self.window, value_dim=self.dv, keep_first=self.keep_first)

    def flops(self, rows, attended=0):
        seen = min(attended, rows * (self.window + self.keep_first)) if self.window else attended
        return super().flops(rows) + 2.0 * seen * (self.d + self.dv) * self.nh

    def forward(self, step, h):
        ops, p, w = self.ctx.ops, self.params, self.w
        g = self.cache.group
        kc, vc = self.cache.k(self.cache_index), self.cache.v(self.cache_index)
        T = step.rows
        proj = linear32(self.ctx, step, h, w["w_proj"], "cwa_proj")
        q = step.ws("cwa_q", (T, self.nh * self.d))
        slots = step.slots(g) if self.cache_owner else None
        source = None
        if self.value_mix is not None:      # the step's rows of values that the "source" layer made, one buffer per size
            key = ("value_mix_source", self.nkv * self.dv)
            if self.value_mix == "source":
                source = step.shared[key] = step.ws("values_of_source", (T, self.nkv * self.dv), torch.float32)
            else:
                source = step.shared.get(key)
                if source is None:
                    raise RuntimeError(f"capped_window_attention {self.prefix!r} blends its values with a layer's that has not run "
                                       "(value_mix 'source' must come first)")
        ops.norm_rotate_store(proj, q, self.nh, self.nkv, self.d, self.dv, p.get("qk_norm_eps") or 0.0,
                              q_weight=w.get("q_norm"), k_weight=w.get("k_norm"),
                              v_other=source if self.value_mix == "blend" else None, mix=self.mix,
                              v_keep=source if self.value_mix == "source" else None,
                              cos_sin=self.position.pairs_table(step), rot=self.position.params["dims"], slots=slots,
                              kcache=kc, vcache=vc, rows=T, halves=True)
        attn = step.ws("cwa_attn", (T, self.nh * self.dv))
        _attend(self, step, q, attn, kc, vc, g, self.nh, self.nkv, self.d, self.dv, p["scale"], self.window,
                keep_first=self.keep_first, softcap=float(p.get("softcap") or 0.0))
        return linear32(self.ctx, step, attn, w["w_o"], "cwa_out", keep_partial=True)      # the stream's next norm adds the slices
