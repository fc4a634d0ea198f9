"""Four attentions over the paged cache that share the kernels of the window attention (ops.attention_window_pool,
its matrix-core form for runs of positions, ops.rotate_store): grouped-query attention with a half-split rotation on
part of each head, rescaled pair by pair for longer contexts, and one sigmoid gate per head; a latent attention
that caches one small normed vector per token from which every head's keys and values are made (optionally with a
rotated key part shared by all heads beside it, queries that go through a latent of their own, and a gate per element);
a grouped-query attention with queries and keys normed over their whole projection, capped scores, a window that keeps a
sequence's first tokens in sight, and values blended with an earlier layer's; and a grouped-query attention with biases,
a norm per head, keys that double as values, a query temperature by position, a bias by distance and a gate per element.
Every size, constant and tensor name is a parameter.
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


def _attend(mixer, step, q, attn, kc, vc, g, nh, nkv, d, dv, scale, window, keep_first=0, softcap=0.0, dist_slope=None, gate=None):
    """Keys and values of one size, no window, no cap on the scores, bfloat16: the kernels every attention over paged
    keys and values takes (parts/paged_attention.py: partitioned for single rows, tiled for runs of positions).
    Otherwise the window attention's: steps with runs of positions take its matrix-core kernel where it has the head
    shape, others one (row, head) per workgroup.  ``gate`` (32-bit logits, one per element of the output): the window
    attention's kernels multiply their output with its sigmoid as they store it; -> True when that was done (False: the
    caller still has to)."""
    ops = mixer.ctx.ops
    if d == dv and window == 0 and not softcap and dist_slope is None and attn.dtype == torch.bfloat16 and d % 8 == 0 and d <= 256:
        paged_attention.attend(step, ops, q, attn, kc, vc, g, nh, nkv, d, scale, 0)
        return False
    if step.max_run > 1 and ops.attention_window_pool_tiles_supported(d, dv, attn.dtype, kc.shape[2]):
        ops.attention_window_pool_tiles(q, attn, kc, vc, None, None, step.tables(g), step.table_stride(g), step.run_start,
                                        step.seq_start, step.seqs, step.max_run, nh, nkv, d, dv, scale, window, 0,
                                        keep_first=keep_first, softcap=softcap, dist_slope=dist_slope, gate=gate)
    else:
        ops.attention_window_pool(q, attn, kc, vc, None, None, step.tables(g), step.table_stride(g), step.row_seq, step.ctx_lens,
                                  nh, nkv, d, dv, scale, window, 0, rows=step.rows, keep_first=keep_first, softcap=softcap,
                                  dist_slope=dist_slope, gate=gate)
    return gate is not None


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
    """Attention whose keys and values are made from one latent vector per token:
    c = n(W_dkv h) * w_norm (n: division by the root mean square, eps), k_h = W_uk,h c, v_h = W_uv,h c, q_h = W_q,h h,
    score = (q_h . k_h) * scale over the last ``window`` tokens (0: all).  Only c is cached.  The products with W_uk and
    W_uv are moved to the query's and the output's side when the weights are bound (q_h . W_uk,h c = (W_uk,h^T q_h) . c,
    and sum_j p_j W_uv,h c_j = W_uv,h sum_j p_j c_j): the step computes q' = (W_uk^T W_q) h per head, attends over the
    cached c as the one key and value head of size kv_rank, and projects with W_o W_uv.

    What a model may add (all off by default):
      rot_dim, position   every head's query has ``rot_dim`` further entries after its ``dim`` and W_dkv ``rot_dim`` further
                          rows after its kv_rank: one key part shared by all heads, not normed; both are rotated
                          (``position``: a PartSpec) and score = (q_h . k_h + q_rot,h . k_rot) * scale.  The pages hold
                          [rotated key part | c] as the one key head and c as the value.
      q_rank              queries go through a latent of their own: c_q = n(W_dq h) * w_dq.norm, q = W_uq c_q.
      gate                True: the heads' outputs are multiplied element by element with sigmoid(W_g h) before the output
                          projection (W_uv then stays a product of its own, one small matrix per head).
      shares_kv           True: the layer has no W_dkv and reads the pages another layer of the same shape wrote
                          (LayerSpec.cache_from names it), with its own W_uk, W_uv, queries and everything else.
    params: heads, dim, vdim, kv_rank, scale, window, eps, rot_dim, position, q_rank, gate, shares_kv.  Tensors under
    the prefix: q (or dq, dq.norm, uq), dkv, dkv.norm, uk, uv, o, g (with gate)."""

    capturable = True
    sub_part_names = ("position",)

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        p = params
        self.nh, self.d, self.dv, self.r = p["heads"], p["dim"], p["vdim"], p["kv_rank"]
        self.rd, self.q_rank = p.get("rot_dim", 0) or 0, p.get("q_rank", 0) or 0
        self.gate, self.shares_kv = bool(p.get("gate")), bool(p.get("shares_kv"))
        self.dk = self.rd + self.r      # a cached key: [rotated part | c]
        pos = p.get("position") or PartSpec("rotary_halves", {"dims": 0, "base": 10000.0})
        self.position = POSITIONS.get(pos.kind)(pos.params, prefix, ctx)
        if self.position.params["dims"] > self.rd:
            raise ValueError(f"latent_attention {prefix!r}: {self.position.params['dims']} rotated entries do not fit a rotated "
                             f"part of {self.rd}")

    def sub_parts(self):
        return (self.position,)

    def param_specs(self):
        H, pre = self.ctx.hidden_size, self.prefix
        nh, d, dv, r, rd = self.nh, self.d, self.dv, self.r, self.rd
        if self.q_rank:
            specs = [ParamSpec("w_dq", ((pre + "dq", (self.q_rank, H)),)),
                     ParamSpec("q_norm", ((pre + "dq.norm", (self.q_rank,)),), role="vector"),
                     ParamSpec("w_uq", ((pre + "uq", (nh * (d + rd), self.q_rank)),))]
        else:
            specs = [ParamSpec("w_q", ((pre + "q", (nh * (d + rd), H)),))]
        if not self.shares_kv:
            specs += [ParamSpec("w_dkv", ((pre + "dkv", (r + rd, H)),)),
                      ParamSpec("c_norm", ((pre + "dkv.norm", (r,)),), role="vector")]
        specs += [ParamSpec("w_uk", ((pre + "uk", (nh * d, r)),)),
                  ParamSpec("w_uv", ((pre + "uv", (nh * dv, r)),)),
                  ParamSpec("w_o", ((pre + "o", (H, nh * dv)),))]
        if self.gate:
            specs.append(ParamSpec("w_g", ((pre + "g", (nh * dv, H)),)))
        return specs

    def bind(self, tensors):
        nh, d, dv, r, rd = self.nh, self.d, self.dv, self.r, self.rd
        t = tensors
        wq = t["w_uq"] if self.q_rank else t["w_q"]      # [nh * (d + rd), K]: every head's [d plain | rd rotated] rows
        K, dt = wq.shape[1], wq.dtype
        # the product with W_uk folded into the queries' matrix, formed in double precision and rounded once; a head's rows
        # become [rotated (rd) | folded (r)], the order of a cached key
        per_head = wq.double().view(nh, d + rd, K)
        folded = torch.einsum("hdr,hdw->hrw", t["w_uk"].double().view(nh, d, r), per_head[:, :d])
        w_query = torch.cat([per_head[:, d:], folded], 1).reshape(nh * (rd + r), K).to(dt).contiguous()
        bound = {}
        first = [] if self.q_rank else [w_query]
        if self.q_rank:
            first.append(t["w_dq"])
            bound["w_query"] = w_query
        if not self.shares_kv:
            c_rows, rot_rows = t["w_dkv"][:r], t["w_dkv"][r:]
            first += [rot_rows, c_rows, c_rows]      # [rotated key part | c | c]: c goes to the pages as part of the key and as the value
            bound.update(f32_params({"c_norm": t["c_norm"]}))
        if self.q_rank:
            bound.update(f32_params({"q_norm": t["q_norm"]}))
        if self.gate:
            first.append(t["w_g"])
            bound["w_uv"] = t["w_uv"].view(nh, dv, r).contiguous()
            bound["w_o"] = t["w_o"]
        else:      # no gate between them: W_uv folded into the output projection
            o_abs = torch.einsum("whv,hvr->whr", t["w_o"].double().view(-1, nh, dv), t["w_uv"].double().view(nh, dv, r))
            bound["w_o"] = o_abs.reshape(-1, nh * r).to(dt).contiguous()
        bound["w_proj"] = _pad_rows(torch.cat(first, 0).contiguous())
        # where the first product's columns start
        self.kv_at = self.q_rank if self.q_rank else nh * self.dk
        self.gate_at = self.kv_at + (0 if self.shares_kv else rd + 2 * r)
        super().bind(bound)

    def cache_need(self):
        return KVCacheNeed(1, self.dk, self.params.get("window", 0), value_dim=self.r)

    def flops(self, rows, attended=0):
        window = self.params.get("window", 0)
        seen = min(attended, rows * window) if window else attended      # a row sees at most its window
        return super().flops(rows) + 2.0 * seen * (self.dk + self.r) * self.nh

    def forward(self, step, h):
        ops, p, w = self.ctx.ops, self.params, self.w
        g = self.cache.group
        kc, vc = self.cache.k(self.cache_index), self.cache.v(self.cache_index)
        T, nh, r, rd, dk = step.rows, self.nh, self.r, self.rd, self.dk
        owner = self.cache_owner and not self.shares_kv
        proj = linear32(self.ctx, step, h, w["w_proj"], "la_proj")
        if owner:      # both copies of c at once
            ops.rms_groups(proj, self.kv_at + rd, r, 2, w["c_norm"], p["eps"], rows=T)
        if self.q_rank:
            cq = step.ws("la_cq", (T, self.q_rank))
            ops.rms_groups(proj, 0, self.q_rank, 1, w["q_norm"], p["eps"], rows=T, out=cq)
            queries, kv = linear32(self.ctx, step, cq, w["w_query"], "la_queries"), (proj[:, self.kv_at:] if owner else None)
        else:
            queries, kv = proj, None
        q = step.ws("la_q", (T, nh * dk))
        slots = step.slots(g) if owner else None
        ops.rotate_store(queries, q, nh, 1, dk, r, cos_sin=self.position.pairs_table(step), rot=self.position.params["dims"],
                         slots=slots, kcache=kc, vcache=vc, rows=T, halves=True, kv=kv)
        attn = step.ws("la_attn", (T, nh * r))
        _attend(self, step, q, attn, kc, vc, g, nh, 1, dk, r, p["scale"], p.get("window", 0))
        if not self.gate:
            return linear32(self.ctx, step, attn, w["w_o"], "la_out", keep_partial=True)
        # every head's W_uv on its stretch of the attended latents, times the gate, in one launch
        o = step.ws("la_values", (T, nh * self.dv))
        ops.gemm_heads(attn, w["w_uv"], o, gate=proj[:, self.gate_at:], rows=T)
        return linear32(self.ctx, step, o, w["w_o"], "la_out", keep_partial=True)


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


def distance_slopes(heads, exponent=8.0):
    """slope of head h = 2^(-exponent * (h + 1) / heads), h = 0 .. heads - 1: what is taken off a score per token of distance."""
    return [2.0 ** (-float(exponent) * (h + 1) / heads) for h in range(heads)]


@MIXERS.register("headnorm_window_attention")
class HeadNormWindowAttention(Mixer):
    """Grouped-query attention whose q and k are each normed per head: divided by the head's own root mean square (eps
    inside the root) and multiplied by one weight of the head's size that all heads share (``q.norm``, ``k.norm``).
    Projections may have biases (``bias``: q, k, (v) and o, the tensor's name + ".b").  ``values``: "keys": there is no
    value projection, a token's values are its keys as projected (biased, before the norm); "projection": W_v h.
    ``q_temp`` (coef, every): the normed query at position p is multiplied by 1 + coef * ln(floor((p + 1) / every) + 1).
    score = (q . k) * scale - slope_h * (i - j) with slope_h = 2^(-slope_exponent (h + 1) / heads) where ``distance_bias``
    is set; position i sees j <= i with i - j < window (0: all); an ordinary softmax.  ``gate``: the heads' outputs are
    multiplied element by element with sigmoid(W_g h) before the output projection.  No rotation.
    params: heads, kv_heads, dim, vdim, scale, window, eps, bias, values, q_temp, distance_bias, slope_exponent, gate.
    Tensors under the prefix: q, k, (v), q.norm, k.norm, o, (g), and with bias q.b, k.b, (v.b), o.b."""

    capturable = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        p = params
        self.nh, self.nkv, self.d, self.dv = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
        if self.nkv <= 0 or self.nh % self.nkv:
            raise ValueError(f"headnorm_window_attention {prefix!r}: heads {self.nh} is not a multiple of kv_heads {self.nkv}")
        self.values = p.get("values", "projection")
        if self.values not in ("keys", "projection"):
            raise ValueError(f"headnorm_window_attention {prefix!r}: values {self.values!r} is not supported (keys | projection)")
        if self.values == "keys" and self.dv != self.d:
            raise ValueError(f"headnorm_window_attention {prefix!r}: keys of {self.d} entries cannot be values of {self.dv}")
        self.bias, self.gate = bool(p.get("bias")), bool(p.get("gate"))
        self.window = p.get("window", 0)
        temp = p.get("q_temp")
        self.temp_coef, self.temp_every = (float(temp[0]), int(temp[1])) if temp else (0.0, 0)

    def _stretches(self):
        sizes = [("q", self.nh * self.d), ("k", self.nkv * self.d)]
        if self.values == "projection":
            sizes.append(("v", self.nkv * self.dv))
        return sizes

    def param_specs(self):
        H, pre = self.ctx.hidden_size, self.prefix
        sizes = self._stretches()
        proj = sizes + ([("g", self.nh * self.dv)] if self.gate else [])
        specs = [ParamSpec("w_proj", tuple((pre + n, (c, H)) for n, c in proj)),
                 ParamSpec("w_o", ((pre + "o", (H, self.nh * self.dv)),)),
                 ParamSpec("q_norm", ((pre + "q.norm", (self.d,)),), role="vector"),
                 ParamSpec("k_norm", ((pre + "k.norm", (self.d,)),), role="vector")]
        if self.bias:
            specs += [ParamSpec("b_proj", tuple((pre + n + ".b", (c,)) for n, c in sizes), role="bias"),
                      ParamSpec("b_o", ((pre + "o.b", (H,)),), role="bias")]
        return specs

    def bind(self, tensors):
        small = f32_params({k: tensors[k] for k in ("q_norm", "k_norm", "b_proj", "b_o") if k in tensors})
        if self.params.get("distance_bias"):
            small["slopes"] = torch.tensor(distance_slopes(self.nh, self.params.get("slope_exponent", 8.0)), dtype=torch.float32,
                                           device=tensors["w_o"].device)
        super().bind({"w_proj": _pad_rows(tensors["w_proj"]), "w_o": tensors["w_o"], **small})
        self.gate_at = sum(c for _, c in self._stretches())

    def cache_need(self):
        return KVCacheNeed(self.nkv, self.d, self.window, value_dim=self.dv)

    def flops(self, rows, attended=0):
        seen = min(attended, rows * self.window) if self.window else attended
        return super().flops(rows) + 2.0 * seen * (self.d + self.dv) * self.nh

    def forward(self, step, h):
        ops, p, w = self.ctx.ops, self.params, self.w
        g = self.cache.group
        kc, vc = self.cache.k(self.cache_index), self.cache.v(self.cache_index)
        T = step.rows
        proj = linear32(self.ctx, step, h, w["w_proj"], "hwa_proj")
        q = step.ws("hwa_q", (T, self.nh * self.d))
        slots = step.slots(g) if self.cache_owner else None
        ops.head_norm_store(proj, q, self.nh, self.nkv, self.d, self.dv, p["eps"], q_weight=w["q_norm"], k_weight=w["k_norm"],
                            bias=w.get("b_proj"), positions=step.positions, temp_coef=self.temp_coef, temp_every=self.temp_every,
                            values_are_keys=self.values == "keys", slots=slots, kcache=kc, vcache=vc, rows=T)
        attn = step.ws("hwa_attn", (T, self.nh * self.dv))
        gate = proj[:, self.gate_at:] if self.gate else None
        gated = _attend(self, step, q, attn, kc, vc, g, self.nh, self.nkv, self.d, self.dv, p["scale"], self.window,
                        dist_slope=w.get("slopes"), gate=gate)
        if self.gate and not gated:
            ops.head_gate(attn, gate, self.nh, self.dv, rows=T, per_element=True)
        out = linear32(self.ctx, step, attn, w["w_o"], "hwa_out", keep_partial=True)      # the stream's next norm adds the slices
        return ops.BiasedOutput(out, w["b_o"]) if self.bias else out
