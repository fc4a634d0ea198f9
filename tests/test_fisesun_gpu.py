"""The Fisesun decoder in the engine against the plain implementation (tests/plain_fisesun.py): every mechanism alone
through its kernels, then whole models of small odd sizes through the step function, the cache and state manager, the
replayer's schedules and the engine's own entry point."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import fisesun_cases as cases
import plain_fisesun as plain
from helpers import replay, schedule_mixed, schedule_portions, schedule_tail_singly, schedule_whole, tokens_needed

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.asarray(a), dtype=dtype).to(DEV).contiguous()


def bf16_grid(a):
    return torch.from_numpy(np.asarray(a, dtype=np.float64)).to(torch.bfloat16).double().numpy()


class Step:
    """The arrays a kernel reads of a step, made by hand: runs = [(state slot, first position, count)]."""

    def __init__(self, runs):
        row_seq, pos, start = [], [], [0]
        for s, (_, p0, n) in enumerate(runs):
            row_seq += [s] * n
            pos += list(range(p0, p0 + n))
            start.append(start[-1] + n)
        i32 = lambda a: torch.tensor(a, dtype=torch.int32, device=DEV)
        self.rows, self.seqs = len(pos), len(runs)
        self.max_run = max(r[2] for r in runs)
        self.row_seq, self.positions, self.ctx_lens = i32(row_seq), i32(pos), i32([p + 1 for p in pos])
        self.run_start, self.seq_start = i32(start), i32([r[1] for r in runs])
        self.seq_end, self.state_slots = i32([r[1] + r[2] for r in runs]), i32([r[0] for r in runs])


# ------------------------------------------------------------------------------ mechanisms alone
def test_the_stream_read_as_it_is_and_capped_logits():
    from kvcm_amd import ops
    rng = np.random.default_rng(0)
    for T, H in ((5, 48), (3, 321), (2, 4100)):
        x, a = rng.normal(size=(T, H)) * 3.0, rng.normal(size=(T, H)) * 0.3
        w = 1.0 + 0.2 * rng.normal(size=H)
        total = x + plain.rms(a, 1e-5) * w
        for dt, tol in ((torch.float32, 3e-6), (torch.bfloat16, 2.0 ** -7)):
            xs, out = dev(x), torch.empty(T, H, dtype=dt, device=DEV)
            ops.rmsnorm_chain(xs, 1e-5, pending=ops.NormedBranches(dev(a), dev(w)), out=out, plain=True)
            np.testing.assert_allclose(xs.cpu().numpy(), total, atol=3e-6)
            np.testing.assert_allclose(out.float().cpu().numpy(), total, atol=tol * np.abs(total).max())
            out2 = torch.empty(T, H, dtype=dt, device=DEV)      # nothing to add: a copy
            ops.rmsnorm_chain(dev(x), 1e-5, out=out2, plain=True)
            np.testing.assert_allclose(out2.float().cpu().numpy(), x, atol=tol * np.abs(x).max())
        # the output still to be added as the slices of a split product
        for S in (3, 9):
            sl = rng.normal(size=(S, T, H))
            xs, out = dev(x), torch.empty(T, H, device=DEV)
            ops.rmsnorm_chain(xs, 1e-5, pending=ops.NormedBranches(ops.PartialSums(dev(sl), S, T, H, torch.empty(T, H, device=DEV)), dev(w)), out=out, plain=True)
            np.testing.assert_allclose(out.cpu().numpy(), x + plain.rms(sl.sum(0), 1e-5) * w, atol=5e-6)
            np.testing.assert_allclose(xs.cpu().numpy(), out.cpu().numpy(), atol=0)      # the stream holds what its reader got
    z = rng.normal(size=(4, 77)) * 20
    zs = dev(z)
    ops.softcap_rows(zs, 7.5)
    np.testing.assert_allclose(zs.cpu().numpy(), plain.tanh_cap(z, 7.5), atol=2e-6)


@pytest.mark.parametrize("case", [dict(nh=3, nkv=1, d=16, dv=6, rot=8, base=100.0, sc=(3.0, 1.0, 4.0, 40)),
                                  dict(nh=6, nkv=2, d=64, dv=40, rot=64, base=5e5, sc=(8.0, 1.0, 4.0, 8192)),
                                  dict(nh=2, nkv=2, d=10, dv=24, rot=0, base=10.0, sc=None),
                                  dict(nh=1, nkv=1, d=32, dv=32, rot=12, base=7.0, sc=None)])
def test_projection_normed_over_all_heads_rotated_blended_and_stored(case):
    from kvcm_amd import ops
    from kvcm_amd.parts.gated_attention_parts import wavelength_scaled_frequencies
    c = case
    nh, nkv, d, dv, rot = c["nh"], c["nkv"], c["d"], c["dv"], c["rot"]
    rng = np.random.default_rng(nh + d)
    T, B, eps, lam = 9, 8, 1e-5, 0.3
    pos = np.array([0, 1, 2, 500, 1999, 7, 64, 65, 3], dtype=np.int64)
    H = 20
    h = rng.normal(size=(T, H))
    w = {"q": rng.normal(size=(nh * d, H)), "k": rng.normal(size=(nkv * d, H)) * 5, "v": rng.normal(size=(nkv * dv, H)),
         "q.norm": 1 + 0.2 * rng.normal(size=nh * d), "k.norm": 1 + 0.2 * rng.normal(size=nkv * d), "vmix": np.array(lam)}
    m = {"heads": nh, "kv_heads": nkv, "dim": d, "vdim": dv}
    if rot:
        m["rot"] = {"dims": rot, "base": c["base"]}
        if c["sc"]:
            m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), c["sc"]))
    v_first = rng.normal(size=(T, nkv * dv))
    want_q, want_k, want_v = plain.attention_qkv(h, w, "", m, eps, pos, v_first)
    proj = np.concatenate([h @ w["q"].T, h @ w["k"].T, h @ w["v"].T], 1)
    table = None
    if rot:
        f = wavelength_scaled_frequencies(rot, c["base"], c["sc"])
        table = torch.empty(T, rot, device=DEV)
        ops.rotary_freq_table(torch.tensor(pos, dtype=torch.int32, device=DEV), torch.tensor(f, dtype=torch.float64, device=DEV), table, rot, 1.0)
    slots = torch.tensor([17, 3, 9, 0, 31, 8, 1, 2, -1], dtype=torch.int32, device=DEV)
    for blend in (True, False):
        q_out = torch.empty(T, nh * d, device=DEV)
        kc, vc = torch.zeros(4, nkv, B, d, device=DEV), torch.zeros(4, nkv, dv, B, device=DEV)
        keep = torch.full((T, nkv * dv + 3), float("nan"), device=DEV)
        ops.norm_rotate_store(dev(proj), q_out, nh, nkv, d, dv, eps, q_weight=dev(w["q.norm"]), k_weight=dev(w["k.norm"]),
                              v_other=dev(v_first) if blend else None, mix=lam, v_keep=None if blend else keep, cos_sin=table, rot=rot,
                              slots=slots, kcache=kc, vcache=vc, halves=True)
        np.testing.assert_allclose(q_out.cpu().numpy(), want_q.reshape(T, -1), atol=1e-5)
        v_ref = want_v.reshape(T, -1) if blend else proj[:, (nh + nkv) * d:]
        if not blend:
            np.testing.assert_allclose(keep[:, :nkv * dv].cpu().numpy(), v_ref, atol=1e-6)
        for t, s in enumerate(slots.tolist()):
            if s >= 0:
                np.testing.assert_allclose(kc[s // B, :, s % B].cpu().numpy(), want_k[t], atol=1e-5)
                np.testing.assert_allclose(vc[s // B, :, :, s % B].cpu().numpy(), v_ref[t].reshape(nkv, dv), atol=2e-6)
    # steps of few rows take a workgroup per head, steps of many one per row: the same bits
    many = 5
    big, slots_big = dev(np.tile(proj, (many, 1))), torch.cat([slots] + [torch.full_like(slots, -1)] * (many - 1))
    table_big = table.repeat(many, 1) if rot else None
    q_big = torch.empty(many * T, nh * d, device=DEV)
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    ops.norm_rotate_store(big, q_big, nh, nkv, d, dv, eps, q_weight=dev(w["q.norm"]), k_weight=dev(w["k.norm"]), cos_sin=table_big, rot=rot,
                          slots=slots_big, kcache=kc2, vcache=vc2, halves=True)
    assert torch.equal(q_big[:T], q_out) and torch.equal(q_big[-T:], q_out) and torch.equal(kc2, kc) and torch.equal(vc2, vc)
    # without weights the projection passes as rotate_store leaves it
    q_a, q_b = torch.empty(T, nh * d, device=DEV), torch.empty(T, nh * d, device=DEV)
    ops.norm_rotate_store(dev(proj), q_a, nh, nkv, d, dv, 0.0, cos_sin=table, rot=rot, halves=True)
    ops.rotate_store(dev(proj), q_b, nh, nkv, d, dv, cos_sin=table, rot=rot, halves=True)
    assert torch.equal(q_a, q_b)


def _paged(rng, k, v, B, dtype, keep_pages, passed):
    """Keys [n, G, d] and values [n, G, dv] of one sequence on shuffled pages, rubbish (NaN) everywhere else; pages
    keep_pages .. passed-1 of the sequence are given back (table entry -1)."""
    n, G, d = k.shape
    dv = v.shape[2]
    pages = -(-n // B)
    ids = rng.permutation(pages + 5)[:pages]
    gone = set(range(keep_pages, passed))
    kc = torch.full((pages + 5, G, B, d), float("nan"), dtype=dtype, device=DEV)
    vc = torch.full((pages + 5, G, dv, B), float("nan"), dtype=dtype, device=DEV)
    for t in range(n):
        if t // B not in gone:
            kc[ids[t // B], :, t % B] = dev(k[t], dtype)
            vc[ids[t // B], :, :, t % B] = dev(v[t], dtype)
    return kc, vc, [-1 if i in gone else int(p) for i, p in enumerate(ids)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [dict(nh=4, nkv=2, d=16, dv=24, B=16, W=20, K=3, cap=5.0), dict(nh=3, nkv=1, d=32, dv=32, B=8, W=33, K=21, cap=0.0),
                                   dict(nh=2, nkv=2, d=10, dv=6, B=8, W=0, K=0, cap=2.0), dict(nh=2, nkv=1, d=64, dv=40, B=16, W=10, K=40, cap=12.0),
                                   dict(nh=2, nkv=1, d=40, dv=40, B=32, W=1, K=2, cap=0.0), dict(nh=2, nkv=1, d=24, dv=24, B=16, W=70, K=70, cap=8.0),
                                   dict(nh=2, nkv=2, d=64, dv=64, B=16, W=150, K=5, cap=25.0)])
def test_window_attention_that_keeps_first_tokens_with_keys_that_stand_out_at_every_edge(shape, dtype):
    """One key is made to dominate the scores; it is put far away, at page borders, at the first position, on the last kept
    token and the one after it, just inside and just outside the window; decoded rows and runs of rows, through shuffled
    pages with rubbish in the others and with the pages given back that the window has passed and that hold no kept token."""
    from kvcm_amd import ops
    s = shape
    nh, nkv, d, dv, B, W, K, cap = (s[k] for k in ("nh", "nkv", "d", "dv", "B", "W", "K", "cap"))
    rng = np.random.default_rng(nh * 100 + d + W)
    n, scale = 230, 0.2
    last = n - 1
    spots = {0, 1, B - 1, B, 2 * B, last - 1, last, 37, 64, 63, 128}
    if W:
        spots |= {last - W + 1, last - W, last - W + 2, max(last - W - 1, 0)}
    if K:
        spots |= {K - 1, K, max(K - 2, 0), K + 1}
    pos = np.arange(n)
    mask = plain.sees(pos, pos, W, K)
    for spot in sorted(p for p in spots if 0 <= p <= last):
        k, v, q = rng.normal(size=(n, nkv, d)), rng.normal(size=(n, nkv, dv)), rng.normal(size=(n, nh, d))
        k[spot] *= 4.0
        q[last] = np.repeat(k[spot], nh // nkv, axis=0) * 1.5      # the last row asks for that key
        if dtype == torch.bfloat16:
            k, v, q = bf16_grid(k), bf16_grid(v), bf16_grid(q)
        want = plain.capped_softmax_attention(q, k, v, scale, cap, mask)
        tol = 2e-5 if dtype == torch.float32 else 3e-2
        for first in (last, last - 9, 100, 0):
            passed = max(first - W + 1, 0) // B if W else 0      # pages wholly before the run's first window
            kc, vc, table = _paged(rng, k, v, B, dtype, -(-K // B) if W else 0, passed)
            st = Step([(0, first, n - first)])
            tables = torch.tensor(table, dtype=torch.int32, device=DEV)
            out = torch.empty(n - first, nh * dv, dtype=dtype, device=DEV)
            qd = dev(q[first:].reshape(n - first, -1), dtype)
            ops.attention_window_pool(qd, out, kc, vc, None, None, tables, len(table), st.row_seq, st.ctx_lens, nh, nkv, d, dv, scale, W, 0,
                                      keep_first=K, softcap=cap)
            np.testing.assert_allclose(out.float().cpu().numpy(), want[first:].reshape(n - first, -1), atol=tol, err_msg=f"key {spot} rows from {first}")
            if ops.attention_window_pool_tiles_supported(d, dv, dtype, B):
                out2 = torch.empty_like(out)
                ops.attention_window_pool_tiles(qd, out2, kc, vc, None, None, tables, len(table), st.run_start, st.seq_start, 1, n - first,
                                                nh, nkv, d, dv, scale, W, 0, keep_first=K, softcap=cap)
                np.testing.assert_allclose(out2.float().cpu().numpy(), want[first:].reshape(n - first, -1), atol=tol, err_msg=f"tiles: key {spot} rows from {first}")


def test_a_kept_token_is_read_back_from_far_beyond_the_window():
    """Attention as a lookup: the query of the last row points along the key of token 2 among 700; with keep_first 3 its
    value comes back, with keep_first 2 it does not."""
    from kvcm_amd import ops
    rng = np.random.default_rng(7)
    n, d, dv, B, W = 700, 32, 16, 16, 50
    k, v = rng.normal(size=(n, 1, d)) * 0.1, rng.normal(size=(n, 1, dv))
    k[2, 0] = 0.0
    k[2, 0, 5] = 3.0
    q = np.zeros((1, 1, d))
    q[0, 0, 5] = 4.0
    for dtype in (torch.float32, torch.bfloat16):
        kc, vc, table = _paged(rng, k, v, B, dtype, 1, (n - W) // B)
        st = Step([(0, n - 1, 1)])
        tables = torch.tensor(table, dtype=torch.int32, device=DEV)
        for keep, hit in ((3, True), (2, False)):
            out = torch.empty(1, dv, dtype=dtype, device=DEV)
            ops.attention_window_pool(dev(q.reshape(1, -1), dtype), out, kc, vc, None, None, tables, len(table), st.row_seq, st.ctx_lens, 1, 1, d, dv,
                                      1.0, W, 0, keep_first=keep)
            close = np.abs(out.float().cpu().numpy()[0] - v[2, 0]).max() < 0.05
            assert close == hit, (dtype, keep)


@pytest.mark.parametrize("sizes", [(8, 2, 48, 32, 64, 16), (5, 3, 52, 20, 9, 24), (3, 1, 33, 7, 40, 0), (2, 2, 64, 16, 130, 8), (1, 1, 16, 40, 3, 0), (70, 6, 32, 16, 200, 0)])
def test_gated_experts_named_by_a_table_by_rows_and_grouped(sizes):
    """Through the part itself: table routing, experts by rows (few rows) and grouped (many rows), sizes that are padded
    to sixteen, the shared expert as where the experts' sum starts."""
    from kvcm_amd import ops
    from kvcm_amd.parts.base import BuildContext, PartSpec
    from kvcm_amd.parts.routed_parts import RoutedExperts, interleave_gate_up
    E, top, H, F, T, SF = sizes
    rng = np.random.default_rng(E * 10 + top)
    V = 50
    w = {"table": np.stack([rng.permutation(E)[:top] for _ in range(V)])}
    for e in range(E):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = (rng.normal(size=s) / np.sqrt(s[1]) for s in ((F, H), (F, H), (H, F)))
    if SF:
        w["shared.gate"], w["shared.up"], w["shared.down"] = (rng.normal(size=s) / np.sqrt(s[1]) for s in ((SF, H), (SF, H), (H, SF)))
    h, tokens = rng.normal(size=(T, H)), rng.integers(0, V, size=T)
    mlp = {"kind": "moe", "router": {"experts": E, "top": top}, "expert": {"ff": F}, **({"shared": {"ff": SF}} if SF else {})}
    for dt, tol in ((torch.float32, 3e-5), (torch.bfloat16, 4e-2)):
        ww = {k: (bf16_grid(a) if dt == torch.bfloat16 and k != "table" else a) for k, a in w.items()}
        hh = bf16_grid(h) if dt == torch.bfloat16 else h
        want = plain.table_mixture(hh, tokens, ww, "", mlp)
        shared = PartSpec("gated_mlp", {"intermediate_size": SF, "activation": "silu"}, "shared.") if SF else None
        part = RoutedExperts({"experts": E, "top": top, "ff": F, "routing": "table", "activation": "silu_gated", "shared": shared, "vocab_size": V},
                             "", BuildContext(dt, torch.device(DEV), H, 16, ops))
        part.bind({"table": dev(ww["table"], torch.int32), "w_gate": dev(np.concatenate([ww[f"e{e}.gate"] for e in range(E)]), dt),
                   "w_up": dev(np.concatenate([ww[f"e{e}.up"] for e in range(E)]), dt),
                   "w_down": dev(np.concatenate([ww[f"e{e}.down"] for e in range(E)]), dt)})
        if SF:
            part.shared.bind({"w_gate_up": dev(np.concatenate([ww["shared.gate"], ww["shared.up"]]), dt), "w_down": dev(ww["shared.down"], dt)})
        assert part.F % 16 == 0 and part.w["w_up"].shape == (E, 2 * part.F, H)

        token_ids = torch.tensor(tokens, dtype=torch.int32, device=DEV)

        class S:
            rows, limits, tune_products = T, None, None
            tokens = token_ids
            bufs = {}

            def ws(self, name, shape, dtype=None):
                return self.bufs.setdefault((name, shape, dtype), torch.full(shape, float("nan") if (dtype or dt).is_floating_point else 0,
                                                                             dtype=dtype or dt, device=DEV))

            def flat(self, name, numel, dtype=torch.float32):
                return torch.empty(numel, dtype=dtype, device=DEV)

            def scratch(self, *a):
                return None
        out = part.forward(S(), dev(hh, dt))
        np.testing.assert_allclose(out.cpu().numpy(), want, atol=tol * max(1.0, np.abs(want).max()), err_msg=str(dt))
    g, u = torch.arange(2 * 32 * 3).reshape(2, 32, 3), -torch.arange(2 * 32 * 3).reshape(2, 32, 3)
    both = interleave_gate_up(g, u)
    assert torch.equal(both[:, :16], g[:, :16]) and torch.equal(both[:, 16:32], u[:, :16]) and torch.equal(both[:, 48:], u[:, 16:])


def test_matrix_memory_of_this_design_against_the_plain_recurrence():
    from kvcm_amd import ops
    heads, d, dv, cap = 3, 24, 40, 7.0
    rng = np.random.default_rng(4)
    n = 90
    q, k, v = rng.normal(size=(n, heads, d)), rng.normal(size=(n, heads, d)), rng.normal(size=(n, heads, dv))
    gi, gf = rng.normal(size=(n, heads)) * 4, rng.normal(size=(n, heads)) * 4 + 2
    bi, bf = rng.normal(size=heads), rng.normal(size=heads)
    want = np.zeros((n, heads, dv))
    for a in range(heads):
        want[:, a], _ = plain.memory_walk(q[:, a] * d ** -0.5, k[:, a], v[:, a], plain.tanh_cap(gi[:, a] + bi[a], cap),
                                          plain.log_logistic(plain.tanh_cap(gf[:, a] + bf[a], cap)))
    S, N, M = torch.full((2, heads, d, dv), 9.0, device=DEV), torch.full((2, heads, d), -3.0, device=DEV), torch.full((2, heads), 50.0, device=DEV)
    got, p = np.zeros((n, heads * dv)), 0
    for c in (1, 2, 40, 1, 17, 29):
        st = Step([(1, p, c)])
        packed = dev(np.concatenate([x[p:p + c].reshape(c, -1) for x in (q, k, v, gi, gf)], 1))
        at = np.cumsum([0, heads * d, heads * d, heads * dv, heads])
        o = torch.empty(c, heads * dv, device=DEV)
        ops.mlstm_scan(*(packed[:, lo:] for lo in at), dev(bi), dev(bf), cap, d ** -0.5, torch.empty(c, 4 * heads, device=DEV),
                       torch.empty(heads * d, device=DEV), o, S, N, M, st, heads, d, dv)
        got[p:p + c] = o.cpu().numpy()
        p += c
    np.testing.assert_allclose(got, want.reshape(n, -1), atol=3e-5 * max(1.0, np.abs(want).max()))


# ------------------------------------------------------------------------------ whole models
LENGTHS = (150, 41, 7, 1, 90, 23)


@pytest.fixture(scope="module")
def models():
    made = {}

    def get(name, dtype):
        if (name, dtype) not in made:
            from kvcm_amd.engine.replay import TraceReplayer
            raw = cases.CONFIGS[name]
            cfg, tensors = cases.tensors_for(raw, seed=len(name) + sum(map(ord, name)))
            reqs = cases.requests_for(raw, LENGTHS, seed=3)
            t = cases.as_numpy(tensors)
            ref = {rid: plain.forward(raw, t, toks) for rid, toks in reqs.items()}
            rp = TraceReplayer(None, dtype, max_tokens=tokens_needed(reqs, 3), block_size=cases.BLOCK_SIZE[name], max_live=3,
                               architecture="Fisesun", model_config=cfg, tensors=tensors)
            made[(name, dtype)] = (rp, reqs, ref, raw, t)
        return made[(name, dtype)]
    return get


def errors(got, ref):
    """Per position: the root mean square over the vocabulary of the difference (means taken off) over the logits' own spread."""
    spread = np.sqrt(np.mean([np.var(r, axis=1).mean() for r in ref.values()]))
    out = {}
    for rid in ref:
        d = got[rid].astype(np.float64) - ref[rid]
        e = np.sqrt(np.var(d, axis=1)) / spread
        assert not np.isnan(e).any(), f"{rid}: positions without logits"
        out[rid] = e
    return out


# float32 is the sharp test: every position within 1e-4 of the logits' spread and 3e-6 on average.  In bfloat16 the inputs of
# every product and the pages are rounded to 8 bits: the mean error is held and at most one position in fifty lies beyond a fifth.
def within(got, ref, dtype, what=""):
    e = errors(got, ref)
    every = np.concatenate(list(e.values()))
    if dtype == "float32":
        rid = max(e, key=lambda r: e[r].max())
        assert every.max() <= 1e-4, f"{what}: request {rid} position {int(e[rid].argmax())} is off by {every.max():.3g} of the logits' spread"
        assert every.mean() <= 3e-6, f"{what}: the mean error is {every.mean():.3g} of the logits' spread"
    else:
        assert every.mean() <= 0.03, f"{what}: the mean error is {every.mean():.3g} of the logits' spread"
        assert (every > 0.2).mean() <= 0.02, f"{what}: {(every > 0.2).sum()} of {every.size} positions are off by more than a fifth"


CASES = [(n, d) for n in cases.CONFIGS for d in ("float32", "bfloat16")]


def check(models, case, make_steps):
    rp, reqs, ref, _, _ = models(*case)
    got = replay(rp, make_steps(reqs), reqs)
    within(got, ref, case[1], str(case))
    assert rp.core.state_slots_free() == 3 and all(rp.core.blocks_in_use(g) == 0 for g in range(rp.core.num_groups)
                                                    if rp.core.groups[g].kind != "state")
    return got


@pytest.mark.parametrize("name", ["P", "Q"])
def test_layer_by_layer_against_the_plain_stream(models, name):
    """The residual stream after every layer of a whole prompt in 32-bit."""
    rp, reqs, _, raw, t = models(name, "float32")
    ops = rp.runner.ops
    toks = reqs["r1"]
    trace = []
    plain.forward(raw, t, toks, trace)
    model = rp.runner.model
    seen = []
    for block in model.blocks:
        original = block.forward

        def wrapped(step, x, pending, original=original):
            if pending is not None:      # the layer before is complete once its normed output is added: done here, ahead of the reader
                ops.rmsnorm_chain(x, raw["norm"]["eps"], pending=pending)
                seen.append(x[:len(toks)].cpu().numpy())
            return original(step, x, None)
        block.forward = wrapped
    try:
        rp.step({"step": 0, "entries": [{"id": "a", "tokens": toks, "want": [0]}], "end": ["a"]})
    finally:
        for block in model.blocks:
            del block.forward
    assert len(seen) == len(trace) - 1 == len(model.blocks) - 1
    for i, (g, w) in enumerate(zip(seen, trace)):
        np.testing.assert_allclose(g, w, atol=2e-5 * max(1.0, np.abs(w).max()), err_msg=f"after layer {i}")


@pytest.mark.parametrize("case", CASES)
def test_whole_prompts(models, case):
    check(models, case, schedule_whole)


@pytest.mark.parametrize("case", CASES)
def test_prompt_then_token_by_token(models, case):
    check(models, case, lambda reqs: schedule_tail_singly(reqs, tail=80))


@pytest.mark.parametrize("case", CASES)
def test_portions_down_to_two_tokens(models, case):
    check(models, case, schedule_portions)
    check(models, case, lambda reqs: schedule_portions(reqs, sizes=(2, 2, 3, 1, 2, 40, 2)))


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("seed", [0, 1])
def test_unequal_requests_in_one_batch_on_reused_pages_and_slots(models, case, seed):
    check(models, case, lambda reqs: schedule_mixed(reqs, seed=seed, max_live=3))


@pytest.mark.parametrize("name", list(cases.CONFIGS))
def test_32bit_logits_do_not_depend_on_cut_batch_or_pages(models, name):
    rp, reqs, _, _, _ = models(name, "float32")
    whole = replay(rp, schedule_whole(reqs), reqs)
    for steps in (schedule_tail_singly(reqs, tail=80), schedule_portions(reqs), schedule_mixed(reqs, seed=2, max_live=3)):
        other = replay(rp, steps, reqs)
        for rid in reqs:
            np.testing.assert_allclose(other[rid], whole[rid], atol=2e-5, rtol=0)


@pytest.mark.parametrize("case", [("P", "float32"), ("Q", "bfloat16"), ("R", "bfloat16"), ("S", "float32")])
def test_steps_replayed_from_recorded_launch_lists(models, case):
    """Every part says it is capturable: a step's shape is recorded once as a list of launches and replayed with only the
    step's metadata changed; padding rows and padding sequences must leave pages and states alone."""
    from kvcm_amd.engine.replay import TraceReplayer
    _, reqs, ref, raw, _ = models(*case)
    cfg, tensors = cases.tensors_for(raw, seed=len(case[0]) + sum(map(ord, case[0])))
    rp = TraceReplayer(None, case[1], max_tokens=tokens_needed(reqs, 3), block_size=cases.BLOCK_SIZE[case[0]], max_live=3,
                       architecture="Fisesun", model_config=cfg, tensors=tensors, use_programs=True)
    assert rp.programs is not None
    for steps in (schedule_mixed(reqs, seed=5, max_live=3), schedule_tail_singly(reqs, tail=20)):
        within(replay(rp, steps, reqs), ref, case[1], str(case))
    assert rp.steps_replayed > 50


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q", "R"])
def test_long_decoding_far_beyond_every_window(name, dtype):
    """300 tokens one by one: every window passes over decoded tokens, pages are given back behind it while those of the
    kept first tokens stay."""
    from kvcm_amd.engine.replay import TraceReplayer
    raw = cases.CONFIGS[name]
    cfg, tensors = cases.tensors_for(raw, seed=1 + ord(name))
    n = 300
    toks = cases.requests_for(raw, (n,), seed=11)["r0"]
    ref = {"r0": plain.forward(raw, cases.as_numpy(tensors), toks)}
    steps = [{"step": 0, "entries": [{"id": "r0", "tokens": toks[:4], "want": [0, 1, 2, 3]}], "end": []}]
    steps += [{"step": i, "entries": [{"id": "r0", "tokens": [toks[i]], "want": [0]}], "end": []} for i in range(4, n)]
    rp = TraceReplayer(None, dtype, max_tokens=320, block_size=cases.BLOCK_SIZE[name], max_live=2, architecture="Fisesun",
                       model_config=cfg, tensors=tensors)
    within(replay(rp, steps, {"r0": toks}), ref, dtype, name)
    B = cases.BLOCK_SIZE[name]
    tables = rp.tables()["r0"]
    for g, spec in enumerate(rp.core.groups):
        if spec.kind == "window":
            first_needed = max(0, n - spec.window + 1) // B
            assert [p >= 0 for p in tables[g]] == [i < -(-spec.keep_first // B) or i >= first_needed for i in range(len(tables[g]))], (g, spec)
    rp.step({"step": n, "entries": [], "end": ["r0"]})


def test_a_short_request_on_a_long_request_s_pages_and_slot(models):
    rp, _, _, raw, t = models("R", "float32")
    long_, short = cases.requests_for(raw, (150, 5), seed=21).values()
    rp.step({"step": 0, "entries": [{"id": "a", "tokens": long_, "want": []}], "end": ["a"]})
    got = rp.step({"step": 1, "entries": [{"id": "b", "tokens": short, "want": list(range(5))}], "end": ["b"]})
    ref = plain.forward(raw, t, short)
    np.testing.assert_allclose(got, ref, atol=3e-5 * np.abs(ref).max())


def _model_folder(path, raw, tensors):
    from kvcm_amd.weights.safetensors_io import write_safetensors
    os.makedirs(path)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(raw, f)
    stored = {k: (v.to(torch.bfloat16) if v.is_floating_point() else v) for k, v in tensors.items()}
    write_safetensors(os.path.join(path, "model.safetensors"), stored)
    return path


@pytest.mark.parametrize("name", list(cases.CONFIGS))
def test_greedy_generation_through_the_engine(name, tmp_path):
    """The entry point a user calls: model folder -> scheduler -> steps (recorded and replayed, decode steps as graphs) ->
    greedy tokens; against the plain implementation's own greedy continuation."""
    from kvcm_amd import Engine, EngineConfig
    raw = cases.CONFIGS[name]
    cfg, tensors = cases.tensors_for(raw, seed=5)
    d = _model_folder(str(tmp_path / "m"), raw, tensors)
    t = cases.as_numpy(tensors)
    prompts = list(cases.requests_for(raw, (9, 30, 1, 17), seed=8).values())
    new = 24
    want = []
    for p in prompts:
        toks = list(p)
        for _ in range(new):
            toks.append(int(np.argmax(plain.forward(raw, t, toks)[-1])))
        want.append(toks[len(p):])
    for chunk in (0, 8):
        eng = Engine(d, EngineConfig(dtype="float32", block_size=cases.BLOCK_SIZE[name], max_seq_len=128, num_blocks=40,
                                     max_num_seqs=3, max_batched_tokens=64, prefill_chunk=chunk))
        assert eng.recorded is not None          # steps are recorded and replayed, decode steps as graphs: as for the other designs
        got = eng.generate(prompts, new)
        assert got == want, f"prefill_chunk={chunk}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program_reads_the_model_folder(dtype, tmp_path):
    raw = cases.CONFIGS["Q"]
    cfg, tensors = cases.tensors_for(raw, seed=9)
    d, out = _model_folder(str(tmp_path / "m"), raw, tensors), str(tmp_path / "out")
    reqs = cases.requests_for(raw, (40, 7, 19, 70), seed=4)
    steps = schedule_mixed(reqs, seed=4, max_live=3)
    p = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", dtype, "--out", out, "--max-tokens", "256"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.split("\n") if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    t = cases.as_numpy(tensors)
    ref = {rid: plain.forward(raw, t, toks) for rid, toks in reqs.items()}
    got = {rid: np.full_like(ref[rid], np.nan, dtype=np.float32) for rid in reqs}
    pos = {rid: 0 for rid in reqs}
    for s in steps:
        rows = np.fromfile(os.path.join(out, f"{s['step']}.f32"), dtype="<f4").reshape(-1, raw["vocab"])
        r = 0
        for e in s["entries"]:
            for w in e["want"]:
                got[e["id"]][pos[e["id"]] + w] = rows[r]
                r += 1
            pos[e["id"]] += len(e["tokens"])
    within(got, ref, dtype, "trace_run")


def test_the_serving_tools_take_the_design(tmp_path):
    """kvmodel writes a random model folder from a configuration file, kvgen generates from it (greedy, against the plain
    implementation on the folder's own tensors), kvbench serves a small workload with random weights of it."""
    cfg_file = str(tmp_path / "p.json")
    with open(cfg_file, "w") as f:
        json.dump(cases.CONFIGS["P"], f)
    d = str(tmp_path / "m")
    tool = lambda name, *args: subprocess.run([sys.executable, os.path.join(ROOT, "bin", name), *args], capture_output=True,
                                              text=True, timeout=300)
    p = tool("kvmodel", "--out", d, "--config-json", cfg_file, "--weights-seed", "3", "--std", "0.15", "--norm-jitter", "0.1")
    assert p.returncode == 0 and "Fisesun" in p.stdout, p.stderr
    prompt = [5, 17, 3, 90, 41, 77, 9]
    p = tool("kvgen", "--model", d, "--dtype", "fp32", "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "10",
             "--max-seq-len", "64", "--num-blocks", "16")
    assert p.returncode == 0, p.stderr
    t = plain.read_tensors(os.path.join(d, "model.safetensors"))
    toks = list(prompt)
    for _ in range(10):
        toks.append(int(np.argmax(plain.forward(cases.CONFIGS["P"], t, toks)[-1])))
    assert [int(x) for x in p.stdout.split()] == toks[len(prompt):]
    p = tool("kvbench", "--random-weights", "--config-json", cfg_file, "--dtype", "bf16", "--requests", "6", "--prompt-len", "9",
             "--output-len", "5", "--max-seq-len", "64", "--num-blocks", "32", "--warmup", "1")
    assert p.returncode == 0, p.stderr + p.stdout
