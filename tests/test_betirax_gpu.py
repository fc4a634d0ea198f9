"""The Betirax decoder in the engine against the plain implementation (tests/plain_betirax.py): every mechanism alone
through its kernels, then whole models of small odd sizes through the step function, the cache manager, the replayer's
schedules and the engine's own entry point."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import betirax_cases as cases
import plain_betirax as plain
from helpers import replay, schedule_mixed, schedule_portions, schedule_tail_singly, schedule_whole, tokens_needed

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.asarray(a), dtype=dtype).to(DEV).contiguous()


def bf16_grid(a):
    return torch.from_numpy(np.asarray(a, dtype=np.float64)).to(torch.bfloat16).double().numpy()


def i32(a):
    return torch.tensor(list(a), dtype=torch.int32, device=DEV)


class Run:
    """The arrays a kernel reads of a step that holds one run: ``count`` rows of one sequence from position ``first``."""

    def __init__(self, first, count):
        pos = list(range(first, first + count))
        self.rows, self.seqs, self.max_run = count, 1, count
        self.row_seq, self.positions, self.ctx_lens = i32([0] * count), i32(pos), i32([p + 1 for p in pos])
        self.run_start, self.seq_start = i32([0, count]), i32([first])


# ------------------------------------------------------------------------------ mechanisms alone
def test_the_norm_after_the_sum():
    """x <- ln(alpha x + y + bias) * w with y a tensor, the slices of a split product, or nothing; rows gathered for the head."""
    from kvcm_amd import ops
    rng = np.random.default_rng(0)
    for T, H in ((5, 48), (3, 321), (2, 4100), (2, 9004)):      # the last two: rows kept in registers, and rows too long for that
        x, y, b = rng.normal(size=(T, H)) * 3.0 + 1.0, rng.normal(size=(T, H)), rng.normal(size=H)
        w = 1.0 + 0.2 * rng.normal(size=H)
        for alpha, bias, splits in ((2.25, True, 1), (0.7, False, 3), (1.0, True, 9)):
            want = plain.layer_norm(alpha * x + y + (b if bias else 0.0), w, 1e-5)
            parts = rng.normal(size=(splits, T, H))
            parts[0] = y - parts[1:].sum(0)
            for dt, tol in ((torch.float32, 4e-6), (torch.bfloat16, 2.0 ** -7)):
                xs, out = dev(x), torch.empty(T, H, dtype=dt, device=DEV)
                add = dev(y) if splits == 1 else ops.PartialSums(dev(parts), splits, T, H, torch.empty(T, H, device=DEV))
                ops.layernorm_post(xs, dev(w), 1e-5, alpha=alpha, add=ops.BiasedOutput(add, dev(b)) if bias else add, out=out)
                np.testing.assert_allclose(xs.cpu().numpy(), want, atol=4e-6 * np.abs(want).max() * (splits ** 0.5 + 1), err_msg=f"{T}x{H} stream")
                np.testing.assert_allclose(out.float().cpu().numpy(), want, atol=tol * np.abs(want).max() * 2, err_msg=f"{T}x{H} {dt}")
        # nothing added, rows gathered, the stream left alone
        rows = [T - 1, 0, T - 1]
        xs, out = dev(x), torch.empty(3, H, device=DEV)
        ops.layernorm_post(xs, dev(w), 1e-5, out=out, rows=i32(rows))
        np.testing.assert_allclose(out.cpu().numpy(), plain.layer_norm(x[rows], w, 1e-5), atol=1e-5)
        assert torch.equal(xs, dev(x))
        ops.layernorm_post(xs, dev(w), 1e-5, alpha=1.0)      # in place, no copy asked for
        np.testing.assert_allclose(xs.cpu().numpy(), plain.layer_norm(x, w, 1e-5), atol=1e-5)


@pytest.mark.parametrize("shape", [dict(nh=4, nkv=2, d=16, every=5), dict(nh=3, nkv=1, d=10, every=16), dict(nh=2, nkv=2, d=128, every=1),
                                   dict(nh=1, nkv=1, d=64, every=0)])
def test_norm_per_head_with_biases_temperature_and_keys_as_values(shape):
    from kvcm_amd import ops
    nh, nkv, d, every = (shape[k] for k in ("nh", "nkv", "d", "every"))
    rng = np.random.default_rng(d + nh)
    B, eps, coef = 8, 1e-5, 0.6
    pos = [0, 1, every - 2, every - 1, every, 2 * every - 1, 2 * every, 7 * every + 3, 1000] if every else [0, 5, 9]
    pos = [max(p, 0) for p in pos]
    T = len(pos)
    proj, bias = rng.normal(size=(T, (nh + nkv) * d + 5)), rng.normal(size=(nh + nkv) * d)
    wq, wk = 1.0 + 0.2 * rng.normal(size=d), 1.0 + 0.2 * rng.normal(size=d)
    x = proj[:, :(nh + nkv) * d] + bias
    q, k = x[:, :nh * d].reshape(T, nh, d), x[:, nh * d:].reshape(T, nkv, d)
    want_q = plain.rms(q, eps) * wq
    if every:
        want_q = want_q * plain.query_temperature(pos, coef, every)[:, None, None]
    want_k = plain.rms(k, eps) * wk
    slots = i32(([17, 3, 9, 0, 31, 8, 1, 2, -1] * 2)[:T])
    for dt, tol in ((torch.float32, 2e-5), (torch.bfloat16, 2.0 ** -7)):
        q_out = torch.empty(T, nh * d, dtype=dt, device=DEV)
        kc, vc = torch.zeros(4, nkv, B, d, dtype=dt, device=DEV), torch.zeros(4, nkv, d, B, dtype=dt, device=DEV)
        ops.head_norm_store(dev(proj), q_out, nh, nkv, d, d, eps, q_weight=dev(wq), k_weight=dev(wk), bias=dev(bias), positions=i32(pos),
                            temp_coef=coef, temp_every=every, values_are_keys=True, slots=slots, kcache=kc, vcache=vc)
        np.testing.assert_allclose(q_out.float().cpu().numpy(), want_q.reshape(T, -1), atol=tol * np.abs(want_q).max())
        for t, s in enumerate(slots.tolist()):
            if s >= 0:
                np.testing.assert_allclose(kc[s // B, :, s % B].float().cpu().numpy(), want_k[t], atol=tol * np.abs(want_k).max())
                np.testing.assert_allclose(vc[s // B, :, :, s % B].float().cpu().numpy(), k[t], atol=tol * np.abs(k).max())      # the keys before their norm
        assert int(kc.float().abs().sum((1, 3)).gt(0).sum()) == sum(s >= 0 for s in slots.tolist())      # the row without a slot stored nothing
    # values of the projection's own, no biases, no weights: everything passes
    dv = 6
    proj = rng.normal(size=(T, (nh + nkv) * d + nkv * dv))
    q_out = torch.empty(T, nh * d, device=DEV)
    kc, vc = torch.zeros(4, nkv, B, d, device=DEV), torch.zeros(4, nkv, dv, B, device=DEV)
    ops.head_norm_store(dev(proj), q_out, nh, nkv, d, dv, eps, slots=slots, kcache=kc, vcache=vc)
    np.testing.assert_allclose(q_out.cpu().numpy(), proj[:, :nh * d], atol=1e-6)
    s = int(slots[1])
    np.testing.assert_allclose(vc[s // B, :, :, s % B].cpu().numpy(), proj[1, (nh + nkv) * d:].reshape(nkv, dv), atol=1e-6)
    np.testing.assert_allclose(kc[s // B, :, s % B].cpu().numpy(), proj[1, nh * d:(nh + nkv) * d].reshape(nkv, d), atol=1e-6)


def _paged(rng, k, v, B, dtype, passed):
    """Keys [n, G, d] and values [n, G, dv] of one sequence on shuffled pages, rubbish (NaN) everywhere else; the sequence's
    first ``passed`` pages are given back (table entry -1)."""
    n, G, d = k.shape
    dv = v.shape[2]
    pages = -(-n // B)
    ids = rng.permutation(pages + 5)[:pages]
    kc = torch.full((pages + 5, G, B, d), float("nan"), dtype=dtype, device=DEV)
    vc = torch.full((pages + 5, G, dv, B), float("nan"), dtype=dtype, device=DEV)
    for t in range(passed * B, n):
        kc[ids[t // B], :, t % B] = dev(k[t], dtype)
        vc[ids[t // B], :, :, t % B] = dev(v[t], dtype)
    return kc, vc, [-1 if i < passed else int(p) for i, p in enumerate(ids)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [dict(nh=4, nkv=2, d=16, dv=16, B=16, W=20), dict(nh=3, nkv=1, d=32, dv=32, B=8, W=33), dict(nh=2, nkv=2, d=10, dv=10, B=8, W=0),
                                   dict(nh=2, nkv=1, d=64, dv=64, B=16, W=1), dict(nh=6, nkv=2, d=128, dv=128, B=32, W=70), dict(nh=8, nkv=1, d=24, dv=16, B=16, W=0),
                                   dict(nh=2, nkv=2, d=64, dv=40, B=16, W=150)])
def test_window_attention_with_a_distance_bias_and_keys_that_stand_out_at_every_edge(shape, dtype):
    """One key is made to dominate the scores in spite of the bias on its distance; it is put far away, at page borders, at the
    first position, just inside and just outside the window; decoded rows and runs of rows, through shuffled pages with rubbish
    in the others and with the pages given back that the window has passed."""
    from kvcm_amd import ops
    s = shape
    nh, nkv, d, dv, B, W = (s[k] for k in ("nh", "nkv", "d", "dv", "B", "W"))
    rng = np.random.default_rng(nh * 100 + d + W)
    n, scale = 230, 0.2
    last = n - 1
    spots = {0, 1, B - 1, B, 2 * B, last - 1, last, 37, 64, 63, 128}
    if W:
        spots |= {last - W + 1, last - W, last - W + 2, max(last - W - 1, 0)}
    slopes = plain.distance_slopes(nh)
    pos = np.arange(n)
    for spot in sorted(p for p in spots if 0 <= p <= last):
        k, v, q = rng.normal(size=(n, nkv, d)), rng.normal(size=(n, nkv, dv)), rng.normal(size=(n, nh, d))
        k[spot] *= 4.0
        # the last row asks for that key, loudly enough for the bias on its distance (up to slope * 229) not to bury it in the first head
        q[last] = np.repeat(k[spot], nh // nkv, axis=0) * (1.5 + slopes[0] * (last - spot) / (scale * (k[spot] ** 2).sum(-1).min()))
        if dtype == torch.bfloat16:
            k, v, q = bf16_grid(k), bf16_grid(v), bf16_grid(q)
        want = plain.softmax_attention(q, k, v, scale, pos, pos, W, slopes)
        tol = 3e-5 if dtype == torch.float32 else 3e-2
        for first in (last, last - 9, 100, 0):
            passed = max(first - W + 1, 0) // B if W else 0      # pages wholly before the run's first window
            kc, vc, table = _paged(rng, k, v, B, dtype, passed)
            st = Run(first, n - first)
            tables = i32(table)
            out = torch.empty(n - first, nh * dv, dtype=dtype, device=DEV)
            qd = dev(q[first:].reshape(n - first, -1), dtype)
            ops.attention_window_pool(qd, out, kc, vc, None, None, tables, len(table), st.row_seq, st.ctx_lens, nh, nkv, d, dv, scale, W, 0,
                                      dist_slope=dev(slopes))
            np.testing.assert_allclose(out.float().cpu().numpy(), want[first:].reshape(n - first, -1), atol=tol, err_msg=f"key {spot} rows from {first}")
            if ops.attention_window_pool_tiles_supported(d, dv, dtype, B):
                out2 = torch.empty_like(out)
                ops.attention_window_pool_tiles(qd, out2, kc, vc, None, None, tables, len(table), st.run_start, st.seq_start, 1, n - first,
                                                nh, nkv, d, dv, scale, W, 0, dist_slope=dev(slopes))
                np.testing.assert_allclose(out2.float().cpu().numpy(), want[first:].reshape(n - first, -1), atol=tol, err_msg=f"tiles: key {spot} rows from {first}")
    # a gate per element in the kernels' epilogue (the inputs of the loop's last round: every row of the sequence as one run)
    gate = rng.normal(size=(n - first, nh * dv + 3)) * 2
    gated = want[first:].reshape(n - first, -1) * plain.logistic(gate[:, :nh * dv])
    out4 = torch.empty_like(out)
    ops.attention_window_pool(qd, out4, kc, vc, None, None, tables, len(table), st.row_seq, st.ctx_lens, nh, nkv, d, dv, scale, W, 0,
                              dist_slope=dev(slopes), gate=dev(gate))
    np.testing.assert_allclose(out4.float().cpu().numpy(), gated, atol=tol)
    if ops.attention_window_pool_tiles_supported(d, dv, dtype, B):
        ops.attention_window_pool_tiles(qd, out4, kc, vc, None, None, tables, len(table), st.run_start, st.seq_start, 1, n - first,
                                        nh, nkv, d, dv, scale, W, 0, dist_slope=dev(slopes), gate=dev(gate))
        np.testing.assert_allclose(out4.float().cpu().numpy(), gated, atol=tol)
    # the bias matters: without it the same inputs give another answer
    out3 = torch.empty_like(out)
    ops.attention_window_pool(qd, out3, kc, vc, None, None, tables, len(table), st.row_seq, st.ctx_lens, nh, nkv, d, dv, scale, W, 0)
    if W != 1:
        assert float((out3.float() - out.float()).abs().max()) > 1e-2


def test_a_far_key_among_hundreds_comes_back_through_the_cached_latents():
    """Attention as a lookup over cached [rotated key part | latent] keys with the latent as the value: the last row's query
    points along token 5 among 900 (no window: everything is seen), for a single decoded row and for a run of rows."""
    from kvcm_amd import ops
    rng = np.random.default_rng(7)
    n, rd, r, B, nh = 900, 8, 24, 16, 3
    dk = rd + r
    k = rng.normal(size=(n, 1, dk)) * 0.1
    k[5, 0] = 0.0
    k[5, 0, rd + 2] = 3.0
    v = k[:, :, rd:].copy()
    q = rng.normal(size=(n, nh, dk)) * 0.1
    q[-1] = 0.0
    q[-1, :, rd + 2] = 5.0
    want = plain.softmax_attention(q, k, v, 1.0, np.arange(n), np.arange(n))
    assert abs(want[-1, 0, 2] - 3.0) < 0.05
    for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 2e-2)):
        kk, vv, qq = (bf16_grid(a) if dtype == torch.bfloat16 else a for a in (k, v, q))
        want = plain.softmax_attention(qq, kk, vv, 1.0, np.arange(n), np.arange(n))
        kc, vc, table = _paged(rng, kk, vv, B, dtype, 0)
        for first in (n - 1, n - 70):
            st = Run(first, n - first)
            out = torch.empty(n - first, nh * r, dtype=dtype, device=DEV)
            qd = dev(qq[first:].reshape(n - first, -1), dtype)
            ops.attention_window_pool(qd, out, kc, vc, None, None, i32(table), len(table), st.row_seq, st.ctx_lens, nh, 1, dk, r, 1.0, 0, 0)
            np.testing.assert_allclose(out.float().cpu().numpy(), want[first:].reshape(n - first, -1), atol=tol)
            if ops.attention_window_pool_tiles_supported(dk, r, dtype, B):
                out2 = torch.empty_like(out)
                ops.attention_window_pool_tiles(qd, out2, kc, vc, None, None, i32(table), len(table), st.run_start, st.seq_start, 1, n - first,
                                                nh, 1, dk, r, 1.0, 0, 0)
                np.testing.assert_allclose(out2.float().cpu().numpy(), want[first:].reshape(n - first, -1), atol=tol)


def test_rotation_with_keys_and_values_in_rows_of_their_own():
    """The queries come from a later product than the keys: rotate_store reads them from two places; rows without a slot store nothing."""
    from kvcm_amd import ops
    from kvcm_amd.parts.gated_attention_parts import rescaled_frequencies
    rng = np.random.default_rng(3)
    nh, rd, r, B, T, dims = 3, 8, 12, 8, 6, 4
    dk = rd + r
    pos = [0, 1, 7, 100, 1000, 31]
    freqs, factor = rescaled_frequencies(dims, 100.0, (3.0, 40, 4.0, 1.0))
    f2, factor2 = plain.ramp_frequencies(dims, 100.0, {"factor": 3.0, "original": 40, "fast": 4.0, "slow": 1.0})
    np.testing.assert_allclose(freqs, f2, rtol=1e-12)
    assert abs(factor - factor2) < 1e-12
    table = torch.empty(T, dims, device=DEV)
    ops.rotary_freq_table(i32(pos), torch.tensor(freqs, dtype=torch.float64, device=DEV), table, dims, factor)
    q, kv = rng.normal(size=(T, nh * dk + 3)), rng.normal(size=(T, 7 + dk + r))
    want_q = plain.rotate_halves(q[:, :nh * dk].reshape(T, nh, dk), pos, dims, f2, factor2).reshape(T, -1)
    want_k = plain.rotate_halves(kv[:, 7:7 + dk].reshape(T, 1, dk), pos, dims, f2, factor2).reshape(T, -1)
    slots = i32([5, 0, 9, -1, 23, 8])
    q_out = torch.empty(T, nh * dk, device=DEV)
    kc, vc = torch.zeros(3, 1, B, dk, device=DEV), torch.zeros(3, 1, r, B, device=DEV)
    ops.rotate_store(dev(q), q_out, nh, 1, dk, r, cos_sin=table, rot=dims, slots=slots, kcache=kc, vcache=vc, halves=True, kv=dev(kv)[:, 7:])
    np.testing.assert_allclose(q_out.cpu().numpy(), want_q, atol=2e-6)
    for t, s in enumerate(slots.tolist()):
        if s >= 0:
            np.testing.assert_allclose(kc[s // B, 0, s % B].cpu().numpy(), want_k[t], atol=2e-6)
            np.testing.assert_allclose(vc[s // B, 0, :, s % B].cpu().numpy(), kv[t, 7 + dk:], atol=1e-6)
    assert float(kc.abs().sum(-1).gt(0).sum()) == 5
    # steps of few rows take a workgroup per head, steps of many one per row: the same bits
    many = 4
    q_big = torch.empty(many * T, nh * dk, device=DEV)
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    ops.rotate_store(dev(np.tile(q, (many, 1))), q_big, nh, 1, dk, r, cos_sin=table.repeat(many, 1), rot=dims,
                     slots=torch.cat([slots] + [torch.full_like(slots, -1)] * (many - 1)), kcache=kc2, vcache=vc2, halves=True,
                     kv=dev(np.tile(kv, (many, 1)))[:, 7:])
    assert torch.equal(q_big[:T], q_out) and torch.equal(q_big[-T:], q_out) and torch.equal(kc2, kc) and torch.equal(vc2, vc)
    # a layer that only reads pages: queries alone, nothing stored
    q_only = torch.empty(T, nh * dk, device=DEV)
    ops.rotate_store(dev(q)[:, :nh * dk].contiguous(), q_only, nh, 1, dk, r, cos_sin=table, rot=dims, halves=True)
    assert torch.equal(q_only, q_out)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_one_product_per_head_with_a_gate(dtype):
    from kvcm_amd import ops
    rng = np.random.default_rng(5)
    for M, heads, N, K in ((1, 3, 12, 20), (5, 2, 80, 96), (16, 4, 64, 64), (17, 1, 7, 9), (70, 8, 40, 24), (130, 2, 130, 72)):
        x, w, g = rng.normal(size=(M, heads * K + 8)), rng.normal(size=(heads, N, K)) / K ** 0.5, rng.normal(size=(M, heads * N + 4))
        if dtype == torch.bfloat16:
            x, w = bf16_grid(x), bf16_grid(w)
        want = np.einsum("mhk,hnk->mhn", x[:, :heads * K].reshape(M, heads, K), w).reshape(M, -1)
        tol = 1e-5 if dtype == torch.float32 else 2.0 ** -7
        out = torch.full((M, heads * N + 2), 7.0, dtype=dtype, device=DEV)
        ops.gemm_heads(dev(x, dtype), dev(w, dtype), out)
        np.testing.assert_allclose(out[:, :heads * N].float().cpu().numpy(), want, atol=tol * np.abs(want).max(), err_msg=str((M, heads, N, K)))
        assert float((out[:, heads * N:].float() - 7.0).abs().max()) == 0.0
        ops.gemm_heads(dev(x, dtype), dev(w, dtype), out, gate=dev(g))
        gated = want * plain.logistic(g[:, :heads * N])
        np.testing.assert_allclose(out[:, :heads * N].float().cpu().numpy(), gated, atol=tol * np.abs(want).max(), err_msg=str((M, heads, N, K)))
        if dtype == torch.bfloat16:      # a 32-bit result of bfloat16 operands
            out32 = torch.empty(M, heads * N, device=DEV)
            ops.gemm_heads(dev(x, dtype), dev(w, dtype), out32)
            np.testing.assert_allclose(out32.cpu().numpy(), want, atol=1e-5 * np.abs(want).max())


def test_small_elementwise_pieces():
    """The gate per element, the activation without a gate, a latent normed into rows of its own, routing weights over the chosen."""
    from kvcm_amd import ops
    rng = np.random.default_rng(6)
    T, heads, dv = 5, 3, 10
    o, g = rng.normal(size=(T, heads * dv)), rng.normal(size=(T, heads * dv + 3)) * 2
    for dt, tol in ((torch.float32, 1e-6), (torch.bfloat16, 2.0 ** -7)):
        od = dev(bf16_grid(o), dt)
        ops.head_gate(od, dev(g), heads, dv, per_element=True)
        np.testing.assert_allclose(od.float().cpu().numpy(), bf16_grid(o) * plain.logistic(g[:, :heads * dv]), atol=tol * 4)
        z = rng.normal(size=(T, 37)) * 3
        act = torch.empty(T, 33, dtype=dt, device=DEV)
        ops.act_rows(dev(z), act, "gelu_tanh")
        np.testing.assert_allclose(act.float().cpu().numpy(), plain.gelu_tanh(z[:, :33]), atol=tol * 12)
        parts = rng.normal(size=(3, T, 33))      # the slices of a split product are added on the way
        parts[0] = z[:, :33] - parts[1:].sum(0)
        ops.act_rows(ops.PartialSums(dev(parts), 3, T, 33, torch.empty(T, 33, device=DEV)), act, "gelu_tanh")
        np.testing.assert_allclose(act.float().cpu().numpy(), plain.gelu_tanh(z[:, :33]), atol=tol * 12)
        x, w = rng.normal(size=(T, 50)), 1.0 + 0.1 * rng.normal(size=20)
        xs, out = dev(x), torch.zeros(T, 24, dtype=dt, device=DEV)
        ops.rms_groups(xs, 7, 20, 1, dev(w), 1e-5, out=out)
        np.testing.assert_allclose(out[:, :20].float().cpu().numpy(), plain.rms(x[:, 7:27], 1e-5) * w, atol=tol * 4)
        assert torch.equal(xs, dev(x)) and float(out[:, 20:].abs().sum()) == 0.0
    for E, top in ((8, 4), (5, 3), (1, 1), (2, 2), (70, 6)):
        z = rng.normal(size=(9, E)) * 2
        want_c, want_w = plain.choose_experts(z, top)
        chosen, weight = torch.empty(9, top, dtype=torch.int32, device=DEV), torch.empty(9, top, device=DEV)
        ops.moe_route(dev(z), E, top, chosen, weight, over_chosen=True)
        assert chosen.cpu().numpy().tolist() == want_c.tolist()
        np.testing.assert_allclose(weight.cpu().numpy(), want_w, atol=2e-6)
        np.testing.assert_allclose(weight.sum(-1).cpu().numpy(), 1.0, atol=1e-6)
        parts = rng.normal(size=(3, 9, E))      # a router product that was split along K: the route adds its slices
        parts[0] = z - parts[1:].sum(0)
        ops.moe_route(ops.PartialSums(dev(parts), 3, 9, E, torch.empty(9, E, device=DEV)), E, top, chosen, weight, over_chosen=True)
        assert chosen.cpu().numpy().tolist() == want_c.tolist()
        np.testing.assert_allclose(weight.cpu().numpy(), want_w, atol=1e-5)


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
                               architecture="Betirax", model_config=cfg, tensors=tensors)
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


# float32 is the sharp test: every position within 1e-4 of the logits' spread and 5e-6 on average.  In bfloat16 the inputs of
# every product and the pages are rounded to 8 bits: the mean error is held and at most one position in fifty lies beyond a fifth.
def within(got, ref, dtype, what=""):
    e = errors(got, ref)
    every = np.concatenate(list(e.values()))
    if dtype == "float32":
        rid = max(e, key=lambda r: e[r].max())
        assert every.max() <= 1e-4, f"{what}: request {rid} position {int(e[rid].argmax())} is off by {every.max():.3g} of the logits' spread"
        assert every.mean() <= 5e-6, f"{what}: the mean error is {every.mean():.3g} of the logits' spread"
    else:
        assert every.mean() <= 0.03, f"{what}: the mean error is {every.mean():.3g} of the logits' spread"
        assert (every > 0.2).mean() <= 0.02, f"{what}: {(every > 0.2).sum()} of {every.size} positions are off by more than a fifth"


CASES = [(n, d) for n in cases.CONFIGS for d in ("float32", "bfloat16")]


def check(models, case, make_steps):
    rp, reqs, ref, _, _ = models(*case)
    got = replay(rp, make_steps(reqs), reqs)
    within(got, ref, case[1], str(case))
    assert all(rp.core.blocks_in_use(g) == 0 for g in range(rp.core.num_groups))
    return got


@pytest.mark.parametrize("name", list(cases.CONFIGS))
def test_layer_by_layer_against_the_plain_stream(models, name):
    """The residual stream after every layer of a whole prompt in 32-bit."""
    rp, reqs, _, raw, t = models(name, "float32")
    toks = reqs["r1"]
    trace = []
    plain.forward(raw, t, toks, trace)
    model = rp.runner.model
    seen = []
    for block in model.blocks:
        original = block.forward

        def wrapped(step, x, pending, original=original):
            out = original(step, x, pending)      # a layer of this design leaves nothing pending: the stream is complete
            seen.append(x[:len(toks)].cpu().numpy())
            return out
        block.forward = wrapped
    try:
        rp.step({"step": 0, "entries": [{"id": "a", "tokens": toks, "want": [0]}], "end": ["a"]})
    finally:
        for block in model.blocks:
            del block.forward
    assert len(seen) == len(trace) == len(model.blocks)
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
def test_unequal_requests_in_one_batch_on_reused_pages(models, case, seed):
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
    step's metadata changed; padding rows and padding sequences must leave the pages alone."""
    from kvcm_amd.engine.replay import TraceReplayer
    _, reqs, ref, raw, _ = models(*case)
    cfg, tensors = cases.tensors_for(raw, seed=len(case[0]) + sum(map(ord, case[0])))
    rp = TraceReplayer(None, case[1], max_tokens=tokens_needed(reqs, 3), block_size=cases.BLOCK_SIZE[case[0]], max_live=3,
                       architecture="Betirax", model_config=cfg, tensors=tensors, use_programs=True)
    assert rp.programs is not None
    for steps in (schedule_mixed(reqs, seed=5, max_live=3), schedule_tail_singly(reqs, tail=20)):
        within(replay(rp, steps, reqs), ref, case[1], str(case))
    assert rp.steps_replayed > 50


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q", "R"])
def test_long_decoding_far_beyond_every_window(name, dtype):
    """300 tokens one by one: every window passes over decoded tokens and the temperature climbs its steps; pages behind a
    window are given back, the latent attentions keep everything."""
    from kvcm_amd.engine.replay import TraceReplayer
    raw = cases.CONFIGS[name] if dtype == "float32" else cases.with_every_expert_chosen(cases.CONFIGS[name])
    cfg, tensors = cases.tensors_for(raw, seed=1 + ord(name))
    n = 300
    toks = cases.requests_for(raw, (n,), seed=11)["r0"]
    ref = {"r0": plain.forward(raw, cases.as_numpy(tensors), toks)}
    steps = [{"step": 0, "entries": [{"id": "r0", "tokens": toks[:4], "want": [0, 1, 2, 3]}], "end": []}]
    steps += [{"step": i, "entries": [{"id": "r0", "tokens": [toks[i]], "want": [0]}], "end": []} for i in range(4, n)]
    rp = TraceReplayer(None, dtype, max_tokens=320, block_size=cases.BLOCK_SIZE[name], max_live=2, architecture="Betirax",
                       model_config=cfg, tensors=tensors)
    within(replay(rp, steps, {"r0": toks}), ref, dtype, name)
    B = cases.BLOCK_SIZE[name]
    tables = rp.tables()["r0"]
    for g, spec in enumerate(rp.core.groups):
        first_needed = max(0, n - spec.window + 1) // B if spec.kind == "window" else 0
        assert [p >= 0 for p in tables[g]] == [i >= first_needed for i in range(len(tables[g]))], (g, spec)
    rp.step({"step": n, "entries": [], "end": ["r0"]})


def test_a_short_request_on_a_long_request_s_pages(models):
    rp, _, _, raw, t = models("P", "float32")
    long_, short = cases.requests_for(raw, (150, 5), seed=21).values()
    rp.step({"step": 0, "entries": [{"id": "a", "tokens": long_, "want": []}], "end": ["a"]})
    got = rp.step({"step": 1, "entries": [{"id": "b", "tokens": short, "want": list(range(5))}], "end": ["b"]})
    ref = plain.forward(raw, t, short)
    np.testing.assert_allclose(got, ref, atol=3e-5 * np.abs(ref).max())


def test_the_first_tokens_of_a_sequence(models):
    """Positions 0, 1, 2 alone and one by one: windows, temperatures and rotations at their start."""
    for name in cases.CONFIGS:
        rp, _, _, raw, t = models(name, "float32")
        toks = cases.requests_for(raw, (3,), seed=31)["r0"]
        ref = plain.forward(raw, t, toks)
        rows = [rp.step({"step": i, "entries": [{"id": "f", "tokens": [toks[i]], "want": [0]}], "end": ["f"] if i == 2 else []})[0] for i in range(3)]
        np.testing.assert_allclose(np.stack(rows), ref, atol=3e-5 * np.abs(ref).max(), err_msg=name)


def _model_folder(path, raw, tensors):
    from kvcm_amd.weights.safetensors_io import write_safetensors
    os.makedirs(path)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(raw, f)
    write_safetensors(os.path.join(path, "model.safetensors"), {k: v.to(torch.bfloat16) for k, v in tensors.items()})
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
    want, margins = [], []
    for p in prompts:
        toks = list(p)
        for _ in range(new):
            row = plain.forward(raw, t, toks)[-1]
            best = np.sort(row)[-2:]
            margins.append(best[1] - best[0])
            toks.append(int(np.argmax(row)))
        want.append(toks[len(p):])
    assert min(margins) > 1e-3      # no choice is so close that 32-bit rounding could decide it
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
    assert p.returncode == 0 and "Betirax" in p.stdout, p.stderr
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
