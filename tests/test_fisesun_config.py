"""The Fisesun design without a GPU: its configuration and the errors it names, the parts, cache groups and tensors a
configuration becomes, the cache manager's pages under a window that keeps a sequence's first tokens, random model
folders, and pins of the plain implementation (tests/plain_fisesun.py) on inputs with known answers."""
import copy
import json
import os

import numpy as np
import pytest
import torch

import fisesun_cases as cases
import plain_fisesun as plain


def test_configurations_round_trip_and_name_every_bad_key():
    from kvcm_amd.config.fisesun_config import FisesunConfig
    from kvcm_amd.config.model_config import ConfigError
    for raw in cases.CONFIGS.values():
        cfg = FisesunConfig.from_dict(raw)
        assert FisesunConfig.from_dict(cfg.to_dict()) == cfg
        assert FisesunConfig.from_dict(json.loads(json.dumps(cfg.to_dict()))) == cfg
    r = FisesunConfig.from_dict(cases.CONFIGS["R"])
    assert (r.embedding_scale, r.logit_softcap, r.layers[2].mlp, r.layers[2].mixer.window, r.layers[0].mixer.softcap) == (1.0, 0.0, None, 0, 0.0)
    bad = copy.deepcopy(cases.CONFIGS["Q"])
    bad["layers"][0]["mixer"]["kv_heads"] = 3
    bad["layers"][0]["mixer"]["rot"]["dims"] = 7
    bad["layers"][0]["mixer"]["rot"]["scaling"]["high"] = 1.0
    bad["layers"][2]["mixer"]["mask"] = {}
    bad["layers"][2]["mixer"]["vdim"] = 40
    bad["layers"][1]["type"] = "lstm"
    bad["layers"][3]["mlp"]["router"]["top"] = 9
    bad["layers"][0]["mlp"]["kind"] = "sparse"
    del bad["width"]
    with pytest.raises(ConfigError) as e:
        FisesunConfig.from_dict(bad)
    text = str(e.value)
    for piece in ("config.width", "kv_heads 3", "rot.dims 7", "low and high must differ", "layers[2].mixer.mask.size", "'lstm' is not supported",
                  "top 9 exceeds", "'sparse' is not supported", "v_mix needs the values of layers[0]"):
        assert piece in text, (piece, text)
    # what a file may leave out: kv_heads (= heads), vdim (= dim), the rotation's base, keep_first, v_mix, the caps
    lean = copy.deepcopy(cases.CONFIGS["P"])
    m = lean["layers"][3]["mixer"]
    del m["kv_heads"], m["vdim"], m["v_mix"], m["mask"]["keep_first"], lean["layers"][1]["mixer"]["rot"]["base"], lean["logit_softcap"]
    cfg = FisesunConfig.from_dict(lean)
    a = cfg.layers[3].mixer
    assert (a.kv_heads, a.vdim, a.v_mix, a.keep_first, cfg.layers[1].mixer.rot_base, cfg.logit_softcap) == (6, 8, False, 0, 10000.0, 0.0)
    assert FisesunConfig.from_dict(cfg.to_dict()) == cfg


def test_parts_cache_groups_and_tensors_of_a_configuration():
    from kvcm_amd.architectures.fisesun import fisesun_spec
    from kvcm_amd.config.fisesun_config import FisesunConfig
    from kvcm_amd.engine.runner import plan_groups
    from kvcm_amd.parts.base import BuildContext, KVCacheNeed, StateNeed
    from kvcm_amd.parts.model import Model
    from kvcm_amd.weights.random_init import expected_tensors
    cfg = FisesunConfig.from_dict(cases.CONFIGS["Q"])
    spec = fisesun_spec(cfg)
    assert [l.block for l in spec.layers] == ["output_norm_residual"] * 4
    mixes = [l.parts["mixer"].params.get("value_mix") for l in spec.layers]
    assert mixes == ["source", None, "blend", None]      # the first blending layer lends, the later ones blend, the last opted out
    assert spec.head.params["softcap"] == 30.0 and spec.layers[0].parts["mixer"].params["position"].params["scaling_kind"] == "wavelength"
    model = Model(spec, BuildContext(torch.bfloat16, torch.device("cpu"), spec.hidden_size, 16, None))
    assert model.capturable, model.not_capturable()
    needs = [g.need for g in model.groups]
    assert KVCacheNeed(1, 64, 33, value_dim=40, keep_first=21) in needs and KVCacheNeed(1, 64, 10, value_dim=40, keep_first=40) in needs
    assert KVCacheNeed(2, 32, 40, value_dim=64, keep_first=5) in needs and StateNeed((2, 32, 16), torch.float32) in needs
    groups = plan_groups(model, 50, 4)
    windows = sorted((g.window, g.keep_first) for g in groups if g.kind == "window")
    assert windows == [(10, 40), (33, 21), (40, 5)]
    names = expected_tensors("Fisesun", cfg)
    for n in ("embed", "final.norm", "head", "l0.norm1", "l0.norm2", "l0.mix.q.norm", "l0.mix.k.norm", "l0.mlp.e3.gate", "l0.mlp.table",
              "l0.mlp.shared.down", "l1.mix.f.b", "l2.mix.vmix", "l2.mlp.gate", "l3.mlp.shared.up"):
        assert n in names, n
    assert "l0.mix.vmix" not in names and "l3.mix.vmix" not in names and "l1.mlp.shared.up" not in names
    assert names["l0.mlp.table"] == ((130, 2), "index") and names["l2.mix.vmix"][0] == ()
    # a layer without a feed-forward has no second norm; without a window every key is kept
    r = Model(fisesun_spec(FisesunConfig.from_dict(cases.CONFIGS["R"])), BuildContext(torch.float32, torch.device("cpu"), 32, 8, None))
    assert "l2.norm2" not in expected_tensors("Fisesun", FisesunConfig.from_dict(cases.CONFIGS["R"]))
    kinds = {(g.kind, g.window, g.keep_first) for g in plan_groups(r, 10, 2)}
    assert ("full", 0, 0) in kinds and ("window", 1, 2) in kinds


def test_pages_under_a_window_that_keeps_the_first_tokens():
    """Pages that the window has passed are given back, except those that hold a sequence's kept first tokens."""
    from kvcm_amd.cache.manager import CacheGroupSpec, HostCore
    B = 8
    core = HostCore([CacheGroupSpec("window", 20, 64, keep_first=11), CacheGroupSpec("window", 20, 64), CacheGroupSpec("window", 5, 64, keep_first=8)],
                    block_size=B, max_seq_len=256, max_num_seqs=2, watermark_blocks=0)
    core.seq_new(1, list(range(30)))
    core.admit(1)
    done = 0
    for n in (30, 7, 1, 1, 50, 1, 40):
        if done:
            core.seq_push_tokens(1, list(range(n)))
            assert core.append_slot(1)
        done += n
        core.set_computed(1, done)
        core.commit(1)
        first_needed = max(0, done - 20 + 1) // B
        t0, t1, t2 = (core.seq_table(1, g) for g in range(3))
        assert all((p >= 0) == (i < 2 or i >= first_needed) for i, p in enumerate(t0)), (done, t0)      # 11 kept tokens: two pages stay
        assert all((p >= 0) == (i >= first_needed) for i, p in enumerate(t1)), (done, t1)
        assert all((p >= 0) == (i < 1 or i >= max(0, done - 5 + 1) // B) for i, p in enumerate(t2)), (done, t2)
    in_use = [core.blocks_in_use(g) for g in range(3)]
    assert in_use[0] == in_use[1] + 2 and in_use[2] == 1 + len([p for p in core.seq_table(1, 2)[1:] if p >= 0])
    core.release(1)
    assert [core.blocks_in_use(g) for g in range(3)] == [0, 0, 0]
    with pytest.raises(Exception, match="only a windowed group"):
        HostCore([CacheGroupSpec("full", 0, 8, keep_first=3)], block_size=B, max_seq_len=64, max_num_seqs=1)


def test_random_model_folders_hold_valid_tables(tmp_path):
    from kvcm_amd.config.fisesun_config import FisesunConfig
    from kvcm_amd.engine.build import read_model_config
    from kvcm_amd.weights.random_init import write_model_dir
    cfg = FisesunConfig.from_dict(cases.CONFIGS["P"])
    d = write_model_dir(str(tmp_path / "m"), "Fisesun", cfg, seed=4, dtype=torch.bfloat16, std=0.1, norm_jitter=0.1, device="cpu")
    arch, again = read_model_config(d)
    assert arch.name == "Fisesun" and again == cfg
    t = plain.read_tensors(os.path.join(d, "model.safetensors"))
    table = t["l1.mlp.table"]
    assert table.shape == (97, 3) and table.min() >= 0 and table.max() < 5 and all(len(set(r)) == 3 for r in table.tolist())
    assert len({tuple(r) for r in table.tolist()}) > 3      # not the same experts for every token
    logits = plain.forward(cases.CONFIGS["P"], t, [5, 1, 90, 33])
    assert logits.shape == (4, 97) and np.isfinite(logits).all() and np.abs(logits).max() < 9.0


# ------------------------------------------------------------------ the plain implementation on inputs with known answers
def test_plain_frequencies_by_wavelength():
    f = plain.pair_frequencies(8, 10.0)
    np.testing.assert_allclose(f, [1.0, 10 ** -0.25, 10 ** -0.5, 10 ** -0.75])
    # wavelengths 2 pi / f = 6.28, 11.2, 19.9, 35.3 against original / high = 10 and original / low = 25: the first keeps its
    # frequency, the last turns four times slower, the two between are blended
    g = plain.pair_frequencies(8, 10.0, {"factor": 4.0, "low": 2.0, "high": 5.0, "original": 50})
    assert g[0] == f[0] and abs(g[3] - f[3] / 4.0) < 1e-15
    for i in (1, 2):
        s = (50 * f[i] / (2 * np.pi) - 2.0) / 3.0
        assert 0 < s < 1 and abs(g[i] - ((1 - s) * f[i] / 4 + s * f[i])) < 1e-15
    from kvcm_amd.parts.gated_attention_parts import wavelength_scaled_frequencies
    for dims, base, sc in ((8, 10.0, (4.0, 2.0, 5.0, 50)), (64, 5e5, (8.0, 1.0, 4.0, 8192)), (2, 3.0, None), (32, 500.0, (2.0, 0.5, 64.0, 100))):
        np.testing.assert_allclose(wavelength_scaled_frequencies(dims, base, sc),
                                   plain.pair_frequencies(dims, base, dict(zip(("factor", "low", "high", "original"), sc)) if sc else None), rtol=1e-13)


def test_plain_rotation_and_what_a_position_sees():
    x = np.zeros((2, 1, 6))
    x[:, 0, 0], x[:, 0, 5] = 1.0, 7.0
    y = plain.rotate_halves(x, [0, 3], 4, np.array([np.pi / 6, 0.0]))      # pairs (0, 2) and (1, 3); entries 4, 5 pass
    np.testing.assert_allclose(y[0, 0], [1, 0, 0, 0, 0, 7], atol=1e-15)
    np.testing.assert_allclose(y[1, 0], [0, 0, 1, 0, 0, 7], atol=1e-15)      # a quarter turn moves entry 0 to its partner
    m = plain.sees(range(8), range(8), 3, 2)
    assert m[7].tolist() == [True, True, False, False, False, True, True, True]
    assert m[3].tolist() == [True, True, True, True, False, False, False, False] and m[0].tolist() == [True] + [False] * 7
    assert plain.sees(range(5), range(5), 0, 9)[4].all() and plain.sees([6], range(8), 2, 0)[0].tolist() == [False] * 5 + [True, True, False]


def test_plain_attention_caps_scores_and_reads_a_kept_token():
    # one query along one key: with a cap the weight of that key cannot outgrow exp(cap) against the others
    q = np.zeros((1, 1, 4))
    q[0, 0, 0] = 100.0
    k, v = np.zeros((3, 1, 4)), np.eye(3)[:, None, :]
    k[1, 0, 0] = 1.0
    free = plain.capped_softmax_attention(q, k, v, 1.0, None, np.ones((1, 3), bool))[0, 0]
    capped = plain.capped_softmax_attention(q, k, v, 1.0, 2.0, np.ones((1, 3), bool))[0, 0]
    np.testing.assert_allclose(free, [0, 1, 0], atol=1e-30)
    np.testing.assert_allclose(capped, np.exp([0, 2.0, 0]) / (2 + np.exp(2.0)), rtol=1e-6)
    hidden = plain.capped_softmax_attention(q, k, v, 1.0, None, np.array([[True, False, True]]))[0, 0]
    np.testing.assert_allclose(hidden, [0.5, 0, 0.5])


def test_plain_memory_maximum_starts_at_zero_and_routing_by_table():
    # shut gates: with m starting at 0 (not at minus infinity) the first token's output is k v^T q exp(li) over max(|n q|, 1)
    q, k, v = np.array([[1.0, 0.0]]), np.array([[2.0, 0.0]]), np.array([[3.0, 5.0]])
    o, (S, n, m) = plain.memory_walk(q, k, v, np.array([-4.0]), np.array([-1.0]))
    assert m == -1.0      # max(lf + 0, li)
    take = np.exp(-4.0 + 1.0)
    np.testing.assert_allclose(o[0], take * 2.0 * np.array([3.0, 5.0]) / (max(take * 2.0, np.exp(1.0)) + 1e-6))
    w = {"e0.gate": np.eye(2), "e0.up": np.eye(2), "e0.down": np.eye(2), "e1.gate": np.eye(2), "e1.up": 2 * np.eye(2), "e1.down": np.eye(2),
         "shared.gate": np.eye(2), "shared.up": np.eye(2), "shared.down": -np.eye(2), "table": np.array([[0, 1], [1, 0], [1, 1]])}
    h = np.array([[1.0, -2.0], [0.5, 0.0]])
    one = plain.silu(h) * h
    mlp = {"kind": "moe", "router": {"experts": 2, "top": 2}, "expert": {"ff": 2}}
    np.testing.assert_allclose(plain.table_mixture(h, [0, 1], w, "", mlp), (one + 2 * one) / 2)
    np.testing.assert_allclose(plain.table_mixture(h, [2, 2], w, "", {**mlp, "shared": {"ff": 2}}), (2 * one + 2 * one) / 2 - one)
    np.testing.assert_allclose(plain.table_mixture(h, [2, 0], w, "", {**mlp, "router": {"experts": 2, "top": 1}}), np.stack([2 * one[0], one[1]]))


def test_plain_layer_order_and_value_blending():
    """x <- x + rms(mixer(x)) w1, then the feed-forward reads the NEW x; a blending layer takes the first such layer's
    values before that layer's own blending (it has none), a layer that does not blend is left alone."""
    raw = cases.CONFIGS["P"]
    cfg, tensors = cases.tensors_for(raw, seed=2)
    t = cases.as_numpy(tensors)
    toks = [3, 50, 96, 0, 7, 7, 21]
    trace = []
    logits = plain.forward(raw, t, toks, trace)
    assert len(trace) == 4 and logits.shape == (7, 97) and np.abs(logits).max() < 9.0
    x0 = t["embed"][toks] * 3.0
    x1 = x0 + plain.rms(plain.mlstm(x0, t, "l0.mix.", raw["layers"][0]["mixer"], 1e-5), 1e-5) * t["l0.norm1"]
    np.testing.assert_allclose(trace[0], x1)
    y, v_first = plain.attention(x1, t, "l1.mix.", raw["layers"][1]["mixer"], 1e-5, None)
    x = x1 + plain.rms(y, 1e-5) * t["l1.norm1"]
    x = x + plain.rms(plain.feed_forward(x, toks, t, "l1.mlp.", raw["layers"][1]["mlp"]), 1e-5) * t["l1.norm2"]
    np.testing.assert_allclose(trace[1], x)
    y2, _ = plain.attention(x, t, "l2.mix.", raw["layers"][2]["mixer"], 1e-5, v_first)
    y2_alone, _ = plain.attention(x, t, "l2.mix.", raw["layers"][2]["mixer"], 1e-5, None)
    assert np.abs(y2 - y2_alone).max() > 1e-3
    x2 = x + plain.rms(y2, 1e-5) * t["l2.norm1"]
    x2 = x2 + plain.rms(plain.gated_ff(x2, t, "l2.mlp."), 1e-5) * t["l2.norm2"]
    np.testing.assert_allclose(trace[2], x2)
    # causal: a later token changes nothing before it
    again = plain.forward(raw, t, toks[:5] + [1, 2])
    np.testing.assert_allclose(again[:5], logits[:5], atol=1e-12)
