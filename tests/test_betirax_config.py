"""The Betirax design without a GPU: its configuration and the errors it names, the parts, cache groups and tensors a
configuration becomes, what binding does to a latent attention's matrices, random model folders, and pins of the plain
implementation (tests/plain_betirax.py) on inputs with known answers."""
import copy
import json

import numpy as np
import pytest
import torch

import betirax_cases as cases
import plain_betirax as plain


def test_configurations_round_trip_and_name_every_bad_key():
    from kvcm_amd.config.betirax_config import BetiraxConfig
    from kvcm_amd.config.model_config import ConfigError
    for raw in cases.CONFIGS.values():
        cfg = BetiraxConfig.from_dict(raw)
        assert BetiraxConfig.from_dict(cfg.to_dict()) == cfg
        assert BetiraxConfig.from_dict(json.loads(json.dumps(cfg.to_dict()))) == cfg
    r = BetiraxConfig.from_dict(cases.CONFIGS["R"])
    assert (r.embedding_scale, r.alpha, r.layers[2].mlp, r.layers[1].mixer.rot_dim, r.layers[1].mixer.rot_dims) == (1.0, 1.0, None, 0, 0)
    assert (r.layers[0].mixer.temp_every, r.layers[3].mixer.kv_from) == (0, 1)
    bad = copy.deepcopy(cases.CONFIGS["Q"])
    bad["layers"][0]["mixer"]["kv_heads"] = 3
    bad["layers"][0]["mixer"]["vdim"] = 48
    bad["layers"][0]["mixer"]["q_temp"]["every"] = 0
    bad["layers"][1]["mixer"]["rot"]["dims"] = 7
    bad["layers"][2]["mixer"]["mask"] = {}
    bad["layers"][3]["mixer"]["kv_rank"] = 32
    bad["layers"][3]["mlp"]["router"]["top"] = 9
    bad["layers"][1]["mlp"]["kind"] = "sparse"
    del bad["width"]
    with pytest.raises(ConfigError) as e:
        BetiraxConfig.from_dict(bad)
    text = str(e.value)
    for piece in ("config.width", "kv_heads 3", "vdim 48 must equal dim 64", "q_temp.every", "rot.dims 7", "layers[2].mixer.mask.size",
                  "kv_rank, rot_dim and rot must equal", "top 9 exceeds", "'sparse' is not supported"):
        assert piece in text, (piece, text)
    for source, piece in ((3, "must name an earlier latent_attention layer"), (0, "must name an earlier latent_attention layer"), ("l1", "must be a layer's number")):
        worse = copy.deepcopy(cases.CONFIGS["Q"])
        worse["layers"][3]["mixer"]["kv_from"] = source
        with pytest.raises(ConfigError, match=piece):
            BetiraxConfig.from_dict(worse)
    chain = copy.deepcopy(cases.CONFIGS["P"])
    chain["layers"].append(copy.deepcopy(chain["layers"][2]))
    chain["layers"][4]["mixer"]["kv_from"] = 2
    with pytest.raises(ConfigError, match="no keys and values of its own"):
        BetiraxConfig.from_dict(chain)
    with pytest.raises(ConfigError, match="'mlstm' is not supported"):
        BetiraxConfig.from_dict(dict(cases.CONFIGS["R"], layers=[{"type": "mlstm", "mixer": {}, "mlp": None}]))
    # what a file may leave out: kv_heads (= heads), vdim (= dim), the rotation's dims (= rot_dim) and base
    lean = copy.deepcopy(cases.CONFIGS["S"])
    del lean["layers"][0]["mixer"]["kv_heads"], lean["layers"][0]["mixer"]["vdim"], lean["layers"][1]["mixer"]["rot"]["dims"]
    del lean["layers"][1]["mixer"]["rot"]["base"], lean["layers"][1]["mixer"]["vdim"]
    cfg = BetiraxConfig.from_dict(lean)
    a, b = cfg.layers[0].mixer, cfg.layers[1].mixer
    assert (a.kv_heads, a.vdim, b.rot_dims, b.rot_base, b.vdim) == (6, 128, 16, 10000.0, 48)
    assert BetiraxConfig.from_dict(cfg.to_dict()) == cfg


def test_parts_cache_groups_and_tensors_of_a_configuration():
    from kvcm_amd.architectures.betirax import betirax_spec
    from kvcm_amd.config.betirax_config import BetiraxConfig
    from kvcm_amd.engine.runner import plan_groups
    from kvcm_amd.parts.base import BuildContext, KVCacheNeed
    from kvcm_amd.parts.model import Model
    from kvcm_amd.weights.random_init import expected_tensors
    cfg = BetiraxConfig.from_dict(cases.CONFIGS["Q"])
    spec = betirax_spec(cfg)
    assert [l.block for l in spec.layers] == ["postnorm_residual"] * 4
    assert [l.parts["mixer"].kind for l in spec.layers] == ["headnorm_window_attention", "latent_attention"] * 2
    assert [l.cache_from for l in spec.layers] == [None, None, None, {"mixer": "l1"}]
    assert spec.head.params["tied"] and spec.layers[0].parts["norm_mixer_out"].params["alpha"] == 0.8 and spec.final_norm.params["alpha"] == 1.0
    assert spec.layers[0].parts["ffn"].params["routing"] == "softmax_chosen" and spec.layers[1].parts["ffn"].kind == "plain_mlp"
    model = Model(spec, BuildContext(torch.bfloat16, torch.device("cpu"), spec.hidden_size, 16, None))
    assert model.capturable, model.not_capturable()
    needs = [g.need for g in model.groups]
    # the reading layer owns no pages: three groups for four layers
    assert needs == [KVCacheNeed(1, 64, 33, value_dim=64), KVCacheNeed(1, 128, 0, value_dim=64), KVCacheNeed(4, 32, 0, value_dim=32)]
    kinds = sorted((g.kind, g.window) for g in plan_groups(model, 50, 4))
    assert kinds == [("full", 0), ("full", 0), ("window", 33)]
    names = expected_tensors("Betirax", cfg)
    for n in ("embed", "final.norm", "l0.norm1", "l0.norm2", "l0.mix.q.b", "l0.mix.k.b", "l0.mix.o.b", "l0.mix.q.norm", "l0.mix.g", "l0.mlp.e3.gate",
              "l0.mlp.router", "l0.mlp.shared.down", "l1.mix.dq.norm", "l1.mix.uq", "l1.mix.dkv", "l1.mix.dkv.norm", "l1.mix.uk", "l1.mix.g",
              "l1.mlp.up", "l3.mix.uv", "l3.mlp.shared.up"):
        assert n in names, n
    for n in ("head", "l0.mix.v", "l3.mix.dkv", "l3.mix.dkv.norm", "l1.mix.o.b", "l1.mlp.gate", "l2.mlp.router"):
        assert n not in names, n
    assert names["l1.mix.dkv"][0] == (64 + 64, 64) and names["l1.mix.uq"][0] == (4 * (32 + 64), 48) and names["l0.mix.q.b"] == ((128,), "bias")
    assert names["l0.mix.q.norm"][0] == (64,) and names["l0.mix.g"][0] == (128, 64)
    # a layer without a feed-forward has no second norm
    assert "l2.norm2" not in expected_tensors("Betirax", BetiraxConfig.from_dict(cases.CONFIGS["R"]))


def test_binding_folds_the_key_matrices_into_the_queries():
    """What the step multiplies with: per head [rotated rows | W_uk^T W_uq's plain rows], so that a query dotted with a cached
    [rotated key part | latent] is the score of the design's own form."""
    from kvcm_amd.parts.base import BuildContext
    from kvcm_amd.parts.gated_attention_parts import LatentAttention
    rng = np.random.default_rng(0)
    nh, d, rd, dv, r, qr, H = 3, 8, 4, 6, 10, 12, 16
    part = LatentAttention({"heads": nh, "dim": d, "vdim": dv, "kv_rank": r, "scale": 1.0, "eps": 1e-5, "rot_dim": rd, "q_rank": qr, "gate": True},
                           "m.", BuildContext(torch.float32, torch.device("cpu"), H, 16, None))
    shapes = {s.name: s.shape for s in part.param_specs()}
    t = {n: torch.from_numpy(rng.normal(size=sh)).float() for n, sh in shapes.items()}
    part.bind(t)
    cq, c, kr = rng.normal(size=qr), rng.normal(size=r), rng.normal(size=rd)
    q = (t["w_uq"].double().numpy() @ cq).reshape(nh, d + rd)
    ku = (t["w_uk"].double().numpy() @ c).reshape(nh, d)
    want = (q[:, :d] * ku).sum(-1) + q[:, d:] @ kr
    got = (part.w["w_query"].double().numpy() @ cq).reshape(nh, rd + r) @ np.concatenate([kr, c])
    np.testing.assert_allclose(got, want, rtol=1e-5)
    assert part.w["w_proj"].shape[0] % 16 == 0 and (part.kv_at, part.gate_at) == (qr, qr + rd + 2 * r)
    assert torch.equal(part.w["w_proj"][qr:qr + rd], t["w_dkv"][r:]) and torch.equal(part.w["w_proj"][qr + rd + r:qr + rd + 2 * r], t["w_dkv"][:r])
    assert part.cache_need().head_dim == rd + r and part.cache_need().value_dim == r


def test_random_model_folders_of_the_design(tmp_path):
    from kvcm_amd.config.betirax_config import BetiraxConfig
    from kvcm_amd.engine.build import read_model_config
    from kvcm_amd.weights.random_init import write_model_dir
    cfg = BetiraxConfig.from_dict(cases.CONFIGS["P"])
    d = write_model_dir(str(tmp_path / "m"), "Betirax", cfg, seed=4, dtype=torch.bfloat16, std=0.1, norm_jitter=0.1, device="cpu")
    arch, again = read_model_config(d)
    assert arch.name == "Betirax" and again == cfg
    t = plain.read_tensors(str(tmp_path / "m" / "model.safetensors"))
    assert abs(t["l1.norm1"].mean() - 1.0) < 0.1 and abs(t["l1.mix.q.b"].mean()) < 0.1 and t["l1.mix.o.b"].shape == (48,)
    logits = plain.forward(cases.CONFIGS["P"], t, [5, 17, 3, 90])
    assert logits.shape == (4, 97) and np.isfinite(logits).all()


# ---------------------------------------------------------------- pins of the plain implementation
def test_plain_norms_and_activations_on_known_inputs():
    x = np.array([[1.0, 2.0, 3.0, 6.0]])
    y = plain.layer_norm(x, np.array([1.0, 1.0, 2.0, 1.0]), 0.0)
    np.testing.assert_allclose(y, [[-2 / 3.5 ** 0.5, -1 / 3.5 ** 0.5, 0.0, 3 / 3.5 ** 0.5]], atol=1e-12)
    assert abs(plain.layer_norm(x + 100.0, np.ones(4), 0.0) - plain.layer_norm(x, np.ones(4), 0.0)).max() < 1e-9      # the mean goes
    np.testing.assert_allclose(plain.rms(np.array([3.0, 4.0]), 0.0), [3 / 12.5 ** 0.5, 4 / 12.5 ** 0.5])
    np.testing.assert_allclose(plain.gelu_tanh(np.array([0.0, 10.0, -10.0])), [0.0, 10.0, 0.0], atol=1e-9)
    assert abs(plain.gelu_tanh(np.array([1.0]))[0] - 0.841192) < 1e-6


def test_plain_temperature_slopes_window_and_routing_on_known_inputs():
    np.testing.assert_allclose(plain.query_temperature([0, 3, 4, 8, 9], 0.5, 5), 1 + 0.5 * np.log([1, 1, 2, 2, 3]))
    np.testing.assert_allclose(plain.distance_slopes(4), [0.25, 0.0625, 2.0 ** -6, 2.0 ** -8])
    # a window of 3 at position 5 sees 3, 4, 5; equal scores: the bias alone weighs them
    q, k, v = np.zeros((6, 1, 2)), np.zeros((6, 1, 2)), np.arange(6.0).reshape(6, 1, 1)
    out = plain.softmax_attention(q, k, v, 1.0, np.arange(6), np.arange(6), window=3, slopes=np.array([np.log(2.0)]))
    np.testing.assert_allclose(out[5, 0, 0], (3 * 0.25 + 4 * 0.5 + 5 * 1.0) / 1.75)
    np.testing.assert_allclose(out[1, 0, 0], (0 * 0.5 + 1 * 1.0) / 1.5)
    chosen, weight = plain.choose_experts(np.array([[0.0, 2.0, 1.0, 2.0 + np.log(3.0)]]), 2)
    assert chosen.tolist() == [[3, 1]]
    np.testing.assert_allclose(weight, [[0.75, 0.25]])


def test_plain_rotation_rescaling_on_known_inputs():
    f, factor = plain.ramp_frequencies(8, 10000.0)
    np.testing.assert_allclose(f, [1.0, 0.1, 0.01, 0.001])
    assert factor == 1.0
    sc = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
    f2, factor2 = plain.ramp_frequencies(8, 10000.0, sc)
    assert abs(factor2 - (0.1 * np.log(4.0) + 1)) < 1e-12
    # pair(8 turns) = 8 ln(64 / (16 pi)) / (2 ln 1e4) = 0.10..: lo 0; pair(1 turn) = 1.007..: hi 2; ramp 0, 0.5, 1, 1
    np.testing.assert_allclose(f2, [1.0, 0.1 * (0.5 / 4 + 0.5), 0.01 / 4, 0.001 / 4])
    x = np.array([[1.0, 0.0, 5.0]])
    np.testing.assert_allclose(plain.rotate_halves(x, [3], 2, np.array([np.pi / 6])), [[0.0, 1.0, 5.0]], atol=1e-12)
