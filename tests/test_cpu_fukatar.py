"""The Fukatar design without a GPU: configuration, registry, frequency tables, and the oracle's own mechanisms against written-out forms."""
import pytest
import torch

from oracle import fukatar_ref as R
from tests.fukatar_shapes import SHAPES, config_of, make_weights, tokens
from tests.test_gpu_fukatar import close

F64 = torch.float64


def test_configuration_round_trip_and_design_flags():
    from vllm_i64_amd.config import FukatarConfig
    for name in SHAPES:
        c = FukatarConfig.from_dict(config_of(name))
        assert FukatarConfig.from_dict(c.to_dict()) == c
        for l in c.layers:
            if l.type == "attention":
                assert (l.mixer.qk_norm, l.mixer.interleaved, l.mixer.rotate_values, l.mixer.head_gate) == ("row", False, True, True)
            elif l.type == "parallel":
                assert (l.mixer.left.qk_norm, l.mixer.left.interleaved, l.mixer.left.rotate_values, l.mixer.left.head_gate) == ("head", True, False, False)
            else:
                assert l.mixer.sink and l.mixer.rot_dim == 0
    plain = FukatarConfig.from_dict(config_of("plain"))
    assert plain.bigram is None and plain.embedding_scale == 1.0 and plain.logit_softcap == 0.0 and plain.layers[1].mixer.kv_heads == 2
    assert plain.layers[1].mixer.softcap == 0.0 and plain.layers[1].mlp is None


def test_configuration_refuses_what_the_design_has_not():
    from vllm_i64_amd.config import FukatarConfig
    bad = config_of("plain")
    bad["layers"][0]["type"] = "mamba2"
    with pytest.raises(ValueError):
        FukatarConfig.from_dict(bad)
    bad = config_of("plain")
    bad["layers"][1]["mixer"]["rot"]["dims"] = 18
    with pytest.raises(ValueError):
        FukatarConfig.from_dict(bad)
    bad = config_of("odd")
    bad["layers"][2]["mixer"]["right"]["kv_heads"] = 3
    with pytest.raises(ValueError):
        FukatarConfig.from_dict(bad)


def test_registry_names_the_design():
    from vllm_i64_amd import registry
    assert "fukatar" in registry.architectures()
    assert registry.architecture_of(config_of("odd")) == "Fukatar"


def test_loader_takes_sizes_a_config_leaves_out_from_the_tensors(monkeypatch):
    from vllm_i64_amd import fukatar, registry
    seen = {}
    monkeypatch.setattr(fukatar, "FukatarModel", lambda cfg, tensors, **kw: seen.update(cfg=cfg, kw=kw))
    cfg = config_of("twotap")
    del cfg["vocab"], cfg["width"], cfg["layers"][0]["mixer"]["right"]["conv"]
    registry._load_fukatar(cfg, make_weights("twotap"), device="cpu", dtype="float32", max_seqs=2, max_tokens=100)
    c = seen["cfg"]
    assert (c.vocab, c.width, c.layers[0].mixer.right.conv) == (SHAPES["twotap"]["vocab"], SHAPES["twotap"]["width"], 2) and seen["kw"]["num_kv_blocks"] == 7


def test_scaled_frequencies_match_the_written_out_ramp():
    from vllm_i64_amd.config import RotaryConfig
    for base, dims, sc in ((10000.0, 64, (4.0, 512, 16.0, 1.0)), (500.0, 6, (4.0, 40, 8.0, 0.5)), (77.0, 10, None), (1e6, 128, (32.0, 8192, 32.0, 1.0))):
        r = {"base": base, "dims": dims}
        if sc:
            r["scaling"] = dict(zip(("factor", "original", "fast", "slow"), sc))
        f, mult = RotaryConfig.from_dict(r).frequencies()
        fo, mo = R.rotary_frequencies(base, dims, r.get("scaling"))
        assert close(torch.tensor(f, dtype=F64), fo, 1e-12) and abs(mult - mo) < 1e-12
        if sc:      # both ends of the ramp are there
            plain, _ = R.rotary_frequencies(base, dims)
            assert float((fo / plain).max()) > 0.99 or dims <= 6
            assert float((fo / plain).min()) < 1.0 / sc[0] + 0.01


def test_oracle_rotation_layouts_turn_pairs():
    x = torch.arange(8, dtype=F64).reshape(1, 1, 8) + 1.0
    f = torch.tensor([0.5, 0.25], dtype=F64)
    pos = torch.tensor([3])
    halves, inter = R.rotate(x, pos, f, 4, False), R.rotate(x, pos, f, 4, True)
    c, s = torch.cos(3 * f), torch.sin(3 * f)
    assert close(halves[0, 0, :4], torch.stack([1 * c[0] - 3 * s[0], 2 * c[1] - 4 * s[1], 3 * c[0] + 1 * s[0], 4 * c[1] + 2 * s[1]]), 1e-12)
    assert close(inter[0, 0, :4], torch.stack([1 * c[0] - 2 * s[0], 2 * c[0] + 1 * s[0], 3 * c[1] - 4 * s[1], 4 * c[1] + 3 * s[1]]), 1e-12)
    assert torch.equal(halves[0, 0, 4:], x[0, 0, 4:]) and torch.equal(inter[0, 0, 4:], x[0, 0, 4:])
    assert close(R.rotate(halves, -pos, f, 4, False), x, 1e-12)


def test_oracle_delta_rule_against_the_unrolled_sum():
    """With beta = 1, g = 1 and orthonormal keys the state stores every value exactly once: reading with a key returns its value."""
    d, dv = 6, 4
    k = torch.eye(d, dtype=F64)[:5].unsqueeze(1)
    g = torch.Generator().manual_seed(0)
    v = torch.randn(5, 1, dv, generator=g, dtype=F64)
    o = R.delta_rule(k, k, v, torch.ones(5, 1, dtype=F64), torch.ones(5, 1, dtype=F64))
    assert close(o, v, 1e-12)
    # a repeated key overwrites (the correction term), and a decay scales what was stored before
    k2 = torch.eye(d, dtype=F64)[[0, 0]].unsqueeze(1)
    o2 = R.delta_rule(k2, k2, v[:2], torch.ones(2, 1, dtype=F64), torch.tensor([[1.0], [0.5]], dtype=F64))
    assert close(o2[1], v[1], 1e-12)
    o3 = R.delta_rule(k2, k2, v[:2], torch.tensor([[1.0], [0.25]], dtype=F64), torch.tensor([[1.0], [0.5]], dtype=F64))
    assert close(o3[1], 0.5 * v[0] + 0.25 * (v[1] - 0.5 * v[0]), 1e-12)


def test_oracle_sink_counts_once_and_unscaled():
    q, k, v = torch.zeros(1, 1, 2, dtype=F64), torch.zeros(1, 1, 2, dtype=F64), torch.ones(1, 1, 3, dtype=F64)
    o = R.causal_attention(q, k, v, 5.0, None, sink=torch.tensor([0.7], dtype=F64))
    assert close(o[0, 0], torch.ones(3, dtype=F64) / (1.0 + torch.exp(torch.tensor(0.7, dtype=F64))), 1e-12)


def test_oracle_first_token_and_hash():
    W = {"embed": torch.arange(12, dtype=F64).reshape(6, 2), "bigram": torch.arange(10, dtype=F64).reshape(5, 2) * 100}
    e = {"scale": 2.0, "bigram": {"buckets": 4, "mul_prev": 3, "mul_cur": 5}}
    x = R.embedding(W, e, [1, 4, 4])
    assert torch.equal(x[0], W["embed"][1] * 2 + W["bigram"][4])
    assert torch.equal(x[1], W["embed"][4] * 2 + W["bigram"][(1 * 3 + 4 * 5) % 4]) and torch.equal(x[2], W["embed"][4] * 2 + W["bigram"][(4 * 3 + 4 * 5) % 4])


def test_oracle_runs_every_shape():
    for name in SHAPES:
        z = R.forward(config_of(name), make_weights(name), tokens(name, 12, 1))
        assert z.shape == (12, SHAPES[name]["vocab"]) and bool(torch.isfinite(z).all())
        cap = SHAPES[name].get("logit_softcap")
        assert cap is None or float(z.abs().max()) < cap
