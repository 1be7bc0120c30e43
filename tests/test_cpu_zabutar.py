"""The Zabutar design without a GPU: configuration, registry, cache layout, distance buckets, and the oracle's own mechanisms against
other forms of the same equations."""
import math

import pytest
import torch

from oracle import zabutar_ref as R
from tests.zabutar_shapes import SHAPES, config_of, make_weights, tokens


def test_config_reads_every_size_and_round_trips():
    from vllm_i64_amd.config import BiasedAttentionConfig, Hgrn2Config, MoeMlpConfig, ZabutarConfig
    for name in SHAPES:
        d = config_of(name)
        c = ZabutarConfig.from_dict(d)
        assert c.vocab == d["vocab"] and c.width == d["width"] and c.canon_taps == d["canon"]["taps"] and c.max_pos == d["max_positions"]
        assert ZabutarConfig.from_dict(c.to_dict()) == c
    c = ZabutarConfig.from_dict(config_of("odd"))
    assert isinstance(c.layers[0].mixer, Hgrn2Config) and isinstance(c.layers[1].mixer, BiasedAttentionConfig) and c.layers[2].mixer.kv_from == 1
    f = c.layers[1].mlp
    assert isinstance(f, MoeMlpConfig) and (f.experts, f.identity, f.entries, f.groups, f.keep, f.top, f.shared_ff) == (5, 1, 6, 3, 2, 2, 20)
    assert c.layers[2].mlp is None and c.layers[3].mlp.groups == 1 and c.layers[3].mlp.shared_ff == 0


@pytest.mark.parametrize("change", ["kv_from_later", "kv_from_recurrent", "kv_sizes", "groups", "type"])
def test_config_refuses_what_the_design_does_not_have(change):
    from vllm_i64_amd.config import ZabutarConfig
    d = config_of("odd")
    if change == "kv_from_later":
        d["layers"][2]["mixer"]["kv_from"] = 4
    elif change == "kv_from_recurrent":
        d["layers"][2]["mixer"]["kv_from"] = 0
    elif change == "kv_sizes":
        d["layers"][2]["mixer"]["vdim"] = 10
    elif change == "groups":
        d["layers"][1]["mlp"]["router"]["groups"] = {"count": 4, "keep": 1}
    else:
        d["layers"][0]["type"] = "mamba2"
    with pytest.raises((ValueError, KeyError)):
        ZabutarConfig.from_dict(d)


def test_registry_names_the_design():
    from vllm_i64_amd import registry
    assert "zabutar" in registry.architectures()
    assert registry.architecture_of(config_of("plain")) == "Zabutar"


def test_loader_takes_missing_sizes_from_the_tensors(monkeypatch):
    from vllm_i64_amd import registry, zabutar
    seen = {}
    monkeypatch.setattr(zabutar, "ZabutarModel", lambda cfg, tensors, **kw: seen.setdefault("cfg", cfg))
    d = config_of("odd")
    for key in ("vocab", "width", "max_positions", "canon"):
        d.pop(key)
    cfg = registry._load_zabutar(d, make_weights("odd"), device="cpu", dtype="float32", max_seqs=2, max_tokens=64)
    assert (cfg.vocab, cfg.width, cfg.max_positions, cfg.canon_taps) == (83, 40, 300, 3)


def test_cache_shares_rows_between_layers_and_bounds_positions():
    from vllm_i64_amd.paged_cache import HybridCache
    kv = HybridCache([{"rows": 12, "kscale": False, "state": {"canon1": (2, 8)}}, {"state": {"gla": (2, 3, 4)}}, {"rows_of": 0, "state": {"canon1": (2, 8)}}],
                     num_blocks=8, max_seqs=2, device="cpu", dtype=torch.float32, block=4, position_limit=10)
    assert kv.rows[2] is kv.rows[0] and kv.rows[1] is None and kv.kscale[0] is None
    assert kv.state[2]["canon1"] is not kv.state[0]["canon1"] and kv.state[1]["gla"].shape == (2, 2, 3, 4)
    kv.reserve(0, 10)
    assert len(kv.blocks_of(0)) == 3
    with pytest.raises(RuntimeError):
        kv.reserve(0, 13)
    kv.free(0)
    assert kv.free_blocks == 8
    with pytest.raises(ValueError):
        HybridCache([{"state": {}}, {"rows_of": 0}], num_blocks=2, max_seqs=1, device="cpu")


@pytest.mark.parametrize("rows,far", [(8, 20.0), (9, 11.0), (16, 100.0), (2, 3.0), (32, 48.0), (7, 29.0)])
def test_distance_table_is_the_oracles_bucket_for_every_distance(rows, far):
    from vllm_i64_amd.dogalorn import distance_bias_table
    rel = torch.arange(rows * 3, dtype=torch.float32).reshape(rows, 3)
    tab = distance_bias_table(rel, far)
    for n in range(int(far) * 3 + 5):
        assert torch.equal(tab[min(n, tab.shape[0] - 1)], rel[R.distance_bucket(n, rows, far)]), n


def test_oracle_recurrence_is_linear_attention_with_cumulative_decays():
    g = torch.Generator().manual_seed(3)
    T, H, d, dv, X = 9, 2, 3, 4, 5
    W = {"q": torch.randn(H * d, X, generator=g), "f": torch.randn(H * d, X, generator=g), "f.b": torch.randn(H * d, generator=g), "lower": torch.rand(H * d, generator=g),
         "v": torch.randn(H * dv, X, generator=g), "norm": torch.ones(dv), "o": torch.eye(H * dv)}
    W = {k: v.double() for k, v in W.items()}
    h = torch.randn(T, X, generator=g).double()
    got = R.hgrn2(W, "", {"heads": H, "dim": d, "vdim": dv}, 0.0, h)
    q = R.silu(h @ W["q"].T).reshape(T, H, d)
    f = (W["lower"] + (1 - W["lower"]) * torch.sigmoid(h @ W["f"].T + W["f.b"])).reshape(T, H, d)
    v = (h @ W["v"].T).reshape(T, H, dv)
    want = torch.zeros(T, H, dv, dtype=torch.float64)
    for t in range(T):
        for s in range(t + 1):
            decay = torch.ones(H, d, dtype=torch.float64)
            for u in range(s + 1, t + 1):
                decay = decay * f[u]
            want[t] += ((q[t] * decay * (1 - f[s])).sum(-1, keepdim=True)) * v[s]
    assert torch.allclose(got, R.rms(want, 0.0).reshape(T, H * dv), atol=1e-10)


def test_oracle_router_keeps_groups_by_corrected_scores_and_weighs_by_plain_ones():
    z = torch.tensor([[2.0, 0.0, 0.1, 0.2, 1.5, 1.4]], dtype=torch.float64)
    corr = torch.tensor([-5.0, 0.0, 0.0, 0.0, 0.0, 0.0], dtype=torch.float64)
    idx, wgt = R.route(z, corr, {"top": 2, "groups": {"count": 3, "keep": 1}, "scale": 2.0})
    assert sorted(idx[0].tolist()) == [4, 5]          # the group of the two runners-up wins although entry 0 has the largest plain score
    s = torch.softmax(z, -1)[0]
    assert torch.allclose(wgt[0].sum(), torch.tensor(2.0, dtype=torch.float64))
    assert torch.allclose(wgt[0], s[idx[0]] / s[idx[0]].sum() * 2.0)
    # all corrected scores negative: the groups that lose count as minus infinity, not as zero
    idx, _ = R.route(z, torch.full((6,), -3.0, dtype=torch.float64), {"top": 2, "groups": {"count": 3, "keep": 1}})
    assert sorted(idx[0].tolist()) == [0, 1]


def test_oracle_pass_through_entries_hand_the_input_on():
    cfg, w = config_of("odd"), {k: v.double() for k, v in make_weights("odd").items()}
    f = cfg["layers"][5]["mlp"]
    h = torch.randn(4, cfg["width"], generator=torch.Generator().manual_seed(1)).double()
    w["l5.mlp.router"] = torch.zeros_like(w["l5.mlp.router"])
    w["l5.mlp.correction"] = torch.tensor([-9.0, -9.0, -9.0, 0.0, 0.0, 0.0], dtype=torch.float64)      # only pass-through entries can win
    out = R.mixture_ff(w, "l5.mlp.", f, h)
    assert torch.allclose(out, h * f["router"]["scale"], atol=1e-12)


def test_oracle_runs_every_shape():
    for name in SHAPES:
        toks = tokens(name, 12, 1)
        rec = []
        lg = R.forward(config_of(name), {k: v.float() for k, v in make_weights(name).items()}, toks, rec)
        assert lg.shape == (12, SHAPES[name]["vocab"]) and len(rec) == len(SHAPES[name]["layers"]) and bool(torch.isfinite(lg).all())
        # causal: a later token changes nothing before it
        lg2 = R.forward(config_of(name), {k: v.float() for k, v in make_weights(name).items()}, toks[:7] + [(toks[7] + 1) % 50] + toks[8:])
        assert torch.equal(lg[:7], lg2[:7]) and not torch.equal(lg[7:], lg2[7:])
