"""Synthetic weights / routing tables / token ids for benchmarks and smoke runs (no checkpoint of the three
registered models is reachable offline).  Protocol: torch CPU generator seeded per purpose; every >=2-D weight
N(0, 0.02) (the config's initializer_range, vllm_i64/models/complexity_deep/config.py:45), norm weights 1;
hash-routing tables per layer from seed 1234 + layer: route 0 = randperm(V) % E (exactly balanced), route 1 a
different, also balanced expert; cyclic tables (v + k) % E otherwise (token_routed_mlp.py:98-107)."""
from __future__ import annotations

from typing import Dict, List

import torch

from .config import ModelConfig


def make_tables(cfg: ModelConfig) -> List[torch.Tensor]:
    V, E = cfg.vocab_size, cfg.num_experts
    out = []
    for layer in range(cfg.num_layers):
        if not cfg.is_moe:
            out.append(torch.zeros(cfg.top_k, V, dtype=torch.long))
        elif not cfg.table_routing:
            ar = torch.arange(V, dtype=torch.long)
            out.append(torch.stack([(ar + k) % E for k in range(cfg.top_k)]))
        else:
            g = torch.Generator().manual_seed(1234 + layer)
            r0 = torch.randperm(V, generator=g) % E
            rows = [r0]
            if cfg.top_k > 1:
                rows.append((r0 + 1 + torch.randperm(V, generator=g) % (E - 1)) % E)
            for k in range(2, cfg.top_k):
                rows.append((rows[1] + k - 1) % E)
            out.append(torch.stack(rows).long())
    return out


def make_weights(cfg: ModelConfig, seed: int = 0, std: float = 0.02) -> Dict[str, torch.Tensor]:
    g = torch.Generator().manual_seed(seed)
    H, kv, hd = cfg.hidden_size, cfg.num_kv_heads * cfg.head_dim, cfg.head_dim

    def rn(*shape):
        return torch.empty(*shape, dtype=torch.float32).normal_(0.0, std, generator=g)

    w: Dict[str, torch.Tensor] = {"embed": rn(cfg.vocab_size, H), "final_norm": torch.ones(H)}
    tables = make_tables(cfg)
    for l in range(cfg.num_layers):
        p = f"l{l}."
        w[p + "ln1"] = torch.ones(H)
        w[p + "qkv"] = rn(H + 2 * kv, H)
        w[p + "q_norm"] = torch.ones(hd)
        w[p + "k_norm"] = torch.ones(hd)
        w[p + "o"] = rn(H, H)
        w[p + "ln2"] = torch.ones(H)
        if cfg.is_moe:
            ei = cfg.expert_inter
            w[p + "exp_gate_up"] = rn(cfg.num_experts, 2 * ei, H)
            w[p + "exp_down"] = rn(cfg.num_experts, H, ei)
            if cfg.shared_intermediate_size:
                S = cfg.shared_intermediate_size
                w[p + "sh_gate_up"] = rn(2 * S, H)
                w[p + "sh_down"] = rn(H, S)
            w[p + "table"] = tables[l]
        else:
            I = cfg.intermediate_size
            w[p + "gate_up"] = rn(2 * I, H)
            w[p + "down"] = rn(H, I)
    return w


def make_token_ids(cfg: ModelConfig, n: int, seed: int = 7, zipf: float = 0.0) -> torch.Tensor:
    """Uniform ids (the benchmark protocol), or with zipf > 0 a Zipf(zipf) distribution over a fixed random permutation of
    the vocabulary (skewed (route, expert) buckets)."""
    g = torch.Generator().manual_seed(seed)
    if zipf <= 0.0:
        return torch.randint(0, cfg.vocab_size, (n,), generator=g, dtype=torch.long)
    ranks = torch.arange(1, cfg.vocab_size + 1, dtype=torch.float64)
    p = ranks.pow(-zipf)
    order = torch.randperm(cfg.vocab_size, generator=torch.Generator().manual_seed(99))
    return order[torch.multinomial(p / p.sum(), n, replacement=True, generator=g)]


def morilorn_config(width: int = 1024, layers: int = 18, heads: int = 16, dim: int = 32, rot_dim: int = 32, vdim: int = 64, kv_rank: int = 256,
                    ff: int = 4096, window: int = 1024, vocab: int = 32000, groups: int = 2):
    """A Morilorn configuration with layers of a real model's proportions (random weights: make_morilorn_weights)."""
    from .config import MorilornConfig
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": (dim + rot_dim) ** -0.5,
             "rot": {"base": 10000.0, "dims": rot_dim}, "mask": {"size": window}}
    layer = {"type": "latent_attention", "mixer": mixer, "mlp": {"kind": "dense", "ff": ff}}
    return MorilornConfig.from_dict({"architecture": "Morilorn", "vocab": vocab, "width": width, "layers": [layer] * layers, "embedding": {"scale": 1.0},
                                     "postln_alpha": 1.0, "norm": {"eps": 1e-6, "groups": groups}, "logit_softcap": 30.0})


def make_morilorn_weights(cfg, seed: int = 0, std: float = 0.02) -> Dict[str, torch.Tensor]:
    """bf16 N(0, std) matrices, norm weights 1, gate biases 0, depth-mix weights 1 / (layers so far)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg.width

    def rn(*shape):
        return torch.empty(*shape, dtype=torch.float32).normal_(0.0, std, generator=g).to(torch.bfloat16)

    one = lambda n: torch.ones(n, dtype=torch.bfloat16)
    w = {"embed": rn(cfg.vocab, W), "head": rn(cfg.vocab, W), "final.norm": one(W)}
    for i, L in enumerate(cfg.layers):
        p, m = f"l{i}.", L.mixer
        w.update({p + "mix.q": rn(m.q_width, W), p + "mix.dkv": rn(m.cache_width, W), p + "mix.dkv.norm": one(m.kv_rank),
                  p + "mix.uk": rn(m.heads * m.dim, m.kv_rank), p + "mix.uv": rn(m.heads * m.vdim, m.kv_rank), p + "mix.g": rn(m.heads * m.vdim, W),
                  p + "mix.o": rn(W, m.heads * m.vdim), p + "rg1": rn(W, W), p + "rg1.b": torch.zeros(W, dtype=torch.bfloat16), p + "norm1": one(W),
                  p + "dwa": torch.full((i + 2,), 1.0 / (i + 2), dtype=torch.bfloat16)})
        if L.mlp is not None:
            w.update({p + "mlp.gate": rn(L.mlp.ff, W), p + "mlp.up": rn(L.mlp.ff, W), p + "mlp.down": rn(W, L.mlp.ff), p + "rg2": rn(W, W),
                      p + "rg2.b": torch.zeros(W, dtype=torch.bfloat16), p + "norm2": one(W)})
    return w


def dogalorn_config(width: int = 1024, blocks: int = 4, ssm_heads: int = 32, ssm_vdim: int = 64, ssm_state: int = 128, heads: int = 16, kv_heads: int = 4,
                    dim: int = 64, chunk: int = 4096, gru_width: int = 1024, ff: int = 4096, streams: int = 2, vocab: int = 32000, rel_rows: int = 32):
    """A Dogalorn configuration with layers of a real model's proportions: `blocks` times (two state-space layers, two layers of
    chunked attention beside a gated recurrence), every layer with a feed-forward (random weights: make_dogalorn_weights)."""
    from .config import DogalornConfig
    mlp = {"kind": "dense", "ff": ff}
    ssm = {"type": "mamba2", "mixer": {"heads": ssm_heads, "vdim": ssm_vdim, "state": ssm_state, "groups": 1, "conv": 4, "norm_groups": 1}, "mlp": mlp}
    par = {"type": "parallel", "mlp": mlp, "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5, "bias_max": float(chunk),
                                                              "mask": {"size": chunk}}, "right": {"width": gru_width}}}
    cfg = DogalornConfig.from_dict({"architecture": "Dogalorn", "vocab": vocab, "width": width, "layers": [ssm, ssm, par, par] * blocks, "streams": streams,
                                    "norm": {"eps": 1e-6}, "logit_scale": 1.0, "embedding": {"bigram": {"buckets": 65521, "mul_prev": 31, "mul_cur": 17}}})
    cfg.rel_rows = rel_rows
    return cfg


def make_dogalorn_weights(cfg, seed: int = 0, std: float = 0.02) -> Dict[str, torch.Tensor]:
    """bf16 N(0, std) matrices, norm weights 1, biases 0, stream weights that start as the ordinary residual (read the mean, write
    to every stream, no mixing), decays exp(-exp(A_log) dt) around 0.9, distance bias 0."""
    g = torch.Generator().manual_seed(seed)
    W, S = cfg.width, cfg.streams

    def rn(*shape):
        return torch.empty(*shape, dtype=torch.float32).normal_(0.0, std, generator=g).to(torch.bfloat16)

    one = lambda *n: torch.ones(*n, dtype=torch.bfloat16)
    zero = lambda *n: torch.zeros(*n, dtype=torch.bfloat16)
    w = {"embed": rn(cfg.vocab, W), "head": rn(cfg.vocab, W), "final.norm": one(())}
    if cfg.bigram is not None:
        w["bigram"] = rn(cfg.bigram.buckets + 1, W)
    for i, L in enumerate(cfg.layers):
        if L.weights_of is not None:
            continue
        p, m = f"l{i}.", L.mixer
        for q in (1, 2) if L.mlp is not None else (1,):
            w[f"{p}norm{q}"] = one(())
            if S:
                w.update({f"{p}hc{q}.in": torch.full((S,), 1.0 / S, dtype=torch.bfloat16), f"{p}hc{q}.out": one(S), f"{p}hc{q}.mix": torch.eye(S, dtype=torch.bfloat16)})
        if L.type == "mamba2":
            w.update({p + "mix.in": rn(m.in_width, W), p + "mix.conv": rn(m.conv_channels, m.conv) * 10, p + "mix.conv.b": zero(m.conv_channels),
                      p + "mix.dt_bias": torch.full((m.heads,), -2.0, dtype=torch.bfloat16), p + "mix.A_log": zero(m.heads), p + "mix.D": one(m.heads),
                      p + "mix.norm": one(m.inner), p + "mix.o": rn(W, m.inner)})
        else:
            a, r = m.left, m.right.width
            nq, nk = a.heads * a.dim, a.kv_heads * a.dim
            w.update({p + "mix.left.q": rn(nq, W), p + "mix.left.k": rn(nk, W), p + "mix.left.q.norm": one(nq), p + "mix.left.k.norm": one(nk),
                      p + "mix.left.rel": zero(getattr(cfg, "rel_rows", 32), a.heads), p + "mix.left.temp": one(a.heads), p + "mix.left.o": rn(W, nq),
                      p + "mix.right.z": rn(r, W), p + "mix.right.z.b": zero(r), p + "mix.right.x": rn(r, W), p + "mix.right.x.b": zero(r),
                      p + "mix.right.g": rn(r, W), p + "mix.right.o": rn(W, r), p + "mix.left.out": one(W), p + "mix.right.out": one(W)})
        if L.mlp is not None:
            w.update({p + "mlp.up": rn(L.mlp.ff, W), p + "mlp.up.b": zero(L.mlp.ff), p + "mlp.down": rn(W, L.mlp.ff), p + "mlp.down.b": zero(W)})
    return w


def zabutar_config(width: int = 1024, blocks: int = 4, rec_heads: int = 8, rec_dim: int = 128, rec_vdim: int = 128, heads: int = 16, kv_heads: int = 4, dim: int = 64,
                   vdim: int = 64, ff: int = 4096, experts: int = 8, top: int = 2, expert_ff: int = 1024, identity: int = 0, groups: int = 4, keep: int = 2,
                   shared_ff: int = 1024, taps: int = 4, vocab: int = 32000, max_positions: int = 4096, rel_rows: int = 32):
    """A Zabutar configuration with layers of a real model's proportions: `blocks` times (recurrent layer with a dense feed-forward,
    attention layer with a mixture of experts, recurrent layer with a mixture, attention layer over the first one's keys and values
    with a dense feed-forward); random weights: make_zabutar_weights."""
    from .config import ZabutarConfig
    dense = {"kind": "dense", "ff": ff}
    moe = {"kind": "moe", "expert": {"ff": expert_ff}, "shared": {"ff": shared_ff},
           "router": {"experts": experts, "top": top, "identity": identity, "scale": 1.0, "groups": {"count": groups, "keep": keep}}}
    rec = {"type": "hgrn2", "mixer": {"heads": rec_heads, "dim": rec_dim, "vdim": rec_vdim}}
    att = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "bias_max": float(max_positions)}
    layers = []
    for b in range(blocks):
        layers += [dict(rec, mlp=dense), {"type": "attention", "mixer": dict(att), "mlp": moe}, dict(rec, mlp=moe),
                   {"type": "attention", "mixer": dict(att, kv_from=4 * b + 1), "mlp": dense}]
    cfg = ZabutarConfig.from_dict({"architecture": "Zabutar", "vocab": vocab, "width": width, "max_positions": max_positions, "norm": {"eps": 1e-6},
                                   "canon": {"taps": taps}, "layers": layers})
    cfg.rel_rows = rel_rows
    return cfg


def make_zabutar_weights(cfg, seed: int = 0, std: float = 0.02) -> Dict[str, torch.Tensor]:
    """bf16 N(0, std) matrices, norm offsets and biases 0, convolution taps small, gate bounds spread over [0, 0.9], distance bias 0,
    a router wide enough that the experts' loads differ from token to token."""
    g = torch.Generator().manual_seed(seed)
    W = cfg.width

    def rn(*shape, s=std):
        return torch.empty(*shape, dtype=torch.float32).normal_(0.0, s, generator=g).to(torch.bfloat16)

    zero = lambda *n: torch.zeros(*n, dtype=torch.bfloat16)
    w = {"embed": rn(cfg.vocab, W), "pos": rn(cfg.max_positions, W), "head": rn(cfg.vocab, W), "final.norm": zero(W)}
    for i, L in enumerate(cfg.layers):
        p, m, f = f"l{i}.", L.mixer, L.mlp
        for q in (1, 2) if f is not None else (1,):
            w.update({f"{p}norm{q}": zero(W), f"{p}norm{q}b": zero(W), f"{p}canon{q}": rn(W, cfg.canon_taps, s=0.1)})
        if L.type == "hgrn2":
            nk, nv = m.heads * m.dim, m.heads * m.vdim
            w.update({p + "mix.q": rn(nk, W), p + "mix.f": rn(nk, W), p + "mix.f.b": zero(nk), p + "mix.lower": (torch.rand(nk, generator=g) * 0.9).to(torch.bfloat16),
                      p + "mix.v": rn(nv, W), p + "mix.norm": torch.ones(m.vdim, dtype=torch.bfloat16), p + "mix.o": rn(W, nv)})
        else:
            w.update({p + "mix.q": rn(m.heads * m.dim, W), p + "mix.rel": zero(getattr(cfg, "rel_rows", 32), m.heads), p + "mix.o": rn(W, m.heads * m.vdim)})
            if m.kv_from is None:
                w.update({p + "mix.k": rn(m.kv_heads * m.dim, W), p + "mix.v": rn(m.kv_heads * m.vdim, W)})
        if f is not None and f.kind == "dense":
            w.update({p + "mlp.up": rn(f.ff, W), p + "mlp.up.b": zero(f.ff), p + "mlp.down": rn(W, f.ff), p + "mlp.down.b": zero(W), p + "mlp.act": zero(2)})
        elif f is not None:
            w.update({p + "mlp.router": rn(f.entries, W, s=0.1), p + "mlp.correction": zero(f.entries)})
            for e in range(f.experts):
                w.update({f"{p}mlp.e{e}.gate": rn(f.ff, W), f"{p}mlp.e{e}.up": rn(f.ff, W), f"{p}mlp.e{e}.down": rn(W, f.ff)})
            if f.shared_ff:
                w.update({p + "mlp.shared.gate": rn(f.shared_ff, W), p + "mlp.shared.up": rn(f.shared_ff, W), p + "mlp.shared.down": rn(W, f.shared_ff)})
    return w


def fukatar_config(width: int = 1024, blocks: int = 4, heads: int = 16, kv_heads: int = 4, dim: int = 64, vdim: int = 64, rot_dims: int = 64, lat_heads: int = 16,
                   lat_dim: int = 64, lat_vdim: int = 64, kv_rank: int = 256, rec_heads: int = 8, rec_kv_heads: int = 4, rec_dim: int = 128, rec_vdim: int = 128,
                   taps: int = 4, ff: int = 4096, vocab: int = 32000):
    """A Fukatar configuration with layers of a real model's proportions: `blocks` times (rotated attention with gated heads, latent
    attention, attention beside a gated delta rule, latent attention), every layer with a dense feed-forward; random weights:
    make_fukatar_weights."""
    from .config import FukatarConfig
    mlp = {"kind": "dense", "ff": ff}
    att = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "softcap": 50.0,
           "rot": {"base": 10000.0, "dims": rot_dims, "scaling": {"factor": 8.0, "original": 2048, "fast": 32.0, "slow": 1.0}}}
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "softcap": 30.0, "rot": {"base": 10000.0, "dims": rot_dims // 2}}
    right = {"heads": rec_heads, "kv_heads": rec_kv_heads, "dim": rec_dim, "vdim": rec_vdim, "conv": taps}
    lat = {"heads": lat_heads, "dim": lat_dim, "vdim": lat_vdim, "kv_rank": kv_rank, "scale": lat_dim ** -0.5}
    layers = []
    for _ in range(blocks):
        layers += [{"type": "attention", "mixer": att, "mlp": mlp}, {"type": "latent_attention", "mixer": lat, "mlp": mlp},
                   {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": mlp}, {"type": "latent_attention", "mixer": lat, "mlp": mlp}]
    return FukatarConfig.from_dict({"architecture": "Fukatar", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "logit_softcap": 30.0,
                                    "embedding": {"scale": width ** 0.5, "bigram": {"buckets": 8191, "mul_prev": 1000003, "mul_cur": 31}}, "layers": layers})


def make_fukatar_weights(cfg, seed: int = 0, std: float = 0.02) -> Dict[str, torch.Tensor]:
    """bf16 N(0, std) matrices, norm weights one, shifts one half, convolution taps small, sinks zero, decays spread over the heads."""
    g = torch.Generator().manual_seed(seed)
    W = cfg.width

    def rn(*shape, s=std):
        return torch.empty(*shape, dtype=torch.float32).normal_(0.0, s, generator=g).to(torch.bfloat16)

    one = lambda *n: torch.ones(*n, dtype=torch.bfloat16)
    w = {"embed": rn(cfg.vocab, W), "head": rn(cfg.vocab, W), "final.norm": one(W)}
    if cfg.bigram is not None:
        w["bigram"] = rn(cfg.bigram.buckets + 1, W)
    for i, L in enumerate(cfg.layers):
        p, m = f"l{i}.", L.mixer
        w.update({p + "norm1": one(W), p + "shift": one(W) * 0.5})
        if L.mlp is not None:
            w.update({p + "norm2": one(W), p + "mlp.up": rn(L.mlp.ff, W), p + "mlp.down": rn(W, L.mlp.ff)})
        if L.type == "latent_attention":
            H, r = m.heads, m.kv_rank
            w.update({p + "mix.q": rn(H * m.dim, W), p + "mix.dkv": rn(r, W), p + "mix.dkv.norm": one(r), p + "mix.uk": rn(H * m.dim, r), p + "mix.uv": rn(H * m.vdim, r),
                      p + "mix.sink": torch.zeros(H, dtype=torch.bfloat16), p + "mix.o": rn(W, H * m.vdim)})
            continue
        a, ap = (m, p + "mix.") if L.type == "attention" else (m.left, p + "mix.left.")
        nq, nk, nv = a.heads * a.dim, a.kv_heads * a.dim, a.kv_heads * a.vdim
        w.update({ap + "q": rn(nq, W), ap + "k": rn(nk, W), ap + "v": rn(nv, W), ap + "o": rn(W, a.heads * a.vdim)})
        if L.type == "attention":
            w.update({ap + "q.norm": one(nq), ap + "k.norm": one(nk), ap + "g": rn(a.heads, W)})
        else:
            r, rp = m.right, p + "mix.right."
            rk, rv = r.kv_heads * r.dim, r.heads * r.vdim
            w.update({rp + "q": rn(rk, W), rp + "k": rn(rk, W), rp + "v": rn(rv, W), rp + "q.conv": rn(rk, r.conv, s=0.3), rp + "k.conv": rn(rk, r.conv, s=0.3),
                      rp + "v.conv": rn(rv, r.conv, s=0.3), rp + "b": rn(r.heads, W), rp + "a": rn(r.heads, W),
                      rp + "A_log": torch.linspace(-4.0, 0.0, r.heads).to(torch.bfloat16), rp + "dt_bias": torch.zeros(r.heads, dtype=torch.bfloat16),
                      rp + "norm": one(r.vdim), rp + "g": rn(rv, W), rp + "o": rn(W, rv), p + "mix.left.out": one(W), p + "mix.right.out": one(W)})
    return w
