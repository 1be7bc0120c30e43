"""Small Zabutar configurations and random weights for the tests (no GPU needed to import)."""
import json

import torch


def hgrn(heads, dim, vdim):
    return {"type": "hgrn2", "mixer": {"heads": heads, "dim": dim, "vdim": vdim}}


def attn(heads, kv_heads, dim, vdim, scale=None, bias_max=20, rel_rows=8, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5, "bias_max": bias_max}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "_rel_rows": rel_rows}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top, identity=0, groups=None, scale=1.0, shared=0):
    r = {"experts": experts, "top": top, "scale": scale}
    if identity:
        r["identity"] = identity
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    d = {"kind": "moe", "expert": {"ff": ff}, "router": r}
    if shared:
        d["shared"] = {"ff": shared}
    return d


def layer(mix, ff):
    d = dict(mix)
    d["mlp"] = ff
    return d


# nothing equal and nothing a power of two / the branches that a config may leave out / sizes that the matrix-core kernels take /
# sizes that fit no 16-byte access (width, head sizes and feed-forward sizes that are no multiples of four)
SHAPES = {
    "odd": {"architecture": "Zabutar", "vocab": 83, "width": 40, "max_positions": 300, "norm": {"eps": 1e-5}, "canon": {"taps": 3},
            "layers": [layer(hgrn(3, 10, 6), dense(36)),
                       layer(attn(6, 2, 10, 14, rel_rows=9, bias_max=11), moe(12, 5, 2, identity=1, groups=(3, 2), scale=0.7, shared=20)),
                       layer(attn(6, 2, 10, 14, rel_rows=7, bias_max=29, kv_from=1), None),
                       layer(hgrn(2, 14, 5), moe(9, 4, 1)),
                       layer(attn(4, 4, 8, 8, rel_rows=4, bias_max=9, scale=0.21), dense(28)),
                       layer(attn(6, 2, 10, 14, rel_rows=5, bias_max=50, kv_from=1), moe(7, 3, 3, identity=3, groups=(2, 2), scale=2.0))]},
    "plain": {"architecture": "Zabutar", "vocab": 64, "width": 32, "max_positions": 256, "norm": {"eps": 1e-6}, "canon": {"taps": 1},
              "layers": [layer(attn(1, 1, 16, 16, bias_max=40, rel_rows=6), dense(48)), layer(hgrn(1, 8, 8), None),
                         layer(attn(2, 1, 16, 16, bias_max=3, rel_rows=2, kv_from=0), moe(16, 2, 2, shared=16))]},
    "ragged": {"architecture": "Zabutar", "vocab": 51, "width": 42, "max_positions": 200, "norm": {"eps": 1e-6}, "canon": {"taps": 2},
               "layers": [layer(attn(3, 1, 6, 10, rel_rows=3, bias_max=7), moe(10, 3, 2, shared=6)), layer(hgrn(2, 9, 7), dense(30)),
                          layer(attn(3, 1, 6, 10, rel_rows=5, bias_max=19, kv_from=0), dense(18)), layer(hgrn(1, 17, 3), None)]},
    "wide": {"architecture": "Zabutar", "vocab": 200, "width": 128, "max_positions": 512, "norm": {"eps": 1e-6}, "canon": {"taps": 5},
             "layers": [layer(hgrn(4, 64, 32), moe(48, 16, 4, groups=(4, 2), scale=1.3, shared=96)),
                        layer(attn(8, 2, 64, 64, rel_rows=32, bias_max=48), dense(160)),
                        layer(attn(8, 2, 64, 64, rel_rows=12, bias_max=200, kv_from=1), moe(40, 6, 2, identity=2, groups=(4, 3))),
                        layer(attn(2, 1, 32, 128, rel_rows=16, bias_max=100), dense(96)),
                        layer(hgrn(2, 24, 80), dense(64))]},
}


def config_of(name):
    cfg = json.loads(json.dumps(SHAPES[name]))
    for l in cfg["layers"]:
        l.pop("_rel_rows", None)
    return cfg


def make_weights(name, seed=0):
    shape = SHAPES[name]
    g = torch.Generator().manual_seed(seed)
    W, taps = shape["width"], shape["canon"]["taps"]
    rn = lambda *s, std=1.0: (torch.randn(*s, generator=g) * std).to(torch.bfloat16)
    un = lambda lo, hi, *s: (torch.rand(tuple(s), generator=g) * (hi - lo) + lo).to(torch.bfloat16)
    lin = lambda o, i: rn(o, i, std=i ** -0.5)
    w = {"embed": rn(shape["vocab"], W), "pos": rn(shape["max_positions"], W, std=0.5), "head": lin(shape["vocab"], W), "final.norm": un(-0.5, 0.5, W)}
    for i, L in enumerate(shape["layers"]):
        p, m, f = f"l{i}.", L["mixer"], L["mlp"]
        for q in (1, 2) if f else (1,):
            w[f"{p}norm{q}"], w[f"{p}norm{q}b"] = un(-0.5, 0.5, W), un(-0.5, 0.5, W)
            w[f"{p}canon{q}"] = rn(W, taps, std=0.4)
        if L["type"] == "hgrn2":
            nk, nv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            w.update({p + "mix.q": lin(nk, W), p + "mix.f": lin(nk, W), p + "mix.f.b": rn(nk, std=0.5), p + "mix.lower": un(0.0, 0.97, nk), p + "mix.v": lin(nv, W),
                      p + "mix.norm": un(0.5, 1.5, m["vdim"]), p + "mix.o": lin(W, nv)})
        else:
            nq, nk, nv = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            w.update({p + "mix.q": lin(nq, W), p + "mix.rel": rn(L["_rel_rows"], m["heads"]), p + "mix.o": lin(W, m["heads"] * m["vdim"])})
            if "kv_from" not in m:
                w.update({p + "mix.k": lin(nk, W), p + "mix.v": lin(nv, W)})
        if f and f["kind"] == "dense":
            w.update({p + "mlp.up": lin(f["ff"], W), p + "mlp.up.b": rn(f["ff"], std=0.3), p + "mlp.down": lin(W, f["ff"]), p + "mlp.down.b": rn(W, std=0.3),
                      p + "mlp.act": rn(2, std=0.8)})
        elif f:
            r, ff = f["router"], f["expert"]["ff"]
            n = r["experts"] + r.get("identity", 0)
            w.update({p + "mlp.router": rn(n, W, std=2.0 * W ** -0.5), p + "mlp.correction": rn(n, std=0.3)})
            for e in range(r["experts"]):
                w.update({f"{p}mlp.e{e}.gate": lin(ff, W), f"{p}mlp.e{e}.up": lin(ff, W), f"{p}mlp.e{e}.down": lin(W, ff)})
            if f.get("shared"):
                s = f["shared"]["ff"]
                w.update({p + "mlp.shared.gate": lin(s, W), p + "mlp.shared.up": lin(s, W), p + "mlp.shared.down": lin(W, s)})
    return w


def tokens(name, n, seed):
    return torch.randint(0, SHAPES[name]["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()
