"""Small Fukatar configurations and random weights for the tests (no GPU needed to import)."""
import json

import torch


def rot(base, dims, scaling=None):
    r = {"base": base, "dims": dims}
    if scaling:
        r["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return r


def attn(heads, kv_heads, dim, vdim, r, softcap=None, scale=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if kv_heads is not None:
        m["kv_heads"] = kv_heads
    if r is not None:
        m["rot"] = r
    if softcap:
        m["softcap"] = softcap
    return m


def latent(heads, dim, vdim, kv_rank, scale=None):
    return {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale if scale is not None else dim ** -0.5}


def delta(heads, kv_heads, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def layer(kind, mixer, ff):
    return {"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}


# nothing equal and no size a multiple of four / the branches a config may leave out (no bigram, no caps, no scaling, one tap, all
# heads their own key head, a layer without feed-forward) / sizes the matrix-core kernels take / another order with two taps
SHAPES = {
    "odd": {"architecture": "Fukatar", "vocab": 83, "width": 42, "norm": {"eps": 1e-5}, "logit_softcap": 9.0,
            "embedding": {"scale": 3.0, "bigram": {"buckets": 31, "mul_prev": 13, "mul_cur": 5}},
            "layers": [layer("attention", attn(6, 2, 10, 14, rot(500.0, 6, (4.0, 40, 8.0, 0.5)), softcap=6.0), 50),
                       layer("latent_attention", latent(3, 10, 6, 18, scale=0.4), 34),
                       layer("parallel", {"left": attn(4, 2, 14, 10, rot(90.0, 10), softcap=11.0, scale=0.3), "right": delta(4, 2, 10, 6, 3)}, None),
                       layer("latent_attention", latent(5, 6, 14, 9), 22),
                       layer("attention", attn(3, 3, 18, 6, rot(3000.0, 18, (1.5, 64, 4.0, 1.0)), softcap=25.0, scale=0.2), 30),
                       layer("parallel", {"left": attn(3, 1, 6, 22, rot(10000.0, 2), softcap=4.0), "right": delta(3, 3, 5, 9, 5)}, 26)]},
    "plain": {"architecture": "Fukatar", "vocab": 64, "width": 32,
              "layers": [layer("parallel", {"left": attn(2, None, 8, 8, rot(100.0, 8)), "right": delta(1, 1, 8, 16, 1)}, 40),
                         layer("attention", attn(2, None, 16, 8, rot(100.0, 4)), None),
                         layer("latent_attention", latent(1, 16, 16, 8), 48)]},
    "wide": {"architecture": "Fukatar", "vocab": 200, "width": 128, "norm": {"eps": 1e-6}, "logit_softcap": 30.0,
             "embedding": {"scale": 8.0, "bigram": {"buckets": 257, "mul_prev": 31, "mul_cur": 3}},
             "layers": [layer("latent_attention", latent(4, 32, 48, 64), 160),
                        layer("attention", attn(8, 2, 64, 32, rot(10000.0, 32, (8.0, 128, 16.0, 2.0)), softcap=50.0), 192),
                        layer("parallel", {"left": attn(4, 2, 32, 64, rot(5000.0, 16), softcap=15.0), "right": delta(4, 2, 64, 32, 4)}, 96),
                        layer("attention", attn(2, 1, 128, 64, rot(1000.0, 128), softcap=20.0), 64),
                        layer("latent_attention", latent(18, 16, 16, 32), None)]},
    "twotap": {"architecture": "Fukatar", "vocab": 51, "width": 36, "norm": {"eps": 1e-6}, "embedding": {"bigram": {"buckets": 7, "mul_prev": 3, "mul_cur": 11}},
               "layers": [layer("parallel", {"left": attn(6, 3, 8, 4, rot(64.0, 8, (2.0, 16, 2.0, 0.25)), softcap=8.0), "right": delta(2, 1, 17, 3, 2)}, 44),
                          layer("latent_attention", latent(2, 12, 20, 24), None),
                          layer("attention", attn(4, 1, 12, 20, rot(777.0, 8), softcap=3.0), 28)]},
}


def config_of(name):
    return json.loads(json.dumps(SHAPES[name]))


def attention_weights(w, p, m, W, lin, un, gate):
    nq, nk, nv = m["heads"] * m["dim"], m.get("kv_heads", m["heads"]) * m["dim"], m.get("kv_heads", m["heads"]) * m["vdim"]
    w.update({p + "q": lin(nq, W), p + "k": lin(nk, W), p + "v": lin(nv, W), p + "o": lin(W, m["heads"] * m["vdim"])})
    if gate:
        w.update({p + "q.norm": un(0.5, 1.5, nq), p + "k.norm": un(0.5, 1.5, nk), p + "g": lin(m["heads"], W)})


def make_weights(name, seed=0):
    shape = SHAPES[name]
    g = torch.Generator().manual_seed(seed)
    W = shape["width"]
    rn = lambda *s, std=1.0: (torch.randn(*s, generator=g) * std).to(torch.bfloat16)
    un = lambda lo, hi, *s: (torch.rand(tuple(s), generator=g) * (hi - lo) + lo).to(torch.bfloat16)
    lin = lambda o, i: rn(o, i, std=i ** -0.5)
    w = {"embed": rn(shape["vocab"], W, std=0.3), "head": lin(shape["vocab"], W), "final.norm": un(0.5, 1.5, W)}
    bg = (shape.get("embedding") or {}).get("bigram")
    if bg:
        w["bigram"] = rn(bg["buckets"] + 1, W)
    for i, L in enumerate(shape["layers"]):
        p, m = f"l{i}.", L["mixer"]
        w[p + "norm1"], w[p + "shift"] = un(0.5, 1.5, W), un(0.0, 1.0, W)
        if L["mlp"]:
            w.update({p + "norm2": un(0.5, 1.5, W), p + "mlp.up": lin(L["mlp"]["ff"], W), p + "mlp.down": lin(W, L["mlp"]["ff"])})
        if L["type"] == "attention":
            attention_weights(w, p + "mix.", m, W, lin, un, True)
        elif L["type"] == "latent_attention":
            H, r = m["heads"], m["kv_rank"]
            w.update({p + "mix.q": rn(H * m["dim"], W, std=2.0 * W ** -0.5), p + "mix.dkv": lin(r, W), p + "mix.dkv.norm": un(0.5, 1.5, r), p + "mix.uk": lin(H * m["dim"], r),
                      p + "mix.uv": lin(H * m["vdim"], r), p + "mix.sink": rn(H, std=2.0), p + "mix.o": lin(W, H * m["vdim"])})
        else:
            attention_weights(w, p + "mix.left.", m["left"], W, lin, un, False)
            r, rp = m["right"], p + "mix.right."
            rk, rv = r["kv_heads"] * r["dim"], r["heads"] * r["vdim"]
            w.update({rp + "q": lin(rk, W), rp + "k": lin(rk, W), rp + "v": lin(rv, W), rp + "q.conv": rn(rk, r["conv"], std=0.6), rp + "k.conv": rn(rk, r["conv"], std=0.6),
                      rp + "v.conv": rn(rv, r["conv"], std=0.6), rp + "b": lin(r["heads"], W), rp + "a": lin(r["heads"], W), rp + "A_log": un(-3.0, 0.5, r["heads"]),
                      rp + "dt_bias": rn(r["heads"]), rp + "norm": un(0.5, 1.5, r["vdim"]), rp + "g": lin(rv, W), rp + "o": lin(W, rv),
                      p + "mix.left.out": un(0.5, 1.5, W), p + "mix.right.out": un(0.5, 1.5, W)})
    return w


def tokens(name, n, seed):
    return torch.randint(0, SHAPES[name]["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()
