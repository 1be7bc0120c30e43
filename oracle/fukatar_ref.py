"""CPU oracle (TEST INFRASTRUCTURE ONLY) of the Fukatar design: a plain, slow restatement of its equations in 64-bit torch, one
function per mechanism, one whole sequence at a time, token-by-token loops for everything recurrent or causal, no cache, no state
object and no code shared with vllm_i64_amd/.  However the product path cuts, batches, pages and slots a sequence, its logits at a
position must agree with this file's.

Notation: T tokens, width w; weights `W[name]` as stored ([out, in] matrices); `m` a mixer's entry of the config; `p` the prefix of
the mixer's tensors.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def layer_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """Centred norm with a weight and no bias."""
    c = x - x.mean(-1, keepdim=True)
    return c / torch.sqrt(c.pow(2).mean(-1, keepdim=True) + eps) * w


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.logaddexp(z, torch.zeros_like(z))


def capped(s: torch.Tensor, cap: Optional[float]) -> torch.Tensor:
    return s if not cap else cap * torch.tanh(s / cap)


# ---- embedding -----------------------------------------------------------------------------------------------------------------
def embedding(W: Dict[str, torch.Tensor], e: dict, tokens: List[int]) -> torch.Tensor:
    """Scaled token row plus the row of a table that a hash of (previous token, token) picks; a sequence's first token takes the
    table's last row."""
    x = W["embed"][tokens] * float(e.get("scale", 1.0))
    b = e.get("bigram")
    if b:
        n = int(b["buckets"])
        rows = [n] + [(tokens[t - 1] * int(b["mul_prev"]) + tokens[t] * int(b["mul_cur"])) % n for t in range(1, len(tokens))]
        x = x + W["bigram"][rows]
    return x


# ---- what a mixer reads: a per-channel blend with the row before ---------------------------------------------------------------
def token_shift(s: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    before = torch.cat([torch.zeros_like(x[:1]), x[:-1]], 0)
    return x + (before - x) * s


# ---- rotations -------------------------------------------------------------------------------------------------------------------
def rotary_frequencies(base: float, dims: int, scaling: Optional[dict] = None):
    """Frequencies f_i, i < dims / 2, and the factor on cosine and sine.  With `scaling` the slow frequencies are divided by its
    factor, the fast ones kept, with a linear ramp between the two pair indices at which `original` positions make `fast` and `slow`
    turns."""
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    if not scaling:
        return torch.tensor(f, dtype=F64), 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])
    at = lambda turns: dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(at(float(scaling["fast"]))), 0)
    hi = min(math.ceil(at(float(scaling["slow"]))), dims - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / factor * ramp + f[i] * (1.0 - ramp))
    return torch.tensor(out, dtype=F64), 0.1 * math.log(factor) + 1.0


def rotate(x: torch.Tensor, pos: torch.Tensor, freq: torch.Tensor, dims: int, interleaved: bool, mult: float = 1.0) -> torch.Tensor:
    """x [T, heads, d]: the first `dims` values of every head turn by pos * freq; pairs are (i, i + dims / 2) or (2i, 2i + 1)."""
    half = dims // 2
    a = pos.to(F64).reshape(-1, 1, 1) * freq.reshape(1, 1, half)
    c, s = torch.cos(a) * mult, torch.sin(a) * mult
    ia = torch.arange(half) * 2 if interleaved else torch.arange(half)
    ib = ia + 1 if interleaved else ia + half
    out = x.clone()
    u, v = x[..., ia], x[..., ib]
    out[..., ia] = u * c - v * s
    out[..., ib] = v * c + u * s
    return out


# ---- softmax attention over grouped key / value heads ----------------------------------------------------------------------------
def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, cap: Optional[float], sink: Optional[torch.Tensor] = None):
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv].  sink [H]: one more term exp(sink) in the denominator, without a value."""
    T, H = q.shape[:2]
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=F64)
    for i in range(T):
        for a in range(H):
            g = a // (H // G)
            s = capped((k[: i + 1, g] @ q[i, a]) * scale, cap)
            if sink is None:
                w = torch.softmax(s, 0)
            else:
                top = torch.maximum(s.max(), sink[a])
                e = torch.exp(s - top)
                w = e / (e.sum() + torch.exp(sink[a] - top))
            out[i, a] = w @ v[: i + 1, g]
    return out


def rotary_attention(W: Dict[str, torch.Tensor], p: str, m: dict, eps: float, h: torch.Tensor) -> torch.Tensor:
    """Whole-row query / key norms, rotation in halves (with scaled frequencies), values rotated by their own position and the sum
    turned back by the query's, capped scores, a sigmoid gate per head."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(T)
    q = rms(h @ W[p + "q"].T, eps) * W[p + "q.norm"]
    k = rms(h @ W[p + "k"].T, eps) * W[p + "k.norm"]
    q, k, v = q.reshape(T, H, d), k.reshape(T, G, d), (h @ W[p + "v"].T).reshape(T, G, dv)
    rot = m.get("rot")
    if rot:
        f, mult = rotary_frequencies(float(rot["base"]), int(rot["dims"]), rot.get("scaling"))
        q, k = rotate(q, pos, f, int(rot["dims"]), False, mult), rotate(k, pos, f, int(rot["dims"]), False, mult)
        fv, _ = rotary_frequencies(float(rot["base"]), dv)
        v = rotate(v, pos, fv, dv, False)
    o = causal_attention(q, k, v, float(m["scale"]), m.get("softcap"))
    if rot:
        o = rotate(o, -pos, fv, dv, False)
    o = o * torch.sigmoid(h @ W[p + "g"].T).unsqueeze(-1)
    return o.reshape(T, H * dv) @ W[p + "o"].T


def unit_norm_attention(W: Dict[str, torch.Tensor], p: str, m: dict, eps: float, h: torch.Tensor) -> torch.Tensor:
    """Rotation in interleaved pairs, then queries and keys divided by their root mean square per head; capped scores."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(T)
    q, k, v = (h @ W[p + "q"].T).reshape(T, H, d), (h @ W[p + "k"].T).reshape(T, G, d), (h @ W[p + "v"].T).reshape(T, G, dv)
    rot = m.get("rot")
    if rot:
        f, mult = rotary_frequencies(float(rot["base"]), int(rot["dims"]), rot.get("scaling"))
        q, k = rotate(q, pos, f, int(rot["dims"]), True, mult), rotate(k, pos, f, int(rot["dims"]), True, mult)
    o = causal_attention(rms(q, eps), rms(k, eps), v, float(m["scale"]), m.get("softcap"))
    return o.reshape(T, H * dv) @ W[p + "o"].T


def latent_attention(W: Dict[str, torch.Tensor], p: str, m: dict, eps: float, h: torch.Tensor) -> torch.Tensor:
    """Keys and values of every head are maps of one normed low-rank row per token; no positions; a learned sink per head."""
    T = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ W[p + "q"].T).reshape(T, H, d)
    c = rms(h @ W[p + "dkv"].T, eps) * W[p + "dkv.norm"]
    k, v = (c @ W[p + "uk"].T).reshape(T, H, d), (c @ W[p + "uv"].T).reshape(T, H, dv)
    o = causal_attention(q, k, v, float(m["scale"]), None, sink=W[p + "sink"])
    return o.reshape(T, H * dv) @ W[p + "o"].T


# ---- gated delta rule --------------------------------------------------------------------------------------------------------------
def short_convolution(w: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """Per channel over time, the last column of w [channels, taps] on the current token, nothing before the first token; then silu."""
    T, taps = x.shape[0], w.shape[1]
    out = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1 - j)
            if s >= 0:
                out[t] = out[t] + w[:, j] * x[s]
    return silu(out)


def delta_rule(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, beta: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    """q, k [T, H, d], v [T, H, dv], beta, g [T, H]: S decays by g, is corrected towards v along k with strength beta, and is read by q
    after the write."""
    T, H, d = q.shape
    dv = v.shape[-1]
    S = torch.zeros(H, d, dv, dtype=F64)
    o = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        S = S * g[t].reshape(H, 1, 1)
        u = beta[t].reshape(H, 1) * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
        S = S + k[t].unsqueeze(-1) * u.unsqueeze(-2)
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return o


def gated_delta(W: Dict[str, torch.Tensor], p: str, m: dict, eps: float, h: torch.Tensor) -> torch.Tensor:
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"])
    q = short_convolution(W[p + "q.conv"], h @ W[p + "q"].T).reshape(T, G, d)
    k = short_convolution(W[p + "k.conv"], h @ W[p + "k"].T).reshape(T, G, d)
    v = short_convolution(W[p + "v.conv"], h @ W[p + "v"].T).reshape(T, H, dv)
    unit = lambda x: x / torch.sqrt(x.pow(2).sum(-1, keepdim=True) + 1e-6)
    own = torch.arange(H) // (H // G)
    q, k = (unit(q) * d ** -0.5)[:, own], unit(k)[:, own]
    beta = torch.sigmoid(h @ W[p + "b"].T)
    g = torch.exp(-torch.exp(W[p + "A_log"]) * softplus(h @ W[p + "a"].T + W[p + "dt_bias"]))
    o = delta_rule(q, k, v, beta, g)
    o = rms(o, eps) * W[p + "norm"] * silu(h @ W[p + "g"].T).reshape(T, H, dv)
    return o.reshape(T, H * dv) @ W[p + "o"].T


def parallel_mixer(W: Dict[str, torch.Tensor], p: str, m: dict, eps: float, h: torch.Tensor) -> torch.Tensor:
    left = unit_norm_attention(W, p + "left.", m["left"], eps, h)
    right = gated_delta(W, p + "right.", m["right"], eps, h)
    return 0.5 * (rms(left, eps) * W[p + "left.out"] + rms(right, eps) * W[p + "right.out"])


# ---- feed-forward --------------------------------------------------------------------------------------------------------------
def dense_ff(W: Dict[str, torch.Tensor], p: str, h: torch.Tensor) -> torch.Tensor:
    return torch.relu(h @ W[p + "up"].T).pow(2) @ W[p + "down"].T


MIXERS = {"attention": rotary_attention, "latent_attention": latent_attention, "parallel": parallel_mixer}


# ---- the model -----------------------------------------------------------------------------------------------------------------
def forward(config: dict, weights: Dict[str, torch.Tensor], tokens: List[int], layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence (64-bit).  layers_out: a list that receives the residual after every layer."""
    W = {k: v.to(F64) for k, v in weights.items()}
    eps = float((config.get("norm") or {}).get("eps", 1e-6))
    x = embedding(W, config.get("embedding") or {}, tokens)
    for i, L in enumerate(config["layers"]):
        p = f"l{i}."
        h = token_shift(W[p + "shift"], x)
        x = x + layer_norm(MIXERS[L["type"]](W, p + "mix.", L["mixer"], eps, h), W[p + "norm1"], eps)
        if L.get("mlp"):
            x = x + layer_norm(dense_ff(W, p + "mlp.", x), W[p + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    z = layer_norm(x, W["final.norm"], eps) @ W["head"].T
    return capped(z, config.get("logit_softcap"))
