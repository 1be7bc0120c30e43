"""CPU oracle (TEST INFRASTRUCTURE ONLY) of the Zabutar design: a plain, slow restatement of its equations in 64-bit torch, one
function per mechanism, one whole sequence at a time, token-by-token loops for everything recurrent or causal, no cache, no state
object and no code shared with vllm_i64_amd/.  However the product path cuts, batches, pages and slots a sequence, its logits at a
position must agree with this file's.

Notation: T tokens, width w; weights `W[name]` as stored ([out, in] matrices); `m` a layer's 'mixer' entry of the config, `f` its
'mlp' entry.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.logaddexp(z, torch.zeros_like(z))


def offset_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose stored weight is the distance from one."""
    return rms(x, eps) * (1.0 + w)


# ---- embedding -----------------------------------------------------------------------------------------------------------------
def embedding(W: Dict[str, torch.Tensor], tokens: List[int]) -> torch.Tensor:
    """Token row plus the learned row of the token's position."""
    return W["embed"][tokens] + W["pos"][: len(tokens)]


# ---- the short convolution in front of every sublayer ------------------------------------------------------------------------------
def input_convolution(w: torch.Tensor, h: torch.Tensor) -> torch.Tensor:
    """h_t + sum_j w[:, j] h_(t - taps + 1 + j) per channel, nothing before the first token.  w [width, taps]."""
    T, taps = h.shape[0], w.shape[1]
    out = h.clone()
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] = out[t] + w[:, j] * h[s]
    return out


# ---- gated linear recurrence whose forget gate also sets the write strength --------------------------------------------------------
def hgrn2(W: Dict[str, torch.Tensor], p: str, m: dict, eps: float, h: torch.Tensor) -> torch.Tensor:
    T = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(h @ W[p + "q"].T).reshape(T, H, d)
    low = W[p + "lower"]
    f = (low + (1.0 - low) * torch.sigmoid(h @ W[p + "f"].T + W[p + "f.b"])).reshape(T, H, d)
    v = (h @ W[p + "v"].T).reshape(T, H, dv)
    S = torch.zeros(H, d, dv, dtype=F64)
    o = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        S = f[t].unsqueeze(-1) * S + (1.0 - f[t]).unsqueeze(-1) * v[t].unsqueeze(-2)
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    o = rms(o, eps) * W[p + "norm"]
    return o.reshape(T, H * dv) @ W[p + "o"].T


# ---- attention with a learned bias by bucketed distance ----------------------------------------------------------------------------
def distance_bucket(n: int, rows: int, far: float) -> int:
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def keys_and_values(W: Dict[str, torch.Tensor], p: str, h: torch.Tensor):
    return h @ W[p + "k"].T, h @ W[p + "v"].T


def biased_attention(W: Dict[str, torch.Tensor], p: str, m: dict, h: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """k, v [T, kv_heads * dim / vdim]: this layer's own, or those of the layer it takes them from."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"])
    q = (h @ W[p + "q"].T).reshape(T, H, d)
    k, v = k.reshape(T, G, d), v.reshape(T, G, dv)
    rel = W[p + "rel"]
    out = torch.zeros(T, H, dv, dtype=F64)
    for i in range(T):
        rows = [distance_bucket(i - j, rel.shape[0], float(m["bias_max"])) for j in range(i + 1)]
        for a in range(H):
            g = a // (H // G)
            s = (k[: i + 1, g] @ q[i, a]) * float(m["scale"]) + rel[rows, a]
            out[i, a] = torch.softmax(s, 0) @ v[: i + 1, g]
    return out.reshape(T, H * dv) @ W[p + "o"].T


# ---- feed-forward --------------------------------------------------------------------------------------------------------------
def xielu(z: torch.Tensor, pq: torch.Tensor) -> torch.Tensor:
    a, b = softplus(pq[0]), 0.5 + softplus(pq[1])
    return torch.where(z > 0, a * z * z + 0.5 * z, b * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z)


def dense_ff(W: Dict[str, torch.Tensor], p: str, h: torch.Tensor) -> torch.Tensor:
    return xielu(h @ W[p + "up"].T + W[p + "up.b"], W[p + "act"]) @ W[p + "down"].T + W[p + "down.b"]


def gated_expert(W: Dict[str, torch.Tensor], p: str, h: torch.Tensor) -> torch.Tensor:
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(z: torch.Tensor, correction: torch.Tensor, r: dict):
    """z [T, experts + identity] router logits -> chosen indices [T, top] and their weights."""
    s = torch.softmax(z, -1)
    choice = s + correction
    n = z.shape[-1]
    groups = r.get("groups")
    if groups:
        size = n // int(groups["count"])
        best = choice.reshape(-1, int(groups["count"]), size).max(-1).values
        kept = best.topk(int(groups["keep"]), -1).indices
        allowed = torch.zeros_like(best, dtype=torch.bool).scatter_(1, kept, True).repeat_interleave(size, 1)
        choice = torch.where(allowed, choice, torch.full_like(choice, -math.inf))
    idx = choice.topk(int(r["top"]), -1).indices
    wgt = s.gather(1, idx)
    return idx, wgt / (wgt.sum(-1, keepdim=True) + 1e-20) * float(r.get("scale", 1.0))


def mixture_ff(W: Dict[str, torch.Tensor], p: str, f: dict, h: torch.Tensor, forced: Optional[torch.Tensor] = None, chosen: Optional[list] = None) -> torch.Tensor:
    """forced [T, top]: entries to use instead of the router's own choice (their weights still come from the router's scores) - for
    comparisons with an implementation in lower precision, where a close call may fall the other way; chosen receives the choice."""
    r = f["router"]
    E = int(r["experts"])
    z = h @ W[p + "router"].T
    idx, wgt = route(z, W[p + "correction"], r)
    if forced is not None:
        idx = forced.to(torch.int64)
        wgt = torch.softmax(z, -1).gather(1, idx)
        wgt = wgt / (wgt.sum(-1, keepdim=True) + 1e-20) * float(r.get("scale", 1.0))
    if chosen is not None:
        chosen.append(idx)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, g in zip(idx[t].tolist(), wgt[t]):
            out[t] += g * (gated_expert(W, f"{p}e{e}.", h[t:t + 1])[0] if e < E else h[t])      # the entries past the experts hand the input through
    if f.get("shared"):
        out = out + gated_expert(W, p + "shared.", h)
    return out


# ---- the whole model ---------------------------------------------------------------------------------------------------------------
def forward(cfg: dict, W32: Dict[str, torch.Tensor], tokens: List[int], record: Optional[list] = None, routes: Optional[dict] = None,
            chosen: Optional[dict] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence; record (a list) receives the residual after every layer; routes: layer -> entries [T, top] to
    use instead of the router's choice; chosen (a dict) receives every mixture layer's choice."""
    W = {k: v.to(F64) for k, v in W32.items()}
    eps = float(cfg["norm"]["eps"])
    x = embedding(W, tokens)
    kv = {}
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = input_convolution(W[p + "canon1"], offset_norm(x, W[p + "norm1"], eps))
        m = L["mixer"]
        if L["type"] == "hgrn2":
            y = hgrn2(W, p + "mix.", m, eps, h)
        elif L["type"] == "attention":
            if m.get("kv_from") is None:
                kv[i] = keys_and_values(W, p + "mix.", h)
            y = biased_attention(W, p + "mix.", m, h, *kv[i if m.get("kv_from") is None else int(m["kv_from"])])
        else:
            raise ValueError(L["type"])
        x = x + offset_norm(y, W[p + "norm1b"], eps)
        f = L.get("mlp")
        if f:
            h = input_convolution(W[p + "canon2"], offset_norm(x, W[p + "norm2"], eps))
            if f.get("kind", "dense") == "dense":
                y = dense_ff(W, p + "mlp.", h)
            else:
                got = []
                y = mixture_ff(W, p + "mlp.", f, h, forced=(routes or {}).get(i), chosen=got)
                if chosen is not None:
                    chosen[i] = got[0]
            x = x + offset_norm(y, W[p + "norm2b"], eps)
        if record is not None:
            record.append(x.clone())
    return offset_norm(x, W["final.norm"], eps) @ W["head"].T
