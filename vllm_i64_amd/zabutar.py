"""Runner of the Zabutar design on one MI355X: a decoder with an RMS norm in front of AND behind every sublayer (weights stored as
distances from one), learned absolute positions, a short causal convolution added to every sublayer's input, and per layer one of two
mixers and one of two feed-forwards:

  x0 = embed[token] + pos[position]
  sublayer:  h = rms(x) (1 + w);  h <- h + conv(h) over the last `taps` positions (the last taps - 1 inputs are per-sequence state);
             x <- x + rms(f(h)) (1 + w_b)
  hgrn2      q = silu(W_q h), f = l + (1 - l) sigmoid(W_f h + b), v = W_v h;  per head S <- diag(f) S + (1 - f) v^T, o = S^T q;
             RMS norm of every head's o, out-projection
  attention  grouped key / value heads, no rotation, score = q . k * scale + rel[bucket(i - j), head], causal softmax; a layer may
             attend over the keys and values that an earlier layer cached instead of projecting its own
  dense      W_down act(W_up h + b) + b, act(z) = a z^2 + z / 2 for z > 0, b' (exp(z) - 1 - z) + z / 2 otherwise
  moe        router softmax over experts + pass-through entries, corrected choice, groups of neighbours, top-k, renormalised weights
             times a scale; experts W_down (silu(W_gate h) * W_up h); a shared expert for every token
  logits = head . (rms(x) (1 + w))

The residual, norms, convolution inputs, gates, the recurrence and its state, router, scores and softmax are fp32 in both modes;
"bfloat16" rounds the inputs of the matrix products to bf16 (fp32 sums on the matrix cores) and keeps cached keys and values in bf16,
"float32" keeps everything in 32 bits.  torch holds memory and streams; every arithmetic step is a libi64hip_dense.so kernel.  The step
interface is I64MoEModel's, so the same engine, scheduler and decoders drive it."""
from __future__ import annotations

import math
import os
from typing import Dict, List, Optional

import torch

from . import ops_dense as D
from .config import ZabutarConfig
from .dogalorn import distance_bias_table
from .model import attention_segments
from .paged_cache import HybridCache


def _softplus(x: float) -> float:
    return max(x, 0.0) + math.log1p(math.exp(-abs(x)))


class _StepBuffers:
    def __init__(self, model: "ZabutarModel", n: int, m: int):
        f32 = dict(dtype=torch.float32, device=model.device)
        i32 = dict(dtype=torch.int32, device=model.device)
        W = model.cfg.width
        self.streams = torch.empty(1, n, W, **f32)              # the residual (one stream of the multi-stream kernel)
        self.h = torch.empty(n, W, **f32)                       # the normed input of the current sublayer
        self.hc = torch.empty(n, W, **f32)                      # ... with its convolution added
        self.y = torch.empty(n, W, **f32)
        self.y2 = torch.empty(n, W, **f32)
        self.p = torch.empty(n * model.max_proj, **f32)         # everything projected from the sublayer input
        self.a = torch.empty(n * model.max_a, **f32)            # queries / recurrence output
        self.b = torch.empty(n * model.max_a, **f32)            # attention output / normed recurrence output
        self.act = torch.empty(n * max(model.max_act, 1), **f32)
        self.sact = torch.empty(n * max(model.max_shared, 1), **f32)
        t = model.max_top
        self.ey = torch.empty(n * t, W, **f32) if t else None   # the chosen experts' outputs, grouped by expert
        self.idx = torch.empty(n * max(t, 1), **i32)
        self.wgt = torch.empty(n * max(t, 1), **f32)
        self.pair_token = torch.empty(n * max(t, 1), **i32)
        self.pair_row = torch.empty(n * max(t, 1), **i32)
        self.group_off = torch.empty(model.max_experts + 1, **i32)
        self.xf = torch.empty(m, W, **f32)
        self.logits = torch.empty(m, model.cfg.vocab, **f32)
        self.attn_ws: Dict[tuple, torch.Tensor] = {}


class ZabutarModel:
    MAX_BUFFER_SETS = int(os.environ.get("I64H_MAX_BUFFER_SETS", "8"))
    ATTN_MAX_SEGMENTS = 4
    ATTN_WAVES = {64: 3072, 128: 2048, 256: 1024}     # waves a decode-sized attention launch aims at, by the width of a key head's cached part

    def __init__(self, cfg: ZabutarConfig, weights: Dict[str, torch.Tensor], device="cuda:0", dtype: str = "bfloat16", max_seqs: int = 4,
                 num_kv_blocks: int = 256, kv_block: int = 16, cache_dtype: Optional[torch.dtype] = None):
        if dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype {dtype}: bfloat16 or float32")
        self.cfg, self.device, self.dtype = cfg, torch.device(device), dtype
        self.exact = dtype == "float32"
        dev = self.device
        bf = lambda t: t.to(device=dev, dtype=torch.bfloat16).contiguous()
        f = lambda t: t.to(device=dev, dtype=torch.float32).contiguous()
        W = cfg.width

        def need(name, shape):
            if name not in weights:
                raise KeyError(f"tensor '{name}' is missing")
            if tuple(weights[name].shape) != tuple(shape):
                raise ValueError(f"'{name}': shape {tuple(weights[name].shape)}, config says {tuple(shape)}")
            return weights[name]

        self._one_plus = lambda t: f(1.0 + t.to(torch.float32))      # norm weights are stored as distances from one
        self.embed, self.head = bf(need("embed", (cfg.vocab, W))), bf(need("head", (cfg.vocab, W)))
        self.pos = bf(need("pos", (cfg.max_positions, W)))
        self.final_norm = self._one_plus(need("final.norm", (W,)))
        self.ones1 = torch.ones(1, dtype=torch.float32, device=dev)
        self.layers: List[dict] = [self._load_layer(i, L, weights, need, bf, f) for i, L in enumerate(cfg.layers)]
        specs = []
        carried = max(cfg.canon_taps - 1, 0)
        for i, L in enumerate(cfg.layers):
            state = {"canon1": (carried, W)} if carried else {}
            if L.mlp is not None and carried:
                state["canon2"] = (carried, W)
            m = L.mixer
            if L.type == "hgrn2":
                state["gla"] = (m.heads, m.vdim, m.dim)
                specs.append({"state": state})
            elif m.kv_from is not None:
                specs.append({"rows_of": m.kv_from, "state": state})
            else:
                specs.append({"rows": m.kv_heads * (m.vdim + m.dim), "kscale": False, "state": state})
        self.max_proj = max(d["n_in"] for d in self.layers)
        self.max_a = max(d["n_a"] for d in self.layers)
        moes = [l.mlp for l in cfg.layers if l.mlp is not None and l.mlp.kind == "moe"]
        self.max_top = max([m.top for m in moes] or [0])
        self.max_experts = max([m.experts for m in moes] or [0])
        self.max_shared = max([m.shared_ff for m in moes] or [0])
        self.max_act = max([l.mlp.ff for l in cfg.layers if l.mlp is not None and l.mlp.kind == "dense"] + [m.ff * m.top for m in moes] +
                           [0])
        if cache_dtype is None:
            cache_dtype = torch.float32 if self.exact else torch.bfloat16
        self.kv = HybridCache(specs, num_kv_blocks, max_seqs, dev, dtype=cache_dtype, block=kv_block, position_limit=cfg.max_positions)
        self._bufs: Dict[tuple, _StepBuffers] = {}
        self._pinned: set = set()
        self._arange: Dict[int, torch.Tensor] = {}

    # ---- load-time layout work: one weight for everything that reads the sublayer input; small vectors in fp32 ----
    def _load_layer(self, i: int, L, weights, need, bf, f) -> dict:
        cfg, W, p = self.cfg, self.cfg.width, f"l{i}."
        d = dict(type=L.type, m=L.mixer, mlp=L.mlp)
        for q in ((1, 2) if L.mlp is not None else (1,)):
            d[f"norm{q}"] = self._one_plus(need(f"{p}norm{q}", (W,)))
            d[f"norm{q}b"] = self._one_plus(need(f"{p}norm{q}b", (W,)))
            d[f"canon{q}"] = f(need(f"{p}canon{q}", (W, cfg.canon_taps)))
        m = L.mixer
        if L.type == "hgrn2":
            nk, nv = m.heads * m.dim, m.heads * m.vdim
            d["w_in"] = bf(torch.cat([need(p + "mix.q", (nk, W)), need(p + "mix.f", (nk, W)), need(p + "mix.v", (nv, W))], 0))
            d["b_in"] = f(torch.cat([torch.zeros(nk), need(p + "mix.f.b", (nk,)).float(), torch.zeros(nv)]))
            d["lower"] = f(need(p + "mix.lower", (nk,)))
            d["norm"] = f(need(p + "mix.norm", (m.vdim,)).float().repeat(m.heads))      # the same weights for every head
            d["o"] = bf(need(p + "mix.o", (W, nv)))
            d["n_in"], d["n_a"] = 2 * nk + nv, nv
        else:
            nq, nk, nv = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
            if m.kv_from is None:
                d["w_in"] = bf(torch.cat([need(p + "mix.q", (nq, W)), need(p + "mix.k", (nk, W)), need(p + "mix.v", (nv, W))], 0))
                d["n_in"] = nq + nk + nv
            else:
                d["w_in"] = bf(need(p + "mix.q", (nq, W)))
                d["n_in"] = nq
            name = p + "mix.rel"
            if name not in weights or weights[name].dim() != 2:
                raise KeyError(f"tensor '{name}' is missing or is no table")
            rel = need(name, (weights[name].shape[0], m.heads))      # the number of distance buckets is the table's height
            d["bias"] = distance_bias_table(rel.float(), m.bias_max).to(self.device)
            d["o"] = bf(need(p + "mix.o", (W, m.heads * m.vdim)))
            d["n_a"] = m.heads * (m.vdim + m.dim)
        ff = L.mlp
        if ff is not None and ff.kind == "dense":
            d["up"], d["up_b"] = bf(need(p + "mlp.up", (ff.ff, W))), f(need(p + "mlp.up.b", (ff.ff,)))
            d["down"], d["down_b"] = bf(need(p + "mlp.down", (W, ff.ff))), f(need(p + "mlp.down.b", (W,)))
            a, b = (float(v) for v in need(p + "mlp.act", (2,)).float())
            d["act_a"], d["act_b"] = _softplus(a), 0.5 + _softplus(b)
        elif ff is not None:
            d["router"] = bf(need(p + "mlp.router", (ff.entries, W)))
            d["correction"] = f(need(p + "mlp.correction", (ff.entries,)))
            # per expert [gate rows; up rows], all experts stacked: one grouped launch for the pair, one for the way down
            d["gate_up"] = bf(torch.stack([torch.cat([need(f"{p}mlp.e{e}.gate", (ff.ff, W)), need(f"{p}mlp.e{e}.up", (ff.ff, W))], 0) for e in range(ff.experts)]))
            d["e_down"] = bf(torch.stack([need(f"{p}mlp.e{e}.down", (W, ff.ff)) for e in range(ff.experts)]))
            if ff.shared_ff:
                s = ff.shared_ff
                d["s_gate_up"] = bf(torch.cat([need(p + "mlp.shared.gate", (s, W)), need(p + "mlp.shared.up", (s, W))], 0))
                d["s_down"] = bf(need(p + "mlp.shared.down", (W, s)))
        return d

    # ---- step buffers (same policy as the other runners: the most recent row counts are kept, pinned sets stay for captured graphs) ----
    def buffers(self, n: int, m: int) -> _StepBuffers:
        key = (n, m)
        B = self._bufs.pop(key, None)
        if B is None:
            B = _StepBuffers(self, n, m)
        self._bufs[key] = B
        loose = [k for k in self._bufs if k not in self._pinned and k != key]
        for k in loose[:max(0, len(loose) + 1 - self.MAX_BUFFER_SETS)]:
            del self._bufs[k]
        return B

    def pin_buffers(self, n: int, m: int) -> None:
        self.buffers(n, m)
        self._pinned.add((n, m))

    def check_sync(self, force: bool = True):
        """No launch of this runner waits on a grid barrier: nothing to read back."""

    def snapshot_state(self):
        """The per-sequence recurrent state, for a caller that runs a step which must not count (a warm-up before a graph capture)."""
        return self.kv.snapshot()

    def restore_state(self, held) -> None:
        self.kv.restore(held)

    def _runs(self, n: int, slot_ids: torch.Tensor, tokens_per_seq, rows_are_slots: bool):
        """First rows of the runs of consecutive rows of one sequence, int32 [runs + 1] on the device, and their number."""
        if rows_are_slots:
            t = self._arange.get(n)
            if t is None:
                t = self._arange[n] = torch.arange(n + 1, dtype=torch.int32, device=self.device)
            return t, n
        if tokens_per_seq is None:      # (a caller that does not say how its rows are grouped: read it off the slot ids)
            s = slot_ids.tolist()
            tokens_per_seq, k = [], 0
            for j in range(1, n + 1):
                if j == n or s[j] != s[j - 1]:
                    tokens_per_seq.append(j - k)
                    k = j
        starts = [0]
        for t in tokens_per_seq:
            if int(t) > 0:
                starts.append(starts[-1] + int(t))
        if starts[-1] != n:
            raise ValueError(f"tokens_per_seq adds up to {starts[-1]} rows, the step has {n}")
        return torch.tensor(starts, dtype=torch.int32).to(self.device), len(starts) - 1

    # ---- mixers and feed-forwards: the sublayer input is B.hc; the result lands in B.y ----
    def _hgrn2(self, B, d, l, n, positions, slot_ids, kvc, seg, nseg) -> None:
        m, ex = d["m"], self.exact
        nk, nv = m.heads * m.dim, m.heads * m.vdim
        P = B.p[: n * d["n_in"]].view(n, d["n_in"])
        D.linear(B.hc, d["w_in"], P, exact=ex, bias=d["b_in"])
        cols = dict(q_off=0, f_off=nk, v_off=2 * nk, heads=m.heads, dim=m.dim, vdim=m.vdim, n=n)
        D.gla_gates(P, lower=d["lower"], q_act=True, **cols)
        O = B.a[: n * nv].view(n, nv)
        D.gla_scan(P, seg_start=seg, nseg=nseg, positions=positions, slot_ids=slot_ids, state=kvc.state[l]["gla"], out=O, **cols)
        G = B.b[: n * nv].view(n, nv)
        D.gate_norm(O, d["norm"], G, groups=m.heads, eps=self.cfg.norm_eps, n=n)
        D.linear(G, d["o"], B.y, exact=ex)

    def _attention(self, B, d, l, n, positions, slot_ids, kvc, runs, ctx_hint) -> None:
        m, ex = d["m"], self.exact
        nq, nk, gs = m.heads * m.dim, m.kv_heads * m.dim, m.vdim + m.dim
        P = B.p[: n * d["n_in"]].view(n, d["n_in"])
        D.linear(B.hc, d["w_in"], P, exact=ex)
        Q = B.a[: n * m.heads * gs].view(n, m.heads * gs)
        rows = kvc.rows[l]
        D.kv_prep(P, q_off=0, k_off=nq, v_off=nq + nk, heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, scale=m.scale, positions=positions,
                  slot_ids=slot_ids, block_table=kvc.block_table, cache=rows if m.kv_from is None else None, q=Q, n=n, block_size=kvc.block)
        O = B.b[: n * m.heads * m.vdim].view(n, m.heads * m.vdim)
        # runs of rows that are one per sequence (a wave takes a token's query heads of one key head, the keys dealt to several waves) and
        # runs of prompt portions (a wave takes 16 consecutive rows of one head), each one launch
        for r0, r1, one_per_seq in runs:
            splits, ws = 1, None
            if one_per_seq and not ex:
                tasks = (r1 - r0) * m.kv_heads * ((m.heads // m.kv_heads + 15) // 16)
                waves = self.ATTN_WAVES[64 if gs <= 64 else (128 if gs <= 128 else 256)]
                splits = max(1, min(waves // max(1, tasks), ctx_hint // 64, 64))
                if splits > 1:
                    key = (r1 - r0, m.heads, m.kv_heads, m.vdim, splits)
                    ws = B.attn_ws.get(key)
                    if ws is None:
                        ws = B.attn_ws[key] = torch.empty(max(1, D.kattn_workspace_floats(r1 - r0, m.heads, m.kv_heads, m.vdim, splits)), dtype=torch.float32,
                                                          device=self.device)
            D.kattn(Q[r0:r1], rows, None, kvc.block_table, slot_ids[r0:r1], positions[r0:r1], chunk=0, bias=d["bias"], sink=False, heads=m.heads,
                    kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, out=O[r0:r1], n=r1 - r0, mode=2 if one_per_seq else 3, splits=splits, workspace=ws)
        D.linear(O, d["o"], B.y, exact=ex)

    def _dense_ff(self, B, d, n) -> None:
        ff = d["mlp"].ff
        act = B.act[: n * ff].view(n, ff)
        D.linear(B.hc, d["up"], act, exact=self.exact, bias=d["up_b"], epilogue=D.EPI_XIELU, act_a=d["act_a"], act_b=d["act_b"])
        D.linear(act, d["down"], B.y, exact=self.exact, bias=d["down_b"])

    def _moe_ff(self, B, d, n, record=None, l=0) -> None:
        f, ex, W = d["mlp"], self.exact, self.cfg.width
        E, top = f.experts, f.top
        # the router's products in 32 bits in both modes (a choice between experts is not rounding's to make), inside the choice's launch
        D.route_topk(None, h=B.hc, w=d["router"], entries=f.entries, correction=d["correction"], groups=f.groups, keep=f.keep, top=top, scale=f.scale,
                     idx=B.idx, wgt=B.wgt, n=n)
        if record is not None:
            record[f"l{l}.route"] = B.idx[: n * top].view(n, top).clone()
        D.moe_plan(B.idx, n=n, top=top, experts=E, group_off=B.group_off, pair_token=B.pair_token, pair_row=B.pair_row)
        # the (token, expert) pairs lie grouped by expert: one launch runs every expert over its own rows, the counts stay on the device
        act = B.act[: n * top * f.ff].view(n * top, f.ff)
        D.linear(B.hc, d["gate_up"], act, m=n, a_rows=B.pair_token, batch=E, w_batch=2 * f.ff * W, exact=ex, epilogue=D.EPI_SILU_MUL, group_off=B.group_off)
        D.linear(act, d["e_down"], B.ey, m=n, batch=E, w_batch=W * f.ff, exact=ex, group_off=B.group_off)
        shared = None
        if f.shared_ff:
            sact = B.sact[: n * f.shared_ff].view(n, f.shared_ff)
            D.linear(B.hc, d["s_gate_up"], sact, exact=ex, epilogue=D.EPI_SILU_MUL)
            shared = D.linear(sact, d["s_down"], B.y2, exact=ex)
        D.moe_combine(B.ey, B.pair_row, B.wgt, B.hc, shared, B.y, n=n, top=top, width=W)

    @torch.no_grad()
    def forward(self, token_ids: torch.Tensor, positions: torch.Tensor, slot_ids: torch.Tensor, ctx_len: Optional[torch.Tensor] = None,
                logit_rows: Optional[torch.Tensor] = None, max_ctx_hint: int = 0, record: Optional[dict] = None, kv=None,
                rows_are_slots: bool = False, tokens_per_seq: Optional[List[int]] = None) -> torch.Tensor:
        """token_ids int64 [N]; positions / slot_ids int32 [N], rows in sequence order (the rows of a sequence consecutive, positions
        consecutive, continuing what the sequence's slot and pages hold; position 0 starts a sequence afresh); logit_rows int32 [M]
        selects the rows whose logits are wanted (None = all).  Returns fp32 logits [M, V].  record: dict filled with the residual after
        every layer ("l<i>.x") and every mixture layer's chosen entries ("l<i>.route", int32 [N, top]).  kv: a HybridCache other than the
        runner's own.  tokens_per_seq (rows per sequence, in order) or rows_are_slots (every row a sequence of its own) say how the rows
        are grouped; without them the slot ids are read back.  ctx_len and max_ctx_hint belong to the shared step interface."""
        cfg = self.cfg
        kvc = kv if kv is not None else self.kv
        n = token_ids.numel()
        M = logit_rows.numel() if logit_rows is not None else n
        B = self.buffers(n, M)
        if n == 0:
            return B.logits
        eps = cfg.norm_eps
        seg, nseg = self._runs(n, slot_ids, tokens_per_seq, rows_are_slots)
        if tokens_per_seq is not None:
            runs = attention_segments(tokens_per_seq, n, self.ATTN_MAX_SEGMENTS)
        else:
            runs = [(0, n, bool(rows_are_slots))]
        # every row the only row of its sequence (a decode step): the convolutions then store their carried inputs in the launch that reads them
        single = bool(rows_are_slots) or (tokens_per_seq is not None and all(int(t) <= 1 for t in tokens_per_seq))
        D.embed_bigram(token_ids, positions, slot_ids, self.embed, B.streams, pos_table=self.pos)
        # every residual launch adds the normed result of the sublayer before it and norms for the sublayer after it
        D.streams_step(B.streams, norm_w=self.layers[0]["norm1"], eps=eps, h=B.h)
        subs = [(l, q) for l, d in enumerate(self.layers) for q in ((1, 2) if d["mlp"] is not None else (1,))]
        for i, (l, q) in enumerate(subs):
            d = self.layers[l]
            D.causal_conv(B.h, off=0, channels=cfg.width, w=d[f"canon{q}"], bias=None, positions=positions, slot_ids=slot_ids,
                          state=kvc.state[l].get(f"canon{q}"), out=B.hc, n=n, added=True, single_rows=single)
            if q == 2 and d["mlp"].kind == "dense":
                self._dense_ff(B, d, n)
            elif q == 2:
                self._moe_ff(B, d, n, record, l)
            elif d["type"] == "hgrn2":
                self._hgrn2(B, d, l, n, positions, slot_ids, kvc, seg, nseg)
            else:
                self._attention(B, d, l, n, positions, slot_ids, kvc, runs, int(max_ctx_hint))
            write = dict(y=B.y, yn_w=d[f"norm{q}b"], y_eps=eps, out_w=self.ones1)
            if i + 1 < len(subs):
                nl, nq_ = subs[i + 1]
                D.streams_step(B.streams, **write, norm_w=self.layers[nl][f"norm{nq_}"], eps=eps, h=B.h)
            else:
                D.streams_step(B.streams, **write)
            if record is not None and (i + 1 == len(subs) or subs[i + 1][0] != l):
                record[f"l{l}.x"] = B.streams.sum(0)
        D.streams_step(B.streams, norm_w=self.final_norm, eps=eps, h=B.xf, rows=logit_rows)
        D.linear(B.xf, self.head, B.logits, exact=self.exact)
        return B.logits
