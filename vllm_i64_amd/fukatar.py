"""Runner of the Fukatar design on one MI355X: a decoder whose sublayers read the residual itself and whose results pass a centred norm
(weight, no bias) before they are added:

  x0 = embed[token] * s + bigram[hash(previous token, token)]          (the first token of a sequence takes the table's last row)
  layer:  h = x + (x_before - x) * shift    per channel, x_before the same layer's input of the token before (zeros at the start; state)
          x <- x + ln1(mixer(h));   x <- x + ln2(W_down relu(W_up x)^2)
  attention         grouped key / value heads; RMS norm with weights over the whole query and key projections; rotation in halves of the
                    first rot.dims values of a head, frequencies optionally scaled (slow ones divided, fast ones kept, a ramp between);
                    every value turned by its own position and the head's sum turned back by the query's; score * scale capped by
                    cap tanh(. / cap); softmax; a sigmoid gate per head; out-projection
  latent_attention  one normed low-rank row per token from which every head's keys and values are maps; no positions; the softmax's
                    denominator also holds exp(sink) per head
  parallel          left: attention with interleaved rotation, then queries and keys divided by their per-head root mean square, capped
                    scores;  right: gated delta rule S <- g S, u = beta (v - S^T k), S <- S + k u^T, o = S^T q on unit q, k behind short
                    causal convolutions + silu, a gated RMS norm per head;  the mean of the two RMS-normed results
  logits = cap tanh(head . ln(x) / cap)

The residual, norms, shift, angles, gates, decays, the recurrence and its state, scores and softmax are fp32 in both modes; "bfloat16"
rounds the inputs of the matrix products to bf16 (fp32 sums on the matrix cores) and keeps cached rows in bf16, "float32" keeps
everything in 32 bits.  torch holds memory and streams; every arithmetic step is a libi64hip_dense.so kernel.  The step interface is
I64MoEModel's, so the same engine, scheduler and decoders drive it."""
from __future__ import annotations

import os
from typing import Dict, List, Optional

import torch

from . import ops_dense as D
from .config import FukatarConfig
from .model import attention_segments
from .paged_cache import HybridCache

UNIT_EPS = 1e-6     # inside the root of the delta rule's unit vectors: a constant of the design, not of a checkpoint


class _StepBuffers:
    def __init__(self, model: "FukatarModel", n: int, m: int):
        f32 = dict(dtype=torch.float32, device=model.device)
        W = model.cfg.width
        self.streams = torch.empty(1, n, W, **f32)              # the residual (one stream of the multi-stream kernel)
        self.h = torch.empty(n, W, **f32)                       # the mixer's input: the residual blended with the row before
        self.y = torch.empty(n, W, **f32)
        self.y2 = torch.empty(n, W, **f32)
        self.p = torch.empty(n * model.max_proj, **f32)         # everything projected from the mixer's input
        self.a = torch.empty(n * model.max_a, **f32)            # query rows / convolution output
        self.b = torch.empty(n * model.max_b, **f32)            # attention output / recurrence output
        self.c = torch.empty(n * model.max_b, **f32)            # values of the latent heads / normed recurrence output
        self.g = torch.empty(n * max(2 * model.max_gdn_heads, 1), **f32)   # write strength and decay per head
        self.act = torch.empty(n * max(model.max_ff, 1), **f32)
        self.xf = torch.empty(m, W, **f32)
        self.logits = torch.empty(m, model.cfg.vocab, **f32)
        self.attn_ws: Dict[tuple, torch.Tensor] = {}


class FukatarModel:
    MAX_BUFFER_SETS = int(os.environ.get("I64H_MAX_BUFFER_SETS", "8"))
    ATTN_MAX_SEGMENTS = 4
    ATTN_WAVES = {64: 3072, 128: 2048, 256: 1024}     # waves a decode-sized attention launch aims at, by the width of a key head's cached part

    def __init__(self, cfg: FukatarConfig, weights: Dict[str, torch.Tensor], device="cuda:0", dtype: str = "bfloat16", max_seqs: int = 4,
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

        self.embed, self.head = bf(need("embed", (cfg.vocab, W))), bf(need("head", (cfg.vocab, W)))
        self.bigram = bf(need("bigram", (cfg.bigram.buckets + 1, W))) if cfg.bigram is not None else None
        self.final_norm = f(need("final.norm", (W,)))
        self.ones1 = torch.ones(1, dtype=torch.float32, device=dev)
        self.layers: List[dict] = [self._load_layer(i, L, need, bf, f) for i, L in enumerate(cfg.layers)]
        specs = []
        for L in cfg.layers:
            state = {"shift": (1, W)}
            m = L.mixer
            if L.type == "latent_attention":
                specs.append({"rows": m.kv_rank, "kscale": False, "state": state})
            elif L.type == "attention":
                specs.append({"rows": m.kv_heads * (m.vdim + m.dim), "kscale": False, "state": state})
            else:
                a, r = m.left, m.right
                if r.conv > 1:
                    state["conv"] = (r.conv - 1, r.conv_channels)
                state["gdn"] = (r.heads, r.vdim, r.dim)
                specs.append({"rows": a.kv_heads * (a.vdim + a.dim), "kscale": False, "state": state})
        self.max_proj = max(d["n_in"] for d in self.layers)
        self.max_a = max(d["n_a"] for d in self.layers)
        self.max_b = max(d["n_b"] for d in self.layers)
        self.max_gdn_heads = max([l.mixer.right.heads for l in cfg.layers if l.type == "parallel"] or [0])
        self.max_ff = max([l.mlp.ff for l in cfg.layers if l.mlp is not None] or [0])
        if cache_dtype is None:
            cache_dtype = torch.float32 if self.exact else torch.bfloat16
        self.kv = HybridCache(specs, num_kv_blocks, max_seqs, dev, dtype=cache_dtype, block=kv_block,
                              seq_state={"prev_token": ((), torch.int64)} if cfg.bigram is not None else None)
        self._bufs: Dict[tuple, _StepBuffers] = {}
        self._pinned: set = set()
        self._arange: Dict[int, torch.Tensor] = {}

    # ---- load-time layout work: one weight for everything that reads the mixer's input; small vectors and tables in fp32 ----
    def _rotary(self, a, d: dict, f) -> None:
        """Frequency tables of a rotated attention: evaluated in 64 bits on the host, rounded once to fp32."""
        d["inv_freq"], d["rot_mult"], d["v_freq"] = None, 1.0, None
        if a.rot is not None and a.rot.dims:
            fr, d["rot_mult"] = a.rot.frequencies()
            d["inv_freq"] = f(torch.tensor(fr, dtype=torch.float64))
        if a.rot is not None and a.rotate_values:
            d["v_freq"] = f(torch.tensor([a.rot.base ** (-2.0 * i / a.vdim) for i in range(a.vdim // 2)], dtype=torch.float64))

    def _load_layer(self, i: int, L, need, bf, f) -> dict:
        W, p = self.cfg.width, f"l{i}."
        d = dict(type=L.type, m=L.mixer, mlp=L.mlp)
        d["norm1"] = f(need(p + "norm1", (W,)))
        s = need(p + "shift", (W,)).float()
        d["shift"] = f(torch.stack([s, -s], 1))      # two taps added to the input: x + s * x_before - s * x
        m = L.mixer
        if L.type == "latent_attention":
            H, r = m.heads, m.kv_rank
            d["w_in"] = bf(torch.cat([need(p + "mix.q", (H * m.dim, W)), need(p + "mix.dkv", (r, W))], 0))
            d["n_in"] = H * m.dim + r
            # a head's score against a cached latent c is q_h . (U_h c) = (U_h^T q_h) . c: the key map transposed per head
            d["uk_t"] = bf(need(p + "mix.uk", (H * m.dim, r)).reshape(H, m.dim, r).transpose(1, 2))      # [H, r, dim]
            d["uv"] = bf(need(p + "mix.uv", (H * m.vdim, r)).reshape(H, m.vdim, r))                      # [H, vdim, r]
            d["c_norm"] = f(need(p + "mix.dkv.norm", (r,)))
            d["sink"] = f(need(p + "mix.sink", (H,))) if m.sink else None
            d["o"] = bf(need(p + "mix.o", (W, H * m.vdim)))
            d["n_a"], d["n_b"] = H * r, max(H * r, H * m.vdim)
        else:
            a = m if L.type == "attention" else m.left
            ap = p + ("mix." if L.type == "attention" else "mix.left.")
            nq, nk, nv = a.heads * a.dim, a.kv_heads * a.dim, a.kv_heads * a.vdim
            parts = [need(ap + "q", (nq, W)), need(ap + "k", (nk, W)), need(ap + "v", (nv, W))]
            d["q_off"], d["k_off"], d["v_off"] = 0, nq, nq + nk
            n_in = nq + nk + nv
            if a.head_gate:
                parts.append(need(ap + "g", (a.heads, W)))
                d["g_off"], n_in = n_in, n_in + a.heads
            d["q_norm"] = f(need(ap + "q.norm", (nq,))) if a.qk_norm == "row" else None
            d["k_norm"] = f(need(ap + "k.norm", (nk,))) if a.qk_norm == "row" else None
            self._rotary(a, d, f)
            d["o"] = bf(need(ap + "o", (W, a.heads * a.vdim)))
            d["n_a"], d["n_b"] = a.heads * (a.vdim + a.dim), a.heads * a.vdim
            if L.type == "parallel":
                r, rp = m.right, p + "mix.right."
                rk, rv = r.kv_heads * r.dim, r.heads * r.vdim
                # [.. left ..| q | k | v | write strength | decay step | output gate]: the three convolved parts side by side
                parts += [need(rp + "q", (rk, W)), need(rp + "k", (rk, W)), need(rp + "v", (rv, W)), need(rp + "b", (r.heads, W)),
                          need(rp + "a", (r.heads, W)), need(rp + "g", (rv, W))]
                d["r_off"], d["rb_off"], d["ra_off"], d["rg_off"] = n_in, n_in + 2 * rk + rv, n_in + 2 * rk + rv + r.heads, n_in + 2 * rk + rv + 2 * r.heads
                n_in += 2 * rk + 2 * rv + 2 * r.heads
                d["conv_w"] = f(torch.cat([need(rp + "q.conv", (rk, r.conv)), need(rp + "k.conv", (rk, r.conv)), need(rp + "v.conv", (rv, r.conv))], 0))
                d["A_log"], d["dt_bias"] = f(need(rp + "A_log", (r.heads,))), f(need(rp + "dt_bias", (r.heads,)))
                d["r_norm"] = f(need(rp + "norm", (r.vdim,)))
                d["o_right"] = bf(need(rp + "o", (W, rv)))
                d["out_left"], d["out_right"] = f(need(p + "mix.left.out", (W,))), f(need(p + "mix.right.out", (W,)))
                d["n_a"], d["n_b"] = max(d["n_a"], r.conv_channels), max(d["n_b"], rv)
            d["w_in"], d["n_in"] = bf(torch.cat(parts, 0)), n_in
        if L.mlp is not None:
            d["norm2"] = f(need(p + "norm2", (W,)))
            d["up"], d["down"] = bf(need(p + "mlp.up", (L.mlp.ff, W))), bf(need(p + "mlp.down", (W, L.mlp.ff)))
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
        """The per-sequence state, for a caller that runs a step which must not count (a warm-up before a graph capture)."""
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

    def _splits(self, B, rows: int, heads: int, kv_heads: int, vals: int, width: int, ctx_hint: int, floats):
        """How many waves share a decode row's keys (about ATTN_WAVES waves in the launch, a wave keeping at least two tiles of 32 keys),
        and the workspace their partial results meet in."""
        tasks = rows * kv_heads * ((heads // kv_heads + 15) // 16)
        waves = self.ATTN_WAVES[64 if width <= 64 else (128 if width <= 128 else 256)]
        splits = max(1, min(waves // max(1, tasks), ctx_hint // 64, 64))
        if splits <= 1:
            return 1, None
        key = (rows, heads, kv_heads, vals, splits)
        ws = B.attn_ws.get(key)
        if ws is None:
            ws = B.attn_ws[key] = torch.empty(max(1, floats(splits)), dtype=torch.float32, device=self.device)
        return splits, ws

    # ---- mixers: the input is B.h; the result lands in B.y (and B.y2 for the second of two side-by-side mixers) ----
    def _rotary_attention(self, B, d, a, P, l, n, positions, slot_ids, kvc, runs, ctx_hint, out) -> None:
        """Rotated attention on the projection rows P (already computed): prep -> paged [values | keys] rows and query rows, attention,
        the turn back and the head gate, out-projection into `out`."""
        ex = self.exact
        gs = a.vdim + a.dim
        Q = B.a[: n * a.heads * gs].view(n, a.heads * gs)
        rows = kvc.rows[l]
        D.rot_prep(P, q_off=d["q_off"], k_off=d["k_off"], v_off=d["v_off"], heads=a.heads, kv_heads=a.kv_heads, dim=a.dim, vdim=a.vdim, q_norm_w=d["q_norm"],
                   k_norm_w=d["k_norm"], eps=self.cfg.norm_eps, rot_dims=a.rot.dims if a.rot is not None else 0, interleaved=a.interleaved,
                   inv_freq=d["inv_freq"], rot_mult=d["rot_mult"], head_norm=a.qk_norm == "head", v_freq=d["v_freq"], scale=a.scale, positions=positions,
                   slot_ids=slot_ids, block_table=kvc.block_table, cache=rows, q=Q, n=n)
        O = B.b[: n * a.heads * a.vdim].view(n, a.heads * a.vdim)
        # runs of rows that are one per sequence (a wave takes a token's query heads of one key head, the keys dealt to several waves) and
        # runs of prompt portions (a wave takes 16 consecutive rows of one head), each one launch
        for r0, r1, one_per_seq in runs:
            splits, ws = 1, None
            if one_per_seq and not ex:
                splits, ws = self._splits(B, r1 - r0, a.heads, a.kv_heads, a.vdim, gs, ctx_hint,
                                          lambda s: D.kattn_workspace_floats(r1 - r0, a.heads, a.kv_heads, a.vdim, s))
            D.kattn(Q[r0:r1], rows, None, kvc.block_table, slot_ids[r0:r1], positions[r0:r1], chunk=0, bias=None, sink=False, heads=a.heads,
                    kv_heads=a.kv_heads, dim=a.dim, vdim=a.vdim, out=O[r0:r1], n=r1 - r0, mode=2 if one_per_seq else 3, splits=splits, workspace=ws,
                    softcap=a.softcap)
        if d["v_freq"] is not None or a.head_gate:
            D.rot_post(O, heads=a.heads, vdim=a.vdim, interleaved=a.interleaved, v_freq=d["v_freq"], positions=positions,
                       gate=P if a.head_gate else None, gate_off=d.get("g_off", 0), ldg=d["n_in"], n=n)
        D.linear(O, d["o"], out, exact=ex)

    def _attention(self, B, d, l, n, positions, slot_ids, kvc, runs, ctx_hint) -> None:
        P = B.p[: n * d["n_in"]].view(n, d["n_in"])
        D.linear(B.h, d["w_in"], P, exact=self.exact)
        self._rotary_attention(B, d, d["m"], P, l, n, positions, slot_ids, kvc, runs, ctx_hint, B.y)

    def _latent(self, B, d, l, n, positions, slot_ids, kvc, runs, ctx_hint) -> None:
        m, ex = d["m"], self.exact
        H, r, N1 = m.heads, m.kv_rank, d["n_in"]
        P = B.p[: n * N1].view(n, N1)
        D.linear(B.h, d["w_in"], P, exact=ex)
        cache = kvc.rows[l]
        Q = B.a[: n * H * r]
        D.latent_prep(P, q_off=0, dkv_off=H * m.dim, heads=H, dim=m.dim, rot_dim=0, kv_rank=r, rot_dims=0, c_norm_w=d["c_norm"], eps=self.cfg.norm_eps,
                      inv_freq=None, positions=positions, slot_ids=slot_ids, block_table=kvc.block_table, block_size=kvc.block, cache=cache, q=Q, n=n)
        # queries into latent space, per head: Q[:, h, :] = q[:, h, :] @ U_h
        D.linear(P, d["uk_t"], Q, m=n, n=r, k=m.dim, a_off=0, lda=N1, ldc=H * r, batch=H, a_batch=m.dim, w_batch=r * m.dim, c_batch=r, exact=ex)
        olat = B.b[: n * H * r]
        for r0, r1, one_per_seq in runs:
            splits, ws = 1, None
            if one_per_seq and not ex:
                splits, ws = self._splits(B, r1 - r0, H, 1, r, r, ctx_hint, lambda s: D.latent_attn_workspace_floats(r1 - r0, H, r, s))
            D.latent_attn(Q[r0 * H * r: r1 * H * r], cache, kvc.block_table, slot_ids[r0:r1], positions[r0:r1], window=0, scale=m.scale, heads=H, kv_rank=r,
                          rot_dim=0, out=olat[r0 * H * r: r1 * H * r], n=r1 - r0, mode=2 if one_per_seq else 3, splits=splits, workspace=ws, sink=d["sink"])
        # summed latents into value space, per head
        og = B.c[: n * H * m.vdim]
        D.linear(olat, d["uv"], og, m=n, n=m.vdim, k=r, lda=H * r, ldc=H * m.vdim, batch=H, a_batch=r, w_batch=m.vdim * r, c_batch=m.vdim, exact=ex)
        D.linear(og, d["o"], B.y, m=n, k=H * m.vdim, lda=H * m.vdim, exact=ex)

    def _parallel(self, B, d, l, n, positions, slot_ids, kvc, seg, nseg, runs, ctx_hint, single) -> None:
        a, r, ex = d["m"].left, d["m"].right, self.exact
        N1 = d["n_in"]
        P = B.p[: n * N1].view(n, N1)
        D.linear(B.h, d["w_in"], P, exact=ex)
        self._rotary_attention(B, d, a, P, l, n, positions, slot_ids, kvc, runs, ctx_hint, B.y)
        st = kvc.state[l]
        C, rk, rv = r.conv_channels, r.kv_heads * r.dim, r.heads * r.vdim
        X = B.a[: n * C].view(n, C)
        D.causal_conv(P, off=d["r_off"], channels=C, w=d["conv_w"], bias=None, positions=positions, slot_ids=slot_ids, state=st.get("conv"), out=X, n=n,
                      single_rows=single)
        G = B.g[: n * 2 * r.heads].view(n, 2 * r.heads)
        cols = dict(q_off=0, k_off=rk, v_off=2 * rk, heads=r.heads, kv_heads=r.kv_heads, dim=r.dim, vdim=r.vdim, n=n)
        D.gdn_gates(X, G, P, b_off=d["rb_off"], a_off=d["ra_off"], a_log=d["A_log"], dt_bias=d["dt_bias"], unit_eps=UNIT_EPS, q_scale=r.dim ** -0.5, **cols)
        R = B.b[: n * rv].view(n, rv)
        D.gdn_scan(X, G, seg_start=seg, nseg=nseg, positions=positions, slot_ids=slot_ids, state=st["gdn"], out=R, **cols)
        Rn = B.c[: n * rv].view(n, rv)
        D.gate_norm(R, d["r_norm"], Rn, groups=r.heads, eps=self.cfg.norm_eps, z=P, z_off=d["rg_off"], ldz=N1, n=n, gate_after=True, width=rv)
        D.linear(Rn, d["o_right"], B.y2, exact=ex)

    @torch.no_grad()
    def forward(self, token_ids: torch.Tensor, positions: torch.Tensor, slot_ids: torch.Tensor, ctx_len: Optional[torch.Tensor] = None,
                logit_rows: Optional[torch.Tensor] = None, max_ctx_hint: int = 0, record: Optional[dict] = None, kv=None,
                rows_are_slots: bool = False, tokens_per_seq: Optional[List[int]] = None) -> torch.Tensor:
        """token_ids int64 [N]; positions / slot_ids int32 [N], rows in sequence order (the rows of a sequence consecutive, positions
        consecutive, continuing what the sequence's slot and pages hold; position 0 starts a sequence afresh); logit_rows int32 [M]
        selects the rows whose logits are wanted (None = all).  Returns fp32 logits [M, V].  record: dict filled with the residual after
        every layer ("l<i>.x").  kv: a HybridCache other than the runner's own.  tokens_per_seq (rows per sequence, in order) or
        rows_are_slots (every row a sequence of its own) say how the rows are grouped; without them the slot ids are read back.
        ctx_len and max_ctx_hint belong to the shared step interface."""
        cfg = self.cfg
        kvc = kv if kv is not None else self.kv
        n = token_ids.numel()
        M = logit_rows.numel() if logit_rows is not None else n
        B = self.buffers(n, M)
        if n == 0:
            return B.logits
        eps, ex = cfg.norm_eps, self.exact
        seg, nseg = self._runs(n, slot_ids, tokens_per_seq, rows_are_slots)
        if tokens_per_seq is not None:
            runs = attention_segments(tokens_per_seq, n, self.ATTN_MAX_SEGMENTS)
        else:
            runs = [(0, n, bool(rows_are_slots))]
        # every row the only row of its sequence (a decode step): the convolutions then store their carried inputs in the launch that reads them
        single = bool(rows_are_slots) or (tokens_per_seq is not None and all(int(t) <= 1 for t in tokens_per_seq))
        bg = cfg.bigram
        D.embed_bigram(token_ids, positions, slot_ids, self.embed, B.streams, bigram=self.bigram, buckets=bg.buckets if bg else 0,
                       mul_prev=bg.mul_prev if bg else 0, mul_cur=bg.mul_cur if bg else 0, prev_token=kvc.seq_state.get("prev_token"),
                       scale=cfg.embedding_scale)
        x = B.streams[0]
        hint = int(max_ctx_hint)
        for l, d in enumerate(self.layers):
            # the blend with the row before, as a convolution of two taps added to its input; the carried input is the layer's own state
            D.causal_conv(x, off=0, channels=cfg.width, w=d["shift"], bias=None, positions=positions, slot_ids=slot_ids, state=kvc.state[l]["shift"],
                          out=B.h, n=n, added=True, single_rows=single)
            write = dict(y=B.y, y_eps=eps, out_w=self.ones1, post_w=d["norm1"], post_center=True)
            if d["type"] == "latent_attention":
                self._latent(B, d, l, n, positions, slot_ids, kvc, runs, hint)
            elif d["type"] == "attention":
                self._attention(B, d, l, n, positions, slot_ids, kvc, runs, hint)
            else:
                self._parallel(B, d, l, n, positions, slot_ids, kvc, seg, nseg, runs, hint, single)
                write.update(y2=B.y2, yn_w=d["out_left"], y2n_w=d["out_right"])
            D.streams_step(B.streams, **write)
            if d["mlp"] is not None:
                act = B.act[: n * d["mlp"].ff].view(n, d["mlp"].ff)
                D.linear(x, d["up"], act, exact=ex, epilogue=D.EPI_RELU_SQ)
                D.linear(act, d["down"], B.y, exact=ex)
                D.streams_step(B.streams, y=B.y, y_eps=eps, out_w=self.ones1, post_w=d["norm2"], post_center=True)
            if record is not None:
                record[f"l{l}.x"] = x.clone()
        D.streams_step(B.streams, norm_w=self.final_norm, eps=eps, h=B.xf, rows=logit_rows, h_center=True)
        cap = cfg.logit_softcap
        D.linear(B.xf, self.head, B.logits, exact=ex, epilogue=D.EPI_SOFTCAP if cap > 0 else D.EPI_STORE, softcap=cap)
        return B.logits
