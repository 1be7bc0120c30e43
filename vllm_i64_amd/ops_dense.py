"""Torch-facing wrappers over libi64hip_dense.so (include/i64h_dense.h): memory and stream plumbing only, no torch math and no
CPU path.  Activations are fp32 tensors, weights bf16 tensors [out, in]."""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import _lib
from ._lib import call_dense, ptr
from .ops import _chk, _stream

EPI_STORE, EPI_GELU_MUL, EPI_MUL_SIGMOID, EPI_SOFTCAP, EPI_GELU_ERF, EPI_SCALE, EPI_SILU_MUL, EPI_XIELU, EPI_RELU_SQ = 0, 1, 2, 3, 4, 5, 6, 7, 8
_DUAL = (EPI_GELU_MUL, EPI_SILU_MUL)
CACHE_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 2}


def _ref(s):
    return ctypes.addressof(s)


def linear(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, *, m: Optional[int] = None, n: Optional[int] = None, k: Optional[int] = None,
           a_off: int = 0, lda: Optional[int] = None, a_rows: Optional[torch.Tensor] = None, c_off: int = 0, ldc: Optional[int] = None,
           batch: int = 1, a_batch: int = 0, w_batch: int = 0, c_batch: int = 0, exact: bool = False, epilogue: int = EPI_STORE,
           e: Optional[torch.Tensor] = None, e_off: int = 0, lde: int = 0, e_batch: int = 0, softcap: float = 0.0,
           bias: Optional[torch.Tensor] = None, bias_batch: int = 0, scale: float = 1.0, act_a: float = 0.0, act_b: float = 0.0,
           group_off: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[b][:, c_off + b * c_batch : + n] = epilogue(a[b][rows, a_off + b * a_batch : + k] @ w[b]^T): see i64h_linear.  a, out and e are
    fp32 matrices addressed by (column offset, row stride); w is bf16 [n, k] (EPI_GELU_MUL / EPI_SILU_MUL: [2n, k], gate rows first), or a
    stack [batch, n, k] with w_batch = n * k.  bias fp32 [n] (per batch: bias_batch apart) is added before the epilogue.  group_off int32
    [batch + 1] on the device: batch b takes the rows [group_off[b], group_off[b + 1]) of a_rows (or a) and out; m is then the most rows a
    batch may have, and a_rows / a / out must hold group_off[batch] rows (the caller's business: the counts stay on the device)."""
    _chk(a, torch.float32, "a"), _chk(w, torch.bfloat16, "w"), _chk(out, torch.float32, "out")
    if a_rows is not None:
        _chk(a_rows, torch.int32, "a_rows")
    N = int(n if n is not None else w.shape[-2] // (2 if epilogue in _DUAL else 1))
    K = int(k if k is not None else w.shape[-1])
    M = int(m if m is not None else (a_rows.numel() if a_rows is not None else a.shape[0]))
    lda = int(lda if lda is not None else a.shape[-1])
    ldc = int(ldc if ldc is not None else out.shape[-1])
    if w.shape[-1] != K or a_off + (batch - 1) * a_batch + K > lda or c_off + (batch - 1) * c_batch + N > ldc:
        raise _lib.I64HError(f"linear: K {K} / N {N} do not fit a (row stride {lda}), w {tuple(w.shape)} or out (row stride {ldc})")
    if out.numel() < (M - 1) * ldc + c_off + (batch - 1) * c_batch + N or (a_rows is None and a.numel() < (M - 1) * lda + a_off + (batch - 1) * a_batch + K):
        raise _lib.I64HError("linear: operand smaller than the launch reads or writes")
    if w.numel() < (batch - 1) * w_batch + N * K * (2 if epilogue in _DUAL else 1):
        raise _lib.I64HError("linear: weight smaller than the launch reads")
    if e is not None:
        _chk(e, torch.float32, "e")
        if e.numel() < (M - 1) * lde + e_off + (batch - 1) * e_batch + N:
            raise _lib.I64HError("linear: gate operand smaller than the launch reads")
    if bias is not None:
        _chk(bias, torch.float32, "bias")
        if bias.numel() < (batch - 1) * bias_batch + N:
            raise _lib.I64HError("linear: bias smaller than the launch reads")
    if group_off is not None:
        _chk(group_off, torch.int32, "group_off")
        if group_off.numel() < batch + 1:
            raise _lib.I64HError("linear: group_off needs batch + 1 entries")
    d = _lib.Linear(A=ptr(a) + 4 * a_off, lda=lda, a_rows=ptr(a_rows), W=ptr(w), C=ptr(out) + 4 * c_off, ldc=ldc, M=M, N=N, K=K, batch=batch,
                    a_batch=a_batch, w_batch=w_batch, c_batch=c_batch, exact=int(exact), epilogue=epilogue,
                    E=(ptr(e) + 4 * e_off) if e is not None else 0, lde=lde, e_batch=e_batch, softcap=float(softcap),
                    bias=ptr(bias), bias_batch=int(bias_batch), scale=float(scale), act_a=float(act_a), act_b=float(act_b), group_off=ptr(group_off))
    call_dense("i64h_linear_run", _ref(d), _stream())
    return out


def embed_scaled(ids: torch.Tensor, table: torch.Tensor, scale: float, out: torch.Tensor) -> torch.Tensor:
    _chk(ids, torch.int64, "ids"), _chk(table, torch.bfloat16, "table"), _chk(out, torch.float32, "out")
    V, W = table.shape
    assert out.numel() >= ids.numel() * W
    call_dense("i64h_embed_scaled", ptr(ids), ptr(table), float(scale), ptr(out), ids.numel(), W, V, _stream())
    return out


def gated_postnorm(x: torch.Tensor, norm_w: torch.Tensor, groups: int, eps: float, *, n: Optional[int] = None, alpha: float = 1.0,
                   y: Optional[torch.Tensor] = None, ldy: Optional[int] = None, gate_pre: Optional[torch.Tensor] = None, gate_off: int = 0,
                   ldg: int = 0, gate_bias: Optional[torch.Tensor] = None, x_rows: Optional[torch.Tensor] = None,
                   out: Optional[torch.Tensor] = None, hist: Optional[torch.Tensor] = None, hist_index: int = 0,
                   mix_w: Optional[torch.Tensor] = None, mix_out: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """See i64h_postnorm.  x fp32 [*, W]; n rows (default: x_rows' count, else x's); hist fp32 [layers + 1, n, W]."""
    _chk(x, torch.float32, "x"), _chk(norm_w, torch.float32, "norm_w")
    W = norm_w.numel()
    rows = int(n if n is not None else (x_rows.numel() if x_rows is not None else x.numel() // W))
    for t, name in ((y, "y"), (gate_pre, "gate_pre"), (gate_bias, "gate_bias"), (out, "out"), (hist, "hist"), (mix_w, "mix_w"), (mix_out, "mix_out")):
        if t is not None:
            _chk(t, torch.float32, name)
    if x_rows is not None:
        _chk(x_rows, torch.int32, "x_rows")
    if mix_w is not None:
        if hist is None or mix_out is None or mix_w.numel() < hist_index + 1 or hist.numel() < (hist_index + 1) * rows * W or hist.shape[-2] != rows:
            raise _lib.I64HError("gated_postnorm: the depth mix needs hist [>= hist_index + 1, n, W], mix_out and hist_index + 1 weights")
    d = _lib.PostNorm(x=ptr(x), x_rows=ptr(x_rows), y=ptr(y), ldy=int(ldy if ldy is not None else W), gate_pre=(ptr(gate_pre) + 4 * gate_off) if gate_pre is not None else 0,
                      ldg=int(ldg), gate_bias=ptr(gate_bias), alpha=float(alpha), norm_w=ptr(norm_w), groups=int(groups), eps=float(eps),
                      out=ptr(out), hist=ptr(hist), hist_index=int(hist_index), mix_w=ptr(mix_w), mix_out=ptr(mix_out), n=rows, W=W)
    call_dense("i64h_gated_postnorm", _ref(d), _stream())
    return out if out is not None else mix_out


def latent_prep(p: torch.Tensor, *, q_off: int, dkv_off: int, heads: int, dim: int, rot_dim: int, kv_rank: int, rot_dims: int,
                c_norm_w: torch.Tensor, eps: float, inv_freq: Optional[torch.Tensor], positions: torch.Tensor, slot_ids: torch.Tensor,
                block_table: torch.Tensor, block_size: int, cache: torch.Tensor, q: torch.Tensor, n: Optional[int] = None) -> None:
    _chk(p, torch.float32, "p"), _chk(c_norm_w, torch.float32, "c_norm_w"), _chk(q, torch.float32, "q")
    _chk(positions, torch.int32, "positions"), _chk(slot_ids, torch.int32, "slot_ids"), _chk(block_table, torch.int32, "block_table")
    _chk(cache, None, "cache")
    rows = int(n if n is not None else positions.numel())
    D = kv_rank + rot_dim
    if cache.shape[-1] != D or cache.shape[-2] != block_size or q.numel() < rows * heads * D or positions.numel() < rows or slot_ids.numel() < rows:
        raise _lib.I64HError("latent_prep: cache / query / position shapes do not fit the sizes")
    if q_off + heads * (dim + rot_dim) > p.shape[-1] or dkv_off + D > p.shape[-1] or c_norm_w.numel() != kv_rank:
        raise _lib.I64HError("latent_prep: projection columns outside the projection rows")
    if rot_dims:
        _chk(inv_freq, torch.float32, "inv_freq")
        assert inv_freq.numel() >= rot_dims // 2
    d = _lib.LatentPrep(P=ptr(p), ldp=p.shape[-1], q_off=q_off, dkv_off=dkv_off, heads=heads, dim=dim, rot_dim=rot_dim, kv_rank=kv_rank,
                        rot_dims=rot_dims, c_norm_w=ptr(c_norm_w), eps=float(eps), inv_freq=ptr(inv_freq) if rot_dims else 0,
                        positions=ptr(positions), slot_ids=ptr(slot_ids), block_table=ptr(block_table), max_blocks_per_seq=block_table.shape[1],
                        block_size=block_size, cache=ptr(cache), cache_dtype=CACHE_DTYPE_CODE[cache.dtype], Q=ptr(q), n=rows)
    call_dense("i64h_latent_prep", _ref(d), _stream())


def latent_attn(q: torch.Tensor, cache: torch.Tensor, block_table: torch.Tensor, slot_ids: torch.Tensor, positions: torch.Tensor, *,
                window: int, scale: float, heads: int, kv_rank: int, rot_dim: int, out: torch.Tensor, n: Optional[int] = None,
                mode: int = 0, splits: int = 1, workspace: Optional[torch.Tensor] = None, sink: Optional[torch.Tensor] = None,
                softcap: float = 0.0) -> torch.Tensor:
    """See i64h_latent_attn.  sink fp32 [heads]: a learned extra score per head in the softmax's denominator."""
    _chk(q, torch.float32, "q"), _chk(out, torch.float32, "out"), _chk(cache, None, "cache")
    _chk(positions, torch.int32, "positions"), _chk(slot_ids, torch.int32, "slot_ids"), _chk(block_table, torch.int32, "block_table")
    rows = int(n if n is not None else positions.numel())
    D = kv_rank + rot_dim
    if sink is not None:
        _chk(sink, torch.float32, "sink")
        if sink.numel() != heads:
            raise _lib.I64HError("latent_attn: the sink scores are not [heads]")
    if cache.shape[-1] != D or q.numel() < rows * heads * D or out.numel() < rows * heads * kv_rank:
        raise _lib.I64HError("latent_attn: cache / query / output shapes do not fit the sizes")
    if splits > 1:
        need = latent_attn_workspace_floats(rows, heads, kv_rank, splits)
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.float32, device=q.device)
        _chk(workspace, torch.float32, "workspace")
        if workspace.numel() < need:
            raise _lib.I64HError(f"latent_attn: workspace of {workspace.numel()} floats, {need} needed")
    d = _lib.LatentAttn(Q=ptr(q), cache=ptr(cache), cache_dtype=CACHE_DTYPE_CODE[cache.dtype], block_table=ptr(block_table),
                        max_blocks_per_seq=block_table.shape[1], block_size=cache.shape[-2], slot_ids=ptr(slot_ids), positions=ptr(positions),
                        window=int(window), scale=float(scale), out=ptr(out), n=rows, heads=heads, kv_rank=kv_rank, rot_dim=rot_dim, mode=mode,
                        splits=int(splits) if splits > 1 else 1, workspace=ptr(workspace) if splits > 1 else 0, sink=int(sink is not None), sink_w=ptr(sink),
                        softcap=float(softcap))
    call_dense("i64h_latent_attn", _ref(d), _stream())
    return out


def latent_attn_workspace_floats(n: int, heads: int, kv_rank: int, splits: int) -> int:
    return int(_lib.load_dense().i64h_latent_attn_workspace_floats(n, heads, kv_rank, splits))


# ---- recurrent and hybrid layers ----------------------------------------------------------------------------------------------------
def _rows_ok(name: str, n: int, *tensors) -> None:
    for t in tensors:
        if t.numel() < n:
            raise _lib.I64HError(f"{name}: a per-row operand has {t.numel()} entries, the launch has {n} rows")


def embed_bigram(ids: torch.Tensor, positions: torch.Tensor, slot_ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, *,
                 bigram: Optional[torch.Tensor] = None, buckets: int = 0, mul_prev: int = 0, mul_cur: int = 0,
                 prev_token: Optional[torch.Tensor] = None, pos_table: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    """See i64h_embed_bigram.  out fp32 [copies, n, W] (or [n, W]); prev_token int64 [slots], read and updated; pos_table bf16 [positions, W];
    scale multiplies the token row."""
    _chk(ids, torch.int64, "ids"), _chk(positions, torch.int32, "positions"), _chk(slot_ids, torch.int32, "slot_ids")
    _chk(table, torch.bfloat16, "table"), _chk(out, torch.float32, "out")
    n = ids.numel()
    V, W = table.shape
    _rows_ok("embed_bigram", n, positions, slot_ids)
    copies = out.numel() // max(1, n * W)
    if out.numel() != copies * n * W:
        raise _lib.I64HError("embed_bigram: out is not [copies, n, W]")
    if bigram is not None:
        _chk(bigram, torch.bfloat16, "bigram"), _chk(prev_token, torch.int64, "prev_token")
        if tuple(bigram.shape) != (buckets + 1, W):
            raise _lib.I64HError(f"embed_bigram: table {tuple(bigram.shape)} for {buckets} buckets of width {W}")
    if pos_table is not None:
        _chk(pos_table, torch.bfloat16, "pos_table")
        if pos_table.dim() != 2 or pos_table.shape[1] != W:
            raise _lib.I64HError(f"embed_bigram: position table {tuple(pos_table.shape)} for width {W}")
    d = _lib.EmbedBigram(ids=ptr(ids), positions=ptr(positions), slot_ids=ptr(slot_ids), table=ptr(table), V=V, W=W, bigram=ptr(bigram),
                         buckets=int(buckets), mul_prev=int(mul_prev), mul_cur=int(mul_cur), prev_token=ptr(prev_token), out=ptr(out),
                         copies=max(1, copies), n=n, pos_table=ptr(pos_table), pos_rows=pos_table.shape[0] if pos_table is not None else 0,
                         scale=float(scale))
    call_dense("i64h_embed_bigram", _ref(d), _stream())
    return out


def streams_step(streams: torch.Tensor, *, y: Optional[torch.Tensor] = None, y2: Optional[torch.Tensor] = None, yn_w: Optional[torch.Tensor] = None,
                 y2n_w: Optional[torch.Tensor] = None, y_eps: float = 0.0, mix: Optional[torch.Tensor] = None, out_w: Optional[torch.Tensor] = None,
                 in_w: Optional[torch.Tensor] = None, norm_w: Optional[torch.Tensor] = None, eps: float = 0.0, h: Optional[torch.Tensor] = None,
                 rows: Optional[torch.Tensor] = None, post_w: Optional[torch.Tensor] = None, post_center: bool = False,
                 h_center: bool = False) -> Optional[torch.Tensor]:
    """See i64h_streams_step.  streams fp32 [S, n, W], updated in place when y is given; h fp32 [n, W] (or [rows, W]).  post_w fp32 [W]: a
    norm over the result as a whole (centred with post_center) before it is added; h_center: the read's norm is centred."""
    _chk(streams, torch.float32, "streams")
    S, n, W = streams.shape
    for t, name in ((y, "y"), (y2, "y2"), (yn_w, "yn_w"), (y2n_w, "y2n_w"), (mix, "mix"), (out_w, "out_w"), (in_w, "in_w"), (norm_w, "norm_w"), (h, "h"),
                    (post_w, "post_w")):
        if t is not None:
            _chk(t, torch.float32, name)
    for t, name in ((y, "y"), (y2, "y2")):
        if t is not None and (t.shape[-1] != W or t.numel() < n * W):
            raise _lib.I64HError(f"streams_step: {name} is not [n, W]")
    if (mix is not None and mix.numel() != S * S) or (out_w is not None and out_w.numel() != S) or (in_w is not None and in_w.numel() != S):
        raise _lib.I64HError("streams_step: stream weights do not fit the number of streams")
    if (yn_w is not None and yn_w.numel() != W) or (y2n_w is not None and y2n_w.numel() != W) or (post_w is not None and post_w.numel() != W):
        raise _lib.I64HError("streams_step: result norm weights are not [W]")
    m_rows = n
    if rows is not None:
        _chk(rows, torch.int32, "rows")
        m_rows = rows.numel()
    if h is not None and h.numel() < m_rows * W:
        raise _lib.I64HError("streams_step: h smaller than the rows it receives")
    d = _lib.Streams(streams=ptr(streams), S=S, n=n, W=W, y=ptr(y), ldy=W, y2=ptr(y2), ldy2=W, yn_w=ptr(yn_w), y2n_w=ptr(y2n_w), y_eps=float(y_eps),
                     mix=ptr(mix), out_w=ptr(out_w), in_w=ptr(in_w), norm_w=ptr(norm_w), norm_w_len=norm_w.numel() if norm_w is not None else 0,
                     eps=float(eps), h=ptr(h), rows=ptr(rows), m_rows=m_rows, post_w=ptr(post_w), post_center=int(bool(post_center)), h_center=int(bool(h_center)))
    call_dense("i64h_streams_step", _ref(d), _stream())
    return h


def causal_conv(p: torch.Tensor, *, off: int, channels: int, w: torch.Tensor, bias: Optional[torch.Tensor], positions: torch.Tensor,
                slot_ids: torch.Tensor, state: Optional[torch.Tensor], out: torch.Tensor, n: Optional[int] = None, added: bool = False,
                single_rows: bool = False) -> torch.Tensor:
    """See i64h_causal_conv.  p fp32 [n, ldp]; w fp32 [channels, taps]; state fp32 [slots, taps - 1, channels]; out fp32 [n, channels].
    added: the convolution is added to its own input and no activation follows (mode 1).  single_rows: the caller vouches that every row
    is the only row of its sequence in this launch; the carried inputs are then stored by the same launch."""
    _chk(p, torch.float32, "p"), _chk(w, torch.float32, "w"), _chk(out, torch.float32, "out")
    _chk(positions, torch.int32, "positions"), _chk(slot_ids, torch.int32, "slot_ids")
    rows = int(n if n is not None else positions.numel())
    taps = w.shape[-1]
    if state is None:
        if taps > 1:
            raise _lib.I64HError("causal_conv: more than one tap needs the carried inputs")
        state = out      # (never read or written with one tap)
    _chk(state, torch.float32, "state")
    _rows_ok("causal_conv", rows, positions, slot_ids)
    if bias is not None:
        _chk(bias, torch.float32, "bias")
    if w.shape[0] != channels or off + channels > p.shape[-1] or p.numel() < rows * p.shape[-1] or out.numel() < rows * channels or \
            (bias is not None and bias.numel() != channels) or (taps > 1 and (state.shape[-1] != channels or state.shape[-2] != taps - 1)):
        raise _lib.I64HError("causal_conv: shapes do not fit the sizes")
    d = _lib.CausalConv(P=ptr(p), ldp=p.shape[-1], off=off, channels=channels, taps=taps, w=ptr(w), bias=ptr(bias), positions=ptr(positions),
                        slot_ids=ptr(slot_ids), state=ptr(state), out=ptr(out), ldo=channels, n=rows, mode=1 if added else 0, single_rows=int(bool(single_rows)))
    call_dense("i64h_causal_conv", _ref(d), _stream())
    return out


def ssm_scan(xbc: torch.Tensor, dt: torch.Tensor, *, dt_off: int, lddt: int, dt_bias: torch.Tensor, a_log: torch.Tensor, d_skip: torch.Tensor,
             heads: int, vdim: int, state: int, groups: int, seg_start: torch.Tensor, nseg: int, positions: torch.Tensor, slot_ids: torch.Tensor,
             ssm_state: torch.Tensor, y: torch.Tensor, n: int) -> torch.Tensor:
    """See i64h_ssm_scan.  xbc fp32 [n, heads * vdim + 2 * groups * state]; dt: the matrix whose columns [dt_off, + heads) hold the raw
    steps (row stride lddt); ssm_state fp32 [slots, heads, vdim, state]; y fp32 [n, heads * vdim]."""
    for t, name in ((xbc, "xbc"), (dt, "dt"), (dt_bias, "dt_bias"), (a_log, "a_log"), (d_skip, "d_skip"), (ssm_state, "ssm_state"), (y, "y")):
        _chk(t, torch.float32, name)
    _chk(seg_start, torch.int32, "seg_start"), _chk(positions, torch.int32, "positions"), _chk(slot_ids, torch.int32, "slot_ids")
    inner = heads * vdim
    _rows_ok("ssm_scan", n, positions, slot_ids)
    if xbc.shape[-1] != inner + 2 * groups * state or xbc.numel() < n * xbc.shape[-1] or y.numel() < n * inner or dt.numel() < (n - 1) * lddt + dt_off + heads or \
            min(dt_bias.numel(), a_log.numel(), d_skip.numel()) < heads or tuple(ssm_state.shape[1:]) != (heads, vdim, state) or seg_start.numel() < nseg + 1:
        raise _lib.I64HError("ssm_scan: shapes do not fit the sizes")
    d = _lib.SsmScan(xbc=ptr(xbc), ldx=xbc.shape[-1], dt=ptr(dt) + 4 * dt_off, lddt=lddt, dt_bias=ptr(dt_bias), A_log=ptr(a_log), Dskip=ptr(d_skip),
                     heads=heads, vdim=vdim, state=state, groups=groups, seg_start=ptr(seg_start), nseg=nseg, positions=ptr(positions),
                     slot_ids=ptr(slot_ids), ssm_state=ptr(ssm_state), y=ptr(y), ldy=inner, n=n)
    call_dense("i64h_ssm_scan", _ref(d), _stream())
    return y


def gate_norm(y: torch.Tensor, w: torch.Tensor, out: torch.Tensor, *, groups: int, eps: float, z: Optional[torch.Tensor] = None, z_off: int = 0,
              ldz: int = 0, n: Optional[int] = None, gate_after: bool = False, width: Optional[int] = None) -> torch.Tensor:
    """out = rms_groups(y * silu(z)) * w: see i64h_gate_norm.  y, out fp32 [n, width]; z the columns [z_off, + width) of a matrix of row stride ldz.
    gate_after: out = rms_groups(y) * w * silu(z).  width (default: w's length): the row's width, w then repeats over it."""
    _chk(y, torch.float32, "y"), _chk(w, torch.float32, "w"), _chk(out, torch.float32, "out")
    w_len = w.numel()
    width = int(width if width is not None else w_len)
    if width % w_len:
        raise _lib.I64HError("gate_norm: the weights do not repeat evenly over the row")
    rows = int(n if n is not None else y.numel() // width)
    if y.numel() < rows * width or out.numel() < rows * width:
        raise _lib.I64HError("gate_norm: operand smaller than the launch reads or writes")
    if z is not None:
        _chk(z, torch.float32, "z")
        if z.numel() < (rows - 1) * ldz + z_off + width:
            raise _lib.I64HError("gate_norm: gate smaller than the launch reads")
    d = _lib.GateNorm(y=ptr(y), ldy=width, z=(ptr(z) + 4 * z_off) if z is not None else 0, ldz=ldz, w=ptr(w), width=width, groups=groups, eps=float(eps),
                      out=ptr(out), ldo=width, n=rows, gate_after=int(bool(gate_after)), w_len=w_len if w_len != width else 0)
    call_dense("i64h_gate_norm", _ref(d), _stream())
    return out


def mingru_scan(p: torch.Tensor, *, z_off: int, x_off: int, g_off: int, width: int, seg_start: torch.Tensor, nseg: int, positions: torch.Tensor,
                slot_ids: torch.Tensor, state: torch.Tensor, out: torch.Tensor, n: int) -> torch.Tensor:
    """See i64h_mingru_scan.  p fp32 [n, ldp]; state fp32 [slots, width]; out fp32 [n, width]."""
    _chk(p, torch.float32, "p"), _chk(state, torch.float32, "state"), _chk(out, torch.float32, "out")
    _chk(seg_start, torch.int32, "seg_start"), _chk(positions, torch.int32, "positions"), _chk(slot_ids, torch.int32, "slot_ids")
    _rows_ok("mingru_scan", n, positions, slot_ids)
    if max(z_off, x_off, g_off) + width > p.shape[-1] or p.numel() < n * p.shape[-1] or out.numel() < n * width or state.shape[-1] != width or \
            seg_start.numel() < nseg + 1:
        raise _lib.I64HError("mingru_scan: shapes do not fit the sizes")
    d = _lib.MinGruScan(P=ptr(p), ldp=p.shape[-1], z_off=z_off, x_off=x_off, g_off=g_off, width=width, seg_start=ptr(seg_start), nseg=nseg,
                        positions=ptr(positions), slot_ids=ptr(slot_ids), state=ptr(state), out=ptr(out), ldo=width, n=n)
    call_dense("i64h_mingru_scan", _ref(d), _stream())
    return out


def kattn_prep(p: torch.Tensor, *, q_off: int, k_off: int, heads: int, kv_heads: int, dim: int, q_norm_w: torch.Tensor, k_norm_w: torch.Tensor,
               temp: Optional[torch.Tensor], scale: float, eps: float, positions: torch.Tensor, slot_ids: torch.Tensor, block_table: torch.Tensor,
               cache: torch.Tensor, kscale: torch.Tensor, q: torch.Tensor, n: Optional[int] = None) -> None:
    """See i64h_kattn_prep.  cache [blocks, block, kv_heads * dim] fp32 / bf16; kscale fp32 [blocks, block]; q fp32 [n, heads * dim]."""
    _chk(p, torch.float32, "p"), _chk(q_norm_w, torch.float32, "q_norm_w"), _chk(k_norm_w, torch.float32, "k_norm_w"), _chk(q, torch.float32, "q")
    _chk(kscale, torch.float32, "kscale"), _chk(cache, None, "cache")
    _chk(positions, torch.int32, "positions"), _chk(slot_ids, torch.int32, "slot_ids"), _chk(block_table, torch.int32, "block_table")
    rows = int(n if n is not None else positions.numel())
    _rows_ok("kattn_prep", rows, positions, slot_ids)
    if temp is not None:
        _chk(temp, torch.float32, "temp")
    if cache.shape[-1] != kv_heads * dim or kscale.numel() != cache.shape[0] * cache.shape[1] or q.numel() < rows * heads * dim or \
            q_norm_w.numel() != heads * dim or k_norm_w.numel() != kv_heads * dim or (temp is not None and temp.numel() != heads) or \
            max(q_off + heads * dim, k_off + kv_heads * dim) > p.shape[-1] or p.numel() < rows * p.shape[-1]:
        raise _lib.I64HError("kattn_prep: shapes do not fit the sizes")
    d = _lib.KAttnPrep(P=ptr(p), ldp=p.shape[-1], q_off=q_off, k_off=k_off, heads=heads, kv_heads=kv_heads, dim=dim, q_norm_w=ptr(q_norm_w),
                       k_norm_w=ptr(k_norm_w), temp=ptr(temp), scale=float(scale), eps=float(eps), positions=ptr(positions), slot_ids=ptr(slot_ids),
                       block_table=ptr(block_table), max_blocks_per_seq=block_table.shape[1], block_size=cache.shape[-2], cache=ptr(cache),
                       cache_dtype=CACHE_DTYPE_CODE[cache.dtype], kscale=ptr(kscale), Q=ptr(q), n=rows)
    call_dense("i64h_kattn_prep", _ref(d), _stream())


def kattn(q: torch.Tensor, cache: torch.Tensor, kscale: torch.Tensor, block_table: torch.Tensor, slot_ids: torch.Tensor, positions: torch.Tensor, *,
          chunk: int, bias: Optional[torch.Tensor], sink: bool, heads: int, kv_heads: int, dim: int, out: torch.Tensor, n: Optional[int] = None,
          mode: int = 0, splits: int = 1, workspace: Optional[torch.Tensor] = None, vdim: int = 0, softcap: float = 0.0) -> torch.Tensor:
    """See i64h_kattn.  q, out fp32 [n, heads * dim]; bias fp32 [distances, heads].  vdim > 0: separate values - the cache rows are
    [kv_heads, vdim + dim], q fp32 [n, heads, vdim + dim], out fp32 [n, heads * vdim], kscale may be None."""
    _chk(q, torch.float32, "q"), _chk(out, torch.float32, "out"), _chk(cache, None, "cache")
    if kscale is not None or vdim <= 0:
        _chk(kscale, torch.float32, "kscale")
    _chk(positions, torch.int32, "positions"), _chk(slot_ids, torch.int32, "slot_ids"), _chk(block_table, torch.int32, "block_table")
    rows = int(n if n is not None else positions.numel())
    _rows_ok("kattn", rows, positions, slot_ids)
    if bias is not None:
        _chk(bias, torch.float32, "bias")
        if bias.dim() != 2 or bias.shape[1] != heads:
            raise _lib.I64HError("kattn: bias is not [distances, heads]")
    gs, vals = (vdim + dim, vdim) if vdim > 0 else (dim, dim)
    if cache.shape[-1] != kv_heads * gs or (kscale is not None and kscale.numel() != cache.shape[0] * cache.shape[1]) or q.numel() < rows * heads * gs or \
            out.numel() < rows * heads * vals:
        raise _lib.I64HError("kattn: shapes do not fit the sizes")
    if splits > 1:
        need = kattn_workspace_floats(rows, heads, kv_heads, vals, splits)
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.float32, device=q.device)
        _chk(workspace, torch.float32, "workspace")
        if workspace.numel() < need:
            raise _lib.I64HError(f"kattn: workspace of {workspace.numel()} floats, {need} needed")
    d = _lib.KAttn(Q=ptr(q), cache=ptr(cache), cache_dtype=CACHE_DTYPE_CODE[cache.dtype], kscale=ptr(kscale), block_table=ptr(block_table),
                   max_blocks_per_seq=block_table.shape[1], block_size=cache.shape[-2], slot_ids=ptr(slot_ids), positions=ptr(positions), chunk=int(chunk),
                   bias=ptr(bias), bias_rows=bias.shape[0] if bias is not None else 0, sink=int(bool(sink)), out=ptr(out), n=rows, heads=heads,
                   kv_heads=kv_heads, dim=dim, mode=int(mode), splits=int(splits) if splits > 1 else 1, workspace=ptr(workspace) if splits > 1 else 0,
                   vdim=int(vdim), softcap=float(softcap))
    call_dense("i64h_kattn", _ref(d), _stream())
    return out


def kattn_workspace_floats(n: int, heads: int, kv_heads: int, dim: int, splits: int) -> int:
    return int(_lib.load_dense().i64h_kattn_workspace_floats(n, heads, kv_heads, dim, splits))


def kv_prep(p: torch.Tensor, *, q_off: int, k_off: int, v_off: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, positions: torch.Tensor,
            slot_ids: torch.Tensor, block_table: torch.Tensor, cache: Optional[torch.Tensor], q: torch.Tensor, n: Optional[int] = None,
            block_size: int = 0) -> None:
    """See i64h_kv_prep.  cache [blocks, block, kv_heads * (vdim + dim)] fp32 / bf16 or None (queries only: the rows are another layer's);
    q fp32 [n, heads, vdim + dim]."""
    _chk(p, torch.float32, "p"), _chk(q, torch.float32, "q")
    _chk(positions, torch.int32, "positions"), _chk(slot_ids, torch.int32, "slot_ids"), _chk(block_table, torch.int32, "block_table")
    rows = int(n if n is not None else positions.numel())
    _rows_ok("kv_prep", rows, positions, slot_ids)
    gs = vdim + dim
    if q.numel() < rows * heads * gs or q_off + heads * dim > p.shape[-1] or p.numel() < rows * p.shape[-1]:
        raise _lib.I64HError("kv_prep: shapes do not fit the sizes")
    if cache is not None:
        _chk(cache, None, "cache")
        if cache.shape[-1] != kv_heads * gs or max(k_off + kv_heads * dim, v_off + kv_heads * vdim) > p.shape[-1]:
            raise _lib.I64HError("kv_prep: cache rows or projection columns do not fit the sizes")
    d = _lib.KvPrep(P=ptr(p), ldp=p.shape[-1], q_off=q_off, k_off=k_off, v_off=v_off, heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=float(scale),
                    positions=ptr(positions), slot_ids=ptr(slot_ids), block_table=ptr(block_table), max_blocks_per_seq=block_table.shape[1],
                    block_size=cache.shape[-2] if cache is not None else int(block_size), cache=ptr(cache),
                    cache_dtype=CACHE_DTYPE_CODE[cache.dtype] if cache is not None else 0, Q=ptr(q), n=rows)
    call_dense("i64h_kv_prep", _ref(d), _stream())


def rot_prep(p: torch.Tensor, *, q_off: int, k_off: int, v_off: int, heads: int, kv_heads: int, dim: int, vdim: int, q_norm_w: Optional[torch.Tensor],
             k_norm_w: Optional[torch.Tensor], eps: float, rot_dims: int, interleaved: bool, inv_freq: Optional[torch.Tensor], rot_mult: float,
             head_norm: bool, v_freq: Optional[torch.Tensor], scale: float, positions: torch.Tensor, slot_ids: torch.Tensor, block_table: torch.Tensor,
             cache: torch.Tensor, q: torch.Tensor, n: Optional[int] = None) -> None:
    """See i64h_rot_prep.  cache [blocks, block, kv_heads * (vdim + dim)] fp32 / bf16; q fp32 [n, heads, vdim + dim]; inv_freq fp32 [rot_dims / 2];
    v_freq fp32 [vdim / 2] or None."""
    _chk(p, torch.float32, "p"), _chk(q, torch.float32, "q"), _chk(cache, None, "cache")
    _chk(positions, torch.int32, "positions"), _chk(slot_ids, torch.int32, "slot_ids"), _chk(block_table, torch.int32, "block_table")
    rows = int(n if n is not None else positions.numel())
    _rows_ok("rot_prep", rows, positions, slot_ids)
    gs = vdim + dim
    if q.numel() < rows * heads * gs or max(q_off + heads * dim, k_off + kv_heads * dim, v_off + kv_heads * vdim) > p.shape[-1] or p.numel() < rows * p.shape[-1] or \
            cache.shape[-1] != kv_heads * gs:
        raise _lib.I64HError("rot_prep: shapes do not fit the sizes")
    for t, name, size in ((q_norm_w, "q_norm_w", heads * dim), (k_norm_w, "k_norm_w", kv_heads * dim), (inv_freq, "inv_freq", rot_dims // 2), (v_freq, "v_freq", vdim // 2)):
        if t is not None:
            _chk(t, torch.float32, name)
            if t.numel() < size:
                raise _lib.I64HError(f"rot_prep: {name} has {t.numel()} values, {size} needed")
    if rot_dims and inv_freq is None:
        raise _lib.I64HError("rot_prep: rotated dimensions without frequencies")
    d = _lib.RotPrep(P=ptr(p), ldp=p.shape[-1], q_off=q_off, k_off=k_off, v_off=v_off, heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, q_norm_w=ptr(q_norm_w),
                     k_norm_w=ptr(k_norm_w), eps=float(eps), rot_dims=int(rot_dims), interleaved=int(bool(interleaved)), inv_freq=ptr(inv_freq), rot_mult=float(rot_mult),
                     head_norm=int(bool(head_norm)), v_freq=ptr(v_freq), scale=float(scale), positions=ptr(positions), slot_ids=ptr(slot_ids),
                     block_table=ptr(block_table), max_blocks_per_seq=block_table.shape[1], block_size=cache.shape[-2], cache=ptr(cache),
                     cache_dtype=CACHE_DTYPE_CODE[cache.dtype], Q=ptr(q), n=rows)
    call_dense("i64h_rot_prep", _ref(d), _stream())


def rot_post(o: torch.Tensor, *, heads: int, vdim: int, interleaved: bool, v_freq: Optional[torch.Tensor], positions: torch.Tensor,
             gate: Optional[torch.Tensor] = None, gate_off: int = 0, ldg: int = 0, n: Optional[int] = None) -> torch.Tensor:
    """See i64h_rot_post: o fp32 [n, heads, vdim] turned back by its row's position and gated per head, in place.  gate: the columns
    [gate_off, + heads) of a matrix of row stride ldg."""
    _chk(o, torch.float32, "o"), _chk(positions, torch.int32, "positions")
    rows = int(n if n is not None else positions.numel())
    _rows_ok("rot_post", rows, positions)
    if o.numel() < rows * heads * vdim:
        raise _lib.I64HError("rot_post: the output rows do not fit the sizes")
    if v_freq is not None:
        _chk(v_freq, torch.float32, "v_freq")
        if v_freq.numel() < vdim // 2:
            raise _lib.I64HError("rot_post: too few frequencies")
    if gate is not None:
        _chk(gate, torch.float32, "gate")
        if gate.numel() < (rows - 1) * ldg + gate_off + heads:
            raise _lib.I64HError("rot_post: gate smaller than the launch reads")
    d = _lib.RotPost(O=ptr(o), heads=heads, vdim=vdim, interleaved=int(bool(interleaved)), v_freq=ptr(v_freq), positions=ptr(positions),
                     gate=(ptr(gate) + 4 * gate_off) if gate is not None else 0, ldg=int(ldg), n=rows)
    call_dense("i64h_rot_post", _ref(d), _stream())
    return o


def _gdn_args(x: torch.Tensor, g: torch.Tensor, *, q_off: int, k_off: int, v_off: int, heads: int, kv_heads: int, dim: int, vdim: int, n: int, **rest) -> "_lib.Gdn":
    _chk(x, torch.float32, "x"), _chk(g, torch.float32, "g")
    ld = x.shape[-1]
    if max(q_off, k_off) + kv_heads * dim > ld or v_off + heads * vdim > ld or x.numel() < n * ld or g.numel() < n * 2 * heads:
        raise _lib.I64HError("gdn: columns outside the rows, or too few gate rows")
    return _lib.Gdn(X=ptr(x), ldx=ld, q_off=q_off, k_off=k_off, v_off=v_off, heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, G=ptr(g), n=n, **rest)


def gdn_gates(x: torch.Tensor, g: torch.Tensor, raw: torch.Tensor, *, q_off: int, k_off: int, v_off: int, heads: int, kv_heads: int, dim: int, vdim: int,
              b_off: int, a_off: int, a_log: torch.Tensor, dt_bias: torch.Tensor, unit_eps: float, q_scale: float, n: int) -> None:
    """See i64h_gdn_gates: unit-vector queries and keys in place on x fp32 [n, ldx]; g fp32 [n, 2 * heads] receives write strength and decay from
    the columns b_off / a_off of raw fp32 [n, ldr]."""
    _chk(raw, torch.float32, "raw"), _chk(a_log, torch.float32, "a_log"), _chk(dt_bias, torch.float32, "dt_bias")
    if max(b_off, a_off) + heads > raw.shape[-1] or raw.numel() < n * raw.shape[-1] or min(a_log.numel(), dt_bias.numel()) < heads:
        raise _lib.I64HError("gdn_gates: shapes do not fit the sizes")
    d = _gdn_args(x, g, q_off=q_off, k_off=k_off, v_off=v_off, heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, n=n, R=ptr(raw), ldr=raw.shape[-1],
                  b_off=b_off, a_off=a_off, A_log=ptr(a_log), dt_bias=ptr(dt_bias), unit_eps=float(unit_eps), q_scale=float(q_scale))
    call_dense("i64h_gdn_gates", _ref(d), _stream())


def gdn_scan(x: torch.Tensor, g: torch.Tensor, *, q_off: int, k_off: int, v_off: int, heads: int, kv_heads: int, dim: int, vdim: int, seg_start: torch.Tensor,
             nseg: int, positions: torch.Tensor, slot_ids: torch.Tensor, state: torch.Tensor, out: torch.Tensor, n: int) -> torch.Tensor:
    """See i64h_gdn_scan.  state fp32 [slots, heads, vdim, dim]; out fp32 [n, heads * vdim]."""
    _chk(state, torch.float32, "state"), _chk(out, torch.float32, "out")
    _chk(seg_start, torch.int32, "seg_start"), _chk(positions, torch.int32, "positions"), _chk(slot_ids, torch.int32, "slot_ids")
    _rows_ok("gdn_scan", n, positions, slot_ids)
    if tuple(state.shape[1:]) != (heads, vdim, dim) or out.numel() < n * heads * vdim or seg_start.numel() < nseg + 1:
        raise _lib.I64HError("gdn_scan: shapes do not fit the sizes")
    d = _gdn_args(x, g, q_off=q_off, k_off=k_off, v_off=v_off, heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, n=n, seg_start=ptr(seg_start), nseg=nseg,
                  positions=ptr(positions), slot_ids=ptr(slot_ids), state=ptr(state), out=ptr(out), ldo=heads * vdim)
    call_dense("i64h_gdn_scan", _ref(d), _stream())
    return out


def _gla_args(p: torch.Tensor, *, q_off: int, f_off: int, v_off: int, heads: int, dim: int, vdim: int, k_off: int = -1, lower: Optional[torch.Tensor] = None,
              q_act: bool = False, n: int, **rest) -> "_lib.Gla":
    _chk(p, torch.float32, "p")
    if lower is not None:
        _chk(lower, torch.float32, "lower")
        if lower.numel() != heads * dim:
            raise _lib.I64HError("gla: the gate's lower bounds are not [heads * dim]")
    ld = p.shape[-1]
    if max(q_off, f_off, max(k_off, 0)) + heads * dim > ld or v_off + heads * vdim > ld or p.numel() < n * ld:
        raise _lib.I64HError("gla: projection columns outside the projection rows")
    return _lib.Gla(P=ptr(p), ldp=ld, q_off=q_off, f_off=f_off, k_off=k_off, v_off=v_off, heads=heads, dim=dim, vdim=vdim, lower=ptr(lower),
                    q_act=int(bool(q_act)), n=n, **rest)


def gla_gates(p: torch.Tensor, *, q_off: int, f_off: int, v_off: int, heads: int, dim: int, vdim: int, lower: Optional[torch.Tensor], q_act: bool,
              n: int) -> None:
    """See i64h_gla_gates: q <- silu(q) (q_act), f <- lower + (1 - lower) * sigmoid(f), in place on the projection rows p fp32 [n, ldp]."""
    d = _gla_args(p, q_off=q_off, f_off=f_off, v_off=v_off, heads=heads, dim=dim, vdim=vdim, lower=lower, q_act=q_act, n=n)
    call_dense("i64h_gla_gates", _ref(d), _stream())


def gla_scan(p: torch.Tensor, *, q_off: int, f_off: int, v_off: int, heads: int, dim: int, vdim: int, seg_start: torch.Tensor, nseg: int,
             positions: torch.Tensor, slot_ids: torch.Tensor, state: torch.Tensor, out: torch.Tensor, n: int, k_off: int = -1) -> torch.Tensor:
    """See i64h_gla_scan.  state fp32 [slots, heads, vdim, dim]; out fp32 [n, heads * vdim]; k_off < 0: the key is one minus the decay."""
    _chk(state, torch.float32, "state"), _chk(out, torch.float32, "out")
    _chk(seg_start, torch.int32, "seg_start"), _chk(positions, torch.int32, "positions"), _chk(slot_ids, torch.int32, "slot_ids")
    _rows_ok("gla_scan", n, positions, slot_ids)
    if tuple(state.shape[1:]) != (heads, vdim, dim) or out.numel() < n * heads * vdim or seg_start.numel() < nseg + 1:
        raise _lib.I64HError("gla_scan: shapes do not fit the sizes")
    d = _gla_args(p, q_off=q_off, f_off=f_off, v_off=v_off, heads=heads, dim=dim, vdim=vdim, k_off=k_off, n=n, seg_start=ptr(seg_start), nseg=nseg,
                  positions=ptr(positions), slot_ids=ptr(slot_ids), state=ptr(state), out=ptr(out), ldo=heads * vdim)
    call_dense("i64h_gla_scan", _ref(d), _stream())
    return out


def route_topk(logits: Optional[torch.Tensor], *, entries: int, correction: Optional[torch.Tensor], groups: int, keep: int, top: int, scale: float, idx: torch.Tensor,
               wgt: torch.Tensor, n: Optional[int] = None, h: Optional[torch.Tensor] = None, w: Optional[torch.Tensor] = None) -> None:
    """See i64h_route_topk.  logits fp32 [n, ld >= entries], or None with h fp32 [n, K] and w bf16 [entries, K]: the launch computes the
    logits itself in 32 bits; idx int32 [n, top]; wgt fp32 [n, top]."""
    _chk(idx, torch.int32, "idx"), _chk(wgt, torch.float32, "wgt")
    if logits is None:
        if h is None or w is None:
            raise _lib.I64HError("route_topk: logits, or the router's input and weight")
        _chk(h, torch.float32, "h"), _chk(w, torch.bfloat16, "w")
        rows = int(n if n is not None else h.shape[0])
        if w.dim() != 2 or w.shape[0] != entries or h.shape[-1] != w.shape[1] or h.numel() < rows * h.shape[-1]:
            raise _lib.I64HError("route_topk: the router's input and weight do not fit the sizes")
    else:
        _chk(logits, torch.float32, "logits")
        rows = int(n if n is not None else logits.shape[0])
        if logits.shape[-1] < entries or logits.numel() < rows * logits.shape[-1]:
            raise _lib.I64HError("route_topk: shapes do not fit the sizes")
    if correction is not None:
        _chk(correction, torch.float32, "correction")
        if correction.numel() != entries:
            raise _lib.I64HError("route_topk: the correction is not [entries]")
    if idx.numel() < rows * top or wgt.numel() < rows * top:
        raise _lib.I64HError("route_topk: shapes do not fit the sizes")
    d = _lib.Route(logits=ptr(logits), ld=logits.shape[-1] if logits is not None else 0, E=entries, correction=ptr(correction), groups=int(groups), keep=int(keep),
                   top=int(top), scale=float(scale), idx=ptr(idx), wgt=ptr(wgt), n=rows, h=ptr(h) if logits is None else 0,
                   ldh=h.shape[-1] if logits is None else 0, W=ptr(w) if logits is None else 0, K=w.shape[1] if logits is None else 0)
    call_dense("i64h_route_topk", _ref(d), _stream())


def moe_plan(idx: torch.Tensor, *, n: int, top: int, experts: int, group_off: torch.Tensor, pair_token: torch.Tensor, pair_row: torch.Tensor) -> None:
    """See i64h_moe_plan."""
    for t, name in ((idx, "idx"), (group_off, "group_off"), (pair_token, "pair_token"), (pair_row, "pair_row")):
        _chk(t, torch.int32, name)
    if idx.numel() < n * top or group_off.numel() < experts + 1 or pair_token.numel() < n * top or pair_row.numel() < n * top:
        raise _lib.I64HError("moe_plan: shapes do not fit the sizes")
    d = _lib.MoePlan(idx=ptr(idx), n=n, top=top, experts=experts, group_off=ptr(group_off), pair_token=ptr(pair_token), pair_row=ptr(pair_row))
    call_dense("i64h_moe_plan", _ref(d), _stream())


def moe_combine(y: torch.Tensor, pair_row: torch.Tensor, wgt: torch.Tensor, h: torch.Tensor, shared: Optional[torch.Tensor], out: torch.Tensor, *,
                n: int, top: int, width: int) -> torch.Tensor:
    """See i64h_moe_combine.  y fp32 [pairs, width]; h, shared, out fp32 [n, width]."""
    _chk(y, torch.float32, "y"), _chk(pair_row, torch.int32, "pair_row"), _chk(wgt, torch.float32, "wgt"), _chk(h, torch.float32, "h"), _chk(out, torch.float32, "out")
    if shared is not None:
        _chk(shared, torch.float32, "shared")
    if min(h.numel(), out.numel(), shared.numel() if shared is not None else out.numel()) < n * width or min(pair_row.numel(), wgt.numel()) < n * top or \
            y.numel() < n * top * width:
        raise _lib.I64HError("moe_combine: shapes do not fit the sizes")
    d = _lib.MoeCombine(Y=ptr(y), pair_row=ptr(pair_row), wgt=ptr(wgt), h=ptr(h), shared=ptr(shared), out=ptr(out), n=n, top=top, W=width)
    call_dense("i64h_moe_combine", _ref(d), _stream())
    return out


def sample_rows(logits: torch.Tensor, out: Optional[torch.Tensor] = None, temperature: Optional[torch.Tensor] = None,
                top_k: Optional[torch.Tensor] = None, top_p: Optional[torch.Tensor] = None, u: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token per row (see i64h_sample_rows); with no temperature tensor every row is greedy."""
    _chk(logits, torch.float32, "logits")
    rows, V = logits.shape
    if out is None:
        out = torch.empty(rows, dtype=torch.int64, device=logits.device)
    for t, dt, name in ((temperature, torch.float32, "temperature"), (top_k, torch.int32, "top_k"), (top_p, torch.float32, "top_p"), (u, torch.float32, "u")):
        if t is not None:
            _chk(t, dt, name)
            assert t.numel() == rows
    call_dense("i64h_sample_rows", ptr(logits), ptr(out), rows, V, ptr(temperature), ptr(top_k), ptr(top_p), ptr(u), _stream())
    return out
