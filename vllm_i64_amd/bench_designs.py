"""`bench.py --design morilorn | dogalorn | zabutar | fukatar`: prefill and decode throughput of a registered design at layer sizes of real models
(random weights), beside the package's closest existing model at equal width, depth, feed-forward size and batch (Morilorn: the dense
int8 decoder; Dogalorn: Morilorn, which shares its library, bf16 Linears and 32-bit residual; Zabutar: Dogalorn, the other design of
recurrent layers beside attention with a distance bias; Fukatar: Zabutar, the other design with a norm behind every sublayer, a matrix-valued
recurrence and attention over separate keys and values), and the design's kernels one by one against their rooflines beside the like
kernel of that model.  Prints one JSON line."""
from __future__ import annotations

import json
import time

import torch

HBM_GBS, BF16_TFLOPS, I8_TOPS = 8000.0, 2500.0, 5000.0      # MI355X: HBM3E, dense bf16 and dense int8 matrix-core peaks

SIZES = {
    "w1024": dict(width=1024, layers=18, heads=16, dim=32, rot_dim=32, vdim=64, kv_rank=256, ff=4096, window=1024, kv_heads=4),
    "w2048": dict(width=2048, layers=8, heads=32, dim=64, rot_dim=32, vdim=64, kv_rank=256, ff=8192, window=1024, kv_heads=8),
}


def _time(fn, reps: int, warm: int = 3) -> float:
    """Seconds per call, device time between two events around `reps` back-to-back calls."""
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps * 1e-3


def _steps(model, dec_cls, batch, ctx, prefill_rows, prefill_seq, steps, warmup, fill, vocab, dev):
    """(prefill tokens/s, decode tokens/s, decode ms/step): one prefill step of prefill_rows rows (sequences of prefill_seq tokens), then a
    batch of `batch` sequences at context ctx (cache contents synthetic) decoding greedily, the step replayed as a HIP graph."""
    g = torch.Generator().manual_seed(3)
    nseq = prefill_rows // prefill_seq
    ids = torch.randint(0, vocab, (prefill_rows,), generator=g).to(dev)
    pos = torch.arange(prefill_seq, dtype=torch.int32).repeat(nseq).to(dev)
    slots = torch.arange(nseq, dtype=torch.int32).repeat_interleave(prefill_seq).to(dev)
    last = (torch.arange(1, nseq + 1, dtype=torch.int32) * prefill_seq - 1).to(dev)
    for s in range(nseq):
        model.kv.reserve(s, prefill_seq)
    t = _time(lambda: model.forward(ids, pos, slots, (pos + 1).contiguous(), logit_rows=last, tokens_per_seq=[prefill_seq] * nseq), reps=3, warm=2)
    prefill_tps = prefill_rows / t
    for s in range(nseq):
        model.kv.free(s)
    fill(model)
    dec = dec_cls(model, batch, use_graph=True)
    dec.set_state(torch.randint(0, vocab, (batch,), generator=g).to(dev), [ctx] * batch, reserve_extra=steps + warmup + 2)
    for _ in range(warmup):
        dec.step()
    torch.cuda.synchronize()
    t0 = time.time()
    for _ in range(steps):
        dec.step()
    torch.cuda.synchronize()
    dt = (time.time() - t0) / steps
    return prefill_tps, batch / dt, dt * 1e3


def _kernels(sz, rows, batch, ctx, dev):
    """Device time of single launches at the step's shapes: the design's kernels and the like kernels of the int8 decoder, each with the
    share of its roofline (matrix products of `rows` rows: matrix-core peak; everything else: bytes moved / HBM rate)."""
    from . import ops, ops_dense as D
    W, ff, H, r, rd, vd = sz["width"], sz["ff"], sz["heads"], sz["kv_rank"], sz["rot_dim"], sz["vdim"]
    Dc = r + rd
    out = {}
    g = torch.Generator(device=dev).manual_seed(1)
    rn = lambda *s: torch.randn(*s, device=dev, generator=g)

    def row(name, t, flops=0.0, bytes_=0.0, peak=BF16_TFLOPS):
        share = max(flops / t / (peak * 1e12), bytes_ / t / (HBM_GBS * 1e9))
        out[name] = {"us": round(t * 1e6, 1), "roofline_share": round(share, 3)}

    # ---- matrix products: the feed-forward's first product (gate and up, activation in the epilogue), prefill- and decode-sized ----
    for n, tag in ((rows, "prefill"), (batch, "decode")):
        a = rn(n, W)
        w_gu = (rn(2 * ff, W) * 0.02).to(torch.bfloat16)
        act = torch.empty(n, ff, device=dev)
        t = _time(lambda: D.linear(a, w_gu, act, epilogue=D.EPI_GELU_MUL), 20)
        row(f"linear_bf16_gate_up_{tag}", t, flops=2.0 * n * 2 * ff * W, bytes_=2.0 * 2 * ff * W + 4.0 * n * (W + ff))
        a8 = torch.randint(-127, 127, (n, W), device=dev, dtype=torch.int8)
        rs = torch.ones(n, device=dev)
        w8 = torch.randint(-127, 127, (1, 2 * ff, W), device=dev, dtype=torch.int8)
        ws = torch.ones(1, device=dev)
        o8 = torch.empty(n, ff, device=dev)
        t = _time(lambda: ops.gemm_i8(a8, rs, w8, ws, out=o8, epilogue=ops.EPI_SWIGLU), 20)
        row(f"int8_decoder_gate_up_{tag}", t, flops=2.0 * n * 2 * ff * W, bytes_=1.0 * 2 * ff * W + 1.0 * n * W + 4.0 * n * ff, peak=I8_TOPS)
    # ---- residual + norm ----
    x, y, gp, b, nw = rn(rows, W), rn(rows, W), rn(rows, W), rn(W), rn(W)
    o = torch.empty(rows, W, device=dev)
    t = _time(lambda: D.gated_postnorm(x, nw, 2, 1e-6, alpha=1.0, y=y, gate_pre=gp, ldg=W, gate_bias=b, out=o), 20)
    row("gated_postnorm_prefill", t, bytes_=4.0 * rows * W * 4)
    st = ops.stats_alloc(4, dev)
    t = _time(lambda: ops.fused_residual_norm(x, nw, 1e-6, add=y, h_out=x, normed=o, slot_base=0, stats=st), 20)
    row("int8_decoder_residual_norm_prefill", t, bytes_=4.0 * rows * W * 4)
    # ---- attention: a prompt's rows (sequences of 512 tokens), and one row per sequence at context ctx ----
    for kind in ("prefill", "decode"):
        if kind == "prefill":
            seq = 512
            n, nseq = rows, rows // seq
            pos = torch.arange(seq, dtype=torch.int32).repeat(nseq).to(dev)
            slots = torch.arange(nseq, dtype=torch.int32).repeat_interleave(seq).to(dev)
            per_seq, keys = seq, seq * (seq + 1) / 2 * nseq
        else:
            n, nseq, per_seq = batch, batch, ctx
            pos = torch.full((n,), ctx - 1, dtype=torch.int32, device=dev)
            slots = torch.arange(n, dtype=torch.int32, device=dev)
            keys = float(min(ctx, sz["window"])) * n
        nb = (per_seq + 15) // 16
        bt = torch.arange(nseq * nb, dtype=torch.int32, device=dev).view(nseq, nb).contiguous()
        cache = (rn(nseq * nb, 16, Dc) * 0.5).to(torch.bfloat16)
        q = rn(n, H, Dc) * 0.3
        ol = torch.empty(n, H, r, device=dev)
        # the launch forms the runner picks: a wave per 16 rows and head for prompts; a wave per token with the keys dealt to several waves for decode rows
        sp = 1 if kind == "prefill" else max(1, min(1024 // max(1, n * ((H + 15) // 16)), int(keys / n) // 64, 64))
        wsp = torch.empty(max(1, D.latent_attn_workspace_floats(n, H, r, sp)), device=dev) if sp > 1 else None
        t = _time(lambda: D.latent_attn(q, cache, bt, slots, pos, window=sz["window"], scale=0.1, heads=H, kv_rank=r, rot_dim=rd, out=ol,
                                        mode=3 if kind == "prefill" else 2, splits=sp, workspace=wsp), 5 if kind == "prefill" else 20)
        row(f"latent_attn_{kind}", t, flops=2.0 * keys * H * (Dc + r), bytes_=(2.0 * keys * Dc if kind == "decode" else 0.0) + 4.0 * n * H * (Dc + r))
        kvh, hd = sz["kv_heads"], W // H
        kc = (rn(nseq * nb, 16, kvh, hd) * 0.5).to(torch.bfloat16)
        vc = (rn(nseq * nb, 16, kvh, hd) * 0.5).to(torch.bfloat16)
        q2 = rn(n, H, hd)
        ctxl = (pos + 1).contiguous()
        splits = 1 if kind == "prefill" else 8
        ws = ops.attn_workspace(n, H, hd, splits, dev) if splits > 1 else None
        o2 = torch.empty(n, H, hd, device=dev)
        keys_full = keys if kind == "prefill" else float(ctx) * n
        t = _time(lambda: ops.paged_attn(q2, kc, vc, bt, ctxl, slot_ids=slots, splits=splits, workspace=ws, out=o2), 5 if kind == "prefill" else 20)
        row(f"int8_decoder_paged_attn_{kind}", t, flops=4.0 * keys_full * H * hd, bytes_=(4.0 * keys_full * kvh * hd if kind == "decode" else 0.0) + 8.0 * n * H * hd)
    return out


def run(args) -> dict:
    from . import _lib, synth
    from .config import ModelConfig
    from .model import GreedyDecoder, I64MoEModel
    from .morilorn import MorilornModel
    _lib.load(), _lib.load_dense()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    batch, ctx, rows = args.batch, args.prompt_len, 4096
    result = {"metric": "prefill / decode tokens/s of the Morilorn design beside the dense int8 decoder at equal sizes", "unit": "tokens/s", "n_gpus": 1,
              "steps": args.steps, "warmup": args.warmup, "dtype": "bf16 matrix products, fp32 residual / norms / attention math (Morilorn); int8 dynamic Linears (closest model)",
              "data": "synthetic", "config": {"batch": batch, "context": ctx, "prefill_step": f"{rows} rows = {rows // 512} prompts of 512 tokens"}, "sizes": {}}
    for name in (args.design_sizes.split(",") if args.design_sizes else sorted(SIZES)):
        sz = SIZES[name]
        need_tokens = batch * (ctx + args.steps + args.warmup + 64)

        def fill_latent(m):
            g = torch.Generator(device=dev).manual_seed(5)
            for t in m.kv.rows:
                t.copy_((0.5 * torch.randn(t.shape, device=dev, generator=g)).to(t.dtype))

        def fill_kv(m):
            g = torch.Generator(device=dev).manual_seed(5)
            for l in range(len(m.kv.k)):
                m.kv.k[l].copy_(torch.randn(m.kv.k[l].shape, device=dev, generator=g).to(m.kv.k[l].dtype))
                m.kv.v[l].copy_((0.6 * torch.randn(m.kv.v[l].shape, device=dev, generator=g)).to(m.kv.v[l].dtype))

        cfg = synth.morilorn_config(width=sz["width"], layers=sz["layers"], heads=sz["heads"], dim=sz["dim"], rot_dim=sz["rot_dim"], vdim=sz["vdim"],
                                    kv_rank=sz["kv_rank"], ff=sz["ff"], window=sz["window"])
        model = MorilornModel(cfg, synth.make_morilorn_weights(cfg), device=dev, dtype="bfloat16", max_seqs=batch, num_kv_blocks=need_tokens // 16)
        p, d, ms = _steps(model, GreedyDecoder, batch, ctx, rows, 512, args.steps, args.warmup, fill_latent, cfg.vocab, dev)
        entry = {"morilorn": {"prefill_tokens_per_s": round(p, 1), "decode_tokens_per_s": round(d, 1), "decode_ms_per_step": round(ms, 3),
                              "shape": {k: v for k, v in sz.items() if k != "kv_heads"}}}
        del model
        torch.cuda.empty_cache()
        ccfg = ModelConfig(name=f"dense-{name}", hidden_size=sz["width"], num_layers=sz["layers"], num_heads=sz["width"] // 64, num_kv_heads=sz["kv_heads"],
                           intermediate_size=sz["ff"], num_experts=1, shared_intermediate_size=0, top_k=1, primary_weight=1.0, table_routing=False,
                           max_pos=(ctx + args.steps + args.warmup + 64 + 255) // 256 * 256)
        cm = I64MoEModel(ccfg, synth.make_weights(ccfg, seed=0), device=dev, kv_dtype=torch.bfloat16, max_seqs=batch, num_kv_blocks=need_tokens // 16)
        p, d, ms = _steps(cm, GreedyDecoder, batch, ctx, rows, 512, args.steps, args.warmup, fill_kv, ccfg.vocab_size, dev)
        entry["int8_decoder"] = {"prefill_tokens_per_s": round(p, 1), "decode_tokens_per_s": round(d, 1), "decode_ms_per_step": round(ms, 3),
                                 "shape": {"hidden": ccfg.hidden_size, "layers": ccfg.num_layers, "heads": ccfg.num_heads, "kv_heads": ccfg.num_kv_heads,
                                           "intermediate": ccfg.intermediate_size}}
        del cm
        torch.cuda.empty_cache()
        entry["kernels"] = _kernels(sz, rows, batch, ctx, dev)
        result["sizes"][name] = entry
    first = result["sizes"][sorted(result["sizes"])[0]]["morilorn"]
    result["value"], result["ms_per_step"] = first["decode_tokens_per_s"], first["decode_ms_per_step"]
    result["higher_is_better"], result["scaling"], result["vs_baseline"] = True, "weak", None
    return result


DOGALORN_SIZES = {
    "w1024": dict(width=1024, blocks=4, ssm_heads=32, ssm_vdim=64, ssm_state=128, heads=16, kv_heads=4, dim=64, chunk=4096, gru_width=1024, ff=4096),
    "w2048": dict(width=2048, blocks=2, ssm_heads=64, ssm_vdim=64, ssm_state=128, heads=32, kv_heads=8, dim=64, chunk=4096, gru_width=2048, ff=8192),
}
F32_TFLOPS = 157.0     # fp32 vector rate (what a recurrence that is not a matrix product can reach at most)


def _dogalorn_kernels(sz, rows, batch, ctx, dev):
    """Single launches at the step's shapes with the share of their roofline (matrix products: bf16 matrix peak; recurrences: the larger
    of bytes / HBM rate and flop / fp32 vector rate; everything else: bytes / HBM rate), beside the like kernel of Morilorn."""
    from . import ops_dense as D
    W, ff, H, G, dm = sz["width"], sz["ff"], sz["heads"], sz["kv_heads"], sz["dim"]
    Hs, P, N, R = sz["ssm_heads"], sz["ssm_vdim"], sz["ssm_state"], sz["gru_width"]
    out = {}
    g = torch.Generator(device=dev).manual_seed(1)
    rn = lambda *s: torch.randn(*s, device=dev, generator=g)

    def row(name, t, flops=0.0, bytes_=0.0, peak=BF16_TFLOPS):
        share = max(flops / t / (peak * 1e12), bytes_ / t / (HBM_GBS * 1e9))
        out[name] = {"us": round(t * 1e6, 1), "roofline_share": round(share, 3)}

    seq = 512
    warm_a, warm_w, warm_c = rn(rows, W), (rn(W, W) * 0.02).to(torch.bfloat16), torch.empty(rows, W, device=dev)
    _time(lambda: D.linear(warm_a, warm_w, warm_c), 20)      # clocks and caches settle before the first timed launch
    for n, tag in ((rows, "prefill"), (batch, "decode")):
        nseq = n // seq if tag == "prefill" else n
        per = seq if tag == "prefill" else 1
        pos0 = 0 if tag == "prefill" else ctx - 1
        pos = (torch.arange(per, dtype=torch.int32) + pos0).repeat(nseq).to(dev)
        slots = torch.arange(nseq, dtype=torch.int32).repeat_interleave(per).to(dev)
        seg = (torch.arange(nseq + 1, dtype=torch.int32) * per).to(dev)
        reps = 5 if tag == "prefill" else 20
        # feed-forward up-projection with bias and activation, beside Morilorn's gate / up pair
        a = rn(n, W)
        w_up, b_up = (rn(ff, W) * 0.02).to(torch.bfloat16), rn(ff)
        act = torch.empty(n, ff, device=dev)
        t = _time(lambda: D.linear(a, w_up, act, bias=b_up, epilogue=D.EPI_GELU_ERF), reps)
        row(f"linear_up_bias_gelu_{tag}", t, flops=2.0 * n * ff * W, bytes_=2.0 * ff * W + 4.0 * n * (W + ff))
        w_gu = (rn(2 * ff, W) * 0.02).to(torch.bfloat16)
        t = _time(lambda: D.linear(a, w_gu, act, epilogue=D.EPI_GELU_MUL), reps)
        row(f"morilorn_linear_gate_up_{tag}", t, flops=2.0 * n * 2 * ff * W, bytes_=2.0 * 2 * ff * W + 4.0 * n * (W + ff))
        # multi-stream residual + norm, beside the gated post-norm
        S = 2
        st, y, h = rn(S, n, W), rn(n, W), torch.empty(n, W, device=dev)
        mix, ow, iw, nw = torch.eye(S, device=dev), torch.ones(S, device=dev), torch.full((S,), 0.5, device=dev), torch.ones(1, device=dev)
        t = _time(lambda: D.streams_step(st, y=y, mix=mix, out_w=ow, in_w=iw, norm_w=nw, eps=1e-6, h=h), reps)
        row(f"streams_step_{tag}", t, bytes_=4.0 * n * W * (2 * S + 2))
        gp, bb, nw2, o = rn(n, W), rn(W), rn(W), torch.empty(n, W, device=dev)
        t = _time(lambda: D.gated_postnorm(st[0], nw2, 2, 1e-6, alpha=1.0, y=y, gate_pre=gp, ldg=W, gate_bias=bb, out=o), reps)
        row(f"morilorn_gated_postnorm_{tag}", t, bytes_=4.0 * n * W * 4)
        # state-space layer: convolution, recurrence, gate + norm
        inner, ch = Hs * P, Hs * P + 2 * N
        nin = inner + ch + Hs
        Pm = rn(n, nin) * 0.5
        cw, cb = rn(ch, 4) * 0.3, rn(ch) * 0.1
        cstate, sstate = torch.zeros(nseq, 3, ch, device=dev), torch.zeros(nseq, Hs, P, N, device=dev)
        xbc, yv, gv = torch.empty(n, ch, device=dev), torch.empty(n, inner, device=dev), torch.empty(n, inner, device=dev)
        t = _time(lambda: D.causal_conv(Pm, off=inner, channels=ch, w=cw, bias=cb, positions=pos, slot_ids=slots, state=cstate, out=xbc, n=n), reps)
        row(f"causal_conv_{tag}", t, bytes_=4.0 * n * ch * 2)
        dtb, al, dk = torch.full((Hs,), -2.0, device=dev), torch.zeros(Hs, device=dev), torch.ones(Hs, device=dev)
        t = _time(lambda: D.ssm_scan(xbc, Pm, dt_off=inner + ch, lddt=nin, dt_bias=dtb, a_log=al, d_skip=dk, heads=Hs, vdim=P, state=N, groups=1, seg_start=seg,
                                     nseg=nseq, positions=pos, slot_ids=slots, ssm_state=sstate, y=yv, n=n), reps)
        row(f"ssm_scan_{tag}", t, flops=6.0 * n * Hs * N * P, bytes_=4.0 * n * (ch + inner) + 8.0 * nseq * Hs * N * P, peak=F32_TFLOPS)
        t = _time(lambda: D.gate_norm(yv, torch.ones(inner, device=dev), gv, groups=1, eps=1e-6, z=Pm, z_off=0, ldz=nin, n=n), reps)
        row(f"gate_norm_{tag}", t, bytes_=4.0 * n * inner * 3)
        # gated recurrence
        Pg = rn(n, 3 * R)
        gstate, go = torch.zeros(nseq, R, device=dev), torch.empty(n, R, device=dev)
        t = _time(lambda: D.mingru_scan(Pg, z_off=0, x_off=R, g_off=2 * R, width=R, seg_start=seg, nseg=nseq, positions=pos, slot_ids=slots, state=gstate, out=go, n=n), reps)
        row(f"mingru_scan_{tag}", t, bytes_=4.0 * n * R * 4)
        # attention: a prompt's rows, and one row per sequence at context ctx, beside the latent attention
        plen = seq if tag == "prefill" else ctx
        nb = (plen + 15) // 16
        bt = torch.arange(nseq * nb, dtype=torch.int32, device=dev).view(nseq, nb).contiguous()
        kc = (rn(nseq * nb, 16, G * dm) * 0.5).to(torch.bfloat16)
        ks = torch.rand(nseq * nb, 16, device=dev, generator=g) + 0.5
        q, oa = rn(n, H * dm) * 0.3, torch.empty(n, H * dm, device=dev)
        bias = torch.zeros(sz["chunk"] + 1, H, device=dev)
        keys = seq * (seq + 1) / 2 * nseq if tag == "prefill" else float(min(ctx, sz["chunk"])) * n
        sp = 1 if tag == "prefill" else max(1, min((3072 if dm <= 64 else 1024) // max(1, n * G * ((H // G + 15) // 16)), int(keys / n) // 64, 64))
        t = _time(lambda: D.kattn(q, kc, ks, bt, slots, pos, chunk=sz["chunk"], bias=bias, sink=True, heads=H, kv_heads=G, dim=dm, out=oa, n=n,
                                  mode=3 if tag == "prefill" else 2, splits=sp), reps)
        row(f"kattn_{tag}", t, flops=4.0 * keys * H * dm, bytes_=(2.0 * keys * G * dm if tag == "decode" else 0.0) + 8.0 * n * H * dm)
        r, rd = 256, 32
        Dc = r + rd
        lc = (rn(nseq * nb, 16, Dc) * 0.5).to(torch.bfloat16)
        q2, ol = rn(n, H, Dc) * 0.3, torch.empty(n, H, r, device=dev)
        lkeys = keys if tag == "prefill" else float(min(ctx, 1024)) * n
        sp2 = 1 if tag == "prefill" else max(1, min(1024 // max(1, n * ((H + 15) // 16)), int(lkeys / n) // 64, 64))
        wsp = torch.empty(max(1, D.latent_attn_workspace_floats(n, H, r, sp2)), device=dev) if sp2 > 1 else None
        t = _time(lambda: D.latent_attn(q2, lc, bt, slots, pos, window=1024, scale=0.1, heads=H, kv_rank=r, rot_dim=rd, out=ol, mode=3 if tag == "prefill" else 2,
                                        splits=sp2, workspace=wsp), reps)
        row(f"morilorn_latent_attn_{tag}", t, flops=2.0 * lkeys * H * (Dc + r), bytes_=(2.0 * lkeys * Dc if tag == "decode" else 0.0) + 4.0 * n * H * (Dc + r))
    return out


def run_dogalorn(args) -> dict:
    from . import _lib, synth
    from .dogalorn import DogalornModel
    from .model import GreedyDecoder
    from .morilorn import MorilornModel
    _lib.load(), _lib.load_dense()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    batch, ctx, rows = args.batch, args.prompt_len, 4096
    result = {"metric": "prefill / decode tokens/s of the Dogalorn design beside Morilorn at equal sizes", "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
              "warmup": args.warmup, "dtype": "bf16 matrix products, fp32 residual / norms / recurrences / attention math (both designs)", "data": "synthetic",
              "config": {"batch": batch, "context": ctx, "prefill_step": f"{rows} rows = {rows // 512} prompts of 512 tokens"}, "sizes": {}}
    for name in (args.design_sizes.split(",") if args.design_sizes else sorted(DOGALORN_SIZES)):
        sz = DOGALORN_SIZES[name]
        need_tokens = batch * (ctx + args.steps + args.warmup + 64)

        def fill_hybrid(m):
            g = torch.Generator(device=dev).manual_seed(5)
            for t in m.kv.rows:
                if t is not None:
                    t.copy_((0.5 * torch.randn(t.shape, device=dev, generator=g)).to(t.dtype))
            for t in m.kv.kscale:
                if t is not None:
                    t.fill_(2.0)
            for d in m.kv.state:
                for t in d.values():
                    t.copy_(0.1 * torch.randn(t.shape, device=dev, generator=g))

        def fill_latent(m):
            g = torch.Generator(device=dev).manual_seed(5)
            for t in m.kv.rows:
                t.copy_((0.5 * torch.randn(t.shape, device=dev, generator=g)).to(t.dtype))

        cfg = synth.dogalorn_config(**sz)
        model = DogalornModel(cfg, synth.make_dogalorn_weights(cfg), device=dev, dtype="bfloat16", max_seqs=batch, num_kv_blocks=need_tokens // 16)
        p, d, ms = _steps(model, GreedyDecoder, batch, ctx, rows, 512, args.steps, args.warmup, fill_hybrid, cfg.vocab, dev)
        entry = {"dogalorn": {"prefill_tokens_per_s": round(p, 1), "decode_tokens_per_s": round(d, 1), "decode_ms_per_step": round(ms, 3), "layers": cfg.num_layers,
                              "shape": sz}}
        del model
        torch.cuda.empty_cache()
        mcfg = synth.morilorn_config(width=sz["width"], layers=4 * sz["blocks"], heads=sz["heads"], dim=32, rot_dim=32, vdim=64, kv_rank=256, ff=sz["ff"], window=1024)
        mm = MorilornModel(mcfg, synth.make_morilorn_weights(mcfg), device=dev, dtype="bfloat16", max_seqs=batch, num_kv_blocks=need_tokens // 16)
        p, d, ms = _steps(mm, GreedyDecoder, batch, ctx, rows, 512, args.steps, args.warmup, fill_latent, mcfg.vocab, dev)
        entry["morilorn"] = {"prefill_tokens_per_s": round(p, 1), "decode_tokens_per_s": round(d, 1), "decode_ms_per_step": round(ms, 3), "layers": mcfg.num_layers}
        del mm
        torch.cuda.empty_cache()
        entry["kernels"] = _dogalorn_kernels(sz, rows, batch, ctx, dev)
        result["sizes"][name] = entry
    first = result["sizes"][sorted(result["sizes"])[0]]["dogalorn"]
    result["value"], result["ms_per_step"] = first["decode_tokens_per_s"], first["decode_ms_per_step"]
    result["higher_is_better"], result["scaling"], result["vs_baseline"] = True, "weak", None
    return result


ZABUTAR_SIZES = {
    "w1024": dict(width=1024, blocks=4, rec_heads=8, rec_dim=128, rec_vdim=128, heads=16, kv_heads=4, dim=64, vdim=64, ff=4096, experts=8, top=2, expert_ff=1024,
                  shared_ff=1024),
    "w2048": dict(width=2048, blocks=2, rec_heads=16, rec_dim=128, rec_vdim=128, heads=32, kv_heads=8, dim=64, vdim=64, ff=8192, experts=8, top=2, expert_ff=2048,
                  shared_ff=2048),
}


def _zabutar_kernels(sz, rows, batch, ctx, dev):
    """Single launches at the step's shapes with the share of their roofline (matrix products: bf16 matrix peak over the products the
    design asks for; recurrences: the larger of bytes / HBM rate and flop / fp32 vector rate; everything else: bytes / HBM rate), beside the
    like kernel of Dogalorn."""
    from . import ops_dense as D
    W, ff, H, G, dm, dv = sz["width"], sz["ff"], sz["heads"], sz["kv_heads"], sz["dim"], sz["vdim"]
    Hr, dk, dr = sz["rec_heads"], sz["rec_dim"], sz["rec_vdim"]
    E, top, eff = sz["experts"], sz["top"], sz["expert_ff"]
    dz = DOGALORN_SIZES["w2048" if W >= 2048 else "w1024"]
    out = {}
    g = torch.Generator(device=dev).manual_seed(1)
    rn = lambda *s: torch.randn(*s, device=dev, generator=g)

    def row(name, t, flops=0.0, bytes_=0.0, peak=BF16_TFLOPS):
        share = max(flops / t / (peak * 1e12), bytes_ / t / (HBM_GBS * 1e9))
        out[name] = {"us": round(t * 1e6, 1), "roofline_share": round(share, 3)}

    seq = 512
    warm_a, warm_w, warm_c = rn(rows, W), (rn(W, W) * 0.02).to(torch.bfloat16), torch.empty(rows, W, device=dev)
    _time(lambda: D.linear(warm_a, warm_w, warm_c), 20)      # clocks and caches settle before the first timed launch
    for n, tag in ((rows, "prefill"), (batch, "decode")):
        nseq = n // seq if tag == "prefill" else n
        per = seq if tag == "prefill" else 1
        pos0 = 0 if tag == "prefill" else ctx - 1
        pos = (torch.arange(per, dtype=torch.int32) + pos0).repeat(nseq).to(dev)
        slots = torch.arange(nseq, dtype=torch.int32).repeat_interleave(per).to(dev)
        seg = (torch.arange(nseq + 1, dtype=torch.int32) * per).to(dev)
        reps = 5 if tag == "prefill" else 20
        a = rn(n, W)
        # dense feed-forward: up-projection with bias and activation (the same Linear under both designs, another epilogue)
        w_up, b_up = (rn(ff, W) * 0.02).to(torch.bfloat16), rn(ff)
        act = torch.empty(n, ff, device=dev)
        t = _time(lambda: D.linear(a, w_up, act, bias=b_up, epilogue=D.EPI_XIELU, act_a=0.7, act_b=1.2), reps)
        row(f"linear_up_bias_xielu_{tag}", t, flops=2.0 * n * ff * W, bytes_=2.0 * ff * W + 4.0 * n * (W + ff))
        t = _time(lambda: D.linear(a, w_up, act, bias=b_up, epilogue=D.EPI_GELU_ERF), reps)
        row(f"dogalorn_linear_up_bias_gelu_{tag}", t, flops=2.0 * n * ff * W, bytes_=2.0 * ff * W + 4.0 * n * (W + ff))
        # mixture of experts: router choice, grouping, the two grouped Linears, the weighted sum (beside the dense gate / up pair of equal work)
        ent = E
        w_r = (rn(ent, W) * 0.1).to(torch.bfloat16)
        idx, wgt = torch.empty(n, top, dtype=torch.int32, device=dev), torch.empty(n, top, device=dev)
        corr = torch.zeros(ent, device=dev)
        t = _time(lambda: D.route_topk(None, h=a, w=w_r, entries=ent, correction=corr, groups=4, keep=2, top=top, scale=1.0, idx=idx, wgt=wgt, n=n), reps)
        row(f"route_topk_{tag}", t, bytes_=4.0 * n * (W + 2 * top) + 2.0 * ent * W)
        goff, ptok, prow = torch.empty(E + 1, dtype=torch.int32, device=dev), torch.empty(n * top, dtype=torch.int32, device=dev), torch.empty(n * top, dtype=torch.int32, device=dev)
        t = _time(lambda: D.moe_plan(idx, n=n, top=top, experts=E, group_off=goff, pair_token=ptok, pair_row=prow), reps)
        row(f"moe_plan_{tag}", t, bytes_=4.0 * n * top * 3)
        pairs = int(goff[-1])
        w_gu = (rn(E, 2 * eff, W) * 0.02).to(torch.bfloat16)
        eact, ey = torch.empty(n * top, eff, device=dev), torch.empty(n * top, W, device=dev)
        t = _time(lambda: D.linear(a, w_gu, eact, m=n, a_rows=ptok, batch=E, w_batch=2 * eff * W, epilogue=D.EPI_SILU_MUL, group_off=goff), reps)
        row(f"experts_gate_up_{tag}", t, flops=2.0 * pairs * 2 * eff * W, bytes_=2.0 * E * 2 * eff * W + 4.0 * pairs * (W + eff))
        w_dn = (rn(E, W, eff) * 0.02).to(torch.bfloat16)
        t = _time(lambda: D.linear(eact, w_dn, ey, m=n, batch=E, w_batch=W * eff, group_off=goff), reps)
        row(f"experts_down_{tag}", t, flops=2.0 * pairs * eff * W, bytes_=2.0 * E * eff * W + 4.0 * pairs * (W + eff))
        w_dgu = (rn(2 * top * eff, W) * 0.02).to(torch.bfloat16)      # a dense pair of the same number of products
        dact = torch.empty(n, top * eff, device=dev)
        t = _time(lambda: D.linear(a, w_dgu, dact, epilogue=D.EPI_GELU_MUL), reps)
        row(f"morilorn_linear_gate_up_{tag}", t, flops=2.0 * n * 2 * top * eff * W, bytes_=2.0 * 2 * top * eff * W + 4.0 * n * (W + top * eff))
        sh, yo = rn(n, W), torch.empty(n, W, device=dev)
        t = _time(lambda: D.moe_combine(ey, prow, wgt, a, sh, yo, n=n, top=top, width=W), reps)
        row(f"moe_combine_{tag}", t, bytes_=4.0 * n * W * (top + 3))
        # residual: add the normed result, norm for the next sublayer; beside Dogalorn's two-stream step
        st, y, h = rn(1, n, W), rn(n, W), torch.empty(n, W, device=dev)
        nb_, nw, one = torch.ones(W, device=dev), torch.ones(W, device=dev), torch.ones(1, device=dev)
        t = _time(lambda: D.streams_step(st, y=y, yn_w=nb_, y_eps=1e-6, out_w=one, norm_w=nw, eps=1e-6, h=h), reps)
        row(f"sandwich_residual_{tag}", t, bytes_=4.0 * n * W * 4)
        S = 2
        st2 = rn(S, n, W)
        mix, ow, iw, nw1 = torch.eye(S, device=dev), torch.ones(S, device=dev), torch.full((S,), 0.5, device=dev), torch.ones(1, device=dev)
        t = _time(lambda: D.streams_step(st2, y=y, mix=mix, out_w=ow, in_w=iw, norm_w=nw1, eps=1e-6, h=h), reps)
        row(f"dogalorn_streams_step_{tag}", t, bytes_=4.0 * n * W * (2 * S + 2))
        # the convolution added to every sublayer's input; beside Dogalorn's convolution + silu over the state-space channels
        cw, cstate, hc = rn(W, 4) * 0.1, torch.zeros(nseq, 3, W, device=dev), torch.empty(n, W, device=dev)
        t = _time(lambda: D.causal_conv(a, off=0, channels=W, w=cw, bias=None, positions=pos, slot_ids=slots, state=cstate, out=hc, n=n, added=True), reps)
        row(f"input_conv_{tag}", t, bytes_=4.0 * n * W * 2)
        ch = dz["ssm_heads"] * dz["ssm_vdim"] + 2 * dz["ssm_state"]
        Pm, cw2, cb2 = rn(n, ch), rn(ch, 4) * 0.3, rn(ch) * 0.1
        cstate2, xbc = torch.zeros(nseq, 3, ch, device=dev), torch.empty(n, ch, device=dev)
        t = _time(lambda: D.causal_conv(Pm, off=0, channels=ch, w=cw2, bias=cb2, positions=pos, slot_ids=slots, state=cstate2, out=xbc, n=n), reps)
        row(f"dogalorn_causal_conv_{tag}", t, bytes_=4.0 * n * ch * 2)
        # gated linear recurrence: gates, scan, head norm; beside Dogalorn's state-space scan
        nk, nv = Hr * dk, Hr * dr
        P = rn(n, 2 * nk + nv) * 0.5
        lower = torch.rand(nk, device=dev, generator=g) * 0.9
        cols = dict(q_off=0, f_off=nk, v_off=2 * nk, heads=Hr, dim=dk, vdim=dr, n=n)
        t = _time(lambda: D.gla_gates(P, lower=lower, q_act=True, **cols), reps)
        row(f"gla_gates_{tag}", t, bytes_=4.0 * n * nk * 4)
        P.uniform_(0.0, 1.0)
        rstate, ro, rg = torch.zeros(nseq, Hr, dr, dk, device=dev), torch.empty(n, nv, device=dev), torch.empty(n, nv, device=dev)
        t = _time(lambda: D.gla_scan(P, seg_start=seg, nseg=nseq, positions=pos, slot_ids=slots, state=rstate, out=ro, **cols), reps)
        row(f"gla_scan_{tag}", t, flops=5.0 * n * Hr * dk * dr, bytes_=4.0 * n * (2 * nk + 2 * nv) + 8.0 * nseq * Hr * dk * dr, peak=F32_TFLOPS)
        t = _time(lambda: D.gate_norm(ro, torch.ones(nv, device=dev), rg, groups=Hr, eps=1e-6, n=n), reps)
        row(f"head_norm_{tag}", t, bytes_=4.0 * n * nv * 2)
        Hs, Pv, N = dz["ssm_heads"], dz["ssm_vdim"], dz["ssm_state"]
        inner, chs = Hs * Pv, Hs * Pv + 2 * N
        Ps, xs = rn(n, inner + chs + Hs) * 0.5, rn(n, chs) * 0.5
        sstate, yv = torch.zeros(nseq, Hs, Pv, N, device=dev), torch.empty(n, inner, device=dev)
        dtb, al, dkp = torch.full((Hs,), -2.0, device=dev), torch.zeros(Hs, device=dev), torch.ones(Hs, device=dev)
        t = _time(lambda: D.ssm_scan(xs, Ps, dt_off=inner + chs, lddt=inner + chs + Hs, dt_bias=dtb, a_log=al, d_skip=dkp, heads=Hs, vdim=Pv, state=N, groups=1,
                                     seg_start=seg, nseg=nseq, positions=pos, slot_ids=slots, ssm_state=sstate, y=yv, n=n), reps)
        row(f"dogalorn_ssm_scan_{tag}", t, flops=6.0 * n * Hs * N * Pv, bytes_=4.0 * n * (chs + inner) + 8.0 * nseq * Hs * N * Pv, peak=F32_TFLOPS)
        # attention: a prompt's rows, and one row per sequence at context ctx; beside Dogalorn's attention whose values are the keys
        plen = seq if tag == "prefill" else ctx
        nb = (plen + 15) // 16
        bt = torch.arange(nseq * nb, dtype=torch.int32, device=dev).view(nseq, nb).contiguous()
        gs = dv + dm
        kc = (rn(nseq * nb, 16, G * gs) * 0.5).to(torch.bfloat16)
        Pq = rn(n, H * dm) * 0.3
        q, oa = torch.empty(n, H * gs, device=dev), torch.empty(n, H * dv, device=dev)
        t = _time(lambda: D.kv_prep(Pq, q_off=0, k_off=0, v_off=0, heads=H, kv_heads=G, dim=dm, vdim=dv, scale=0.125, positions=pos, slot_ids=slots, block_table=bt,
                                    cache=None, q=q, n=n, block_size=16), reps)
        row(f"kv_prep_queries_{tag}", t, bytes_=4.0 * n * H * (dm + gs))
        bias = torch.zeros(4097, H, device=dev)
        keys = seq * (seq + 1) / 2 * nseq if tag == "prefill" else float(ctx) * n
        waves = 3072 if gs <= 64 else (2048 if gs <= 128 else 1024)
        sp = 1 if tag == "prefill" else max(1, min(waves // max(1, n * G * ((H // G + 15) // 16)), int(keys / n) // 64, 64))
        t = _time(lambda: D.kattn(q, kc, None, bt, slots, pos, chunk=0, bias=bias, sink=False, heads=H, kv_heads=G, dim=dm, vdim=dv, out=oa, n=n,
                                  mode=3 if tag == "prefill" else 2, splits=sp), reps)
        row(f"kv_attention_{tag}", t, flops=2.0 * keys * H * (dm + dv), bytes_=(2.0 * keys * G * gs if tag == "decode" else 0.0) + 4.0 * n * H * (gs + dv))
        kc2 = (rn(nseq * nb, 16, G * dm) * 0.5).to(torch.bfloat16)
        ks = torch.rand(nseq * nb, 16, device=dev, generator=g) + 0.5
        q2, oa2 = rn(n, H * dm) * 0.3, torch.empty(n, H * dm, device=dev)
        sp2 = 1 if tag == "prefill" else max(1, min((3072 if dm <= 64 else 1024) // max(1, n * G * ((H // G + 15) // 16)), int(keys / n) // 64, 64))
        t = _time(lambda: D.kattn(q2, kc2, ks, bt, slots, pos, chunk=4096, bias=bias, sink=True, heads=H, kv_heads=G, dim=dm, out=oa2, n=n,
                                  mode=3 if tag == "prefill" else 2, splits=sp2), reps)
        row(f"dogalorn_kattn_{tag}", t, flops=4.0 * keys * H * dm, bytes_=(2.0 * keys * G * dm if tag == "decode" else 0.0) + 8.0 * n * H * dm)
    return out


def run_zabutar(args) -> dict:
    from . import _lib, synth
    from .dogalorn import DogalornModel
    from .model import GreedyDecoder
    from .zabutar import ZabutarModel
    _lib.load(), _lib.load_dense()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    batch, ctx, rows = args.batch, args.prompt_len, 4096
    result = {"metric": "prefill / decode tokens/s of the Zabutar design beside Dogalorn at equal sizes", "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
              "warmup": args.warmup, "dtype": "bf16 matrix products, fp32 residual / norms / recurrences / attention math (both designs)", "data": "synthetic",
              "config": {"batch": batch, "context": ctx, "prefill_step": f"{rows} rows = {rows // 512} prompts of 512 tokens"}, "sizes": {}}
    for name in (args.design_sizes.split(",") if args.design_sizes else sorted(ZABUTAR_SIZES)):
        sz = ZABUTAR_SIZES[name]
        need_tokens = batch * (ctx + args.steps + args.warmup + 64)

        def fill(m):
            g = torch.Generator(device=dev).manual_seed(5)
            for t in {id(t): t for t in m.kv.rows if t is not None}.values():
                t.copy_((0.5 * torch.randn(t.shape, device=dev, generator=g)).to(t.dtype))
            for t in m.kv.kscale:
                if t is not None:
                    t.fill_(2.0)
            for d in m.kv.state:
                for t in d.values():
                    t.copy_(0.1 * torch.randn(t.shape, device=dev, generator=g))

        cfg = synth.zabutar_config(max_positions=max(4096, ctx + args.steps + args.warmup + 64), **sz)
        model = ZabutarModel(cfg, synth.make_zabutar_weights(cfg), device=dev, dtype="bfloat16", max_seqs=batch, num_kv_blocks=need_tokens // 16)
        p, d, ms = _steps(model, GreedyDecoder, batch, ctx, rows, 512, args.steps, args.warmup, fill, cfg.vocab, dev)
        entry = {"zabutar": {"prefill_tokens_per_s": round(p, 1), "decode_tokens_per_s": round(d, 1), "decode_ms_per_step": round(ms, 3), "layers": cfg.num_layers,
                             "shape": sz}}
        del model
        torch.cuda.empty_cache()
        dz = DOGALORN_SIZES[name]
        dcfg = synth.dogalorn_config(**dz)
        dm = DogalornModel(dcfg, synth.make_dogalorn_weights(dcfg), device=dev, dtype="bfloat16", max_seqs=batch, num_kv_blocks=need_tokens // 16)
        p, d, ms = _steps(dm, GreedyDecoder, batch, ctx, rows, 512, args.steps, args.warmup, fill, dcfg.vocab, dev)
        entry["dogalorn"] = {"prefill_tokens_per_s": round(p, 1), "decode_tokens_per_s": round(d, 1), "decode_ms_per_step": round(ms, 3), "layers": dcfg.num_layers}
        del dm
        torch.cuda.empty_cache()
        entry["kernels"] = _zabutar_kernels(sz, rows, batch, ctx, dev)
        result["sizes"][name] = entry
    first = result["sizes"][sorted(result["sizes"])[0]]["zabutar"]
    result["value"], result["ms_per_step"] = first["decode_tokens_per_s"], first["decode_ms_per_step"]
    result["higher_is_better"], result["scaling"], result["vs_baseline"] = True, "weak", None
    return result


FUKATAR_SIZES = {
    "w1024": dict(width=1024, blocks=4, heads=16, kv_heads=4, dim=64, vdim=64, rot_dims=64, lat_heads=16, lat_dim=64, lat_vdim=64, kv_rank=256, rec_heads=8,
                  rec_kv_heads=4, rec_dim=128, rec_vdim=128, taps=4, ff=4096),
    "w2048": dict(width=2048, blocks=2, heads=32, kv_heads=8, dim=64, vdim=64, rot_dims=64, lat_heads=32, lat_dim=64, lat_vdim=64, kv_rank=256, rec_heads=16,
                  rec_kv_heads=8, rec_dim=128, rec_vdim=128, taps=4, ff=8192),
}


def _fukatar_kernels(sz, rows, batch, ctx, dev):
    """Single launches at the step's shapes with the share of their roofline (matrix products: bf16 matrix peak; recurrences: the larger of
    bytes / HBM rate and flop / fp32 vector rate; everything else: bytes / HBM rate), each beside the like kernel of Zabutar (of Morilorn
    for the latent attention, of Dogalorn for the convolution with silu)."""
    from . import ops_dense as D
    W, ff, H, G, dm, dv = sz["width"], sz["ff"], sz["heads"], sz["kv_heads"], sz["dim"], sz["vdim"]
    Hr, Gr, dk, dr, taps = sz["rec_heads"], sz["rec_kv_heads"], sz["rec_dim"], sz["rec_vdim"], sz["taps"]
    Hl, dl, r = sz["lat_heads"], sz["lat_dim"], sz["kv_rank"]
    out = {}
    g = torch.Generator(device=dev).manual_seed(1)
    rn = lambda *s: torch.randn(*s, device=dev, generator=g)

    def row(name, t, flops=0.0, bytes_=0.0, peak=BF16_TFLOPS):
        share = max(flops / t / (peak * 1e12), bytes_ / t / (HBM_GBS * 1e9))
        out[name] = {"us": round(t * 1e6, 1), "roofline_share": round(share, 3)}

    seq = 512
    warm_a, warm_w, warm_c = rn(rows, W), (rn(W, W) * 0.02).to(torch.bfloat16), torch.empty(rows, W, device=dev)
    _time(lambda: D.linear(warm_a, warm_w, warm_c), 20)      # clocks and caches settle before the first timed launch
    for n, tag in ((rows, "prefill"), (batch, "decode")):
        nseq = n // seq if tag == "prefill" else n
        per = seq if tag == "prefill" else 1
        pos0 = 0 if tag == "prefill" else ctx - 1
        pos = (torch.arange(per, dtype=torch.int32) + pos0).repeat(nseq).to(dev)
        slots = torch.arange(nseq, dtype=torch.int32).repeat_interleave(per).to(dev)
        seg = (torch.arange(nseq + 1, dtype=torch.int32) * per).to(dev)
        single = tag == "decode"
        reps = 5 if tag == "prefill" else 20
        a = rn(n, W)
        # feed-forward: up-projection with the squared relu; beside the same Linear with Zabutar's bias and two-branch activation
        w_up, b_up = (rn(ff, W) * 0.02).to(torch.bfloat16), rn(ff)
        act = torch.empty(n, ff, device=dev)
        t = _time(lambda: D.linear(a, w_up, act, epilogue=D.EPI_RELU_SQ), reps)
        row(f"linear_up_relu_sq_{tag}", t, flops=2.0 * n * ff * W, bytes_=2.0 * ff * W + 4.0 * n * (W + ff))
        t = _time(lambda: D.linear(a, w_up, act, bias=b_up, epilogue=D.EPI_XIELU, act_a=0.7, act_b=1.2), reps)
        row(f"zabutar_linear_up_bias_xielu_{tag}", t, flops=2.0 * n * ff * W, bytes_=2.0 * ff * W + 4.0 * n * (W + ff))
        # residual: the centred norm of one result, and of the mean of two normed results, added; beside Zabutar's norm behind + norm in front
        st, y, y2, h = rn(1, n, W), rn(n, W), rn(n, W), torch.empty(n, W, device=dev)
        wn, one = torch.ones(W, device=dev), torch.ones(1, device=dev)
        t = _time(lambda: D.streams_step(st, y=y, y_eps=1e-6, out_w=one, post_w=wn, post_center=True), reps)
        row(f"residual_centred_norm_{tag}", t, bytes_=4.0 * n * W * 3)
        t = _time(lambda: D.streams_step(st, y=y, y2=y2, yn_w=wn, y2n_w=wn, y_eps=1e-6, out_w=one, post_w=wn, post_center=True), reps)
        row(f"residual_two_results_centred_norm_{tag}", t, bytes_=4.0 * n * W * 4)
        t = _time(lambda: D.streams_step(st, y=y, yn_w=wn, y_eps=1e-6, out_w=one, norm_w=wn, eps=1e-6, h=h), reps)
        row(f"zabutar_sandwich_residual_{tag}", t, bytes_=4.0 * n * W * 4)
        # token shift (two taps added to the input); beside Zabutar's four-tap added convolution
        sw, sstate, hs = rn(W, 2) * 0.5, torch.zeros(nseq, 1, W, device=dev), torch.empty(n, W, device=dev)
        t = _time(lambda: D.causal_conv(a, off=0, channels=W, w=sw, bias=None, positions=pos, slot_ids=slots, state=sstate, out=hs, n=n, added=True, single_rows=single), reps)
        row(f"token_shift_{tag}", t, bytes_=4.0 * n * W * 2)
        cw, cstate = rn(W, 4) * 0.1, torch.zeros(nseq, 3, W, device=dev)
        t = _time(lambda: D.causal_conv(a, off=0, channels=W, w=cw, bias=None, positions=pos, slot_ids=slots, state=cstate, out=hs, n=n, added=True, single_rows=single), reps)
        row(f"zabutar_input_conv_{tag}", t, bytes_=4.0 * n * W * 2)
        # rotated attention: prep (norms, rotation of q, k and v, cache write), attention with capped scores, the turn back + gate
        plen = seq if tag == "prefill" else ctx
        nb = (plen + 15) // 16
        bt = torch.arange(nseq * nb, dtype=torch.int32, device=dev).view(nseq, nb).contiguous()
        gs = dv + dm
        kc = (rn(nseq * nb, 16, G * gs) * 0.5).to(torch.bfloat16)
        nq, nk, nv = H * dm, G * dm, G * dv
        ldp = nq + nk + nv + H
        P = rn(n, ldp) * 0.3
        q, oa = torch.empty(n, H * gs, device=dev), torch.empty(n, H * dv, device=dev)
        inv = torch.rand(dm // 2, device=dev, generator=g)
        vfr = torch.rand(dv // 2, device=dev, generator=g)
        qw, kw = torch.ones(nq, device=dev), torch.ones(nk, device=dev)
        t = _time(lambda: D.rot_prep(P, q_off=0, k_off=nq, v_off=nq + nk, heads=H, kv_heads=G, dim=dm, vdim=dv, q_norm_w=qw, k_norm_w=kw, eps=1e-6, rot_dims=dm,
                                     interleaved=False, inv_freq=inv, rot_mult=1.1, head_norm=False, v_freq=vfr, scale=0.125, positions=pos, slot_ids=slots,
                                     block_table=bt, cache=kc, q=q, n=n), reps)
        row(f"rot_prep_{tag}", t, bytes_=4.0 * n * (nq + nk + nv + H * gs) + 2.0 * n * G * gs)
        t = _time(lambda: D.kv_prep(P, q_off=0, k_off=nq, v_off=nq + nk, heads=H, kv_heads=G, dim=dm, vdim=dv, scale=0.125, positions=pos, slot_ids=slots, block_table=bt,
                                    cache=kc, q=q, n=n), reps)
        row(f"zabutar_kv_prep_{tag}", t, bytes_=4.0 * n * (nq + nk + nv + H * gs) + 2.0 * n * G * gs)
        keys = seq * (seq + 1) / 2 * nseq if tag == "prefill" else float(ctx) * n
        waves = 3072 if gs <= 64 else (2048 if gs <= 128 else 1024)
        sp = 1 if tag == "prefill" else max(1, min(waves // max(1, n * G * ((H // G + 15) // 16)), int(keys / n) // 64, 64))
        mode = 3 if tag == "prefill" else 2
        t = _time(lambda: D.kattn(q, kc, None, bt, slots, pos, chunk=0, bias=None, sink=False, heads=H, kv_heads=G, dim=dm, vdim=dv, out=oa, n=n, mode=mode, splits=sp,
                                  softcap=50.0), reps)
        abytes = (2.0 * keys * G * gs if tag == "decode" else 0.0) + 4.0 * n * H * (gs + dv)
        row(f"capped_attention_{tag}", t, flops=2.0 * keys * H * (dm + dv), bytes_=abytes)
        bias = torch.zeros(4097, H, device=dev)
        t = _time(lambda: D.kattn(q, kc, None, bt, slots, pos, chunk=0, bias=bias, sink=False, heads=H, kv_heads=G, dim=dm, vdim=dv, out=oa, n=n, mode=mode, splits=sp), reps)
        row(f"zabutar_kv_attention_{tag}", t, flops=2.0 * keys * H * (dm + dv), bytes_=abytes)
        t = _time(lambda: D.rot_post(oa, heads=H, vdim=dv, interleaved=False, v_freq=vfr, positions=pos, gate=P, gate_off=nq + nk + nv, ldg=ldp, n=n), reps)
        row(f"rot_post_{tag}", t, bytes_=4.0 * n * H * dv * 2)
        # latent attention with learned sinks; beside the same launch without them (Morilorn's)
        lc = (rn(nseq * nb, 16, r) * 0.5).to(torch.bfloat16)
        ql, ol = rn(n, Hl * r) * 0.1, torch.empty(n, Hl * r, device=dev)
        sink = torch.zeros(Hl, device=dev)
        spl = 1 if tag == "prefill" else max(1, min(1024 // max(1, n * ((Hl + 15) // 16)), int(keys / n) // 64, 64))
        lflops, lbytes = 4.0 * keys * Hl * r, (2.0 * keys * r if tag == "decode" else 0.0) + 8.0 * n * Hl * r
        t = _time(lambda: D.latent_attn(ql, lc, bt, slots, pos, window=0, scale=0.125, heads=Hl, kv_rank=r, rot_dim=0, out=ol, n=n, mode=mode, splits=spl, sink=sink), reps)
        row(f"latent_attention_sink_{tag}", t, flops=lflops, bytes_=lbytes)
        t = _time(lambda: D.latent_attn(ql, lc, bt, slots, pos, window=0, scale=0.125, heads=Hl, kv_rank=r, rot_dim=0, out=ol, n=n, mode=mode, splits=spl), reps)
        row(f"morilorn_latent_attention_{tag}", t, flops=lflops, bytes_=lbytes)
        # gated delta rule: convolution + silu, gates, scan, gated head norm; beside Dogalorn's convolution and Zabutar's gates, scan, head norm
        rk, rv = Gr * dk, Hr * dr
        C = 2 * rk + rv
        Pr = rn(n, C + 2 * Hr + rv) * 0.5
        cw2, cst2, X = rn(C, taps) * 0.3, torch.zeros(nseq, taps - 1, C, device=dev), torch.empty(n, C, device=dev)
        t = _time(lambda: D.causal_conv(Pr, off=0, channels=C, w=cw2, bias=None, positions=pos, slot_ids=slots, state=cst2, out=X, n=n, single_rows=single), reps)
        row(f"delta_conv_silu_{tag}", t, bytes_=4.0 * n * C * 2)
        Gt = torch.empty(n, 2 * Hr, device=dev)
        cols = dict(q_off=0, k_off=rk, v_off=2 * rk, heads=Hr, kv_heads=Gr, dim=dk, vdim=dr, n=n)
        al, db = torch.linspace(-4.0, 0.0, Hr, device=dev), torch.zeros(Hr, device=dev)
        t = _time(lambda: D.gdn_gates(X, Gt, Pr, b_off=C, a_off=C + Hr, a_log=al, dt_bias=db, unit_eps=1e-6, q_scale=dk ** -0.5, **cols), reps)
        row(f"delta_gates_{tag}", t, bytes_=4.0 * n * rk * 4)
        nkz = Hr * dk
        Pz = rn(n, 2 * nkz + rv) * 0.5
        lower = torch.rand(nkz, device=dev, generator=g) * 0.9
        zc = dict(q_off=0, f_off=nkz, v_off=2 * nkz, heads=Hr, dim=dk, vdim=dr, n=n)
        t = _time(lambda: D.gla_gates(Pz, lower=lower, q_act=True, **zc), reps)
        row(f"zabutar_gla_gates_{tag}", t, bytes_=4.0 * n * nkz * 4)
        dstate, ro, rg = torch.zeros(nseq, Hr, dr, dk, device=dev), torch.empty(n, rv, device=dev), torch.empty(n, rv, device=dev)
        t = _time(lambda: D.gdn_scan(X, Gt, seg_start=seg, nseg=nseq, positions=pos, slot_ids=slots, state=dstate, out=ro, **cols), reps)
        row(f"delta_scan_{tag}", t, flops=7.0 * n * Hr * dk * dr, bytes_=4.0 * n * (2 * rk + 2 * rv) + 8.0 * nseq * Hr * dk * dr, peak=F32_TFLOPS)
        Pz.uniform_(0.0, 1.0)
        t = _time(lambda: D.gla_scan(Pz, seg_start=seg, nseg=nseq, positions=pos, slot_ids=slots, state=dstate, out=ro, **zc), reps)
        row(f"zabutar_gla_scan_{tag}", t, flops=5.0 * n * Hr * dk * dr, bytes_=4.0 * n * (2 * nkz + 2 * rv) + 8.0 * nseq * Hr * dk * dr, peak=F32_TFLOPS)
        nwv = torch.ones(dr, device=dev)
        t = _time(lambda: D.gate_norm(ro, nwv, rg, groups=Hr, eps=1e-6, z=Pr, z_off=C + 2 * Hr, ldz=C + 2 * Hr + rv, n=n, gate_after=True, width=rv), reps)
        row(f"gated_head_norm_{tag}", t, bytes_=4.0 * n * rv * 3)
        t = _time(lambda: D.gate_norm(ro, torch.ones(rv, device=dev), rg, groups=Hr, eps=1e-6, n=n), reps)
        row(f"zabutar_head_norm_{tag}", t, bytes_=4.0 * n * rv * 2)
    return out


def run_fukatar(args) -> dict:
    from . import _lib, synth
    from .fukatar import FukatarModel
    from .model import GreedyDecoder
    from .zabutar import ZabutarModel
    _lib.load(), _lib.load_dense()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    batch, ctx, rows = args.batch, args.prompt_len, 4096
    result = {"metric": "prefill / decode tokens/s of the Fukatar design beside Zabutar at equal sizes", "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
              "warmup": args.warmup, "dtype": "bf16 matrix products, fp32 residual / norms / recurrences / attention math (both designs)", "data": "synthetic",
              "config": {"batch": batch, "context": ctx, "prefill_step": f"{rows} rows = {rows // 512} prompts of 512 tokens"}, "sizes": {}}
    for name in (args.design_sizes.split(",") if args.design_sizes else sorted(FUKATAR_SIZES)):
        sz = FUKATAR_SIZES[name]
        need_tokens = batch * (ctx + args.steps + args.warmup + 64)

        def fill(m):
            g = torch.Generator(device=dev).manual_seed(5)
            for t in {id(t): t for t in m.kv.rows if t is not None}.values():
                t.copy_((0.5 * torch.randn(t.shape, device=dev, generator=g)).to(t.dtype))
            for d in m.kv.state:
                for t in d.values():
                    t.copy_(0.1 * torch.randn(t.shape, device=dev, generator=g))

        cfg = synth.fukatar_config(**sz)
        model = FukatarModel(cfg, synth.make_fukatar_weights(cfg), device=dev, dtype="bfloat16", max_seqs=batch, num_kv_blocks=need_tokens // 16)
        p, d, ms = _steps(model, GreedyDecoder, batch, ctx, rows, 512, args.steps, args.warmup, fill, cfg.vocab, dev)
        entry = {"fukatar": {"prefill_tokens_per_s": round(p, 1), "decode_tokens_per_s": round(d, 1), "decode_ms_per_step": round(ms, 3), "layers": cfg.num_layers,
                             "shape": sz}}
        del model
        torch.cuda.empty_cache()
        zs = ZABUTAR_SIZES[name]
        zcfg = synth.zabutar_config(max_positions=max(4096, ctx + args.steps + args.warmup + 64), **zs)
        zm = ZabutarModel(zcfg, synth.make_zabutar_weights(zcfg), device=dev, dtype="bfloat16", max_seqs=batch, num_kv_blocks=need_tokens // 16)
        p, d, ms = _steps(zm, GreedyDecoder, batch, ctx, rows, 512, args.steps, args.warmup, fill, zcfg.vocab, dev)
        entry["zabutar"] = {"prefill_tokens_per_s": round(p, 1), "decode_tokens_per_s": round(d, 1), "decode_ms_per_step": round(ms, 3), "layers": zcfg.num_layers}
        del zm
        torch.cuda.empty_cache()
        entry["kernels"] = _fukatar_kernels(sz, rows, batch, ctx, dev)
        result["sizes"][name] = entry
    first = result["sizes"][sorted(result["sizes"])[0]]["fukatar"]
    result["value"], result["ms_per_step"] = first["decode_tokens_per_s"], first["decode_ms_per_step"]
    result["higher_is_better"], result["scaling"], result["vs_baseline"] = True, "weak", None
    return result


def main(args) -> int:
    print(json.dumps({"dogalorn": run_dogalorn, "zabutar": run_zabutar, "fukatar": run_fukatar}.get(args.design, run)(args)), flush=True)
    return 0
