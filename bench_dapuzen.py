"""Side benchmark of the Dapuzen design (``bench.py --design dapuzen``): prefill and decode throughput of a Dapuzen
stack at layer sizes that resemble a real model's (random weights), beside the package's closest existing model, Geponex
(fp32 stream, attention in the same paged kernels, a linear attention with a constant decay per head, routed experts beside
a shared expert, layers that reuse weights), at equal sizes -- same width, heads, layers, experts and expert size, the
recurrent heads of 128 x 128 -- and, kernel by kernel, how far each new kernel is from its roofline next to the like kernel
of that model.

Not the headline benchmark: ``bench.py`` without ``--design`` is unchanged.  Prints one JSON line.
"""
from __future__ import annotations

import json

import torch

from bench_geponex import geponex_checkpoint, geponex_config
from bench_sonuzen import BLOCK, HBM_GBS, MFMA_TFLOPS, SonuzenRunner, _events_ms


def dapuzen_config(width, heads, kv_heads, layers, experts, identity, top, ff, vocab, window, dim=128, state=128, ssm_vdim=64):
    """``layers``: the mixer type per layer; every feed-forward is the mixture (with a shared expert of a quarter of the
    experts' active size, as the neighbour's)."""
    ls = []
    attn = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5, mask=dict(size=window))
    for kind in layers:
        if kind == "attention":
            mixer = dict(attn, rot=dict(base=10000.0, dims=dim))
        elif kind == "retention":
            mixer = dict(heads=heads, dim=dim, vdim=dim, rot=dict(base=10000.0, dims=dim),
                         decay=[1.0 - 2.0 ** (-5 - 3 * h / max(heads - 1, 1)) for h in range(heads)])
        else:
            mixer = dict(left=dict(attn, softcap=30.0), left_scale=1.0, right_scale=1.0,
                         right=dict(heads=width // ssm_vdim, vdim=ssm_vdim, state=state, groups=2, norm_groups=2, conv=4))
        mlp = dict(kind="moe", expert=dict(ff=ff), shared=dict(ff=ff // 4),
                   router=dict(experts=experts, identity=identity, top=top, groups=dict(count=(experts + identity) // 4, keep=2)))
        ls.append(dict(type=kind, mixer=mixer, mlp=mlp))
    return dict(architecture="Dapuzen", vocab=vocab, width=width, layers=ls, norm=dict(eps=1e-6), embedding=dict(scale=1.0))


def dapuzen_checkpoint(cfg, dev, seed=0):
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, std=1.0):
        return (torch.randn(shape, device=dev, generator=g, dtype=torch.float32) * std).to(torch.bfloat16)

    def lin(o, i):
        return rnd(o, i, std=i ** -0.5)

    def attention(p, m, biased, gated):
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        for n, o in (("q", H * D), ("k", G * D), ("v", G * Dv)):
            yield p + n, lin(o, W)
            if biased:
                yield p + n + ".b", rnd(o, std=0.1)
        yield p + "o", lin(W, H * Dv)
        if biased:
            yield p + "o.b", rnd(W, std=0.1)
        if gated:
            yield p + "g", lin(H, W)

    yield "embed", rnd(V, W, std=0.5)
    yield "head", lin(V, W)
    yield "final.norm", 1 + rnd(std=0.05)
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}.", spec["mixer"]
        yield p + "norm1", 1 + rnd(std=0.05)
        if spec["type"] == "attention":
            yield from attention(p + "mix.", m, False, True)
        elif spec["type"] == "retention":
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            for n, o in (("q", H * D), ("k", H * D), ("v", H * Dv), ("g", H * Dv)):
                yield p + "mix." + n, lin(o, W)
            yield p + "mix.o", lin(W, H * Dv)
        else:
            yield from attention(p + "mix.left.", m["left"], True, False)
            r, q = m["right"], p + "mix.right."
            inner, ch = r["heads"] * r["vdim"], r["heads"] * r["vdim"] + 2 * r["groups"] * r["state"]
            yield q + "in", lin(inner + ch + r["heads"], W)
            yield q + "conv", rnd(ch, r["conv"], std=0.5)
            yield q + "conv.b", rnd(ch, std=0.1)
            yield q + "dt_bias", rnd(r["heads"], std=0.5)
            yield q + "A_log", rnd(r["heads"], std=0.5) - 2.0
            yield q + "D", 1 + rnd(r["heads"], std=0.1)
            yield q + "norm", 1 + rnd(inner, std=0.05)
            yield q + "o", lin(W, inner)
        e = spec["mlp"]
        for j in range(e["router"]["experts"]):
            yield f"{p}mlp.e{j}.gate", lin(e["expert"]["ff"], W)
            yield f"{p}mlp.e{j}.up", lin(e["expert"]["ff"], W)
            yield f"{p}mlp.e{j}.down", lin(W, e["expert"]["ff"])
        n = e["router"]["experts"] + e["router"]["identity"]
        yield p + "mlp.router", lin(n, W)
        yield p + "mlp.correction", rnd(n, std=0.01)
        Fs = e["shared"]["ff"]
        yield p + "mlp.shared.gate", lin(Fs, W)
        yield p + "mlp.shared.up", lin(Fs, W)
        yield p + "mlp.shared.down", lin(W, Fs)
        yield p + "mlp.shared.sg", lin(1, W)


def kernel_table(dev, W, H, G, D, B, ctx, L, E, I, top, ff, window, N=128, P=64):
    """(name, ms, fraction of the roofline that bounds it) for each new kernel and the like kernel of the neighbours."""
    from vllm_hymeta import hip_ops
    rows = []
    bf = torch.bfloat16

    def rnd(*shape, std=1.0, dtype=bf):
        return (torch.randn(*shape, device=dev, dtype=torch.float32) * std).to(dtype)

    def i32(v):
        return torch.tensor(v, dtype=torch.int32, device=dev)

    def add(name, fn, nbytes=0, flops=0, iters=20):
        ms = _events_ms(fn, iters=iters)
        t_mem, t_mma = nbytes / (HBM_GBS * 1e9) * 1e3, flops / (MFMA_TFLOPS * 1e12) * 1e3
        rows.append(dict(kernel=name, ms=round(ms, 4), roofline_ms=round(max(t_mem, t_mma), 4), bound="hbm" if t_mem >= t_mma else "mfma",
                         fraction_of_roofline=round(max(t_mem, t_mma) / ms, 3)))

    # ---- attention over one prompt of L tokens in a window: plain, with capped scores, with the heads' gates; beside the same
    # kernel as Sonuzen runs it (distance bias and sink)
    nblk = (L + BLOCK - 1) // BLOCK
    bt = torch.arange(nblk, dtype=torch.int32, device=dev).view(1, nblk)
    qs, kvs, gate = rnd(L, H, D), rnd(nblk, BLOCK, G, 2 * D), rnd(L, H)
    r1, r2 = torch.full((H,), 0.5, device=dev), torch.full((H,), 0.1, device=dev)
    seen = sum(min(i + 1, window) for i in range(L))
    for name, kw in (("gated", dict(head_gate=gate)), ("capped", dict(softcap=30.0))):
        add(f"window attention prefill, {name}, L={L}, window {window} (H={H}, {G} kv heads of {D})",
            lambda: hip_ops.sink_attention(qs, kvs, bt, i32([0, L]), i32([L]), G, D, D, D ** -0.5, L, L, sink=False, window_left=window - 1, **kw),
            flops=4 * H * D * seen, iters=5)
    add(f"sink_attention prefill (Sonuzen) L={L}, window {window}",
        lambda: hip_ops.sink_attention(qs, kvs, bt, i32([0, L]), i32([L]), G, D, D, D ** -0.5, L, L, r1, r2, True, window - 1), flops=4 * H * D * seen, iters=5)
    bps = (ctx + 1 + BLOCK - 1) // BLOCK
    btd = torch.randperm(B * bps).to(torch.int32).view(B, bps).to(dev)
    sl = torch.full((B,), ctx + 1, dtype=torch.int32, device=dev)
    qsl = torch.arange(B + 1, dtype=torch.int32, device=dev)
    qd, kvd, gd = rnd(B, H, D), rnd(B * bps, BLOCK, G, 2 * D), rnd(B, H)
    wkeys = min(ctx + 1, window)
    for name, kw in (("gated", dict(head_gate=gd)), ("capped", dict(softcap=30.0))):
        add(f"window attention decode, {name}, B={B} ctx={ctx}, window {window}",
            lambda: hip_ops.sink_attention(qd, kvd, btd, qsl, sl, G, D, D, D ** -0.5, 1, ctx + 1, sink=False, window_left=window - 1, **kw),
            nbytes=B * G * wkeys * 2 * D * 2)
    add(f"sink_attention decode (Sonuzen) B={B} ctx={ctx}, window {window}",
        lambda: hip_ops.sink_attention(qd, kvd, btd, qsl, sl, G, D, D, D ** -0.5, 1, ctx + 1, r1, r2, True, window - 1), nbytes=B * G * wkeys * 2 * D * 2)
    # ---- between the projection and the attention
    freqs = torch.tensor([10000.0 ** (-2.0 * i / D) for i in range(D // 2)], dtype=torch.float64, device=dev)
    w1 = torch.ones(D, device=dev)
    for T in (B, L):
        qkv = rnd(T, (H + 2 * G) * D + (H + 7) // 8 * 8)        # the heads' gate columns ride behind, padded to whole eights
        sm = torch.arange(T, dtype=torch.int64, device=dev)
        pos = torch.arange(T, dtype=torch.int64, device=dev)
        cache = kvd if T == B else kvs
        add(f"rotary_cache T={T}", lambda: hip_ops.rotary_cache_(qkv, H, G, D, D, D, freqs, 1.0, cache, sm, positions=pos),
            nbytes=T * ((H + 2 * G) * D * 2 + (H + G) * D * 2 + 2 * G * D * 2))
        qkv2 = rnd(T, (H + 2 * G) * D)
        add(f"qk_norm_cache (Sonuzen) T={T}", lambda: hip_ops.qk_norm_cache_(qkv2, H, G, D, D, w1, w1, 1e-5, cache, sm),
            nbytes=T * ((H + 2 * G) * D * 2 + H * D * 2 + 2 * G * D * 2))
    # ---- recurrences: retention (H heads of D x D) and the state-space scan (W / P heads of N x P) beside lightning attention
    Hs = W // P
    ones = torch.ones(B, dtype=torch.int32, device=dev)
    sidx = torch.arange(B, dtype=torch.int32, device=dev)
    decay = torch.full((H,), 0.99, device=dev)
    proj = rnd(L, 4 * H * D)
    st = torch.zeros(2, H, D, D, device=dev)
    q_, k_, v_ = proj[:, :H * D].view(L, H, D), proj[:, H * D:2 * H * D].view(L, H, D), proj[:, 2 * H * D:3 * H * D].view(L, H, D)
    add(f"decay_scan prefill, retention, L={L} (H={H}, {D}x{D})",
        lambda: hip_ops.decay_scan(q_, k_, v_, st, i32([0, L]), i32([0]), i32([1]), L, decay=decay),
        nbytes=L * H * (3 * D * 2 + D * 4), flops=L * H * (4 * D * D + 4 * 64 * D), iters=5)
    add(f"lightning_attention prefill (Geponex) L={L} (H={H}, {D}x{D})",
        lambda: hip_ops.lightning_attention(proj, st, decay, H, D, D, i32([0, L]), i32([0]), i32([1]), L),
        nbytes=L * H * (3 * D * 2 + D * 4), flops=L * H * (4 * D * D + 4 * 64 * D), iters=5)
    Gs = 2
    xbc = rnd(L, Hs * P + 2 * Gs * N)
    sts = torch.zeros(2, Hs, N, P, device=dev)
    ld, dt, skip = -torch.rand(L, Hs, device=dev) * 0.1, torch.rand(L, Hs, device=dev), torch.ones(Hs, device=dev)
    x_, b_, c_ = xbc[:, :Hs * P].view(L, Hs, P), xbc[:, Hs * P:Hs * P + Gs * N].view(L, Gs, N), xbc[:, Hs * P + Gs * N:].view(L, Gs, N)
    add(f"decay_scan prefill, state space, L={L} ({Hs} heads, {N}x{P}, {Gs} groups)",
        lambda: hip_ops.decay_scan(c_, b_, x_, sts, i32([0, L]), i32([0]), i32([1]), L, log2_decay=ld, v_scale=dt, skip=skip),
        nbytes=L * Hs * (P * 2 + P * 4 + 8) + L * 2 * Gs * N * 2, flops=L * Hs * (4 * N * P + 2 * 64 * N + 2 * 64 * P), iters=5)
    projd = rnd(B, 4 * H * D)
    std_ = torch.zeros(B, H, D, D, device=dev)
    qd_, kd_, vd_ = projd[:, :H * D].view(B, H, D), projd[:, H * D:2 * H * D].view(B, H, D), projd[:, 2 * H * D:3 * H * D].view(B, H, D)
    add(f"decay_scan decode, retention, B={B}", lambda: hip_ops.decay_scan(qd_, kd_, vd_, std_, qsl, ones, sidx, 1, decay=decay),
        nbytes=B * H * (2 * D * D * 4 + 3 * D * 2 + D * 4))
    add(f"lightning_attention decode (Geponex) B={B}", lambda: hip_ops.lightning_attention(projd, std_, decay, H, D, D, qsl, ones, sidx, 1),
        nbytes=B * H * (2 * D * D * 4 + 3 * D * 2 + D * 4))
    xbcd = rnd(B, Hs * P + 2 * Gs * N)
    stsd = torch.zeros(B, Hs, N, P, device=dev)
    ldd, dtd = -torch.rand(B, Hs, device=dev) * 0.1, torch.rand(B, Hs, device=dev)
    xd_, bd_, cd_ = xbcd[:, :Hs * P].view(B, Hs, P), xbcd[:, Hs * P:Hs * P + Gs * N].view(B, Gs, N), xbcd[:, Hs * P + Gs * N:].view(B, Gs, N)
    add(f"decay_scan decode, state space, B={B}", lambda: hip_ops.decay_scan(cd_, bd_, xd_, stsd, qsl, ones, sidx, 1, log2_decay=ldd, v_scale=dtd, skip=skip),
        nbytes=B * Hs * (2 * N * P * 4 + P * 2 + P * 4))
    # ---- the convolution, the norms and the stream
    for T in (B, L):
        lay = (qsl, ones, sidx) if T == B else (i32([0, T]), i32([0]), i32([1]))
        C = Hs * P + 2 * Gs * N
        pin = rnd(T, C + Hs)
        cw, cb = rnd(C, 4, std=0.5, dtype=torch.float32).contiguous(), rnd(C, std=0.1, dtype=torch.float32)
        cstate = torch.zeros(max(B, 4), 3, C, dtype=bf, device=dev)
        dtb, alog = torch.zeros(Hs, device=dev), torch.zeros(Hs, device=dev)
        add(f"causal_conv_silu (+ step sizes) T={T}", lambda: hip_ops.causal_conv_silu(pin[:, :C], cw, cb, cstate, *lay, dt_in=pin[:, C:], dt_bias=dtb, a_log=alog,
                                                                                          max_query_len=1 if T == B else T),
            nbytes=T * C * 4)
        x = rnd(T, W, dtype=torch.float32)
        wn = 1 + rnd(W, std=0.1, dtype=torch.float32)
        cw3 = rnd(W, 3, std=0.2, dtype=torch.float32).contiguous()
        cs = torch.zeros(max(T, 4), 2, W, dtype=bf, device=dev)
        add(f"norm_conv (Sonuzen) T={T}", lambda: hip_ops.norm_conv(x, wn, 1e-5, bf, 1.0, cw3, cs, *lay), nbytes=T * W * (4 + 2))
        ys = [rnd(T, W) for _ in range(4)]
        rs = torch.rand(T, device=dev)
        add(f"stream_add_norm (4 terms + next norm) T={T}",
            lambda: hip_ops.stream_add_norm_(x, [(ys[0], 1.0, None), (ys[1], 1.0, None), (ys[2], 1.0, rs), (ys[3], 1.0, rs)], 1.1, 1e-6, bf), nbytes=T * W * (8 + 4 * 2 + 2))
        add(f"stream_add_norm (1 term + next norm) T={T}", lambda: hip_ops.stream_add_norm_(x, [(ys[0], 1.0, None)], 1.1, 1e-6, bf), nbytes=T * W * (8 + 2 + 2))
        add(f"add_group_norm (Geponex) T={T}", lambda: hip_ops.add_group_norm(x, ys[0], wn, 2, 1e-6, 2.0, out_dtype=bf), nbytes=T * W * (2 + 4 + 4 + 2))
        o, gt = rnd(T, H * D, dtype=torch.float32), rnd(T, H * D)
        wg = torch.ones(H * D, device=dev)
        add(f"gated_rms_norm per head, silu gate T={T}", lambda: hip_ops.gated_rms_norm(o, gt, None, 1e-6, groups=H, gate_act="silu"), nbytes=T * H * D * (4 + 2 + 2))
        add(f"gated_rms_norm 2 groups, gate first T={T}", lambda: hip_ops.gated_rms_norm(o, gt, wg, 1e-6, groups=2, gate_act="silu", gate_first=True),
            nbytes=T * H * D * (4 + 2 + 2))
        add(f"gated_rms_norm (Geponex) T={T}", lambda: hip_ops.gated_rms_norm(o, gt, wg, 1e-6), nbytes=T * H * D * (4 + 2 + 2))
    # ---- experts
    w13, w2 = rnd(E, 2 * ff, W, std=W ** -0.5), rnd(E, W, ff, std=ff ** -0.5)
    router = rnd(E, W, std=W ** -0.5, dtype=torch.float32)
    rows_g = rnd(E + I + 1, W, std=W ** -0.5, dtype=torch.float32)
    corr = rnd(E + I, std=0.01, dtype=torch.float32)
    choice = hip_ops.GroupedChoice(corr, (E + I) // 4, 2, I, 1)
    rows_0 = rows_g[:E + 1].contiguous()
    choice_0 = hip_ops.GroupedChoice(corr[:E].contiguous(), max(E // 4, 1), max(E // 4, 1), 0, 1)
    for T in (B, L):
        xm = rnd(T, W)
        wbytes = min(E, T * top) * 3 * ff * W * 2
        fl = T * top * 3 * ff * W * 2
        # like for like: every chosen output is an expert with matrices
        add(f"moe_routed_forward grouped softmax, silu experts T={T} (E={E}, no identity experts, top {top})",
            lambda: hip_ops.moe_routed_forward(xm, rows_0, None, w13, w2, top, hip_ops.ROUTE_SOFTMAX_GROUPED, 1.0, "silu_glu", choice=choice_0),
            nbytes=wbytes, flops=fl, iters=10 if T > 256 else 20)
        # as the model runs it: with random router rows E / (E + I) of the chosen outputs have matrices, the others cost nothing
        add(f"moe_routed_forward grouped softmax, silu experts T={T} (E={E} + {I} identity, top {top}; flops of the expected {E}/{E + I} share)",
            lambda: hip_ops.moe_routed_forward(xm, rows_g, None, w13, w2, top, hip_ops.ROUTE_SOFTMAX_GROUPED, 1.0, "silu_glu", choice=choice),
            nbytes=wbytes, flops=fl * E // (E + I), iters=10 if T > 256 else 20)
        add(f"moe_sigmoid_forward (Geponex) T={T} (E={E}, top {top})", lambda: hip_ops.moe_sigmoid_forward(xm, router, w13, w2, top, 1.0, 7.0), nbytes=wbytes,
            flops=fl, iters=10 if T > 256 else 20)
    return rows


def main(args):
    from vllm_hymeta.models.configuration_dapuzen import DapuzenConfig
    from vllm_hymeta.models.configuration_geponex import GeponexConfig
    from vllm_hymeta.models.modeling_dapuzen import DapuzenForCausalLM
    from vllm_hymeta.models.modeling_geponex import GeponexForCausalLM

    torch.cuda.set_device(0)
    dev = torch.device("cuda", 0)
    B, ctx, L = args.batch, args.ctx if args.ctx_given else 4096, min(args.prefill_ctx, 8192)
    vocab, window = 32768, 1024
    out = {"metric": "dapuzen_vs_geponex_tokens_per_s", "dtype": "bf16", "data": "synthetic", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "sizes": []}
    for (W, H, inter) in ((2048, 16, 8192), (3584, 28, 18944)):
        E, I, top = 8, 8, 2
        ff = inter // top
        res = {}
        for name in ("geponex", "dapuzen"):
            if name == "geponex":
                cfg = geponex_config(W, H, ("latent_attention_2", "lightning", "latent_attention", "lightning"), E, top, ff, vocab)
                model = GeponexForCausalLM(GeponexConfig(cfg), max_num_seqs=max(B, 4), dtype=torch.bfloat16, device=dev)
                model.load_weights(geponex_checkpoint(cfg, dev))
            else:
                cfg = dapuzen_config(W, H, 4, ("attention", "retention", "parallel", "retention"), E, I, top, ff, vocab, window)
                model = DapuzenForCausalLM(DapuzenConfig(cfg), max_num_seqs=max(B, 4), dtype=torch.bfloat16, device=dev)
                model.load_weights(dapuzen_checkpoint(cfg, dev))
            run = SonuzenRunner(model, dev)
            dec = run.decode(B, ctx, args.steps, args.warmup)
            pre = run.prefill(L)
            res[name] = {"decode_ms_per_step": round(dec, 3), "decode_tokens_per_s": round(B / dec * 1e3, 1), "prefill_ms": round(pre, 2),
                         "prefill_tokens_per_s": round(L / pre * 1e3, 1)}
            del run, model
            torch.cuda.empty_cache()
        out["sizes"].append({"width": W, "heads": H, "kv_heads": 4, "head_dim": 128, "layers": 4, "experts": E, "identity": I, "top": top, "expert_ff": ff,
                             "batch": B, "ctx": ctx, "prompt": L, "window": window, "state_space": {"heads": W // 64, "vdim": 64, "state": 128}, **res})
        print(json.dumps(out["sizes"][-1]), flush=True)
    out["kernels"] = kernel_table(dev, 3584, 28, 4, 128, B, ctx, L, 8, 8, 2, 9472, window)
    s = out["sizes"][-1]
    out["value"], out["unit"] = s["dapuzen"]["decode_tokens_per_s"], "tokens/s"
    out["config"] = {"model": "Dapuzen 4 layers (gated window attention, retention, capped attention beside a state-space layer; grouped-choice experts "
                              "with identity experts and a gated shared expert)", "global_batch": B, "seq_len": ctx, "parallelism": "tp1"}
    print(json.dumps(out))
