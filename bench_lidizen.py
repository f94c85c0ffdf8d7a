"""Side benchmark of the Lidizen design (``bench.py --design lidizen``): prefill and decode throughput of a Lidizen
stack at layer sizes that resemble a real model's (random weights), beside the package's closest existing model, Sonuzen
(fp32 stream, softmax attention over pages with grouped key/value heads in the same attention kernels, routed experts),
at equal sizes -- same width, heads, key/value heads, head size, layers, experts and expert size -- and, kernel by
kernel, how far each new kernel is from its roofline next to the like kernel of that model.

Not the headline benchmark: ``bench.py`` without ``--design`` is unchanged.  Prints one JSON line.
"""
from __future__ import annotations

import json

import torch

from bench_sonuzen import BLOCK, HBM_GBS, MFMA_TFLOPS, SonuzenRunner, _events_ms, sonuzen_checkpoint, sonuzen_config


def lidizen_config(width, heads, kv_heads, dim, layers, experts, top, ff, vocab, window, keep_first, streams=4):
    """``layers``: "dense" or "moe" per layer (the feed-forward; every mixer is the attention).  The dense feed-forward has
    the experts' active size."""
    ls = []
    for kind in layers:
        mixer = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5, rot=dict(base=10000.0, dims=dim),
                     mask=dict(size=window, keep_first=keep_first), v_mix=True)
        mlp = dict(kind="dense", ff=top * ff) if kind == "dense" else dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top))
        ls.append(dict(type="attention", mixer=mixer, mlp=mlp))
    return dict(architecture="Lidizen", vocab=vocab, width=width, streams=streams, layers=ls, norm=dict(eps=1e-5),
                embedding=dict(bigram=dict(buckets=65521, mul_prev=37, mul_cur=19)))


def lidizen_checkpoint(cfg, dev, seed=0):
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    W, V, S = cfg["width"], cfg["vocab"], cfg["streams"]

    def rnd(*shape, std=1.0):
        return (torch.randn(*shape, device=dev, generator=g, dtype=torch.float32) * std).to(torch.bfloat16)

    def lin(o, i):
        return rnd(o, i, std=i ** -0.5)

    yield "embed", rnd(V, W, std=0.5)
    yield "bigram", rnd(cfg["embedding"]["bigram"]["buckets"] + 1, W, std=0.5)
    yield "embed.norm", 1 + rnd(W, std=0.05)
    yield "final.norm", 1 + rnd(W, std=0.05)
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}.", spec["mixer"]
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        yield p + "norm1", 1 + rnd(W, std=0.05)
        yield p + "norm2", 1 + rnd(W, std=0.05)
        for n, o in (("q", H * D), ("k", G * D), ("v", G * Dv)):
            yield p + "mix." + n, lin(o, W)
            yield p + "mix." + n + ".b", rnd(o, std=0.1)
        yield p + "mix.q.norm", 1 + rnd(H * D, std=0.05)
        yield p + "mix.k.norm", 1 + rnd(G * D, std=0.05)
        yield p + "mix.talk", (torch.eye(H, device=dev) + 0.1 * torch.randn(H, H, device=dev, generator=g)).to(torch.bfloat16)
        yield p + "mix.vmix", torch.tensor(0.3, device=dev, dtype=torch.bfloat16)
        yield p + "mix.o", lin(W, H * Dv)
        e = spec["mlp"]
        if e["kind"] == "dense":
            for n in ("gate", "up"):
                yield p + "mlp." + n, lin(e["ff"], W)
                yield p + "mlp." + n + ".b", rnd(e["ff"], std=0.1)
            yield p + "mlp.down", lin(W, e["ff"])
            yield p + "mlp.down.b", rnd(W, std=0.1)
        else:
            for j in range(e["router"]["experts"]):
                yield f"{p}mlp.e{j}.up", lin(e["expert"]["ff"], W)
                yield f"{p}mlp.e{j}.down", lin(W, e["expert"]["ff"])
            yield p + "mlp.router", lin(e["router"]["experts"], W)
            yield p + "mlp.router.b", rnd(e["router"]["experts"], std=0.1)
        for q in (1, 2):
            yield f"{p}hc{q}.in", rnd(S, std=0.1) + 1.0 / S
            yield f"{p}hc{q}.out", rnd(S, std=0.1) + 0.5
            yield f"{p}hc{q}.mix", (torch.eye(S, device=dev) + 0.05 * torch.randn(S, S, device=dev, generator=g)).to(torch.bfloat16)


def kernel_table(dev, W, H, G, D, B, ctx, L, E, top, ff, window, keep, S=4):
    """(name, ms, fraction of the roofline that bounds it) for each new kernel and the like kernel of Sonuzen."""
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

    Dk = G * D
    nblk = (L + BLOCK - 1) // BLOCK
    bt = torch.arange(nblk, dtype=torch.int32, device=dev).view(1, nblk)
    ql, kvl = rnd(L, H, Dk), rnd(nblk, BLOCK, 1, Dk + G * D)
    qs, kvs = rnd(L, H, D), rnd(nblk, BLOCK, G, 2 * D)
    r1, r2 = torch.full((H,), 0.5, device=dev), torch.full((H,), 0.1, device=dev)
    # ---- attention over one prompt of L tokens: all keys (the like-for-like case), then the window the model runs
    # (flops: the kernel's own products, a shared key of G * D and a value of D per query head and visible key)
    add(f"shared-key attention prefill L={L}, no window (H={H}, key {Dk}, value {D})",
        lambda: hip_ops.sink_attention(ql, kvl, bt, i32([0, L]), i32([L]), G, Dk, D, 0.05, L, L, sink=False, shared_key=True),
        flops=H * L * L * (Dk + D), iters=3)
    add(f"sink_attention prefill (Sonuzen) L={L}, no window (H={H}, {G} kv heads of {D})",
        lambda: hip_ops.sink_attention(qs, kvs, bt, i32([0, L]), i32([L]), G, D, D, D ** -0.5, L, L, r1, r2), flops=2 * H * D * L * L, iters=5)
    seen = sum(min(i + 1, window) for i in range(L))
    add(f"shared-key attention prefill L={L}, window {window} + {keep} kept",
        lambda: hip_ops.sink_attention(ql, kvl, bt, i32([0, L]), i32([L]), G, Dk, D, 0.05, L, L, sink=False, window_left=window - 1, shared_key=True,
                                       keep_first=keep), flops=2 * H * seen * (Dk + D), iters=5)
    add(f"sink_attention prefill (Sonuzen) L={L}, window {window}",
        lambda: hip_ops.sink_attention(qs, kvs, bt, i32([0, L]), i32([L]), G, D, D, D ** -0.5, L, L, r1, r2, True, window - 1), flops=4 * H * D * seen, iters=5)
    # ---- decode rows at context ctx
    bps = (ctx + 1 + BLOCK - 1) // BLOCK
    btd = torch.randperm(B * bps).to(torch.int32).view(B, bps).to(dev)
    sl = torch.full((B,), ctx + 1, dtype=torch.int32, device=dev)
    qsl = torch.arange(B + 1, dtype=torch.int32, device=dev)
    qd, kvd = rnd(B, H, Dk), rnd(B * bps, BLOCK, 1, Dk + G * D)
    qd2, kvd2 = rnd(B, H, D), rnd(B * bps, BLOCK, G, 2 * D)
    add(f"shared-key attention decode B={B} ctx={ctx}, no window",
        lambda: hip_ops.sink_attention(qd, kvd, btd, qsl, sl, G, Dk, D, 0.05, 1, ctx + 1, sink=False, shared_key=True), nbytes=B * (ctx + 1) * 2 * Dk * 2)
    add(f"sink_attention decode (Sonuzen) B={B} ctx={ctx}, no window",
        lambda: hip_ops.sink_attention(qd2, kvd2, btd, qsl, sl, G, D, D, D ** -0.5, 1, ctx + 1, r1, r2), nbytes=B * G * (ctx + 1) * 2 * D * 2)
    wkeys = min(ctx + 1, window + keep)
    add(f"shared-key attention decode B={B} ctx={ctx}, window {window} + {keep} kept",
        lambda: hip_ops.sink_attention(qd, kvd, btd, qsl, sl, G, Dk, D, 0.05, 1, ctx + 1, sink=False, window_left=window - 1, shared_key=True,
                                       keep_first=keep), nbytes=B * wkeys * 2 * Dk * 2)
    add(f"sink_attention decode (Sonuzen) B={B} ctx={ctx}, window {window}",
        lambda: hip_ops.sink_attention(qd2, kvd2, btd, qsl, sl, G, D, D, D ** -0.5, 1, ctx + 1, r1, r2, True, window - 1),
        nbytes=B * G * min(ctx + 1, window) * 2 * D * 2)
    # ---- between the projection and the attention
    freqs = torch.tensor([10000.0 ** (-2.0 * i / D) for i in range(D // 2)], dtype=torch.float64, device=dev)
    wq, wk = torch.ones(H * D, device=dev), torch.ones(G * D, device=dev)
    talk = torch.eye(H, device=dev) + 0.1 * torch.randn(H, H, device=dev)
    for T in (B, L):
        qkv, vo = rnd(T, (H + 2 * G) * D), rnd(T, G * D)
        sm = torch.arange(T, dtype=torch.int64, device=dev)
        lay = (qsl, sl) if T == B else (i32([0, T]), i32([T]))
        cache = kvd if T == B else kvl
        add(f"talk_qkv_prep T={T}", lambda: hip_ops.talk_qkv_prep(qkv, H, G, D, D, wq, wk, talk, 1e-5, D, freqs, cache, sm, *lay, v_other=vo, v_blend=0.3),
            nbytes=T * ((H + 3 * G) * D * 2 + H * Dk * 2 + 2 * Dk * 2))
        qkv2 = rnd(T, (H + 2 * G) * D)
        cache2 = kvd2 if T == B else kvs
        w1 = torch.ones(D, device=dev)
        add(f"qk_norm_cache (Sonuzen) T={T}", lambda: hip_ops.qk_norm_cache_(qkv2, H, G, D, D, w1, w1, 1e-5, cache2, sm),
            nbytes=T * ((H + 2 * G) * D * 2 + H * D * 2 + 2 * G * D * 2))
    # ---- stream kernels
    ones = torch.ones(B, dtype=torch.int32, device=dev)
    sidx = torch.arange(B, dtype=torch.int32, device=dev)
    for T in (B, L):
        x = rnd(T, S, W, dtype=torch.float32)
        y = rnd(T, W)
        wn = 1 + rnd(W, std=0.1, dtype=torch.float32)
        mix = (torch.eye(S, device=dev) + 0.05 * torch.randn(S, S, device=dev)).contiguous()
        ow, iw = torch.full((S,), 0.5, device=dev), torch.full((S,), 1.0 / S, device=dev)
        add(f"hyper_stream (write + read, {S} streams) T={T}", lambda: hip_ops.hyper_stream_(x, y, mix, ow, iw, wn, 1e-5, bf), nbytes=T * W * (S * 8 + 2 + 2))
        x1 = rnd(T, 1, W, dtype=torch.float32)
        o1 = torch.ones(1, device=dev)
        add(f"hyper_stream (1 stream: add + norm) T={T}", lambda: hip_ops.hyper_stream_(x1, y, o1, o1, o1, wn, 1e-5, bf), nbytes=T * W * (8 + 2 + 2))
        xs = rnd(T, W, dtype=torch.float32)
        add(f"add_group_norm (Geponex) T={T}", lambda: hip_ops.add_group_norm(xs, y, wn, 1, 1e-5, 1.0, out_dtype=bf), nbytes=T * W * (2 + 4 + 4 + 2))
        add(f"norm_residual (Sonuzen) T={T}", lambda: hip_ops.norm_residual_(xs, y, wn, 1e-5, 0.5, 1.0), nbytes=T * W * (2 + 4 + 4))
        ids = torch.randint(0, 32768, (T,), device=dev)
        table, pair = rnd(32768, W), rnd(65522, W)
        prev = torch.zeros(max(B, 4), dtype=torch.int32, device=dev)
        lay = (qsl, ones, sidx) if T == B else (i32([0, T]), i32([0]), i32([1]))
        add(f"embed_pair ({S} streams) T={T}", lambda: hip_ops.embed_pair(ids, table, pair, wn, 1e-5, S, 65521, 37, 19, prev, *lay), nbytes=T * W * (4 + S * 4))
        add(f"embed_rows (Sonuzen) T={T}", lambda: hip_ops.embed_rows(ids, table), nbytes=T * W * (2 + 4))
        gu = rnd(T, 2 * top * ff)
        add(f"silu_mul T={T}", lambda: hip_ops.silu_mul(gu), nbytes=T * top * ff * 6)
        add(f"silu_and_mul (7B family) T={T}", lambda: hip_ops.silu_and_mul(gu), nbytes=T * top * ff * 6)
    # ---- experts
    w1, w13, w2 = rnd(E, ff, W, std=W ** -0.5), rnd(E, 2 * ff, W, std=W ** -0.5), rnd(E, W, ff, std=ff ** -0.5)
    router = rnd(E, W, std=W ** -0.5, dtype=torch.float32)
    rb = rnd(E, std=0.1, dtype=torch.float32)
    table = torch.rand(1024, E, device=dev).argsort(1)[:, :top].to(torch.int32).contiguous()
    for T in (B, L):
        xm = rnd(T, W)
        ids = torch.randint(0, 1024, (T,), device=dev)
        add(f"moe_routed_forward relu^2, softmax over the chosen T={T} (E={E}, top {top}, 2 matrices per expert)",
            lambda: hip_ops.moe_routed_forward(xm, router, rb, w1, w2, top, hip_ops.ROUTE_SOFTMAX_CHOSEN, 1.0, "relu2"),
            nbytes=min(E, T * top) * 2 * ff * W * 2, flops=T * top * 2 * ff * W * 2, iters=10 if T > 256 else 20)
        add(f"moe_table_forward (Sonuzen) T={T} (E={E}, top {top}, 3 matrices per expert)", lambda: hip_ops.moe_table_forward(xm, ids, table, w13, w2),
            nbytes=min(E, T * top) * 3 * ff * W * 2, flops=T * top * 3 * ff * W * 2, iters=10 if T > 256 else 20)
    return rows


def main(args):
    from vllm_hymeta.models.configuration_lidizen import LidizenConfig
    from vllm_hymeta.models.configuration_sonuzen import SonuzenConfig
    from vllm_hymeta.models.modeling_lidizen import LidizenForCausalLM
    from vllm_hymeta.models.modeling_sonuzen import SonuzenForCausalLM

    torch.cuda.set_device(0)
    dev = torch.device("cuda", 0)
    B, ctx, L = args.batch, args.ctx if args.ctx_given else 4096, min(args.prefill_ctx, 8192)
    vocab, window, keep = 32768, 1024, 4
    out = {"metric": "lidizen_vs_sonuzen_tokens_per_s", "dtype": "bf16", "data": "synthetic", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "sizes": []}
    for (W, H, G, inter) in ((2048, 16, 2, 8192), (3584, 28, 4, 18944)):
        E, top = 8, 2
        ff = inter // top
        res = {}
        for name in ("sonuzen", "lidizen", "lidizen_all_keys"):
            if name == "sonuzen":
                cfg = sonuzen_config(W, H, G, 128, ("attention",) * 4, E, top, ff, vocab)
                model = SonuzenForCausalLM(SonuzenConfig(cfg), max_num_seqs=max(B, 4), dtype=torch.bfloat16, device=dev)
                model.load_weights(sonuzen_checkpoint(cfg, dev))
            else:
                win = window if name == "lidizen" else 1 << 20
                cfg = lidizen_config(W, H, G, 128, ("moe",) * 4, E, top, ff, vocab, win, keep)
                model = LidizenForCausalLM(LidizenConfig(cfg), max_num_seqs=max(B, 4), dtype=torch.bfloat16, device=dev)
                model.load_weights(lidizen_checkpoint(cfg, dev))
            run = SonuzenRunner(model, dev)
            dec = run.decode(B, ctx, args.steps, args.warmup)
            pre = run.prefill(L)
            res[name] = {"decode_ms_per_step": round(dec, 3), "decode_tokens_per_s": round(B / dec * 1e3, 1), "prefill_ms": round(pre, 2),
                         "prefill_tokens_per_s": round(L / pre * 1e3, 1)}
            del run, model
            torch.cuda.empty_cache()
        out["sizes"].append({"width": W, "heads": H, "kv_heads": G, "head_dim": 128, "layers": 4, "experts": E, "top": top, "expert_ff": ff, "batch": B,
                             "ctx": ctx, "prompt": L, "window": window, "keep_first": keep, "streams": 4, **res})
        print(json.dumps(out["sizes"][-1]), flush=True)
    out["kernels"] = kernel_table(dev, 3584, 28, 4, 128, B, ctx, L, 8, 2, 9472, window, keep)
    s = out["sizes"][-1]
    out["value"], out["unit"] = s["lidizen"]["decode_tokens_per_s"], "tokens/s"
    out["config"] = {"model": "Lidizen 4 layers (head-mixed attention with a window, 4 residual streams, routed relu^2 experts)", "global_batch": B,
                     "seq_len": ctx, "parallelism": "tp1"}
    print(json.dumps(out))
