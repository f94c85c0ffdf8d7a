"""The Lidizen building blocks and the model under the engine, against the plain CPU statement in ``oracle/lidizen.py``.

Mechanisms alone first (the pair embedding with its carried token, the residual streams' write-and-read step, the
attention over one shared key per token with a window that keeps the first keys, the whole attention sublayer with its
norms, rotation, head mixing and value blend, the activations, the router and its experts), then whole models of several
shapes: a prompt in one step against the oracle, and the same tokens cut into steps in every way the engine allows
(token by token, portions down to two tokens, unequal requests in one batch, pages and state slots used again) against
the one-step result.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle.lidizen import (attention_config, bigram_rows_ref, hyper_step_ref, layer_norm_ref, lidizen_config,  # noqa: E402
                            lidizen_random_weights, lidizen_ref, moe_ff_ref, shared_key_attention_ref, talking_attention_ref)

DEV = "cuda"


def rel_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    got, ref = got.double().cpu(), ref.double().cpu()
    return float((got - ref).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt().clamp_min(1e-30))


def rows_close(got: torch.Tensor, ref: torch.Tensor, tol: float, exact: bool) -> bool:
    """fp32 (``exact``): the whole tensor within ``tol``.  bf16: the typical row within ``0.6 tol`` and at most one row in
    ten beyond ``tol``."""
    if exact:
        return rel_err(got, ref) < tol
    got, ref = got.double().cpu(), ref.double().cpu()
    err = (got - ref).pow(2).mean(-1).sqrt() / ref.pow(2).mean(-1).sqrt().clamp_min(1e-30)
    return float(err.median()) < 0.6 * tol and float((err > tol).float().mean()) <= 0.1


def i32(v):
    return torch.tensor(v, dtype=torch.int32, device=DEV)


def layout_of(portions, contexts, slots, block_tables=None, block_size=16):
    """A step's layout from (rows, tokens before them, state slot) per sequence."""
    from itertools import accumulate
    from vllm_hymeta.models.stream_block import StepLayout
    qsl = list(accumulate(portions, initial=0))
    slot_mapping = bt = None
    if block_tables is not None:
        width = max(len(t) for t in block_tables)
        bt = torch.zeros(len(block_tables), width, dtype=torch.int32)
        sm = []
        for s, (n, ctx) in enumerate(zip(portions, contexts)):
            bt[s, :len(block_tables[s])] = torch.tensor(block_tables[s], dtype=torch.int32)
            sm += [block_tables[s][p // block_size] * block_size + p % block_size for p in range(ctx, ctx + n)]
        bt, slot_mapping = bt.to(DEV), torch.tensor(sm, dtype=torch.int64, device=DEV)
    return StepLayout(query_start_loc=i32(qsl), context_lens=i32(contexts), seq_lens=i32([c + n for c, n in zip(contexts, portions)]),
                      slot_idx=i32(slots), block_tables=bt, slot_mapping=slot_mapping, max_query_len=max(portions),
                      max_seq_len=max(c + n for c, n in zip(contexts, portions)))


# --------------------------------------------------------------------------- embedding
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,copies,buckets,mp,mc", [(48, 3, 53, 7, 5), (256, 1, 1, 1, 1), (600, 4, 997, 29, 23), (1024, 2, 64, 0, 3)])
def test_pair_embedding_in_portions_carries_the_previous_token(dtype, width, copies, buckets, mp, mc):
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(width)
    V = 90
    table = torch.randn(V, width, generator=g).to(dtype)
    pair = torch.randn(buckets + 1, width, generator=g).to(dtype)
    pair[buckets] += 3.0                                        # the first token's row stands out
    w = 1 + 0.1 * torch.randn(width, generator=g)
    eps = 1e-5
    seqs = [torch.randint(0, V, (n,), generator=g).tolist() for n in (37, 1, 9)]

    def ref(toks):
        rows = bigram_rows_ref(toks, buckets, mp, mc)
        return layer_norm_ref(table.double()[torch.tensor(toks)] + pair.double()[torch.tensor(rows)], w.double(), eps)

    refs = [ref(t) for t in seqs]
    prev = torch.full((4,), 77, dtype=torch.int32, device=DEV)     # stale values: a new sequence must not read them
    slots = [2, 0, 3]
    got = [[] for _ in seqs]
    at = [0, 0, 0]
    for step in ([(0, 2)], [(0, 1), (1, 1)], [(0, 5), (2, 4)], [(2, 5), (0, 29)]):
        toks = torch.tensor(sum((seqs[k][at[k]:at[k] + n] for k, n in step), []), dtype=torch.int64, device=DEV)
        lay = layout_of([n for _, n in step], [at[k] for k, _ in step], [slots[k] for k, _ in step])
        out = hip_ops.embed_pair(toks, table.to(DEV), pair.to(DEV), w.to(DEV), eps, copies, buckets, mp, mc, prev, lay.query_start_loc,
                                 lay.context_lens, lay.slot_idx)
        assert out.shape == (toks.numel(), copies, width) and out.dtype == torch.float32
        for c in range(1, copies):
            assert torch.equal(out[:, c], out[:, 0])
        r = 0
        for k, n in step:
            got[k].append(out[r:r + n, 0])
            r += n
            at[k] += n
    for k in range(3):
        assert rel_err(torch.cat(got[k]), refs[k]) < 2e-6, k
    assert prev.tolist() == [seqs[1][-1], 77, seqs[0][-1], seqs[2][-1]]
    # a slot that changes hands: the new sequence's first token reads the extra row, not the old owner's token
    lay = layout_of([3], [0], [2])
    out = hip_ops.embed_pair(torch.tensor(seqs[2][:3], dtype=torch.int64, device=DEV), table.to(DEV), pair.to(DEV), w.to(DEV), eps, 1, buckets, mp,
                             mc, prev, lay.query_start_loc, lay.context_lens, lay.slot_idx)
    assert rel_err(out[:, 0], refs[2][:3]) < 2e-6
    # without a pair table and without a norm: the table's rows
    out = hip_ops.embed_pair(torch.tensor(seqs[0], dtype=torch.int64, device=DEV), table.to(DEV), None, None, eps, 2)
    assert torch.equal(out[:, 1].cpu(), table.float()[torch.tensor(seqs[0])])


# --------------------------------------------------------------------------- residual streams
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("S,width", [(1, 48), (2, 256), (3, 600), (4, 1024), (8, 130), (5, 2048), (11, 96), (4, 3584)])
def test_streams_write_and_read_in_one_launch(dtype, S, width):
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(S * 1000 + width)
    T, eps = 13, 1e-5
    xs = torch.randn(T, S, width, generator=g) * 3 + 1.5             # a mean far from zero: an RMS norm in place of the layer norm shows
    y = torch.randn(T, width, generator=g).to(dtype)
    mix = torch.eye(S) + 0.3 * torch.randn(S, S, generator=g)        # not symmetric: [from, to] read the other way shows
    out_w, in_w = torch.randn(S, generator=g), torch.randn(S, generator=g)
    w = 1 + 0.1 * torch.randn(width, generator=g)
    tol = 2e-6 if dtype == torch.float32 else 4e-3
    new = hyper_step_ref(xs.double(), y.double(), mix.double(), out_w.double())
    h_ref = layer_norm_ref(torch.einsum("s,nsw->nw", in_w.double(), new), w.double(), eps)
    if S > 1:
        assert rel_err(hyper_step_ref(xs.double(), y.double(), mix.double().T, out_w.double()), new) > 0.05
    x = xs.clone().to(DEV)
    h = hip_ops.hyper_stream_(x, y.to(DEV), mix.to(DEV), out_w.to(DEV), in_w.to(DEV), w.to(DEV), eps, dtype)
    assert rel_err(x, new) < 2e-6 and rel_err(h, h_ref) < tol and h.dtype == dtype
    # write alone, then read alone: the same streams and the same rows
    x2 = xs.clone().to(DEV)
    assert hip_ops.hyper_stream_(x2, y.to(DEV), mix.to(DEV), out_w.to(DEV), None, None, eps, None) is None
    assert torch.equal(x2, x)
    h2 = hip_ops.hyper_stream_(x2, None, None, None, in_w.to(DEV), w.to(DEV), eps, dtype)
    assert torch.equal(h2, h) and torch.equal(x2, x)
    # read without a norm weight: the weighted sum itself
    u = hip_ops.hyper_stream_(x2, None, None, None, in_w.to(DEV), None, eps, torch.float32)
    assert rel_err(u, torch.einsum("s,nsw->nw", in_w.double(), new)) < 2e-6


# --------------------------------------------------------------------------- attention over one shared key per token
def _paged(rows, dtype, block_size, seed=0, spare=3):
    """``rows [L, E]`` written into a shuffled page pool; returns (cache [blocks, block_size, 1, E], block table)."""
    L, E = rows.shape
    nb = (L + block_size - 1) // block_size
    perm = torch.randperm(nb + spare, generator=torch.Generator().manual_seed(seed)).tolist()[:nb]
    cache = torch.full((nb + spare, block_size, 1, E), float("nan"), dtype=dtype)
    for p in range(L):
        cache[perm[p // block_size], p % block_size, 0] = rows[p].to(dtype)
    return cache.to(DEV), perm


def _attend(q, cache, perm, G, Dk, Dv, scale, portions, contexts, window, keep, block_size):
    """The step's rows of several sequences that share one page list (each reads its own prefix of it)."""
    from vllm_hymeta import hip_ops
    lay = layout_of(portions, contexts, [0] * len(portions), [perm] * len(portions), block_size)
    return hip_ops.sink_attention(q, cache, lay.block_tables, lay.query_start_loc, lay.seq_lens, G, Dk, Dv, scale, lay.max_query_len,
                                  lay.max_seq_len, sink=False, window_left=-1 if window is None else window - 1, shared_key=True,
                                  keep_first=keep)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,Dk,Dv,window,keep,page", [
    (4, 2, 32, 24, 12, 2, 16), (3, 1, 40, 16, None, 0, 16), (8, 2, 128, 64, 70, 4, 64), (8, 4, 256, 64, 80, 5, 16), (6, 6, 64, 128, 33, 0, 32),
    (16, 2, 128, 128, 64, 64, 64), (4, 1, 512, 128, 100, 3, 64), (34, 2, 128, 64, 50, 1, 16), (5, 5, 200, 48, 17, 70, 16), (2, 2, 64, 64, 1, 1, 64)])
def test_attention_over_a_shared_key_with_a_window_that_keeps_the_first_keys(dtype, H, G, Dk, Dv, window, keep, page):
    """Portions of a prompt and single rows over scattered pages against the plain statement: sizes of the matrix-core
    kernels and others, windows shorter and longer than a tile, kept keys within and beyond the first tile."""
    g = torch.Generator().manual_seed(H * 100 + Dk)
    L = 230
    rows = torch.randn(L, Dk + G * Dv, generator=g).to(dtype)
    q = torch.randn(L, H, Dk, generator=g).to(dtype)
    scale = Dk ** -0.5 * 2.0
    ref = shared_key_attention_ref(q.double(), rows.double(), G, Dv, scale, 0, window, keep)
    cache, perm = _paged(rows, dtype, page, seed=Dk)
    tol = 3e-6 if dtype == torch.float32 else 6e-3
    qd = q.to(DEV)
    # the whole prompt; then portions that end before / on / after tile and page borders; then rows one by one
    got = _attend(qd, cache, perm, G, Dk, Dv, scale, [L], [0], window, keep, page)
    assert rel_err(got, ref) < tol
    at = 0
    for n in (70, 2, 1, 55, 1, 64, 37):
        got = _attend(qd[at:at + n], cache, perm, G, Dk, Dv, scale, [n], [at], window, keep, page)
        assert rel_err(got, ref[at:at + n]) < tol, (at, n)
        at += n
    assert at == L
    # a batch: single rows of four "sequences" (prefixes of the same pages) beside a portion
    pos = [0, 63, 64, 129, 229]
    qs = torch.cat([qd[p:p + 1] for p in pos[:4]] + [qd[150:230]])
    got = _attend(qs, cache, perm, G, Dk, Dv, scale, [1, 1, 1, 1, 80], pos[:4] + [150], window, keep, page)
    want = torch.cat([ref[p:p + 1] for p in pos[:4]] + [ref[150:230]])
    assert rel_err(got, want) < tol


@pytest.mark.parametrize("dtype,H,G,Dk,Dv", [(torch.float32, 4, 2, 48, 24), (torch.bfloat16, 8, 2, 128, 64), (torch.bfloat16, 6, 1, 64, 128), (torch.bfloat16, 4, 4, 96, 40)])
def test_a_window_far_into_a_long_sequence(dtype, H, G, Dk, Dv):
    """2100 keys on scattered pages, a window of 88 and 6 kept keys: the whole prompt, a late portion, and single rows at
    tile borders far from the start (most of a decode launch's key splits see no key at all)."""
    g = torch.Generator().manual_seed(Dk)
    L, window, keep, page = 2100, 88, 6, 64
    rows = torch.randn(L, Dk + G * Dv, generator=g).to(dtype)
    q = torch.randn(L, H, Dk, generator=g).to(dtype)
    scale = Dk ** -0.5 * 2.0
    ref = shared_key_attention_ref(q.double(), rows.double(), G, Dv, scale, 0, window, keep)
    cache, perm = _paged(rows, dtype, page, seed=L)
    tol = 3e-6 if dtype == torch.float32 else 6e-3
    qd = q.to(DEV)
    assert rel_err(_attend(qd, cache, perm, G, Dk, Dv, scale, [L], [0], window, keep, page), ref) < tol
    assert rel_err(_attend(qd[1900:2077], cache, perm, G, Dk, Dv, scale, [177], [1900], window, keep, page), ref[1900:2077]) < tol
    pos = [2099, 2048, 2047, 1983, 1152, 99, 88, 87]
    got = _attend(torch.cat([qd[p:p + 1] for p in pos]), cache, perm, G, Dk, Dv, scale, [1] * len(pos), pos, window, keep, page)
    assert rel_err(got, torch.cat([ref[p:p + 1] for p in pos])) < tol


@pytest.mark.parametrize("dtype,Dk,Dv", [(torch.float32, 48, 24), (torch.bfloat16, 128, 64), (torch.bfloat16, 256, 128), (torch.bfloat16, 40, 16)])
@pytest.mark.parametrize("page", [16, 64])
def test_one_key_decides_at_the_edges_of_the_window_and_of_the_kept_keys(dtype, Dk, Dv, page):
    """One key is made to win the softmax wherever it is visible (its score stands far out), and its value is unlike any
    other.  Queries exactly ``window - 1`` and ``window`` behind it, the last kept key and the first one not kept, a key
    hundreds of tokens back on a page border: the output is the key's value or far from it, for prompt rows and for
    single rows."""
    H, G, L, window, keep = 4, 2, 400, 90, 5
    g = torch.Generator().manual_seed(page + Dk)
    scale = 1.0
    for special, seen_by, hidden_from in ((200, 200 + window - 1, 200 + window), (keep - 1, 399, None), (keep, keep + window - 1, keep + window),
                                          (page * 3, page * 3 + window - 1, page * 3 + window), (0, 350, None), (255, 255 + window - 1, 255 + window)):
        rows = (0.05 * torch.randn(L, Dk + G * Dv, generator=g)).to(dtype)
        direction = torch.randn(Dk, generator=g)
        direction /= direction.norm()
        rows[special, :Dk] = (direction * 8).to(dtype)
        rows[special, Dk:] = 5.0
        q = (direction * 8)[None, None, :].expand(L, H, Dk).contiguous().to(dtype)            # score 64 with the special key, about 0 with others
        ref = shared_key_attention_ref(q.double(), rows.double(), G, Dv, scale, 0, window, keep)
        assert float(ref[seen_by].mean()) > 4.9 and (hidden_from is None or abs(float(ref[hidden_from].mean())) < 0.5)
        cache, perm = _paged(rows, dtype, page, seed=special)
        tol = 1e-5 if dtype == torch.float32 else 2e-2
        qd = q.to(DEV)
        got = _attend(qd, cache, perm, G, Dk, Dv, scale, [L], [0], window, keep, page)
        assert float((got.double().cpu() - ref).abs().max()) < tol * 5
        for p in (seen_by, hidden_from):
            if p is None:
                continue
            one = _attend(qd[p:p + 1], cache, perm, G, Dk, Dv, scale, [1], [p], window, keep, page)
            assert float((one.double().cpu() - ref[p:p + 1]).abs().max()) < tol * 5, (special, p)
            two = _attend(qd[p - 1:p + 1], cache, perm, G, Dk, Dv, scale, [2], [p - 1], window, keep, page)
            assert float((two.double().cpu() - ref[p - 1:p + 1]).abs().max()) < tol * 5, (special, p)


# --------------------------------------------------------------------------- the attention sublayer
def _mixer(m, w, dtype, eps, prefix, first_blend_seen):
    from vllm_hymeta.linear import HymetaLinear
    from vllm_hymeta.models.talking_attention import PagedSharedKeyAttention, TalkingHeadsAttentionMixer
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    mask, rot = m.get("mask") or {}, m.get("rot") or {}
    attn = PagedSharedKeyAttention(H, G, D, Dv, m["scale"], prefix, sliding_window=mask.get("size"), keep_first=mask.get("keep_first", 0), dtype=dtype)
    dims = int(rot.get("dims", 0))
    freqs = torch.tensor([rot["base"] ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64, device=DEV) if dims else None

    def a(n):
        return w[n].to(device=DEV, dtype=dtype).contiguous()

    blend = None
    if m.get("v_mix"):
        blend = float(w["vmix"]) if first_blend_seen else 0.0
    qkv = HymetaLinear.from_weight(torch.cat([a("q"), a("k"), a("v")]).contiguous(), torch.cat([a("q.b"), a("k.b"), a("v.b")]).contiguous())
    return TalkingHeadsAttentionMixer(qkv, HymetaLinear.from_weight(a("o")), attn, w["q.norm"].to(DEV), w["k.norm"].to(DEV),
                                      w["talk"].to(DEV) if "talk" in w else None, eps, dims, freqs, blend), attn


_LAYER_SERIAL = [0]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mixer", [
    attention_config(), attention_config(heads=6, kv_heads=1, dim=12, vdim=8, size=5, keep_first=0, rot_dims=12),
    attention_config(heads=2, kv_heads=2, dim=64, vdim=64, size=40, keep_first=3, rot_dims=32, base=10000.0),
    attention_config(heads=8, kv_heads=2, dim=64, vdim=128, size=64, keep_first=1, rot_dims=64, scale=0.2),
    attention_config(heads=3, kv_heads=3, dim=10, vdim=7, size=1000, keep_first=2, rot_dims=0)])
def test_attention_sublayer_in_portions(dtype, mixer):
    """Two layers' mixers in a row (the second blends its values with the first's) on scattered pages, in portions,
    against the plain statement; then that every mechanism shows: the head mix, the rotation, the whole-projection norm,
    the blend."""
    from vllm_hymeta.models.attention import bind_kv_cache
    W, T, eps, page = 48, 75, 1e-5, 16
    cfg = lidizen_config(width=W, layers=[{"type": "attention", "mixer": mixer, "mlp": None}] * 2, streams=0, bigram=None)
    weights = lidizen_random_weights(cfg, seed=3)
    g = torch.Generator().manual_seed(5)
    h = torch.randn(T, W, generator=g).to(dtype)
    w0 = {k[len("l0.mix."):]: v.double() for k, v in weights.items() if k.startswith("l0.mix.")}
    w1 = {k[len("l1.mix."):]: v.double() for k, v in weights.items() if k.startswith("l1.mix.")}
    ref0, v_first = talking_attention_ref(h.double(), w0, mixer, eps, None, True)
    ref1, _ = talking_attention_ref(h.double(), w1, mixer, eps, v_first, True)
    _LAYER_SERIAL[0] += 1
    m0, a0 = _mixer(mixer, w0, dtype, eps, f"test_lidizen_{_LAYER_SERIAL[0]}.a", False)
    m1, a1 = _mixer(mixer, w1, dtype, eps, f"test_lidizen_{_LAYER_SERIAL[0]}.b", True)
    nb = (T + page - 1) // page
    perm = torch.randperm(nb + 2, generator=g).tolist()[:nb]
    for attn in (a0, a1):
        bind_kv_cache(attn, torch.full(attn.kv_cache_shape(nb + 2, page), float("nan"), dtype=dtype, device=DEV))
    got0, got1 = [], []
    at = 0
    for n in (33, 2, 1, 1, 30, 8):
        lay = layout_of([n], [at], [0], [perm], page)
        y0, vf = m0(h[at:at + n].to(DEV), lay, a0, None)
        y1, _ = m1(h[at:at + n].to(DEV), lay, a1, vf)
        got0.append(y0), got1.append(y1)
        at += n
    tol = 1e-5 if dtype == torch.float32 else 1.5e-2
    assert rel_err(torch.cat(got0), ref0) < tol and rel_err(torch.cat(got1), ref1) < tol
    # what would hide a missing mechanism: each of them moves the result by much more than the tolerance
    no_talk = dict(w1, talk=torch.eye(mixer["heads"], dtype=torch.float64))
    assert rel_err(talking_attention_ref(h.double(), no_talk, mixer, eps, v_first, True)[0], ref1) > 0.05
    assert rel_err(talking_attention_ref(h.double(), w1, mixer, eps, None, False)[0], ref1) > 0.05
    if mixer["rot"]["dims"]:
        assert rel_err(talking_attention_ref(h.double(), w1, dict(mixer, rot={"dims": 0, "base": 1.0}), eps, v_first, True)[0], ref1) > 0.05
    if mixer["mask"]["size"] < T:
        assert rel_err(talking_attention_ref(h.double(), w1, dict(mixer, mask={"size": T, "keep_first": 0}), eps, v_first, True)[0], ref1) > 0.02


# --------------------------------------------------------------------------- activations and experts
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_silu_gate_and_squared_relu(dtype):
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(1)
    for rows, n in ((5, 40), (33, 1024), (2, 7)):
        x = (3 * torch.randn(rows, 2 * n, generator=g)).to(dtype)
        tol = 1e-6 if dtype == torch.float32 else 4e-3
        gate, up = x.double()[:, :n], x.double()[:, n:]
        assert rel_err(hip_ops.silu_mul(x.to(DEV)), gate * torch.sigmoid(gate) * up) < tol
        assert rel_err(hip_ops.relu_squared(x.to(DEV)), torch.relu(x.double()) ** 2) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W,F,E,top", [(48, 40, 6, 2), (64, 64, 16, 4), (128, 128, 3, 1), (72, 24, 5, 5), (256, 160, 10, 3)])
def test_experts_weighed_by_the_softmax_over_the_chosen_logits(dtype, W, F, E, top):
    from vllm_hymeta.models.feed_forward import Relu2RoutedMoE
    g = torch.Generator().manual_seed(W + E)
    mlp = {"kind": "moe", "expert": {"ff": F}, "router": {"experts": E, "top": top}}
    w = {"router": torch.randn(E, W, generator=g) * W ** -0.5 * 3, "router.b": torch.randn(E, generator=g)}
    for e in range(E):
        w[f"e{e}.up"] = (torch.randn(F, W, generator=g) * W ** -0.5).to(torch.bfloat16).float()
        w[f"e{e}.down"] = (torch.randn(W, F, generator=g) * F ** -0.5).to(torch.bfloat16).float()
    h = torch.randn(70, W, generator=g).to(dtype)
    ref = moe_ff_ref(h.double(), {k: v.double() for k, v in w.items()}, mlp)
    moe = Relu2RoutedMoE(w["router"].to(DEV), w["router.b"].to(DEV), torch.stack([w[f"e{e}.up"] for e in range(E)]).to(DEV, dtype),
                         torch.stack([w[f"e{e}.down"] for e in range(E)]).to(DEV, dtype), top)
    got = moe(h.to(DEV))
    assert rows_close(got, ref, 1e-5 if dtype == torch.float32 else 1.5e-2, dtype == torch.float32)
    # the router's bias and the softmax over the chosen alone both show
    if top < E:
        assert rel_err(moe_ff_ref(h.double(), {k: (v.double() if k != "router.b" else torch.zeros(E, dtype=torch.float64)) for k, v in w.items()}, mlp), ref) > 0.05


# --------------------------------------------------------------------------- whole models under the engine
def build_engine(cfg, weights, dtype, max_tokens=512, block_size=16, max_num_seqs=4, max_num_batched_tokens=1 << 30):
    from vllm_hymeta.engine import LLMEngine
    from vllm_hymeta.models.configuration_lidizen import LidizenConfig
    from vllm_hymeta.models.modeling_lidizen import LidizenForCausalLM
    model = LidizenForCausalLM(LidizenConfig(cfg), max_num_seqs=max_num_seqs, dtype=dtype, device=DEV)
    model.load_weights(weights.items())
    return LLMEngine(model, num_blocks=max_tokens // block_size, block_size=block_size, max_num_seqs=max_num_seqs,
                     max_num_batched_tokens=max_num_batched_tokens, device=DEV)


def _layer(mixer, mlp):
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


_DENSE = {"kind": "dense", "ff": 72}


def _moe(experts=6, top=2, ff=40):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


MODELS = {
    "default": dict(),
    "plain_residual_no_pair_table_no_blend": dict(width=40, streams=0, bigram=None, layers=[
        _layer(attention_config(heads=1, kv_heads=1, dim=8, vdim=16, size=9, keep_first=0, rot_dims=8, v_mix=False), None),
        _layer(attention_config(heads=2, kv_heads=2, dim=8, vdim=4, size=300, keep_first=1, rot_dims=0, v_mix=False), _moe(3, 1, 24)),
        _layer(attention_config(heads=4, kv_heads=1, dim=6, vdim=10, size=20, keep_first=7, rot_dims=2, v_mix=False), _DENSE)]),
    "matrix_core_sizes": dict(width=128, streams=4, bigram=(509, 3, 11), layers=[
        _layer(attention_config(heads=4, kv_heads=2, dim=64, vdim=64, size=70, keep_first=3, rot_dims=64, base=10000.0, v_mix=False), {"kind": "dense", "ff": 192}),
        _layer(attention_config(heads=8, kv_heads=4, dim=64, vdim=32, size=40, keep_first=66, rot_dims=32, v_mix=True), _moe(8, 2, 64)),
        _layer(attention_config(heads=2, kv_heads=1, dim=128, vdim=128, size=130, keep_first=0, rot_dims=16, v_mix=False), _moe(8, 2, 64)),
        _layer(attention_config(heads=4, kv_heads=4, dim=16, vdim=32, size=64, keep_first=64, rot_dims=16, v_mix=True), None)]),
    "one_stream_with_weights_blend_from_the_second_layer": dict(width=64, streams=1, bigram=(1, 1, 1), layers=[
        _layer(attention_config(heads=4, kv_heads=2, dim=16, vdim=16, size=25, keep_first=2, v_mix=False), _moe(4, 4, 32)),
        _layer(attention_config(heads=2, kv_heads=2, dim=16, vdim=16, size=12, keep_first=0, v_mix=True), _DENSE),
        _layer(attention_config(heads=8, kv_heads=2, dim=16, vdim=16, size=33, keep_first=5, v_mix=True), _DENSE)]),
}


def _tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


@pytest.mark.parametrize("name", sorted(MODELS))
def test_model_whole_prompt_against_the_oracle_fp32(name):
    cfg = lidizen_config(**MODELS[name])
    weights = lidizen_random_weights(cfg, seed=len(name))
    toks = _tokens(45, cfg["vocab"], 1)
    layers_ref = []
    ref = lidizen_ref(cfg, weights, toks, residuals=layers_ref)
    eng = build_engine(cfg, weights, torch.float32)
    layers_got = []
    inner = eng.model.model
    plain = inner.forward
    inner.forward = lambda *a, **k: plain(*a, residual_out=layers_got, **k)
    got = eng.run_batch([("a", toks, list(range(len(toks))))])
    inner.forward = plain
    assert len(layers_got) == len(layers_ref)
    for i, (x, r) in enumerate(zip(layers_got, layers_ref)):
        assert rel_err(x, r) < 2e-5, i
    assert got.shape == ref.shape and got.dtype == torch.float32
    assert rel_err(got, ref) < 3e-5
    eng.finish_request("a")
    assert rel_err(eng.run_batch([("b", toks, list(range(len(toks))))]), ref) < 3e-5       # the fused write-and-read launches


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", sorted(MODELS))
def test_model_schedules_agree_with_the_whole_prompt(name, dtype):
    """Decoding token by token (the windows pass over decoded tokens), portions of several sizes (down to two tokens, and
    one), and a mixed batch of four requests whose pages and state slots come from requests that ended: every position's
    logits equal the one-step logits up to rounding, and the oracle's.  In bf16 every token runs all its layer's experts:
    with fewer, a choice between two nearly equal logits falls differently under bf16 rounding now and then, which moves
    that row by much more than rounding does (the choice itself is tested in fp32 here and alone in bf16 above)."""
    cfg = lidizen_config(**MODELS[name])
    if dtype == torch.bfloat16:
        for entry in cfg["layers"]:
            if entry["mlp"] and entry["mlp"]["kind"] == "moe":
                entry["mlp"] = dict(entry["mlp"], router=dict(entry["mlp"]["router"], top=entry["mlp"]["router"]["experts"]))
    weights = lidizen_random_weights(cfg, seed=len(name))
    V = cfg["vocab"]
    seqs = {k: _tokens(n, V, 10 + k) for k, n in enumerate([150, 33, 1, 70, 19, 64])}
    refs = {k: lidizen_ref(cfg, weights, t) for k, t in seqs.items()}
    exact = dtype == torch.float32
    tol_ref = 5e-5 if exact else 0.12
    tol_self = 5e-5 if exact else 0.1
    page = 64 if name == "matrix_core_sizes" else 16
    pages = 320 // page
    eng = build_engine(cfg, weights, dtype, max_tokens=pages * page, block_size=page, max_num_seqs=4)
    whole = {}
    for k, t in seqs.items():
        whole[k] = eng.run_batch([(f"w{k}", t, list(range(len(t))))])
        eng.finish_request(f"w{k}")
        assert rows_close(whole[k], refs[k], tol_ref, exact), k
    assert eng.pool.num_free == pages

    def replay(plan):
        at = {k: 0 for k in seqs}
        got = {k: [] for k in seqs}
        for step in plan:
            entries = [(f"r{k}", seqs[k][at[k]:at[k] + n], list(range(n))) for k, n in step]
            out = eng.run_batch(entries)
            row = 0
            for k, n in step:
                got[k].append(out[row:row + n])
                row += n
                at[k] += n
                if at[k] == len(seqs[k]):
                    eng.finish_request(f"r{k}")
        return {k: torch.cat(v) for k, v in got.items() if v}

    # token by token after a prompt that ends inside a page
    got = replay([[(0, 85)]] + [[(0, 1)]] * 65)
    assert rows_close(got[0], whole[0], tol_self, exact) and rows_close(got[0], refs[0], tol_ref, exact)
    # token by token from the very first token
    got = replay([[(1, 1)]] * 33)
    assert rows_close(got[1], whole[1], tol_self, exact)
    # portions: 2, 1, 3, ... across page borders and multiples of 64 rows
    got = replay([[(0, 2)], [(0, 1)], [(0, 3)], [(0, 10)], [(0, 2)], [(0, 45)], [(0, 2)], [(0, 64)], [(0, 2)], [(0, 19)]])
    assert rows_close(got[0], whole[0], tol_self, exact)
    # mixed: up to four live requests, portions beside single tokens, requests that end and free pages and slots for new ones
    plan = [[(0, 70), (1, 2)], [(0, 1), (1, 31), (2, 1)], [(0, 1), (3, 16), (4, 2)], [(0, 78), (3, 1), (4, 17)],
            [(3, 53), (5, 3)], [(5, 2)], [(5, 59)]]
    got = replay(plan)
    for k in seqs:
        if len(seqs[k]) < 10 and not exact:
            continue                                      # too few rows for the statistics of rows_close
        assert rows_close(got[k], whole[k], tol_self, exact), k
        assert rows_close(got[k], refs[k], tol_ref, exact), k
    assert eng.pool.num_free == pages and not eng.requests


def test_greedy_generation_through_the_scheduler_matches_the_oracle():
    """engine.generate: six prompts, two state slots, a token budget that cuts prompts into portions -- the scheduler
    batches portions beside decoded tokens and reuses slots and pages; every generated token is the oracle's argmax."""
    from vllm_hymeta.engine import SamplingParams
    cfg = lidizen_config(**MODELS["default"])
    weights = lidizen_random_weights(cfg, seed=4)
    prompts = [_tokens(n, cfg["vocab"], 40 + n) for n in (23, 5, 1, 37, 12, 18)]
    new = 5
    eng = build_engine(cfg, weights, torch.float32, max_tokens=128, block_size=16, max_num_seqs=2, max_num_batched_tokens=16)
    outs = eng.generate(prompts, SamplingParams(max_tokens=new))
    assert eng.pool.num_free == 8 and not eng.requests
    for p, o in zip(prompts, outs):
        assert len(o) == new
        toks = list(p)
        for t in o:
            logits = lidizen_ref(cfg, weights, toks)[-1]
            top2 = logits.topk(2).values
            if float(top2[0] - top2[1]) > 1e-3:        # a clear winner: the engine must have picked it
                assert t == int(logits.argmax())
            toks.append(t)


@pytest.mark.parametrize("dtype,name", [(torch.float32, "default"), (torch.bfloat16, "matrix_core_sizes")])
def test_long_decode_keeps_its_pages_and_its_previous_token(dtype, name):
    """400 tokens decoded one by one after a two-token prompt: every window passes over decoded tokens many times, the
    kept first tokens stay, the pair embedding follows the decoded tokens."""
    cfg = lidizen_config(**MODELS[name])
    if dtype == torch.bfloat16:
        for entry in cfg["layers"]:
            if entry["mlp"] and entry["mlp"]["kind"] == "moe":
                entry["mlp"] = dict(entry["mlp"], router=dict(entry["mlp"]["router"], top=entry["mlp"]["router"]["experts"]))
    weights = lidizen_random_weights(cfg, seed=8)
    toks = _tokens(402, cfg["vocab"], 3)
    page = 64 if dtype == torch.bfloat16 else 32
    eng = build_engine(cfg, weights, dtype, max_tokens=448, block_size=page, max_num_seqs=1)
    places = [17, 200, 333, 401]
    whole = eng.run_batch([("w", toks, places)])
    eng.finish_request("w")
    tol = 5e-5 if dtype == torch.float32 else 0.1
    eng.run_batch([("d", toks[:2], [])])
    for i in range(2, 402):
        out = eng.run_batch([("d", toks[i:i + 1], [0] if i in places else [])])
        if i in places:
            assert rel_err(out, whole[places.index(i):places.index(i) + 1]) < tol, i
    eng.finish_request("d")
    if dtype == torch.float32:
        ref = lidizen_ref(cfg, weights, toks[:201])[-1:]
        assert rel_err(eng.run_batch([("x", toks[:201], [200])]), ref) < 5e-5


def test_trace_runner_and_generate_command_lines(tmp_path):
    """A checkpoint folder (config.json + model.safetensors) served by the two programs under bin/: the trace replayer
    runs portions, single tokens and two requests side by side, gives pages back at a request's end and writes the logits
    asked for (fp32 against the oracle); the generator's greedy tokens are the oracle's argmax."""
    import json
    import os
    import subprocess
    import sys
    import numpy as np
    from safetensors.torch import save_file
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = lidizen_config(**MODELS["default"])
    weights = {k: v.to(torch.bfloat16).float() for k, v in lidizen_random_weights(cfg, seed=12).items()}      # what a bf16 file holds
    model_dir = tmp_path / "model"
    model_dir.mkdir()
    (model_dir / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in weights.items()}, str(model_dir / "model.safetensors"))
    a, b = _tokens(90, cfg["vocab"], 5), _tokens(40, cfg["vocab"], 6)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:50], "want": [0, 49]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[50:52], "want": []}, {"id": "b", "tokens": b[:39], "want": [38]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[39:], "want": [0]}, {"id": "a", "tokens": a[52:53], "want": [0]}], "end": ["b"]},
        {"step": 3, "entries": [{"id": "a", "tokens": a[53:], "want": [36]}, {"id": "c", "tokens": b[:7], "want": [6]}], "end": ["a", "c"]},
    ]
    out_dir = tmp_path / "out"
    run = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(model_dir), "--dtype", "float32", "--out", str(out_dir),
                          "--max-tokens", "192"], input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [l for l in run.stdout.splitlines() if l.startswith("done")] == [f"done {k}" for k in range(4)]
    ra, rb = lidizen_ref(cfg, weights, a), lidizen_ref(cfg, weights, b)
    want = {0: torch.stack([ra[0], ra[49]]), 1: rb[38:39], 2: torch.stack([rb[39], ra[52]]), 3: torch.stack([ra[89], rb[6]])}
    for k, ref in want.items():
        got = torch.from_numpy(np.fromfile(str(out_dir / f"{k}.f32"), dtype="<f4").reshape(ref.shape[0], -1))
        assert rel_err(got, ref) < 5e-5, k
    gen = subprocess.run([sys.executable, os.path.join(root, "bin", "generate"), "--model", str(model_dir), "--dtype", "float32", "--prompt-ids",
                          ",".join(map(str, a[:20])), "--max-new-tokens", "3", "--max-tokens", "128"], capture_output=True, text=True, timeout=300)
    assert gen.returncode == 0, gen.stderr[-2000:]
    line = json.loads([l for l in gen.stdout.splitlines() if l.startswith("{")][-1])
    toks = list(a[:20])
    for t in line["output"]:
        logits = lidizen_ref(cfg, weights, toks)[-1]
        top2 = logits.topk(2).values
        if float(top2[0] - top2[1]) > 1e-3:
            assert t == int(logits.argmax())
        toks.append(t)
    assert len(line["output"]) == 3


def _random_model(seed):
    """Sizes drawn at random: head counts, group sizes, key and value sizes (also such that a layer's concatenated keys
    and its values take the matrix-core kernels), windows around a page and a tile, kept keys, streams, feed-forwards."""
    import random
    r = random.Random(seed)
    width = r.choice([24, 40, 64, 96, 128, 200])
    layers = []
    blend_shape = None
    for _ in range(r.randint(1, 4)):
        G = r.choice([1, 2, 3, 4])
        H = G * r.choice([1, 2, 3, 5])
        if r.random() < 0.4:
            D, Dv = r.choice([(64 // G if G in (1, 2, 4) else 32, 64), (128 // G if G in (1, 2, 4) else 64, 64), (64, 128), (32, 64)])
        else:
            D, Dv = 2 * r.randint(2, 20), r.randint(3, 40)
        v_mix = r.random() < 0.6
        if v_mix:
            if blend_shape is None:
                blend_shape = (G, Dv)
            elif blend_shape != (G, Dv):
                H, (G, Dv) = blend_shape[0] * r.choice([1, 2, 4]), blend_shape
        size = r.choice([1, 2, 7, 15, 16, 17, 63, 64, 65, 100, 128, 1000])
        mixer = attention_config(heads=H, kv_heads=G, dim=D, vdim=Dv, size=size, keep_first=r.choice([0, 0, 1, 3, 16, 64, 70]),
                                 rot_dims=r.choice([0, 2, D // 2 * 2, D // 4 * 2]), base=r.choice([10.0, 10000.0, 500000.0]),
                                 scale=r.choice([D ** -0.5, 0.3, 0.05]), v_mix=v_mix)
        kind = r.choice(["dense", "moe", "moe", None])
        mlp = None if kind is None else {"kind": "dense", "ff": r.choice([16, 72, 128])} if kind == "dense" else _moe(r.randint(1, 9), 1, r.choice([8, 40, 64, 128]))
        if mlp and mlp["kind"] == "moe":
            mlp["router"]["top"] = r.randint(1, mlp["router"]["experts"])
        layers.append(_layer(mixer, mlp))
    bigram = None if r.random() < 0.2 else (r.choice([1, 7, 251, 4099]), r.randint(0, 40), r.randint(1, 40))
    return lidizen_config(vocab=r.choice([50, 130]), width=width, layers=layers, streams=r.choice([0, 1, 2, 3, 4, 6]), eps=r.choice([1e-5, 1e-6, 1e-3]),
                          bigram=bigram)


@pytest.mark.parametrize("seed", range(12))
def test_models_of_random_sizes_under_the_engine(seed):
    """fp32: a prompt of 210 tokens in one step, then in portions and single tokens beside a second request, against the
    oracle; bf16 (every expert chosen): the same schedule against the one-step result."""
    cfg = _random_model(seed)
    weights = lidizen_random_weights(cfg, seed=seed)
    V = cfg["vocab"]
    a, b = _tokens(210, V, 100 + seed), _tokens(75, V, 200 + seed)
    ra, rb = lidizen_ref(cfg, weights, a), lidizen_ref(cfg, weights, b)
    page = 64 if seed % 2 else 16
    plan = [[(0, 3)], [(0, 64), (1, 2)], [(0, 1), (1, 1)], [(0, 62), (1, 70)], [(0, 1), (1, 1)], [(0, 2), (1, 1)], [(0, 77)]]
    for dtype in (torch.float32, torch.bfloat16):
        c = cfg
        if dtype == torch.bfloat16:
            import copy
            c = copy.deepcopy(cfg)
            for entry in c["layers"]:
                if entry["mlp"] and entry["mlp"]["kind"] == "moe":
                    entry["mlp"]["router"]["top"] = entry["mlp"]["router"]["experts"]
        exact = dtype == torch.float32
        eng = build_engine(c, weights, dtype, max_tokens=448, block_size=page, max_num_seqs=2)
        wa = eng.run_batch([("wa", a, list(range(len(a))))])
        eng.finish_request("wa")
        if exact:
            assert rel_err(wa, ra) < 5e-5
        seqs, at, got = {0: a, 1: b}, {0: 0, 1: 0}, {0: [], 1: []}
        for step in plan:
            out = eng.run_batch([(f"r{k}", seqs[k][at[k]:at[k] + n], list(range(n))) for k, n in step])
            row = 0
            for k, n in step:
                got[k].append(out[row:row + n])
                row += n
                at[k] += n
                if at[k] == len(seqs[k]):
                    eng.finish_request(f"r{k}")
        assert at == {0: 210, 1: 75} and not eng.requests
        ga, gb = torch.cat(got[0]), torch.cat(got[1])
        if exact:
            assert rel_err(ga, ra) < 5e-5 and rel_err(gb, rb) < 5e-5
        else:
            assert rows_close(ga, wa, 0.1, False)
