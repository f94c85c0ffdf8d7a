"""The Dapuzen building blocks and the model under the engine, against the plain CPU statement in ``oracle/dapuzen.py``.

Mechanisms alone first (the stream's sum with the next norm, the half-split rotation with the paged write, the windowed
attention with capped scores and a gate per head, the causal convolution with its carried inputs, the decayed scan as a
retention and as a state-space recurrence, the gated grouped norm, the grouped choice of experts with identity experts
and a gated shared expert), then whole models of several shapes: a prompt in one step against the oracle, and the same
tokens cut into steps in every way the engine allows (token by token, portions down to two tokens, unequal requests in
one batch, pages and state slots used again) against the one-step result.
"""
import copy
import math

import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu

from oracle.dapuzen import (attention_mixer_config, causal_conv_ref, dapuzen_config, dapuzen_random_weights, dapuzen_ref,  # noqa: E402
                            gated_attention_ref, grouped_route_ref, moe_config, moe_ff_ref, parallel_mixer_config, retention_mixer_config,
                            rotate_half_ref, ssd_scan_ref, unit_rms_ref, window_attention_ref)

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
    positions = torch.tensor(sum((list(range(c, c + n)) for n, c in zip(portions, contexts)), []), dtype=torch.int64, device=DEV)
    return StepLayout(query_start_loc=i32(qsl), context_lens=i32(contexts), seq_lens=i32([c + n for c, n in zip(contexts, portions)]),
                      slot_idx=i32(slots), block_tables=bt, slot_mapping=slot_mapping, max_query_len=max(portions),
                      max_seq_len=max(c + n for c, n in zip(contexts, portions)), positions=positions)


def in_steps(seqs, plan, run):
    """Cut the sequences' rows into the plan's steps (lists of (sequence, rows)), call ``run(step rows per sequence, contexts,
    sequence ids)`` per step, and return every sequence's outputs joined."""
    at = {k: 0 for k in seqs}
    got = {k: [] for k in seqs}
    for step in plan:
        out = run([(k, at[k], n) for k, n in step])
        r = 0
        for k, n in step:
            got[k].append(out[r:r + n])
            r += n
            at[k] += n
    return {k: torch.cat(v) for k, v in got.items() if v}


# --------------------------------------------------------------------------- the stream's sum and the next norm
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,terms", [(48, 1), (256, 5), (600, 2), (4096, 3), (5000, 6), (64, 0)])
def test_stream_sum_with_the_next_norm_in_one_launch(dtype, width, terms):
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(width + terms)
    T, eps, scale = 11, 1e-5, 1.37
    x0 = torch.randn(T, width, generator=g) * 3 + 0.5
    ys = [torch.randn(T, width, generator=g).to(dtype) for _ in range(terms)]
    coefs = [1.0, 1.2, -0.7, 1.0, 0.5, 2.0][:terms]
    rows = [None if i % 2 == 0 else torch.rand(T, generator=g) for i in range(terms)]
    new = x0.double()
    for y, c, r in zip(ys, coefs, rows):
        new = new + c * y.double() * (1.0 if r is None else r.double()[:, None])
    h_ref = unit_rms_ref(new, eps) * scale
    x = x0.clone().to(DEV)
    h = hip_ops.stream_add_norm_(x, [(y.to(DEV), c, None if r is None else r.to(DEV)) for y, c, r in zip(ys, coefs, rows)], scale, eps, dtype)
    tol = 2e-6 if dtype == torch.float32 else 4e-3
    assert rel_err(x, new) < 2e-6 and rel_err(h, h_ref) < tol and h.dtype == dtype
    if terms:
        # the sum alone: the same stream, nothing returned
        x2 = x0.clone().to(DEV)
        assert hip_ops.stream_add_norm_(x2, [(y.to(DEV), c, None if r is None else r.to(DEV)) for y, c, r in zip(ys, coefs, rows)], None, eps) is None
        assert torch.equal(x2, x)


# --------------------------------------------------------------------------- rotation and the paged write
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,Dv,rot,extra", [(6, 2, 24, 40, 16, 6), (4, 4, 64, 64, 64, 0), (2, 1, 10, 3, 0, 1), (3, 3, 32, 8, 2, 0), (8, 2, 128, 128, 64, 8)])
def test_half_split_rotation_with_the_paged_write(dtype, H, G, D, Dv, rot, extra):
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(H * D + rot)
    page, base = 16, 5000.0
    portions, contexts = [5, 1, 40], [0, 1000, 27]                  # a far position: the angle's reduction shows
    T = sum(portions)
    width = (H + G) * D + G * Dv + extra
    qkv = torch.randn(T, width, generator=g).to(dtype)
    tables = [[3], [9 + i for i in range(63)], [1, 5, 2, 7, 8]]
    tables[1] = list(range(10, 10 + 63))
    lay = layout_of(portions, contexts, [0, 1, 2], tables, page)
    cache = torch.zeros(80, page, G, D + Dv, dtype=dtype, device=DEV)
    freqs = torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float64, device=DEV) if rot else None
    ks = 0.25
    tol = 2e-6 if dtype == torch.float32 else 4e-3
    for use_positions in (True, False):
        buf = qkv.clone().to(DEV)
        cache.zero_()
        hip_ops.rotary_cache_(buf, H, G, D, Dv, rot, freqs, ks, cache, lay.slot_mapping, positions=lay.positions if use_positions else None,
                              query_start_loc=lay.query_start_loc, seq_lens=lay.seq_lens)
        r = 0
        for n, ctx, tab in zip(portions, contexts, tables):
            rows = qkv[r:r + n].double()
            q = rows[:, :H * D].view(n, H, D)
            k = rows[:, H * D:(H + G) * D].view(n, G, D)
            # the oracle turns a whole sequence from position 0: put the rows at their places
            pad = lambda t: torch.cat([torch.zeros(ctx, *t.shape[1:], dtype=t.dtype), t], 0)      # noqa: E731
            q_ref = rotate_half_ref(pad(q), rot, base)[ctx:]
            k_ref = rotate_half_ref(pad(k), rot, base)[ctx:] * ks
            assert rel_err(buf[r:r + n, :H * D].view(n, H, D), q_ref) < tol
            assert rel_err(buf[r:r + n, H * D:(H + G) * D].view(n, G, D), k_ref) < tol
            assert torch.equal(buf[r:r + n, (H + G) * D:].cpu(), qkv[r:r + n, (H + G) * D:])       # values and what rides behind: untouched
            for j in range(n):
                p = ctx + j
                row = cache[tab[p // page], p % page].cpu()
                assert torch.equal(row[:, :D], buf[r + j, H * D:(H + G) * D].view(G, D).cpu())
                assert torch.equal(row[:, D:], qkv[r + j, (H + G) * D:(H + G) * D + G * Dv].view(G, Dv))
            r += n
    # without a cache (a recurrence's queries and keys): the same rotation
    buf2 = qkv.clone().to(DEV)
    hip_ops.rotary_cache_(buf2, H, G, D, Dv, rot, freqs, ks, positions=lay.positions)
    assert torch.equal(buf2, buf)


# --------------------------------------------------------------------------- windowed attention
def _fill_cache(k, v, tables, page, dtype, blocks):
    """``k [n, G, D]``, ``v [n, G, Dv]`` of one sequence into pages (key then value per head)."""
    G, D, Dv = k.shape[1], k.shape[2], v.shape[2]
    cache = torch.randn(blocks, page, G, D + Dv).to(dtype)          # stale rows everywhere else
    for p in range(k.shape[0]):
        cache[tables[p // page], p % page, :, :D] = k[p].to(dtype)
        cache[tables[p // page], p % page, :, D:] = v[p].to(dtype)
    return cache.to(DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,Dv,window,cap,gated,page", [
    (6, 2, 24, 40, 13, None, True, 16), (4, 2, 16, 24, 9, 3.0, False, 16), (8, 4, 64, 64, 70, 2.0, True, 64), (4, 1, 128, 128, 64, None, True, 64),
    (2, 2, 64, 128, 200, 5.0, False, 16), (8, 8, 128, 64, 17, 1.5, True, 32), (3, 1, 20, 7, 1, None, False, 16), (5, 5, 8, 8, None, 0.7, True, 16)])
def test_windowed_attention_with_capped_scores_and_head_gates(dtype, H, G, D, Dv, window, cap, gated, page):
    """Prompts, portions and single rows of three sequences in one launch against the plain attention of each."""
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(H * 100 + D)
    lens = [150, 70, 33]
    scale = D ** -0.5
    blocks = 40
    perm = torch.randperm(blocks, generator=g).tolist()
    tables, used = [], 0
    for n in lens:
        nb = (n + page - 1) // page
        tables.append(perm[used:used + nb])
        used += nb
    qs = [torch.randn(n, H, D, generator=g).to(dtype) * 1.5 for n in lens]
    ks = [torch.randn(n, G, D, generator=g).to(dtype) * 1.5 for n in lens]
    vs = [torch.randn(n, G, Dv, generator=g).to(dtype) for n in lens]
    gates = [torch.randn(n, H, generator=g).to(dtype) for n in lens]
    cache = torch.randn(blocks, page, G, D + Dv, generator=g).to(dtype)
    for s, n in enumerate(lens):
        for p in range(n):
            cache[tables[s][p // page], p % page, :, :D] = ks[s][p]
            cache[tables[s][p // page], p % page, :, D:] = vs[s][p]
    cache = cache.to(DEV)
    refs = []
    for s in range(3):
        o = window_attention_ref(qs[s].double(), ks[s].double(), vs[s].double(), scale, window, cap)
        refs.append(o * torch.sigmoid(gates[s].double())[:, :, None] if gated else o)
    tol = 3e-6 if dtype == torch.float32 else 8e-3
    # (rows, context) per sequence: whole prompts; a portion, a single row, a portion from the start; single rows only
    for plan in ([(150, 0), (70, 0), (33, 0)], [(37, 113), (1, 69), (20, 0)], [(1, 149), (1, 42), (1, 0)], [(2, 100), (64, 6), (1, 32)]):
        q = torch.cat([qs[s][c:c + n] for s, (n, c) in enumerate(plan)]).to(DEV)
        gate = torch.cat([gates[s][c:c + n] for s, (n, c) in enumerate(plan)]).to(DEV) if gated else None
        lay = layout_of([n for n, _ in plan], [c for _, c in plan], [0, 1, 2], tables, page)
        out = hip_ops.sink_attention(q, cache, lay.block_tables, lay.query_start_loc, lay.seq_lens, G, D, Dv, scale, lay.max_query_len,
                                     lay.max_seq_len, sink=False, window_left=-1 if window is None else window - 1, softcap=cap or 0.0, head_gate=gate)
        ref = torch.cat([refs[s][c:c + n] for s, (n, c) in enumerate(plan)])
        assert rel_err(out, ref) < tol, plan


@pytest.mark.parametrize("dtype,D,Dv", [(torch.float32, 48, 24), (torch.bfloat16, 64, 64), (torch.bfloat16, 128, 128), (torch.bfloat16, 40, 16)])
@pytest.mark.parametrize("page", [16, 64])
def test_one_key_decides_at_the_edges_of_the_window(dtype, D, Dv, page):
    """Among hundreds of keys ONE matches the query (a large score) and carries a value of its own: placed at the window's
    first position it makes the whole output, one further back it must not be seen.  In prompts and decoding."""
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(D + page)
    n, window, H, G = 300, 70, 2, 1
    q_dir = F.normalize(torch.randn(D, generator=g), dim=0)
    for query_pos in (299, 131, 70, 69):
        for back, seen in ((window - 1, True), (window, False), (0, True)):
            key_pos = query_pos - back
            if key_pos < 0:
                continue
            k = torch.randn(n, G, D, generator=g) * 0.1
            v = torch.randn(n, G, Dv, generator=g) * 0.1
            k[key_pos, 0] = q_dir * 6.0
            v[key_pos, 0] = 5.0
            q = (q_dir * 6.0).expand(H, D).contiguous()
            tables = list(range(3, 3 + (n + page - 1) // page))
            cache = _fill_cache(k, v, tables, page, dtype, 30)
            for rows, ctx in ((1, query_pos), (query_pos + 1, 0), (2, query_pos - 1)):        # decoded; in a prompt; in a portion of two
                if ctx < 0:
                    continue
                qq = torch.randn(rows, H, D, generator=g) * 0.1
                qq[-1] = q
                lay = layout_of([rows], [ctx], [0], [tables], page)
                out = hip_ops.sink_attention(qq.to(dtype).to(DEV), cache, lay.block_tables, lay.query_start_loc, lay.seq_lens, G, D, Dv, 1.0,
                                             lay.max_query_len, lay.max_seq_len, sink=False, window_left=window - 1)
                got = float(out[-1].float().mean())
                assert (got > 4.5) == seen, (query_pos, back, rows, got)


# --------------------------------------------------------------------------- causal convolution
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("C,taps,heads", [(40, 4, 6), (512, 4, 8), (300, 2, 3), (64, 1, 1), (33, 5, 2), (1000, 3, 16)])
def test_causal_convolution_in_portions_carries_its_inputs(dtype, C, taps, heads):
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(C + taps)
    lens = {0: 300, 1: 1, 2: 145}
    row = C + heads + 5                                          # a wider row: the stride shows
    if C % 4 == 0:
        row = (row + 3) // 4 * 4                                 # ... in whole fours where the channels are: the strips of rows run
    xs = {k: torch.randn(n, row, generator=g).to(dtype) for k, n in lens.items()}
    w = torch.randn(C, taps, generator=g) * taps ** -0.5
    b = torch.randn(C, generator=g) * 0.1
    dt_bias, a_log = torch.randn(heads, generator=g), torch.randn(heads, generator=g) * 0.5 - 1
    refs = {k: F.silu(causal_conv_ref(x[:, :C].double(), w.double(), b.double())) for k, x in xs.items()}
    state = torch.full((4, max(taps - 1, 1), C), 7.0, dtype=dtype, device=DEV)        # stale values: a new sequence must not read them
    slots = {0: 2, 1: 0, 2: 3}
    dts, lds = {k: [] for k in lens}, {k: [] for k in lens}

    def run(step):
        rows = torch.cat([xs[k][at:at + n] for k, at, n in step]).to(DEV)
        lay = layout_of([n for _, _, n in step], [at for _, at, _ in step], [slots[k] for k, _, _ in step])
        out, dt, ld = hip_ops.causal_conv_silu(rows[:, :C], w.to(DEV), b.to(DEV), state, lay.query_start_loc, lay.context_lens, lay.slot_idx,
                                               dt_in=rows[:, C:C + heads], dt_bias=dt_bias.to(DEV), a_log=a_log.to(DEV), max_query_len=lay.max_query_len)
        r = 0
        for k, _, n in step:
            dts[k].append(dt[r:r + n])
            lds[k].append(ld[r:r + n])
            r += n
        return out

    # (the last step: a sequence that ends inside a strip of rows, the next one starting there with a state of its own)
    got = in_steps(lens, [[(0, 2)], [(0, 1), (1, 1)], [(0, 1), (2, 4)], [(0, 3), (2, 1)], [(0, 1), (2, 1)], [(2, 6), (0, 29)], [(0, 263), (2, 133)]], run)
    tol = 2e-6 if dtype == torch.float32 else 6e-3
    for k in lens:
        assert rel_err(got[k], refs[k]) < tol, k
        dt_ref = F.softplus(xs[k][:, C:C + heads].double() + dt_bias.double())
        assert rel_err(torch.cat(dts[k]), dt_ref) < 2e-6
        assert rel_err(torch.cat(lds[k]), -torch.exp(a_log.double()) * dt_ref * math.log2(math.e)) < 2e-6
    # a slot that changes hands: the new sequence starts from zeros, not from the old owner's rows
    lay = layout_of([5], [0], [2])
    out = hip_ops.causal_conv_silu(xs[2][:5, :C].to(DEV), w.to(DEV), b.to(DEV), state, lay.query_start_loc, lay.context_lens, lay.slot_idx)
    assert rel_err(out, refs[2][:5]) < tol


# --------------------------------------------------------------------------- the decayed scan
def _scan_ref(q, k, v, log2_decay, v_scale, skip):
    """``q, k [T, G, D]``, ``v [T, H, P]``, ``log2_decay, v_scale [T, H]``, ``skip [H]``, all double."""
    T, H, P = v.shape
    G, D = q.shape[1], q.shape[2]
    out = torch.zeros(T, H, P, dtype=torch.float64)
    for h in range(H):
        gq = h // (H // G)
        S = torch.zeros(D, P, dtype=torch.float64)
        for t in range(T):
            S = 2.0 ** log2_decay[t, h] * S + v_scale[t, h] * torch.outer(k[t, gq], v[t, h])
            out[t, h] = S.T @ q[t, gq] + skip[h] * v[t, h]
    return out.reshape(T, H * P)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,P,per_token", [(3, 3, 16, 24, False), (6, 3, 12, 8, True), (8, 2, 32, 48, True), (4, 4, 32, 64, False), (4, 1, 64, 64, True),
                                                (2, 2, 128, 32, False), (2, 1, 128, 128, True), (5, 5, 40, 20, False), (1, 1, 200, 16, True)])
def test_decayed_scan_in_portions_and_single_rows(dtype, H, G, D, P, per_token):
    """A constant decay per head (retention) or a decay and an input weight per token (state-space), heads that share
    queries and keys, the skip term: whole sequences, portions of every size, single rows, a state slot used again."""
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(H * D + P)
    lens = {0: 150, 1: 1, 2: 70}
    qs = {k: (torch.randn(n, G, D, generator=g) * D ** -0.25).to(dtype) for k, n in lens.items()}
    ks = {k: (torch.randn(n, G, D, generator=g) * D ** -0.25).to(dtype) for k, n in lens.items()}
    vs = {k: torch.randn(n, H, P, generator=g).to(dtype) for k, n in lens.items()}
    decay = torch.tensor([1 - 2.0 ** (-2 - h) for h in range(H)])
    lds = {k: (-torch.rand(n, H, generator=g) * 0.4) if per_token else torch.log2(decay).expand(n, H).contiguous() for k, n in lens.items()}
    bs = {k: (torch.rand(n, H, generator=g) + 0.2) if per_token else torch.ones(n, H) for k, n in lens.items()}
    skip = torch.randn(H, generator=g) if per_token else torch.zeros(H)
    refs = {k: _scan_ref(qs[k].double(), ks[k].double(), vs[k].double(), lds[k].double(), bs[k].double(), skip.double()) for k in lens}
    state = torch.full((4, H, D, P), 3.0, dtype=torch.float32, device=DEV)          # stale values: a new sequence must not read them
    slots = {0: 1, 1: 3, 2: 0}

    def run(step):
        cat = lambda d: torch.cat([d[k][at:at + n] for k, at, n in step]).to(DEV)      # noqa: E731
        lay = layout_of([n for _, _, n in step], [at for _, at, _ in step], [slots[k] for k, _, _ in step])
        kw = dict(log2_decay=cat(lds), v_scale=cat(bs), skip=skip.to(DEV)) if per_token else dict(decay=decay.to(DEV))
        return hip_ops.decay_scan(cat(qs), cat(ks), cat(vs), state, lay.query_start_loc, lay.context_lens, lay.slot_idx, lay.max_query_len, **kw)

    tol = 5e-6 if dtype == torch.float32 else 6e-3
    whole = in_steps(lens, [[(0, 150), (1, 1), (2, 70)]], run)
    for k in lens:
        assert rel_err(whole[k], refs[k]) < tol, k
    state.fill_(-2.0)
    plan = [[(0, 2)], [(0, 1), (2, 64)], [(0, 1), (1, 1), (2, 1)], [(0, 7), (2, 2)], [(0, 65), (2, 1)], [(0, 1)], [(0, 73), (2, 2)]]
    got = in_steps(lens, plan, run)
    for k in lens:
        assert rel_err(got[k], refs[k]) < tol, k
    # the state after the last row is what one more row starts from, whatever the cut
    q1, k1, v1 = torch.randn(1, G, D, generator=g).to(dtype), torch.randn(1, G, D, generator=g).to(dtype), torch.randn(1, H, P, generator=g).to(dtype)
    lay = layout_of([1], [150], [1])
    kw = dict(log2_decay=lds[0][:1].to(DEV), v_scale=bs[0][:1].to(DEV), skip=skip.to(DEV)) if per_token else dict(decay=decay.to(DEV))
    more = hip_ops.decay_scan(q1.to(DEV), k1.to(DEV), v1.to(DEV), state, lay.query_start_loc, lay.context_lens, lay.slot_idx, 1, **kw)
    ref = _scan_ref(torch.cat([qs[0], q1]).double(), torch.cat([ks[0], k1]).double(), torch.cat([vs[0], v1]).double(),
                    torch.cat([lds[0], lds[0][:1]]).double(), torch.cat([bs[0], bs[0][:1]]).double(), skip.double())[-1:]
    assert rel_err(more, ref) < 4 * tol


@pytest.mark.parametrize("per_token", [False, True])
def test_decayed_scan_of_a_long_portion_in_segments(per_token):
    """A portion long enough to run as segments side by side (bf16, matrix-core sizes) beside a short one, after a carried
    state: the same rows as the chunks one after the other, and as the plain recurrence."""
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(11)
    H, G, D, P = 2, 1, 64, 32
    lens = {0: 2700, 1: 40}
    dtype = torch.bfloat16
    qs = {k: (torch.randn(n, G, D, generator=g) * D ** -0.25).to(dtype) for k, n in lens.items()}
    ks = {k: (torch.randn(n, G, D, generator=g) * D ** -0.25).to(dtype) for k, n in lens.items()}
    vs = {k: torch.randn(n, H, P, generator=g).to(dtype) for k, n in lens.items()}
    decay = torch.tensor([0.97, 0.999])
    lds = {k: (-torch.rand(n, H, generator=g) * 0.1) if per_token else torch.log2(decay).expand(n, H).contiguous() for k, n in lens.items()}
    bs = {k: (torch.rand(n, H, generator=g) + 0.2) if per_token else torch.ones(n, H) for k, n in lens.items()}
    skip = torch.randn(H, generator=g) if per_token else torch.zeros(H)
    refs = {k: _scan_ref(qs[k].double(), ks[k].double(), vs[k].double(), lds[k].double(), bs[k].double(), skip.double()) for k in lens}
    state = torch.full((2, H, D, P), 3.0, dtype=torch.float32, device=DEV)

    def run(step):
        cat = lambda d: torch.cat([d[k][at:at + n] for k, at, n in step]).to(DEV)      # noqa: E731
        lay = layout_of([n for _, _, n in step], [at for _, at, _ in step], [k for k, _, _ in step])
        kw = dict(log2_decay=cat(lds), v_scale=cat(bs), skip=skip.to(DEV)) if per_token else dict(decay=decay.to(DEV))
        return hip_ops.decay_scan(cat(qs), cat(ks), cat(vs), state, lay.query_start_loc, lay.context_lens, lay.slot_idx, lay.max_query_len, **kw)

    got = in_steps(lens, [[(0, 100)], [(0, 2600), (1, 40)]], run)            # 2600 rows from a carried state: three segments
    for k in lens:
        assert rel_err(got[k], refs[k]) < 6e-3, k
    end = state.clone()
    got = in_steps(lens, [[(0, 1500)], [(0, 1200), (1, 40)]], run)           # below the segments' threshold: chunk after chunk
    assert rel_err(state, end) < 1e-4
    for k in lens:
        assert rel_err(got[k], refs[k]) < 6e-3, k


def test_state_space_recurrence_is_the_scan_with_its_step_sizes():
    """The oracle's state-space recurrence (decay from A and dt, input weighed by dt, the skip) through the scan."""
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(5)
    T, H, G, N, P = 45, 6, 3, 12, 8
    x, B, C = torch.randn(T, H, P, generator=g), torch.randn(T, G, N, generator=g) * 0.5, torch.randn(T, G, N, generator=g) * 0.5
    dt, a_log, D = torch.rand(T, H, generator=g) + 0.1, torch.randn(H, generator=g) * 0.5 - 1, torch.randn(H, generator=g)
    ref = ssd_scan_ref(x.double(), dt.double(), a_log.double(), B.double(), C.double(), D.double()).reshape(T, H * P)
    ld = (-torch.exp(a_log) * dt * math.log2(math.e)).contiguous()
    state = torch.zeros(1, H, N, P, device=DEV)
    lay = layout_of([T], [0], [0])
    out = hip_ops.decay_scan(C.to(DEV), B.to(DEV), x.to(DEV), state, lay.query_start_loc, lay.context_lens, lay.slot_idx, T, log2_decay=ld.to(DEV),
                             v_scale=dt.to(DEV), skip=D.to(DEV))
    assert rel_err(out, ref) < 5e-6


# --------------------------------------------------------------------------- the gated norm in groups
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W,groups,act,first,weighted", [(96, 4, "silu", False, False), (384, 2, "silu", True, True), (4096, 1, "sigmoid", False, True),
                                                        (5120, 1, "silu", True, True), (60, 60, "silu", False, False), (9000, 2, "sigmoid", True, False)])
def test_gated_norm_in_groups_gate_before_or_after(dtype, W, groups, act, first, weighted):
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(W + groups)
    T, eps = 9, 1e-5
    x = torch.randn(T, W, generator=g) * 2
    gate = torch.randn(T, W + 8, generator=g).to(dtype)
    w = 1 + 0.1 * torch.randn(W, generator=g) if weighted else None
    gd = gate[:, :W].double()
    a = F.silu(gd) if act == "silu" else torch.sigmoid(gd)
    norm = lambda t: unit_rms_ref(t.view(T, groups, W // groups), eps).reshape(T, W)      # noqa: E731
    ref = norm(x.double() * a) if first else norm(x.double()) * a
    if weighted:
        ref = ref * w.double()
    out = hip_ops.gated_rms_norm(x.to(DEV), gate.to(DEV)[:, :W], None if w is None else w.to(DEV), eps, groups=groups, gate_act=act, gate_first=first)
    assert rel_err(out, ref) < (2e-6 if dtype == torch.float32 else 4e-3) and out.dtype == dtype


# --------------------------------------------------------------------------- the mixture
def _moe_weights(W, mlp, g, dtype):
    r = mlp["router"]
    n = r["experts"] + r.get("identity", 0)
    lin = lambda o, i: (torch.randn(o, i, generator=g) * i ** -0.5).to(torch.bfloat16).float()      # noqa: E731
    w = {"router": (torch.randn(n, W, generator=g) * 3 * W ** -0.5).to(torch.bfloat16).float(),
         "correction": (torch.randn(n, generator=g) * 0.1).to(torch.bfloat16).float()}
    for e in range(r["experts"]):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = lin(mlp["expert"]["ff"], W), lin(mlp["expert"]["ff"], W), lin(W, mlp["expert"]["ff"])
    if mlp.get("shared"):
        Fs = mlp["shared"]["ff"]
        w["shared.gate"], w["shared.up"], w["shared.down"], w["shared.sg"] = lin(Fs, W), lin(Fs, W), lin(W, Fs), lin(1, W)
    return w


def _moe_module(W, mlp, w, dtype):
    from vllm_hymeta.linear import HymetaLinear
    from vllm_hymeta.models.feed_forward import GroupedSoftmaxMoE, SiluGluMLP
    r = mlp["router"]
    cast = lambda t: t.to(dtype).to(DEV)      # noqa: E731
    w13 = torch.stack([torch.cat([cast(w[f"e{e}.gate"]), cast(w[f"e{e}.up"])], 0) for e in range(r["experts"])])
    w2 = torch.stack([cast(w[f"e{e}.down"]) for e in range(r["experts"])])
    shared = gate = None
    if mlp.get("shared"):
        shared = SiluGluMLP(HymetaLinear.from_weight(torch.cat([cast(w["shared.gate"]), cast(w["shared.up"])], 0).contiguous()),
                            HymetaLinear.from_weight(cast(w["shared.down"])))
        gate = w["shared.sg"].to(DEV)
    grp = r.get("groups") or {"count": 1, "keep": 1}
    return GroupedSoftmaxMoE(w["router"].to(DEV), w["correction"].to(DEV), w13, w2, r["top"], grp["count"], grp["keep"], r.get("identity", 0), shared, gate)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W,cfg", [(48, dict()), (64, dict(experts=9, identity=3, top=4, groups=3, keep=2, ff=64, shared_ff=80)),
                                   (128, dict(experts=6, identity=0, top=2, groups=1, keep=1, ff=32, shared_ff=0)),
                                   (72, dict(experts=2, identity=6, top=3, groups=4, keep=3, ff=24, shared_ff=16)),
                                   (256, dict(experts=16, identity=0, top=1, groups=8, keep=1, ff=128, shared_ff=64)),
                                   (64, dict(experts=7, identity=2, top=9, groups=3, keep=3, ff=40, shared_ff=0))])
def test_experts_chosen_by_corrected_scores_within_the_best_groups(dtype, W, cfg):
    """The block's terms summed, against the oracle: rows whose choice hangs on a margin below the inputs' rounding are
    left out (bf16: the router reads the rounded input, as the oracle here does)."""
    mlp = moe_config(**cfg)
    g = torch.Generator().manual_seed(W + mlp["router"]["experts"])
    w = _moe_weights(W, mlp, g, dtype)
    T = 150
    h = torch.randn(T, W, generator=g).to(dtype)
    ref = moe_ff_ref(h.double(), {k: v.double() for k, v in w.items()}, mlp)
    r = mlp["router"]
    n = r["experts"] + r.get("identity", 0)
    # margins of the choice: the groups' and the outputs'
    s = torch.softmax(h.double() @ w["router"].double().T, -1) + w["correction"].double()
    grp = r["groups"]
    gb = s.view(T, grp["count"], n // grp["count"]).max(-1).values.sort(-1, descending=True).values
    clear = torch.ones(T, dtype=torch.bool)
    if grp["keep"] < grp["count"]:
        clear &= (gb[:, grp["keep"] - 1] - gb[:, grp["keep"]]) > 1e-4
    chosen, _ = grouped_route_ref(h.double() @ w["router"].double().T, w["correction"].double(), r["top"], grp["count"], grp["keep"])
    srt = s.sort(-1, descending=True).values
    if r["top"] < n:
        picked = s.gather(1, chosen).min(-1).values
        rest = s.clone().scatter_(1, chosen, -1e9)
        kept_mask = torch.zeros(T, grp["count"], dtype=torch.bool).scatter_(1, s.view(T, grp["count"], -1).max(-1).values.topk(grp["keep"]).indices, True)
        rest = torch.where(kept_mask[:, :, None].expand(T, grp["count"], n // grp["count"]).reshape(T, n), rest, torch.full_like(rest, -1e9))
        clear &= (picked - rest.max(-1).values) > 1e-4
    assert int(clear.sum()) > T // 2
    mod = _moe_module(W, mlp, w, dtype)
    terms = mod(h.to(DEV))
    out = torch.zeros(T, W, dtype=torch.float64)
    for y, c, rows in terms:
        out += c * y.double().cpu() * (1.0 if rows is None else rows.double().cpu()[:, None])
    assert len(terms) == 1 + (1 if r.get("identity") else 0) + (1 if mlp.get("shared") else 0)
    tol = 5e-6 if dtype == torch.float32 else 1.5e-2
    assert rel_err(out[clear], ref[clear]) < tol


def test_identity_experts_and_a_masked_group_show_in_the_output():
    """A router built by hand: every token's best outputs lie in a group that the correction pushes out of the kept
    groups, and an identity expert takes the largest share -- a choice by uncorrected scores, a masked score of 0
    instead of minus infinity, or a dropped identity term would each change the result."""
    W = 32
    mlp = moe_config(experts=4, identity=4, top=3, groups=4, keep=2, ff=16, shared_ff=0)
    g = torch.Generator().manual_seed(1)
    w = _moe_weights(W, mlp, g, torch.float32)
    w["router"].zero_()
    w["router"][:, 0] = torch.tensor([2.0, 1.9, 0.5, 0.4, 1.0, 0.9, 0.2, 0.1])        # group 0 = outputs 0, 1 ... group 3 = 6, 7
    w["correction"] = torch.tensor([-1.0, -1.0, 0.0, 0.0, 0.0, 0.0, -0.5, -0.5])       # pushes group 0 (and 3) behind 1 and 2; negative scores stay candidates
    h = torch.randn(20, W, generator=g)
    h[:, 0] = 1.0
    chosen, weights = grouped_route_ref(h.double() @ w["router"].double().T, w["correction"].double(), 3, 4, 2)
    assert sorted(chosen[0].tolist()) == [2, 4, 5]                                      # experts of groups 1 and 2, two of them identity experts
    ref = moe_ff_ref(h.double(), {k: v.double() for k, v in w.items()}, mlp)
    terms = _moe_module(W, mlp, w, torch.float32)(h.to(DEV))
    out = sum(c * y.double().cpu() * (1.0 if rows is None else rows.double().cpu()[:, None]) for y, c, rows in terms)
    assert rel_err(out, ref) < 5e-6
    assert rel_err(terms[0][0].double().cpu(), ref) > 0.3                               # without the identity term it is far off


# --------------------------------------------------------------------------- whole models under the engine
def build_engine(cfg, weights, dtype, max_tokens=512, block_size=16, max_num_seqs=4, max_num_batched_tokens=1 << 30):
    from vllm_hymeta.engine import LLMEngine
    from vllm_hymeta.models.configuration_dapuzen import DapuzenConfig
    from vllm_hymeta.models.modeling_dapuzen import DapuzenForCausalLM
    model = DapuzenForCausalLM(DapuzenConfig(cfg), max_num_seqs=max_num_seqs, dtype=dtype, device=DEV)
    model.load_weights(weights.items())
    return LLMEngine(model, num_blocks=max_tokens // block_size, block_size=block_size, max_num_seqs=max_num_seqs,
                     max_num_batched_tokens=max_num_batched_tokens, device=DEV)


_DENSE = {"kind": "dense", "ff": 72}

MODELS = {
    "default": dict(),
    "ones_and_equals": dict(width=40, embed_scale=1.0, layers=[       # one head, one group, window 1, no rotation, no identity, no shared, top 1
        ("attention", attention_mixer_config(heads=1, kv_heads=1, dim=8, vdim=8, window=1, rot_dims=0), None),
        ("parallel", parallel_mixer_config(heads=1, kv_heads=1, dim=8, vdim=8, window=None, softcap=None, ssm_heads=1, ssm_vdim=8, state=4, groups=1,
                                           norm_groups=1, conv=1, left_scale=1.0, right_scale=1.0), moe_config(experts=3, identity=0, top=1, groups=1, keep=1, ff=16, shared_ff=0)),
        ("retention", retention_mixer_config(heads=1, dim=8, vdim=8, rot_dims=0, decay=[1.0]), _DENSE),
        ("weights_of", 0)]),
    "matrix_core_sizes": dict(width=128, layers=[
        ("attention", attention_mixer_config(heads=8, kv_heads=2, dim=64, vdim=64, window=70, rot_dims=64), {"kind": "dense", "ff": 192}),
        ("parallel", parallel_mixer_config(heads=8, kv_heads=4, dim=128, vdim=128, window=130, softcap=8.0, ssm_heads=4, ssm_vdim=64, state=64, groups=2,
                                           norm_groups=4, conv=4), moe_config(experts=10, identity=2, top=3, groups=4, keep=2, ff=64, shared_ff=128)),
        ("retention", retention_mixer_config(heads=4, dim=32, vdim=64, rot_dims=32), None),
        ("attention", attention_mixer_config(heads=16, kv_heads=16, dim=64, vdim=128, window=64, rot_dims=16), moe_config(experts=8, identity=0, top=2, groups=2, keep=1, ff=64, shared_ff=0)),
        ("weights_of", 1), ("weights_of", 2)]),
    "retention_first_parallel_last": dict(width=64, layers=[
        ("retention", retention_mixer_config(heads=2, dim=64, vdim=32, rot_dims=20), moe_config(experts=4, identity=2, top=2, groups=2, keep=2, ff=32, shared_ff=24)),
        ("weights_of", 0),
        ("parallel", parallel_mixer_config(heads=6, kv_heads=3, dim=20, vdim=12, window=33, softcap=1.0, ssm_heads=8, ssm_vdim=16, state=128, groups=1,
                                           norm_groups=8, conv=2), _DENSE)]),
}


def _tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def _all_chosen(cfg):
    """bf16: every router output chosen, every group kept, so that a rounding cannot flip the choice."""
    c = copy.deepcopy(cfg)
    for entry in c["layers"]:
        if entry["mlp"] and entry["mlp"]["kind"] == "moe":
            r = entry["mlp"]["router"]
            r["top"] = r["experts"] + r.get("identity", 0)
            r["groups"] = dict(r["groups"], keep=r["groups"]["count"])
    return c


@pytest.mark.parametrize("name", sorted(MODELS))
def test_model_whole_prompt_against_the_oracle_fp32(name):
    """One step for the whole prompt, every position's logits and the stream after every layer."""
    cfg = dapuzen_config(**MODELS[name])
    weights = dapuzen_random_weights(cfg, seed=len(name))
    toks = _tokens(170, cfg["vocab"], 7)
    stream_ref = []
    ref = dapuzen_ref(cfg, weights, toks, residual_out=stream_ref)
    eng = build_engine(cfg, weights, torch.float32, max_tokens=256, block_size=16)
    stream = []
    inner = eng.model.model
    plain = inner.forward
    inner.forward = lambda *a, **k: plain(*a, residual_out=stream, **k)
    got = eng.run_batch([("a", toks, list(range(len(toks))))])
    assert len(stream) == len(cfg["layers"])
    for i, (s, r) in enumerate(zip(stream, stream_ref)):
        assert rel_err(s, r) < 2e-5, (i, cfg["layers"][i]["type"])
    assert rel_err(got, ref) < 5e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", sorted(MODELS))
def test_model_schedules_agree_with_the_whole_prompt(name, dtype):
    cfg = dapuzen_config(**MODELS[name])
    if dtype == torch.bfloat16:
        cfg = _all_chosen(cfg)
    weights = dapuzen_random_weights(cfg, seed=len(name))
    V = cfg["vocab"]
    seqs = {k: _tokens(n, V, 10 + k) for k, n in enumerate([150, 33, 1, 70, 19, 64])}
    refs = {k: dapuzen_ref(cfg, weights, t) for k, t in seqs.items()}
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
    cfg = dapuzen_config(**MODELS["default"])
    weights = dapuzen_random_weights(cfg, seed=4)
    prompts = [_tokens(n, cfg["vocab"], 40 + n) for n in (23, 5, 1, 37, 12, 18)]
    new = 5
    eng = build_engine(cfg, weights, torch.float32, max_tokens=128, block_size=16, max_num_seqs=2, max_num_batched_tokens=16)
    outs = eng.generate(prompts, SamplingParams(max_tokens=new))
    assert eng.pool.num_free == 8 and not eng.requests
    for p, o in zip(prompts, outs):
        assert len(o) == new
        toks = list(p)
        for t in o:
            logits = dapuzen_ref(cfg, weights, toks)[-1]
            top2 = logits.topk(2).values
            if float(top2[0] - top2[1]) > 1e-3:        # a clear winner: the engine must have picked it
                assert t == int(logits.argmax())
            toks.append(t)


@pytest.mark.parametrize("dtype,name", [(torch.float32, "default"), (torch.bfloat16, "matrix_core_sizes")])
def test_long_decode_passes_every_window_and_keeps_its_states(dtype, name):
    """400 tokens decoded one by one after a two-token prompt: every window passes over decoded tokens many times, the
    recurrent and convolution states are carried 400 times."""
    cfg = dapuzen_config(**MODELS[name])
    if dtype == torch.bfloat16:
        cfg = _all_chosen(cfg)
    weights = dapuzen_random_weights(cfg, seed=8)
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
        ref = dapuzen_ref(cfg, weights, toks[:201])[-1:]
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
    cfg = dapuzen_config(**MODELS["default"])
    weights = {k: v.to(torch.bfloat16).float() for k, v in dapuzen_random_weights(cfg, seed=12).items()}      # what a bf16 file holds
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
    ra, rb = dapuzen_ref(cfg, weights, a), dapuzen_ref(cfg, weights, b)
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
        logits = dapuzen_ref(cfg, weights, toks)[-1]
        top2 = logits.topk(2).values
        if float(top2[0] - top2[1]) > 1e-3:
            assert t == int(logits.argmax())
        toks.append(t)
    assert len(line["output"]) == 3


def _random_model(seed):
    """Sizes drawn at random: layer order, head counts, group sizes, key, value and state sizes (also such that a layer
    takes the matrix-core kernels), windows around a page and a tile, rotated parts, taps, routers."""
    import random
    r = random.Random(seed)
    width = r.choice([24, 40, 64, 96, 128, 200])

    def attn(biased):
        G = r.choice([1, 2, 3, 4])
        H = G * r.choice([1, 2, 3, 5])
        D, Dv = r.choice([(64, 64), (128, 64), (64, 128), (128, 128)]) if r.random() < 0.4 else (2 * r.randint(2, 24), r.randint(3, 50))
        window = r.choice([None, 1, 2, 7, 15, 16, 17, 63, 64, 65, 100, 128, 1000])
        return dict(heads=H, kv_heads=G, dim=D, vdim=Dv, window=window), D

    layers = []
    for _ in range(r.randint(1, 5)):
        kind = r.choice(["attention", "parallel", "retention", "weights_of"])
        if kind == "weights_of" and not any(l[0] != "weights_of" for l in layers):
            kind = "attention"
        ff = r.choice(["dense", "moe", "moe", None])
        if ff == "moe":
            groups = r.choice([1, 2, 3, 4])
            per = r.randint(1, 4)
            outputs = groups * per
            identity = r.randint(0, outputs - 1)
            keep = r.randint(1, groups)
            mlp = moe_config(experts=outputs - identity, identity=identity, top=r.randint(1, keep * per), groups=groups, keep=keep,
                             ff=r.choice([8, 40, 64, 128]), shared_ff=r.choice([0, 16, 64]))
        else:
            mlp = None if ff is None else {"kind": "dense", "ff": r.choice([16, 72, 128])}
        if kind == "weights_of":
            layers.append(("weights_of", r.choice([i for i, l in enumerate(layers) if l[0] != "weights_of"])))
        elif kind == "attention":
            a, D = attn(False)
            layers.append((kind, attention_mixer_config(**a, rot_dims=r.choice([0, 2, D // 2 * 2, D // 4 * 2]), base=r.choice([10.0, 10000.0, 500000.0]),
                                                        scale=r.choice([D ** -0.5, 0.3, 0.05])), mlp))
        elif kind == "retention":
            H, D = r.choice([1, 2, 3, 4]), r.choice([8, 16, 32, 64, 128, 20])
            layers.append((kind, retention_mixer_config(heads=H, dim=D, vdim=r.choice([8, 32, 64, 24, 100]), rot_dims=r.choice([0, 2, D, D // 4 * 2]),
                                                        base=r.choice([10.0, 2e6]), decay=[r.choice([1.0, 0.99, 0.9, 0.5]) for _ in range(H)]), mlp))
        else:
            a, D = attn(True)
            G = r.choice([1, 2, 3])
            P = r.choice([8, 16, 64, 12, 32])
            ssm_heads = G * r.choice([1, 2, 4])
            ng = r.choice([g for g in (1, 2, 4, ssm_heads) if (ssm_heads * P) % g == 0])
            layers.append((kind, parallel_mixer_config(heads=a["heads"], kv_heads=a["kv_heads"], dim=a["dim"], vdim=a["vdim"], window=a["window"],
                                                       softcap=r.choice([None, 0.5, 5.0, 50.0]), ssm_heads=ssm_heads, ssm_vdim=P,
                                                       state=r.choice([4, 16, 32, 64, 128, 24]), groups=G, norm_groups=ng, conv=r.choice([1, 2, 3, 4, 5]),
                                                       left_scale=r.choice([1.0, 0.6]), right_scale=r.choice([1.0, 1.7])), mlp))
    return dapuzen_config(vocab=r.choice([50, 130]), width=width, layers=layers, eps=r.choice([1e-5, 1e-6, 1e-3]), embed_scale=r.choice([1.0, 2.5, 8.0]))


@pytest.mark.parametrize("seed", range(12))
def test_models_of_random_sizes_under_the_engine(seed):
    """fp32: a prompt of 210 tokens in one step, then in portions and single tokens beside a second request, against the
    oracle; bf16 (every expert chosen): the same schedule against the one-step result."""
    cfg = _random_model(seed)
    weights = dapuzen_random_weights(cfg, seed=seed)
    V = cfg["vocab"]
    a, b = _tokens(210, V, 100 + seed), _tokens(75, V, 200 + seed)
    ra, rb = dapuzen_ref(cfg, weights, a), dapuzen_ref(cfg, weights, b)
    page = 64 if seed % 2 else 16
    plan = [[(0, 3)], [(0, 64), (1, 2)], [(0, 1), (1, 1)], [(0, 62), (1, 70)], [(0, 1), (1, 1)], [(0, 2), (1, 1)], [(0, 77)]]
    for dtype in (torch.float32, torch.bfloat16):
        c = cfg if dtype == torch.float32 else _all_chosen(cfg)
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
