"""Host side of the Lidizen family: configuration, registry, kernel sources, and the oracle's own consistency (no GPU)."""
import json

import pytest
import torch

from oracle.lidizen import (attention_config, bigram_rows_ref, hyper_step_ref, lidizen_config, lidizen_random_weights, lidizen_ref,
                            shared_key_attention_ref, talking_attention_ref, visible_ref)


def _layer(mixer, mlp):
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def test_config_reads_every_size_and_constant():
    from vllm_hymeta.models.configuration_lidizen import LidizenConfig, Relu2MoeSpec, SiluMlpSpec
    raw = lidizen_config(vocab=90, width=60, streams=5, eps=3e-6, bigram=(97, 13, 3), layers=[
        _layer(attention_config(heads=6, kv_heads=3, dim=10, vdim=14, size=21, keep_first=4, rot_dims=6, base=5000.0, scale=0.3, v_mix=False), None),
        _layer(attention_config(heads=2, kv_heads=1, dim=8, vdim=42, size=7, keep_first=0, rot_dims=8, v_mix=True),
               {"kind": "moe", "expert": {"ff": 20}, "router": {"experts": 7, "top": 3}}),
        _layer(attention_config(heads=7, kv_heads=7, dim=4, vdim=6, rot_dims=2, v_mix=True), {"kind": "dense", "ff": 44})])
    cfg = LidizenConfig(raw)
    assert (cfg.vocab_size, cfg.hidden_size, cfg.streams, cfg.norm_eps, cfg.num_hidden_layers) == (90, 60, 5, 3e-6, 3)
    assert (cfg.bigram.buckets, cfg.bigram.mul_prev, cfg.bigram.mul_cur) == (97, 13, 3)
    a = cfg.layers[0].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.window, a.keep_first, a.rot_dims, a.rot_base, a.scale, a.v_mix) == (6, 3, 10, 14, 21, 4, 6, 5000.0, 0.3, False)
    assert a.frequencies() == [5000.0 ** (-2.0 * i / 6) for i in range(3)] and cfg.layers[0].mlp is None
    moe, dense = cfg.layers[1].mlp, cfg.layers[2].mlp
    assert isinstance(moe, Relu2MoeSpec) and (moe.experts, moe.top, moe.ff) == (7, 3, 20)
    assert isinstance(dense, SiluMlpSpec) and dense.ff == 44
    # what a file may leave out: streams, the pair table, the window
    bare = lidizen_config(streams=0, bigram=None)
    del bare["layers"][0]["mixer"]["mask"]
    cfg = LidizenConfig(bare)
    assert cfg.streams == 0 and cfg.bigram is None and cfg.layers[0].mixer.window is None and cfg.layers[0].mixer.keep_first == 0
    for breaker in (lambda c: c["layers"][0].update(type="lstm"), lambda c: c["layers"][0]["mixer"].update(kv_heads=3),
                    lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), lambda c: c["layers"][0]["mixer"]["rot"].update(dims=64),
                    lambda c: c["layers"][1]["mlp"]["router"].update(top=9), lambda c: c["layers"][1]["mlp"].update(kind="conv"),
                    lambda c: c["layers"][1]["mixer"].update(vdim=5)):
        bad = json.loads(json.dumps(lidizen_config()))
        breaker(bad)
        with pytest.raises(ValueError):
            LidizenConfig(bad)


def test_registry_serves_the_family(tmp_path):
    from vllm_hymeta import registry
    from vllm_hymeta.models.configuration_lidizen import LidizenConfig
    (tmp_path / "config.json").write_text(json.dumps(lidizen_config()))
    assert registry.architecture_of(str(tmp_path)) == "Lidizen" and "Lidizen" in registry.known_architectures()
    cls, cfg = registry.resolve(str(tmp_path))
    assert cls.__name__ == "LidizenForCausalLM" and isinstance(cfg, LidizenConfig)
    sources = registry.kernel_sources(str(tmp_path))
    assert tuple(sources) == tuple(cls.kernel_sources) and {"hyper_stream", "talk_attn", "sink_attn"} <= set(sources)
    import os
    csrc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "vllm-hymeta_amd", "csrc")
    assert all(os.path.exists(os.path.join(csrc, s + ".hip")) for s in sources)


def test_pair_rows_and_visibility():
    assert bigram_rows_ref([3, 4, 4, 0], 10, 7, 5) == [10, (3 * 7 + 4 * 5) % 10, (4 * 7 + 4 * 5) % 10, (4 * 7) % 10]
    vis = visible_ref(8, 3, 2)
    assert vis[7].tolist() == [True, True, False, False, False, True, True, True]
    assert vis[2].tolist() == [True, True, True] + [False] * 5 and vis[4].tolist() == [True, True, True, True, True, False, False, False]


def test_every_mechanism_shows_in_the_oracles_logits():
    cfg = lidizen_config()
    w = lidizen_random_weights(cfg, seed=1)
    toks = torch.randint(0, cfg["vocab"], (40,), generator=torch.Generator().manual_seed(0)).tolist()
    ref = lidizen_ref(cfg, w, toks)

    def moved(cfg2=None, w2=None):
        out = lidizen_ref(cfg2 or cfg, w2 or w, toks)
        return float((out - ref).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt())

    def with_mixer(**kw):
        c = json.loads(json.dumps(cfg))
        for layer in c["layers"]:
            for k, v in kw.items():
                if isinstance(v, dict):
                    layer["mixer"][k].update(v)
                else:
                    layer["mixer"][k] = v
        return c

    assert moved(with_mixer(mask={"size": 13})) > 1e-3 and moved(with_mixer(mask={"keep_first": 3})) > 1e-3
    assert moved(with_mixer(rot={"dims": 6})) > 1e-3 and moved(with_mixer(rot={"base": 50.0})) > 1e-3
    assert moved(with_mixer(v_mix=False)) > 1e-3 and moved(with_mixer(scale=0.3)) > 1e-3
    assert moved(w2=dict(w, **{"l1.mix.talk": torch.eye(4)})) > 1e-3
    assert moved(w2=dict(w, **{"l1.mix.vmix": torch.tensor(0.9)})) > 1e-3
    assert moved(w2=dict(w, **{"l0.mix.vmix": torch.tensor(0.9)})) == 0.0                 # the first blending layer's weight is not used
    assert moved(w2=dict(w, **{"l0.hc2.mix": w["l0.hc2.mix"].T.contiguous()})) > 1e-3
    assert moved(w2=dict(w, **{"l1.mlp.router.b": torch.zeros(6)})) > 1e-3
    c = json.loads(json.dumps(cfg))
    c["embedding"]["bigram"]["mul_prev"] = 11
    assert moved(c) > 1e-3
    # one stream with unit weights is the plain residual
    plain = lidizen_config(streams=0)
    wp = lidizen_random_weights(plain, seed=2)
    one = lidizen_config(streams=1)
    w1 = dict(wp)
    for i, layer in enumerate(one["layers"]):
        for q in (1, 2):
            w1[f"l{i}.hc{q}.in"], w1[f"l{i}.hc{q}.out"], w1[f"l{i}.hc{q}.mix"] = torch.ones(1), torch.ones(1), torch.ones(1, 1)
    assert torch.allclose(lidizen_ref(plain, wp, toks), lidizen_ref(one, w1, toks), rtol=1e-12, atol=1e-12)


def test_the_mix_of_the_scores_moves_onto_the_queries():
    """What the product path rests on: scores mixed across heads equal the mixed queries against the concatenated keys."""
    g = torch.Generator().manual_seed(3)
    m = attention_config(heads=6, kv_heads=3, dim=8, vdim=5, size=9, keep_first=2, rot_dims=0)
    T, W = 30, 20
    cfg = lidizen_config(width=W, layers=[_layer(m, None)], streams=0, bigram=None)
    w = {k[len("l0.mix."):]: v.double() for k, v in lidizen_random_weights(cfg, seed=5).items() if k.startswith("l0.mix.")}
    w["q.norm"], w["k.norm"] = torch.ones(48, dtype=torch.float64), torch.ones(24, dtype=torch.float64)
    h = torch.randn(T, W, generator=g, dtype=torch.float64)
    ref, _ = talking_attention_ref(h, w, m, 0.0, None, False)
    q = (h @ w["q"].T + w["q.b"])
    k = (h @ w["k"].T + w["k.b"])
    q = (q / q.pow(2).mean(-1, keepdim=True).sqrt()).reshape(T, 6, 8)
    k = k / k.pow(2).mean(-1, keepdim=True).sqrt()
    v = h @ w["v"].T + w["v.b"]
    mixed = torch.zeros(T, 6, 24, dtype=torch.float64)
    for hh in range(6):
        for j in range(6):
            mixed[:, hh, (j // 2) * 8:(j // 2) * 8 + 8] += w["talk"][hh, j] * q[:, j]
    o = shared_key_attention_ref(mixed, torch.cat([k, v], 1), 3, 5, m["scale"], 0, 9, 2).reshape(T, 30)
    assert torch.allclose(o @ w["o"].T, ref, rtol=1e-10, atol=1e-10)
    xs = torch.randn(4, 3, 7, generator=g, dtype=torch.float64)
    eye = torch.eye(3, dtype=torch.float64)
    assert torch.equal(hyper_step_ref(xs, None, eye, torch.zeros(3, dtype=torch.float64)), xs)
