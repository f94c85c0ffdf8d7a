"""Host side of the Dapuzen family: configuration, registry, kernel sources, and the oracle's own consistency (no GPU)."""
import json
import os

import pytest
import torch

from oracle.dapuzen import (attention_mixer_config, causal_conv_ref, dapuzen_config, dapuzen_random_weights, dapuzen_ref, grouped_route_ref,
                            moe_config, parallel_mixer_config, retention_mixer_config, rotate_half_ref, window_attention_ref)


def test_config_reads_every_size_and_constant():
    from vllm_hymeta.models.configuration_dapuzen import (DapuzenConfig, DenseMlpSpec, GroupedMoeSpec, RetentionSpec, SideBySideSpec,
                                                          WindowAttentionSpec)
    raw = dapuzen_config(vocab=90, width=60, eps=3e-6, embed_scale=7.5, layers=[
        ("attention", attention_mixer_config(heads=6, kv_heads=3, dim=10, vdim=14, window=21, rot_dims=6, base=5000.0, scale=0.3), None),
        ("parallel", parallel_mixer_config(heads=4, kv_heads=2, dim=12, vdim=20, window=5, softcap=7.0, ssm_heads=6, ssm_vdim=10, state=14, groups=3,
                                           norm_groups=5, conv=3, left_scale=0.4, right_scale=1.6),
         moe_config(experts=5, identity=3, top=3, groups=4, keep=2, ff=20, shared_ff=36)),
        ("retention", retention_mixer_config(heads=2, dim=8, vdim=42, rot_dims=4, base=77.0, decay=[0.5, 0.75]), {"kind": "dense", "ff": 44}),
        ("weights_of", 1)])
    cfg = DapuzenConfig(raw)
    assert (cfg.vocab_size, cfg.hidden_size, cfg.norm_eps, cfg.embedding_scale, cfg.num_hidden_layers) == (90, 60, 3e-6, 7.5, 4)
    a = cfg.layers[0].mixer
    assert isinstance(a, WindowAttentionSpec) and (a.heads, a.kv_heads, a.dim, a.vdim, a.window, a.rot_dims, a.rot_base, a.scale) == (6, 3, 10, 14, 21, 6, 5000.0, 0.3)
    assert a.gate and not a.bias and a.softcap is None and a.frequencies() == [5000.0 ** (-2.0 * i / 6) for i in range(3)] and cfg.layers[0].mlp is None
    p = cfg.layers[1].mixer
    assert isinstance(p, SideBySideSpec) and (p.left_scale, p.right_scale) == (0.4, 1.6) and p.left.bias and not p.left.gate
    assert (p.left.softcap, p.left.window, p.left.rot_dims) == (7.0, 5, 0)
    r = p.right
    assert (r.heads, r.vdim, r.state, r.groups, r.norm_groups, r.conv, r.inner, r.conv_channels) == (6, 10, 14, 3, 5, 3, 60, 60 + 2 * 3 * 14)
    moe = cfg.layers[1].mlp
    assert isinstance(moe, GroupedMoeSpec) and (moe.experts, moe.identity, moe.top, moe.groups, moe.keep, moe.ff, moe.shared_ff) == (5, 3, 3, 4, 2, 20, 36)
    t = cfg.layers[2].mixer
    assert isinstance(t, RetentionSpec) and (t.heads, t.dim, t.vdim, t.decay, t.rot_dims, t.rot_base) == (2, 8, 42, [0.5, 0.75], 4, 77.0)
    assert isinstance(cfg.layers[2].mlp, DenseMlpSpec) and cfg.layers[2].mlp.ff == 44
    assert [l.weights_of for l in cfg.layers] == [0, 1, 2, 1] and cfg.layers[3].type == "parallel"
    # what a file may leave out: the window, the rotation, the cap, identity experts, groups, the shared expert
    bare = dapuzen_config()
    del bare["layers"][0]["mixer"]["mask"], bare["layers"][0]["mixer"]["rot"], bare["layers"][1]["mixer"]["left"]["softcap"]
    del bare["layers"][1]["mlp"]["router"]["identity"], bare["layers"][1]["mlp"]["router"]["groups"], bare["layers"][1]["mlp"]["shared"]
    bare["layers"][1]["mlp"]["router"]["top"] = 2
    cfg = DapuzenConfig(bare)
    assert cfg.layers[0].mixer.window is None and cfg.layers[0].mixer.rot_dims == 0 and cfg.layers[1].mixer.left.softcap is None
    m = cfg.layers[1].mlp
    assert (m.identity, m.groups, m.keep, m.shared_ff) == (0, 1, 1, 0)
    for breaker in (lambda c: c["layers"][0].update(type="lstm"), lambda c: c["layers"][0]["mixer"].update(kv_heads=4),
                    lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), lambda c: c["layers"][0]["mixer"]["rot"].update(dims=64),
                    lambda c: c["layers"][1]["mlp"]["router"].update(top=9), lambda c: c["layers"][1]["mlp"].update(kind="conv"),
                    lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=3), lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(keep=1),
                    lambda c: c["layers"][2]["mixer"].update(decay=[0.5]), lambda c: c["layers"][1]["mixer"]["right"].update(groups=4),
                    lambda c: c["layers"][3].update(weights_of=7), lambda c: c["layers"][0]["mixer"]["mask"].update(size=0)):
        bad = json.loads(json.dumps(dapuzen_config()))
        breaker(bad)
        with pytest.raises(ValueError):
            DapuzenConfig(bad)


def test_registry_serves_the_family(tmp_path):
    from vllm_hymeta import registry
    from vllm_hymeta.models.configuration_dapuzen import DapuzenConfig
    (tmp_path / "config.json").write_text(json.dumps(dapuzen_config()))
    assert registry.architecture_of(str(tmp_path)) == "Dapuzen" and "Dapuzen" in registry.known_architectures()
    cls, cfg = registry.resolve(str(tmp_path))
    assert cls.__name__ == "DapuzenForCausalLM" and isinstance(cfg, DapuzenConfig)
    sources = registry.kernel_sources(str(tmp_path))
    assert tuple(sources) == tuple(cls.kernel_sources) and {"parallel_ops", "decay_scan", "sink_attn", "moe_sigmoid"} <= set(sources)
    csrc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "vllm-hymeta_amd", "csrc")
    assert all(os.path.exists(os.path.join(csrc, s + ".hip")) for s in sources)


def test_checkpoint_names_load_into_the_model_on_the_cpu():
    """Every tensor of the oracle's checkpoint is taken by name and shape; a missing or misshapen one is refused."""
    from vllm_hymeta.models.configuration_dapuzen import DapuzenConfig
    from vllm_hymeta.models.modeling_dapuzen import DapuzenForCausalLM
    cfg = dapuzen_config()
    w = dapuzen_random_weights(cfg, seed=2)
    model = DapuzenForCausalLM(DapuzenConfig(cfg), max_num_seqs=2, dtype=torch.float32, device="cpu")
    assert model.load_weights(w.items()) == set(w)
    assert sorted(model.model.blocks) == ["0", "1", "2", "4"] and sorted(model.model.attn_layers) == ["0", "1", "3", "4"]
    rec, conv = model.model.state_cache.cache
    assert [tuple(t.shape) for t in rec] == [(1, 2, 6, 12, 8), (1, 2, 3, 16, 24), (1, 2, 6, 12, 8)] and [tuple(t.shape) for t in conv] == [(1, 2, 2, 120)] * 2
    short = dict(w)
    del short["l1.mix.right.A_log"]
    with pytest.raises(KeyError):
        DapuzenForCausalLM(DapuzenConfig(cfg), max_num_seqs=2, dtype=torch.float32, device="cpu").load_weights(short.items())
    bad = dict(w, **{"l0.mix.g": torch.zeros(7, cfg["width"])})
    with pytest.raises(ValueError):
        DapuzenForCausalLM(DapuzenConfig(cfg), max_num_seqs=2, dtype=torch.float32, device="cpu").load_weights(bad.items())


def test_rotation_window_convolution_and_choice_of_the_oracle():
    x = torch.arange(2 * 1 * 6, dtype=torch.float64).view(2, 1, 6) + 1
    out = rotate_half_ref(x, 4, 10.0)
    assert torch.equal(out[0], x[0]) and torch.equal(out[:, :, 4:], x[:, :, 4:])          # position 0 and the unrotated rest pass
    c, s = torch.cos(torch.tensor(1.0, dtype=torch.float64)), torch.sin(torch.tensor(1.0, dtype=torch.float64))
    assert torch.allclose(out[1, 0, 0], x[1, 0, 0] * c - x[1, 0, 2] * s) and torch.allclose(out[1, 0, 2], x[1, 0, 2] * c + x[1, 0, 0] * s)
    # a window of 3: query 5 sees keys 3, 4, 5
    T = 8
    q, k = torch.ones(T, 1, 2, dtype=torch.float64), torch.zeros(T, 1, 2, dtype=torch.float64)
    v = torch.arange(T, dtype=torch.float64).view(T, 1, 1)
    assert torch.allclose(window_attention_ref(q, k, v, 1.0, 3)[5, 0, 0], torch.tensor(4.0, dtype=torch.float64))
    assert torch.allclose(window_attention_ref(q, k, v, 1.0, None)[5, 0, 0], torch.tensor(2.5, dtype=torch.float64))
    # the last tap weighs the current token
    xs = torch.tensor([[1.0], [10.0], [100.0]], dtype=torch.float64)
    y = causal_conv_ref(xs, torch.tensor([[3.0, 2.0]], dtype=torch.float64), torch.tensor([0.5], dtype=torch.float64))
    assert y[:, 0].tolist() == [2.5, 23.5, 230.5]
    # a masked group is out whatever its scores; the weights are the uncorrected scores
    logits = torch.log(torch.tensor([[0.4, 0.3, 0.2, 0.1]], dtype=torch.float64))
    chosen, weights = grouped_route_ref(logits, torch.tensor([-1.0, -1.0, 0.0, 0.0], dtype=torch.float64), 2, 2, 1)
    assert sorted(chosen[0].tolist()) == [2, 3] and torch.allclose(weights.sum(), torch.tensor(0.3, dtype=torch.float64))


def test_every_mechanism_shows_in_the_oracles_logits():
    cfg = dapuzen_config()
    w = dapuzen_random_weights(cfg, seed=1)
    toks = torch.randint(0, cfg["vocab"], (40,), generator=torch.Generator().manual_seed(0)).tolist()
    ref = dapuzen_ref(cfg, w, toks)

    def moved(cfg2=None, w2=None):
        out = dapuzen_ref(cfg2 or cfg, w2 or w, toks)
        return float((out - ref).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt())

    def changed(path, value):
        c = json.loads(json.dumps(cfg))
        node = c
        for key in path[:-1]:
            node = node[key]
        node[path[-1]] = value
        return c

    assert moved() == 0.0
    for path, value in ((("embedding", "scale"), 1.0), (("layers", 0, "mixer", "mask", "size"), 12), (("layers", 0, "mixer", "rot", "dims"), 8),
                        (("layers", 1, "mixer", "left", "softcap"), 0.5), (("layers", 1, "mixer", "left_scale"), 0.1),
                        (("layers", 1, "mixer", "right", "norm_groups"), 1), (("layers", 1, "mlp", "router", "groups", "keep"), 4),
                        (("layers", 2, "mixer", "decay"), [0.5, 0.5, 0.5]), (("layers", 2, "mixer", "rot", "base"), 10.0), (("norm", "eps"), 0.5)):
        assert moved(changed(path, value)) > 1e-4, path
    for name in ("l0.mix.g", "l1.mix.left.k.b", "l1.mix.right.D", "l1.mix.right.conv.b", "l1.mix.right.dt_bias", "l1.mlp.correction", "l1.mlp.shared.sg",
                 "l2.mix.g", "l0.norm1", "final.norm", "l0.mlp.act"):
        w2 = dict(w)
        # (the same amount on every correction would leave the order as it is)
        w2[name] = w[name] + (0.5 * (torch.arange(w[name].numel()) % 2).reshape(w[name].shape) if name.endswith("correction") else 0.5)
        assert moved(w2=w2) > 1e-4, name
    # a layer that runs another's weights has a state of its own: its output differs from the owner's
    stream = []
    dapuzen_ref(cfg, w, toks, residual_out=stream)
    assert float((stream[3] - stream[2]).abs().max()) > 1e-3
