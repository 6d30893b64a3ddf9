"""Host side of the Geponex family: configuration, rotary frequencies, registry, kernel sources, and the oracle's own
consistency (no GPU)."""
import json
import math

import pytest
import torch

from oracle.geponex import (geponex_config, geponex_random_weights, geponex_ref, group_norm_ref, latent_mixer_config,
                            lightning_mixer_config, moe_config, rotary_frequencies_ref, xielu_ref)


def test_config_reads_every_size_and_the_layers_that_share_weights():
    from vllm_hymeta.models.configuration_geponex import DenseMlpSpec, GeponexConfig, LatentAttentionSpec, LightningSpec, MoeMlpSpec
    raw = geponex_config(vocab=90, width=60, groups=5, eps=3e-6, alpha=1.25, layers=[
        ("lightning", lightning_mixer_config(heads=5, dim=4, vdim=12), None),
        ("latent_attention", latent_mixer_config(heads=3, dim=8, rot_dim=6, vdim=10, kv_rank=14, q_rank=22, base=5000.0, scale=0.3,
                                                 scaling={"factor": 2.0, "original": 32, "fast": 8.0, "slow": 1.0}),
         moe_config(experts=7, top=3, ff=20, limit=0.9, scale=1.5, shared_ff=12, shared_limit=3.0)),
        ("latent_attention_2", latent_mixer_config(), {"kind": "dense", "ff": 44}),
        ("weights_of", 1)])
    cfg = GeponexConfig(raw)
    assert (cfg.vocab_size, cfg.hidden_size, cfg.norm_groups, cfg.norm_eps, cfg.postln_alpha) == (90, 60, 5, 3e-6, 1.25)
    assert [l.weights_of for l in cfg.layers] == [0, 1, 2, 1]
    lt, la, l2 = cfg.layers[0].mixer, cfg.layers[1].mixer, cfg.layers[2].mixer
    assert isinstance(lt, LightningSpec) and (lt.heads, lt.dim, lt.vdim, len(lt.decay)) == (5, 4, 12, 5) and cfg.layers[0].mlp is None
    assert isinstance(la, LatentAttentionSpec) and (la.heads, la.dim, la.rot_dim, la.vdim, la.kv_rank, la.q_rank, la.scale) == (3, 8, 6, 10, 14, 22, 0.3)
    assert (la.sink, la.gate, l2.sink, l2.gate) == (False, False, True, True) and la.rot.scaling["factor"] == 2.0 and l2.rot.scaling is None
    moe = cfg.layers[1].mlp
    assert isinstance(moe, MoeMlpSpec) and (moe.experts, moe.top, moe.route_scale, moe.expert.ff, moe.expert.limit) == (7, 3, 1.5, 20, 0.9)
    assert (moe.shared.ff, moe.shared.limit) == (12, 3.0) and isinstance(cfg.layers[2].mlp, DenseMlpSpec) and cfg.layers[2].mlp.ff == 44
    assert cfg.layers[3].type == "latent_attention" and cfg.layers[3].mlp.top == 3
    bad = geponex_config()
    bad["layers"][0]["type"] = "lstm"
    with pytest.raises(ValueError):
        GeponexConfig(bad)
    with pytest.raises(ValueError):
        GeponexConfig(geponex_config(width=50, groups=3))
    ahead = geponex_config()
    ahead["layers"].insert(0, dict(ahead["layers"][1], weights_of=2))         # a layer may run the weights of a later one
    ahead["layers"][4]["weights_of"] = 2
    assert [l.weights_of for l in GeponexConfig(ahead).layers] == [2, 1, 2, 3, 2]
    chain = geponex_config()
    chain["layers"].append(dict(chain["layers"][3], weights_of=3))          # a layer without tensors cannot lend them
    with pytest.raises(ValueError):
        GeponexConfig(chain)


@pytest.mark.parametrize("dims,base,scaling", [(24, 300000.0, {"factor": 6.0, "original": 2048, "fast": 24.0, "slow": 2.0}),
                                               (8, 10000.0, {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}),
                                               (64, 10000.0, {"factor": 40.0, "original": 4096, "fast": 32.0, "slow": 1.0}),
                                               (16, 1000000.0, None)])
def test_rotary_frequencies_with_and_without_the_blend(dims, base, scaling):
    from vllm_hymeta.models.configuration_geponex import RotarySpec
    freqs, mag = RotarySpec(dims, base, scaling).frequencies()
    ref, ref_mag = rotary_frequencies_ref(dims, base, scaling)
    assert len(freqs) == dims // 2 and torch.allclose(torch.tensor(freqs, dtype=torch.float64), ref, rtol=1e-14, atol=0)
    assert mag == pytest.approx(ref_mag, rel=1e-15)
    if scaling:
        plain = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
        assert freqs[0] == pytest.approx(plain[0]) or freqs[0] < plain[0]           # fast pairs keep their frequency ...
        assert freqs[-1] == pytest.approx(plain[-1] / scaling["factor"]) or freqs[-1] > plain[-1] / scaling["factor"]
        assert any(abs(f - p) > 1e-12 * p for f, p in zip(freqs, plain))            # ... some pair is slowed down
        assert mag == pytest.approx(0.1 * math.log(scaling["factor"]) + 1.0)
    else:
        assert mag == 1.0


def test_registry_picks_the_class_and_names_its_kernel_sources(tmp_path):
    import os
    from vllm_hymeta import registry
    from vllm_hymeta.models.modeling_geponex import GeponexForCausalLM
    (tmp_path / "config.json").write_text(json.dumps(geponex_config()))
    cls, cfg = registry.resolve(str(tmp_path))
    assert cls is GeponexForCausalLM and cfg.hidden_size == 48 and "Geponex" in registry.known_architectures()
    assert registry.kernel_sources(str(tmp_path)) == GeponexForCausalLM.kernel_sources
    csrc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "vllm-hymeta_amd", "csrc")
    for name in GeponexForCausalLM.kernel_sources:
        assert os.path.exists(os.path.join(csrc, name + ".hip")), name


def test_oracle_is_causal_and_its_mechanisms_show_in_the_logits():
    """The plain statement itself: a later token changes nothing before it; the shift, the sink, the gate, the norms'
    groups, the stream's factor, YaRN, the experts' clamp and the layers that share weights each move the logits (a fault
    that drops one of them cannot hide behind the random weights)."""
    cfg = geponex_config()
    w = geponex_random_weights(cfg, 2)
    toks = [3, 14, 15, 9, 65, 35, 8, 79, 32, 38, 46, 26]
    full = geponex_ref(cfg, w, toks)
    assert torch.allclose(geponex_ref(cfg, w, toks[:7]), full[:7], atol=1e-12)
    for name in ("l0.shift", "l1.shift", "l0.mix.sink", "l0.mlp.up.b", "l1.mlp.router"):
        w2 = dict(w)
        w2[name] = torch.zeros_like(w[name]) if name != "l0.mix.sink" else w[name] + 4.0
        assert (geponex_ref(cfg, w2, toks) - full).abs().max() > 1e-3, name

    def changed(**kw):
        c = json.loads(json.dumps(cfg))
        for path, v in kw.items():
            node = c
            keys = path.split("__")
            for k in keys[:-1]:
                node = node[int(k)] if k.isdigit() else node[k]
            node[keys[-1]] = v
        return (geponex_ref(c, w, toks) - full).abs().max()

    assert changed(postln_alpha=1.0) > 1e-3 and changed(norm__groups=1) > 1e-3
    assert changed(layers__2__mixer__rot__scaling=None) > 1e-3
    assert changed(layers__1__mlp__expert__limit=9.0) > 1e-3 and changed(layers__1__mlp__router__scale=1.0) > 1e-3
    assert changed(layers__1__mixer__decay=[0.3, 0.3, 0.3]) > 1e-3
    drop = json.loads(json.dumps(cfg))
    drop["layers"] = drop["layers"][:3]                                  # the layer that runs layer 1's weights again
    assert (geponex_ref(drop, w, toks) - full).abs().max() > 1e-3
    x = torch.tensor([[3.0, 4.0, 0.0, 0.5]], dtype=torch.float64)
    assert torch.allclose(group_norm_ref(x, torch.ones(4, dtype=torch.float64), 2, 0.0),
                          torch.tensor([[3 / 12.5 ** 0.5, 4 / 12.5 ** 0.5, 0.0, 2 ** 0.5]], dtype=torch.float64))
    z = torch.tensor([-1.0, 0.0, 2.0], dtype=torch.float64)
    p = q = torch.tensor(0.0, dtype=torch.float64)
    ln2 = math.log(2.0)
    assert torch.allclose(xielu_ref(z, p, q), torch.tensor([(0.5 + ln2) * (math.exp(-1) - 1 + 1) - 0.5, 0.0, ln2 * 4 + 1.0], dtype=torch.float64))
