"""Host side of the Sonuzen family and of the package's own engine: configuration, layer order, registry, page pool,
scheduler, and the oracle's own consistency (no GPU)."""
import json

import pytest
import torch

from oracle.sonuzen import causal_conv_add_ref, layer_runs_ref, sink_attention_ref, sonuzen_config, sonuzen_random_weights, sonuzen_ref


def test_config_reads_every_size_and_orders_the_looped_layers():
    from vllm_hymeta.models.configuration_sonuzen import SonuzenConfig
    raw = sonuzen_config(layers=("mingru", "attention", "attention", "mingru"), loop=(1, 3, 3), heads=6, kv_heads=3, dim=8, vdim=40,
                         mingru_width=80, taps=4, top=1, experts=7, ff=24, no_mlp=(3,))
    cfg = SonuzenConfig(raw)
    assert cfg.layer_runs() == [(0, 0), (1, 0), (2, 0), (1, 1), (2, 1), (1, 2), (2, 2), (3, 0)]
    assert [i for i, _ in cfg.layer_runs()] == [i for i, _ in layer_runs_ref(raw)]
    a = cfg.layers[1].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim) == (6, 3, 8, 40) and cfg.layers[0].mixer.width == 80
    assert cfg.layers[3].mlp is None and cfg.layers[0].mlp.top == 1 and cfg.layers[0].mlp.experts == 7 and cfg.conv_taps == 4
    plain = SonuzenConfig(sonuzen_config(layers=("attention",), taps=0))
    assert not plain.has_loop and not plain.has_conv and plain.layer_runs() == [(0, 0)]
    with pytest.raises(ValueError):
        SonuzenConfig(sonuzen_config(layers=("attention",), heads=5, kv_heads=2))
    bad = sonuzen_config(layers=("attention",))
    bad["layers"][0]["type"] = "lstm"
    with pytest.raises(ValueError):
        SonuzenConfig(bad)


def test_registry_picks_the_class_by_config_json(tmp_path):
    from vllm_hymeta import registry
    (tmp_path / "config.json").write_text(json.dumps(sonuzen_config()))
    cls, cfg = registry.resolve(str(tmp_path))
    assert cls.__name__ == "SonuzenForCausalLM" and cfg.hidden_size == 64
    (tmp_path / "config.json").write_text(json.dumps({"architectures": ["NoSuchModel"]}))
    with pytest.raises(ValueError):
        registry.resolve(str(tmp_path))
    assert "GLAswaForCausalLM" in registry.known_architectures()


def test_page_pool_reuses_the_pages_freed_last():
    from vllm_hymeta.engine import BlockPool
    pool = BlockPool(6, 16)
    a, b = [], []
    pool.grow(a, 17)
    pool.grow(b, 16)
    assert a == [0, 1] and b == [2] and pool.num_free == 3
    pool.grow(a, 32)
    assert a == [0, 1]
    pool.grow(a, 33)
    assert a == [0, 1, 3]
    pool.release(a)
    assert a == [] and pool.num_free == 5
    c = []
    pool.grow(c, 40)
    assert c == [0, 1, 3]                        # the pages that came back are handed out first
    with pytest.raises(RuntimeError):
        pool.grow(b, 16 * 5)


def test_scheduler_batches_decodes_before_portions_and_respects_slots_and_budget():
    from vllm_hymeta.engine import BlockPool, Request, Scheduler
    pool = BlockPool(16, 16)
    sch = Scheduler(pool, max_num_seqs=2, max_num_batched_tokens=20)
    rs = [Request(f"r{k}", list(range(n)), n) for k, n in enumerate([30, 4, 9])]
    for r in rs:
        sch.add(r)
    batch = sch.schedule()
    assert [(r.request_id, n) for r, n in batch] == [("r0", 20)]            # the budget cuts the prompt
    rs[0].num_computed = 20
    batch = sch.schedule()
    assert [(r.request_id, n) for r, n in batch] == [("r0", 10), ("r1", 4)]  # the rest of it, then the next request
    rs[0].num_computed, rs[1].num_computed = 30, 4
    rs[0].token_ids.append(1), rs[1].token_ids.append(1)
    batch = sch.schedule()
    assert sorted((r.request_id, n) for r, n in batch) == [("r0", 1), ("r1", 1)]      # two slots: r2 waits
    sch.retire(rs[1])
    rs[0].num_computed = 31
    rs[0].token_ids.append(2)
    batch = sch.schedule()
    assert [(r.request_id, n) for r, n in batch] == [("r0", 1), ("r2", 9)]   # the single token first, then the new prompt


def test_oracle_is_causal_and_its_mechanisms_show_in_the_logits():
    """The plain statement itself: a later token changes nothing before it; the sink, the distance bias, the convolution
    and the loop's vectors each move the logits (a fault that drops one of them cannot hide behind the random weights)."""
    cfg = sonuzen_config(layers=("attention", "mingru"), loop=(0, 2, 2))
    w = sonuzen_random_weights(cfg, 2)
    toks = [3, 14, 15, 92, 65, 35, 89, 79, 32, 38]
    full = sonuzen_ref(cfg, w, toks)
    assert torch.allclose(sonuzen_ref(cfg, w, toks[:6]), full[:6], atol=1e-12)
    for name in ("l0.mix.r1", "l0.canon1", "l1.canon2", "loop.step", "l0.mix.k.norm", "l1.mix.z.b"):
        w2 = dict(w)
        w2[name] = torch.zeros_like(w[name])
        assert (sonuzen_ref(cfg, w2, toks) - full).abs().max() > 1e-3, name
    q, k, v = torch.randn(5, 2, 4).double(), torch.randn(5, 1, 4).double(), torch.randn(5, 1, 3).double()
    with_sink, without = sink_attention_ref(q, k, v, 0.5, None, None, True), sink_attention_ref(q, k, v, 0.5, None, None, False)
    assert torch.allclose(without[0, 0], v[0, 0]) and not torch.allclose(with_sink[0, 0], v[0, 0])
    h = torch.arange(12, dtype=torch.float64).view(4, 3)
    cw = torch.tensor([[1.0, 0.0], [0.0, 1.0], [2.0, 3.0]], dtype=torch.float64)
    out = causal_conv_add_ref(h, cw)
    assert out[0].tolist() == [0.0, 2.0, 8.0] and out[2].tolist() == [6 + 3, 7 + 7, 8 + 2 * 5 + 3 * 8]


def test_registry_names_the_kernel_sources_the_model_class_names():
    """The table a first run reads before torch is imported says what the class says, and every name is a source file."""
    import os
    from vllm_hymeta import registry
    from vllm_hymeta.models.modeling_sonuzen import SonuzenForCausalLM
    assert registry._KERNEL_SOURCES["SonuzenForCausalLM"] == SonuzenForCausalLM.kernel_sources
    csrc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "vllm-hymeta_amd", "csrc")
    for name in SonuzenForCausalLM.kernel_sources:
        assert os.path.exists(os.path.join(csrc, name + ".hip")), name
