"""The package's own engine around the 7B model class: the scheduler's batches (two whole prompts, then single tokens,
a third request in the slot and pages the first one gave back) through ``LLMEngine.execute`` against the CPU
restatement of the model on each whole sequence."""
import pytest
import torch

from _util import assert_bf16_close, gen
from test_gpu_model_7b import _checkpoint

pytestmark = pytest.mark.gpu


def test_engine_serves_the_7b_model_class():
    from oracle.model import glaswa_model_ref
    from vllm_hymeta.engine import LLMEngine
    from vllm_hymeta.model_for_7B.configuration_gla_swa import GLAswaConfig
    from vllm_hymeta.model_for_7B.modeling_gla_swa import GLAswaForCausalLM

    dev = torch.device("cuda")
    g_ = gen(23)
    cfg = GLAswaConfig(vocab_size=512, hidden_size=512, num_hidden_layers=4, num_attention_heads=4, num_key_value_heads=2,
                       intermediate_size=1024, sliding_window=48, max_position_embeddings=1024)
    ckpt = _checkpoint(g_, cfg)
    model = GLAswaForCausalLM(cfg, max_num_seqs=2, device=dev)
    model.load_weights(ckpt.items())
    eng = LLMEngine(model, num_blocks=12, block_size=16, max_num_seqs=2, device=dev)
    seqs = {k: torch.randint(0, cfg.vocab_size, (n,), generator=g_).tolist() for k, n in (("a", 61), ("b", 34), ("c", 50))}
    refs = {k: glaswa_model_ref(torch.tensor(t), ckpt, cfg)[1] for k, t in seqs.items()}

    def check(out, rows, what):
        assert out.dtype == torch.float32
        assert_bf16_close(out.cpu(), torch.stack(rows), what, rel=2e-2, frac=2.0 ** -4)

    # two whole prompts (all but their last 3 tokens) in one batch, then three steps of single tokens
    out = eng.run_batch([("a", seqs["a"][:58], [57]), ("b", seqs["b"][:31], [30, 0])])
    check(out, [refs["a"][57], refs["b"][30], refs["b"][0]], "engine, 7B, prompts")
    for i in range(3):
        out = eng.run_batch([("b", seqs["b"][31 + i:32 + i], [0]), ("a", seqs["a"][58 + i:59 + i], [0])])
        check(out, [refs["b"][31 + i], refs["a"][58 + i]], f"engine, 7B, decode step {i}")
    eng.finish_request("a")
    assert eng.pool.num_free == 12 - 3
    # a new request takes the slot and the pages that came back, beside a request that goes on
    out = eng.run_batch([("c", seqs["c"][:49], [48])])
    check(out, [refs["c"][48]], "engine, 7B, prompt in a used slot")
    out = eng.run_batch([("c", seqs["c"][49:], [0])])
    check(out, [refs["c"][49]], "engine, 7B, decode in a used slot")
