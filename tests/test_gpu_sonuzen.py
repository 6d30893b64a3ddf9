"""The Sonuzen building blocks and the model under the engine, against the plain CPU statement in ``oracle/sonuzen.py``.

Mechanisms alone first (norm + convolution with its carried state, output norm + residual, minGRU, biased sink
attention over pages, table-routed experts), then whole models of several shapes: a prompt in one step against the
oracle, and the same tokens cut into steps in every way the engine allows (token by token, portions down to two
tokens, unequal requests in one batch, pages and state slots used again) against the one-step result.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle.sonuzen import (causal_conv_add_ref, mingru_ref, norm_one_plus_ref, rms_unit, sink_attention_ref,  # noqa: E402
                            sonuzen_config, sonuzen_random_weights, sonuzen_ref, table_moe_ref)

DEV = "cuda"
TOL = {torch.float32: 2e-5, torch.bfloat16: 2e-2}


def rel_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    got, ref = got.double().cpu(), ref.double().cpu()
    return float((got - ref).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt().clamp_min(1e-30))


def i32(v):
    return torch.tensor(v, dtype=torch.int32, device=DEV)


def bf16_values(*shape, std=1.0, gen=None):
    return (torch.randn(*shape, generator=gen) * std).to(torch.bfloat16).double()


# --------------------------------------------------------------------------- norm + convolution
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps,width", [(3, 96), (1, 64), (2, 40), (5, 272)])
def test_norm_conv_in_portions_carries_its_state(dtype, taps, width):
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(taps * 100 + width)
    lens = [11, 1, 7]
    xs = [torch.randn(n, width, generator=g, dtype=torch.float64) * 2 for n in lens]
    w, cw, eps = torch.randn(width, generator=g).double() * 0.2, torch.randn(width, taps, generator=g).double() * 0.5, 1e-5
    refs = [causal_conv_add_ref(norm_one_plus_ref(x, w, eps), cw) for x in xs]
    state = torch.full((4, max(taps - 1, 1), width), 7.0, dtype=dtype, device=DEV)[:, :taps - 1].contiguous() if taps > 1 else None
    slots = [2, 0, 3]
    # portions: sequence 0 in 2 + 1 + 3 + 5, sequence 1 whole, sequence 2 in 4 + 1 + 2, interleaved in shared steps
    plan = [[(0, 2), (2, 4)], [(0, 1), (1, 1)], [(2, 1), (0, 3)], [(0, 5), (2, 2)]]
    done = [0, 0, 0]
    outs = [[], [], []]
    for step in plan:
        rows = torch.cat([xs[s][done[s]:done[s] + n] for s, n in step]).float().to(DEV)
        qsl = [0]
        for s, n in step:
            qsl.append(qsl[-1] + n)
        out = hip_ops.norm_conv(rows, w.float().to(DEV), eps, dtype, 1.0, cw.float().to(DEV).contiguous(), state, i32(qsl),
                                i32([done[s] for s, _ in step]), i32([slots[s] for s, _ in step]))
        for k, (s, n) in enumerate(step):
            outs[s].append(out[qsl[k]:qsl[k + 1]])
            done[s] += n
    assert done == lens
    for s in range(3):
        assert rel_err(torch.cat(outs[s]), refs[s]) < TOL[dtype], (s, taps)
    if taps > 1:
        # a new sequence in a used slot starts from zeros, whatever the slot holds
        out = hip_ops.norm_conv(xs[2].float().to(DEV), w.float().to(DEV), eps, dtype, 1.0, cw.float().to(DEV).contiguous(), state,
                                i32([0, lens[2]]), i32([0]), i32([2]))
        assert rel_err(out, refs[2]) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps,width", [(3, 96), (4, 272), (2, 64), (5, 40), (3, 4200)])
def test_norm_conv_of_long_steps(dtype, taps, width):
    """Steps of a thousand rows and more run in strips of rows whose inputs are read once; strips that hold a portion's
    first rows or a boundary between two sequences do not.  Two sequences in one step, then their next portions."""
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(taps + width)
    lens = [1301, 702]
    xs = [torch.randn(n, width, generator=g, dtype=torch.float64) for n in lens]
    w, cw, eps = torch.randn(width, generator=g).double() * 0.2, torch.randn(width, taps, generator=g).double() * 0.5, 1e-5
    refs = [causal_conv_add_ref(norm_one_plus_ref(x, w, eps), cw) for x in xs]
    state = torch.zeros(2, taps - 1, width, dtype=dtype, device=DEV)
    first = [1027, 601]                                   # the second sequence starts inside a strip
    step1 = torch.cat([xs[0][:first[0]], xs[1][:first[1]]]).float().to(DEV)
    args = (w.float().to(DEV), eps, dtype, 1.0, cw.float().to(DEV).contiguous(), state)
    out1 = hip_ops.norm_conv(step1, *args, i32([0, first[0], first[0] + first[1]]), i32([0, 0]), i32([1, 0]))
    step2 = torch.cat([xs[1][first[1]:], xs[0][first[0]:], ]).float().to(DEV)
    n1, n0 = lens[1] - first[1], lens[0] - first[0]
    out2 = hip_ops.norm_conv(step2, *args, i32([0, n1, n1 + n0]), i32([first[1], first[0]]), i32([0, 1]))
    assert rel_err(torch.cat([out1[:first[0]], out2[n1:]]), refs[0]) < TOL[dtype]
    assert rel_err(torch.cat([out1[first[0]:], out2[:n1]]), refs[1]) < TOL[dtype]
    # the strip form and the row form give the same values: the same rows in a step too short for strips
    short = hip_ops.norm_conv(step1[100:900].contiguous(), *args[:5], None, i32([0, 800]), i32([0]), None)
    long_ = hip_ops.norm_conv(step1[100:1300].contiguous(), *args[:5], None, i32([0, 1200]), i32([0]), None)
    assert rel_err(long_[8:800], short[8:800]) < (1e-6 if dtype == torch.float32 else 4e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_plain_norm_and_output_norm_with_residual(dtype):
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(3)
    T, W, eps = 9, 200, 1e-6
    x, w = torch.randn(T, W, generator=g).double(), torch.randn(W, generator=g).double() * 0.3
    out = hip_ops.norm_conv(x.float().to(DEV), w.float().to(DEV), eps, dtype, 1.0)
    assert rel_err(out, norm_one_plus_ref(x, w, eps)) < TOL[dtype]
    out = hip_ops.norm_conv(x.float().to(DEV), w.float().to(DEV), eps, dtype, 0.0)
    assert rel_err(out, rms_unit(x, eps) * w) < TOL[dtype]
    y = bf16_values(T, W, std=3.0, gen=g)
    add = torch.randn(W, generator=g).double()
    xd = x.float().to(DEV)
    hip_ops.norm_residual_(xd, y.to(dtype).to(DEV), w.float().to(DEV), eps, 0.25, 1.0, add.float().to(DEV))
    assert xd.dtype == torch.float32
    assert rel_err(xd, x + 0.25 * norm_one_plus_ref(y, w, eps) + add) < 2e-6      # the stream is fp32 in both types


# --------------------------------------------------------------------------- minGRU
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [64, 80])
def test_mingru_prefill_equals_token_by_token_and_portions(dtype, width):
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(width)
    T = 150
    zug = bf16_values(T, 3 * width, std=1.5, gen=g)
    # the recurrence alone: the oracle's mixer with projections that pick the three column blocks, identity on the way out
    eye, zero = torch.eye(width, dtype=torch.float64), torch.zeros(width, width, dtype=torch.float64)
    pick = [torch.cat([eye if j == n else zero for j in range(3)], 1) for n in range(3)]
    ref = mingru_ref(zug, pick[0], torch.zeros(width).double(), pick[1], torch.zeros(width).double(), pick[2], eye)
    S = torch.zeros(width, dtype=torch.float64)
    for t in range(T):
        z, u = torch.sigmoid(zug[t, :width]), zug[t, width:2 * width]
        S = (1 - z) * S + z * torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    zd = zug.to(dtype).to(DEV)
    for portions in ([T], [1] * T, [2, 3, 64, 1, 9, 65, 6], [8, 9, 133]):
        assert sum(portions) == T
        state = torch.full((3, width), 5.0, dtype=torch.float32, device=DEV)       # stale values of an earlier owner
        outs, at = [], 0
        for n in portions:
            outs.append(hip_ops.mingru(zd[at:at + n], state, i32([0, n]), i32([at]), i32([1]), n))
            at += n
        assert rel_err(torch.cat(outs), ref) < TOL[dtype], portions
        assert rel_err(state[1], S) < 1e-5                                        # the carried state is fp32 in both types
        assert float(state[0].min()) == 5.0 and float(state[2].max()) == 5.0      # other slots untouched


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mingru_long_portions_run_in_segments(dtype):
    """Portions of thousands of rows are scanned in segments side by side and chained; a short sequence shares the step, and
    the long one goes on from the state a first portion left."""
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(21)
    width, T, first = 72, 2400, 37
    zug, short = bf16_values(T, 3 * width, std=1.5, gen=g), bf16_values(5, 3 * width, gen=g)
    eye, zero = torch.eye(width, dtype=torch.float64), torch.zeros(width, width, dtype=torch.float64)
    pick = [torch.cat([eye if j == n else zero for j in range(3)], 1) for n in range(3)]
    none = torch.zeros(width).double()
    ref, ref_short = mingru_ref(zug, pick[0], none, pick[1], none, pick[2], eye), mingru_ref(short, pick[0], none, pick[1], none, pick[2], eye)
    state = torch.full((3, width), 9.0, dtype=torch.float32, device=DEV)
    zd = zug.to(dtype).to(DEV)
    a = hip_ops.mingru(zd[:first], state, i32([0, first]), i32([0]), i32([2]), first)
    rows = torch.cat([short.to(dtype).to(DEV), zd[first:]])
    b = hip_ops.mingru(rows, state, i32([0, 5, 5 + T - first]), i32([0, first]), i32([0, 2]), T - first)
    assert rel_err(torch.cat([a, b[5:]]), ref) < TOL[dtype]
    assert rel_err(b[:5], ref_short) < TOL[dtype]
    whole = hip_ops.mingru(zd, state, i32([0, T]), i32([0]), i32([1]), T)
    assert rel_err(whole, ref) < TOL[dtype]
    assert rel_err(state[1], state[2]) < 1e-5        # the same final state whichever way the rows were cut


def test_mingru_batches_unequal_sequences():
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(9)
    width, lens = 72, [1, 40, 3, 17]
    zs = [bf16_values(n, 3 * width, gen=g) for n in lens]
    state = torch.zeros(6, width, dtype=torch.float32, device=DEV)
    alone = [hip_ops.mingru(z.float().to(DEV), state, i32([0, n]), i32([0]), i32([5]), n) for z, n in zip(zs, lens)]
    qsl = [0]
    for n in lens:
        qsl.append(qsl[-1] + n)
    both = hip_ops.mingru(torch.cat(zs).float().to(DEV), state, i32(qsl), i32([0] * 4), i32([3, 0, 4, 1]), max(lens))
    for k in range(4):
        assert rel_err(both[qsl[k]:qsl[k + 1]], alone[k]) < 1e-6       # (short sequences run the plain update when alone)


# --------------------------------------------------------------------------- attention
def _paged_attention(q, k, v, dtype, block_size, portions, scale, r1, r2, qw, kw, eps, sink=True, shuffle_seed=0):
    """Runs one sequence through qk_norm_cache_ + sink_attention in ``portions`` over scattered pages."""
    from vllm_hymeta import hip_ops
    T, H, D = q.shape
    G, Dv = k.shape[1], v.shape[2]
    nblk = (T + block_size - 1) // block_size + 3
    perm = torch.randperm(nblk, generator=torch.Generator().manual_seed(shuffle_seed)).tolist()
    table = perm[:(T + block_size - 1) // block_size]
    kv = torch.full((nblk, block_size, G, D + Dv), float("nan"), dtype=dtype, device=DEV)
    qkv = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], 1).to(dtype).to(DEV)
    outs, at = [], 0
    f = lambda t: None if t is None else t.float().to(DEV)
    for n in portions:
        rows = qkv[at:at + n].clone()
        slots = torch.tensor([table[p // block_size] * block_size + p % block_size for p in range(at, at + n)], dtype=torch.int64, device=DEV)
        hip_ops.qk_norm_cache_(rows, H, G, D, Dv, f(qw), f(kw), eps, kv, slots)
        outs.append(hip_ops.sink_attention(rows[:, :H * D].view(n, H, D), kv, i32([table]), i32([0, n]), i32([at + n]), G, D, Dv, scale,
                                           n, at + n, f(r1), f(r2), sink))
        at += n
    return torch.cat(outs)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,Dv", [(4, 2, 16, 24), (3, 3, 8, 8), (6, 1, 40, 16), (2, 1, 128, 128), (4, 2, 64, 64), (8, 2, 64, 128),
                                     (5, 1, 128, 64)])
def test_sink_attention_over_pages_in_portions(dtype, H, G, D, Dv):
    g = torch.Generator().manual_seed(H * 31 + D)
    T, eps, scale = 150, 1e-5, 0.3
    q, k, v = bf16_values(T, H, D, gen=g), bf16_values(T, G, D, gen=g), bf16_values(T, G, Dv, gen=g)
    qw, kw = 1 + bf16_values(D, std=0.2, gen=g), 1 + bf16_values(D, std=0.2, gen=g)
    r1, r2 = torch.rand(H, generator=g).double() + 0.2, torch.rand(H, generator=g).double() * 0.5 + 0.05
    qn, kn = rms_unit(q, eps) * qw, rms_unit(k, eps) * kw
    if dtype == torch.bfloat16:      # what the cache and the query rows hold
        qn, kn = qn.to(dtype).double(), kn.to(dtype).double()
    ref = sink_attention_ref(qn, kn, v, scale, r1, r2)
    for portions in ([T], [115] + [1] * 35, [2, 14, 16, 1, 31, 2, 9, 64, 11]):       # page size 16: portions end on, before and after borders
        for page in (16, 64):
            out = _paged_attention(q, k, v, dtype, page, portions, scale, r1, r2, qw, kw, eps, shuffle_seed=len(portions))
            assert rel_err(out, ref) < (3e-5 if dtype == torch.float32 else 1e-2), (portions, page)
    no_sink = sink_attention_ref(qn, kn, v, scale, r1, r2, sink=False)
    assert rel_err(ref, no_sink) > 0.05           # the inputs do tell a softmax with a sink from one without
    out = _paged_attention(q, k, v, dtype, 16, [T], scale, r1, r2, qw, kw, eps, sink=False)
    assert rel_err(out, no_sink) < (3e-5 if dtype == torch.float32 else 1e-2)
    out = _paged_attention(q, k, v, dtype, 16, [T], scale, None, None, qw, kw, eps)
    assert rel_err(out, sink_attention_ref(qn, kn, v, scale, None, None)) < (3e-5 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D", [16, 64])
def test_a_key_far_back_decides_the_output(dtype, D):
    """Hundreds of keys, one of which (far back, on a page border) matches the last queries many times better than the
    rest even after the distance bias: the output is that key's value row, in a prompt's portion and for a decoded token."""
    g = torch.Generator().manual_seed(5)
    T, H, G, Dv, bs = 700, 2, 1, D, 64
    q, k, v = bf16_values(T, H, D, std=0.3, gen=g), bf16_values(T, G, D, std=0.3, gen=g), bf16_values(T, G, Dv, gen=g)
    far = 64                                                    # first row of the second page
    k[far] = 0
    k[far, 0, 3] = 4.0
    q[-3:] = 0
    q[-3:, :, 3] = 4.0
    r1, r2 = torch.tensor([1.0, 0.5]).double(), torch.tensor([0.1, 0.3]).double()
    scale = 2.0
    # the oracle on the last three rows only
    rows = []
    for i in range(T - 3, T):
        for h in range(H):
            s = torch.stack([(q[i, h] * k[j, 0]).sum() * scale - r1[h] * torch.log1p(r2[h] * (i - j)) for j in range(i + 1)])
            e = torch.exp(s)
            rows.append(((e / (1 + e.sum()))[:, None] * v[:i + 1, 0]).sum(0))
    ref = torch.stack(rows).view(3, H, Dv)
    assert rel_err(ref[:, 0], v[far, 0].expand(3, Dv)) < 0.05       # the far key does decide
    for portions in ([T], [T - 2, 1, 1], [far, 1, T - far - 2, 1]):
        out = _paged_attention(q, k, v, dtype, bs, portions, scale, r1, r2, None, None, 1e-5)
        assert rel_err(out[-3:], ref) < (3e-5 if dtype == torch.float32 else 1e-2), portions


def test_sink_attention_batches_unequal_sequences_like_each_alone():
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(11)
    H, G, D, Dv, bs = 4, 2, 16, 8, 16
    lens, ctx = [33, 1, 5], [0, 48, 17]                      # a whole prompt, a decoded token, a portion
    nblk = 16
    kv = torch.randn(nblk, bs, G, D + Dv, generator=g).to(DEV)
    tables = [[3, 7, 9, 0], [1, 2, 4, 8], [5, 6, 10, 11]]
    qs = [torch.randn(n, H, D, generator=g).to(DEV) for n in lens]
    r1, r2 = torch.rand(H, generator=g).to(DEV), torch.rand(H, generator=g).to(DEV)
    alone = [hip_ops.sink_attention(qs[s], kv, i32([tables[s]]), i32([0, lens[s]]), i32([ctx[s] + lens[s]]), G, D, Dv, 0.25, lens[s],
                                    ctx[s] + lens[s], r1, r2) for s in range(3)]
    both = hip_ops.sink_attention(torch.cat(qs), kv, i32(tables), i32([0, 33, 34, 39]), i32([c + n for c, n in zip(ctx, lens)]),
                                  G, D, Dv, 0.25, 33, 49, r1, r2)
    assert torch.equal(both, torch.cat(alone))


# --------------------------------------------------------------------------- experts by table
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,I,E,top", [(64, 32, 4, 2), (128, 64, 8, 1), (48, 20, 5, 3), (64, 32, 3, 3), (72, 8, 2, 2)])
def test_table_routed_experts(dtype, H, I, E, top):
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(H + I + E + top)
    T, V = 37, 50
    x = bf16_values(T, H, gen=g)
    gates, ups = [bf16_values(I, H, std=H ** -0.5, gen=g) for _ in range(E)], [bf16_values(I, H, std=H ** -0.5, gen=g) for _ in range(E)]
    downs = [bf16_values(H, I, std=I ** -0.5, gen=g) for _ in range(E)]
    table = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(V)]).to(torch.int32)
    tokens = torch.randint(0, V, (T,), generator=g)
    ref = table_moe_ref(x, tokens.tolist(), table, gates, ups, downs)
    w13 = torch.stack([torch.cat([a, b]) for a, b in zip(gates, ups)]).to(dtype).to(DEV)
    w2 = torch.stack(downs).to(dtype).to(DEV)
    out = hip_ops.moe_table_forward(x.to(dtype).to(DEV), tokens.to(DEV), table.to(DEV), w13, w2)
    assert out.dtype == dtype
    assert rel_err(out, ref) < (2e-5 if dtype == torch.float32 else 2e-2)
    # a token's row does not depend on what else is in the batch
    one = hip_ops.moe_table_forward(x[5:6].to(dtype).to(DEV), tokens[5:6].to(DEV), table.to(DEV), w13, w2)
    assert rel_err(one, out[5:6]) < (1e-6 if dtype == torch.float32 else 1e-2)


# --------------------------------------------------------------------------- whole models under the engine
def build_engine(cfg, weights, dtype, max_tokens=512, block_size=16, max_num_seqs=4, max_num_batched_tokens=1 << 30):
    from vllm_hymeta.engine import LLMEngine
    from vllm_hymeta.models.configuration_sonuzen import SonuzenConfig
    from vllm_hymeta.models.modeling_sonuzen import SonuzenForCausalLM
    model = SonuzenForCausalLM(SonuzenConfig(cfg), max_num_seqs=max_num_seqs, dtype=dtype, device=DEV)
    model.load_weights(weights.items())
    return LLMEngine(model, num_blocks=max_tokens // block_size, block_size=block_size, max_num_seqs=max_num_seqs,
                     max_num_batched_tokens=max_num_batched_tokens, device=DEV)


MODELS = {
    "hybrid_loop": dict(layers=("mingru", "attention", "attention", "mingru", "attention"), loop=(1, 4, 2)),
    "loop_from_first_layer_three_times": dict(layers=("mingru", "attention"), loop=(0, 2, 3), taps=2, top=1, experts=3),
    "no_loop_wide_gru_no_mlp_on_one": dict(layers=("attention", "mingru", "mingru"), mingru_width=96, no_mlp=(1,), taps=4,
                                           heads=6, kv_heads=3, dim=8, vdim=8, top=3, experts=5, ff=24, width=48, residual_mult=1.0,
                                           logit_scale=1.0),
    "one_tap_one_head": dict(layers=("attention",), heads=1, kv_heads=1, dim=32, vdim=16, taps=1, loop=(0, 1, 2), experts=2, top=2,
                             ff=40, width=72, scale=0.4),
    "matrix_core_head_sizes": dict(layers=("attention", "mingru", "attention"), loop=(1, 3, 2), width=128, heads=4, kv_heads=2, dim=64,
                                   vdim=128, ff=64, experts=4, top=2),
    "no_convolution": dict(layers=("mingru", "attention"), taps=0, width=128, ff=64, heads=8, kv_heads=2, dim=16, vdim=32),
}


def _tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


@pytest.mark.parametrize("name", sorted(MODELS))
def test_model_whole_prompt_against_the_oracle_fp32(name):
    cfg = sonuzen_config(**MODELS[name])
    weights = sonuzen_random_weights(cfg, seed=len(name))
    toks = _tokens(45, cfg["vocab"], 1)
    ref = sonuzen_ref(cfg, weights, toks)
    eng = build_engine(cfg, weights, torch.float32)
    got = eng.run_batch([("a", toks, list(range(len(toks))))])
    assert got.shape == ref.shape and got.dtype == torch.float32
    assert rel_err(got, ref) < 2e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", sorted(MODELS))
def test_model_schedules_agree_with_the_whole_prompt(name, dtype):
    """Decoding token by token, portions of several sizes (down to two tokens, and one), and a mixed batch of four
    requests whose pages and state slots come from requests that ended: every position's logits equal the one-step
    logits up to rounding, and (fp32) the oracle's."""
    cfg = sonuzen_config(**MODELS[name])
    weights = sonuzen_random_weights(cfg, seed=len(name))
    V = cfg["vocab"]
    seqs = {k: _tokens(n, V, 10 + k) for k, n in enumerate([70, 33, 1, 50, 19, 64])}
    refs = {k: sonuzen_ref(cfg, weights, t) for k, t in seqs.items()}
    tol_ref = 3e-5 if dtype == torch.float32 else 4e-2
    tol_self = 3e-5 if dtype == torch.float32 else 3e-2
    # pool of 12 pages of 16 tokens (64 for the model whose attention runs on the matrix cores, where a page holds a whole
    # tile of keys): never room for everything at once
    page = 64 if name == "matrix_core_head_sizes" else 16
    eng = build_engine(cfg, weights, dtype, max_tokens=12 * page, block_size=page, max_num_seqs=4)
    whole = {}
    for k, t in seqs.items():
        whole[k] = eng.run_batch([(f"w{k}", t, list(range(len(t))))])
        eng.finish_request(f"w{k}")
        assert rel_err(whole[k], refs[k]) < tol_ref, k
    assert eng.pool.num_free == 12

    def replay(plan):
        """plan: steps, each a list of (sequence, tokens in this step); returns per-sequence logits of every position."""
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
    got = replay([[(0, 21)]] + [[(0, 1)]] * 49)
    assert rel_err(got[0], whole[0]) < tol_self and rel_err(got[0], refs[0]) < tol_ref
    # portions: 2, 1, 3, ... across page borders (16, 32, 48) and the convolution's reach
    got = replay([[(0, 2)], [(0, 1)], [(0, 3)], [(0, 10)], [(0, 2)], [(0, 14)], [(0, 17)], [(0, 2)], [(0, 19)]])
    assert rel_err(got[0], whole[0]) < tol_self
    # mixed: up to four live requests, portions beside single tokens, requests that end and free pages and slots for new ones
    plan = [[(0, 30), (1, 2)], [(0, 1), (1, 31), (2, 1)], [(0, 1), (3, 16), (4, 2)], [(0, 38), (3, 1), (4, 17)],
            [(3, 33), (5, 3)], [(5, 2)], [(5, 59)]]
    got = replay(plan)
    for k in seqs:
        assert rel_err(got[k], whole[k]) < tol_self, k
        assert rel_err(got[k], refs[k]) < tol_ref, k
    assert eng.pool.num_free == 12 and not eng.requests


def test_greedy_generation_through_the_scheduler_matches_the_oracle():
    """engine.generate: six prompts, two state slots, a token budget that cuts prompts into portions -- the scheduler
    batches portions beside decoded tokens and reuses slots and pages; every generated token is the oracle's argmax."""
    from vllm_hymeta.engine import SamplingParams
    cfg = sonuzen_config(**MODELS["hybrid_loop"])
    weights = sonuzen_random_weights(cfg, seed=4)
    prompts = [_tokens(n, cfg["vocab"], 40 + n) for n in (23, 5, 1, 37, 12, 18)]
    new = 5
    eng = build_engine(cfg, weights, torch.float32, max_tokens=128, block_size=16, max_num_seqs=2, max_num_batched_tokens=16)
    outs = eng.generate(prompts, SamplingParams(max_tokens=new))
    assert eng.pool.num_free == 8 and not eng.requests
    for p, o in zip(prompts, outs):
        assert len(o) == new
        toks = list(p)
        for t in o:
            logits = sonuzen_ref(cfg, weights, toks)[-1]
            best = int(logits.argmax())
            top2 = logits.topk(2).values
            if float(top2[0] - top2[1]) > 1e-3:        # a clear winner: the engine must have picked it
                assert t == best
            toks.append(t)


def test_long_decode_keeps_its_states():
    """400 tokens decoded one by one after a two-token prompt (fp32): recurrent, convolution and page bookkeeping hold."""
    cfg = sonuzen_config(**MODELS["hybrid_loop"])
    weights = sonuzen_random_weights(cfg, seed=8)
    toks = _tokens(402, cfg["vocab"], 3)
    eng = build_engine(cfg, weights, torch.float32, max_tokens=416, block_size=32, max_num_seqs=1)
    whole = eng.run_batch([("w", toks, [401, 200, 17])])
    eng.finish_request("w")
    eng.run_batch([("d", toks[:2], [])])
    last = None
    for i in range(2, 402):
        out = eng.run_batch([("d", toks[i:i + 1], [0] if i in (17, 200, 401) else [])])
        if i == 17:
            assert rel_err(out, whole[2:3]) < 3e-5
        if i == 200:
            assert rel_err(out, whole[1:2]) < 3e-5
        last = out
    assert rel_err(last, whole[0:1]) < 3e-5
    ref = sonuzen_ref(cfg, weights, toks[:201])[-1:]
    eng.finish_request("d")
    got = eng.run_batch([("x", toks[:201], [200])])
    assert rel_err(got, ref) < 3e-5
