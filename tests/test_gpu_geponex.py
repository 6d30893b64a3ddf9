"""The Geponex building blocks and the model under the engine, against the plain CPU statement in ``oracle/geponex.py``.

Mechanisms alone first (token shift with its carried row, the grouped norm after the sum, the latent attention's cache
rows and queries, attention over rows shared by keys and values with a sink logit, lightning attention with its state,
the activations, the sigmoid router and its experts), then whole models of several shapes: a prompt in one step against
the oracle, and the same tokens cut into steps in every way the engine allows (token by token, portions down to two
tokens, unequal requests in one batch, pages and state slots used again) against the one-step result.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle.geponex import (geponex_config, geponex_random_weights, geponex_ref, group_norm_ref,  # noqa: E402
                            latent_attention_ref, latent_mixer_config, lightning_mixer_config, lightning_ref, moe_config, moe_ff_ref,
                            rotary_frequencies_ref, rotate_pairs_ref, shared_row_attention_ref, token_shift_ref, xielu_ref)

DEV = "cuda"


def rel_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    got, ref = got.double().cpu(), ref.double().cpu()
    return float((got - ref).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt().clamp_min(1e-30))


def rows_close(got: torch.Tensor, ref: torch.Tensor, tol: float, exact: bool) -> bool:
    """fp32 (``exact``): the whole tensor within ``tol``.  bf16: a router's choice between two experts with nearly equal
    scores may fall the other way for a few rows, which moves those rows by much more than rounding does; so the typical
    row is within ``0.6 tol`` and at most one row in ten beyond ``tol``."""
    if exact:
        return rel_err(got, ref) < tol
    got, ref = got.double().cpu(), ref.double().cpu()
    err = (got - ref).pow(2).mean(-1).sqrt() / ref.pow(2).mean(-1).sqrt().clamp_min(1e-30)
    return float(err.median()) < 0.6 * tol and float((err > tol).float().mean()) <= 0.1


def i32(v):
    return torch.tensor(v, dtype=torch.int32, device=DEV)


def bf16_values(*shape, std=1.0, gen=None):
    return (torch.randn(*shape, generator=gen) * std).to(torch.bfloat16).double()


def layout_of(portions, contexts, slots, block_tables=None, block_size=16):
    """A step's layout from (rows, tokens before them, state slot) per sequence."""
    from itertools import accumulate
    from vllm_hymeta.models.stream_block import StepLayout
    qsl = list(accumulate(portions, initial=0))
    slot_mapping = None
    bt = None
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


# --------------------------------------------------------------------------- token shift
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [48, 256, 600])
def test_token_shift_in_portions_carries_the_last_row(dtype, width):
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(width)
    xs = [torch.randn(n, width, generator=g) for n in (37, 1, 9)]
    mix = torch.rand(width, generator=g)
    refs = [token_shift_ref(x.double(), mix.double()) for x in xs]
    state = torch.full((4, width), 7.0, device=DEV)                      # stale values: a new sequence must not read them
    slots = [2, 0, 3]
    got = [[] for _ in xs]
    at = [0, 0, 0]
    # sequence 0 in portions of 2, 1, 5, 29; sequence 1 a single token; sequence 2 in 4 + 5, starting later
    for step in ([(0, 2)], [(0, 1), (1, 1)], [(0, 5), (2, 4)], [(2, 5), (0, 29)]):
        rows = torch.cat([xs[k][at[k]:at[k] + n] for k, n in step]).to(DEV)
        lay = layout_of([n for _, n in step], [at[k] for k, _ in step], [slots[k] for k, _ in step])
        out = hip_ops.token_shift(rows, mix.to(DEV), state, dtype, lay.query_start_loc, lay.context_lens, lay.slot_idx)
        r = 0
        for k, n in step:
            got[k].append(out[r:r + n])
            r += n
            at[k] += n
    for k in range(3):
        assert rel_err(torch.cat(got[k]), refs[k]) < (1e-6 if dtype == torch.float32 else 4e-3), k
    assert torch.equal(state[2].cpu(), xs[0][-1]) and torch.equal(state[3].cpu(), xs[2][-1])
    assert torch.all(state[1] == 7.0)
    # the slot of the sequence that ended is taken by a new one: it starts from zeros, not from the old row
    x_new = torch.randn(3, width, generator=g)
    lay = layout_of([3], [0], [2])
    out = hip_ops.token_shift(x_new.to(DEV), mix.to(DEV), state, torch.float32, lay.query_start_loc, lay.context_lens, lay.slot_idx)
    assert rel_err(out, token_shift_ref(x_new.double(), mix.double())) < 1e-6


# --------------------------------------------------------------------------- norm after the sum
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,groups", [(48, 3), (256, 2), (520, 1), (1024, 8)])
def test_grouped_norm_after_the_sum(dtype, width, groups):
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(groups)
    x = torch.randn(11, width, generator=g)
    x[:, :width // groups] *= 30.0                     # one group much larger than the others: a norm over the whole row shows
    y, y2 = torch.randn(11, width, generator=g).to(dtype), torch.randn(11, width, generator=g).to(dtype)
    w = 1 + 0.1 * torch.randn(width, generator=g)
    eps, alpha = 1e-5, 1.5
    tol = 1e-6 if dtype == torch.float32 else 4e-3
    ref = group_norm_ref(alpha * x.double() + y.double() + y2.double(), w.double(), groups, eps)
    xs = x.clone().to(DEV)
    out = hip_ops.add_group_norm(xs, y.to(DEV), w.to(DEV), groups, eps, alpha, y2.to(DEV), in_place=True, out_dtype=dtype)
    assert rel_err(xs, ref) < 1e-6 and rel_err(out, ref) < tol and out.dtype == dtype
    # the last norm of a model: no sublayer output, the stream is left alone
    xs = x.clone().to(DEV)
    out = hip_ops.add_group_norm(xs, None, w.to(DEV), groups, eps, 1.0, in_place=False, out_dtype=dtype)
    assert torch.equal(xs.cpu(), x) and rel_err(out, group_norm_ref(x.double(), w.double(), groups, eps)) < tol
    # groups matter: the same row normed as one group differs
    if groups > 1:
        assert rel_err(group_norm_ref(x.double(), w.double(), 1, eps), group_norm_ref(x.double(), w.double(), groups, eps)) > 0.1


# --------------------------------------------------------------------------- attention over shared rows
def _paged_rows(rows, dtype, block_size, shuffle_seed=0):
    """``rows [T, Dk]`` written into a shuffled page pool; returns (cache [blocks, block_size, 1, Dk], block table)."""
    T, Dk = rows.shape
    nb = (T + block_size - 1) // block_size
    perm = torch.randperm(nb + 3, generator=torch.Generator().manual_seed(shuffle_seed)).tolist()[:nb]
    cache = torch.full((nb + 3, block_size, 1, Dk), float("nan"), dtype=dtype)
    for p in range(T):
        cache[perm[p // block_size], p % block_size, 0] = rows[p].to(dtype)
    return cache.to(DEV), perm


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,C,R,sink", [(3, 40, 8, True), (4, 64, 32, False), (8, 128, 64, True), (1, 24, 0, True), (16, 64, 32, True),
                                       (4, 256, 64, True), (3, 384, 64, False), (20, 512, 64, True), (40, 64, 32, True), (36, 256, 64, False)])
def test_attention_over_rows_shared_by_keys_and_values(dtype, H, C, R, sink):
    """Portions of a prompt and single rows over pages, against the plain statement; the sink logit of every head counts."""
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(H * C)
    T, bs = 150, 16 if C != 64 else 64
    rows = bf16_values(T, C + R, gen=g)
    q = bf16_values(T, H, C + R, gen=g)
    sk = bf16_values(H, std=2.0, gen=g) if sink else None
    scale = (C + R) ** -0.5 * 2.0
    ref = shared_row_attention_ref(q, rows, C, scale, sk)
    if sink:
        assert rel_err(shared_row_attention_ref(q, rows, C, scale, torch.zeros(H, dtype=torch.float64)), ref) > 1e-2
    cache, table = _paged_rows(rows, dtype, bs, shuffle_seed=C)
    outs, at = [], 0
    for n in (70, 2, 1, 1, 63, 1, 12):
        lay = layout_of([n], [at], [0], [table], bs)
        outs.append(hip_ops.sink_attention(q[at:at + n].to(dtype).to(DEV), cache, lay.block_tables, lay.query_start_loc, lay.seq_lens, 1, C + R, C,
                                           scale, n, at + n, sink=sink, sink_logits=None if sk is None else sk.float().to(DEV), value_in_key=True))
        at += n
    assert at == T
    assert rel_err(torch.cat(outs), ref) < (2e-6 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("C,R", [(64, 32), (512, 64)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_row_far_back_decides_the_output(dtype, C, R):
    """Among 700 rows one (at a page border, far from the query) matches the query's direction with a large score: the
    output is that row's value part, in a prompt's portion and for a single decoded row alike."""
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(5)
    T, H, bs = 700, 4, 64
    rows = bf16_values(T, C + R, std=0.3, gen=g)
    q = bf16_values(T, H, C + R, std=0.3, gen=g)
    far = 64                                            # first row of the second page
    direction = torch.nn.functional.normalize(torch.randn(C + R, generator=g).double(), dim=0)
    rows[far] = (direction * 6).to(torch.bfloat16).double()
    q[-1, :] = (direction * 8).to(torch.bfloat16).double()
    q[500, 2] = (direction * 8).to(torch.bfloat16).double()
    sk = torch.zeros(H, dtype=torch.float64)
    cache, table = _paged_rows(rows, dtype, bs, shuffle_seed=1)
    lay = layout_of([T - 1], [0], [0], [table], bs)
    out = hip_ops.sink_attention(q[:T - 1].to(dtype).to(DEV), cache, lay.block_tables, lay.query_start_loc, lay.seq_lens, 1, C + R, C, 1.0,
                                 T - 1, T - 1, sink=True, sink_logits=sk.float().to(DEV), value_in_key=True)
    assert rel_err(out[500, 2], rows[far, :C]) < 2e-2
    lay = layout_of([1], [T - 1], [0], [table], bs)
    one = hip_ops.sink_attention(q[T - 1:].to(dtype).to(DEV), cache, lay.block_tables, lay.query_start_loc, lay.seq_lens, 1, C + R, C, 1.0,
                                 1, T, sink=True, sink_logits=sk.float().to(DEV), value_in_key=True)
    for h in range(H):
        assert rel_err(one[0, h], rows[far, :C]) < 2e-2


def test_attention_batches_unequal_sequences_like_each_alone():
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(9)
    H, C, R, bs = 4, 64, 32, 64
    lens, ctxs = [90, 1, 130, 1], [0, 77, 40, 0]
    seqs = [(bf16_values(c + n, C + R, gen=g), bf16_values(n, H, C + R, gen=g)) for n, c in zip(lens, ctxs)]
    sk = bf16_values(H, gen=g).float().to(DEV)
    nb = [(c + n + bs - 1) // bs for n, c in zip(lens, ctxs)]
    cache = torch.zeros(sum(nb), bs, 1, C + R, dtype=torch.bfloat16)
    tables, base = [], 0
    for (rows, _), k in zip(seqs, nb):
        tables.append(list(range(base, base + k)))
        for p in range(rows.shape[0]):
            cache[base + p // bs, p % bs, 0] = rows[p].to(torch.bfloat16)
        base += k
    cache = cache.to(DEV)
    lay = layout_of(lens, ctxs, [0, 1, 2, 3], tables, bs)
    q = torch.cat([s[1] for s in seqs]).to(torch.bfloat16).to(DEV)
    both = hip_ops.sink_attention(q, cache, lay.block_tables, lay.query_start_loc, lay.seq_lens, 1, C + R, C, 0.2, max(lens), 170, sink=True,
                                  sink_logits=sk, value_in_key=True)
    r = 0
    for k, (n, c) in enumerate(zip(lens, ctxs)):
        lay1 = layout_of([n], [c], [0], [tables[k]], bs)
        alone = hip_ops.sink_attention(seqs[k][1].to(torch.bfloat16).to(DEV), cache, lay1.block_tables, lay1.query_start_loc, lay1.seq_lens, 1,
                                       C + R, C, 0.2, n, c + n, sink=True, sink_logits=sk, value_in_key=True)
        assert rel_err(both[r:r + n], alone) < 1e-6, k
        r += n


# --------------------------------------------------------------------------- the latent attention sublayer
def _latent_mixer(m, w, dtype, eps, prefix):
    from vllm_hymeta.linear import HymetaLinear
    from vllm_hymeta.models.configuration_geponex import RotarySpec
    from vllm_hymeta.models.latent_attention import LatentAttentionMixer, PagedLatentAttention
    H, D, R, Dv, C, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]

    def dev(t, dt=dtype):
        return t.to(dt).to(DEV).contiguous()

    gate = "g" in w
    attn = PagedLatentAttention(H, C, R, m["scale"], prefix, sink_logits=dev(w["sink"], torch.float32) if "sink" in w else None, dtype=dtype)
    freqs, mag = RotarySpec(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling")).frequencies()
    down = torch.cat([w["dq"], w["dkv"]] + ([w["g"]] if gate else []), 0)
    return LatentAttentionMixer(HymetaLinear.from_weight(dev(down)), HymetaLinear.from_weight(dev(w["uq"])), dev(w["uk"]).view(H, D, C),
                                dev(w["uv"]).view(H, Dv, C).transpose(1, 2).contiguous(), HymetaLinear.from_weight(dev(w["o"])), attn,
                                H, D, R, Dv, C, Q, dev(w["dq.norm"], torch.float32), dev(w["dkv.norm"], torch.float32), eps, m["rot"]["dims"],
                                torch.tensor(freqs, dtype=torch.float64, device=DEV), mag, gate), attn


_YARN = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind,mixer", [
    ("latent_attention_2", latent_mixer_config()),
    ("latent_attention", latent_mixer_config(scaling=_YARN)),
    ("latent_attention", latent_mixer_config(heads=5, dim=16, rot_dim=32, vdim=48, kv_rank=64, q_rank=72, base=300000.0, scaling=_YARN)),
    ("latent_attention_2", latent_mixer_config(heads=1, dim=8, rot_dim=16, vdim=8, kv_rank=24, q_rank=16)),
])
def test_latent_attention_sublayer_in_portions(dtype, kind, mixer):
    """The whole sublayer over a paged cache, a prompt cut into portions and decoded rows, against the plain statement
    that writes keys and values out per head.  YaRN's blended frequencies and magnitude, the sink and the gate each show."""
    from vllm_hymeta.models.attention import bind_kv_cache, standalone_prefix
    W, eps, T, bs = 48, 1e-5, 100, 16
    cfg = geponex_config(width=W, layers=[(kind, mixer, None)])
    weights = geponex_random_weights(cfg, seed=mixer["heads"])
    w = {k[len("l0.mix."):]: v.double() for k, v in weights.items() if k.startswith("l0.mix.")}
    h = bf16_values(T, W, gen=torch.Generator().manual_seed(2))
    ref = latent_attention_ref(h, w, mixer, eps)
    if mixer["rot"].get("scaling"):
        plain = dict(mixer, rot={k: v for k, v in mixer["rot"].items() if k != "scaling"})
        assert rel_err(latent_attention_ref(h, w, plain, eps), ref) > 1e-2
    if "sink" in w:
        assert rel_err(latent_attention_ref(h, dict(w, sink=w["sink"] - 3.0), mixer, eps), ref) > 1e-2
    mod, attn = _latent_mixer(mixer, w, dtype, eps, standalone_prefix("latent"))
    nb = (T + bs - 1) // bs
    table = torch.randperm(nb + 2, generator=torch.Generator().manual_seed(3)).tolist()[:nb]
    bind_kv_cache(attn, torch.zeros(attn.kv_cache_shape(nb + 2, bs), dtype=dtype, device=DEV))
    outs, at = [], 0
    for n in (33, 2, 1, 31, 1, 1, 30, 1):
        lay = layout_of([n], [at], [0], [table], bs)
        outs.append(mod(h[at:at + n].to(dtype).to(DEV), lay, attn))
        at += n
    assert at == T
    assert rel_err(torch.cat(outs), ref) < (1e-5 if dtype == torch.float32 else 2e-2)


def test_rotation_of_the_first_dimensions_only():
    """``rot.dims`` smaller than the rotated part: the pairs behind it pass unchanged, into the cache and into the query."""
    from vllm_hymeta import hip_ops
    T, H, D, R, dims, C = 9, 2, 8, 16, 6, 24
    g = torch.Generator().manual_seed(1)
    freqs, mag = rotary_frequencies_ref(dims, 100.0, None)
    q = torch.randn(T, H, D + R, generator=g)
    q_abs = torch.randn(H, T, C, generator=g)
    lay = layout_of([T], [40], [0])
    out = hip_ops.latent_q_assemble(q.to(DEV), q_abs.to(DEV), D, R, dims, freqs.to(DEV), mag, lay.query_start_loc, lay.seq_lens)
    pos = torch.arange(40, 40 + T)
    assert torch.equal(out[:, :, :C].cpu(), q_abs.transpose(0, 1))
    assert rel_err(out[:, :, C:C + dims], rotate_pairs_ref(q[:, :, D:D + dims].double(), pos, freqs, mag)) < 1e-6
    assert torch.equal(out[:, :, C + dims:].cpu(), q[:, :, D + dims:])


# --------------------------------------------------------------------------- lightning attention
def _lightning_mixer(m, w, dtype, eps):
    from vllm_hymeta.linear import HymetaLinear
    from vllm_hymeta.models.lightning_attention import LightningAttentionMixer

    def dev(t, dt=dtype):
        return t.to(dt).to(DEV).contiguous()

    return LightningAttentionMixer(HymetaLinear.from_weight(dev(torch.cat([w["q"], w["k"], w["v"], w["g"]], 0))), HymetaLinear.from_weight(dev(w["o"])),
                                   m["heads"], m["dim"], m["vdim"], torch.tensor(m["decay"], dtype=torch.float32, device=DEV),
                                   dev(w["norm"], torch.float32), eps)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mixer", [lightning_mixer_config(), lightning_mixer_config(heads=2, dim=32, vdim=64, decay=[0.6, 0.999]),
                                   lightning_mixer_config(heads=1, dim=128, vdim=32, decay=[0.97]),
                                   lightning_mixer_config(heads=5, dim=8, vdim=40)])
def test_lightning_attention_prefill_equals_token_by_token_and_portions(dtype, mixer):
    """One step over the prompt, token by token, and portions whose edges fall before, on and behind multiples of 64
    rows: the same outputs; the state is carried in fp32 and a slot that is used again starts from zero."""
    W, eps, T = 48, 1e-5, 200
    cfg = geponex_config(width=W, layers=[("lightning", mixer, None)])
    weights = geponex_random_weights(cfg, seed=mixer["heads"])
    w = {k[len("l0.mix."):]: v.double() for k, v in weights.items() if k.startswith("l0.mix.")}
    h = bf16_values(T, W, gen=torch.Generator().manual_seed(4))
    ref = lightning_ref(h, w, mixer, eps)
    mod = _lightning_mixer(mixer, w, dtype, eps)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    state = torch.full((3, mixer["heads"], mixer["dim"], mixer["vdim"]), 5.0, device=DEV)       # stale: must not be read
    hd = h.to(dtype).to(DEV)
    whole = mod(hd, layout_of([T], [0], [1]), state)
    assert rel_err(whole, ref) < tol
    s_whole = state[1].clone()
    assert torch.all(state[0] == 5.0) and torch.all(state[2] == 5.0)
    for plan in ([1] * 70, [63, 1, 64, 2, 65, 5], [2, 130, 1, 67], [128, 72]):
        outs, at = [], 0
        for n in plan:
            outs.append(mod(hd[at:at + n], layout_of([n], [at], [2]), state))
            at += n
        assert rel_err(torch.cat(outs), ref[:at]) < tol, plan
        if at == T:
            assert rel_err(state[2], s_whole) < (1e-5 if dtype == torch.float32 else 1e-2)


def test_lightning_long_portions_run_in_segments():
    """A portion of 2300 rows (segments of 1024 side by side, chained through their states) behind 70 rows that left a
    state, beside a short portion and a decoding sequence in the same step: outputs and final states as token by token."""
    mixer = lightning_mixer_config(heads=2, dim=32, vdim=64, decay=[0.97, 0.9995])
    W, eps, T = 32, 1e-6, 2370
    cfg = geponex_config(width=W, layers=[("lightning", mixer, None)])
    weights = geponex_random_weights(cfg, seed=11)
    w = {k[len("l0.mix."):]: v.double() for k, v in weights.items() if k.startswith("l0.mix.")}
    g = torch.Generator().manual_seed(12)
    h, h2, h3 = bf16_values(T, W, gen=g), bf16_values(90, W, gen=g), bf16_values(31, W, gen=g)
    ref, ref2, ref3 = lightning_ref(h, w, mixer, eps), lightning_ref(h2, w, mixer, eps), lightning_ref(h3, w, mixer, eps)
    mod = _lightning_mixer(mixer, w, torch.bfloat16, eps)
    state = torch.full((4, 2, 32, 64), 3.0, device=DEV)
    dev = lambda t: t.to(torch.bfloat16).to(DEV)
    first = mod(torch.cat([dev(h[:70]), dev(h3[:30])]), layout_of([70, 30], [0, 0], [1, 3]), state)
    step = mod(torch.cat([dev(h[70:]), dev(h2), dev(h3[30:])]), layout_of([T - 70, 90, 1], [70, 0, 30], [1, 0, 3]), state)
    assert rel_err(first[:70], ref[:70]) < 2e-2
    assert rel_err(step[:T - 70], ref[70:]) < 2e-2 and rel_err(step[T - 70:T - 70 + 90], ref2) < 2e-2 and rel_err(step[-1:], ref3[30:]) < 2e-2
    # the final states against a token-by-token run of the same rows
    state2 = torch.zeros_like(state)
    for t in range(T):
        mod(dev(h[t:t + 1]), layout_of([1], [t], [2]), state2)
    assert rel_err(state[1], state2[2]) < 2e-3
    assert torch.all(state[2] == 3.0)


def test_lightning_attention_batches_unequal_sequences():
    mixer = lightning_mixer_config(heads=2, dim=32, vdim=64, decay=[0.8, 0.99])
    W, eps = 64, 1e-6
    cfg = geponex_config(width=W, layers=[("lightning", mixer, None)])
    weights = geponex_random_weights(cfg, seed=3)
    w = {k[len("l0.mix."):]: v.double() for k, v in weights.items() if k.startswith("l0.mix.")}
    mod = _lightning_mixer(mixer, w, torch.bfloat16, eps)
    g = torch.Generator().manual_seed(6)
    lens = [100, 1, 65, 1, 2]
    hs = [bf16_values(n, W, gen=g).to(torch.bfloat16).to(DEV) for n in lens]
    state = torch.zeros(5, 2, 32, 64, device=DEV)
    # sequences 1 and 3 decode from states that earlier steps left
    for k in (1, 3):
        mod(bf16_values(40 + k, W, gen=g).to(torch.bfloat16).to(DEV), layout_of([40 + k], [0], [k]), state)
    before = state.clone()
    ctxs = [0, 41, 0, 43, 0]
    both = mod(torch.cat(hs), layout_of(lens, ctxs, [0, 1, 2, 3, 4]), state)
    after = state.clone()
    state.copy_(before)
    r = 0
    for k, n in enumerate(lens):
        alone = mod(hs[k], layout_of([n], [ctxs[k]], [k]), state)
        assert rel_err(both[r:r + n], alone) < 1e-6, k
        r += n
    assert rel_err(after, state) < 1e-6


def test_lightning_state_keeps_a_token_from_far_back():
    """With a decay close to one the first token's key and value still decide the output 300 tokens later; with a small
    decay they are gone."""
    from vllm_hymeta import hip_ops
    H, D, Dv, T = 2, 32, 32, 300
    qkv = torch.zeros(T, 2 * H * D + H * Dv)
    qkv[:, :] = -20.0                                   # silu(-20) ~ 0: empty tokens
    qkv[0, H * D:2 * H * D] = 4.0                       # the first token's key ...
    qkv[0, 2 * H * D:] = torch.arange(H * Dv) % 7 + 1.0    # ... and value
    qkv[-1, :H * D] = 4.0                               # the last token asks for it
    decay = torch.tensor([0.9999, 0.5])
    for dtype in (torch.float32, torch.bfloat16):
        state = torch.zeros(1, H, D, Dv, device=DEV)
        lay = layout_of([T], [0], [0])
        out = hip_ops.lightning_attention(qkv.to(dtype).to(DEV), state, decay.to(DEV), H, D, Dv, lay.query_start_loc, lay.context_lens, lay.slot_idx, T)
        silu = torch.nn.functional.silu
        k0, v0, q = silu(torch.tensor(4.0)), silu(qkv[0, 2 * H * D:2 * H * D + Dv].to(dtype).float()), silu(torch.tensor(4.0))
        want = 0.9999 ** (T - 1) * D * float(k0) * float(q) * v0
        assert rel_err(out[-1, :Dv], want) < 1e-2
        assert float(out[-1, Dv:].abs().max()) < 1e-6


# --------------------------------------------------------------------------- activations, router, experts
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_activations(dtype):
    from vllm_hymeta import hip_ops
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(7, 2 * 72, generator=g) * 3).to(dtype)
    tol = 1e-6 if dtype == torch.float32 else 5e-3
    sp = torch.nn.functional.softplus
    p, q = torch.tensor(0.3, dtype=torch.float64), torch.tensor(-0.7, dtype=torch.float64)
    got = hip_ops.xielu(x.to(DEV), float(sp(p)), float(0.5 + sp(q)))
    assert rel_err(got, xielu_ref(x.double(), p, q)) < tol
    limit = 1.25
    gate, up = x[:, :72].double(), x[:, 72:].double()
    ref = torch.clamp(gate, max=limit) * torch.sigmoid(1.702 * torch.clamp(gate, max=limit)) * (torch.clamp(up, -limit, limit) + 1)
    assert rel_err(hip_ops.clamped_glu(x.to(DEV), limit), ref) < tol
    assert float((gate > limit).float().mean()) > 0.1 and float((up.abs() > limit).float().mean()) > 0.1      # the clamps are at work
    gt = (torch.randn(7, 144, generator=g)).to(dtype)
    assert rel_err(hip_ops.sigmoid_gate_mul(x.to(DEV), gt.to(DEV)), x.double() * torch.sigmoid(gt.double())) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W,F,E,top,shared", [(48, 40, 6, 2, True), (64, 64, 16, 4, True), (128, 32, 3, 1, False), (72, 24, 5, 5, False)])
def test_sigmoid_routed_experts(dtype, W, F, E, top, shared):
    from vllm_hymeta.linear import HymetaLinear
    from vllm_hymeta.models.feed_forward import ClampedGluMLP, SigmoidRoutedMoE
    mlp = moe_config(experts=E, top=top, ff=F, limit=0.8, scale=2.5, shared_ff=56 if shared else 0, shared_limit=1.5)
    cfg = geponex_config(width=W, layers=[("lightning", lightning_mixer_config(), mlp)])
    weights = geponex_random_weights(cfg, seed=E)
    w = {k[len("l0.mlp."):]: v.double() for k, v in weights.items() if k.startswith("l0.mlp.")}
    w["router"] = w["router"] * 6.0                    # scores spread out: no close calls between the chosen and the rest
    h = bf16_values(50, W, gen=torch.Generator().manual_seed(top))
    ref = moe_ff_ref(h, w, mlp)

    def dev(t, dt=dtype):
        return t.to(dt).to(DEV).contiguous()

    w13 = torch.stack([torch.cat([w[f"e{e}.gate"], w[f"e{e}.up"]], 0) for e in range(E)])
    w2 = torch.stack([w[f"e{e}.down"] for e in range(E)])
    sh = None
    if shared:
        sh = ClampedGluMLP(HymetaLinear.from_weight(dev(torch.cat([w["shared.gate"], w["shared.up"]], 0))), HymetaLinear.from_weight(dev(w["shared.down"])), 1.5)
    moe = SigmoidRoutedMoE(dev(w["router"], torch.float32), dev(w13), dev(w2), top, 2.5, 0.8, sh)
    y, y2 = moe(dev(h))
    got = y.double() + (0 if y2 is None else y2.double())
    assert rel_err(got, ref) < (1e-5 if dtype == torch.float32 else 2e-2)
    # the constant on the weights and the experts' clamp both show in the result
    assert rel_err(moe_ff_ref(h, w, dict(mlp, router=dict(mlp["router"], scale=1.0))), ref) > 1e-2
    assert rel_err(moe_ff_ref(h, w, dict(mlp, expert=dict(mlp["expert"], limit=8.0))), ref) > 1e-2


# --------------------------------------------------------------------------- whole models under the engine
def build_engine(cfg, weights, dtype, max_tokens=512, block_size=16, max_num_seqs=4, max_num_batched_tokens=1 << 30):
    from vllm_hymeta.engine import LLMEngine
    from vllm_hymeta.models.configuration_geponex import GeponexConfig
    from vllm_hymeta.models.modeling_geponex import GeponexForCausalLM
    model = GeponexForCausalLM(GeponexConfig(cfg), max_num_seqs=max_num_seqs, dtype=dtype, device=DEV)
    model.load_weights(weights.items())
    return LLMEngine(model, num_blocks=max_tokens // block_size, block_size=block_size, max_num_seqs=max_num_seqs,
                     max_num_batched_tokens=max_num_batched_tokens, device=DEV)


_DENSE = {"kind": "dense", "ff": 72}
MODELS = {
    "default": dict(),
    "one_head_one_group_no_mlp_on_one": dict(width=40, groups=1, alpha=1.0, layers=[
        ("lightning", lightning_mixer_config(heads=1, dim=8, vdim=16, decay=[0.9]), None),
        ("latent_attention", latent_mixer_config(heads=1, dim=8, rot_dim=4, vdim=8, kv_rank=12, q_rank=10), moe_config(experts=3, top=1, ff=24, shared_ff=0)),
        ("latent_attention_2", latent_mixer_config(heads=2, dim=8, rot_dim=8, vdim=4, kv_rank=20, q_rank=16), _DENSE)]),
    "matrix_core_sizes": dict(width=128, groups=2, alpha=2.0, layers=[
        ("latent_attention_2", latent_mixer_config(heads=6, dim=16, rot_dim=32, vdim=48, kv_rank=64, q_rank=96), {"kind": "dense", "ff": 192}),
        ("lightning", lightning_mixer_config(heads=2, dim=32, vdim=64, decay=[0.7, 0.995]), moe_config(experts=8, top=2, ff=64, shared_ff=64)),
        ("latent_attention", latent_mixer_config(heads=3, dim=64, rot_dim=64, vdim=32, kv_rank=128, q_rank=64, base=200000.0, scaling=_YARN),
         moe_config(experts=8, top=2, ff=64, shared_ff=64)),
        ("weights_of", 1), ("weights_of", 0)]),
    "lightning_first_weights_shared_twice": dict(width=64, groups=4, alpha=0.5, layers=[
        ("lightning", lightning_mixer_config(heads=4, dim=16, vdim=16), moe_config(experts=4, top=3, ff=32)),
        ("latent_attention", latent_mixer_config(heads=2, dim=16, rot_dim=16, vdim=32, kv_rank=32, q_rank=24), _DENSE),
        ("weights_of", 0), ("weights_of", 1), ("weights_of", 0)]),
}


def _tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


@pytest.mark.parametrize("name", sorted(MODELS))
def test_model_whole_prompt_against_the_oracle_fp32(name):
    cfg = geponex_config(**MODELS[name])
    weights = geponex_random_weights(cfg, seed=len(name))
    toks = _tokens(45, cfg["vocab"], 1)
    layers_ref = []
    ref = geponex_ref(cfg, weights, toks, residual_out=layers_ref)
    eng = build_engine(cfg, weights, torch.float32)
    got = eng.run_batch([("a", toks, list(range(len(toks))))])
    assert got.shape == ref.shape and got.dtype == torch.float32
    assert rel_err(got, ref) < 3e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", sorted(MODELS))
def test_model_schedules_agree_with_the_whole_prompt(name, dtype):
    """Decoding token by token, portions of several sizes (down to two tokens, and one), and a mixed batch of four
    requests whose pages and state slots come from requests that ended: every position's logits equal the one-step
    logits up to rounding, and the oracle's.  In bf16 every token runs all its layer's experts: with fewer, a choice
    between two nearly equal scores falls differently under bf16 rounding now and then, and the lightning state carries
    such a row's difference to every later row, so that a comparison says nothing (the choice itself is tested in fp32
    here and alone in bf16 above)."""
    cfg = geponex_config(**MODELS[name])
    if dtype == torch.bfloat16:
        for entry in cfg["layers"]:
            if entry["mlp"] and entry["mlp"]["kind"] == "moe":
                entry["mlp"] = dict(entry["mlp"], router=dict(entry["mlp"]["router"], top=entry["mlp"]["router"]["experts"]))
    weights = geponex_random_weights(cfg, seed=len(name))
    V = cfg["vocab"]
    seqs = {k: _tokens(n, V, 10 + k) for k, n in enumerate([150, 33, 1, 70, 19, 64])}
    refs = {k: geponex_ref(cfg, weights, t) for k, t in seqs.items()}
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


def test_a_layer_may_run_the_weights_of_a_later_layer():
    cfg = geponex_config(**MODELS["default"])
    cfg["layers"].insert(0, dict(cfg["layers"][1], weights_of=2))              # layer 0 runs (what is now) layer 2's lightning weights
    cfg["layers"][4]["weights_of"] = 2
    weights = {k.replace("l3.", "l4.").replace("l2.", "l3.").replace("l1.", "l2.").replace("l0.", "l1.") if k[0] == "l" else k: v
               for k, v in geponex_random_weights(geponex_config(**MODELS["default"]), seed=2).items()}
    toks = _tokens(40, cfg["vocab"], 9)
    ref = geponex_ref(cfg, weights, toks)
    eng = build_engine(cfg, weights, torch.float32)
    got = eng.run_batch([("a", toks[:25], list(range(25)))])
    got = torch.cat([got, eng.run_batch([("a", toks[25:], list(range(15)))])])
    assert rel_err(got, ref) < 5e-5


def test_greedy_generation_through_the_scheduler_matches_the_oracle():
    """engine.generate: six prompts, two state slots, a token budget that cuts prompts into portions -- the scheduler
    batches portions beside decoded tokens and reuses slots and pages; every generated token is the oracle's argmax."""
    from vllm_hymeta.engine import SamplingParams
    cfg = geponex_config(**MODELS["default"])
    weights = geponex_random_weights(cfg, seed=4)
    prompts = [_tokens(n, cfg["vocab"], 40 + n) for n in (23, 5, 1, 37, 12, 18)]
    new = 5
    eng = build_engine(cfg, weights, torch.float32, max_tokens=128, block_size=16, max_num_seqs=2, max_num_batched_tokens=16)
    outs = eng.generate(prompts, SamplingParams(max_tokens=new))
    assert eng.pool.num_free == 8 and not eng.requests
    for p, o in zip(prompts, outs):
        assert len(o) == new
        toks = list(p)
        for t in o:
            logits = geponex_ref(cfg, weights, toks)[-1]
            top2 = logits.topk(2).values
            if float(top2[0] - top2[1]) > 1e-3:        # a clear winner: the engine must have picked it
                assert t == int(logits.argmax())
            toks.append(t)


def test_long_decode_keeps_its_states():
    """400 tokens decoded one by one after a two-token prompt (fp32): lightning states, shifted rows and pages hold."""
    cfg = geponex_config(**MODELS["default"])
    weights = geponex_random_weights(cfg, seed=8)
    toks = _tokens(402, cfg["vocab"], 3)
    eng = build_engine(cfg, weights, torch.float32, max_tokens=416, block_size=32, max_num_seqs=1)
    whole = eng.run_batch([("w", toks, [401, 200, 17])])
    eng.finish_request("w")
    eng.run_batch([("d", toks[:2], [])])
    last = None
    for i in range(2, 402):
        out = eng.run_batch([("d", toks[i:i + 1], [0] if i in (17, 200, 401) else [])])
        if i == 17:
            assert rel_err(out, whole[2:3]) < 5e-5
        if i == 200:
            assert rel_err(out, whole[1:2]) < 5e-5
        last = out
    assert rel_err(last, whole[0:1]) < 5e-5
    ref = geponex_ref(cfg, weights, toks[:201])[-1:]
    eng.finish_request("d")
    got = eng.run_batch([("x", toks[:201], [200])])
    assert rel_err(got, ref) < 5e-5


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
    cfg = geponex_config(**MODELS["default"])
    weights = {k: v.to(torch.bfloat16).float() for k, v in geponex_random_weights(cfg, seed=12).items()}      # what a bf16 file holds
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
    ra, rb = geponex_ref(cfg, weights, a), geponex_ref(cfg, weights, b)
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
        logits = geponex_ref(cfg, weights, toks)[-1]
        top2 = logits.topk(2).values
        if float(top2[0] - top2[1]) > 1e-3:
            assert t == int(logits.argmax())
        toks.append(t)
    assert len(line["output"]) == 3
