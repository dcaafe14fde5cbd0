"""The Ravelorn design (gated delta rule with per-channel or per-head decay, sink attention with unit-RMS queries and
keys and a query temperature, the two side by side, score-routed experts with identity experts, post-norm layers,
learned positions, soft-capped logits) on the GPU against the plain CPU implementation in oracle/ravelorn.py.

Every test makes its own small configuration and random weights. fp32 weights are compared tightly (the kernels then
run plain fp32); bf16 weights within the noise of bf16 operands. Schedules (whole prompt, token by token, portions,
batches, reused slots) must not change a position's logits beyond rounding. Where random weights would hide a fault
(a key far back, a sink, a token the state must keep) the operation is called on crafted inputs that show it.
"""

from pathlib import Path

import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import ravelorn as orc  # noqa: E402


# ------------------------------------------------------------------------------------------------ configurations
def delta(heads=4, kv_heads=2, dim=8, vdim=12, conv=3, decay_rank=5, gate_rank=7):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                                               "conv": conv, "decay_rank": decay_rank, "gate_rank": gate_rank}}


def pair(heads=4, kv_heads=2, dim=8, vdim=12, coef=0.7, every=5, scale=None, rheads=3, rkv=3, rdim=12, rvdim=8, conv=4,
         left_scale=1.3, right_scale=0.6):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5 if scale is None else scale}
    if every:
        left["q_temp"] = {"coef": coef, "every": every}
    right = {"heads": rheads, "kv_heads": rkv, "dim": rdim, "vdim": rvdim, "conv": conv}
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}}


def moe(experts=5, identity=2, top=3, ff=20):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "identity": identity, "top": top}}


def make_cfg(layers, width=40, vocab=53, eps=1e-5, mult=0.6, cap=9.0, positions=400):
    return {"architecture": "Ravelorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult,
            "logit_softcap": cap, "max_positions": positions, "layers": [dict(l[0], mlp=l[1]) for l in layers]}


MIXED = [(delta(), moe()), (pair(), moe(experts=7, identity=0, top=2, ff=12)), (delta(heads=3, kv_heads=3, dim=12, vdim=6, conv=5), None),
         (pair(heads=3, kv_heads=1, dim=12, vdim=20, every=0, rheads=4, rkv=2, rdim=6, rvdim=10, conv=2), moe(experts=2, identity=3, top=4))]


def build(cfg, dtype=torch.float32, seed=0, edit=None):
    from lit_gpt.config import LayeredConfig
    from lit_gpt.layered import LayeredGPT

    config = LayeredConfig.from_dict(cfg)
    weights = LayeredGPT.random_weights(config, seed=seed)
    if edit:
        edit(weights)
    model = LayeredGPT(config, weights, device=torch.device("cuda", 0), dtype=dtype)
    return model, weights


def tokens_of(n, vocab, seed=0):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def rel_err(got, want):
    """Per row: rms of the mean-free difference over the rms of the mean-free reference."""
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-9)


def engine_logits(model, seqs, cuts, max_seq=None, engine=None):
    """Run sequences together through the BatchEngine: ``cuts[i]`` lists how many tokens request i brings per step
    (0: it sits the step out). Returns the logits of every position per request."""
    from generate.batch import BatchEngine

    eng = engine or BatchEngine(model, max_seq_length=max_seq or max(len(s) for s in seqs), slots=1)
    out = [[] for _ in seqs]
    at = [0] * len(seqs)
    ids = [object() for _ in seqs]
    for step in range(max(len(c) for c in cuts)):
        entries, who, end = [], [], []
        for i, s in enumerate(seqs):
            n = cuts[i][step] if step < len(cuts[i]) else 0
            if n:
                entries.append((ids[i], s[at[i]:at[i] + n], list(range(n))))
                who.append((i, n))
                at[i] += n
                if at[i] == len(s):
                    end.append(ids[i])
        lg = eng.step(entries, end)
        row = 0
        for i, n in who:
            out[i].append(lg[row:row + n].cpu())
            row += n
    assert all(a == len(s) for a, s in zip(at, seqs))
    return [torch.cat(o) for o in out]


def portions(n, size):
    return [size] * (n // size) + ([n % size] if n % size else [])


TOL32, TOL16, SAME = 2e-4, 6e-2, 2e-5


# ------------------------------------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("layers", [
    [(delta(), None)],
    [(delta(heads=1, kv_heads=1, dim=5, vdim=3, conv=1, decay_rank=1, gate_rank=2), None)],  # no history, odd sizes
    [(delta(heads=6, kv_heads=2, dim=20, vdim=70, conv=7), None)],  # three value heads per key head, two column blocks
    [(delta(heads=2, kv_heads=1, dim=72, vdim=8, conv=2), None)],
    [(delta(heads=2, kv_heads=2, dim=132, vdim=4, conv=4), None)],  # more than 128 state rows
    [(pair(), None)],
    [(pair(heads=6, kv_heads=2, dim=6, vdim=10, every=1, coef=0.3), None)],  # key size no multiple of 4; every step
    [(pair(heads=3, kv_heads=3, dim=16, vdim=136, every=0, rheads=2, rkv=1, rdim=8, rvdim=72), None)],  # no temperature
    [(pair(heads=1, kv_heads=1, dim=12, vdim=8, every=4, coef=2.0, scale=0.9, left_scale=1.0, right_scale=0.0), None)],
    [(pair(left_scale=0.0, right_scale=1.0, conv=1), None)],  # the delta rule alone, per-head decay
    [(delta(), moe())],
    [(delta(), moe(experts=1, identity=0, top=1, ff=9))],
    [(delta(), moe(experts=3, identity=4, top=5, ff=33))],  # more identity experts than real ones
    [(delta(), moe(experts=70, identity=1, top=2, ff=6))],  # two lanes' worth of router outputs
    [(pair(), moe()), (delta(), None)],
])
def test_mechanism_against_plain(layers):
    cfg = make_cfg(layers)
    model, w = build(cfg)
    toks = tokens_of(29, cfg["vocab"])
    want = orc.forward(cfg, w, toks)
    got = engine_logits(model, [toks], [[len(toks)]])[0]
    assert rel_err(got, want).max() < TOL32
    got = engine_logits(model, [toks], [[1] * len(toks)])[0]
    assert rel_err(got, want).max() < TOL32


@pytest.mark.parametrize("mult,cap", [(1.0, 0.0), (0.25, 2.0)])
def test_residual_factor_and_cap(mult, cap):
    cfg = make_cfg(MIXED[:2], mult=mult, cap=cap)
    model, w = build(cfg, seed=9)
    toks = tokens_of(17, cfg["vocab"])
    assert rel_err(engine_logits(model, [toks], [[len(toks)]])[0], orc.forward(cfg, w, toks)).max() < TOL32


def test_residual_after_every_layer():
    from lit_gpt.mixers import StepBatch

    cfg = make_cfg(MIXED)
    model, w = build(cfg)
    toks = tokens_of(23, cfg["vocab"])
    want = []
    orc.forward(cfg, w, toks, layers_out=want)
    model.set_kv_cache(1, 32)
    got = []
    with torch.inference_mode():
        model._forward_post(StepBatch.build([(0, 0, toks)], model.device), after_layer=lambda run, x: got.append(x.cpu().clone()))
    assert len(got) == len(want) == len(MIXED)
    for g, e in zip(got, want):
        assert (g.double() - e).abs().max() < 1e-4 * e.abs().max()


@pytest.mark.parametrize("width,vocab", [(8, 11), (50, 300), (136, 70)])
def test_other_widths(width, vocab):
    cfg = make_cfg(MIXED, width=width, vocab=vocab)
    model, w = build(cfg, seed=3)
    toks = tokens_of(21, vocab, seed=2)
    assert rel_err(engine_logits(model, [toks], [[len(toks)]])[0], orc.forward(cfg, w, toks)).max() < TOL32


def test_wide_rows_through_the_norm():
    """Rows wider than the norm kernel keeps in registers."""
    from lit_gpt import seq_ops

    dev = torch.device("cuda", 0)
    for n in (8, 50, 1030, 4096, 5000):
        g = torch.Generator().manual_seed(n)
        y, x = torch.randn(5, n, generator=g) * 3 + 1, torch.randn(5, n, generator=g)
        w, b = torch.randn(n, generator=g), torch.randn(n, generator=g)
        want = x.double() + 0.7 * orc.layer_norm(y.double(), w.double(), b.double(), 1e-5)
        xd = x.to(dev)
        out, o16 = seq_ops.layernorm(y.to(dev), w.to(dev), b.to(dev), eps=1e-5, x=xd, mult=0.7, bf16_copy=True)
        assert out.data_ptr() == xd.data_ptr() and (xd.cpu().double() - want).abs().max() < 2e-5
        assert torch.equal(o16.cpu(), xd.cpu().bfloat16())
        plain = seq_ops.layernorm(y.to(dev), w.to(dev), None, eps=1e-5)
        assert (plain.cpu().double() - orc.layer_norm(y.double(), w.double(), torch.zeros(n).double(), 1e-5)).abs().max() < 2e-5


def test_bf16_within_operand_noise():
    cfg = make_cfg(MIXED)
    model, w = build(cfg, dtype=torch.bfloat16)
    toks = tokens_of(40, cfg["vocab"])
    want = orc.forward(cfg, w, toks)
    whole = engine_logits(model, [toks], [[len(toks)]])[0]
    single = engine_logits(model, [toks], [[24] + [1] * 16])[0]
    # (routing is a hard choice: a bf16 product may flip a near tie, so the bulk of the rows is what is compared)
    assert rel_err(whole, want).median() < TOL16 and rel_err(single, want).median() < TOL16


@pytest.mark.parametrize("width,vocab", [(50, 300), (136, 70), (200, 97)])
def test_bf16_without_routing_is_within_operand_noise_everywhere(width, vocab):
    """No hard choices in the model: every row must be within bf16 operand noise, also at widths and head sizes that
    are no multiples of the vector widths, as a whole prompt (MFMA tiles), in portions and token by token."""
    layers = [(delta(heads=3, kv_heads=1, dim=10, vdim=14, conv=2), None),
              (pair(heads=6, kv_heads=3, dim=6, vdim=10, every=7, rheads=2, rkv=2, rdim=20, rvdim=6), None),
              (delta(heads=2, kv_heads=2, dim=16, vdim=24, conv=4), None)]
    cfg = make_cfg(layers, width=width, vocab=vocab)
    model, w = build(cfg, dtype=torch.bfloat16, seed=5)
    toks = tokens_of(61, vocab, seed=3)
    want = orc.forward(cfg, w, toks)
    for cuts in ([61], [40] + [1] * 21, [13, 9, 20, 19]):
        assert rel_err(engine_logits(model, [toks], [cuts])[0], want).max() < TOL16, cuts


# ------------------------------------------------------------------------------------------------ schedules
def slow_state(w):
    for k in w:
        if k.endswith("A_log"):
            w[k] = torch.full_like(w[k], -20.0)  # decay exp(-exp(-20) ...) = 1: what the state took in stays


@pytest.mark.parametrize("edit", [None, slow_state])
def test_prompt_portions_and_single_tokens_agree(edit):
    cfg = make_cfg(MIXED)
    model, w = build(cfg, edit=edit)
    n = 45
    toks = tokens_of(n, cfg["vocab"], seed=5)
    want = orc.forward(cfg, w, toks)
    whole = engine_logits(model, [toks], [[n]])[0]
    assert rel_err(whole, want).max() < TOL32
    for cuts in ([1] * n, portions(n, 2), portions(n, 3), portions(n, 7), portions(n, 16), [17, 1, 1, 2, 24],
                 [30] + [1] * 15):
        got = engine_logits(model, [toks], [cuts])[0]
        assert rel_err(got, whole).max() < SAME, cuts


def test_unequal_batch_equals_each_alone():
    cfg = make_cfg(MIXED)
    model, w = build(cfg, seed=1)
    lens = [1, 37, 9, 22]
    seqs = [tokens_of(n, cfg["vocab"], seed=i) for i, n in enumerate(lens)]
    alone = [engine_logits(model, [s], [[len(s)]])[0] for s in seqs]
    # prompts of unequal lengths in one step (all but the last 4 tokens), then decoded together; shorter ones end earlier
    cuts = [[max(1, n - 4)] + [1] * (n - max(1, n - 4)) for n in lens]
    together = engine_logits(model, seqs, cuts, max_seq=40)
    for a, b in zip(alone, together):
        assert rel_err(b, a).max() < SAME
    assert rel_err(alone[1], orc.forward(cfg, w, seqs[1])).max() < TOL32


def test_slots_freed_reused_and_grown():
    from generate.batch import BatchEngine

    cfg = make_cfg(MIXED)
    model, w = build(cfg, seed=2)
    a, b, c, d = (tokens_of(n, cfg["vocab"], seed=10 + n) for n in (33, 12, 27, 18))
    ref = {id(s): engine_logits(model, [s], [[len(s)]])[0] for s in (a, b, c, d)}
    eng = BatchEngine(model, max_seq_length=40, slots=1)
    # a fills slot 0 with a long sequence and ends; b takes the same slot and must not see what a left
    got_a = engine_logits(model, [a], [[20, 13]], engine=eng)[0]
    got_b = engine_logits(model, [b], [[5] + [1] * 7], engine=eng)[0]
    assert eng.pool.size == 1
    assert rel_err(got_a, ref[id(a)]).max() < SAME and rel_err(got_b, ref[id(b)]).max() < SAME
    # three at once: the caches grow while c is in flight
    lg_c0 = eng.step([("c", c[:10], list(range(10)))])
    both = eng.step([("c", c[10:], list(range(17))), ("d", d, list(range(18))), ("a", a, list(range(33)))],
                    end=["c", "d", "a"])
    got_c = torch.cat([lg_c0.cpu(), both[:17].cpu()])
    assert model.slots >= 3
    assert rel_err(got_c, ref[id(c)]).max() < SAME
    assert rel_err(both[17:35], ref[id(d)]).max() < SAME
    assert rel_err(both[35:], ref[id(a)]).max() < SAME


def test_first_token_alone_and_long_decoding():
    cfg = make_cfg([(delta(), None), (pair(every=64), moe()), (delta(heads=2, kv_heads=1, dim=16, vdim=8), None)])
    model, w = build(cfg, seed=4, edit=slow_state)
    n = 300
    toks = tokens_of(n, cfg["vocab"], seed=8)
    whole = engine_logits(model, [toks], [[n]])[0]
    single = engine_logits(model, [toks], [[1] * n])[0]
    assert rel_err(single, whole).max() < SAME
    short = orc.forward(cfg, w, toks[:70])
    assert rel_err(single[:70], short).max() < TOL32
    first = engine_logits(model, [toks[:1]], [[1]])[0]
    assert rel_err(first, short[:1]).max() < TOL32


def test_positions_are_bounded_by_the_table():
    cfg = make_cfg(MIXED[:1], positions=12)
    model, _ = build(cfg)
    from generate.batch import BatchEngine

    eng = BatchEngine(model, max_seq_length=64)
    assert model.max_seq_length == 12
    with pytest.raises(ValueError):
        eng.step([("a", tokens_of(13, cfg["vocab"]), [])])


# ------------------------------------------------------------------------------------------------ crafted attention
def plain_sinkattn(q, k, v, pos_q, scale, sink, post, group):
    """q (n, H, d) prepared queries at positions pos_q of one sequence whose cache holds k (S, G, d), v (S, G, dv)."""
    n, H = q.shape[:2]
    out = torch.zeros(n, H, v.shape[-1], dtype=torch.float64)
    for i in range(n):
        p = pos_q[i]
        for h in range(H):
            g = h // group
            s = (k[: p + 1, g].double() @ q[i, h].double()) * scale
            if sink is not None:
                s = torch.cat([s, sink[h].double().view(1)])
            a = torch.softmax(s, 0)
            out[i, h] = a[: p + 1] @ v[: p + 1, g].double() * post
    return out.reshape(n, -1)


@pytest.mark.parametrize("cache_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("S,with_sink", [(700, True), (300, False), (257, True)])
def test_attention_far_keys_and_the_sink(S, with_sink, cache_dtype):
    """One key per probe is made to dominate (its value is then the head's output): the sequence's first key, a key
    far back, keys 255 / 256 rows back (a key-tile border), the key before the query and the query's own; one head's
    sink is made as large as the dominating score, so that leaving it out would double the output. Prompt rows
    (16-query tiles) and one-token steps, also split over the keys."""
    from lit_gpt import seq_ops
    from lit_gpt.mixers import StepBatch

    dev = torch.device("cuda", 0)
    H, G, d, dv = 4, 2, 16, 24
    g = torch.Generator().manual_seed(S)
    k = torch.randn(S, G, d, generator=g) * 0.3
    v = torch.randn(S, G, dv, generator=g)
    nq = 37
    p0 = S - nq
    q = torch.randn(nq, H, d, generator=g) * 0.3
    pos_q = list(range(p0, S))
    for i in range(nq):  # query i's head i % H points at one chosen key
        p = pos_q[i]
        target = [0, 1, max(0, p - 256), max(0, p - 255), p, p - 1, p // 2][i % 7]
        gsel = (i % H) // (H // G)
        q[i, i % H] = 25.0 * k[target, gsel] / k[target, gsel].norm() ** 2
    sink = torch.tensor([25.0, -3.0, 0.5, 24.0]) if with_sink else None
    if cache_dtype == torch.bfloat16:
        k, v = k.bfloat16().float(), v.bfloat16().float()
    want = plain_sinkattn(q, k, v, pos_q, 1.0, sink, 0.8, H // G)
    ck = torch.zeros(2, S, G, d, dtype=cache_dtype, device=dev)
    cv = torch.zeros(2, S, G, dv, dtype=cache_dtype, device=dev)
    ck[1] = k.to(dev, cache_dtype)
    cv[1] = v.to(dev, cache_dtype)
    ck[0].fill_(7.0)  # another sequence's slot: never read
    kw = dict(H=H, G=G, d=d, dv=dv, scale=1.0, post=0.8)
    sk = None if sink is None else sink.to(dev)
    proj = q.reshape(nq, -1).to(dev).contiguous()
    step = StepBatch.build([(1, p0, [0] * nq)], dev)
    got = seq_ops.sinkattn(proj, 0, ck, cv, sk, step.seq_start, step.seq_slot, step.seq_pos0, nq, **kw)
    assert (got.double().cpu() - want).abs().max() < 2e-4
    for i in (0, 1, 2, 3, 4, 5, nq - 1):  # one-token steps, whole and split over the keys
        one = StepBatch.build([(1, pos_q[i], [0])], dev)
        for splits in (1, 3, None):
            got = seq_ops.sinkattn(proj[i:i + 1].contiguous(), 0, ck, cv, sk, one.seq_start, one.seq_slot, one.seq_pos0,
                                   1, splits=splits, **kw)
            assert (got.double().cpu() - want[i]).abs().max() < 2e-4, (i, splits)


def test_query_temperature_steps_with_the_position():
    """Unit-RMS queries and keys, then the temperature: it changes exactly where floor((p + 1) / every) does."""
    from lit_gpt import seq_ops

    dev = torch.device("cuda", 0)
    H, G, d, dv, every, coef = 2, 1, 8, 4, 4, 0.9
    g = torch.Generator().manual_seed(5)
    T = 14
    proj = torch.randn(T, H * d + G * d + G * dv, generator=g)
    ck = torch.zeros(1, 20, G, d, device=dev)
    cv = torch.zeros(1, 20, G, dv, device=dev)
    pd = proj.to(dev)
    pos = torch.arange(3, 3 + T, dtype=torch.int32, device=dev)
    seq_ops.normattn_prepare(pd, 0, H * d, H * d + G * d, ck, cv, torch.zeros(T, dtype=torch.int32, device=dev), pos, H=H,
                             G=G, d=d, dv=dv, eps=1e-5, temp_coef=coef, temp_every=every)
    import math
    for t in range(T):
        p = 3 + t
        temp = 1.0 + coef * math.log((p + 1) // every + 1)
        qn = orc.rms_unit(proj[t, :H * d].view(H, d).double(), 1e-5) * temp
        kn = orc.rms_unit(proj[t, H * d:H * d + G * d].view(G, d).double(), 1e-5)
        assert (pd[t, :H * d].cpu().double().view(H, d) - qn).abs().max() < 1e-5
        assert (ck[0, p].cpu().double() - kn).abs().max() < 1e-5
        assert torch.equal(cv[0, p].cpu().reshape(-1), proj[t, H * d + G * d:])
    assert float(ck[0, :3].abs().max()) == 0.0 and float(ck[0, 3 + T:].abs().max()) == 0.0


# ------------------------------------------------------------------------------------------------ crafted delta rule
@pytest.mark.parametrize("per_channel", [True, False])
@pytest.mark.parametrize("H,G,d,dv,lanes", [(2, 1, 5, 3, 0), (4, 2, 8, 16, 4), (2, 2, 20, 70, 8), (3, 1, 64, 64, 16),
                                            (1, 1, 72, 8, 0), (2, 1, 130, 24, 0), (1, 1, 260, 17, 0), (1, 1, 512, 5, 0),
                                            (2, 2, 128, 40, 4), (2, 2, 128, 40, 8), (2, 2, 128, 40, 16)])
def test_delta_rule_kernel_every_form(H, G, d, dv, lanes, per_channel):
    """lgs_gated_delta against float64 for sequences of 1 ... 90 tokens in one packed batch: started at position 0
    over a stale slot, or continued from a stored state; every lanes-per-column form and row count per lane."""
    from lit_gpt import seq_ops
    from lit_gpt.mixers import StepBatch

    dev = torch.device("cuda", 0)
    g = torch.Generator().manual_seed(d * 7 + dv)
    lens, first = [1, 90, 17, 33], [0, 5, 0, 40]
    slots = [3, 0, 2, 1]
    state = torch.randn(5, H, d, dv, generator=g)
    step = StepBatch.build([(s, p, [0] * n) for s, p, n in zip(slots, first, lens)], dev)
    T = sum(lens)
    unit = lambda x: x / x.norm(dim=-1, keepdim=True)  # noqa: E731
    q = unit(torch.randn(T, G, d, generator=g)) * d ** -0.5
    k = unit(torch.randn(T, G, d, generator=g))
    v = torch.randn(T, H, dv, generator=g)
    beta = torch.rand(T, H, generator=g)
    dec = torch.rand(T, H, d if per_channel else 1, generator=g) * 0.5 + 0.5
    qkv = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], 1).contiguous()
    sd = state.to(dev)
    kq = (q * k).sum(-1)
    got = seq_ops.gated_delta(qkv.to(dev), dec.reshape(T, -1).contiguous().to(dev), beta.to(dev), kq.to(dev), sd, step.seq_start,
                              step.seq_slot, step.seq_pos0, H=H, G=G, d=d, dv=dv, per_channel=per_channel, lanes=lanes)
    at = 0
    for s, p, n in zip(slots, first, lens):
        for h in range(H):
            S = state[s, h].double() if p > 0 else torch.zeros(d, dv, dtype=torch.float64)
            kv = h // (H // G)
            for t in range(at, at + n):
                S = dec[t, h].double().expand(d)[:, None] * S
                u = beta[t, h].double() * (v[t, h].double() - S.T @ k[t, kv].double())
                S = S + torch.outer(k[t, kv].double(), u)
                o = S.T @ q[t, kv].double()
                assert (got[t, h * dv:(h + 1) * dv].double().cpu() - o).abs().max() < 2e-5 * max(1.0, float(o.abs().max()))
            assert (sd[s, h].double().cpu() - S).abs().max() < 2e-5 * max(1.0, float(S.abs().max()))
        at += n
    assert torch.equal(sd[4].cpu(), state[4])  # a slot no sequence owns is left alone


def test_delta_prepare():
    from lit_gpt import seq_ops

    dev = torch.device("cuda", 0)
    H, G, d, T = 4, 2, 10, 6
    g = torch.Generator().manual_seed(2)
    qkv = torch.randn(T, 2 * G * d + 7, generator=g)
    a = torch.randn(T, 3 + H * d, generator=g) * 3
    b = torch.randn(T, H + 2, generator=g)
    A_log, bias = torch.randn(H, generator=g), torch.randn(H * d, generator=g)
    qd = qkv.to(dev)
    dec, beta, kq = seq_ops.delta_prepare(qd, a.to(dev), 3, b.to(dev), 2, A_log.to(dev), bias.to(dev), H=H, G=G, d=d,
                                          per_channel=True, q_scale=0.25)
    x = qkv[:, :2 * G * d].double().view(T, 2 * G, d)
    want = x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)
    want[:, :G] *= 0.25
    assert (qd[:, :2 * G * d].cpu().double().view(T, 2 * G, d) - want).abs().max() < 1e-6
    assert torch.equal(qd[:, 2 * G * d:].cpu(), qkv[:, 2 * G * d:])
    assert (kq.cpu().double() - (want[:, :G] * want[:, G:]).sum(-1)).abs().max() < 1e-6
    wd = torch.exp(-torch.exp(A_log.double())[None, :, None] * orc.softplus(a[:, 3:].double() + bias.double()).view(T, H, d))
    assert (dec.cpu().double().view(T, H, d) - wd).abs().max() < 1e-6
    assert (beta.cpu().double() - torch.sigmoid(b[:, 2:].double())).abs().max() < 1e-6
    dec1, _, _ = seq_ops.delta_prepare(qkv.to(dev), a.to(dev), 1, b.to(dev), 0, A_log.to(dev), bias[:H].contiguous().to(dev),
                                    H=H, G=G, d=d, per_channel=False, q_scale=1.0)
    w1 = torch.exp(-torch.exp(A_log.double()) * orc.softplus(a[:, 1:1 + H].double() + bias[:H].double()))
    assert (dec1.cpu().double() - w1).abs().max() < 1e-6


@pytest.mark.parametrize("per_channel,taps", [(True, 4), (False, 1), (True, 2), (False, 7)])
def test_one_token_step_form_equals_the_separate_launches(per_channel, taps):
    """Convolution + preparation in one launch (with the low-rank second map inside) against conv_silu, the product
    and delta_prepare, over steps that start one sequence over a stale history and continue two others; and the
    low-rank gate inside the head gate against the product followed by the plain head gate."""
    from lit_gpt import seq_ops
    from lit_gpt.mixers import StepBatch

    dev = torch.device("cuda", 0)
    H, G, d, dv, rank = 4, 2, 6, 5, 3
    C, n = 2 * G * d + H * dv, H * d if per_channel else H
    g = torch.Generator().manual_seed(taps)
    conv_w = torch.randn(C, taps, generator=g).to(dev)
    w_a2 = torch.randn(n, rank, generator=g).to(dev) if per_channel else None
    A_log, bias = torch.randn(H, generator=g).to(dev), torch.randn(n, generator=g).to(dev)
    hist = max(1, taps - 1)
    st_a = torch.randn(4, hist, C, generator=g).to(dev)
    st_b = st_a.clone()
    acols = rank if per_channel else H
    ld = C + 3 + acols + H
    pos = {0: 5, 2: 0, 3: 9}  # slot -> position: slot 2 starts a sequence over what the slot still holds
    for it in range(3):
        proj = torch.randn(3, ld, generator=g).to(dev)
        step = StepBatch.build([(s, p, [0]) for s, p in pos.items()], dev)
        kw = dict(H=H, G=G, d=d, per_channel=per_channel, q_scale=0.4)
        qkv1, dec1, beta1, kq1 = seq_ops.delta_step_prepare(proj, 0, conv_w, st_a, step.seq_slot, step.seq_pos0, C + 3,
                                                            C + 3 + acols, A_log, bias, dv=dv, w_a2=w_a2, **kw)
        qkv2 = seq_ops.conv_silu(proj, 0, conv_w, torch.zeros(C, device=dev), st_b, step.seq_start, step.seq_slot,
                                 step.seq_pos0, 1)
        if per_channel:
            a = torch.empty(3, n, device=dev)
            seq_ops.linear(proj, w_a2, M=3, N=n, K=rank, y=a, a_off=C + 3, lda=ld, ldy=n)
            dec2, beta2, kq2 = seq_ops.delta_prepare(qkv2, a, 0, proj, C + 3 + acols, A_log, bias, **kw)
        else:
            dec2, beta2, kq2 = seq_ops.delta_prepare(qkv2, proj, C + 3, proj, C + 3 + acols, A_log, bias, **kw)
        for name, x, y in (("qkv", qkv1, qkv2), ("dec", dec1, dec2), ("beta", beta1, beta2), ("kq", kq1, kq2)):
            assert (x - y).abs().max() < 1e-5, (it, name, (x - y).abs().max(1).values.tolist())
        assert float((st_a - st_b).abs().max()) == 0.0, it
        pos = {s: p + 1 for s, p in pos.items()}
    o = torch.randn(3, H * dv, generator=g).to(dev)
    w_g2 = torch.randn(H * dv, rank, generator=g).to(dev)
    nw = torch.randn(dv, generator=g).to(dev)
    gate = torch.empty(3, H * dv, device=dev)
    seq_ops.linear(proj, w_g2, M=3, N=H * dv, K=rank, y=gate, a_off=2, lda=ld, ldy=H * dv)
    kw = dict(H=H, dv=dv, unit_norm=True, eps=1e-5, act=seq_ops.ACT_SIGMOID, weight=nw, post=0.7)
    want = seq_ops.head_gate(o.clone(), gate, 0, **kw)
    got = seq_ops.head_gate(o.clone(), proj, 2, w_g2=w_g2, **kw)
    assert (got - want).abs().max() < 1e-5


def test_router_in_one_launch_equals_product_then_routing():
    from lit_gpt import seq_ops

    dev = torch.device("cuda", 0)
    g = torch.Generator().manual_seed(8)
    for E, K, top, dtype in ((5, 40, 3, torch.float32), (70, 33, 4, torch.float32), (18, 64, 4, torch.bfloat16)):
        w = torch.randn(E, K, generator=g).to(dev, dtype)
        h = torch.randn(6, K, generator=g).to(dev)
        corr = (torch.randn(E, generator=g) * 0.05).to(dev)
        z = torch.empty(6, E, device=dev)
        seq_ops.linear(h, w, M=6, N=E, K=K, y=z, lda=K, ldy=E)
        ids2, wts2 = seq_ops.moe_route_scores(z, 0, E, top, corr)
        ids1, wts1 = seq_ops.moe_router(h, w, top, corr)
        assert torch.equal(ids1, ids2) and (wts1 - wts2).abs().max() < 1e-5


@pytest.mark.parametrize("schedule", ["whole", "portions", "single", "stale"])
def test_state_carries_an_early_token(schedule):
    """With decay 1 (and beta one half) the memory keeps what the first tokens wrote for the whole sequence, so every
    late position depends on them. Losing the state at a step's edge, or starting from a stale slot, shows."""
    def edit(w):
        slow_state(w)
        for name in w:
            if name.endswith("mix.b"):
                w[name] = torch.zeros_like(w[name])
    cfg = make_cfg([(delta(heads=2, kv_heads=1, dim=8, vdim=8), None)])
    model, w = build(cfg, seed=12, edit=edit)
    n = 150
    toks = tokens_of(n, cfg["vocab"], seed=4)
    want = orc.forward(cfg, w, toks)
    from generate.batch import BatchEngine
    eng = BatchEngine(model, max_seq_length=n, slots=1)
    if schedule == "stale":  # another sequence leaves its state in the slot first
        engine_logits(model, [tokens_of(40, cfg["vocab"], seed=9)], [[40]], engine=eng)
    cuts = {"whole": [n], "portions": portions(n, 17), "single": [1] * n, "stale": [100] + [1] * 50}[schedule]
    got = engine_logits(model, [toks], [cuts], engine=eng)[0]
    assert rel_err(got, want).max() < TOL32


# ------------------------------------------------------------------------------------------------ routing
def test_routing_scores_correction_and_identity():
    """The choice adds the correction, the weights do not; weights are not renormalised; equal scores go to the lowest
    index; identity experts return the input."""
    from lit_gpt import seq_ops

    dev = torch.device("cuda", 0)
    z = torch.tensor([[2.0, 1.0, 0.0, -1.0, 0.5, 0.5], [0.0, 0.0, 0.0, 0.0, 0.0, 0.0], [3.0, -2.0, 1.0, 1.0, 0.2, 0.1]])
    corr = torch.tensor([-5.0, 0.0, 0.0, 5.0, 0.0, 0.0])
    proj = torch.cat([torch.zeros(3, 8), z], 1).contiguous().to(dev)
    ids, wts = seq_ops.moe_route_scores(proj, 8, 6, 3, corr.to(dev))
    s = torch.softmax(z.double(), -1)
    assert ids.cpu().tolist() == [[3, 1, 4], [3, 1, 2], [3, 2, 4]]
    for t in range(3):
        assert (wts[t].cpu().double() - s[t][ids[t].cpu().long()]).abs().max() < 1e-6
    ids2, wts2 = seq_ops.moe_route_scores(proj, 8, 6, 2, None)
    assert ids2.cpu().tolist() == [[0, 1], [0, 1], [0, 2]]
    assert float(wts2.sum(1).max()) < 1.0  # not renormalised


def test_both_expert_forms_agree_and_identity_counts():
    """The streaming form (few pairs) and the sorted grouped form (many) of the same layer, rows compared one by one;
    a router that always picks an identity expert returns weight * input for it."""
    from lit_gpt import mixers as mx
    from lit_gpt.config import FeedForwardSpec

    dev = torch.device("cuda", 0)
    W, E, I, F, top = 24, 3, 2, 10, 3
    g = torch.Generator().manual_seed(3)
    w = {"router": torch.randn(E + I, W, generator=g), "correction": torch.tensor([0.0, 0.0, 0.0, 9.0, 0.0])}
    for e in range(E):
        w.update({f"e{e}.gate": torch.randn(F, W, generator=g) * 0.3, f"e{e}.up": torch.randn(F, W, generator=g) * 0.3,
                  f"e{e}.down": torch.randn(W, F, generator=g) * 0.3})
    ff = mx.SparseFeedForward(FeedForwardSpec("moe", F, E, top, identity=I), W, w, dev, torch.float32, route="scores")
    ff.bind({"router": 0})
    T = 40
    h = torch.randn(T, W, generator=g)
    want = orc.moe_ff(h.double(), {k: v.double() for k, v in w.items()}, {"router": {"experts": E, "top": top}})
    hd = h.to(dev)
    from lit_gpt import seq_ops
    proj = torch.empty(T, E + I, device=dev)
    seq_ops.linear(hd, w["router"].to(dev), M=T, N=E + I, K=W, y=proj, lda=W, ldy=E + I)
    big = torch.empty(T, W, device=dev)
    ff(proj, hd, big, accumulate=False)
    assert (big.cpu().double() - want).abs().max() < 1e-4
    small = torch.full((5, W), 3.0, device=dev)
    ff(proj[:5].contiguous(), hd[:5].contiguous(), small, accumulate=True)
    assert (small.cpu().double() - 3.0 - want[:5]).abs().max() < 1e-4


# ------------------------------------------------------------------------------------------------ entry points
def follows_plain_greedy(cfg, w, prompt, out):
    """Every continued token is the plain implementation's argmax wherever that has a clear margin."""
    lg = orc.forward(cfg, w, out[:-1])
    clear = [i for i in range(len(prompt) - 1, len(out) - 1) if float(torch.topk(lg[i], 2).values.diff().abs()) > 1e-3]
    return bool(clear) and all(out[i + 1] == int(lg[i].argmax()) for i in clear)


def test_greedy_generation_through_the_entry_points():
    from generate.base import generate
    from generate.batch import BatchEngine

    cfg = make_cfg(MIXED[:3])
    model, w = build(cfg, seed=7)
    prompts = [tokens_of(9, cfg["vocab"], seed=1), tokens_of(4, cfg["vocab"], seed=2), tokens_of(15, cfg["vocab"], seed=3)]
    new = 8
    eng = BatchEngine(model, max_seq_length=24)
    batched = eng.generate(prompts, new)
    assert not eng.live
    for p, out in zip(prompts, batched):
        assert out[:len(p)] == p and len(out) == len(p) + new
        assert follows_plain_greedy(cfg, w, p, out)
    assert BatchEngine(model, max_seq_length=24).generate(prompts, new, use_graph=True) == batched
    model.set_kv_cache(1, 24)
    single = generate(model, torch.tensor(prompts[0], dtype=torch.int32, device="cuda"), len(prompts[0]) + new,
                      temperature=0.0).cpu().tolist()
    assert single == batched[0]
    sampled = BatchEngine(model, max_seq_length=24).generate(prompts, 3, temperature=0.8, top_k=5)
    assert [len(o) for o in sampled] == [len(p) + 3 for p in prompts]


def test_captured_decode_step_replays():
    """One-token steps as replays of one HIP graph, every replay against the eager step, with eager work between."""
    from generate.batch import BatchEngine

    cfg = make_cfg(MIXED)
    model, _ = build(cfg, seed=21)
    prompts = [tokens_of(11, cfg["vocab"], seed=4), tokens_of(3, cfg["vocab"], seed=5)]
    eager = BatchEngine(model, max_seq_length=40).generate(prompts, 12)
    eng = BatchEngine(model, max_seq_length=40)
    ids = ["a", "b"]
    lg = eng.step([(ids[i], p, [len(p) - 1]) for i, p in enumerate(prompts)])
    first = [int(lg[i].argmax()) for i in range(2)]
    graph = eng.decode_graph(ids, first)
    outs = [list(p) + [first[i]] for i, p in enumerate(prompts)]
    for n in range(11):
        drawn = graph.step().cpu().tolist()
        torch.cuda.synchronize()
        (torch.randn(64, 64, device="cuda") @ torch.randn(64, 64, device="cuda")).sum().item()  # other eager work
        for i in range(2):
            outs[i].append(drawn[i])
    assert outs == eager


def test_command_line_serves_a_checkpoint_folder(tmp_path, capsys):
    import json

    from safetensors.torch import save_file

    from generate.base import main
    from lit_gpt.config import LayeredConfig
    from lit_gpt.layered import LayeredGPT

    cfg = make_cfg(MIXED[:3], vocab=70)
    w = LayeredGPT.random_weights(LayeredConfig.from_dict(cfg), seed=15)
    save_file({k: v.contiguous() for k, v in w.items()}, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    main(checkpoint_dir=tmp_path, max_new_tokens=5, temperature=0.0, top_k=None, prompt_len=7, precision="32-true")
    ids = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert len(ids) == 12
    assert follows_plain_greedy(cfg, w, ids[:7], ids)


def test_checkpoint_folder_through_registry_and_runner(tmp_path):
    import json
    import subprocess
    import sys

    import numpy as np
    from safetensors.torch import save_file

    from lit_gpt.config import LayeredConfig, load_config, model_class
    from lit_gpt.layered import LayeredGPT

    REPO = Path(__file__).resolve().parent.parent
    cfg = make_cfg(MIXED)
    weights = LayeredGPT.random_weights(LayeredConfig.from_dict(cfg), seed=11)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in weights.items()}, str(tmp_path / "model.safetensors"))
    config = load_config(tmp_path)
    assert model_class(config) is LayeredGPT
    a, b = tokens_of(14, cfg["vocab"], seed=1), tokens_of(6, cfg["vocab"], seed=2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:10], "want": [3, 9]}, {"id": "b", "tokens": b[:5], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[10:11], "want": [0]}, {"id": "b", "tokens": b[5:], "want": [0]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[11:12], "want": []}], "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": a[12:], "want": [1]}], "end": ["a"]}]
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, str(REPO / "bin" / "trace_run"), "--model", str(tmp_path), "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "32"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.split("\n") if l.startswith("done")] == [f"done {i}" for i in range(4)]
    wa, wb = orc.forward(cfg, weights, a), orc.forward(cfg, weights, b)
    V = cfg["vocab"]
    got0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, V))
    got1 = torch.from_numpy(np.fromfile(out / "1.f32", dtype="<f4").reshape(-1, V))
    got3 = torch.from_numpy(np.fromfile(out / "3.f32", dtype="<f4").reshape(-1, V))
    assert not (out / "2.f32").exists()
    assert rel_err(got0, wa[[3, 9]]).max() < TOL32
    assert rel_err(got1, torch.stack([wa[10], wb[5]])).max() < TOL32
    assert rel_err(got3, wa[13:14]).max() < TOL32


def test_two_streams_equal_one():
    """The parallel mixer's branches on two streams against the same steps on one stream, bit for bit, over prompts,
    portions and a batch (the second stream's kernels read only what was made before the fork)."""
    from lit_gpt.mixers import ParallelMixer

    cfg = make_cfg(MIXED)
    model, _ = build(cfg, seed=13)
    seqs = [tokens_of(n, cfg["vocab"], seed=20 + n) for n in (70, 33, 12)]
    cuts = [[40, 30], [33], [0, 12]]
    assert ParallelMixer.overlap
    two = engine_logits(model, seqs, cuts, max_seq=80)
    try:
        ParallelMixer.overlap = False
        one = engine_logits(model, seqs, cuts, max_seq=80)
    finally:
        ParallelMixer.overlap = True
    for a, b in zip(one, two):
        assert torch.equal(a, b)
