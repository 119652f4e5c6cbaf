"""Ronavik decoder: the framework (model registry -> LLMEngine -> native scheduler -> ops) against the slow float64 oracle
in tests/ronavik_oracle.py. Small made-up configurations and random weights; strong position vectors, query temperatures
that step every few tokens, sizeable biases and gate matrices, so that a key that is one token off, a lost state, a
missing bias or temperature, a wrong head / group mapping, a wrong expert or a wrong page moves the logits far beyond
the tolerance. CPU runs use the reference ops, GPU runs the HIP kernels (fp32: tight tolerance; bf16: rounding level).
"""
import json
import math
import os

import pytest
import torch

from generativeaiexamples_amd import ops
from generativeaiexamples_amd.engine import EngineConfig, LLMEngine, SamplingParams
from generativeaiexamples_amd.models.registry import build_llm
from generativeaiexamples_amd.models.ronavik import RonavikConfig, RonavikModel

from . import ronavik_oracle as O

_GPU = pytest.mark.gpu
TARGETS = [pytest.param("cpu", torch.float32, id="cpu-fp32"),
           pytest.param("cuda", torch.float32, id="gpu-fp32", marks=_GPU),
           pytest.param("cuda", torch.bfloat16, id="gpu-bf16", marks=_GPU)]
FP32_TARGETS = TARGETS[:2]


def row_err(got, want):
    """RMS of the difference (mean over the vocabulary taken off) over the RMS of the centred reference, per row."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    w = want.double() - want.double().mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-9)


def rel_err(got, want):
    return row_err(got, want).max().item()


def close(got, want, dtype):
    """fp32: every row within 2e-4. bf16: rounding level - rows within 4 % on average and no row beyond 15 %; a wrong
    mechanism is off by tens of percent on most rows."""
    e = row_err(got, want)
    if dtype == torch.float32:
        return e.max().item() < 2e-4
    return e.mean().item() < 4e-2 and e.max().item() < 0.15


def make_engine(cfg, sd, device, dtype, max_tokens=512, max_seqs=4, graphs=None):
    model = RonavikModel(RonavikConfig.from_json(cfg), device=device, dtype=dtype).load_state(sd)
    from generativeaiexamples_amd.engine.tokenizer import load_tokenizer
    graphs = (device != "cpu") if graphs is None else graphs
    return LLMEngine(model, load_tokenizer(None, "llama3", cfg["vocab"]), EngineConfig(
        max_num_seqs=max_seqs, num_blocks=max_tokens // ops.BLOCK, max_model_len=max_tokens, max_batched_tokens=1 << 20,
        use_graphs=graphs, graph_batch_sizes=(1, 2, 4), decode_steps=1))


def run_schedule(eng, prompts, schedule):
    """schedule: list of steps, each a list of (request name, count). Returns {name: logits [len, vocab]} with every
    position's logits; requests end when their tokens are used up."""
    at = {n: 0 for n in prompts}
    got = {n: [] for n in prompts}
    for step in schedule:
        entries, end = [], []
        for name, count in step:
            lo = at[name]
            entries.append((name, prompts[name][lo:lo + count], list(range(count))))
            at[name] = lo + count
            if at[name] == len(prompts[name]):
                end.append(name)
        out = eng.replay_step(entries, end)
        r = 0
        for name, count in step:
            got[name].append(out[r:r + count])
            r += count
    return {n: torch.cat(v) for n, v in got.items() if v}


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def config_for(dtype, layers, **kw):
    """The test's configuration. An expert choice is a discrete decision: with random weights some position always has
    two router scores closer than bf16 rounding of the router's input, and the other expert's output is a different
    vector altogether. So bf16 runs take every expert (top = experts: the same expert kernels, no decision), and the
    choice itself is tested in fp32 (CPU and GPU), on prompts without a near-tie (clear_tokens)."""
    if dtype == torch.bfloat16:
        layers = [l if l.get("mlp") is None else
                  dict(l, mlp=dict(l["mlp"], router=dict(l["mlp"]["router"], top=min(8, l["mlp"]["router"]["experts"]),
                                                         experts=min(8, l["mlp"]["router"]["experts"])))) for l in layers]
    return O.make_config(layers, **kw)


def clear_tokens(n, cfg, sd, seed, gap=1e-4):
    """Random tokens whose router scores have no near-tie between the last chosen and the first rejected expert."""
    for s in range(seed, seed + 50):
        t = tokens(n, cfg["vocab"], s)
        if O.router_margin(cfg, sd, t) > gap:
            return t
    raise AssertionError("no clear-cut prompt found")


def cuts(n, sizes):
    out, i = [], 0
    while n > 0:
        c = min(n, sizes[i % len(sizes)])
        out.append(c)
        n -= c
        i += 1
    return out


FULL = [O.with_mlp(O.ssm()), O.with_mlp(O.par()), O.with_mlp(O.par(kv_heads=4, blocks=1, conv=2), None),
        O.with_mlp(O.ssm(groups=1, norm_groups=1, conv=2), top=1), O.with_mlp(O.par(kv_heads=1, q_temp=(0.3, 7)), top=3)]


# ------------------------------------------------------------------------------------------------ each mechanism alone
@pytest.mark.parametrize("device,dtype", TARGETS)
@pytest.mark.parametrize("layer", [
    O.with_mlp(O.par(), None), O.with_mlp(O.par(dim=12, vdim=20, heads=6, kv_heads=1, q_temp=(0.9, 3)), None),
    O.with_mlp(O.par(heads=1, kv_heads=1, q_temp=None, width=8, blocks=1, conv=1, left_scale=1.0, right_scale=1.0), None),
    O.with_mlp(O.par(dim=16, vdim=16, heads=2, kv_heads=2, width=40, blocks=5, conv=5, q_temp=(0.2, 1)), None),
    O.with_mlp(O.ssm(), None), O.with_mlp(O.ssm(heads=6, vdim=4, state=20, groups=3, norm_groups=2, conv=3), None),
    O.with_mlp(O.ssm(heads=1, vdim=16, state=8, groups=1, norm_groups=1, conv=1), None),
    O.with_mlp(O.ssm(heads=2, vdim=12, state=70, groups=2, norm_groups=8, conv=2), None),
    O.with_mlp(O.ssm(), ff=40, experts=6, top=1), O.with_mlp(O.par(), ff=20, experts=3, top=3),
    O.with_mlp(O.ssm(), ff=72, experts=9, top=4)],
    ids=["par", "par-gqa1-uneven", "par-1head-conv1", "par-mha-5blocks", "ssm", "ssm-3groups", "ssm-1head-conv1",
         "ssm-wide-state", "moe-top1", "moe-all", "moe-top4"])
def test_single_mechanism(layer, device, dtype):
    cfg = config_for(dtype, [layer], width=40)
    sd = O.random_checkpoint(cfg, 1)
    toks = clear_tokens(37, cfg, sd, 2)
    want = O.forward(cfg, sd, toks)
    eng = make_engine(cfg, sd, device, dtype)
    got = run_schedule(eng, {"a": toks}, [[("a", len(toks))]])["a"]
    assert close(got, want, dtype)


@pytest.mark.parametrize("device,dtype", FP32_TARGETS)
def test_ops_against_oracle_mechanisms(device, dtype):
    """Single ops against the oracle's functions: the post-norm gated residual, the gated group norm, the recurrence
    gates and scan, the sigmoid router with input-side weights."""
    g = torch.Generator().manual_seed(0)
    rn = lambda *s: torch.randn(*s, generator=g)  # noqa: E731
    dev = torch.device(device)
    # post-norm gated residual + the next opening norm
    res, y, gate, wp, wn = rn(5, 70), rn(5, 70), rn(5, 70), rn(70), rn(70)
    r = res.clone().to(dev)
    out = ops.gated_norm_add_f32(r, y.to(dev), gate.to(dev), wp.to(dev), 1e-5, wn.to(dev), torch.float32).cpu()
    x = res.double() + O.norm(y.double() * torch.sigmoid(gate.double()), wp.double(), 1e-5)
    assert torch.allclose(r.cpu().double(), x, atol=1e-5)
    assert torch.allclose(out.double(), O.norm(x, wn.double(), 1e-5), atol=1e-5)
    # gate before the norm, norm in groups
    yy, z, w = rn(6, 48), rn(6, 48), rn(48)
    got = ops.gate_group_norm(yy.to(dev), z.to(dev), w.to(dev), 4, 1e-5, torch.float32).cpu().double()
    gz = yy.double() * torch.nn.functional.silu(z.double())
    assert torch.allclose(got, O.rms_div(gz.reshape(6, 4, 12), 1e-5).reshape(6, 48) * w.double(), atol=1e-5)
    # recurrence of the gated linear unit from a state that is not zero
    W, nb, T = 30, 3, 9
    u, ya = rn(T, W), rn(T, W)
    wa, wi, ba, bi, lam = rn(nb, 10, 10), rn(nb, 10, 10), rn(W), rn(W), rn(W) - 2
    wa_t, wi_t = wa.transpose(1, 2).contiguous().to(dev), wi.transpose(1, 2).contiguous().to(dev)
    a, b = ops.rglru_gates(u.to(dev), wa_t, ba.to(dev), wi_t, bi.to(dev), lam.to(dev), 8.0)
    blocks = lambda w: torch.cat([u[:, 10 * i:10 * i + 10].double() @ w[i].double().T for i in range(nb)], 1)  # noqa: E731
    r_, i_ = torch.sigmoid(blocks(wa) + ba.double()), torch.sigmoid(blocks(wi) + bi.double())
    a_ = torch.exp(-8.0 * r_ * torch.nn.functional.softplus(lam.double()))
    assert torch.allclose(a.cpu().double(), a_, atol=1e-5)
    assert torch.allclose(b.cpu().double(), torch.sqrt(1 - a_ ** 2) * i_ * u.double(), atol=1e-5)
    state = torch.zeros(3, W)
    state[1] = rn(W)
    S = state[1].double()
    want = []
    for t in range(T):
        S = a_[t] * S + torch.sqrt(1 - a_[t] ** 2) * i_[t] * u[t].double()
        want.append(1.5 * S * O.gelu_tanh(ya[t].double()))
    st = state.clone().to(dev)
    cu, slots = torch.tensor([0, T], dtype=torch.int32, device=dev), torch.tensor([1], dtype=torch.int32, device=dev)
    got = ops.rglru_scan(a, b, ya.to(dev), st, cu, slots, torch.float32, act="gelu_tanh", out_scale=1.5).cpu().double()
    assert torch.allclose(got, torch.stack(want), atol=1e-5) and torch.allclose(st[1].cpu().double(), S, atol=1e-5)
    assert st[0].abs().max() == 0 and st[2].abs().max() == 0
    # router: sigmoid scores, weights not renormalised, applied to the expert's input
    E, k, D, F_ = 6, 2, 24, 16
    h, wr = rn(7, D), rn(E, D)
    Wm = {"router": wr.double()}
    for e in range(E):
        Wm[f"e{e}.up"], Wm[f"e{e}.down"] = rn(F_, D).double(), rn(D, F_).double()
    want = O.moe(h.double(), Wm, "", dict(router=dict(experts=E, top=k)))
    ids, wts = ops.moe_route((h @ wr.T).to(dev), k, renorm=False, score="sigmoid")
    _, offs, pos = ops.moe_dispatch(ids, E)
    xs = ops.moe_scale_rows(h.to(dev), pos, wts)
    up = ops.moe_gemm(xs, None, torch.stack([Wm[f"e{e}.up"] for e in range(E)]).float().to(dev), offs, 7 * k, act="relu2")
    dn = ops.moe_gemm(up, None, torch.stack([Wm[f"e{e}.down"] for e in range(E)]).float().to(dev), offs, 7 * k)
    got = ops.moe_combine(dn, pos, None).cpu().double()
    assert torch.allclose(got, want, atol=1e-4, rtol=1e-4)


# ------------------------------------------------------------------------------------ whole model, schedules, batches
@pytest.mark.parametrize("device,dtype", TARGETS)
def test_prefill_decode_portions(device, dtype):
    """Whole prompt, token-by-token decoding from the first token on, and portions of 2 / 3 / 5 / 17 / 1 tokens: every
    position's logits equal the oracle's, so they do not depend on how the prompt was cut. The query temperature steps
    every 4 and every 7 tokens, inside and at the edges of portions."""
    cfg = config_for(dtype, FULL)
    sd = O.random_checkpoint(cfg, 3)
    toks = clear_tokens(61, cfg, sd, 4)
    want = O.forward(cfg, sd, toks)
    eng = make_engine(cfg, sd, device, dtype)
    for name, sizes in (("whole", [61]), ("decode", [1]), ("prefill+decode", [30] + [1] * 31), ("small", [2, 3, 5, 17, 1]),
                        ("twos", [2])):
        sched = [[(name, c)] for c in cuts(61, sizes)]
        got = run_schedule(eng, {name: toks}, sched)[name]
        assert close(got, want, dtype), name


@pytest.mark.parametrize("device,dtype", TARGETS)
def test_mixed_batches_and_reuse(device, dtype):
    """Unequal requests in one batch (portions beside single tokens) against each alone; a pool of two state slots and
    few pages, so slots and pages of finished requests are used again by later ones."""
    cfg = config_for(dtype, FULL[:4])
    sd = O.random_checkpoint(cfg, 5)
    lens = dict(a=45, b=18, c=33, d=1, e=26)
    prompts = {n: clear_tokens(L, cfg, sd, 10 + 50 * i) for i, (n, L) in enumerate(lens.items())}
    want = {n: O.forward(cfg, sd, t) for n, t in prompts.items()}
    eng = make_engine(cfg, sd, device, dtype, max_tokens=96, max_seqs=2)
    sched = [[("a", 20), ("b", 3)], [("a", 1), ("b", 15)],          # b ends: its slot and pages go back
             [("a", 1), ("c", 2)], [("c", 17), ("a", 5)], [("a", 1), ("c", 1)], [("a", 17), ("c", 13)],  # a, c end
             [("d", 1), ("e", 7)], [("e", 2)], [("e", 1)], [("e", 16)]]
    got = run_schedule(eng, prompts, sched)
    for n in prompts:
        assert close(got[n], want[n], dtype), n
    assert eng.sched.num_free_blocks() == 96 // ops.BLOCK and not eng.model.pool.slot_of


@pytest.mark.parametrize("device,dtype", TARGETS)
def test_first_tokens_and_long_decode(device, dtype):
    """Positions 0..4 of a sequence (zero-padded convolutions, zero states, one-key attention) and 150 single-token
    steps across many page borders and temperature steps."""
    cfg = config_for(dtype, [O.with_mlp(O.par(conv=4, q_temp=(0.4, 16))), O.with_mlp(O.ssm(conv=4), top=1),
                                 O.with_mlp(O.par(q_temp=(0.6, 5)), None)])
    sd = O.random_checkpoint(cfg, 7)
    toks = clear_tokens(155, cfg, sd, 8)
    want = O.forward(cfg, sd, toks)
    eng = make_engine(cfg, sd, device, dtype)
    got = run_schedule(eng, {"a": toks}, [[("a", 1)] for _ in toks])["a"]
    assert close(got[:5], want[:5], dtype)
    assert close(got, want, dtype)


@pytest.mark.parametrize("device,dtype", FP32_TARGETS)
def test_far_token_through_state(device, dtype):
    """Slowly forgetting recurrent layers (no attention): changing four tokens 300 positions back changes the last
    logits (oracle), and the framework follows it, through a prompt cut at odd places and single-token steps."""
    cfg = O.make_config([O.with_mlp(O.ssm(heads=2, vdim=8, state=8, groups=1, norm_groups=1), None),
                         O.with_mlp(O.par(dim=4, vdim=4, heads=1, kv_heads=1, left_scale=0.0, q_temp=None, width=16, blocks=2),
                                    None)], width=32, vocab=64)
    sd = O.random_checkpoint(cfg, 9, slow_decay=True)
    sd["pos"] = sd["pos"] * 0.0  # the far tokens reach the last position through the states only
    a = tokens(320, cfg["vocab"], 11)
    b = list(a)
    for i in (5, 6, 7, 8):
        b[i] = (b[i] + 13) % cfg["vocab"]
    wa, wb = O.forward(cfg, sd, a)[-1:], O.forward(cfg, sd, b)[-1:]
    assert rel_err(wb, wa) > 2e-3  # the far tokens matter
    eng = make_engine(cfg, sd, device, dtype)
    sched = lambda n: [[(n, c)] for c in cuts(320, [33, 2, 64, 1, 100])]  # noqa: E731
    got = run_schedule(eng, {"a": a, "b": b}, sched("a") + sched("b"))
    assert rel_err(got["a"][-1:], wa) < 2e-4 and rel_err(got["b"][-1:], wb) < 2e-4


def _attention_probe(device, dtype, n_ctx, hot, portion, dk=8, dv=16, query=-1, bias=-12.0):
    """ops-level: one head, keys of n_ctx positions through the paged cache (pages deliberately scattered). The sigmoid
    bias is so low that an ordinary key weighs nothing; the key at position `hot` is aligned with the query at
    `query` and scaled so that its weight is about one half. Returns that query's output: v[hot] / 2 if the key was
    seen, zero if not."""
    B = ops.BLOCK
    dev = torch.device(device)
    nb = (n_ctx + B - 1) // B
    pages = list(range(nb + 3))[::-1][:nb]  # not the identity
    kc = torch.zeros(nb + 4, 1, B, dk, dtype=dtype, device=dev)
    vc = torch.zeros(nb + 4, 1, dv, B, dtype=dtype, device=dev)
    g = torch.Generator().manual_seed(0)
    qi = query % n_ctx
    k = torch.randn(n_ctx, dk, generator=g)
    q_hot = torch.randn(dk, generator=g)
    qh = q_hot / q_hot.norm()
    k = k - torch.outer(k @ qh, qh)  # every other key is orthogonal to the probing query: score 0
    k[hot] = qh
    v = torch.zeros(n_ctx, dv)
    v[hot, 5] = 2.0
    q = torch.randn(n_ctx, dk, generator=g)
    q[qi] = qh
    ones = torch.ones(dk, device=dev)
    # unit-RMS rows after the per-head norm: |q| = |k| = sqrt(dk), so q.k = dk for the aligned pair; scale it to -bias
    scale = -bias / dk
    bt = torch.tensor([pages], dtype=torch.int32, device=dev)
    pb = torch.tensor([bias], device=dev)
    done, res = 0, None
    for c in cuts(n_ctx, portion):
        pos = torch.arange(done, done + c)
        slots = torch.tensor([pages[p // B] * B + p % B for p in pos.tolist()], dtype=torch.int32, device=dev)
        qn = ops.headnorm_kv_write(q[pos].to(dev, dtype), k[pos].to(dev, dtype), v[pos].to(dev, dtype), ones, ones, slots,
                                   kc, vc, 1, 1, dk, dv, 1e-12)
        cu = torch.tensor([0, c], dtype=torch.int32, device=dev)
        ctx = torch.tensor([done + c], dtype=torch.int32, device=dev)
        out = ops.sigmoid_attention(qn, kc, vc, bt, cu, ctx, 1, 1, dk, dv, scale, pb)
        if done <= qi < done + c:
            res = out[qi - done].float().cpu()
        done += c
    return res


@pytest.mark.parametrize("device,dtype", FP32_TARGETS)
@pytest.mark.parametrize("portion", [[1000], [1], [7, 2, 30]], ids=["prompt", "decode", "portions"])
def test_far_keys_page_borders_and_causal_edge(device, dtype, portion):
    """One key among hundreds carries the output (no softmax: a lost key is not renormalised away): at page borders,
    at the first position, far back; the key at the query's own position is seen, the one after it is not."""
    n = 330
    for hot in (0, 1, 15, 16, 17, 31, 32, 200, n - 2, n - 1):
        out = _attention_probe(device, dtype, n, hot, portion if portion != [1] else [300, 1])
        assert abs(out[5].item() - 1.0) < 1e-3 and out.abs().sum().item() < 1.01, (hot, out)
    for qi in (0, 5, 15, 16, 40):   # causal edge inside a portion: own position in, next position out
        p = portion if portion != [1] else [1]
        assert abs(_attention_probe(device, dtype, 70, qi, p, query=qi)[5].item() - 1.0) < 1e-3, qi
        assert _attention_probe(device, dtype, 70, qi + 1, p, query=qi).abs().max().item() < 1e-3, qi


@_GPU
@pytest.mark.parametrize("dk,dv", [(64, 64), (128, 64), (64, 128), (128, 128), (256, 256)])
def test_far_keys_matrix_core_kernel(dk, dv):
    """The same stand-out key probes on the bf16 query-tiled matrix-core kernel (head sizes it is built for, portions of
    8 rows and more), beside shorter portions that stay on the one-wave-per-row kernel."""
    n, dt = 330, torch.bfloat16
    for portion in ([1000], [170, 140, 9, 11], [220, 3, 107]):
        for hot in (0, 15, 16, 31, 32, 63, 64, 200, n - 1):
            out = _attention_probe("cuda", dt, n, hot, portion, dk, dv)
            assert abs(out[5].item() - 1.0) < 0.05 and out.abs().sum().item() < 1.1, (portion, hot, out)
        for qi in (0, 31, 32, 100):
            assert abs(_attention_probe("cuda", dt, 150, qi, portion, dk, dv, query=qi)[5].item() - 1.0) < 0.05, qi
            assert _attention_probe("cuda", dt, 150, qi + 1, portion, dk, dv, query=qi).abs().max().item() < 1e-2, qi


@_GPU
def test_matrix_core_attention_in_model():
    """bf16 model with 64- and 128-wide heads: portions of 8+ rows take the matrix-core attention kernel, shorter ones
    and decoded tokens the row kernel; both against the oracle, alone and in a mixed batch."""
    layers = [O.with_mlp(O.par(dim=64, vdim=64, heads=4, kv_heads=2, q_temp=(0.3, 32), width=64, blocks=2)),
              O.with_mlp(O.ssm(heads=4, vdim=16, state=16)),
              O.with_mlp(O.par(dim=128, vdim=64, heads=2, kv_heads=1, q_temp=(0.2, 50), width=128, blocks=1), top=1)]
    cfg = config_for(torch.bfloat16, layers, width=128, vocab=128)
    sd = O.random_checkpoint(cfg, 61)
    prompts = {"a": clear_tokens(150, cfg, sd, 62), "b": clear_tokens(90, cfg, sd, 163)}
    want = {n: O.forward(cfg, sd, t) for n, t in prompts.items()}
    eng = make_engine(cfg, sd, "cuda", torch.bfloat16)
    sched = [[("a", 70)], [("a", 33), ("b", 50)], [("a", 9), ("b", 1)], [("a", 1), ("b", 39)], [("a", 37)]]
    got = run_schedule(eng, prompts, sched)
    for n in prompts:
        assert close(got[n], want[n], torch.bfloat16), n


# ------------------------------------------------------------------------------------------- shapes of other models
@pytest.mark.parametrize("device,dtype", TARGETS)
@pytest.mark.parametrize("case", ["ssm-only", "par-only-no-ff", "tiny-odd", "wide-odd"])
def test_other_shapes(case, device, dtype):
    if case == "ssm-only":
        cfg = config_for(dtype, [O.with_mlp(O.ssm(), top=1),
                                 O.with_mlp(O.ssm(heads=2, vdim=12, state=5, groups=2, norm_groups=3))], width=24, eps=1e-3)
    elif case == "par-only-no-ff":
        cfg = config_for(dtype, [O.with_mlp(O.par(), None), O.with_mlp(O.par(kv_heads=4, q_temp=None), None)], width=16,
                         vocab=33)
    elif case == "tiny-odd":
        cfg = config_for(dtype, [O.with_mlp(O.par(dim=4, vdim=4, heads=1, kv_heads=1, width=6, blocks=1, conv=2), ff=5,
                                            experts=2, top=1),
                                 O.with_mlp(O.ssm(heads=1, vdim=6, state=3, groups=1, norm_groups=2, conv=2), ff=7, experts=3,
                                            top=2)], width=10, vocab=21)
    else:
        cfg = config_for(dtype, [O.with_mlp(O.par(dim=72, vdim=136, heads=2, kv_heads=1, width=208, blocks=2), ff=200,
                                            experts=3),
                                 O.with_mlp(O.ssm(heads=3, vdim=40, state=72, groups=1, norm_groups=3), ff=200, experts=3)],
                         width=136, vocab=150)
    sd = O.random_checkpoint(cfg, 21)
    toks = clear_tokens(40, cfg, sd, 22)
    want = O.forward(cfg, sd, toks)
    eng = make_engine(cfg, sd, device, dtype)
    got = run_schedule(eng, {"a": toks}, [[("a", c)] for c in cuts(40, [9, 1, 1, 14])])["a"]
    assert close(got, want, dtype)


# ------------------------------------------------------------------------------- registry, generation, runner script
def _save(tmp_path, cfg, sd, name):
    from safetensors.torch import save_file

    d = tmp_path / name
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in sd.items()}, str(d / "model.safetensors"))
    return d


@pytest.mark.parametrize("device,dtype", TARGETS)
def test_greedy_generation_through_engine(tmp_path, device, dtype):
    """A checkpoint directory -> model registry -> LLMEngine.generate (its own scheduler, chunked prefill, decode graphs on
    the GPU): greedy tokens equal the oracle's argmax (up to a near-tie of the oracle's top two logits)."""
    cfg = config_for(dtype, FULL[:4])
    sd = O.random_checkpoint(cfg, 31)
    d = _save(tmp_path, cfg, sd, "ckpt")
    model, tok, _ = build_llm(weights=str(d), device=device, dtype=dtype)
    assert isinstance(model, RonavikModel) and model.dtype == dtype
    eng = LLMEngine(model, tok, EngineConfig(max_num_seqs=4, num_blocks=64, max_model_len=256, prefill_chunk=16,
                                             max_batched_tokens=24, graph_batch_sizes=(1, 2, 4), decode_steps=1))
    prompts = [tokens(n, cfg["vocab"], 40 + n) for n in (23, 5, 41)]
    reqs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    margin = 1e-3 if dtype == torch.float32 else 0.15
    for p, r in zip(prompts, reqs):
        assert len(r.output_ids) == 12
        seq = list(p)
        for t in r.output_ids:
            row = O.forward(cfg, sd, seq)[-1]
            assert row[t] >= row.max() - margin * (row.max() - row.min()), (len(seq), t, int(row.argmax()))
            seq.append(t)


def test_trace_runner_script(tmp_path):
    """bin/trace_run on the CPU: steps from stdin, logits files and 'done' lines out."""
    import subprocess
    import sys

    import numpy as np

    cfg = O.make_config([O.with_mlp(O.par()), O.with_mlp(O.ssm()), O.with_mlp(O.par(kv_heads=1), None)])
    sd = O.random_checkpoint(cfg, 51)
    d = _save(tmp_path, cfg, sd, "m")
    a, b = clear_tokens(20, cfg, sd, 1), clear_tokens(9, cfg, sd, 102)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:12], "want": [0, 11]}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[:8], "want": []}, {"id": "a", "tokens": a[12:13], "want": [0]}],
              "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[13:], "want": [6]}, {"id": "b", "tokens": b[8:], "want": [0]}],
              "end": ["a", "b"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(d), "--dtype", "float32",
                        "--out", str(tmp_path / "out"), "--max-tokens", "128", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    wa, wb = O.forward(cfg, sd, a), O.forward(cfg, sd, b)
    rd = lambda n: torch.from_numpy(np.fromfile(tmp_path / "out" / f"{n}.f32", dtype="<f4").reshape(-1, cfg["vocab"]))  # noqa: E731
    assert rel_err(rd(0), wa[[0, 11]]) < 2e-4
    assert rel_err(rd(1), wa[[12]]) < 2e-4
    assert rel_err(rd(2), torch.stack([wa[19], wb[8]])) < 2e-4


def test_config_rejects_unknown_branches():
    with pytest.raises(ValueError):
        RonavikConfig.from_json(O.make_config([{"type": "mystery", "mixer": {}, "mlp": None}]))
    with pytest.raises(ValueError):
        RonavikConfig.from_json(O.make_config([dict(O.par(), mlp={"kind": "dense", "ff": 8})]))
    with pytest.raises(ValueError):
        RonavikConfig.from_json(O.make_config([O.with_mlp(O.par(heads=3, kv_heads=2))]))
    with pytest.raises(ValueError):
        RonavikConfig.from_json(O.make_config([O.with_mlp(O.ssm(), experts=2, top=3)]))


def test_query_temperature_steps():
    """The temperature is a step function of the position: constant inside a period, changing exactly at p + 1 = n * every."""
    q = torch.ones(12, 4)
    kc, vc = torch.zeros(2, 1, 16, 4), torch.zeros(2, 1, 4, 16)
    out = ops.headnorm_kv_write(q, q, q, torch.ones(4), torch.ones(4), torch.arange(12, dtype=torch.int32), kc, vc, 1, 1, 4, 4,
                                0.0, torch.arange(12, dtype=torch.int32), 0.5, 5)
    want = [1 + 0.5 * math.log((p + 1) // 5 + 1) for p in range(12)]
    assert torch.allclose(out[:, 0], torch.tensor(want), atol=1e-6)
    assert want[3] == 1.0 and want[4] > 1.0 and want[8] == want[4] and want[9] > want[8]


@_GPU
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_kernel_shape_variants(dtype):
    """Kernel variants that the small models above do not reach - workgroup-per-row norms (few wide rows), the
    decode-sized and the wide-block gate kernels, the chunk-parallel recurrence over several chunks and sequences -
    against the same ops on the CPU (which the tests above tie to the oracle)."""
    g = torch.Generator().manual_seed(0)
    rn = lambda *s: torch.randn(*s, generator=g)  # noqa: E731
    lim = 2e-5 if dtype == torch.float32 else 2e-2
    rel = lambda a, b: ((a.float().cpu() - b.float()).norm() / b.float().norm()).item()  # noqa: E731
    for T, D in ((3, 600), (5, 4500), (600, 520)):
        res, y, gate, wp, wn = rn(T, D), rn(T, D).to(dtype), rn(T, D).to(dtype), rn(D), rn(D)
        r1, r2 = res.clone(), res.clone().cuda()
        o1 = ops.gated_norm_add_f32(r1, y, gate, wp, 1e-5, wn, dtype)
        o2 = ops.gated_norm_add_f32(r2, y.cuda(), gate.cuda(), wp.cuda(), 1e-5, wn.cuda(), dtype)
        assert rel(r2, r1) < 1e-5 and rel(o2, o1) < lim, (T, D)
        yy, z, w = rn(T, D), rn(T, D).to(dtype), rn(D)
        for ng in (1, 4):
            assert rel(ops.gate_group_norm(yy.cuda(), z.cuda(), w.cuda(), ng, 1e-5, dtype),
                       ops.gate_group_norm(yy, z, w, ng, 1e-5, dtype)) < lim, (T, D, ng)
    if dtype == torch.float32:
        for T, W, nb in ((1, 512, 2), (7, 2200, 2), (70, 2200, 1), (3, 3300, 1), (100, 192, 3)):
            bs = W // nb
            u, wa, wi = rn(T, W), rn(nb, bs, bs) * bs ** -0.5, rn(nb, bs, bs) * bs ** -0.5
            ba, bi, lam = rn(W), rn(W), rn(W) - 2
            a1, b1 = ops.rglru_gates(u, wa, ba, wi, bi, lam, 8.0)
            a2, b2 = ops.rglru_gates(u.cuda(), wa.cuda(), ba.cuda(), wi.cuda(), bi.cuda(), lam.cuda(), 8.0)
            assert rel(a2, a1) < 1e-5 and rel(b2, b1) < 1e-4, (T, W, nb)
    T, W = 700, 300
    cu = torch.tensor([0, 400, 401, 465, 700], dtype=torch.int32)
    slots = torch.tensor([2, 0, 1, 3], dtype=torch.int32)
    a, b, yv, st = torch.rand(T, W, generator=g) * 0.5 + 0.5, rn(T, W) * 0.3, rn(T, W + 8).to(dtype), rn(5, W)
    s1, s2 = st.clone(), st.clone().cuda()
    o1 = ops.rglru_scan(a, b, yv[:, 8:], s1, cu, slots, dtype, act="gelu_tanh", out_scale=1.1)
    o2 = ops.rglru_scan(a.cuda(), b.cuda(), yv.cuda()[:, 8:], s2, cu.cuda(), slots.cuda(), dtype, act="gelu_tanh", out_scale=1.1)
    assert rel(o2, o1) < lim and rel(s2, s1) < 1e-5
    # state-space scan: long portions of few sequences take the chunk-parallel form (several chunks, a single token
    # between them, a state that does not start at zero)
    for (H, G, N, DV) in ((4, 2, 32, 32), (2, 1, 100, 24)):
        inner, T = H * DV, 1300
        cu = torch.tensor([0, 600, 601, 1300], dtype=torch.int32)
        slots = torch.tensor([1, 3, 0], dtype=torch.int32)
        cv, dtr = rn(T, inner + 2 * G * N) * 0.5, rn(T, H + 3).to(dtype)
        dtb, A, Dk, st = rn(H) - 1, rn(H) * 0.5, rn(H), rn(4, H, N, DV) * 0.3
        s1, s2, cg, dg = st.clone(), st.clone().cuda(), cv.cuda(), dtr.cuda()
        o1 = ops.ssd_scan(cv[:, :inner], cv[:, inner:inner + G * N], cv[:, inner + G * N:], dtr[:, 1:H + 1], dtb, A, Dk, s1,
                          cu, slots, G)
        o2 = ops.ssd_scan(cg[:, :inner], cg[:, inner:inner + G * N], cg[:, inner + G * N:], dg[:, 1:H + 1], dtb.cuda(),
                          A.cuda(), Dk.cuda(), s2, cu.cuda(), slots.cuda(), G)
        assert rel(o2, o1) < 5e-5 and rel(s2, s1) < 5e-5, (H, G, N, DV)
