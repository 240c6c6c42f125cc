"""Kuzanex (layer-list decoder with window attention, mLSTM layers, norm after the sum) against the plain float64
formulation in ``kuzanex_oracle.py``: every mechanism alone, then the serving engine - scheduler, paged cache, state
slots, prefill and decode plans - on small random models of several shapes. Every test runs on the CPU formulations
of the ops and, marked `gpu`, on the HIP kernels."""
import math
import os
import sys

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import kuzanex_oracle as O  # noqa: E402

from areal_vllm_amd.api.cli_args import InferenceServerConfig  # noqa: E402
from areal_vllm_amd.inference.engine import NativeInferenceEngine  # noqa: E402
from areal_vllm_amd.models.config import ModelConfig  # noqa: E402
from areal_vllm_amd.ops import mlstm as mlstm_ops  # noqa: E402
from areal_vllm_amd.ops import post_norm, window_attention as wattn  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
CASES = [("cpu", "float32"), pytest.param("cuda", "float32", marks=pytest.mark.gpu),
         pytest.param("cuda", "bfloat16", marks=pytest.mark.gpu)]
F64 = torch.float64


def tol(dtype):
    return 2e-4 if dtype in ("float32", torch.float32) else 6e-2


def rel_err(got, want):
    """Per row: rms of the difference (mean taken off) over the rms of the reference row."""
    got, want = torch.as_tensor(got).to(F64), torch.as_tensor(want).to(F64)
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    ref = (want - want.mean(-1, keepdim=True)).pow(2).mean(-1).sqrt().clamp(min=1e-9)
    return float((d.pow(2).mean(-1).sqrt() / ref).max())


# ------------------------------------------------------------------------------------ mechanisms
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_scaled_add_norm_and_xielu(device, dtype):
    g = torch.Generator().manual_seed(3)
    for T, W in ((5, 48), (3, 257), (1, 8), (2, 1030), (1, 2100), (1, 4100), (1, 8200)):  # every kernel variant
        x = torch.randn(T, W, generator=g)
        y = torch.randn(T, W, generator=g).to(dtype)
        gain = torch.tensor([1.37]).to(dtype)
        want = O.scalar_norm(2.5 * x.to(F64) + y.to(F64), gain, 1e-5)
        x32, xc = post_norm.scaled_add_norm(x.clone().to(device), y.to(device), gain.to(device), 2.5, 1e-5, dtype)
        assert x32.dtype == torch.float32 and xc.dtype == dtype
        assert rel_err(x32.cpu(), want) < 1e-5
        assert rel_err(xc.float().cpu(), want) < tol(dtype)
        nx, _ = post_norm.scaled_add_norm(x.clone().to(device), None, gain.to(device), 1.0, 1e-5, dtype, inplace=False)
        assert rel_err(nx.cpu(), O.scalar_norm(x.to(F64), gain, 1e-5)) < 1e-5
    z = (torch.randn(7, 33, generator=g) * 3).to(dtype)
    act = torch.tensor([0.4, -0.7]).to(dtype)
    got = post_norm.xielu(z.to(device), act.to(device)).float().cpu()
    assert rel_err(got, O.xielu(z.to(F64), act.to(F64))) < tol(dtype)


def _attention_reference(qn, kn, v, scale, softcap, talk, window):
    H, G = qn.shape[1], kn.shape[1]
    p = O.sink_softmax(O.shaped_scores(qn, kn.repeat_interleave(H // G, 1), scale, softcap, talk, window))
    return torch.einsum("hij,jhv->ihv", p, v.repeat_interleave(H // G, 1))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,V,window", [(4, 2, 16, 24, 37), (3, 3, 8, 8, 32), (6, 1, 40, 16, 5), (2, 2, 64, 64, 0),
                                            # head sizes the matrix-core kernel takes (bf16 rows of several queries)
                                            (4, 2, 64, 64, 37), (16, 4, 128, 128, 70), (8, 8, 128, 64, 33),
                                            (2, 1, 64, 128, 0), (6, 2, 64, 64, 40), (12, 4, 64, 64, 45), (5, 1, 64, 64, 20),
                                            (1, 1, 64, 64, 9)])
def test_window_attention_edges_pages_portions_and_splits(device, dtype, H, G, D, V, window):
    """A key that dominates its query's scores sits just inside and just outside the window, on both sides of page
    borders and at position 0; whole prompt, portions down to two tokens and split decoding must all agree."""
    g = torch.Generator().manual_seed(11)
    n, eps, scale, softcap = 150, 1e-5, 0.3, 9.0
    q = torch.randn(n, H, D, generator=g)
    k = torch.randn(n, G, D, generator=g)
    v = torch.randn(n, G, V, generator=g)
    w_eff = window if window else 10 ** 6
    pairs = [(140, 140 - min(w_eff, 140) + 1), (141, 141 - min(w_eff, 141)), (100, 64), (100, 63), (149, 128),
             (149, 127), (w_eff - 1 if w_eff < n else 40, 0), (min(w_eff, n - 1), 0), (31, 31), (32, 31), (1, 0)]
    for i, j in pairs:
        if 0 <= j <= i < n:  # the query's direction copied into the key, scaled: one score stands out
            k[j] = 1.5 * q[i].view(G, H // G, D).mean(1) + 0.3 * k[j]
    qw = 1 + 0.2 * torch.randn(D, generator=g)
    kw = 1 + 0.2 * torch.randn(D, generator=g)
    talk = torch.eye(H) + 0.2 * torch.randn(H, H, generator=g)
    proj = torch.cat([q.reshape(n, -1), k.reshape(n, -1), v.reshape(n, -1), torch.randn(n, H, generator=g)], 1).to(dtype)
    qw, kw, talk = qw.to(dtype), kw.to(dtype), talk.to(dtype)
    p64 = proj.to(F64)
    qn = O.unit_rms(p64[:, :H * D].view(n, H, D), eps) * qw.to(F64)
    kn = O.unit_rms(p64[:, H * D:(H + G) * D].view(n, G, D), eps) * kw.to(F64)
    if dtype == torch.bfloat16:  # what the cache and the query buffer can hold
        qn, kn = qn.to(dtype).to(F64), kn.to(dtype).to(F64)
    want = _attention_reference(qn, kn, p64[:, (H + G) * D:(H + G) * D + G * V].view(n, G, V), scale, softcap,
                                talk.to(F64), window)
    want = want * torch.sigmoid(p64[:, -H:]).unsqueeze(-1)  # one gate per head and token
    shape = wattn.ScoreShape(scale=scale, softcap=softcap, slope_exp=8.0, window=window, sink=True)
    pages = [7, 2, 9, 4, 1]  # scattered, out of order
    bt = torch.tensor([pages], dtype=torch.int32, device=device)
    slots = torch.tensor([pages[t // 32] * 32 + t % 32 for t in range(n)], dtype=torch.int64, device=device)
    pj, qwd, kwd, tk = proj.to(device), qw.to(device), kw.to(device), talk.to(device)

    def run(portions, nsplit=1, matrix_cores=True):
        kc, vc = wattn.alloc_window_cache(12, G, D, V, dtype, device)
        kc.fill_(float("nan") if dtype == torch.float32 else 1e4)  # stale pages must never leak into a result
        vc.fill_(1e4)
        outs, at = [], 0
        for c in portions:
            qq = wattn.qk_norm_cache_write(pj[at:at + c], qwd, kwd, slots[at:at + c], kc, vc, H, eps)
            cu = torch.tensor([0, c], dtype=torch.int32, device=device)
            ctx = torch.tensor([at + c], dtype=torch.int32, device=device)
            outs.append(wattn.window_attention(qq, kc, vc, bt, cu, ctx, c, shape, tk,
                                               nsplit=nsplit if c == 1 else 1, gate=pj[at:at + c, -H:],
                                               matrix_cores=matrix_cores))
            at += c
        return torch.cat(outs).float().cpu()

    whole = run([n])
    assert rel_err(whole.reshape(n, -1), want.reshape(n, -1)) < tol(dtype)
    cut = run([3, 64, 2, 50, 29, 2])
    assert rel_err(cut.reshape(n, -1), want.reshape(n, -1)) < tol(dtype)
    assert rel_err(cut.reshape(n, -1), whole.reshape(n, -1)) < 1e-5 + (1e-2 if dtype == torch.bfloat16 else 0)
    plain = run([3, 64, 2, 50, 29, 2], matrix_cores=False)  # the kernel for every shape and type
    assert rel_err(plain.reshape(n, -1), want.reshape(n, -1)) < tol(dtype)
    for nsplit in (1, 3):
        dec = run([100] + [1] * 50, nsplit=nsplit)
        assert rel_err(dec.reshape(n, -1), want.reshape(n, -1)) < tol(dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("NH,D,V", [(3, 24, 40), (1, 8, 8), (2, 64, 72), (2, 130, 16), (2, 128, 128), (2, 48, 64)])
def test_mlstm_state_carried_over_portions_and_reused_slots(device, dtype, NH, D, V):
    g = torch.Generator().manual_seed(5)
    n, W, cap, eps = 150, 32, 6.0, 1e-5
    x = torch.randn(n, W, generator=g).to(dtype)
    wg = (torch.randn(2 * NH, W, generator=g) * 0.6).to(dtype)
    bg = torch.randn(2 * NH, generator=g).to(dtype)
    proj = (torch.randn(n, 2 * NH * D + 2 * NH * V + 5, generator=g)).to(dtype)
    nw = (1 + 0.2 * torch.randn(NH * V, generator=g)).to(dtype)
    z = x.to(F64) @ wg.to(F64).T + bg.to(F64)
    ig = cap * torch.tanh(z[:, :NH] / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh(z[:, NH:] / cap))
    p64 = proj.to(F64)
    heads = []
    for h in range(NH):
        y = O.mlstm_recurrence(p64[:, h * D:(h + 1) * D] * D ** -0.5, p64[:, NH * D + h * D:NH * D + (h + 1) * D],
                               p64[:, 2 * NH * D + h * V:2 * NH * D + (h + 1) * V], ig[:, h], fg[:, h])
        heads.append(O.unit_rms(y, eps))
    gate = p64[:, 2 * NH * D + NH * V:2 * NH * D + 2 * NH * V]
    want = torch.cat(heads, -1) * nw.to(F64) * torch.sigmoid(gate)
    state = mlstm_ops.RecurrentState(3, NH, D, V, device)
    xd, pd, wgd, bgd, nwd = x.to(device), proj.to(device), wg.to(device), bg.to(device), nw.to(device)

    def run(portions, slot):
        outs, at = [], 0
        for c in portions:
            i_, f_ = mlstm_ops.mlstm_gates(xd[at:at + c].contiguous(), wgd, bgd, NH, cap)
            cu = torch.tensor([0, c], dtype=torch.int32, device=device)
            hb, nq, mt = mlstm_ops.mlstm_scan(pd[at:at + c], 0, NH * D, 2 * NH * D, i_, f_, cu,
                                              torch.tensor([at], dtype=torch.int32, device=device),
                                              torch.tensor([slot], dtype=torch.int32, device=device), state,
                                              max_q=c)  # long portions take the chunk-parallel kernel on the GPU
            outs.append(mlstm_ops.mlstm_out(hb, nq, mt, pd[at:at + c, 2 * NH * D + NH * V:2 * NH * D + 2 * NH * V], nwd,
                                            eps))
            at += c
        return torch.cat(outs).float().cpu()

    assert rel_err(run([n], 1), want) < tol(dtype)
    state.S.fill_(123.0)  # a slot is handed on as it is: a sequence that starts at position 0 must not see this
    state.n.fill_(-7.0)
    state.m.fill_(3.0)
    assert rel_err(run([2, 9, 1, 1, 17, 8, 30, 2, 64, 16], 1), want) < tol(dtype)
    assert rel_err(run([40, 65] + [1] * 45, 2), want) < tol(dtype)
    # a row without a slot is skipped and leaves every slot alone
    before = state.S.clone()
    i_, f_ = mlstm_ops.mlstm_gates(xd[:4].contiguous(), wgd, bgd, NH, cap)
    mlstm_ops.mlstm_scan(pd[:4], 0, NH * D, 2 * NH * D, i_, f_, torch.tensor([0, 4], dtype=torch.int32, device=device),
                         torch.tensor([0], dtype=torch.int32, device=device),
                         torch.tensor([-1], dtype=torch.int32, device=device), state)
    assert torch.equal(before, state.S)


# ------------------------------------------------------------------------------------------ engine
def attn_layer(heads=4, kv=2, dim=16, vdim=24, window=37, ff=80, scale=0.35, softcap=7.0):
    mixer = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "softcap": softcap}
    if window:
        mixer["mask"] = {"size": window}
    return {"type": "attention", "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def mlstm_layer(heads=3, dim=16, vdim=24, cap=5.0, ff=80):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(layers, width=48, vocab=101, alpha=1.7, eps=1e-5):
    return {"architecture": "Kuzanex", "layers": layers, "norm": {"eps": eps}, "postln_alpha": alpha, "vocab": vocab,
            "width": width}


MIXED = config([attn_layer(), mlstm_layer(), mlstm_layer(heads=1, dim=8, vdim=8, ff=0), attn_layer(4, 4, 8, 8, 5)])


def make_engine(cfg_dict, device, dtype, num_pages=40, max_running=4, context=512, score=True, graphs=True):
    cfg = ModelConfig.from_hf_dict(cfg_dict)
    srv = InferenceServerConfig(model_path="", dtype=dtype, context_length=context, max_running_requests=max_running,
                                num_continuous_decode_steps=1, max_prefill_tokens=context,
                                disable_cuda_graph=not graphs)
    eng = NativeInferenceEngine(srv, model_config=cfg, device=torch.device(device), num_pages=num_pages,
                                score_mode=score)
    eng.initialize(load_weights=False)
    weights = {k: v.detach().float().cpu() for k, v in eng.model.checkpoint_tensors().items()}
    return eng, weights


def replay(eng, steps):
    """steps: list of lists of (request id, tokens, wanted places, ends after this step) -> {id: {position: logits}}."""
    out, fed, live = {}, {}, set()
    for step in steps:
        for rid, toks, want, _ in step:
            if rid not in live:
                eng.open_replay(rid)
                live.add(rid)
                fed[rid] = 0
        logits = eng.replay_step([(rid, toks, want) for rid, toks, want, _ in step])
        at = 0
        for rid, toks, want, end in step:
            for w in want:
                out.setdefault(rid, {})[fed[rid] + w] = logits[at]
                at += 1
            fed[rid] += len(toks)
            if end:
                eng.close_replay(rid)
                live.discard(rid)
        assert at == logits.shape[0]
    return out


def cut(rid, tokens, sizes):
    """One request alone, fed in portions of the given sizes (the last size repeats); every position is wanted."""
    steps, at, i = [], 0, 0
    while at < len(tokens):
        c = min(sizes[min(i, len(sizes) - 1)], len(tokens) - at)
        steps.append([(rid, tokens[at:at + c], list(range(c)), at + c == len(tokens))])
        at += c
        i += 1
    return steps


def check_against_oracle(got, tokens, weights, cfg_dict, dtype, rid):
    want = O.forward(tokens, weights, cfg_dict)
    rows = torch.from_numpy(np.stack([got[rid][p] for p in range(len(tokens))]))
    assert rel_err(rows, want) < tol(dtype), rel_err(rows, want)


def tokens_of(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


@pytest.mark.parametrize("device,dtype", CASES)
def test_whole_prompt_and_every_layer(device, dtype):
    eng, w = make_engine(MIXED, device, dtype)
    try:
        toks = tokens_of(75, MIXED["vocab"], 1)
        eng.runner.layer_trace = []
        got = replay(eng, cut("a", toks, [len(toks)]))
        trace, eng.runner.layer_trace = eng.runner.layer_trace, None
        layers = []
        O.forward(toks, w, MIXED, layers)
        assert len(trace) == len(layers)
        for a, b in zip(trace, layers):
            assert rel_err(a.cpu(), b) < tol(dtype)
        check_against_oracle(got, toks, w, MIXED, dtype, "a")
    finally:
        eng.destroy()


@pytest.mark.parametrize("device,dtype", CASES)
def test_prefill_against_token_by_token_and_portions(device, dtype):
    eng, w = make_engine(MIXED, device, dtype)
    try:
        toks = tokens_of(140, MIXED["vocab"], 2)
        for k, sizes in enumerate(([1], [60, 1], [2], [3, 64, 2, 31, 33, 1, 1, 5], [1, 32, 32, 32, 1])):
            got = replay(eng, cut(f"r{k}", toks, list(sizes)))
            check_against_oracle(got, toks, w, MIXED, dtype, f"r{k}")
        assert eng.sched.num_free_state_slots() == 4 and eng.sched.num_free_pages() == eng.sched.num_total_pages()
    finally:
        eng.destroy()


@pytest.mark.parametrize("device,dtype", CASES)
def test_unequal_requests_in_one_batch_with_pages_and_slots_used_again(device, dtype):
    """Seven requests of very different lengths through three slots and a pool that cannot hold them all at once:
    portions of some beside single tokens of others; each must equal the request computed alone."""
    eng, w = make_engine(MIXED, device, dtype, num_pages=15, max_running=3)
    try:
        V = MIXED["vocab"]
        reqs = {f"q{i}": tokens_of(n, V, 10 + i) for i, n in enumerate((1, 70, 23, 130, 2, 97, 40))}
        plan = {"q0": [1], "q1": [5, 1, 1, 33, 2, 1], "q2": [23], "q3": [64, 2, 1, 1, 40, 1], "q4": [1, 1], "q5": [31, 33, 1],
                "q6": [2, 1]}
        waiting, live, at, steps = list(reqs), [], {r: 0 for r in reqs}, []
        nth = {r: 0 for r in reqs}
        while waiting or live:
            while waiting and len(live) < 3:
                need = sum((len(reqs[r]) + 31) // 32 for r in live) + (len(reqs[waiting[0]]) + 31) // 32
                if need > 13:
                    break
                live.append(waiting.pop(0))
            step = []
            for r in list(live):
                sizes = plan[r]
                c = min(sizes[min(nth[r], len(sizes) - 1)], len(reqs[r]) - at[r])
                end = at[r] + c == len(reqs[r])
                step.append((r, reqs[r][at[r]:at[r] + c], list(range(c)), end))
                at[r] += c
                nth[r] += 1
                if end:
                    live.remove(r)
            steps.append(step)
        assert max(len(s) for s in steps) == 3 and any(len(t) == 1 for s in steps if len(s) > 1 for _, t, _, _ in s)
        got = replay(eng, steps)
        for r, toks in reqs.items():
            check_against_oracle(got, toks, w, MIXED, dtype, r)
        assert eng.sched.num_free_state_slots() == 3 and eng.sched.num_free_pages() == eng.sched.num_total_pages()
    finally:
        eng.destroy()


SHAPES = [
    # kv heads = heads, key size = value size, feed-forward as wide as the model, one head: values that hide mix-ups
    config([attn_layer(2, 2, 16, 16, 33, ff=32), mlstm_layer(1, 16, 16, ff=32)], width=32),
    # grouped heads, sizes that are no multiples of 8 or of each other, no feed-forward, window below a page
    config([mlstm_layer(5, 12, 20, ff=0), attn_layer(6, 2, 12, 20, 7, ff=0), attn_layer(3, 1, 20, 12, 64)], width=40,
           vocab=67, alpha=0.9),
    config([attn_layer(4, 2, 16, 24, 0)], width=24),  # no window: every earlier token is seen
    config([mlstm_layer(2, 72, 80, cap=12.0)], width=56, alpha=3.0, eps=1e-3),
    config([attn_layer(4, 2, 64, 64, 37), mlstm_layer(2, 64, 64), attn_layer(8, 2, 64, 128, 50, ff=0)], width=64),
]


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("which", range(len(SHAPES)))
def test_other_sizes_windows_and_layer_orders(device, dtype, which):
    cfg = SHAPES[which]
    eng, w = make_engine(cfg, device, dtype)
    try:
        toks = tokens_of(110, cfg["vocab"], 30 + which)
        got = replay(eng, cut("whole", toks, [len(toks)]))
        check_against_oracle(got, toks, w, cfg, dtype, "whole")
        got = replay(eng, cut("cut", toks, [31, 2, 34, 1]))
        check_against_oracle(got, toks, w, cfg, dtype, "cut")
    finally:
        eng.destroy()


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_shapes_orders_and_schedules(device, seed):
    """Random layer lists (sizes, head layouts, windows, constants, with and without feed-forward) fed through random
    schedules of up to three live requests: portions of 1 .. 100 tokens, requests that skip steps; 32-bit, so that
    any deviation beyond rounding shows."""
    import random

    rng = random.Random(seed)
    for case in range(3):
        width, vocab, layers = rng.choice([32, 48, 72]), rng.choice([37, 101]), []
        for _ in range(rng.randint(1, 4)):
            ff = rng.choice([0, 40, width])
            if rng.random() < 0.5:
                G = rng.choice([1, 2, 3])
                H = G * rng.choice([1, 2, 4])
                D = rng.choice([8, 24, 64])
                V = rng.choice([64, 128]) if D == 64 else rng.choice([8, 40])
                layers.append(attn_layer(H, G, D, V, rng.choice([1, 2, 31, 32, 33, 100, 0]), ff,
                                         scale=rng.choice([0.1, 0.3]), softcap=rng.choice([3.0, 50.0])))
            else:
                layers.append(mlstm_layer(rng.choice([1, 2, 3]), rng.choice([8, 24, 64, 136]), rng.choice([8, 40, 72]),
                                          rng.choice([4.0, 12.0]), ff))
        cfg = config(layers, width=width, vocab=vocab, alpha=rng.choice([0.8, 2.5]), eps=rng.choice([1e-5, 1e-6]))
        reqs = {f"q{i}": tokens_of(rng.choice([1, 2, 17, 97, 150]), vocab, 100 * case + i)
                for i in range(rng.randint(1, 3))}
        at, steps = {r: 0 for r in reqs}, []
        while any(at[r] < len(t) for r, t in reqs.items()):
            step = []
            for r, t in reqs.items():
                if at[r] < len(t) and rng.random() > 0.2:
                    c = min(rng.choice([1, 1, 1, 2, 3, 16, 31, 33, 64, 100]), len(t) - at[r])
                    step.append((r, t[at[r]:at[r] + c], list(range(c)), at[r] + c == len(t)))
                    at[r] += c
            if step:
                steps.append(step)
        eng, w = make_engine(cfg, device, "float32", num_pages=24, max_running=3)
        try:
            got = replay(eng, steps)
            for r, t in reqs.items():
                check_against_oracle(got, t, w, cfg, "float32", r)
        finally:
            eng.destroy()


@pytest.mark.parametrize("device,dtype", CASES)
def test_first_tokens_and_long_decoding(device, dtype):
    cfg = config([attn_layer(4, 2, 16, 24, 40), mlstm_layer()])
    eng, w = make_engine(cfg, device, dtype)
    try:
        for n in (1, 2, 3):
            toks = tokens_of(n, cfg["vocab"], 40 + n)
            check_against_oracle(replay(eng, cut(f"s{n}", toks, [1])), toks, w, cfg, dtype, f"s{n}")
        toks = tokens_of(230, cfg["vocab"], 44)  # the window passes over decoded tokens several times
        check_against_oracle(replay(eng, cut("long", toks, [20, 1])), toks, w, cfg, dtype, "long")
    finally:
        eng.destroy()


@pytest.mark.parametrize("device,dtype", CASES)
def test_greedy_generation_through_the_engine(device, dtype):
    """The engine's own entry point: prompts of unequal length generated together, prefill plans, then decode
    plans (captured graphs on the GPU), more requests than request slots."""
    cfg = config([attn_layer(4, 2, 16, 24, 21), mlstm_layer(2, 16, 24), attn_layer(2, 1, 16, 16, 70)], vocab=61)
    eng, w = make_engine(cfg, device, dtype, max_running=3, score=False)
    try:
        prompts = [tokens_of(n, cfg["vocab"], 50 + n) for n in (3, 41, 18, 1, 66)]
        res = eng.generate_blocking(prompts, max_new_tokens=12, greedy=True)
        for p, r in zip(prompts, res):
            assert r.finish_reason == "length" and len(r.output_tokens) == 12
            want = O.greedy(p, 12, w, cfg)
            if dtype == "float32":
                assert r.output_tokens == want
            else:  # a near-tie may flip under bf16: the tokens before the first difference must still agree
                same = sum(1 for a, b in zip(r.output_tokens, want) if a == b)
                assert r.output_tokens[:4] == want[:4] and same >= 6
        assert eng.sched.num_free_state_slots() == 3
    finally:
        eng.destroy()


@pytest.mark.parametrize("device", DEVICES)
def test_served_from_a_checkpoint_directory(device, tmp_path):
    """The framework's own path from a directory with config.json and model.safetensors: the model class is chosen by
    the configuration, the weights come through the engine's loader."""
    from areal_vllm_amd.models import build_model

    cfg_dict = config([mlstm_layer(2, 8, 16), attn_layer(4, 1, 8, 16, 9, ff=0)], width=32, vocab=53)
    m = build_model(ModelConfig.from_hf_dict(cfg_dict), dtype=torch.bfloat16)
    m.flatten()
    m.init_weights(seed=9)
    m.save_checkpoint(str(tmp_path))
    w = {k: v.float() for k, v in m.checkpoint_tensors().items()}
    srv = InferenceServerConfig(model_path=str(tmp_path), dtype="float32", context_length=128, max_running_requests=2,
                                num_continuous_decode_steps=2)
    eng = NativeInferenceEngine(srv, device=torch.device(device), num_pages=12)
    eng.initialize()
    try:
        prompts = [tokens_of(n, 53, 70 + n) for n in (5, 33, 17)]
        res = eng.generate_blocking(prompts, max_new_tokens=7, greedy=True)
        for p, r in zip(prompts, res):
            assert r.output_tokens == O.greedy(p, 7, w, cfg_dict)
    finally:
        eng.destroy()


def test_http_server_command_line_serves_a_checkpoint(tmp_path):
    """The server's own command line -> engine -> POST /generate, greedy, against the float64 formulation."""
    import asyncio
    import socket
    import threading

    import requests
    from aiohttp import web

    from areal_vllm_amd.inference.server import InferenceServer, build_engine, parse_server_args
    from areal_vllm_amd.models import build_model

    cfg_dict = config([attn_layer(2, 1, 8, 8, 11), mlstm_layer(1, 8, 16, ff=0)], width=24, vocab=41)
    m = build_model(ModelConfig.from_hf_dict(cfg_dict), dtype=torch.float32)
    m.flatten()
    m.init_weights(seed=13)
    m.save_checkpoint(str(tmp_path))
    w = {k: v.float() for k, v in m.checkpoint_tensors().items()}
    args, srv_cfg = parse_server_args(["--model-path", str(tmp_path), "--device", "cpu", "--num-pages", "16", "--dtype",
                                       "float32", "--context-length", "128", "--max-running-requests", "2"])
    eng = build_engine(args, srv_cfg)
    with socket.socket() as sk:
        sk.bind(("127.0.0.1", 0))
        port = sk.getsockname()[1]
    loop, started = asyncio.new_event_loop(), threading.Event()

    def run():
        asyncio.set_event_loop(loop)
        runner = web.AppRunner(InferenceServer(eng).app)
        loop.run_until_complete(runner.setup())
        loop.run_until_complete(web.TCPSite(runner, "127.0.0.1", port).start())
        started.set()
        loop.run_forever()

    threading.Thread(target=run, daemon=True).start()
    assert started.wait(30)
    try:
        prompt = tokens_of(19, 41, 3)
        r = requests.post(f"http://127.0.0.1:{port}/generate", json={
            "input_ids": prompt, "sampling_params": {"max_new_tokens": 6, "temperature": 0.0}}, timeout=120).json()
        assert r["output_ids"] == O.greedy(prompt, 6, w, cfg_dict)
    finally:
        loop.call_soon_threadsafe(loop.stop)
        eng.destroy()


def test_config_reader_and_checkpoint_save_then_load(tmp_path):
    cfg = ModelConfig.from_hf_dict(SHAPES[1])
    assert cfg.family == "kuzanex" and cfg.n_layers == 3 and cfg.has_recurrent_state
    from areal_vllm_amd.models import build_model

    m = build_model(cfg, dtype=torch.float32)
    m.flatten()
    m.init_weights(seed=4)
    assert sum(p.numel() for p in m.parameters()) == cfg.n_params()
    m.save_checkpoint(str(tmp_path))
    cfg2 = ModelConfig.from_pretrained(str(tmp_path))
    assert cfg2.layers == cfg.layers and cfg2.postln_alpha == cfg.postln_alpha
    m2 = build_model(cfg2, dtype=torch.float32)
    m2.flatten()
    m2.load_checkpoint(str(tmp_path))
    for (n1, a), (n2, b) in zip(m.checkpoint_tensors().items(), m2.checkpoint_tensors().items()):
        assert n1 == n2 and torch.equal(a, b)
    with pytest.raises(ValueError):
        ModelConfig.from_hf_dict(config([dict(attn_layer(), type="conv")]))
