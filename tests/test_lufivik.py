"""Lufivik (layer-list decoder: latent attention, routed clamped-GLU experts, sublayers between two layer norms with
gated residuals, input convolution, bigram embedding, looped layers) against the plain float64 formulation in
``lufivik_oracle.py``: every mechanism alone, then the serving engine - scheduler, paged latent cache, state slots,
prefill and decode plans - on small random models of several shapes. Every test runs on the CPU formulations of the
ops and, marked `gpu`, on the HIP kernels."""
import os
import sys

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import lufivik_oracle as O  # noqa: E402

from areal_vllm_amd.api.cli_args import InferenceServerConfig  # noqa: E402
from areal_vllm_amd.inference.engine import NativeInferenceEngine  # noqa: E402
from areal_vllm_amd.models.config import ModelConfig  # noqa: E402
from areal_vllm_amd.models.hybrid import RoutedGLUExperts  # noqa: E402
from areal_vllm_amd.ops import latent_attention as lattn  # noqa: E402
from areal_vllm_amd.ops import sandwich  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
CASES = [("cpu", "float32"), pytest.param("cuda", "float32", marks=pytest.mark.gpu),
         pytest.param("cuda", "bfloat16", marks=pytest.mark.gpu)]
OP_CASES = [("cpu", torch.float32), ("cpu", torch.bfloat16),
            pytest.param("cuda", torch.float32, marks=pytest.mark.gpu),
            pytest.param("cuda", torch.bfloat16, marks=pytest.mark.gpu)]
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


def rows_agree(got, want, dtype):
    """32-bit: every row within the tolerance. bf16: a router's near-tie may pick another expert for a token (and what
    reads that token shifts with it), and small random models amplify rounding through their norms: the median row
    must be inside the tolerance and four rows of five within 2.5 times it (a wrong kernel is off by the rows' own
    size; the matrix-core kernels are held to the sharp bound by the mechanism tests above)."""
    got, want = torch.as_tensor(got).to(F64), torch.as_tensor(want).to(F64)
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    ref = (want - want.mean(-1, keepdim=True)).pow(2).mean(-1).sqrt().clamp(min=1e-9)
    e = d.pow(2).mean(-1).sqrt() / ref
    if dtype in ("float32", torch.float32):
        return bool(e.max() < tol(dtype))
    return bool(e.median() < tol(dtype) and (e < 2.5 * tol(dtype)).double().mean() >= 0.8)


def i32(x, device):
    return torch.tensor(x, dtype=torch.int32, device=device)


# ------------------------------------------------------------------------------------ mechanisms
@pytest.mark.parametrize("device,dtype", OP_CASES)
def test_layer_norm_and_gated_norm_scale_sum(device, dtype):
    g = torch.Generator().manual_seed(3)
    for T, W in ((5, 48), (3, 257), (1, 8), (2, 1030), (1, 4100)):
        x = torch.randn(T, W, generator=g) * 3 + 0.5
        w, b = (1 + 0.2 * torch.randn(W, generator=g)).to(dtype), (0.3 * torch.randn(W, generator=g)).to(dtype)
        want = O.layer_norm(x.to(F64), w.to(F64), b.to(F64), 1e-5)
        h32, hc = sandwich.layer_norm(x.to(device), w.to(device), b.to(device), 1e-5, dtype)
        assert h32.dtype == torch.float32 and hc.dtype == dtype
        assert rel_err(h32.cpu(), want) < 1e-5 and rel_err(hc.float().cpu(), want) < tol(dtype)
        y = (2 * torch.randn(T, W, generator=g)).to(dtype)
        r = (2 * torch.randn(T, W, generator=g)).to(dtype)
        s = (0.5 + torch.rand(W, generator=g)).to(dtype)
        nw, nb = (1 + 0.2 * torch.randn(W, generator=g)).to(dtype), (0.3 * torch.randn(W, generator=g)).to(dtype)
        x_want = x.to(F64) + O.layer_norm(y.to(F64) * torch.sigmoid(r.to(F64)), w.to(F64), b.to(F64), 1e-5) * s.to(F64)
        h_want = O.layer_norm(x_want, nw.to(F64), nb.to(F64), 1e-5)
        xd = x.clone().to(device)
        x2, h2, hc2 = sandwich.gated_norm_add(xd, y.to(device), r.to(device), w.to(device), b.to(device), s.to(device),
                                              1e-5, (nw.to(device), nb.to(device)))
        assert x2 is xd and rel_err(x2.cpu(), x_want) < 1e-5 and rel_err(h2.cpu(), h_want) < 1e-5
        assert rel_err(hc2.float().cpu(), h_want) < tol(dtype)
        # no gate, no scale, no following norm
        xd = x.clone().to(device)
        x3, h3, _ = sandwich.gated_norm_add(xd, y.to(device), None, w.to(device), b.to(device), None, 1e-5)
        assert h3 is None and rel_err(x3.cpu(), x.to(F64) + O.layer_norm(y.to(F64), w.to(F64), b.to(F64), 1e-5)) < 1e-5


@pytest.mark.parametrize("device,dtype", OP_CASES)
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_input_convolution_portions_rows_and_slots_used_again(device, dtype, taps):
    g = torch.Generator().manual_seed(taps)
    n, W, n_slots = 45, 24, 5
    h = torch.randn(n, W, generator=g)
    w = torch.randn(W, taps, generator=g).to(dtype)
    want = h.to(F64) + O.causal_conv(h.to(F64), w.to(F64))
    state = torch.full((n_slots, taps - 1, W), 1e3, device=device) if taps > 1 else None  # what an earlier request left

    def run(portions, slot):
        outs, at = [], 0
        for c in portions:
            outs.append(sandwich.canon_conv(h[at:at + c].contiguous().to(device), w.to(device), state, i32([0, c], device),
                                            i32([at], device), i32([slot], device), dtype))
            at += c
        return torch.cat(outs).float().cpu()

    assert rel_err(run([n], 1), want) < tol(dtype)
    for k, sizes in enumerate(([1] * n, [2] * 22 + [1], [3, 1, 7, 2, 1, 1, 30], [40, 1, 1, 1, 1, 1], [1, 2, 42])):
        assert rel_err(run(sizes, k % n_slots), want) < tol(dtype)
    # two sequences side by side in one call, at different places, beside a row that owns no slot
    if taps > 1:
        state.fill_(-7.0)
    a = run([10], 0)  # slot 0 now continues at position 10
    before = state.clone() if state is not None else None
    both = torch.cat([h[10:13], h[:6], h[:2]]).contiguous().to(device)
    out = sandwich.canon_conv(both, w.to(device), state, i32([0, 3, 9, 11], device), i32([10, 0, 0], device),
                              i32([0, 3, -1], device), dtype).float().cpu()
    assert rel_err(torch.cat([a, out[:3]]), want[:13]) < tol(dtype) and rel_err(out[3:9], want[:6]) < tol(dtype)
    assert torch.isfinite(out).all()
    if state is not None:
        assert torch.equal(state[[1, 2, 4]], before[[1, 2, 4]])  # untouched slots


@pytest.mark.parametrize("device,dtype", OP_CASES)
@pytest.mark.parametrize("buckets,mul_prev,mul_cur", [(13, 29, 5), (1, 1, 1), (512, 1, 0), (64, 1000003, 999983)])
def test_bigram_embedding_portions_first_token_and_slots(device, dtype, buckets, mul_prev, mul_cur):
    g = torch.Generator().manual_seed(5)
    V, W, n = 70, 40, 37
    toks = torch.randint(0, V, (n,), generator=g)
    E, B = torch.randn(V, W, generator=g).to(dtype), torch.randn(buckets + 1, W, generator=g).to(dtype)
    w, b = (1 + 0.2 * torch.randn(W, generator=g)).to(dtype), (0.3 * torch.randn(W, generator=g)).to(dtype)
    rows = O.bigram_rows(toks.tolist(), buckets, mul_prev, mul_cur)
    assert rows[0] == buckets
    want = O.layer_norm(E.to(F64)[toks] + B.to(F64)[rows], w.to(F64), b.to(F64), 1e-5)
    prev = torch.full((4,), V - 1, dtype=torch.int32, device=device)  # left behind by earlier requests

    def run(portions, slot):
        outs, at = [], 0
        for c in portions:
            outs.append(sandwich.embed_bigram_norm(toks[at:at + c].to(device), E.to(device), B.to(device), mul_prev,
                                                   mul_cur, w.to(device), b.to(device), 1e-5, i32([0, c], device),
                                                   i32([at], device), i32([slot], device), prev))
            at += c
        assert int(prev[slot]) == int(toks[at - 1])
        return torch.cat(outs).cpu()

    assert rel_err(run([n], 0), want) < 1e-5
    for k, sizes in enumerate(([1] * n, [2] * 18 + [1], [5, 1, 1, 30], [36, 1])):
        assert rel_err(run(sizes, k), want) < 1e-5
    # rows of one batch: a continuation, a fresh sequence, a row without a slot (token embedding alone)
    run([4], 2)
    both = torch.cat([toks[4:9], toks[:3], toks[:2]]).to(device)
    out = sandwich.embed_bigram_norm(both, E.to(device), B.to(device), mul_prev, mul_cur, w.to(device), b.to(device), 1e-5,
                                     i32([0, 5, 8, 10], device), i32([4, 0, 0], device), i32([2, 1, -1], device), prev).cpu()
    assert rel_err(out[:5], want[4:9]) < 1e-5 and rel_err(out[5:8], want[:3]) < 1e-5
    assert rel_err(out[8:], O.layer_norm(E.to(F64)[toks[:2]], w.to(F64), b.to(F64), 1e-5)) < 1e-5
    assert int(prev[2]) == int(toks[8]) and int(prev[1]) == int(toks[2])
    # without a bigram table the embedding is the token's row
    out = sandwich.embed_bigram_norm(toks.to(device), E.to(device), None, 0, 0, w.to(device), b.to(device), 1e-5,
                                     i32([0, n], device), i32([0], device), i32([0], device), None).cpu()
    assert rel_err(out, O.layer_norm(E.to(F64)[toks], w.to(F64), b.to(F64), 1e-5)) < 1e-5


def _mixer_cfg(H, D, P, V, R, window, scale=0.3, base=10000.0):
    m = {"heads": H, "dim": D, "rot_dim": P, "vdim": V, "kv_rank": R, "q_rank": 8, "scale": scale,
         "rot": {"base": base, "dims": P}}
    if window:
        m["mask"] = {"size": window}
    return m


@pytest.mark.parametrize("device,dtype", OP_CASES)
@pytest.mark.parametrize("H,D,P,V,R,window", [(4, 16, 8, 24, 32, 37), (3, 8, 8, 8, 8, 32), (1, 40, 4, 16, 24, 5),
                                              (6, 40, 32, 24, 128, 41), (2, 64, 64, 128, 72, 0), (5, 24, 2, 8, 40, 1),
                                              (16, 16, 16, 16, 64, 33),
                                              # latent / rotary sizes the matrix-core kernel takes (bf16 prompt rows)
                                              (16, 64, 64, 64, 512, 70), (9, 16, 32, 16, 256, 45), (3, 24, 64, 8, 64, 33),
                                              (4, 8, 64, 24, 256, 0), (2, 12, 64, 16, 128, 31)])
def test_latent_attention_edges_pages_portions_and_splits(device, dtype, H, D, P, V, R, window):
    """A key that dominates its query's scores sits just inside and just outside the window, on both sides of page
    borders, at position 0 and hundreds of tokens back; whole prompt, portions down to two tokens, several rows in
    one call and split decoding must all agree with the unabsorbed formulation."""
    g = torch.Generator().manual_seed(11)
    n, eps = 330 if window == 0 else 150, 1e-5
    m = _mixer_cfg(H, D, P, V, R, window)
    down = torch.randn(n, R + P, generator=g)
    w_uk = torch.randn(H * D, R, generator=g) / R ** 0.5
    w_uv = torch.randn(H * V, R, generator=g) / R ** 0.5
    cw = 1 + 0.2 * torch.randn(R, generator=g)
    q = torch.randn(n, H, D + P, generator=g)
    gates = torch.randn(n, H, generator=g)
    # query i of head h points at the (unrotated) key of token j: its score stands out among all others
    c64 = O.rms_norm(down[:, :R].to(F64), cw.to(F64), eps)
    keys = (c64 @ w_uk.to(F64).T).view(n, H, D)
    far = max(window, 1) if window > 0 else 300
    for i, j in ((far + 3, 4), (far + 2, 2), (far + 40, 40 + 1), (far + 33, 33), (70, 70 - min(far, 70) + 1), (64, 32),
                 (65, 31), (95, 64), (96, 63), (n - 1, n - far), (n - 2, n - 1 - far), (n - 3, 0), (31, 0), (1, 0)):
        if 0 <= j <= i < n:
            q[i, :, :D] = (8.0 * keys[j] / keys[j].norm(dim=-1, keepdim=True)).float()
    down, w_uk, w_uv, cw, q, gates = (t.to(dtype) for t in (down, w_uk, w_uv, cw, q, gates))
    want = O.latent_core(q.to(F64), down.to(F64), gates.to(F64), w_uk.to(F64), w_uv.to(F64), cw.to(F64), m, eps)
    want = want.reshape(n, H * V)

    n_pages = 40
    cache = lattn.alloc_latent_cache(n_pages, R, P, dtype, device)
    cache.fill_(50.0)  # stale rows of freed pages
    table = lattn.rotary_table(m["rot"]["base"], P, 512, device)
    perm = (torch.randperm(n_pages - 1, generator=g) + 1).tolist()
    Q = 8
    proj = torch.cat([torch.randn(n, Q, generator=g).to(dtype), down, gates], 1).to(device)
    ones = torch.ones(Q, dtype=dtype, device=device)
    qd, ukd, uvd, cwd = q.to(device), w_uk.to(device), w_uv.to(device), cw.to(device)

    def rows_step(rows, nsplit=1):
        """rows: (page list, first position, count) of each row; one call of every op for all of them."""
        idx = torch.cat([torch.arange(a, a + c) for _, a, c in rows])
        pos = idx.to(torch.int32).to(device)
        slots = torch.cat([torch.tensor([pg[p // 32] * 32 + p % 32 for p in range(a, a + c)]) for pg, a, c in rows])
        bt = torch.zeros(len(rows), 16, dtype=torch.int32)
        for r, (pg, _, _) in enumerate(rows):
            bt[r, :len(pg)] = torch.tensor(pg, dtype=torch.int32)
        cu = i32(np.concatenate([[0], np.cumsum([c for _, _, c in rows])]).tolist(), device)
        ctx = i32([a + c for _, a, c in rows], device)
        pr = proj[idx.to(device)]
        lattn.latent_prep(pr, Q, R, P, ones, cwd, pos, slots.to(device), cache, table, eps)
        qq = qd[idx.to(device)].contiguous()
        q_lat = torch.bmm(qq[:, :, :D].transpose(0, 1), ukd.view(H, D, R)).transpose(0, 1).contiguous()
        max_q = max(c for _, _, c in rows)
        o = lattn.latent_attention(qq, q_lat, cache, bt.to(device), cu, ctx, max_q, D, P, m["scale"], window, table,
                                   gate=pr[:, Q + R + P:], nsplit=nsplit if max_q == 1 else 1)
        return torch.bmm(o.transpose(0, 1), uvd.view(H, V, R).transpose(1, 2)).transpose(0, 1).reshape(len(idx), H * V)

    def run(portions, pages, nsplit=1):
        outs, at = [], 0
        for c in portions:
            c = min(c, n - at)
            if c > 0:
                outs.append(rows_step([(pages, at, c)], nsplit))
                at += c
        assert at == n
        return torch.cat(outs).float().cpu()

    pa, pb = perm[:12], perm[12:24]
    t = tol(dtype) if dtype == torch.float32 else 8e-2
    assert rel_err(run([n], pa), want) < t
    assert rel_err(run([2] * (n // 2), pb), want) < t
    assert rel_err(run([1, 31, 1, 33, 30, 3, 1, 1, 9] + [40] * 9, pa), want) < t
    for ns in (1, 2, 5):
        got = run([n - 45] + [1] * 45, pb if ns != 2 else pa, nsplit=ns)
        assert rel_err(got, want) < t
    # two copies of the sequence at different places of their progress, in one call each time
    ga, gb, a, b = [], [], 0, 0
    for ca, cb in ((40, 1), (1, 70), (30, 1), (2, 2), (1, 1), (n - 74, n - 75)):
        out = rows_step([(pa, a, ca), (pb, b, cb)], nsplit=3).float().cpu()
        ga.append(out[:ca])
        gb.append(out[ca:])
        a, b = a + ca, b + cb
    assert a == n and b == n
    assert rel_err(torch.cat(ga), want) < t and rel_err(torch.cat(gb), want) < t


@pytest.mark.parametrize("device,dtype", OP_CASES)
@pytest.mark.parametrize("W,ff,E,top,limit", [(48, 20, 5, 2, 0.7), (24, 8, 3, 3, 2.0), (64, 64, 4, 1, 1.0),
                                              (128, 64, 10, 4, 7.0)])
def test_routed_experts(device, dtype, W, ff, E, top, limit):
    g = torch.Generator().manual_seed(7)
    mod = RoutedGLUExperts(W, ff, E, top, limit, 1.702, dtype, device)
    wt = {"router": torch.randn(E, W, generator=g) / W ** 0.5}
    for e in range(E):
        wt[f"e{e}.gate"] = torch.randn(ff, W, generator=g) * (3.0 / W ** 0.5)  # pre-activations beyond the limit
        wt[f"e{e}.up"] = torch.randn(ff, W, generator=g) * (3.0 / W ** 0.5)
        wt[f"e{e}.down"] = torch.randn(W, ff, generator=g) / ff ** 0.5
    wt = {k: v.to(dtype) for k, v in wt.items()}
    mod.router.data.copy_(wt["router"])
    for e in range(E):
        mod.gate_up.data[e, :ff].copy_(wt[f"e{e}.gate"])
        mod.gate_up.data[e, ff:].copy_(wt[f"e{e}.up"])
        mod.down.data[e].copy_(wt[f"e{e}.down"])
    spec = {"router": {"experts": E, "top": top}, "expert": {"ff": ff, "limit": limit}}
    for T in (1, 2, 37):
        h = torch.randn(T, W, generator=g).to(dtype)
        want = O.routed_experts(h.to(F64), wt, "", spec)
        with torch.no_grad():
            got = mod(h.to(device), h.float().to(device))
        assert rel_err(got.float().cpu(), want) < tol(dtype)
        # the weights are the softmax scores themselves: with more than `top` experts they sum to less than one
        if top < E:
            s = torch.softmax(h.to(F64) @ wt["router"].to(F64).T, -1)
            assert float(torch.topk(s, top, -1).values.sum(-1).min()) < 0.97


# ------------------------------------------------------------------------------------------ engine
def layer(heads=4, dim=16, rot=8, vdim=24, q_rank=20, kv_rank=32, window=37, ff=24, experts=5, top=2, limit=1.5,
          scale=0.3, base=10000.0):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
             "scale": scale, "rot": {"base": base, "dims": rot}}
    if window:
        mixer["mask"] = {"size": window}
    mlp = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}} if ff else None
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


def config(layers, width=48, vocab=101, eps=1e-5, taps=3, bigram=(53, 29, 5), loop=None):
    d = {"architecture": "Lufivik", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if taps:
        d["canon"] = {"taps": taps}
    if bigram:
        d["embedding"] = {"bigram": {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}}
    if loop:
        d["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return d


MIXED = config([layer(), layer(heads=2, dim=8, rot=4, vdim=8, kv_rank=16, window=5, ff=0),
                layer(heads=3, window=64, experts=3, top=3, ff=16)], loop=(1, 3, 2))


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
    assert rows_agree(rows, want, dtype), rel_err(rows, want)


def tokens_of(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


@pytest.mark.parametrize("device,dtype", CASES)
def test_whole_prompt_and_every_layer_run(device, dtype):
    eng, w = make_engine(MIXED, device, dtype)
    try:
        toks = tokens_of(75, MIXED["vocab"], 1)
        eng.runner.layer_trace = []
        got = replay(eng, cut("a", toks, [len(toks)]))
        trace, eng.runner.layer_trace = eng.runner.layer_trace, None
        layers = []
        O.forward(toks, w, MIXED, layers)
        assert len(trace) == len(layers) == 5  # layers 1 and 2 run twice
        for a, b in zip(trace, layers):
            assert rows_agree(a.cpu(), b, dtype)
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
    # one head, key size = rotary size = value size = ranks, as many experts as are chosen, one tap: values that hide
    # mix-ups; no loop
    config([layer(1, 16, 16, 16, 16, 16, 33, ff=16, experts=2, top=2)], width=16, taps=1),
    # sizes that are no multiples of 8 or of each other, no feed-forward in the middle, windows of one token and of
    # more than the sequence, other constants, the whole model looped
    config([layer(5, 12, 6, 20, 28, 36, 1, ff=10, experts=3, top=1, limit=0.4, scale=0.11, base=500.0),
            layer(3, 20, 2, 12, 36, 12, 500, ff=0), layer(6, 8, 10, 8, 12, 20, 7, ff=30, experts=7, top=3, limit=9.0)],
           width=40, vocab=67, eps=1e-3, taps=6, bigram=(7, 3, 2), loop=(0, 3, 2)),
    config([layer(4, 16, 8, 24, window=0)], width=24, bigram=None, taps=0),  # every earlier token seen; plain embedding
    config([layer(2, 8, 4, 8, ff=0), layer(2, 8, 4, 8, window=31)], width=56, taps=2, bigram=(1, 1, 1), loop=(1, 2, 3)),
    # nothing a multiple of 4: width, ranks, head sizes, expert width, vocabulary
    config([layer(3, 10, 6, 14, 18, 22, 13, ff=9, experts=4, top=2), layer(7, 6, 2, 5, 9, 11, 3, ff=0)], width=50, vocab=59,
           taps=5, bigram=(97, 3, 11), loop=(0, 1, 3)),
    # sizes the matrix-core paths take
    config([layer(4, 64, 64, 64, 64, 128, 40, ff=64, experts=4, top=2), layer(8, 64, 32, 64, 128, 64, 70, ff=128)],
           width=64, loop=(0, 1, 2)),
]


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("which", range(len(SHAPES)))
def test_other_sizes_windows_constants_and_loops(device, dtype, which):
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
    """Random layer lists (sizes, windows, constants, with and without feed-forward, loops) fed through random
    schedules of up to three live requests: portions of 1 .. 100 tokens, requests that skip steps; 32-bit, so that
    any deviation beyond rounding shows."""
    import random

    rng = random.Random(seed)
    for case in range(2):
        width, vocab, layers = rng.choice([32, 48, 72]), rng.choice([37, 101]), []
        for _ in range(rng.randint(1, 3)):
            E = rng.choice([2, 5, 9])
            layers.append(layer(rng.choice([1, 2, 3, 6]), rng.choice([8, 24, 64]), rng.choice([2, 8, 32]),
                                rng.choice([8, 40, 64]), rng.choice([8, 20]), rng.choice([8, 24, 72]),
                                rng.choice([1, 2, 31, 32, 33, 100, 0]), rng.choice([0, 12, 64]), E, rng.randint(1, E),
                                rng.choice([0.5, 2.0]), rng.choice([0.1, 0.3]), rng.choice([100.0, 10000.0])))
        a = rng.randint(0, len(layers))
        b = rng.randint(a, len(layers))
        cfg = config(layers, width=width, vocab=vocab, eps=rng.choice([1e-5, 1e-6]), taps=rng.choice([0, 1, 2, 4]),
                     bigram=rng.choice([None, (11, 5, 3), (200, 17, 3)]),
                     loop=rng.choice([None, (a, b, rng.randint(1, 3))]))
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
    cfg = config([layer(window=40), layer(heads=2, window=9, ff=0)], taps=4)
    eng, w = make_engine(cfg, device, dtype)
    try:
        for n in (1, 2, 3, 4, 5):  # shorter than, as long as and longer than the convolution
            toks = tokens_of(n, cfg["vocab"], 40 + n)
            check_against_oracle(replay(eng, cut(f"s{n}", toks, [1])), toks, w, cfg, dtype, f"s{n}")
            check_against_oracle(replay(eng, cut(f"w{n}", toks, [n])), toks, w, cfg, dtype, f"w{n}")
        toks = tokens_of(230, cfg["vocab"], 44)  # the windows pass over decoded tokens several times
        check_against_oracle(replay(eng, cut("long", toks, [20, 1])), toks, w, cfg, dtype, "long")
    finally:
        eng.destroy()


@pytest.mark.parametrize("device,dtype", CASES)
def test_greedy_generation_through_the_engine(device, dtype):
    """The engine's own entry point: prompts of unequal length generated together, prefill plans, then decode
    plans (captured graphs on the GPU), more requests than request slots."""
    cfg = config([layer(window=21), layer(heads=2, dim=16, vdim=16, window=70, ff=0)], vocab=61, loop=(0, 2, 2))
    eng, w = make_engine(cfg, device, dtype, max_running=3, score=False)
    try:
        prompts = [tokens_of(n, cfg["vocab"], 50 + n) for n in (3, 41, 18, 1, 66)]
        res = eng.generate_blocking(prompts, max_new_tokens=12, greedy=True)
        agree = 0
        for p, r in zip(prompts, res):
            assert r.finish_reason == "length" and len(r.output_tokens) == 12
            want = O.greedy(p, 12, w, cfg)
            if dtype == "float32":
                assert r.output_tokens == want
            else:  # a near-tie (of two tokens, of two experts) may flip under bf16
                agree += r.output_tokens[0] == want[0]
        assert dtype == "float32" or agree >= 4
        assert eng.sched.num_free_state_slots() == 3
    finally:
        eng.destroy()


@pytest.mark.parametrize("device", DEVICES)
def test_served_from_a_checkpoint_directory(device, tmp_path):
    """The framework's own path from a directory with config.json and model.safetensors: the model class is chosen by
    the configuration, the weights come through the engine's loader; several decode steps per plan."""
    from areal_vllm_amd.models import build_model

    cfg_dict = config([layer(2, 8, 4, 16, 12, 16, 9), layer(3, 8, 8, 8, 8, 24, 30, ff=0)], width=32, vocab=53, loop=(1, 2, 2))
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

    cfg_dict = config([layer(2, 8, 4, 8, 12, 16, 11, ff=12, experts=3, top=2), layer(1, 8, 8, 16, 8, 8, 0, ff=0)], width=24,
                      vocab=41, taps=2, loop=(0, 1, 2))
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
    assert cfg.family == "lufivik" and cfg.n_layers == 3 and cfg.has_recurrent_state
    assert cfg.layer_runs == [0, 1, 2, 0, 1, 2] and ModelConfig.from_hf_dict(MIXED).layer_runs == [0, 1, 2, 1, 2]
    from areal_vllm_amd.models import build_model

    m = build_model(cfg, dtype=torch.float32)
    m.flatten()
    m.init_weights(seed=4)
    assert sum(p.numel() for p in m.parameters()) == cfg.n_params()
    m.save_checkpoint(str(tmp_path))
    cfg2 = ModelConfig.from_pretrained(str(tmp_path))
    assert cfg2.layers == cfg.layers and cfg2.loop == cfg.loop and cfg2.bigram == cfg.bigram
    assert cfg2.canon_taps == cfg.canon_taps
    m2 = build_model(cfg2, dtype=torch.float32)
    m2.flatten()
    m2.load_checkpoint(str(tmp_path))
    for (n1, a), (n2, b) in zip(m.checkpoint_tensors().items(), m2.checkpoint_tensors().items()):
        assert n1 == n2 and torch.equal(a, b)
    with pytest.raises(ValueError):
        ModelConfig.from_hf_dict(config([dict(layer(), type="conv")]))
    with pytest.raises(ValueError):
        ModelConfig.from_hf_dict(config([layer()], loop=(1, 0, 2)))
