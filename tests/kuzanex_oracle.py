"""Plain, slow formulation of the Kuzanex design in float64: one function per mechanism, whole sequences at a
time, no cache, no batching. The tests compare the framework against it; it shares no code with the framework.

Notation: x [n, W] residual stream of one sequence (positions 0 .. n-1); weights `w` is a dict name -> tensor with
the checkpoint's names ('l3.mix.q', 'l3.mlp.up.b', ...); linear weights are [out, in].
"""
import math

import torch

F64 = torch.float64


def unit_rms(z, eps):
    return z / torch.sqrt((z * z).mean(-1, keepdim=True) + eps)


def scalar_norm(z, gain, eps):
    return unit_rms(z, eps) * gain.to(F64).reshape(())


def xielu(z, pq):
    p, q = float(pq[0]), float(pq[1])
    sp = math.log1p(math.exp(p))
    sq = math.log1p(math.exp(q))
    pos = sp * z * z + z / 2
    neg = (0.5 + sq) * (torch.exp(torch.clamp(z, max=0.0)) - 1 - z) + z / 2
    return torch.where(z > 0, pos, neg)


def feed_forward(x, w, pre):
    up = x @ w[pre + "up"].to(F64).T + w[pre + "up.b"].to(F64)
    return xielu(up, w[pre + "act"].to(F64)) @ w[pre + "down"].to(F64).T + w[pre + "down.b"].to(F64)


def shaped_scores(q, k, scale, softcap, talk, window):
    """q [n, H, D], k [n, H, D] (key heads already repeated) -> masked pre-softmax scores [H, n, n]."""
    n, H, _ = q.shape
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    i = torch.arange(n).view(n, 1)
    j = torch.arange(n).view(1, n)
    slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=F64)
    s = s - slopes.view(H, 1, 1) * (i - j).to(F64)
    if talk is not None:
        s = torch.einsum("hg,gij->hij", talk.to(F64), s)
    seen = (i - j >= 0)
    if window:
        seen = seen & (i - j < window)
    return s.masked_fill(~seen, float("-inf"))


def sink_softmax(s):
    """exp(s_j) / (1 + sum_j exp(s_j)) along the last axis."""
    m = torch.clamp(s.max(-1, keepdim=True).values, min=0.0)
    e = torch.exp(s - m)
    return e / (torch.exp(-m) + e.sum(-1, keepdim=True))


def attention(x, w, pre, m, eps):
    n = x.shape[0]
    H, G, D = m["heads"], m.get("kv_heads", m["heads"]), m["dim"]
    V = m.get("vdim", D)
    q = (x @ w[pre + "q"].to(F64).T + w[pre + "q.b"].to(F64)).view(n, H, D)
    k = (x @ w[pre + "k"].to(F64).T + w[pre + "k.b"].to(F64)).view(n, G, D)
    v = (x @ w[pre + "v"].to(F64).T + w[pre + "v.b"].to(F64)).view(n, G, V)
    q = unit_rms(q, eps) * w[pre + "q.norm"].to(F64)
    k = unit_rms(k, eps) * w[pre + "k.norm"].to(F64)
    k = k.repeat_interleave(H // G, 1)
    v = v.repeat_interleave(H // G, 1)
    window = (m.get("mask") or {}).get("size") or 0
    p = sink_softmax(shaped_scores(q, k, m["scale"], m.get("softcap") or 0.0, w.get(pre + "talk"), window))
    o = torch.einsum("hij,jhv->ihv", p, v)
    gate = torch.sigmoid(x @ w[pre + "g"].to(F64).T)  # [n, H]
    return (o * gate.unsqueeze(-1)).reshape(n, H * V) @ w[pre + "o"].to(F64).T


def mlstm_recurrence(q, k, v, ig, fg):
    """One head. q, k [n, D]; v [n, V]; log gates ig, fg [n] -> read-out [n, V] (already divided)."""
    n, D = q.shape
    S = torch.zeros(D, v.shape[1], dtype=F64)
    nv = torch.zeros(D, dtype=F64)
    m = 0.0
    out = []
    for t in range(n):
        f, i = float(fg[t]), float(ig[t])
        m_new = max(f + m, i)
        a, b = math.exp(f + m - m_new), math.exp(i - m_new)
        S = a * S + b * torch.outer(k[t], v[t])
        nv = a * nv + b * k[t]
        m = m_new
        den = max(abs(float(nv @ q[t])), math.exp(-m)) + 1e-6
        out.append((S.T @ q[t]) / den)
    return torch.stack(out)


def mlstm(x, w, pre, m, eps):
    n = x.shape[0]
    H, D = m["heads"], m["dim"]
    V = m.get("vdim", D)
    cap = m["gate_cap"]
    q = (x @ w[pre + "q"].to(F64).T).view(n, H, D) * D ** -0.5
    k = (x @ w[pre + "k"].to(F64).T).view(n, H, D)
    v = (x @ w[pre + "v"].to(F64).T).view(n, H, V)
    ig = cap * torch.tanh((x @ w[pre + "i"].to(F64).T + w[pre + "i.b"].to(F64)) / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh((x @ w[pre + "f"].to(F64).T + w[pre + "f.b"].to(F64)) / cap))
    heads = [unit_rms(mlstm_recurrence(q[:, h], k[:, h], v[:, h], ig[:, h], fg[:, h]), eps) for h in range(H)]
    y = torch.cat(heads, -1) * w[pre + "norm"].to(F64) * torch.sigmoid(x @ w[pre + "g"].to(F64).T)
    return y @ w[pre + "o"].to(F64).T


def forward(tokens, w, cfg, layers_out=None):
    """Logits [n, vocab] of one sequence; `cfg` is the config.json dictionary."""
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    x = w["embed"].to(F64)[torch.as_tensor(tokens)]
    for li, layer in enumerate(cfg["layers"]):
        pre = f"l{li}."
        mix = attention if layer["type"] == "attention" else mlstm
        x = scalar_norm(alpha * x + mix(x, w, pre + "mix.", layer["mixer"], eps), w[pre + "norm1"], eps)
        if layer.get("mlp") is not None:
            x = scalar_norm(alpha * x + feed_forward(x, w, pre + "mlp."), w[pre + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x)
    return scalar_norm(x, w["final.norm"], eps) @ w["head"].to(F64).T


def greedy(prompt, n_new, w, cfg):
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(forward(toks, w, cfg)[-1].argmax()))
    return toks[len(prompt):]
