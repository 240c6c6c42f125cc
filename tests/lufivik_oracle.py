"""Plain, slow float64 formulation of the Lufivik design, one function per mechanism, written from its equations.
Shares no code with the framework: tests compare the framework's ops, runner and engine against it.

Notation: W width, t time, H heads. Weights are a dict {checkpoint name: tensor}; linear weights are [out, in].
"""
import math

import torch

F64 = torch.float64


def f64(t):
    return t.to(F64)


def layer_norm(x, w, b, eps):
    """(x - mean) / sqrt(mean squared deviation + eps) * w + b over the last axis."""
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def rotate(x, positions, base):
    """x [n, ..., P]: entry i pairs with entry i + P/2; the pair turns by the angle position * base^(-2i/P)."""
    P = x.shape[-1]
    out = torch.empty_like(x)
    for i in range(P // 2):
        ang = positions.to(F64) * (base ** (-2.0 * i / P))
        ang = ang.view(-1, *([1] * (x.dim() - 2)))
        u, v = x[..., i], x[..., i + P // 2]
        out[..., i] = u * torch.cos(ang) - v * torch.sin(ang)
        out[..., i + P // 2] = v * torch.cos(ang) + u * torch.sin(ang)
    return out


def causal_conv(h, w):
    """h [n, W], w [W, taps]: out_t = sum_j w[:, j] h_(t - taps + 1 + j), nothing before t = 0."""
    n, taps = h.shape[0], w.shape[1]
    out = torch.zeros_like(h)
    for t in range(n):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    rows = []
    for t, tok in enumerate(tokens):
        rows.append(buckets if t == 0 else (tokens[t - 1] * mul_prev + tok * mul_cur) % buckets)
    return rows


def latent_core(q, down, gate_logits, w_uk, w_uv, c_weight, m, eps):
    """q [n, H, D + P] (rotary part last, unrotated), down [n, R + P] (raw latent | raw rotary key), gate logits
    [n, H] -> gated head outputs [n, H, V]. Keys and values are expanded from the normalised latent per head."""
    n = q.shape[0]
    H, D, P, V, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    base, scale, window = m["rot"]["base"], m["scale"], (m.get("mask") or {}).get("size") or 0
    pos = torch.arange(n)
    c = rms_norm(down[:, :R], c_weight, eps)
    k_rot = rotate(down[:, R:], pos, base)
    q_rot = rotate(q[:, :, D:], pos, base)
    k = (c @ w_uk.T).view(n, H, D)
    v = (c @ w_uv.T).view(n, H, V)
    gate = torch.sigmoid(gate_logits)
    out = torch.zeros(n, H, V, dtype=F64)
    i, j = pos.view(n, 1), pos.view(1, n)
    seen = (j <= i) & ((i - j < window) if window > 0 else (j <= i))
    for hd in range(H):
        s = (q[:, hd, :D] @ k[:, hd].T + q_rot[:, hd] @ k_rot.T) * scale
        w = torch.softmax(s.masked_fill(~seen, -math.inf), -1)
        out[:, hd] = (w @ v[:, hd]) * gate[:, hd:hd + 1]
    return out


def latent_attention(h, wt, p, m, eps):
    """The whole mixer on its input h [n, W]; wt: weights, p: prefix of the mixer's tensors, m: its config."""
    n = h.shape[0]
    H, D, P = m["heads"], m["dim"], m["rot_dim"]
    q = (rms_norm(h @ f64(wt[p + "dq"]).T, f64(wt[p + "dq.norm"]), eps) @ f64(wt[p + "uq"]).T).view(n, H, D + P)
    out = latent_core(q, h @ f64(wt[p + "dkv"]).T, h @ f64(wt[p + "g"]).T, f64(wt[p + "uk"]), f64(wt[p + "uv"]),
                      f64(wt[p + "dkv.norm"]), m, eps)
    return out.reshape(n, -1) @ f64(wt[p + "o"]).T


def routed_experts(h, wt, p, e):
    """h [n, W]: softmax over all experts, the `top` largest scores weigh their experts' outputs as they are."""
    E, top, lim = e["router"]["experts"], e["router"]["top"], e["expert"]["limit"]
    s = torch.softmax(h @ f64(wt[p + "router"]).T, -1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for ex in torch.argsort(s[t], descending=True, stable=True)[:top].tolist():
            g = torch.clamp(f64(wt[p + f"e{ex}.gate"]) @ h[t], max=lim)
            u = torch.clamp(f64(wt[p + f"e{ex}.up"]) @ h[t], -lim, lim)
            out[t] += s[t, ex] * (f64(wt[p + f"e{ex}.down"]) @ (g * torch.sigmoid(1.702 * g) * (u + 1.0)))
    return out


def layer_runs(cfg):
    n, lp = len(cfg["layers"]), cfg.get("loop")
    if not lp:
        return list(range(n))
    return list(range(lp["start"])) + list(range(lp["start"], lp["stop"])) * lp["times"] + list(range(lp["stop"], n))


def forward(tokens, wt, cfg, layers_out=None):
    """Logits [n, vocab] (float64) of a whole sequence; `layers_out` collects the stream after every layer run."""
    eps = cfg["norm"]["eps"]
    x = f64(wt["embed"])[tokens]
    big = (cfg.get("embedding") or {}).get("bigram")
    if big:
        x = x + f64(wt["bigram"])[bigram_rows(tokens, big["buckets"], big["mul_prev"], big["mul_cur"])]
    x = layer_norm(x, f64(wt["embed.norm"]), f64(wt["embed.norm.b"]), eps)
    for li in layer_runs(cfg):
        spec, p = cfg["layers"][li], f"l{li}."

        def ln(z, name):
            return layer_norm(z, f64(wt[p + name]), f64(wt[p + name + ".b"]), eps)

        h = ln(x, "norm1")
        gate = torch.sigmoid(h @ f64(wt[p + "rg1"]).T + f64(wt[p + "rg1.b"]))
        if (cfg.get("canon") or {}).get("taps"):
            h = h + causal_conv(h, f64(wt[p + "canon1"]))
        y = latent_attention(h, wt, p + "mix.", spec["mixer"], eps) * gate
        x = x + ln(y, "norm1b") * f64(wt[p + "ls1"])
        if spec.get("mlp"):
            h = ln(x, "norm2")
            gate = torch.sigmoid(h @ f64(wt[p + "rg2"]).T + f64(wt[p + "rg2.b"]))
            y = routed_experts(h, wt, p + "mlp.", spec["mlp"]) * gate
            x = x + ln(y, "norm2b") * f64(wt[p + "ls2"])
        if layers_out is not None:
            layers_out.append(x.clone())
    return layer_norm(x, f64(wt["final.norm"]), f64(wt["final.norm.b"]), eps) @ f64(wt["head"]).T


def greedy(prompt, n_new, wt, cfg):
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(torch.argmax(forward(toks, wt, cfg)[-1])))
    return toks[len(prompt):]
