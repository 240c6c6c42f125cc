"""Sublayers between two norms on an fp32 residual stream, and what feeds them.

    h        = LN(x)                                   layer norm with weight and bias, fp32 statistics
    x       <- x + s * LN'(y * sigmoid(r))             y: the sublayer's output, r: gate logits (a projection of h),
                                                       s: one scale per channel ("layer scale")
    conv(h)_t = sum_j w[:, j] * h_(t - taps + 1 + j)   causal per-channel convolution over time; the last taps - 1
                                                       inputs of every sequence live in a state slot
    x_0      = LN(E[tok] + B[(prev * a + tok * b) mod n])   token plus hashed-bigram embedding (row n of B for a
                                                       sequence's first token); the previous token lives in a slot

GPU: ``csrc/hip/sandwich.hip``. CPU: PyTorch formulations of the same arithmetic (fp32).

Rows of a packed batch are described as everywhere in the serving path: row b owns tokens cu_q[b]:cu_q[b+1], its
first token has position first_pos[b] and its state lives in slot state_slots[b] (negative: the row is padding and
touches nothing).
"""
from typing import Optional, Tuple

import torch

from . import _lib as L


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float, dtype: torch.dtype,
               want32: bool = True) -> Tuple[Optional[torch.Tensor], torch.Tensor]:
    """x fp32 [T, W] -> (LN(x) in fp32 or None when `want32` is False, LN(x) in `dtype`; one tensor when `dtype` is
    fp32)."""
    assert x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous()
    T, W = x.shape
    if L.use_hip(x):
        assert weight.dtype == dtype and bias.dtype == dtype and weight.numel() == W and bias.numel() == W
        f32 = dtype == torch.float32
        o32 = torch.empty_like(x) if (want32 or f32) else None
        oc = o32 if f32 else torch.empty(T, W, dtype=dtype, device=x.device)
        L.check(L.lib().areal_layer_norm32(L.ptr(x), L.ptr(weight), L.ptr(bias), L.ptr(o32),
                                           None if f32 else L.ptr(oc), L.c_int(T), L.c_int(W), L.c_float(eps),
                                           L.c_int(L.dtype_flag(weight)), L.stream_ptr()), "layer_norm32")
        return o32, oc
    m = x.mean(-1, keepdim=True)
    d = x - m
    h = d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * weight.float() + bias.float()
    return h, (h if dtype == torch.float32 else h.to(dtype))


def gated_norm_add(x: torch.Tensor, y: torch.Tensor, gate: Optional[torch.Tensor], weight: torch.Tensor,
                   bias: torch.Tensor, scale: Optional[torch.Tensor], eps: float,
                   next_norm: Optional[Tuple[torch.Tensor, torch.Tensor]] = None, want32: bool = True):
    """x <- x + scale * LN(y * sigmoid(gate); weight, bias) in place on the fp32 stream x [T, W]; y and gate [T, W] in
    the compute dtype (gate / scale None: left out). With `next_norm` = (weight, bias) the norm of the new x that the
    next sublayer reads is produced by the same launch: returns (x, h32 or None, h in the compute dtype)."""
    assert x.dtype == torch.float32 and x.is_contiguous() and y.shape == x.shape
    T, W = x.shape
    dtype = y.dtype
    if L.use_hip(x):
        assert y.is_contiguous() and (gate is None or (gate.is_contiguous() and gate.dtype == dtype))
        assert weight.dtype == dtype and bias.dtype == dtype and (scale is None or scale.dtype == dtype)
        f32 = dtype == torch.float32
        h32 = hc = None
        if next_norm is not None:
            h32 = torch.empty_like(x) if (want32 or f32) else None
            hc = h32 if f32 else torch.empty(T, W, dtype=dtype, device=x.device)
        L.check(L.lib().areal_gated_norm_add(
            L.ptr(x), L.ptr(y), L.ptr(gate), L.ptr(weight), L.ptr(bias), L.ptr(scale),
            L.ptr(next_norm[0]) if next_norm else None, L.ptr(next_norm[1]) if next_norm else None, L.ptr(h32),
            None if (f32 or hc is None) else L.ptr(hc), L.c_int(T), L.c_int(W), L.c_float(eps),
            L.c_int(L.dtype_flag(y)), L.stream_ptr()), "gated_norm_add")
        return x, h32, hc
    z = y.float()
    if gate is not None:
        z = z * torch.sigmoid(gate.float())
    m = z.mean(-1, keepdim=True)
    d = z - m
    z = d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * weight.float() + bias.float()
    if scale is not None:
        z = z * scale.float()
    x.add_(z)
    if next_norm is None:
        return x, None, None
    h32, hc = layer_norm(x, next_norm[0], next_norm[1], eps, dtype)
    return x, h32, hc


def canon_conv(h: torch.Tensor, weight: torch.Tensor, state: Optional[torch.Tensor], cu_q: torch.Tensor,
               first_pos: torch.Tensor, state_slots: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """h fp32 [T, W] -> h + conv(h) in `dtype`, with weight [W, taps] and state fp32 [slots, taps - 1, W] (entry k of a
    slot: the input taps - 1 - k tokens before the row's first token; None when taps == 1). Positions before a
    sequence's start count as zeros, so a slot's old contents do not matter to a row that starts at position 0.
    Afterwards every row's slot holds its last taps - 1 inputs."""
    assert h.dtype == torch.float32 and h.is_contiguous()
    T, W = h.shape
    taps = weight.shape[1]
    assert weight.shape[0] == W and weight.is_contiguous()
    assert taps == 1 or (state is not None and state.shape[1:] == (taps - 1, W) and state.dtype == torch.float32)
    B = cu_q.numel() - 1
    if L.use_hip(h):
        assert weight.dtype == dtype and cu_q.dtype == torch.int32 and first_pos.dtype == torch.int32
        assert state_slots.dtype == torch.int32
        out = torch.empty(T, W, dtype=dtype, device=h.device)
        L.check(L.lib().areal_canon_conv(L.ptr(h), L.ptr(weight), L.ptr(state), L.ptr(cu_q), L.ptr(first_pos),
                                         L.ptr(state_slots), L.ptr(out), L.c_int(B), L.c_int(T), L.c_int(W),
                                         L.c_int(taps), L.c_int(L.dtype_flag(weight)), L.stream_ptr()), "canon_conv")
        return out
    out = torch.empty_like(h)
    w = weight.float()
    cq, fp, ss = cu_q.tolist(), first_pos.tolist(), state_slots.tolist()
    K = taps - 1
    for b in range(B):
        lo, hi = cq[b], cq[b + 1]
        if hi <= lo or ss[b] < 0:
            out[lo:hi] = h[lo:hi]
            continue
        if K == 0:
            out[lo:hi] = h[lo:hi] * (1.0 + w[:, 0])
            continue
        hist = state[ss[b]].clone()  # [K, W], oldest first
        if fp[b] < K:  # before the sequence's start there is nothing
            hist[:K - fp[b]] = 0
        ext = torch.cat([hist, h[lo:hi]], 0)
        n = hi - lo
        acc = h[lo:hi].clone()
        for j in range(taps):
            acc += w[:, j] * ext[j:j + n]
        out[lo:hi] = acc
        state[ss[b]] = ext[n:n + K]
    return out if dtype == torch.float32 else out.to(dtype)


def embed_bigram_norm(tokens: torch.Tensor, embed: torch.Tensor, bigram: Optional[torch.Tensor], mul_prev: int,
                      mul_cur: int, weight: torch.Tensor, bias: torch.Tensor, eps: float, cu_q: torch.Tensor,
                      first_pos: torch.Tensor, state_slots: torch.Tensor, prev_state: Optional[torch.Tensor]
                      ) -> torch.Tensor:
    """tokens int64 [T] -> fp32 stream [T, W] = LN(embed[tok] + bigram[row]); row = (prev * mul_prev + tok * mul_cur)
    mod buckets with buckets = bigram rows - 1, the last row for a token at position 0. `prev_state` int32 [slots]:
    the last token every sequence has seen (read by a row's first token, then replaced by the row's last token).
    `bigram` None: the token embedding alone."""
    T = tokens.numel()
    W = embed.shape[1]
    B = cu_q.numel() - 1
    if L.use_hip(embed):
        assert tokens.dtype == torch.int64 and embed.is_contiguous() and (bigram is None or bigram.is_contiguous())
        assert bigram is None or (bigram.dtype == embed.dtype and prev_state is not None
                                  and prev_state.dtype == torch.int32)
        out = torch.empty(T, W, dtype=torch.float32, device=embed.device)
        L.check(L.lib().areal_embed_bigram_norm(
            L.ptr(tokens), L.ptr(embed), L.ptr(bigram), L.c_int(bigram.shape[0] - 1 if bigram is not None else 0),
            L.c_int64(mul_prev), L.c_int64(mul_cur), L.ptr(weight), L.ptr(bias), L.c_float(eps), L.ptr(cu_q),
            L.ptr(first_pos), L.ptr(state_slots), L.ptr(prev_state), L.ptr(out), L.c_int(B), L.c_int(T), L.c_int(W),
            L.c_int(embed.shape[0]), L.c_int(L.dtype_flag(embed)), L.stream_ptr()), "embed_bigram_norm")
        return out
    x = embed[tokens].float()
    if bigram is not None:
        n = bigram.shape[0] - 1
        cq, fp, ss = cu_q.tolist(), first_pos.tolist(), state_slots.tolist()
        rows = torch.zeros(T, dtype=torch.long)
        live = torch.zeros(T, dtype=torch.bool)
        for b in range(B):
            lo, hi = cq[b], cq[b + 1]
            if hi <= lo or ss[b] < 0:
                continue
            tk = tokens[lo:hi].cpu().long()
            prev = torch.cat([prev_state[ss[b]:ss[b] + 1].cpu().long(), tk[:-1]])
            r = (prev * mul_prev + tk * mul_cur) % n
            if fp[b] == 0:
                r[0] = n
            rows[lo:hi] = r
            live[lo:hi] = True
            prev_state[ss[b]] = int(tk[-1])
        add = bigram[rows.to(bigram.device)].float()
        x = x + add * live.to(add.device).unsqueeze(-1)
    m = x.mean(-1, keepdim=True)
    d = x - m
    return d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * weight.float() + bias.float()
