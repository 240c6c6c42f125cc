"""Matrix-memory recurrence (mLSTM) with a carried fp32 state per request slot.

GPU: ``csrc/hip/mlstm.hip``. CPU: the same recurrence in PyTorch, token by token (fp32).
"""
import math
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from . import _lib as L


class RecurrentState:
    """State slots of one mLSTM layer: S [slots, heads, D, V], n [slots, heads, D], m [slots, heads], fp32. A row
    that starts at position 0 ignores what its slot held, so slots are handed on without clearing."""

    def __init__(self, n_slots: int, n_heads: int, k_dim: int, v_dim: int, device):
        self.S = torch.zeros(n_slots, n_heads, k_dim, v_dim, dtype=torch.float32, device=device)
        self.n = torch.zeros(n_slots, n_heads, k_dim, dtype=torch.float32, device=device)
        self.m = torch.zeros(n_slots, n_heads, dtype=torch.float32, device=device)

    def nbytes(self) -> int:
        return 4 * (self.S.numel() + self.n.numel() + self.m.numel())


def mlstm_gates(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], n_heads: int, cap: float
                ) -> Tuple[torch.Tensor, torch.Tensor]:
    """x [T, W]; w [2 heads, W] (input-gate rows, then forget-gate rows); -> log input gate, log forget gate
    [T, heads] fp32: i = cap tanh(z_i / cap), f = logsigmoid(cap tanh(z_f / cap)); dot products accumulate in fp32."""
    T, W = x.shape
    if L.use_hip(x):
        assert x.is_contiguous() and w.is_contiguous() and w.dtype == x.dtype and w.shape == (2 * n_heads, W)
        ig = torch.empty(T, n_heads, dtype=torch.float32, device=x.device)
        fg = torch.empty_like(ig)
        L.check(L.lib().areal_mlstm_gates(L.ptr(x), L.ptr(w), L.ptr(bias), L.ptr(ig), L.ptr(fg), L.c_int(T), L.c_int(W),
                                          L.c_int(n_heads), L.c_float(cap), L.c_int(L.dtype_flag(x)), L.stream_ptr()),
                "mlstm_gates")
        return ig, fg
    z = x.float() @ w.float().t()
    if bias is not None:
        z = z + bias.float()
    if cap > 0:
        z = cap * torch.tanh(z / cap)
    return z[:, :n_heads].contiguous(), F.logsigmoid(z[:, n_heads:]).contiguous()


def mlstm_scan(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, ig: torch.Tensor, fg: torch.Tensor,
               cu_q: torch.Tensor, first_pos: torch.Tensor, state_slots: torch.Tensor, state: RecurrentState,
               max_q: int = 1) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Advance the state of every row's slot over the row's tokens. proj [T, *] holds heads x D queries at column
    q_off, heads x D keys at k_off, heads x V values at v_off. first_pos [B] int32: position of each row's first
    token (0: fresh state); state_slots [B] int32 (negative: the row is skipped). `max_q`: the longest row; from 16
    tokens on (key size <= 128) the GPU runs the chunk-parallel kernel on the fp32 matrix cores, otherwise the
    token-by-token one. Returns the unnormalised read-out [T, heads, V], n . q [T, heads] and m [T, heads], fp32."""
    T = proj.shape[0]
    NH, D, V = state.S.shape[1], state.S.shape[2], state.S.shape[3]
    B = cu_q.numel() - 1
    hip = L.use_hip(proj)
    new = torch.empty if hip else torch.zeros  # the kernel writes every element (zeros for skipped rows)
    hbuf = new(T, NH, V, dtype=torch.float32, device=proj.device)
    nq = new(T, NH, dtype=torch.float32, device=proj.device)
    mt = new(T, NH, dtype=torch.float32, device=proj.device)
    if hip:
        assert proj.stride(1) == 1 and cu_q.dtype == torch.int32 and first_pos.dtype == torch.int32
        assert state_slots.dtype == torch.int32 and ig.is_contiguous() and fg.is_contiguous()
        if D > 256:
            raise RuntimeError("mLSTM scan: key size above 256 is not built")
        L.check(L.lib().areal_mlstm_scan(
            L.ptr(proj), L.c_int64(proj.stride(0)), L.c_int(q_off), L.c_int(k_off), L.c_int(v_off), L.ptr(ig),
            L.ptr(fg), L.ptr(cu_q), L.ptr(first_pos), L.ptr(state_slots), L.ptr(state.S), L.ptr(state.n),
            L.ptr(state.m), L.ptr(hbuf), L.ptr(nq), L.ptr(mt), L.c_int(B), L.c_int(NH), L.c_int(D), L.c_int(V),
            L.c_int(int(max_q)), L.c_int(L.dtype_flag(proj)), L.stream_ptr()), "mlstm_scan")
        return hbuf, nq, mt
    cq, fp, sl = cu_q.tolist(), first_pos.tolist(), state_slots.tolist()
    qs = 1.0 / math.sqrt(D)
    for b in range(B):
        if sl[b] < 0 or cq[b + 1] <= cq[b]:
            continue
        if fp[b] == 0:
            S = torch.zeros(NH, D, V)
            n = torch.zeros(NH, D)
            m = torch.zeros(NH)
        else:
            S, n, m = state.S[sl[b]].clone(), state.n[sl[b]].clone(), state.m[sl[b]].clone()
        for t in range(cq[b], cq[b + 1]):
            q = proj[t, q_off:q_off + NH * D].float().view(NH, D) * qs
            k = proj[t, k_off:k_off + NH * D].float().view(NH, D)
            v = proj[t, v_off:v_off + NH * V].float().view(NH, V)
            m2 = torch.maximum(fg[t] + m, ig[t])
            a, bb = torch.exp(fg[t] + m - m2), torch.exp(ig[t] - m2)
            m = m2
            S = a.view(NH, 1, 1) * S + bb.view(NH, 1, 1) * k.unsqueeze(2) * v.unsqueeze(1)
            n = a.view(NH, 1) * n + bb.view(NH, 1) * k
            hbuf[t] = torch.einsum("hdv,hd->hv", S, q)
            nq[t] = (n * q).sum(-1)
            mt[t] = m
        state.S[sl[b]], state.n[sl[b]], state.m[sl[b]] = S, n, m
    return hbuf, nq, mt


def mlstm_out(hbuf: torch.Tensor, nq: torch.Tensor, mt: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor,
              eps: float) -> torch.Tensor:
    """y = h / (max(|n.q|, exp(-m)) + 1e-6); per head y / rms(y); times weight [heads V], times sigmoid(gate).
    gate: [T, heads V] view (unit stride along the last axis) in the compute dtype; returns [T, heads V] in it."""
    T, NH, V = hbuf.shape
    if L.use_hip(hbuf):
        assert gate.stride(1) == 1 and weight.dtype == gate.dtype and weight.numel() == NH * V
        out = torch.empty(T, NH * V, dtype=gate.dtype, device=gate.device)
        L.check(L.lib().areal_mlstm_out(L.ptr(hbuf), L.ptr(nq), L.ptr(mt), L.ptr(gate), L.c_int64(gate.stride(0)),
                                        L.ptr(weight), L.ptr(out), L.c_int(T), L.c_int(NH), L.c_int(V), L.c_float(eps),
                                        L.c_int(L.dtype_flag(gate)), L.stream_ptr()), "mlstm_out")
        return out
    y = hbuf / (torch.maximum(nq.abs(), torch.exp(-mt)) + 1e-6).unsqueeze(-1)
    y = y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + eps)
    return (y.reshape(T, NH * V) * weight.float() * torch.sigmoid(gate.float())).to(gate.dtype)
