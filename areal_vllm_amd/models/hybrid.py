"""Layer-list decoders: every layer names its own token mixer, the residual stream is fp32 and normalised AFTER
each sum. The Kuzanex design is the first member: sliding-window attention with shaped scores and mLSTM layers in
any order, feed-forward blocks with the xIELU activation, one gain per norm.

Layer:      x <- norm1(alpha x + mixer(x));  x <- norm2(alpha x + ff(x))       (sublayers read x itself)
Norm:       z / sqrt(mean(z^2) + eps) * g, g one number.
Output:     logits = head . norm(x).

The mechanisms are separate modules with their constants as constructor arguments (``WindowAttentionMixer``,
``MLSTMMixer``, ``XieluMLP``); what they compute is documented with their kernels (``ops/window_attention.py``,
``ops/mlstm.py``, ``ops/post_norm.py``). The modules hold parameters and know how to run ONE step on the tensors of a
batch plan; paged caches, state slots and the loop over layers belong to the model runner
(``inference/model_runner.py::HybridModelRunner``).
"""
import dataclasses
import json
import os
from typing import Any, Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops
from ..ops import mlstm as mlstm_ops
from ..ops import post_norm, window_attention as wattn
from .config import ModelConfig
from .transformer import FlatParams


@dataclasses.dataclass
class HybridConfig(ModelConfig):
    """`layers`: one dict per layer, {"type": "attention" | "mlstm", "mixer": {...sizes and constants...},
    "mlp": {"kind": "dense", "ff": F} | None}, as the checkpoint's config.json lists them."""
    layers: List[Dict[str, Any]] = dataclasses.field(default_factory=list)
    postln_alpha: float = 1.0

    @property
    def has_recurrent_state(self) -> bool:
        return any(l["type"] == "mlstm" for l in self.layers)

    def n_params(self, with_embedding: bool = True) -> int:
        W, n = self.hidden_size, 1
        for l in self.layers:
            m = l["mixer"]
            if l["type"] == "attention":
                H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
                n += (W + 1) * ((H + G) * D + G * V + H) + 2 * D + H * H + W * H * V
            else:
                H, D, V = m["heads"], m["dim"], m["vdim"]
                n += W * (2 * H * D + 2 * H * V) + 2 * H * (W + 1) + H * V + W * H * V
            n += 1
            if l.get("mlp"):
                n += 2 * W * l["mlp"]["ff"] + W + l["mlp"]["ff"] + 3
        return n + (2 * self.vocab_size * W if with_embedding else 0)

    def to_hf_dict(self) -> Dict[str, Any]:
        layers = [{k: v for k, v in l.items() if k != "second_norm" or v} for l in self.layers]
        return {"architecture": "Kuzanex", "layers": layers, "norm": {"eps": self.rms_norm_eps},
                "postln_alpha": self.postln_alpha, "vocab": self.vocab_size, "width": self.hidden_size}


def kuzanex_config(d: Dict[str, Any]) -> HybridConfig:
    """config.json of a Kuzanex checkpoint -> HybridConfig. Every size and constant is taken from it."""
    layers = []
    for i, l in enumerate(d["layers"]):
        if l["type"] not in ("attention", "mlstm"):
            raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
        mlp = l.get("mlp")
        if mlp is not None and mlp.get("kind", "dense") != "dense":
            raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
        layers.append({"type": l["type"], "mixer": dict(l["mixer"]), "mlp": dict(mlp) if mlp is not None else None,
                       "second_norm": bool(l.get("second_norm", False))})
    att = next((l["mixer"] for l in layers if l["type"] == "attention"), None)
    return HybridConfig(
        family="kuzanex", vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), n_layers=len(layers),
        n_q_heads=int(att["heads"]) if att else 1, n_kv_heads=int(att["kv_heads"]) if att else 1,
        head_dim=int(att["dim"]) if att else 1, intermediate_size=max([l["mlp"]["ff"] for l in layers if l["mlp"]] or [0]),
        rms_norm_eps=float(d["norm"]["eps"]), max_position_embeddings=int(d.get("max_positions", 1 << 17)),
        tie_word_embeddings=False, qkv_bias=True, qk_norm=True, pos_embed="none", layers=layers,
        postln_alpha=float(d["postln_alpha"]), eos_token_id=d.get("eos_token_id"), pad_token_id=d.get("pad_token_id"))


def kuzanex_config_from_dir(path: str) -> HybridConfig:
    """config.json plus one look at the checkpoint's tensor names (which layers without a feed-forward block own
    a second norm gain)."""
    with open(os.path.join(path, "config.json")) as f:
        cfg = kuzanex_config(json.load(f))
    names = set()
    for fn in sorted(os.listdir(path)):
        if fn.endswith(".safetensors"):
            from safetensors import safe_open

            with safe_open(os.path.join(path, fn), framework="pt") as f:
                names.update(f.keys())
    for i, l in enumerate(cfg.layers):
        if l["mlp"] is None and f"l{i}.norm2" in names:
            l["second_norm"] = True
    return cfg


class StepTensors:
    """What one batch plan hands to the mixers (all on the device): rows of the packed token batch (`cu_q`, longest
    row `max_q`), each row's context length after the step, cache slot of every token, page tables, position of each
    row's first token, state slot of each row, and the decode launch's split count / workspace."""

    def __init__(self, cu_q, ctx_len, max_q, slots, block_tables, first_pos, state_slots, nsplit=1, workspace=None):
        self.cu_q, self.ctx_len, self.max_q, self.slots = cu_q, ctx_len, int(max_q), slots
        self.block_tables, self.first_pos, self.state_slots = block_tables, first_pos, state_slots
        self.nsplit, self.workspace = int(nsplit), workspace


class WindowAttentionMixer(nn.Module):
    """Grouped-query attention on RMS-normalised queries and keys (no rotation), scores through soft cap, distance
    bias and head mixing, sliding window, optional sink, one sigmoid gate per head ahead of the output projection.
    q | k | v | gate come out of ONE projection (the gate rows carry no bias)."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, softcap: float,
                 window: int, slope_exp: float, sink: bool, head_mixing: bool, eps: float, dtype, device):
        super().__init__()
        assert heads % kv_heads == 0
        self.H, self.G, self.D, self.V, self.eps = heads, kv_heads, dim, vdim, eps
        self.shape = wattn.ScoreShape(scale=scale, softcap=softcap, slope_exp=slope_exp, window=window, sink=sink)
        n = (heads + kv_heads) * dim + kv_heads * vdim + heads
        self.proj = nn.Parameter(torch.empty(n, width, dtype=dtype, device=device))
        self.proj_bias = nn.Parameter(torch.zeros(n, dtype=dtype, device=device))
        self.q_norm = nn.Parameter(torch.ones(dim, dtype=dtype, device=device))
        self.k_norm = nn.Parameter(torch.ones(dim, dtype=dtype, device=device))
        self.talk = nn.Parameter(torch.eye(heads, dtype=dtype, device=device)) if head_mixing else None
        self.o = nn.Parameter(torch.empty(width, heads * vdim, dtype=dtype, device=device))

    def cache_shape(self):
        return self.G, self.D, self.V

    def step(self, xc: torch.Tensor, st: StepTensors, cache) -> torch.Tensor:
        kc, vc = cache
        T = xc.shape[0]
        H, G, D, V = self.H, self.G, self.D, self.V
        proj = F.linear(xc, self.proj, self.proj_bias)
        q = wattn.qk_norm_cache_write(proj, self.q_norm, self.k_norm, st.slots, kc, vc, H, self.eps)
        o = wattn.window_attention(q, kc, vc, st.block_tables, st.cu_q, st.ctx_len, st.max_q, self.shape, self.talk,
                                   nsplit=st.nsplit if st.max_q == 1 else 1, workspace=st.workspace,
                                   gate=proj[:, (H + G) * D + G * V:])
        return F.linear(o.view(T, H * V), self.o)


class MLSTMMixer(nn.Module):
    """Matrix-memory recurrence: q | k | v | output gate from one projection, the two log gates from a small one
    with fp32 accumulation, capped by `gate_cap`; per-head RMS norm, weight and sigmoid gate on the read-out."""

    def __init__(self, width: int, heads: int, dim: int, vdim: int, gate_cap: float, eps: float, dtype, device):
        super().__init__()
        self.H, self.D, self.V, self.cap, self.eps = heads, dim, vdim, gate_cap, eps
        self.proj = nn.Parameter(torch.empty(2 * heads * dim + 2 * heads * vdim, width, dtype=dtype, device=device))
        self.gates = nn.Parameter(torch.empty(2 * heads, width, dtype=dtype, device=device))
        self.gates_bias = nn.Parameter(torch.zeros(2 * heads, dtype=dtype, device=device))
        self.norm = nn.Parameter(torch.ones(heads * vdim, dtype=dtype, device=device))
        self.o = nn.Parameter(torch.empty(width, heads * vdim, dtype=dtype, device=device))

    def state_shape(self):
        return self.H, self.D, self.V

    def step(self, xc: torch.Tensor, st: StepTensors, state) -> torch.Tensor:
        H, D, V = self.H, self.D, self.V
        proj = F.linear(xc, self.proj)
        ig, fg = mlstm_ops.mlstm_gates(xc, self.gates, self.gates_bias, H, self.cap)
        hbuf, nq, mt = mlstm_ops.mlstm_scan(proj, 0, H * D, 2 * H * D, ig, fg, st.cu_q, st.first_pos, st.state_slots,
                                            state, max_q=st.max_q)
        y = mlstm_ops.mlstm_out(hbuf, nq, mt, proj[:, 2 * H * D + H * V:], self.norm, self.eps)
        return F.linear(y, self.o)


class XieluMLP(nn.Module):
    def __init__(self, width: int, ff: int, dtype, device):
        super().__init__()
        self.up = nn.Parameter(torch.empty(ff, width, dtype=dtype, device=device))
        self.up_bias = nn.Parameter(torch.zeros(ff, dtype=dtype, device=device))
        self.down = nn.Parameter(torch.empty(width, ff, dtype=dtype, device=device))
        self.down_bias = nn.Parameter(torch.zeros(width, dtype=dtype, device=device))
        self.act = nn.Parameter(torch.zeros(2, dtype=dtype, device=device))

    def forward(self, xc: torch.Tensor) -> torch.Tensor:
        return F.linear(post_norm.xielu(F.linear(xc, self.up, self.up_bias), self.act), self.down, self.down_bias)


class HybridBlock(nn.Module):
    def __init__(self, cfg: HybridConfig, spec: Dict[str, Any], dtype, device):
        super().__init__()
        W, m, eps = cfg.hidden_size, spec["mixer"], cfg.rms_norm_eps
        self.kind = spec["type"]
        if self.kind == "attention":
            mask = m.get("mask") or {}
            self.mix = WindowAttentionMixer(
                W, int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m.get("vdim", m["dim"])),
                float(m.get("scale", float(m["dim"]) ** -0.5)), float(m.get("softcap") or 0.0),
                int(mask.get("size") or 0), slope_exp=8.0, sink=True, head_mixing=True, eps=eps, dtype=dtype,
                device=device)
        else:
            self.mix = MLSTMMixer(W, int(m["heads"]), int(m["dim"]), int(m.get("vdim", m["dim"])),
                                  float(m.get("gate_cap") or 0.0), eps, dtype, device)
        self.norm1 = nn.Parameter(torch.ones(1, dtype=dtype, device=device))
        self.mlp = XieluMLP(W, int(spec["mlp"]["ff"]), dtype, device) if spec.get("mlp") else None
        # a layer without a feed-forward block ends after norm1, unless its checkpoint carries a second gain
        # (`second_norm`, found by `from_pretrained`): then x <- norm2(alpha x) follows
        second = self.mlp is not None or bool(spec.get("second_norm"))
        self.norm2 = nn.Parameter(torch.ones(1, dtype=dtype, device=device)) if second else None


class HybridDecoder(nn.Module):
    """Parameters of a layer-list decoder in one flat buffer (the rollout engine's weight updates address it), random
    initialisation, checkpoint loading. Inference only; one rank."""

    hybrid = True

    def __init__(self, cfg: HybridConfig, dtype=torch.bfloat16, device="cpu", tp_size: int = 1, tp_rank: int = 0,
                 tp_group=None, **unused):
        super().__init__()
        if tp_size != 1:
            raise NotImplementedError("layer-list decoders are served by one rank")
        self.cfg, self.dtype = cfg, dtype
        self.tp_size, self.tp_rank, self.tp_group, self.ep_group = 1, 0, None, None
        self.has_embed = self.has_head = True
        self.layer_ids = list(range(cfg.n_layers))
        self.vocab_range = (0, cfg.vocab_size)
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, cfg.hidden_size, dtype=dtype, device=device))
        self.layers = nn.ModuleList([HybridBlock(cfg, spec, dtype, device) for spec in cfg.layers])
        self.norm = nn.Parameter(torch.ones(1, dtype=dtype, device=device))
        self.head = nn.Parameter(torch.empty(cfg.vocab_size, cfg.hidden_size, dtype=dtype, device=device))
        self.flat: Optional[FlatParams] = None
        self.flat_experts = None

    @property
    def head_weight(self) -> torch.Tensor:
        return self.head

    def flatten(self, pad_to: int = 1, expert_pad_to=None) -> FlatParams:
        self.flat = FlatParams(self, self.dtype, next(self.parameters()).device, pad_to)
        return self.flat

    def init_weights(self, seed: int = 0, std: float = 0.02):
        g = torch.Generator(device="cpu").manual_seed(seed)
        W = self.cfg.hidden_size
        for n, p in self.named_parameters():
            leaf = n.rsplit(".", 1)[-1]
            if leaf == "talk":
                p.data.copy_(torch.eye(p.shape[0]) + 0.1 * torch.randn(p.shape, generator=g))
            elif leaf in ("norm1", "norm2") or n == "norm" or leaf in ("q_norm", "k_norm") or n.endswith("mix.norm"):
                p.data.copy_(1.0 + 0.1 * torch.randn(p.shape, generator=g))
            elif leaf == "act":
                p.data.copy_(0.3 * torch.randn(p.shape, generator=g))
            elif leaf.endswith("bias"):
                p.data.copy_(0.1 * torch.randn(p.shape, generator=g))
            elif leaf == "embed":
                p.data.copy_(torch.randn(p.shape, generator=g))
            else:  # projections: unit-variance outputs for a unit-variance input
                p.data.copy_(torch.randn(p.shape, generator=g) / (p.shape[-1] ** 0.5))
            if leaf == "proj_bias":  # the gate rows of the attention projection have no bias
                p.data[-self._mixer_of(n).H:] = 0

    def _mixer_of(self, name: str):
        return self.layers[int(name.split(".")[1])].mix

    def embed_tokens(self, input_ids, positions=None, scatter: bool = False):
        return ops.embedding(input_ids, self.embed)

    # ------------------------------------------------------------------------- checkpoint names
    def checkpoint_tensors(self) -> Dict[str, torch.Tensor]:
        """Checkpoint name -> the view of this model's parameters that holds it (fused projections are sliced)."""
        out: Dict[str, torch.Tensor] = {"embed": self.embed.data, "head": self.head.data,
                                        "final.norm": self.norm.data.view(())}
        for i, blk in enumerate(self.layers):
            p, m = f"l{i}.", blk.mix
            out[p + "norm1"] = blk.norm1.data.view(())
            if blk.norm2 is not None:
                out[p + "norm2"] = blk.norm2.data.view(())
            if blk.kind == "attention":
                H, G, D, V = m.H, m.G, m.D, m.V
                a, b, c = H * D, (H + G) * D, (H + G) * D + G * V
                for nm, lo, hi in (("q", 0, a), ("k", a, b), ("v", b, c)):
                    out[p + f"mix.{nm}"] = m.proj.data[lo:hi]
                    out[p + f"mix.{nm}.b"] = m.proj_bias.data[lo:hi]
                out[p + "mix.g"] = m.proj.data[c:]
                out[p + "mix.q.norm"], out[p + "mix.k.norm"] = m.q_norm.data, m.k_norm.data
                if m.talk is not None:
                    out[p + "mix.talk"] = m.talk.data
                out[p + "mix.o"] = m.o.data
            else:
                H, D, V = m.H, m.D, m.V
                a, b, c = H * D, 2 * H * D, 2 * H * D + H * V
                for nm, lo, hi in (("q", 0, a), ("k", a, b), ("v", b, c), ("g", c, c + H * V)):
                    out[p + f"mix.{nm}"] = m.proj.data[lo:hi]
                out[p + "mix.i"], out[p + "mix.f"] = m.gates.data[:H], m.gates.data[H:]
                out[p + "mix.i.b"], out[p + "mix.f.b"] = m.gates_bias.data[:H], m.gates_bias.data[H:]
                out[p + "mix.norm"], out[p + "mix.o"] = m.norm.data, m.o.data
            if blk.mlp is not None:
                q = p + "mlp."
                out[q + "up"], out[q + "up.b"] = blk.mlp.up.data, blk.mlp.up_bias.data
                out[q + "down"], out[q + "down.b"] = blk.mlp.down.data, blk.mlp.down_bias.data
                out[q + "act"] = blk.mlp.act.data
        return out

    def assign_named_tensors(self, tensors: Dict[str, torch.Tensor], strict: bool = True):
        views = self.checkpoint_tensors()
        unknown = [n for n in tensors if n not in views]
        if strict and unknown:
            raise KeyError(f"{len(unknown)} tensor(s) map onto no parameter of this model: {sorted(unknown)[:8]}")
        for n, t in tensors.items():
            if n in views:
                v = views[n]
                if tuple(v.shape) != tuple(t.shape):
                    raise ValueError(f"{n}: checkpoint shape {tuple(t.shape)}, model expects {tuple(v.shape)}")
                v.copy_(t.to(v.dtype))

    def load_checkpoint(self, path: str, strict: bool = True):
        from safetensors import safe_open

        files = sorted(f for f in os.listdir(path) if f.endswith(".safetensors"))
        if not files:
            raise FileNotFoundError(f"no safetensors files under {path}")
        seen = set()
        for fn in files:
            with safe_open(os.path.join(path, fn), framework="pt") as f:
                names = list(f.keys())
                self.assign_named_tensors({k: f.get_tensor(k) for k in names}, strict=strict)
                seen.update(names)
        missing = sorted(set(self.checkpoint_tensors()) - seen)
        if strict and missing:
            raise KeyError(f"checkpoint lacks {len(missing)} tensor(s): {missing[:8]}")

    def save_checkpoint(self, path: str):
        from safetensors.torch import save_file

        os.makedirs(path, exist_ok=True)
        save_file({k: v.detach().cpu().contiguous().clone() for k, v in self.checkpoint_tensors().items()},
                  os.path.join(path, "model.safetensors"))
        with open(os.path.join(path, "config.json"), "w") as f:
            json.dump(self.cfg.to_hf_dict(), f, indent=1)
