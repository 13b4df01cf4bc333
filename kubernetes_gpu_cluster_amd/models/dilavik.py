"""Dilavik: a hybrid decoder of mLSTM and windowed-attention layers.

Per layer, on an fp32 residual stream x (width W):
  h = group_norm1(x);  x += mixer(h)          mixer: MLSTMMixer | WindowedAttention
  h = group_norm2(x);  x += down(xIELU(up h)) (layers with a feed-forward)
  X_(i+1) = x;  x = sum_{j <= i+1} dwa_i[j] X_j   (X_0: the scaled embedding)
and after the last layer the model's grouped norm and the LM head.  The GEMMs run in the
activation dtype (bf16, fp32 accumulation); the stream, the norms, the depth average,
the gates, the recurrence and the attention softmax stay in fp32.

Kernel sequence per layer (ops/__init__.py, "hybrid decoders"):
  [depth_mix_norm of the previous layer -> h]  qkv GEMM -> gate_proj -> rope_kv_store ->
  window_attention (head gate in its epilogue) -> o GEMM -> group_rms_norm(add) -> up
  GEMM -> xielu -> down GEMM -> depth_mix_norm
  mLSTM: qkvg GEMM -> gate_proj -> mlstm_scan -> head_norm_gate -> o GEMM -> depth_mix_norm
One GPU per replica (TP = PP = 1).
"""
from __future__ import annotations

import re
from typing import Iterable, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops
from ..parallel.layers import ParallelLMHead, ReplicatedLinear, VocabParallelEmbedding
from ..parallel.state import get_state
from .attention import ForwardContext, WindowedAttention
from .configs import ModelConfig
from .recurrent import MLSTMMixer


def _f32(shape, device, fill=0.0):
    return nn.Parameter(torch.full(shape, fill, dtype=torch.float32, device=device),
                        requires_grad=False)


class XIELUMLP(nn.Module):
    """down(xIELU(up h)); the activation's two parameters are kept as
    (softplus(p), 1/2 + softplus(q)) in fp32."""

    def __init__(self, hidden: int, ff: int, dtype, device):
        super().__init__()
        self.up_proj = ReplicatedLinear(hidden, ff, dtype=dtype, device=device)
        self.down_proj = ReplicatedLinear(ff, hidden, dtype=dtype, device=device)
        self.act = _f32((2,), device, 1.0)

    def load_act(self, pq: torch.Tensor) -> None:
        sp = F.softplus(pq.float())
        self.act.data.copy_(torch.stack([sp[0], 0.5 + sp[1]]))

    def forward(self, h):
        return self.down_proj(ops.xielu(self.up_proj(h), self.act))


class DilavikLayer(nn.Module):
    def __init__(self, cfg: ModelConfig, idx: int, cache_idx: int, state_idx: int, dtype, device):
        super().__init__()
        sp = cfg.layer_specs[idx]
        W = cfg.hidden_size
        self.idx = idx
        self.norm1 = _f32((W,), device, 1.0)
        if sp.kind == "attention":
            self.mix = WindowedAttention(W, sp, cache_idx, dtype, device)
        else:
            self.mix = MLSTMMixer(W, sp, state_idx, cfg.rms_eps, dtype, device)
        if sp.ff:
            self.norm2 = _f32((W,), device, 1.0)
            self.mlp = XIELUMLP(W, sp.ff, dtype, device)
        else:
            self.norm2 = self.mlp = None
        # depth-average weights over X_0 .. X_(idx+1); identity: the layer's own result
        self.dwa = _f32((idx + 2,), device)
        self.dwa.data[idx + 1] = 1.0


class DilavikForCausalLM(nn.Module):
    def __init__(self, cfg: ModelConfig, dtype=torch.bfloat16, device=None):
        super().__init__()
        s = get_state()
        assert s.tp_size == 1 and s.pp_size == 1, "Dilavik runs on one GPU per replica"
        assert cfg.hidden_size % cfg.norm_groups == 0
        self.cfg, self.dtype = cfg, dtype
        self.start, self.end = 0, cfg.num_layers
        self.first = self.last = True
        self.embed_tokens = VocabParallelEmbedding(cfg.vocab_size, cfg.hidden_size, dtype, device)
        layers, nc, ns = [], 0, 0
        for i, sp in enumerate(cfg.layer_specs):
            layers.append(DilavikLayer(cfg, i, nc, ns, dtype, device))
            nc += sp.kind == "attention"
            ns += sp.kind != "attention"
        self.layers = nn.ModuleList(layers)
        self.final_norm = _f32((cfg.hidden_size,), device, 1.0)
        self.lm_head = ParallelLMHead(cfg.vocab_size, cfg.hidden_size, dtype, device)
        self.hist = None            # [L + 1, Tcap, W] fp32: X_0 .. X_L of the step's rows
        self.stream = None          # [Tcap, W] fp32: the residual stream

    # ------------------------------------------------------------------ engine hooks
    @property
    def num_local_layers(self) -> int:
        return len(self.layers)

    def local_kv_heads(self) -> int:
        return max((sp.kv_heads for sp in self.cfg.layer_specs if sp.kind == "attention"),
                   default=1)

    def cache_layout(self) -> list:
        """(kv heads, key size, value size) of every attention layer's paged cache."""
        return [(sp.kv_heads, sp.dim, sp.vdim) for sp in self.cfg.layer_specs
                if sp.kind == "attention"]

    def state_layout(self) -> list:
        """Per recurrent layer, the per-slot shapes of its state tensors."""
        return [l.mix.state_shapes() for l in self.layers if isinstance(l.mix, MLSTMMixer)]

    def prepare(self, max_pos: int, max_tokens: int, device) -> None:
        """Rotary tables for ``max_pos`` positions and the step buffers for ``max_tokens``
        rows (static, so captured decode graphs replay over them)."""
        tables: dict = {}
        for l in self.layers:
            if isinstance(l.mix, WindowedAttention):
                l.mix.prepare(tables, max_pos, device)
        L, W = len(self.layers), self.cfg.hidden_size
        self.hist = torch.zeros(L + 1, max_tokens, W, dtype=torch.float32, device=device)
        self.stream = torch.zeros(max_tokens, W, dtype=torch.float32, device=device)

    @torch.no_grad()
    def init_random(self, seed: int = 0, std: float = 0.02) -> None:
        """Random weights for benchmarking: projections ~ N(0, std), norm weights near 1,
        depth-average weights near "take the layer's own result", small gate biases."""
        g = torch.Generator(device="cpu").manual_seed(seed)

        def rnd(p, scale, base=0.0):
            p.copy_((torch.randn(p.shape, generator=g) * scale + base).to(p.device, p.dtype))
        for name, p in self.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("norm1", "norm2", "final_norm", "norm_weight"):
                rnd(p, 0.05, 1.0)
            elif leaf == "dwa":
                rnd(p, 0.05 / p.numel())
                p[-1] += 1.0
            elif leaf == "act":
                p.copy_(torch.tensor([0.8, 1.0], device=p.device))
            elif leaf == "if_bias":
                rnd(p, 0.5)
                p[p.numel() // 2:] += 3.0        # forget gates start open
            else:
                rnd(p, std)

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, ctx: ForwardContext,
                hidden=None, residual=None, taps: Optional[list] = None):
        """-> the final-normed hidden rows.  ``taps``: the residual stream after every
        layer is appended (fp32 copies; debugging and tests)."""
        cfg = self.cfg
        T = input_ids.shape[0]
        if self.hist is None or self.hist.shape[1] < T:
            self.prepare(cfg.max_position, max(T, 1), input_ids.device)
        G, eps, dt = cfg.norm_groups, cfg.rms_eps, self.dtype
        x = self.stream[:T]
        torch.mul(self.embed_tokens(input_ids), cfg.embed_scale, out=x)
        self.hist[0, :T].copy_(x)
        h = ops.group_rms_norm(x, self.layers[0].norm1, G, eps, dt)
        for i, layer in enumerate(self.layers):
            y = layer.mix(h, positions, ctx)
            if layer.mlp is not None:
                h = ops.group_rms_norm(x, layer.norm2, G, eps, dt, add=y)
                y = layer.mlp(h)
            nxt = self.layers[i + 1].norm1 if i + 1 < len(self.layers) else self.final_norm
            h = ops.depth_mix_norm(x, self.hist, i, y, layer.dwa, nxt, G, eps, dt)
            if taps is not None:
                taps.append(x.clone())
        return h

    def compute_logits(self, hidden: torch.Tensor, gather: bool = True) -> torch.Tensor:
        return self.lm_head(hidden, gather)

    # ------------------------------------------------------------------ weights
    def load_weights(self, weights: Iterable[tuple[str, torch.Tensor]]) -> int:
        """Checkpoint names: ``embed``, ``head``, ``final.norm``, and per layer i
        ``l<i>.norm1|norm2|dwa``, ``l<i>.mix.q|k|v|g|o`` (+ ``norm``, ``i``, ``i.b``, ``f``,
        ``f.b`` for mLSTM) and ``l<i>.mlp.up|down|act``."""
        n, seen = 0, set()
        for name, w in weights:
            if self._load_one(name, w):
                n += 1
                seen.add(name)
        return n

    def _load_one(self, name: str, w: torch.Tensor) -> bool:
        if name == "embed":
            self.embed_tokens.weight.weight_loader(self.embed_tokens.weight, w.to(self.dtype))
            return True
        if name == "head":
            self.lm_head.weight.weight_loader(self.lm_head.weight, w.to(self.dtype))
            return True
        if name == "final.norm":
            self.final_norm.data.copy_(w.float())
            return True
        m = re.match(r"l(\d+)\.(.*)", name)
        if m is None or int(m.group(1)) >= len(self.layers):
            return False
        layer, rest = self.layers[int(m.group(1))], m.group(2)
        sp, mix = self.cfg.layer_specs[layer.idx], layer.mix
        H, d, dv = sp.heads, sp.dim, sp.vdim
        if rest in ("norm1", "norm2", "dwa"):
            getattr(layer, rest).data.copy_(w.float())
            return True
        if rest == "mlp.up":
            layer.mlp.up_proj.weight.data.copy_(w.to(self.dtype))
        elif rest == "mlp.down":
            layer.mlp.down_proj.weight.data.copy_(w.to(self.dtype))
        elif rest == "mlp.act":
            layer.mlp.load_act(w)
        elif rest == "mix.o":
            mix.o_proj.weight.data.copy_(w.to(self.dtype))
        elif sp.kind == "attention":
            G = sp.kv_heads
            off = {"mix.q": (0, H * d), "mix.k": (H * d, G * d), "mix.v": ((H + G) * d, G * dv)}
            if rest in off:
                a, ln = off[rest]
                mix.qkv_proj.weight.data.narrow(0, a, ln).copy_(w.to(self.dtype))
            elif rest == "mix.g":
                mix.gate.data.copy_(w.to(self.dtype))
            else:
                return False
        else:
            off = {"mix.q": (0, H * d), "mix.k": (H * d, H * d), "mix.v": (2 * H * d, H * dv),
                   "mix.g": (2 * H * d + H * dv, H * dv)}
            if rest in off:
                a, ln = off[rest]
                mix.qkvg_proj.weight.data.narrow(0, a, ln).copy_(w.to(self.dtype))
            elif rest in ("mix.i", "mix.f"):
                mix.if_weight.data.narrow(0, 0 if rest == "mix.i" else H, H).copy_(w.to(self.dtype))
            elif rest in ("mix.i.b", "mix.f.b"):
                mix.if_bias.data.narrow(0, 0 if rest == "mix.i.b" else H, H).copy_(w.float())
            elif rest == "mix.norm":
                mix.norm_weight.data.copy_(w.float())
            else:
                return False
        return True
