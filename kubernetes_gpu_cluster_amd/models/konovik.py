"""Konovik: a decoder of latent-attention and minGRU layers with token shift, a looped
span of layers, scalar-weight norms, sigmoid-routed experts and a per-token side input.

On an fp32 residual stream x (width W), with m the config's residual multiplier:
  x = RMSNorm(embed[token]) * g_e                       (kept as E when layers are looped)
  per layer run (layers [start, stop) of the loop run ``times`` times in a row with the
  same weights, each pass with its own cache and state, x += E before every pass but the
  first):
    h = token_shift(RMSNorm(x) * g_1);  x += m * mixer(h)     LatentAttention | MinGRUMixer
    x += m * ff(RMSNorm(x) * g_2)                             gated dense | routed experts
    y = side_proj(gelu_tanh(side_gate x) * side_embed[token, layer's columns])
    x += m * RMSNorm(y) * w_side
  logits = head(RMSNorm(x) * g_f)
The model's norms carry a single number as weight (kept as a constant vector so the row
kernels are the ones other decoders use).  Projections run in the activation dtype with
fp32 accumulation; the stream, every norm, the shift, the recurrence, routing and the
attention softmax are fp32.

Kernel sequence per layer run (ops/__init__.py, "Konovik-style decoders"):
  residual_norm (previous sublayer joins x; norm, fp32) -> token_shift -> mixer:
    latent attention: merged GEMM -> batched GEMM (queries into latent space) ->
      latent_rope_store -> window_attention -> batched GEMM (values) -> gate_mul -> o GEMM
    minGRU: merged GEMM -> mingru_scan -> o GEMM
  -> residual_norm -> feed-forward (gate_up GEMM -> silu_mul -> down GEMM | gate_proj ->
  moe_route_sigmoid -> expert GEMMs with relu_sq -> moe_finish) -> side_input (decode-size
  batches: one kernel; otherwise residual_norm (cast) -> side gate GEMM -> side_gate -> side
  proj GEMM -> residual_norm (normed add + next norm)).
One GPU per replica (TP = PP = 1).
"""
from __future__ import annotations

import re
from typing import Iterable, Optional

import torch
import torch.nn as nn

from .. import ops
from ..ops.gemm import linear_silu
from ..parallel.layers import ParallelLMHead, ReplicatedLinear, VocabParallelEmbedding
from ..parallel.state import get_state
from .attention import ForwardContext, LatentAttention
from .configs import ModelConfig
from .moe import SigmoidRoutedExperts
from .recurrent import MinGRUMixer


def _f32(shape, device, fill=0.0):
    return nn.Parameter(torch.full(shape, fill, dtype=torch.float32, device=device),
                        requires_grad=False)


class GatedMLP(nn.Module):
    """down(silu(gate h) * up h) with gate and up as one merged projection."""

    def __init__(self, hidden: int, ff: int, dtype, device):
        super().__init__()
        self.ff = ff
        self.gate_up_proj = ReplicatedLinear(hidden, 2 * ff, dtype=dtype, device=device)
        self.down_proj = ReplicatedLinear(ff, hidden, dtype=dtype, device=device)

    def forward(self, h):
        return self.down_proj(linear_silu(h, self.gate_up_proj.weight))


class KonovikLayer(nn.Module):
    def __init__(self, cfg: ModelConfig, idx: int, dtype, device):
        super().__init__()
        sp = cfg.layer_specs[idx]
        W = cfg.hidden_size
        self.idx = idx
        self.norm1 = _f32((W,), device, 1.0)        # the checkpoint's single number, repeated
        self.shift = _f32((W,), device)
        if sp.kind == "latent_attention":
            self.mix = LatentAttention(W, sp, cfg.rms_eps, dtype, device)
        else:
            self.mix = MinGRUMixer(W, sp, dtype, device)
        f = sp.mlp
        if f is None:
            self.norm2 = self.mlp = None
        else:
            self.norm2 = _f32((W,), device, 1.0)
            self.mlp = (GatedMLP(W, f.ff, dtype, device) if f.kind == "dense"
                        else SigmoidRoutedExperts(W, f, dtype, device))
        if cfg.side_dim:
            self.side_gate = ReplicatedLinear(W, cfg.side_dim, dtype=dtype, device=device)
            self.side_proj = ReplicatedLinear(cfg.side_dim, W, dtype=dtype, device=device)
            self.side_norm = _f32((W,), device, 1.0)
        else:
            self.side_gate = self.side_proj = self.side_norm = None


class KonovikForCausalLM(nn.Module):
    def __init__(self, cfg: ModelConfig, dtype=torch.bfloat16, device=None):
        super().__init__()
        s = get_state()
        assert s.tp_size == 1 and s.pp_size == 1, "Konovik runs on one GPU per replica"
        self.cfg, self.dtype = cfg, dtype
        self.start, self.end = 0, cfg.num_layers
        self.first = self.last = True
        W, L = cfg.hidden_size, cfg.num_layers
        self.embed_tokens = VocabParallelEmbedding(cfg.vocab_size, W, dtype, device)
        self.embed_norm = _f32((W,), device, 1.0)
        self.side_embed = (nn.Parameter(torch.zeros(cfg.vocab_size, L * cfg.side_dim, dtype=dtype,
                                                    device=device), requires_grad=False)
                           if cfg.side_dim else None)
        self.layers = nn.ModuleList([KonovikLayer(cfg, i, dtype, device) for i in range(L)])
        self.final_norm = _f32((W,), device, 1.0)
        self.lm_head = ParallelLMHead(cfg.vocab_size, W, dtype, device)
        # execution order: (layer, cache index or -1, state index, x += E first)
        self.runs, nc, ns = [], 0, 0
        for i, again in cfg.layer_runs():
            att = cfg.layer_specs[i].is_attention
            self.runs.append((i, nc if att else -1, ns, again))
            nc += att
            ns += 1
        self.looped = any(r[3] for r in self.runs)
        self.stream = self.embed_out = None     # [Tcap, W] fp32 step buffers

    # ------------------------------------------------------------------ engine hooks
    @property
    def num_local_layers(self) -> int:
        return len(self.runs)

    def local_kv_heads(self) -> int:
        return 1

    def cache_layout(self) -> list:
        """Per attention layer run (kv groups, row width, 0): one group whose rows hold the
        latent and the rotary key part; values are read from the latent columns."""
        sp = self.cfg.layer_specs
        return [(1, sp[i].kv_rank + sp[i].rot_dims, 0) for i, c, _, _ in self.runs if c >= 0]

    def state_layout(self) -> list:
        """Per layer run: the token-shift row, and for a minGRU run its state vector."""
        out = []
        for i, c, _, _ in self.runs:
            shapes = ((self.cfg.hidden_size,),)
            if c < 0:
                shapes += self.layers[i].mix.state_shapes()
            out.append(shapes)
        return out

    def prepare(self, max_pos: int, max_tokens: int, device) -> None:
        """Rotary tables for ``max_pos`` positions and the step buffers for ``max_tokens``
        rows (static, so captured decode graphs replay over them)."""
        tables: dict = {}
        for l in self.layers:
            if isinstance(l.mix, LatentAttention):
                l.mix.prepare(tables, max_pos, device)
        W = self.cfg.hidden_size
        self.stream = torch.zeros(max_tokens, W, dtype=torch.float32, device=device)
        self.embed_out = (torch.zeros(max_tokens, W, dtype=torch.float32, device=device)
                          if self.looped else None)

    @torch.no_grad()
    def init_random(self, seed: int = 0, std: float = 0.02) -> None:
        """Random weights for benchmarking: projections ~ N(0, std), norm weights near 1,
        shifts in (0, 1), small corrections and biases."""
        g = torch.Generator(device="cpu").manual_seed(seed)

        def rnd(p, scale, base=0.0):
            p.copy_((torch.randn(p.shape, generator=g) * scale + base).to(p.device, p.dtype))
        for name, p in self.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("norm1", "norm2", "final_norm", "embed_norm"):
                p.fill_(1.0 + 0.05 * float(torch.randn((), generator=g)))
            elif leaf in ("norm_weight", "side_norm"):
                rnd(p, 0.05, 1.0)
            elif leaf == "shift":
                p.copy_(torch.rand(p.shape, generator=g).to(p.device))
            elif leaf in ("correction", "zx_bias"):
                rnd(p, 0.1)
            else:
                rnd(p, std)

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, ctx: ForwardContext,
                hidden=None, residual=None, taps: Optional[list] = None):
        """-> the final-normed hidden rows.  ``taps``: the residual stream after every
        layer run is appended (fp32 copies; debugging and tests)."""
        cfg = self.cfg
        T = input_ids.shape[0]
        if self.stream is None or self.stream.shape[0] < T:
            self.prepare(cfg.max_position, max(T, 1), input_ids.device)
        eps, dt, m, f32 = cfg.rms_eps, self.dtype, cfg.residual_mult, torch.float32
        x = self.stream[:T]
        x.copy_(self.embed_tokens(input_ids))
        ops.residual_norm(x, None, 1.0, self.embed_norm, eps, f32, out=x)
        if self.looped:
            self.embed_out[:T].copy_(x)
        h = ops.residual_norm(x, None, 1.0, self.layers[self.runs[0][0]].norm1, eps, f32)
        for n, (i, cache_idx, state_idx, _) in enumerate(self.runs):
            layer = self.layers[i]
            st = ctx.states[state_idx]
            h = ops.token_shift(h, layer.shift, st[0], ctx.attn, dt)
            if cache_idx >= 0:
                y = layer.mix(h, positions, ctx, cache_idx)
            else:
                y = layer.mix(h, positions, ctx, st[1])
            if layer.mlp is not None:
                y = layer.mlp(ops.residual_norm(x, y, m, layer.norm2, eps, dt))
            last = n + 1 == len(self.runs)
            nxt = self.final_norm if last else self.layers[self.runs[n + 1][0]].norm1
            again = not last and self.runs[n + 1][3]
            out_dt = dt if last else f32
            split = again or taps is not None       # the stream is needed before the next norm
            if layer.side_gate is not None:
                h = ops.side_input(x, y, m, layer.side_gate.weight, layer.side_proj.weight,
                                   input_ids, self.side_embed, i * cfg.side_dim, layer.side_norm,
                                   None if split else nxt, eps, None if split else out_dt)
            else:
                h = ops.residual_norm(x, y, m, None if split else nxt, eps,
                                      None if split else out_dt)
            if split:
                if taps is not None:
                    taps.append(x.clone())
                h = ops.residual_norm(x, self.embed_out[:T] if again else None, 1.0, nxt, eps,
                                      out_dt)
        return h

    def compute_logits(self, hidden: torch.Tensor, gather: bool = True) -> torch.Tensor:
        return self.lm_head(hidden, gather)

    # ------------------------------------------------------------------ weights
    def load_weights(self, weights: Iterable[tuple[str, torch.Tensor]]) -> int:
        """Checkpoint names: ``embed``, ``embed.norm``, ``side.embed``, ``head``,
        ``final.norm`` and per layer i ``l<i>.norm1|norm2|shift``, ``l<i>.mix.*``,
        ``l<i>.mlp.*``, ``l<i>.side.gate|proj|norm``.  Returns the number loaded and raises
        on a name it does not know."""
        n = 0
        for name, w in weights:
            if not self._load_one(name, w):
                raise KeyError(f"unexpected tensor {name!r} in a Konovik checkpoint")
            n += 1
        return n

    def _load_one(self, name: str, w: torch.Tensor) -> bool:
        dt = self.dtype

        def put(p, src):
            p.data.copy_(src.to(p.dtype).reshape(p.shape) if src.numel() == p.numel()
                         else src.to(p.dtype).expand_as(p))
            return True
        if name == "embed":
            self.embed_tokens.weight.weight_loader(self.embed_tokens.weight, w.to(dt))
            return True
        if name == "head":
            self.lm_head.weight.weight_loader(self.lm_head.weight, w.to(dt))
            return True
        if name == "embed.norm":
            return put(self.embed_norm, w.float().reshape(1))
        if name == "final.norm":
            return put(self.final_norm, w.float().reshape(1))
        if name == "side.embed":
            return self.side_embed is not None and put(self.side_embed, w)
        mm = re.match(r"l(\d+)\.(.*)", name)
        if mm is None or int(mm.group(1)) >= len(self.layers):
            return False
        layer, rest = self.layers[int(mm.group(1))], mm.group(2)
        sp, mix = self.cfg.layer_specs[layer.idx], layer.mix
        if rest in ("norm1", "norm2"):
            p = getattr(layer, rest)
            return p is not None and put(p, w.float().reshape(1))
        if rest == "shift":
            return put(layer.shift, w.float())
        if rest.startswith("side."):
            tgt = {"side.gate": layer.side_gate and layer.side_gate.weight,
                   "side.proj": layer.side_proj and layer.side_proj.weight,
                   "side.norm": layer.side_norm}.get(rest)
            return tgt is not None and put(tgt, w)
        if rest == "mix.o":
            return put(mix.o_proj.weight, w)
        if rest.startswith("mix.") and sp.kind == "latent_attention":
            H, d, r, dv, rank = sp.heads, sp.dim, sp.rot_dims, sp.vdim, sp.kv_rank
            P = mix.proj.weight.data
            if rest == "mix.q":
                P[: mix.n_q].copy_(w.to(dt))
            elif rest == "mix.dkv":
                P[mix.n_q: mix.n_q + mix.n_kv].copy_(w.to(dt))
            elif rest == "mix.g":
                P[mix.n_q + mix.n_kv:].copy_(w.to(dt))
            elif rest == "mix.dkv.norm":
                put(mix.norm_weight, w.float())
            elif rest == "mix.uk":          # [H d, rank] -> [H, d, rank]
                mix.w_uk.data.copy_(w.to(dt).view(H, d, rank))
            elif rest == "mix.uv":          # [H dv, rank] -> [H, rank, dv]
                mix.w_uv.data.copy_(w.to(dt).view(H, dv, rank).transpose(1, 2))
            else:
                return False
            return True
        if rest.startswith("mix."):
            n = sp.width
            off = {"mix.z": 0, "mix.x": n, "mix.g": 2 * n}
            if rest in off:
                mix.zxg_proj.weight.data.narrow(0, off[rest], n).copy_(w.to(dt))
            elif rest in ("mix.z.b", "mix.x.b"):
                mix.zx_bias.data.narrow(0, 0 if rest == "mix.z.b" else n, n).copy_(w.float())
            else:
                return False
            return True
        if not rest.startswith("mlp.") or layer.mlp is None:
            return False
        f, mlp, leaf = sp.mlp, layer.mlp, rest[4:]
        if f.kind == "dense":
            if leaf == "gate":
                mlp.gate_up_proj.weight.data[: f.ff].copy_(w.to(dt))
            elif leaf == "up":
                mlp.gate_up_proj.weight.data[f.ff:].copy_(w.to(dt))
            elif leaf == "down":
                put(mlp.down_proj.weight, w)
            else:
                return False
            return True
        me = re.match(r"e(\d+)\.(up|down)$", leaf)
        if me:
            e = int(me.group(1))
            if e >= f.experts:
                return False
            (mlp.w_up if me.group(2) == "up" else mlp.w_down).data[e].copy_(w.to(dt))
            return True
        if leaf == "router":
            mlp.gates.data[: f.experts].copy_(w.to(dt))
        elif leaf == "correction":
            put(mlp.correction, w.float())
        elif leaf == "shared.up" and f.shared_ff:
            put(mlp.shared_up.weight, w)
        elif leaf == "shared.down" and f.shared_ff:
            put(mlp.shared_down.weight, w)
        elif leaf == "shared.sg" and f.shared_ff:
            mlp.gates.data[f.experts].copy_(w.to(dt).reshape(-1))
        else:
            return False
        return True
