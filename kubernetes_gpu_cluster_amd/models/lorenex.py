"""Lorenex: gated-linear-attention layers and layers that run an attention beside a
selective scan, with the norm on every sublayer's result.

On an fp32 residual stream x (width W), m the residual multiplier:
  x = embed[token] * embed_scale + pos[p]                (learned positions, from 0 per sequence)
  per layer:   x += m * RMSNorm(mixer(x)) w_1;   x += m * RMSNorm(ff(x)) w_2
  logits = embed . (RMSNorm(x) w_f)                      (the embedding table is the head)
The sublayers read x itself (rounded to the activation dtype); only their results are
normed.  Layer type "gla": gated linear attention (a decay per key channel).  Type
"parallel": left_scale * attention + right_scale * selective scan, the attention with
biased q / k / v projections that pass a short causal convolution, unit-RMS q, k and v per
head, a query factor that grows with the position, no rotation.  Feed-forward: PolyNorm
dense (down(a N(z) + b N(z^2) + c N(z^3) + e), z = up h), or clamped gated experts under a
softmax router with a choice correction and identity experts, or none.  A layer may run
with another layer's weights; its cache and state are its own.  Projections run in the
activation dtype with fp32 accumulation; the stream, every norm, the decays, step sizes,
recurrent states, softmax and routing are fp32.

Kernel sequence per layer (ops/__init__.py, "Lorenex-style decoders" and "parallel mixers"):
  residual_norm (the previous sublayer's normed result joins x; x in the activation dtype) ->
  gla:       merged projection GEMM -> gla_scan (decay projection inside) -> gated_rms_norm
             -> output GEMM
  parallel:  ONE merged projection GEMM -> causal_conv -> norm_kv_store -> window_attention
             into the left columns | causal_conv -> two small GEMMs -> selective_scan (gate
             in its epilogue) into the right columns -> ONE output GEMM
  -> residual_norm -> up GEMM -> polynorm -> down GEMM | gate_proj -> moe_route_softmax_all ->
  expert GEMMs with swiglu_clamp -> moe_finish (identity experts).
One GPU per replica (TP = PP = 1).
"""
from __future__ import annotations

import re
from typing import Iterable, Optional

import torch
import torch.nn as nn

from .. import ops
from ..ops.gemm import linear
from ..parallel.layers import ReplicatedLinear, VocabParallelEmbedding
from ..parallel.state import get_state
from .attention import ForwardContext
from .configs import ModelConfig
from .moe import SoftmaxAllRoutedExperts
from .nolesun import ParallelMixer
from .recurrent import GLAMixer


def _f32(shape, device, fill=0.0):
    return nn.Parameter(torch.full(shape, fill, dtype=torch.float32, device=device),
                        requires_grad=False)


class PolyNormMLP(nn.Module):
    """down(a N(z) + b N(z^2) + c N(z^3) + e), z = up h, N = division by the row's RMS."""

    def __init__(self, hidden: int, ff: int, eps: float, dtype, device):
        super().__init__()
        self.eps = eps
        self.up_proj = ReplicatedLinear(hidden, ff, dtype=dtype, device=device)
        self.down_proj = ReplicatedLinear(ff, hidden, dtype=dtype, device=device)
        self.coef = _f32((4,), device)

    def forward(self, h):
        return self.down_proj(ops.polynorm(self.up_proj(h), self.coef, self.eps))


class LorenexLayer(nn.Module):
    def __init__(self, cfg: ModelConfig, idx: int, dtype, device):
        super().__init__()
        sp = cfg.layer_specs[idx]
        W = cfg.hidden_size
        self.idx = idx
        self.norm1 = _f32((W,), device, 1.0)
        self.mix = (GLAMixer(W, sp, cfg.rms_eps, dtype, device) if sp.kind == "gla"
                    else ParallelMixer(W, sp, cfg.rms_eps, dtype, device))
        f = sp.mlp
        if f is None:
            self.norm2 = self.mlp = None
        else:
            self.norm2 = _f32((W,), device, 1.0)
            self.mlp = (PolyNormMLP(W, f.ff, cfg.rms_eps, dtype, device) if f.kind == "dense"
                        else SoftmaxAllRoutedExperts(W, f, dtype, device))


class LorenexForCausalLM(nn.Module):
    def __init__(self, cfg: ModelConfig, dtype=torch.bfloat16, device=None):
        super().__init__()
        s = get_state()
        assert s.tp_size == 1 and s.pp_size == 1, "Lorenex runs on one GPU per replica"
        self.cfg, self.dtype = cfg, dtype
        self.start, self.end = 0, cfg.num_layers
        self.first = self.last = True
        W, L = cfg.hidden_size, cfg.num_layers
        share = cfg.weights_of or tuple(range(L))
        self.embed_tokens = VocabParallelEmbedding(cfg.vocab_size, W, dtype, device)
        self.pos = _f32((cfg.max_position, W), device)
        # a layer that runs with another layer's weights has no module of its own
        self.layers = nn.ModuleDict({str(i): LorenexLayer(cfg, i, dtype, device)
                                     for i in range(L) if share[i] == i})
        self.final_norm = _f32((W,), device, 1.0)
        # execution order: (layer whose weights run, cache index or -1, state index)
        self.runs, nc = [], 0
        for n in range(L):
            has_cache = cfg.layer_specs[n].kind == "parallel"
            self.runs.append((share[n], nc if has_cache else -1, n))
            nc += has_cache
        self.stream = None          # [Tcap, W] fp32 step buffer

    def layer(self, i: int) -> LorenexLayer:
        return self.layers[str(i)]

    # ------------------------------------------------------------------ engine hooks
    @property
    def num_local_layers(self) -> int:
        return len(self.runs)

    def local_kv_heads(self) -> int:
        return max((sp.left.kv_heads for sp in self.cfg.layer_specs if sp.kind == "parallel"),
                   default=1)

    def cache_layout(self) -> list:
        """(kv heads, key size, value size) of every attention-carrying layer run's cache."""
        return [self.layer(i).mix.cache_shape() for i, c, _ in self.runs if c >= 0]

    def state_layout(self) -> list:
        """Per layer run, the per-slot shapes of its state tensors (gla: S; parallel: the
        attention's convolution inputs, the scan's convolution inputs, the scan's state)."""
        return [self.layer(i).mix.state_shapes() for i, _, _ in self.runs]

    def prepare(self, max_pos: int, max_tokens: int, device) -> None:
        """The step buffer for ``max_tokens`` rows (static, so captured decode graphs replay
        over it)."""
        self.stream = torch.zeros(max_tokens, self.cfg.hidden_size, dtype=torch.float32,
                                  device=device)

    @torch.no_grad()
    def init_random(self, seed: int = 0, std: float = 0.02) -> None:
        """Random weights for benchmarking: projections ~ N(0, std), norm weights near 1,
        decays and step sizes in the range trained models use."""
        g = torch.Generator(device="cpu").manual_seed(seed)

        def rnd(p, scale, base=0.0):
            p.copy_((torch.randn(p.shape, generator=g) * scale + base).to(p.device, p.dtype))
        for name, p in self.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("norm1", "norm2", "final_norm", "norm_weight"):
                rnd(p, 0.05, 1.0)
            elif leaf == "A":
                p.copy_(-(1.0 + 15.0 * torch.rand(p.shape, generator=g)).to(p.device))
            elif leaf == "dt_bias":
                rnd(p, 0.5, -3.0)
            elif leaf == "a2_bias":
                rnd(p, 1.0, 3.0)
            elif leaf == "a2":
                rnd(p, 0.3)
            elif leaf == "dskip":
                rnd(p, 0.1, 1.0)
            elif leaf == "conv_w":
                rnd(p, 0.3)
            elif leaf == "coef":
                p.copy_(torch.tensor([1.0, 0.3, 0.1, 0.0]))
            elif leaf in ("conv_b", "correction", "bias"):
                rnd(p, 0.02)
            elif leaf == "router":
                rnd(p, 0.2)
            elif leaf == "pos":
                rnd(p, 0.02)
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
        eps, dt, m = cfg.rms_eps, self.dtype, cfg.residual_mult
        x = self.stream[:T]
        ops.embed_pos(input_ids, positions, self.embed_tokens.weight, cfg.embed_scale, self.pos, x)
        y = post = None                     # a sublayer result that has not joined x yet
        for i, c, n in self.runs:
            layer = self.layer(i)
            h = ops.residual_norm(x, y, m, None, eps, dt, add_norm_w=post)
            y, post = layer.mix(h, positions, ctx, c, ctx.states[n]), layer.norm1
            if layer.mlp is not None:
                h = ops.residual_norm(x, y, m, None, eps, dt, add_norm_w=post)
                y, post = layer.mlp(h), layer.norm2
            if taps is not None:
                ops.residual_norm(x, y, m, None, eps, None, add_norm_w=post)
                y = post = None
                taps.append(x.clone())
        return ops.residual_norm(x, y, m, self.final_norm, eps, dt, add_norm_w=post)

    def compute_logits(self, hidden: torch.Tensor, gather: bool = True) -> torch.Tensor:
        return linear(hidden, self.embed_tokens.weight)

    # ------------------------------------------------------------------ weights
    def load_weights(self, weights: Iterable[tuple[str, torch.Tensor]]) -> int:
        """Checkpoint names: ``embed``, ``pos``, ``final.norm`` and per layer i with tensors
        of its own ``l<i>.norm1|norm2``, ``l<i>.mix.*`` (gla: q k v g o norm a1 a2 a2.b;
        parallel: left.q|k|v (+ .b, .conv), left.o, right.in|conv|conv.b|x|dt|dt.b|A_log|D|o),
        ``l<i>.mlp.*`` (up down act | e<j>.gate|up|down, router, correction).  Returns the
        number loaded and raises on a name or a shape it does not know."""
        n = 0
        for name, w in weights:
            if not self._load_one(name, w):
                raise KeyError(f"unexpected tensor {name!r} in a Lorenex checkpoint")
            n += 1
        return n

    @staticmethod
    def _put(tgt: torch.Tensor, w: torch.Tensor) -> bool:
        if tuple(tgt.shape) != tuple(w.shape):
            raise ValueError(f"shape {tuple(w.shape)} does not fit {tuple(tgt.shape)}")
        tgt.copy_(w.to(tgt.dtype))
        return True

    def _load_one(self, name: str, w: torch.Tensor) -> bool:
        put = self._put
        if name == "embed":
            self.embed_tokens.weight.weight_loader(self.embed_tokens.weight, w.to(self.dtype))
            return True
        if name == "pos":
            return put(self.pos.data, w)
        if name == "final.norm":
            return put(self.final_norm.data, w)
        mm = re.match(r"l(\d+)\.(.*)", name)
        if mm is None or mm.group(1) not in self.layers:
            return False
        layer, rest = self.layers[mm.group(1)], mm.group(2)
        sp, mix = self.cfg.layer_specs[layer.idx], layer.mix
        if rest == "norm1" or (rest == "norm2" and layer.norm2 is not None):
            return put(getattr(layer, rest).data, w)
        if rest.startswith("mix."):
            if sp.kind == "gla":
                return self._load_gla(mix, sp, rest[4:], w)
            if rest.startswith("mix.left."):
                return self._load_left(mix, sp.left, rest[9:], w)
            if rest.startswith("mix.right."):
                return self._load_right(mix, sp.right, rest[10:], w)
            return False
        if not rest.startswith("mlp.") or layer.mlp is None:
            return False
        f, mlp, leaf = sp.mlp, layer.mlp, rest[4:]
        if f.kind == "dense":
            tgt = {"up": mlp.up_proj.weight, "down": mlp.down_proj.weight,
                   "act": mlp.coef}.get(leaf)
            return tgt is not None and put(tgt.data, w)
        me = re.match(r"e(\d+)\.(gate|up|down)$", leaf)
        if me:
            e, which = int(me.group(1)), me.group(2)
            if e >= f.experts:
                return False
            if which == "down":
                return put(mlp.w2.data[e], w)
            return put(mlp.w13.data[e].narrow(0, 0 if which == "gate" else f.ff, f.ff), w)
        tgt = {"router": mlp.router, "correction": mlp.correction}.get(leaf)
        return tgt is not None and put(tgt.data, w)

    def _load_gla(self, mix: GLAMixer, sp, leaf: str, w: torch.Tensor) -> bool:
        put = self._put
        H, d, dv, r = sp.heads, sp.dim, sp.vdim, sp.decay_rank
        off = {"q": (0, H * d), "k": (H * d, H * d), "v": (2 * H * d, H * dv),
               "g": (mix.n_qkv, H * dv), "a1": (mix.n_qkv + mix.n_g, r)}
        if leaf in off:
            a, n = off[leaf]
            return put(mix.proj.weight.data.narrow(0, a, n), w)
        if leaf == "o":
            return put(mix.o_proj.weight.data, w)
        if leaf == "norm":
            return put(mix.norm_weight.data, w.float().repeat(H))
        tgt = {"a2": mix.a2, "a2.b": mix.a2_bias}.get(leaf)
        return tgt is not None and put(tgt.data, w)

    def _load_left(self, mix: ParallelMixer, l, leaf: str, w: torch.Tensor) -> bool:
        put = self._put
        H, G, dk, dv = l.heads, l.kv_heads, l.dim, l.vdim
        off = {"q": (0, H * dk), "k": (H * dk, G * dk), "v": ((H + G) * dk, G * dv)}
        base = leaf.split(".")[0]
        if base in off:
            a, n = off[base]
            if leaf == base:
                return put(mix.in_proj.weight.data.narrow(0, a, n), w)
            if leaf == base + ".b" and l.bias:
                return put(mix.in_proj.bias.data.narrow(0, a, n), w)
            if leaf == base + ".conv" and l.conv:
                return put(mix.left.conv_w.data.narrow(0, a, n), w)
            return False
        if leaf == "o":
            return put(mix.o_proj.weight.data[:, : mix.left.n_out], w)
        return False

    def _load_right(self, mix: ParallelMixer, r, leaf: str, w: torch.Tensor) -> bool:
        put = self._put
        core, c0 = mix.right, mix.left.n_in
        if leaf == "in":
            return put(mix.in_proj.weight.data.narrow(0, c0, core.n_in), w)
        if leaf == "o":
            return put(mix.o_proj.weight.data[:, mix.left.n_out:], w)
        if leaf == "A_log":
            return put(core.A.data, -torch.exp(w.float()).t())
        tgt = {"conv": core.conv_w, "conv.b": core.conv_b, "x": core.x_proj.weight,
               "dt": core.dt_proj.weight, "dt.b": core.dt_bias, "D": core.dskip}.get(leaf)
        return tgt is not None and put(tgt.data, w)
