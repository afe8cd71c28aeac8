"""Gukirax: a config-driven looped decoder with talking-heads attention.

``config.layers`` describes every layer on its own (mixer sizes and the
feed-forward: dense, mixture of experts, or none), so sizes may differ
from layer to layer. ``config.loop`` = {start, stop, times} runs layers
start..stop-1 ``times`` times in a row with the same weights; every run
of a layer owns a KV cache of its own. Each pass opens with
x <- W_in [x ; x0], x0 being the normed embedding.

* stream: fp32; token embedding -> weight-only LayerNorm; every
  sublayer is x += LN_post(sigmoid(W_g h + b_g) * f(h)) with
  h = LN_pre(x) (weight-only LayerNorms, sigmoid gate from the
  sublayer's own input)
* mixer ``attention``: q and k projections only (values are the keys as
  projected), rotate-half rotary on the first ``rot.dims`` dims, unit
  RMS per head, cross-head mixing of the score planes before the causal
  softmax, a learned per-head sink in the denominator
* feed-forward: dense up -> xIELU -> down, or softmax-router MoE (top-k
  of the probabilities, weights not renormalised) of ungated relu^2
  experts plus an always-on shared expert of the same form
* logits: final LayerNorm, tied embedding table, scale, tanh soft cap

Framework mapping: merged projections q | k | gate (layers/linear.py),
LayerNorm.add_into with the fused gate (layers/layernorm.py),
TalkingHeadsAttention + HalfRotary (layers/attention.py,
layers/rotary.py), FusedMoE with ``activation="relu2"``
(layers/moe/layer.py), XIELU / ReLU2 (layers/activation.py), the paged KV
pool with one entry per layer RUN (core/kv_cache.py). Prompt portions and
decode tokens of a mixed batch go through the same ragged kernels.
"""

from typing import Iterable, List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from gllm_amd import ops
from gllm_amd.layers.activation import ReLU2, XIELU
from gllm_amd.layers.attention import TalkingHeadsAttention
from gllm_amd.layers.embedding import ParallelLMHead, VocabParallelEmbedding
from gllm_amd.layers.layernorm import LayerNorm
from gllm_amd.layers.linear import (MergedColumnParallelLinear,
                                    ReplicatedLinear, RowParallelLinear)
from gllm_amd.layers.moe.layer import FusedMoE
from gllm_amd.layers.rotary import HalfRotary
from gllm_amd.runtime.forward_context import ForwardContext


def _get(d, key, default=None):
    """config.json sub-objects arrive as dicts (or namespaces)."""
    if d is None:
        return default
    if isinstance(d, dict):
        return d.get(key, default)
    return getattr(d, key, default)


class TalkingMixer(nn.Module):
    """q | k | residual-gate in one projection, attention, out proj."""

    def __init__(self, width: int, m, eps: float, dtype):
        super().__init__()
        H, G = int(_get(m, "heads")), int(_get(m, "kv_heads"))
        D = int(_get(m, "dim"))
        Dv = int(_get(m, "vdim", D))
        if Dv != D:
            raise ValueError("values are the projected keys: vdim must "
                             f"equal dim (got {Dv} vs {D})")
        # the gate's bias rides on the merged projection; q and k rows
        # keep a zero bias
        self.sizes = [H * D, G * D, width]
        self.in_proj = MergedColumnParallelLinear(width, self.sizes,
                                                  bias=True,
                                                  params_dtype=dtype)
        self.in_proj.bias.data.zero_()
        self.out_proj = RowParallelLinear(H * D, width, params_dtype=dtype)
        rot = _get(m, "rot")
        rotary = None
        if rot and int(_get(rot, "dims", 0) or 0) > 0:
            rotary = HalfRotary(int(_get(rot, "dims")),
                                float(_get(rot, "base")))
        self.attn = TalkingHeadsAttention(-1, H, G, D,
                                          float(_get(m, "scale")), eps,
                                          rotary=rotary, sink=True)

    def forward(self, h: torch.Tensor, fctx: ForwardContext, kv_index: int):
        """Returns (mixer output, gate logits) — the gate is applied by
        the norm that follows (LayerNorm.add_into)."""
        q, k, gate = self.in_proj(h).split(self.sizes, dim=-1)
        return self.out_proj(self.attn(q, k, fctx, kv_index)), gate


class DenseFF(nn.Module):
    """up | gate in one projection -> xIELU -> down."""

    def __init__(self, width: int, mlp, dtype):
        super().__init__()
        ff = int(_get(mlp, "ff"))
        self.sizes = [ff, width]
        self.in_proj = MergedColumnParallelLinear(width, self.sizes,
                                                  bias=True,
                                                  params_dtype=dtype)
        self.in_proj.bias.data.zero_()
        self.act = XIELU()
        self.down = RowParallelLinear(ff, width, params_dtype=dtype)

    def forward(self, h: torch.Tensor):
        up, gate = self.in_proj(h).split(self.sizes, dim=-1)
        return self.down(self.act(up)), gate


class RoutedFF(nn.Module):
    """Softmax router in fp32 -> top-k probabilities as they are ->
    ungated relu^2 experts, plus a shared expert of the same form whose
    up projection is merged with the residual gate."""

    def __init__(self, width: int, mlp, engine_config, dtype):
        super().__init__()
        router = _get(mlp, "router")
        self.num_experts = int(_get(router, "experts"))
        self.top = int(_get(router, "top"))
        ff = int(_get(_get(mlp, "expert"), "ff"))
        self.router = ReplicatedLinear(width, self.num_experts,
                                       params_dtype=dtype)
        self.experts = FusedMoE(self.num_experts, self.top, width, ff,
                                renormalize=False,
                                use_ep=engine_config.use_ep,
                                params_dtype=dtype, activation="relu2",
                                fp32_routing_weights=True)
        shared = _get(mlp, "shared")
        self.shared_ff = int(_get(shared, "ff")) if shared else 0
        # shared-expert up rows (possibly none) | residual gate
        self.sizes = [self.shared_ff, width]
        self.in_proj = MergedColumnParallelLinear(width, self.sizes,
                                                  bias=True,
                                                  params_dtype=dtype)
        self.in_proj.bias.data.zero_()
        self.act = ReLU2()
        self.shared_down = RowParallelLinear(
            self.shared_ff, width, params_dtype=dtype) \
            if self.shared_ff else None
        self._r32 = None

    def forward(self, h: torch.Tensor):
        if self._r32 is None or self._r32.device != h.device:
            self._r32 = self.router.weight.float()
        logits = F.linear(h.float(), self._r32)
        weights, ids = ops.topk_softmax(logits, self.top, False)
        y = self.experts.forward_routed(h, weights, ids)
        up, gate = self.in_proj(h).split(self.sizes, dim=-1)
        if self.shared_down is not None:
            y = y + self.shared_down(self.act(up))
        return y, gate


class GukiraxLayer(nn.Module):
    def __init__(self, width: int, layer, eps: float, engine_config, dtype):
        super().__init__()
        kind = _get(layer, "type")
        if kind != "attention":
            raise ValueError(f"unknown mixer type {kind!r}")
        self.mix = TalkingMixer(width, _get(layer, "mixer"), eps, dtype)
        self.norm1 = LayerNorm(width, eps, dtype, bias=False)
        self.norm1b = LayerNorm(width, eps, dtype, bias=False)
        mlp = _get(layer, "mlp")
        if mlp:
            kind = _get(mlp, "kind")
            if kind == "dense":
                self.mlp = DenseFF(width, mlp, dtype)
            elif kind == "moe":
                self.mlp = RoutedFF(width, mlp, engine_config, dtype)
            else:
                raise ValueError(f"unknown feed-forward kind {kind!r}")
            self.norm2 = LayerNorm(width, eps, dtype, bias=False)
            self.norm2b = LayerNorm(width, eps, dtype, bias=False)
        else:
            self.mlp = None

    def forward(self, x: torch.Tensor, h: torch.Tensor,
                fctx: ForwardContext, nxt: Optional[LayerNorm],
                kv_index: int):
        """x: fp32 stream (updated in place); h = norm1(x). Returns
        ``nxt`` applied to the updated x (None without ``nxt``)."""
        y, gate = self.mix(h, fctx, kv_index)
        if self.mlp is None:
            return self.norm1b.add_into(x, y, nxt, gate)
        h = self.norm1b.add_into(x, y, self.norm2, gate)
        y, gate = self.mlp(h)
        return self.norm2b.add_into(x, y, nxt, gate)


class GukiraxForCausalLM(nn.Module):
    def __init__(self, cfg, engine_config):
        super().__init__()
        from gllm_amd.parallel import get_pp_size, get_tp_size
        assert get_tp_size() == 1 and get_pp_size() == 1, \
            "Gukirax serves on one GPU per replica (tp = pp = 1)"
        self.cfg = cfg
        dtype = engine_config.torch_dtype()
        self.dtype = dtype
        layers = list(cfg.layers)
        width = int(cfg.width)
        vocab = int(cfg.vocab)
        eps = float(_get(cfg.norm, "eps"))
        self.logit_scale = float(getattr(cfg, "logit_scale", 1.0))
        cap = getattr(cfg, "logit_softcap", None)
        self.logit_softcap = float(cap) if cap else 0.0
        # names the rest of the framework reads off a model config
        cfg.vocab_size = vocab
        cfg.hidden_size = width
        cfg.num_hidden_layers = len(layers)
        self.layer_start, self.layer_end = 0, len(layers)
        self.is_first_stage = self.is_last_stage = True
        self.embed = VocabParallelEmbedding(vocab, width, params_dtype=dtype)
        self.embed_norm = LayerNorm(width, eps, dtype, bias=False)
        self.layers = nn.ModuleList(
            GukiraxLayer(width, layer, eps, engine_config, dtype)
            for layer in layers)
        # the order layers run in: (layer, opens a pass, cache index)
        loop = getattr(cfg, "loop", None)
        n = len(layers)
        order: List[Tuple[int, bool]] = []
        if loop:
            a, b = int(_get(loop, "start")), int(_get(loop, "stop"))
            times = int(_get(loop, "times"))
            if not 0 <= a <= b <= n or times < 1:
                raise ValueError(f"bad loop {loop!r} for {n} layers")
            order += [(i, False) for i in range(a)]
            for _ in range(times):
                order += [(i, i == a) for i in range(a, b)]
            order += [(i, False) for i in range(b, n)]
            # (an empty span has no pass to open; the tensor still loads)
            self.loop_in = ReplicatedLinear(2 * width, width,
                                            params_dtype=dtype)
        else:
            order = [(i, False) for i in range(n)]
            self.loop_in = None
        self.runs = [(li, opens, r) for r, (li, opens) in enumerate(order)]
        self.kv_layer_shapes = []
        for li, _, _ in self.runs:
            at = self.layers[li].mix.attn
            self.kv_layer_shapes.append(
                (at.num_kv_heads, at.head_dim, at.head_dim))
        self.num_kv_layers = len(self.kv_layer_shapes)
        self.ssm_spec = None
        self.final_norm = LayerNorm(width, eps, dtype, bias=False)
        self.lm_head = ParallelLMHead(vocab, width, params_dtype=dtype)
        self.lm_head.tie_to(self.embed)
        # hipGraph decode buckets need a sync-free forward: bf16 with
        # every MoE on the grouped GEMM (8-aligned width and ff)
        self.supports_graph = dtype == torch.bfloat16 and all(
            not isinstance(lay.mlp, RoutedFF) or
            (width % 8 == 0 and
             lay.mlp.experts.intermediate_per_rank % 8 == 0)
            for lay in self.layers)
        # called as layer_probe(run index, x) after every layer run
        self.layer_probe = None

    @property
    def num_local_layers(self):
        return len(self.layers)

    def forward(self, input_ids, positions, fctx, hidden_states=None,
                residual=None):
        x0 = self.embed_norm.forward_f32(self.embed(input_ids).float())
        x = x0
        if self.loop_in is not None and self.runs and not self.runs[0][1]:
            x = x0.clone()     # layers ahead of the loop update x in place
        h = None
        last = len(self.runs) - 1
        for r, (li, opens, kv) in enumerate(self.runs):
            layer = self.layers[li]
            if opens:
                x = self.loop_in(
                    torch.cat([x, x0], dim=-1).to(self.dtype)).float()
                h = None
            if h is None:
                h = layer.norm1(x)
            if r == last:
                nxt = self.final_norm
            elif self.runs[r + 1][1]:
                nxt = None
            else:
                nxt = self.layers[self.runs[r + 1][0]].norm1
            h = layer(x, h, fctx, nxt, kv)
            if self.layer_probe is not None:
                self.layer_probe(r, x)
        if not self.runs:
            h = self.final_norm(x)
        return h, None

    def compute_logits(self, hidden_states, fctx):
        rows = hidden_states
        if fctx.logits_indices is not None:
            rows = hidden_states.index_select(0, fctx.logits_indices)
        logits = self.lm_head(rows).float() * self.logit_scale
        if self.logit_softcap:
            logits = torch.tanh(logits / self.logit_softcap) \
                * self.logit_softcap
        return logits

    # ------------------------------------------------------------------
    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]):
        """Checkpoint names: ``embed``, ``embed.norm``, ``loop.in``,
        ``final.norm`` and per layer ``l<i>.norm{1,1b,2,2b}``,
        ``l<i>.rg{1,2}[.b]``, ``l<i>.mix.{q,k,o,talk,sink}``,
        ``l<i>.mlp.{up,down,act}`` (dense) or ``l<i>.mlp.{router,
        e<j>.{up,down}, shared.{up,down}}`` (experts)."""
        seen = set()
        for name, w in weights:
            if self._load_one(name, w):
                seen.add(name)
            elif w.is_floating_point():
                raise KeyError(f"unexpected tensor {name!r}")
        return seen

    @staticmethod
    def _copy(param, w):
        assert tuple(param.shape) == tuple(w.shape), \
            (tuple(param.shape), tuple(w.shape))
        param.data.copy_(w.to(param.dtype))

    def _load_one(self, name: str, w: torch.Tensor) -> bool:
        if name == "embed":
            self.embed.weight.weight_loader(self.embed.weight, w)
            return True
        simple = {"embed.norm": self.embed_norm.weight,
                  "final.norm": self.final_norm.weight}
        if self.loop_in is not None:
            simple["loop.in"] = self.loop_in.weight
        if name in simple:
            self._copy(simple[name], w)
            return True
        parts = name.split(".")
        if not (parts[0].startswith("l") and parts[0][1:].isdigit()):
            return False
        layer = self.layers[int(parts[0][1:])]
        rest = parts[1:]
        if rest[0] in ("norm1", "norm1b", "norm2", "norm2b") \
                and len(rest) == 1:
            self._copy(getattr(layer, rest[0]).weight, w)
            return True
        if rest[0] in ("rg1", "rg2"):
            proj = layer.mix.in_proj if rest[0] == "rg1" \
                else layer.mlp.in_proj
            shard = len(proj.output_sizes) - 1
            p = proj.bias if rest[1:] == ["b"] else proj.weight
            if rest[1:] not in ([], ["b"]):
                return False
            p.weight_loader(p, w, shard)
            return True
        if rest[0] == "mlp":
            return self._load_mlp(layer.mlp, rest[1:], w)
        if rest[0] != "mix" or len(rest) != 2:
            return False
        mix = layer.mix
        if rest[1] == "o":
            self._copy(mix.out_proj.weight, w)
        elif rest[1] in ("q", "k"):
            p = mix.in_proj.weight
            p.weight_loader(p, w, ("q", "k").index(rest[1]))
        elif rest[1] == "talk":
            self._copy(mix.attn.talk, w)
        elif rest[1] == "sink":
            self._copy(mix.attn.sink, w)
        else:
            return False
        return True

    def _load_mlp(self, mlp, sub: List[str], w) -> bool:
        if isinstance(mlp, DenseFF):
            if sub == ["up"]:
                p = mlp.in_proj.weight
                p.weight_loader(p, w, 0)
            elif sub == ["down"]:
                self._copy(mlp.down.weight, w)
            elif sub == ["act"]:
                mlp.act.load(w)
            else:
                return False
            return True
        if sub == ["router"]:
            self._copy(mlp.router.weight, w)
            return True
        if sub == ["shared", "up"] and mlp.shared_ff:
            p = mlp.in_proj.weight
            p.weight_loader(p, w, 0)
            return True
        if sub == ["shared", "down"] and mlp.shared_ff:
            self._copy(mlp.shared_down.weight, w)
            return True
        if len(sub) == 2 and sub[0].startswith("e") and sub[0][1:].isdigit():
            e = int(sub[0][1:])
            ex = mlp.experts
            if sub[1] == "up":
                ex.w13_weight.weight_loader(ex.w13_weight, w, e, 0)
            elif sub[1] == "down":
                ex.w2_weight.weight_loader(ex.w2_weight, w, e)
            else:
                return False
            return True
        return False
