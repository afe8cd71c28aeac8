"""Sudevik: a config-driven hybrid decoder.

Every layer is described by its own entry of ``config.layers`` — mixer
type, mixer sizes and feed-forward — so layers may differ in every size
and come in any order. Two mixers:

* ``attention``: GQA with separate key and value sizes, per-head q/k RMS
  norm, interleaved-pair rotary (optionally YaRN-scaled, optionally on a
  prefix of the head), a sliding window that keeps the first tokens, a
  softmax sink (denominator 1 + sum exp) and a sigmoid output gate. A
  layer with ``kv_from: j`` owns no key/value tensors and attends over
  layer j's cache with its own queries.
* ``delta``: gated delta rule with short causal convolutions on q, k, v,
  unit-norm q/k, per-head decay and write strength, and a gated per-head
  RMS norm on the read-out.

Each sublayer is wrapped in LayerNorms (weight + bias) before and
after; the residual stream is fp32. Feed-forward: top-k-of-logits
mixture of SwiGLU experts with a biased fp32 router, or none.

Framework mapping: merged projections (layers/linear.py), LayerNorm
over the fp32 stream (layers/layernorm.py), WindowAttention + PairRotary
(layers/attention.py, layers/rotary.py), FusedMoE (layers/moe/layer.py),
the paged KV pool with per-layer shapes (core/kv_cache.py) and the
recurrent state pool with per-layer specs (core/ssm.py). Prompt
portions and decode tokens of a mixed batch run through the same ragged
kernels (ops.window_attention, ops.delta_rule_varlen), so results do
not depend on how a sequence was cut into steps.
"""

from typing import Iterable, List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from gllm_amd import ops
from gllm_amd.core.ssm import SSMLayerSpec, SSMSpec
from gllm_amd.layers.attention import WindowAttention
from gllm_amd.layers.embedding import ParallelLMHead, VocabParallelEmbedding
from gllm_amd.layers.layernorm import LayerNorm
from gllm_amd.layers.linear import (MergedColumnParallelLinear,
                                    ReplicatedLinear, RowParallelLinear)
from gllm_amd.layers.moe.layer import FusedMoE
from gllm_amd.layers.rotary import PairRotary
from gllm_amd.runtime.forward_context import ForwardContext


def _get(d, key, default=None):
    """config.json sub-objects arrive as dicts (or namespaces)."""
    if d is None:
        return default
    if isinstance(d, dict):
        return d.get(key, default)
    return getattr(d, key, default)


class RoutedExperts(nn.Module):
    """Top-k-of-logits MoE: the router (weight + bias) runs in fp32, the
    ``top`` largest logits win and their softmax weights the experts."""

    def __init__(self, width: int, mlp, engine_config, dtype):
        super().__init__()
        router = _get(mlp, "router")
        self.num_experts = int(_get(router, "experts"))
        self.top = int(_get(router, "top"))
        ff = int(_get(_get(mlp, "expert"), "ff"))
        self.router = ReplicatedLinear(width, self.num_experts, bias=True,
                                       params_dtype=dtype)
        self.experts = FusedMoE(self.num_experts, self.top, width, ff,
                                renormalize=True,
                                use_ep=engine_config.use_ep,
                                params_dtype=dtype)
        self._r32 = None

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        if self._r32 is None or self._r32[0].device != h.device:
            self._r32 = (self.router.weight.float(),
                         self.router.bias.float())
        logits = F.linear(h.float(), self._r32[0], self._r32[1])
        weights, ids = ops.topk_then_softmax(logits, self.top)
        return self.experts.forward_routed(h, weights, ids)


class AttentionMixer(nn.Module):
    def __init__(self, width: int, m, eps: float, kv_index: int,
                 owns_kv: bool, dtype):
        super().__init__()
        H, G = int(_get(m, "heads")), int(_get(m, "kv_heads"))
        D, Dv = int(_get(m, "dim")), int(_get(m, "vdim"))
        self.sizes = [H * D, G * D, G * Dv, H * Dv] if owns_kv \
            else [H * D, H * Dv]
        self.owns_kv = owns_kv
        self.in_proj = MergedColumnParallelLinear(width, self.sizes,
                                                  params_dtype=dtype)
        self.out_proj = RowParallelLinear(H * Dv, width, params_dtype=dtype)
        rot = _get(m, "rot")
        rotary = None
        if rot:
            rotary = PairRotary(int(_get(rot, "dims")),
                                float(_get(rot, "base")),
                                _get(rot, "scaling"))
        mask = _get(m, "mask")
        self.attn = WindowAttention(
            kv_index, H, G, D, Dv, float(_get(m, "scale")), eps,
            window=int(_get(mask, "size", 0) or 0),
            keep_first=int(_get(mask, "keep_first", 0) or 0),
            sink=True, rotary=rotary, owns_kv=owns_kv, params_dtype=dtype)

    def shard_of(self, name: str) -> Optional[int]:
        order = ["q", "k", "v", "g"] if self.owns_kv else ["q", "g"]
        return order.index(name) if name in order else None

    def forward(self, h: torch.Tensor, fctx: ForwardContext):
        parts = self.in_proj(h).split(self.sizes, dim=-1)
        if self.owns_kv:
            q, k, v, gate = parts
        else:
            (q, gate), k, v = parts, None, None
        return self.out_proj(self.attn(q, k, v, gate, fctx))


class DeltaMixer(nn.Module):
    def __init__(self, width: int, m, eps: float, ssm_layer_id: int, dtype):
        super().__init__()
        self.H, self.G = int(_get(m, "heads")), int(_get(m, "kv_heads"))
        self.Dk, self.Dv = int(_get(m, "dim")), int(_get(m, "vdim"))
        self.taps = int(_get(m, "conv"))
        self.ssm_layer_id = ssm_layer_id
        self.eps = eps
        H, G, Dk, Dv = self.H, self.G, self.Dk, self.Dv
        # q | k | v feed the convolution (one contiguous column block),
        # then the output gate and the two per-head gate projections
        self.sizes = [G * Dk, G * Dk, H * Dv, H * Dv, H, H]
        self.conv_dim = 2 * G * Dk + H * Dv
        self.in_proj = MergedColumnParallelLinear(width, self.sizes,
                                                  params_dtype=dtype)
        self.conv_weight = nn.Parameter(
            torch.empty(self.conv_dim, self.taps, dtype=dtype),
            requires_grad=False)
        self.A_log = nn.Parameter(torch.zeros(H, dtype=torch.float32),
                                  requires_grad=False)
        self.dt_bias = nn.Parameter(torch.zeros(H, dtype=torch.float32),
                                    requires_grad=False)
        self.norm_weight = nn.Parameter(torch.ones(Dv, dtype=dtype),
                                        requires_grad=False)
        self.out_proj = RowParallelLinear(H * Dv, width, params_dtype=dtype)
        self._ones = None

    def shard_of(self, name: str) -> Optional[int]:
        order = ["q", "k", "v", "g", "a", "b"]
        return order.index(name) if name in order else None

    def spec(self) -> SSMLayerSpec:
        return SSMLayerSpec(self.conv_dim, self.taps, self.H, self.Dk,
                            self.Dv, layout="kv")

    def forward(self, h: torch.Tensor, fctx: ForwardContext):
        T = h.shape[0]
        if fctx.is_profile_run or fctx.ssm_pool is None:
            return h.new_zeros(T, self.out_proj.output_size)
        proj = self.in_proj(h)
        gk, hv = self.G * self.Dk, self.H * self.Dv
        mixed = proj[:, :self.conv_dim]
        z = proj[:, self.conv_dim:self.conv_dim + hv]
        a = proj[:, self.conv_dim + hv:self.conv_dim + hv + self.H]
        b = proj[:, self.conv_dim + hv + self.H:]
        pool = fctx.ssm_pool
        if fctx.ssm_slots_dev is not None:
            # captured decode bucket: persistent slot buffer, every row
            # a one-token step on carried state (padding rows work on
            # the pool's scratch slot)
            slots = fctx.ssm_slots_dev[:T]
            if self._ones is None or self._ones.numel() < T \
                    or self._ones.device != h.device:
                self._ones = torch.ones(max(T, 1024), dtype=torch.int32,
                                        device=h.device)
            init = self._ones[:T]
        else:
            slots, init = fctx.ssm_slots_t, fctx.ssm_has_init_t
        qsl = fctx.query_start_loc
        conv = ops.causal_conv_silu(
            mixed, self.conv_weight, pool.conv_state[self.ssm_layer_id],
            slots, init, qsl)
        o = ops.delta_rule_varlen(
            conv[:, :gk], conv[:, gk:2 * gk], conv[:, 2 * gk:], a, b,
            self.A_log, self.dt_bias, pool.ssm_state[self.ssm_layer_id],
            slots, init, qsl, self.Dk ** -0.5, fctx.max_query_len)
        gated = ops.rms_gate(o, z, self.norm_weight, self.H, self.eps,
                             h.dtype)
        return self.out_proj(gated)


class SudevikLayer(nn.Module):
    def __init__(self, width: int, layer, eps: float, index: int,
                 engine_config, dtype, kv_index: int = -1,
                 owns_kv: bool = True):
        super().__init__()
        self.kind = _get(layer, "type")
        m = _get(layer, "mixer")
        if self.kind == "attention":
            self.mix = AttentionMixer(width, m, eps, kv_index, owns_kv,
                                      dtype)
        elif self.kind == "delta":
            self.mix = DeltaMixer(width, m, eps, index, dtype)
        else:
            raise ValueError(f"unknown mixer type {self.kind!r}")
        self.norm1 = LayerNorm(width, eps, dtype)
        self.norm1b = LayerNorm(width, eps, dtype)
        mlp = _get(layer, "mlp")
        if mlp:
            kind = _get(mlp, "kind", "moe")
            if kind != "moe":
                raise ValueError(f"unknown feed-forward kind {kind!r}")
            self.mlp = RoutedExperts(width, mlp, engine_config, dtype)
            self.norm2 = LayerNorm(width, eps, dtype)
            self.norm2b = LayerNorm(width, eps, dtype)
        else:
            self.mlp = None

    def forward(self, x: torch.Tensor, h: torch.Tensor,
                fctx: ForwardContext, nxt: LayerNorm) -> torch.Tensor:
        """x: fp32 stream (updated in place); h = norm1(x) from the
        previous boundary. Returns ``nxt`` applied to the updated x."""
        y = self.mix(h, fctx)
        if self.mlp is None:
            return self.norm1b.add_into(x, y, nxt)
        h = self.norm1b.add_into(x, y, self.norm2)
        return self.norm2b.add_into(x, self.mlp(h), nxt)


class SudevikForCausalLM(nn.Module):
    # ragged state kernels read slots / flags from device tensors
    wants_state_tensors = True

    def __init__(self, cfg, engine_config):
        super().__init__()
        from gllm_amd.parallel import get_pp_size, get_tp_size
        assert get_tp_size() == 1 and get_pp_size() == 1, \
            "Sudevik serves on one GPU per replica (tp = pp = 1)"
        self.cfg = cfg
        dtype = engine_config.torch_dtype()
        layers = list(cfg.layers)
        width = int(cfg.width)
        vocab = int(cfg.vocab)
        eps = float(_get(cfg.norm, "eps"))
        # names the rest of the framework reads off a model config
        cfg.vocab_size = vocab
        cfg.hidden_size = width
        cfg.num_hidden_layers = len(layers)
        self.layer_start, self.layer_end = 0, len(layers)
        self.is_first_stage = self.is_last_stage = True
        self.embed = VocabParallelEmbedding(vocab, width, params_dtype=dtype)
        mods: List[SudevikLayer] = []
        kv_index_of = {}
        kv_shapes: List[Tuple[int, int, int]] = []
        ssm_specs: List[SSMLayerSpec] = []
        for i, layer in enumerate(layers):
            kind = _get(layer, "type")
            m = _get(layer, "mixer")
            if kind == "attention":
                src = _get(m, "kv_from")
                if src is None:
                    kv_index_of[i] = len(kv_shapes)
                    kv_shapes.append((int(_get(m, "kv_heads")),
                                      int(_get(m, "dim")),
                                      int(_get(m, "vdim"))))
                    mods.append(SudevikLayer(width, layer, eps, i,
                                             engine_config, dtype,
                                             kv_index_of[i], True))
                else:
                    if int(src) not in kv_index_of:
                        raise ValueError(
                            f"layer {i}: kv_from {src} is not an earlier "
                            "attention layer with keys of its own")
                    mods.append(SudevikLayer(width, layer, eps, i,
                                             engine_config, dtype,
                                             kv_index_of[int(src)], False))
            else:
                lay = SudevikLayer(width, layer, eps, len(ssm_specs),
                                   engine_config, dtype)
                ssm_specs.append(lay.mix.spec())
                mods.append(lay)
        self.layers = nn.ModuleList(mods)
        self.kv_layer_shapes = kv_shapes
        self.num_kv_layers = len(kv_shapes)
        self.ssm_spec = None
        if ssm_specs:
            s0 = ssm_specs[0]
            self.ssm_spec = SSMSpec(len(ssm_specs), s0.conv_dim,
                                    s0.conv_kernel, s0.num_v_heads,
                                    s0.head_k_dim, s0.head_v_dim,
                                    layers=ssm_specs)
        self.final_norm = LayerNorm(width, eps, dtype)
        self.lm_head = ParallelLMHead(vocab, width, params_dtype=dtype)
        # hipGraph decode buckets need a sync-free forward: bf16 with
        # every MoE on the grouped GEMM (8-aligned width and ff); fp32
        # and odd expert shapes take the host segment loop
        self.supports_graph = dtype == torch.bfloat16 and all(
            lay.mlp is None or (width % 8 == 0 and
                                lay.mlp.experts.intermediate_per_rank % 8
                                == 0)
            for lay in mods)

    @property
    def num_local_layers(self):
        return len(self.layers)

    def forward(self, input_ids, positions, fctx, hidden_states=None,
                residual=None):
        x = self.embed(input_ids).float()
        h = self.layers[0].norm1(x) if len(self.layers) else None
        for i, layer in enumerate(self.layers):
            nxt = self.layers[i + 1].norm1 if i + 1 < len(self.layers) \
                else self.final_norm
            h = layer(x, h, fctx, nxt)
        if h is None:
            h = self.final_norm(x)
        return h, None

    def compute_logits(self, hidden_states, fctx):
        rows = hidden_states
        if fctx.logits_indices is not None:
            rows = hidden_states.index_select(0, fctx.logits_indices)
        return self.lm_head(rows)

    # ------------------------------------------------------------------
    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]):
        """Checkpoint names: ``embed``, ``head``, ``final.norm[.b]`` and
        per layer ``l<i>.norm{1,1b,2,2b}[.b]``, ``l<i>.mix.<t>`` (with
        ``.conv`` / ``.norm`` suffixes) and ``l<i>.mlp.{router[.b],
        e<j>.{gate,up,down}}``."""
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

    def _load_norm(self, norm: LayerNorm, is_bias: bool, w):
        self._copy(norm.bias if is_bias else norm.weight, w)
        return True

    def _load_one(self, name: str, w: torch.Tensor) -> bool:
        if name == "embed":
            self.embed.weight.weight_loader(self.embed.weight, w)
            return True
        if name == "head":
            self.lm_head.weight.weight_loader(self.lm_head.weight, w)
            return True
        if name in ("final.norm", "final.norm.b"):
            return self._load_norm(self.final_norm, name.endswith(".b"), w)
        parts = name.split(".")
        if not (parts[0].startswith("l") and parts[0][1:].isdigit()):
            return False
        layer = self.layers[int(parts[0][1:])]
        rest = parts[1:]
        if rest[0] in ("norm1", "norm1b", "norm2", "norm2b"):
            return self._load_norm(getattr(layer, rest[0]),
                                   rest[1:] == ["b"], w)
        if rest[0] == "mlp":
            return self._load_mlp(layer.mlp, rest[1:], w)
        if rest[0] != "mix":
            return False
        mix, sub = layer.mix, rest[1:]
        if sub == ["o"]:
            p = mix.out_proj.weight
            p.weight_loader(p, w)
            return True
        if len(sub) == 1 and mix.shard_of(sub[0]) is not None:
            p = mix.in_proj.weight
            p.weight_loader(p, w, mix.shard_of(sub[0]))
            return True
        if isinstance(mix, AttentionMixer):
            if sub == ["q", "norm"]:
                self._copy(mix.attn.q_norm, w)
                return True
            if sub == ["k", "norm"] and mix.owns_kv:
                self._copy(mix.attn.k_norm, w)
                return True
            return False
        if len(sub) == 2 and sub[1] == "conv" and sub[0] in ("q", "k", "v"):
            off = sum(mix.sizes[:mix.shard_of(sub[0])])
            self._copy(mix.conv_weight.data.narrow(0, off, w.shape[0]), w)
            return True
        if sub in (["A_log"], ["dt_bias"]):
            self._copy(getattr(mix, sub[0]), w)
            return True
        if sub == ["norm"]:
            self._copy(mix.norm_weight, w)
            return True
        return False

    @staticmethod
    def _load_mlp(mlp: RoutedExperts, sub: List[str], w) -> bool:
        if sub == ["router"]:
            mlp.router.weight.data.copy_(w)
            return True
        if sub == ["router", "b"]:
            mlp.router.bias.data.copy_(w)
            return True
        if len(sub) == 2 and sub[0].startswith("e") and sub[0][1:].isdigit():
            e = int(sub[0][1:])
            ex = mlp.experts
            if sub[1] == "gate":
                ex.w13_weight.weight_loader(ex.w13_weight, w, e, 0)
            elif sub[1] == "up":
                ex.w13_weight.weight_loader(ex.w13_weight, w, e, 1)
            elif sub[1] == "down":
                ex.w2_weight.weight_loader(ex.w2_weight, w, e)
            else:
                return False
            return True
        return False
