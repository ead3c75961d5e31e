"""Mixture-of-experts decoders (Mixtral-8x7B #9, Llama-4-Scout #5;
plus Qwen2-MoE / Qwen3-MoE).

* ``MixtralForCausalLM``  softmax top-2 routing over 8 SwiGLU experts
  (core/helm-charts/vllm/gaudi-values.yaml:354-375); also Qwen3-MoE
  (``norm_topk_prob``) and Qwen2-MoE (+ gated shared expert).
* ``Llama4ForCausalLM``   text path of Llama-4-Scout-17B-16E
  (core/helm-charts/vllm/gaudi-values.yaml:258-278, gaudi3-values.yaml:492-501):
  sigmoid top-1 routing applied to the expert *input*, a shared expert, chunked
  local attention (8192) on RoPE layers, GPT-J-style (interleaved) RoPE, weightless
  QK L2-norm on RoPE layers, NoPE every 4th layer with attention temperature tuning.

Experts live in one ``FusedMoE`` module ([E, 2I, H] / [E, H, I] tensors, K9 kernels in
ops/moe.py).  Tensor parallel shards each expert's I; ``--enable-expert-parallel``
instead gives each rank E/tp whole experts (the reference's EP on Gaudi 3,
``VLLM_EP_SIZE``); either way the layer output is all-reduced over the TP group.
"""

from __future__ import annotations

import math
import os
from typing import Iterable, List, Optional, Tuple

import torch
import torch.nn as nn

from ..config import ModelConfig
from ..ops import moe as moe_ops
from ..parallel import comm, state
from .layers import (MergedColumnParallelLinear, PendingAllReduce, ReplicatedLinear,
                     RowParallelLinear, _param)


def _deferred_reduce(out: torch.Tensor):
    """TP>1: hand the MoE partial sums to the next add+RMSNorm (fused xGMI all-reduce)."""
    return PendingAllReduce(out) if state.tp_size() > 1 else out
from .llama import LlamaAttention, LlamaDecoderLayer, LlamaForCausalLM, LlamaMLP


class FusedMoE(nn.Module):
    def __init__(self, num_experts: int, top_k: int, hidden: int, inter: int,
                 renormalize: bool = True, scoring: str = "softmax", scale_input: bool = False,
                 dtype=torch.bfloat16, device=None):
        super().__init__()
        tp, r = state.tp_size(), state.tp_rank()
        self.E, self.k, self.H = num_experts, top_k, hidden
        self.ep = state.ep_enabled()
        if self.ep:
            if num_experts % tp:
                raise ValueError("num_experts must be divisible by the EP size")
            self.e_per = num_experts // tp
            self.e_lo = r * self.e_per
            self.I_local = inter
        else:
            self.e_per, self.e_lo = num_experts, 0
            if inter % tp:
                raise ValueError("moe intermediate size must be divisible by tp")
            self.I_local = inter // tp
        self.I = inter
        self.renormalize, self.scoring, self.scale_input = renormalize, scoring, scale_input
        self.w13 = _param((self.e_per, 2 * self.I_local, hidden), dtype, device)
        self.w2 = _param((self.e_per, hidden, self.I_local), dtype, device)
        self.w13.weight_loader = self._load_w13
        self.w2.weight_loader = self._load_w2

    # shard helpers: loaded tensors are full [I, H] / [H, I] per expert
    def _local(self, expert: int) -> Optional[int]:
        e = expert - self.e_lo
        return e if 0 <= e < self.e_per else None

    def _ishard(self, t: torch.Tensor, dim: int) -> torch.Tensor:
        if self.ep or state.tp_size() == 1:
            return t
        n = self.I_local
        return t.narrow(dim, state.tp_rank() * n, n)

    def _load_w13(self, param, loaded, shard_id):
        expert, which = shard_id               # which: "w1" (gate) | "w3" (up) | "w13"
        e = self._local(expert)
        if e is None:
            return
        if which == "w13":                     # fused [2I, H] (gate rows then up rows)
            g, u = loaded.chunk(2, dim=0)
            param.data[e, :self.I_local].copy_(self._ishard(g, 0))
            param.data[e, self.I_local:].copy_(self._ishard(u, 0))
            return
        off = 0 if which == "w1" else self.I_local
        param.data[e, off:off + self.I_local].copy_(self._ishard(loaded, 0))

    def _load_w2(self, param, loaded, shard_id):
        expert, _ = shard_id
        e = self._local(expert)
        if e is not None:
            param.data[e].copy_(self._ishard(loaded, 1))

    def forward(self, x: torch.Tensor, router_logits: Optional[torch.Tensor] = None,
                reduce: bool = True, router_w: Optional[torch.Tensor] = None,
                routing: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                defer_combine: bool = False):
        if routing is not None:       # routed by the preceding norm (MixtralMoE.norm_and_route)
            w, ids = routing
        elif router_logits is None:   # fused router GEMM + top-k
            w, ids = moe_ops.route(x, router_w, self.k, self.renormalize, self.scoring)
        else:
            w, ids = moe_ops.topk_route(router_logits, self.k, self.renormalize, self.scoring)
        if self.scale_input:
            # Llama-4 applies the routing score to the expert input (k = 1), as the reference
            # model does: bf16 score x bf16 activation (one elementwise launch)
            x = x * w[:, :1].to(x.dtype)
            w = self._unit_weights(w)
        if self.a2a:
            from ..parallel.expert_parallel import moe_all_to_all_replicated
            return moe_all_to_all_replicated(x, w, ids, self.w13, self.w2, self.e_lo,
                                             self.e_per, state.tp_group())
        out = moe_ops.fused_moe(x, self.w13, self.w2, w, ids,
                                (self.e_lo, self.e_lo + self.e_per) if self.ep else None,
                                defer_combine=defer_combine and not (reduce and
                                                                     state.tp_size() > 1))
        if reduce and state.tp_size() > 1:
            out = comm.all_reduce(out)
        return out

    def _unit_weights(self, w: torch.Tensor) -> torch.Tensor:
        """All-ones routing weights shaped like ``w``: a slice of a cached buffer (no fill
        launch per layer and step), grown outside graph capture only."""
        buf = getattr(self, "_ones", None)
        if (buf is None or buf.device != w.device or buf.shape[0] < w.shape[0]
                or buf.shape[1] != w.shape[1]):
            if torch.cuda.is_available() and torch.cuda.is_current_stream_capturing():
                return torch.ones_like(w)
            buf = torch.ones(max(256, w.shape[0]), w.shape[1], dtype=w.dtype, device=w.device)
            self._ones = buf
        return buf[:w.shape[0]]

    @property
    def a2a(self) -> bool:
        """All-to-all EP: the output comes back complete (no all-reduce follows).  Llama-4
        (routing score applied to the expert input, shared expert summed before one
        all-reduce) keeps the all-reduce form."""
        return self.ep and not self.scale_input and state.ep_dispatch() == "all_to_all"


class MixtralMoE(nn.Module):
    """block_sparse_moe (Mixtral) / mlp (Qwen-MoE): router + FusedMoE [+ shared expert]."""

    def __init__(self, cfg: ModelConfig, dtype, device):
        super().__init__()
        H = cfg.hidden_size
        inter = cfg.moe_intermediate_size or cfg.intermediate_size
        self.gate = ReplicatedLinear(H, cfg.num_local_experts, dtype=dtype, device=device)
        renorm = cfg.norm_topk_prob if cfg.architecture.startswith("Qwen") else True
        self.experts = FusedMoE(cfg.num_local_experts, cfg.num_experts_per_tok, H, inter, renorm,
                                dtype=dtype, device=device)
        self.shared_expert = None
        if cfg.shared_expert_intermediate_size:
            self.shared_expert = LlamaMLP(H, cfg.shared_expert_intermediate_size, "silu", dtype,
                                          device)
            self.shared_expert.down_proj.reduce_results = False   # one all-reduce for the sum
            self.shared_expert_gate = ReplicatedLinear(H, 1, dtype=dtype, device=device)

    def norm_and_route(self, h, residual, norm, md=None):
        """Decode: the O projection's split-K add + RMSNorm (``norm``) with this block's router
        and top-k in the same launch -> (x, residual, routing), or None when not applicable.
        A pure-decode batch on one rank (``md``) routes its bucket-padding rows (context 0) to
        no expert."""
        ex = self.experts
        if (self.gate.bias is not None or ex.scale_input or
                not moe_ops.splitk_norm_route_ok(h, residual, self.gate.weight, ex.k)):
            return None
        row_len = None
        if (md is not None and md.num_prefill_tokens == 0 and md.decode_seq_lens is not None
                and md.num_decode == h.M and state.tp_size() == 1 and not ex.ep):
            row_len = md.decode_seq_lens
        return moe_ops.splitk_norm_route(h, residual, norm.weight, norm.eps, self.gate.weight,
                                         ex.k, ex.renormalize, ex.scoring, row_len=row_len)

    def forward(self, x, routing=None):
        # one rank, no shared expert: the combine may be left to the next add + RMSNorm
        defer = self.shared_expert is None and state.tp_size() == 1
        if routing is not None:
            out = self.experts(x, None, reduce=False, routing=routing, defer_combine=defer)
        elif self.gate.bias is None and x.dim() == 2:
            out = self.experts(x, None, reduce=False, router_w=self.gate.weight,
                               defer_combine=defer)
        else:
            out = self.experts(x, self.gate(x), reduce=False)
        a2a = self.experts.a2a          # all-to-all EP: `out` is already complete
        if self.shared_expert is not None:
            s = self.shared_expert(x)
            s = s.materialize() if hasattr(s, "materialize") else s
            if a2a:
                s = comm.all_reduce(s)
            out = out + torch.sigmoid(self.shared_expert_gate(x).float()).to(x.dtype) * s
        if a2a:
            return out
        return _deferred_reduce(out)


class UngatedMLP(nn.Module):
    """W_down act(W_up x) without a gate branch.  ``act``: "relu2" (squared ReLU) or "xielu"
    (softplus(p) z^2 + z/2 above zero, (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2 below, with
    the layer's two learned numbers (p, q) in the parameter ``act``).  With ``defer`` the
    decode-sized products hand their split-K partial sums on: the up-projection's to the
    activation kernel, the down-projection's to the caller's boundary step.  ``own_up=False``:
    the up-projection's rows live in another module's fused projection of the same input, and
    ``forward(None, pre=...)`` takes its output (a tensor or split-K partial columns)."""

    def __init__(self, hidden: int, inter: int, dtype, device, act: str = "relu2",
                 defer: bool = False, own_up: bool = True):
        super().__init__()
        if act not in ("relu2", "xielu"):
            raise ValueError(f"UngatedMLP: unknown activation {act!r}")
        self.up = ReplicatedLinear(hidden, inter, dtype=dtype, device=device) if own_up else None
        self.down = ReplicatedLinear(inter, hidden, dtype=dtype, device=device)
        self.kind, self.defer = act, defer
        if act == "xielu":
            self.act = _param((2,), dtype, device)
            self.act.weight_loader = lambda p, t, sid=None: p.data.copy_(t.reshape(2))

    def forward(self, x, pre=None):
        from ..ops import activation, gemm
        from ..ops.gemm import SplitK, SplitKSlice
        if pre is None:
            pre = gemm.linear(x, self.up.weight, defer_reduce=self.defer and self.kind == "xielu")
        if self.kind == "relu2":
            if isinstance(pre, SplitKSlice):
                pre = pre.dense(self.down.weight.dtype)
            elif isinstance(pre, SplitK):
                pre = pre.materialize()
            return self.down(activation.relu2(pre.contiguous()))
        z = activation.xielu(pre, self.act)
        return gemm.linear(z, self.down.weight, defer_reduce=self.defer)


class GroupRoutedMoE(nn.Module):
    """Ungated experts behind a group-limited sigmoid router (ops/moe.py route_grouped +
    ungated_moe), plus an optional always-on shared expert.  One rank."""

    def __init__(self, hidden: int, inter: int, num_experts: int, top_k: int, num_groups: int,
                 keep_groups: int, route_scale: float, shared_inter: int = 0,
                 dtype=torch.bfloat16, device=None):
        super().__init__()
        if state.tp_size() != 1:
            raise NotImplementedError("GroupRoutedMoE runs on one rank")
        if num_experts % num_groups or not (1 <= keep_groups <= num_groups) or \
                top_k > keep_groups * (num_experts // num_groups):
            raise ValueError("router groups do not fit the expert count / top-k")
        self.E, self.k, self.groups, self.keep = num_experts, top_k, num_groups, keep_groups
        self.route_scale = float(route_scale)
        self.router = _param((num_experts, hidden), dtype, device)
        # a shared expert of the routed experts' size is stored as expert E and named by an extra
        # routing column of weight 1: it then rides in the routed experts' grouped launches
        self.merged_shared = shared_inter == inter and shared_inter > 0
        n = num_experts + (1 if self.merged_shared else 0)
        self.w_up = _param((n, inter, hidden), dtype, device)
        self.w_down = _param((n, hidden, inter), dtype, device)
        self.router.weight_loader = lambda p, t, sid=None: p.data.copy_(t)
        self.w_up.weight_loader = self.w_down.weight_loader = \
            lambda p, t, sid=None: p.data[sid].copy_(t)
        self.shared = UngatedMLP(hidden, shared_inter, dtype, device) \
            if (shared_inter and not self.merged_shared) else None

    def _route(self, x, md):
        row_len = None
        if md is not None and md.num_prefill_tokens == 0 and md.decode_seq_lens is not None:
            row_len = md.decode_seq_lens          # bucket-padding rows route nowhere
        return moe_ops.route_grouped(x, self.router, self.k, self.groups, self.keep,
                                     self.route_scale, row_len, always_on=self.merged_shared)

    def forward(self, x, md=None):
        tw, ids = self._route(x, md)
        out = moe_ops.ungated_moe(x, self.w_up, self.w_down, tw, ids, "relu2")
        if self.shared is not None:
            out = out + self.shared(x)
        return out

    def forward_post_norm(self, x, md, norm_w, eps: float, resid: torch.Tensor):
        """resid += layernorm(block(x)) * norm_w (fp32, in place); returns resid in x's dtype.
        On the GPU the experts' weighted sum, the shared expert's add, the norm and the
        residual update are one launch."""
        from ..ops import norm as norm_ops
        if not x.is_cuda:
            return norm_ops.post_norm_residual(self.forward(x, md), norm_w, eps, resid)
        tw, ids = self._route(x, md)
        h2, inv = moe_ops.ungated_moe(x, self.w_up, self.w_down, tw, ids, "relu2",
                                      rows_only=True)
        shared = self.shared(x) if self.shared is not None else None
        return moe_ops.combine_post_norm(h2, tw, inv, shared, norm_w, eps, resid)


class GroupLimitedMoE(nn.Module):
    """Gated experts  W_down (act(W_gate x) * (W_up x))  behind a group-limited router
    (ops/moe.py route_grouped + fused_moe): fp32 router logits over ``num_experts + identity``
    outputs, softmax (or sigmoid) scores, a stored per-output ``correction`` that is added for
    the selection only, groups of neighbouring outputs of which the best ``keep_groups`` (by
    their largest, or two largest, corrected scores) stay eligible, ``top_k`` winners weighing
    their plain scores times ``route_scale`` without renormalisation.  The last ``identity``
    outputs are identity experts: no weights, their output is the input.  An optional shared
    expert of size ``shared_inter`` runs for every token, times sigmoid(w_sg . x) when
    ``shared_gate``.  One rank."""

    def __init__(self, hidden: int, inter: int, num_experts: int, top_k: int, num_groups: int = 1,
                 keep_groups: int = 1, identity: int = 0, shared_inter: int = 0,
                 shared_gate: bool = True, scoring: str = "softmax", group_score: str = "max",
                 route_scale: float = 1.0, act: str = "silu", dtype=torch.bfloat16, device=None):
        super().__init__()
        if state.tp_size() != 1:
            raise NotImplementedError("GroupLimitedMoE runs on one rank")
        n_out = num_experts + identity
        if n_out % num_groups or not (1 <= keep_groups <= num_groups) or \
                top_k > keep_groups * (n_out // num_groups):
            raise ValueError("router groups do not fit the output count / top-k")
        self.E, self.identity, self.k = num_experts, int(identity), top_k
        self.groups, self.keep = num_groups, keep_groups
        self.scoring, self.group_score, self.route_scale = scoring, group_score, float(route_scale)
        self.act = act
        self.router = _param((n_out, hidden), dtype, device)
        self.correction = _param((n_out,), dtype, device)
        self.correction.data.zero_()
        self.router.weight_loader = self.correction.weight_loader = \
            lambda p, t, sid=None: p.data.copy_(t)
        # fp32 copy of the correction for the router launch, refreshed IN PLACE after a weight
        # load (captured decode graphs hold its address)
        self.corr_f32 = torch.zeros(n_out, dtype=torch.float32, device=device)
        self.w13 = _param((num_experts, 2 * inter, hidden), dtype, device)     # [gate; up] rows
        self.w2 = _param((num_experts, hidden, inter), dtype, device)
        self.w13.weight_loader = self._load_w13
        self.w2.weight_loader = lambda p, t, sid=None: p.data[sid].copy_(t)
        self.I = inter
        self.shared = LlamaMLP(hidden, shared_inter, act, dtype, device) if shared_inter else None
        # zero until a checkpoint (or the random init) fills it: an all-zero row means the
        # checkpoint has no gate, and the shared expert then counts whole
        self.shared_gate = None
        self.gated = False
        if self.shared is not None and shared_gate:
            self.shared_gate = _param((hidden,), dtype, device)
            self.shared_gate.data.zero_()
            self.shared_gate.weight_loader = lambda p, t, sid=None: p.data.copy_(t.reshape(-1))

    def _load_w13(self, param, loaded, shard_id):
        e, which = shard_id
        off = 0 if which == "gate" else self.I
        param.data[e, off:off + self.I].copy_(loaded)

    def refresh(self) -> None:
        self.corr_f32.copy_(self.correction.float())
        self.gated = self.shared_gate is not None and bool((self.shared_gate != 0).any())

    def forward(self, x: torch.Tensor, md=None) -> torch.Tensor:
        row_len = None
        if md is not None and md.num_prefill_tokens == 0 and md.decode_seq_lens is not None:
            row_len = md.decode_seq_lens          # bucket-padding rows route nowhere
        r = moe_ops.route_grouped(x, self.router, self.k, self.groups, self.keep,
                                  self.route_scale, row_len, scoring=self.scoring,
                                  group_score=self.group_score, correction=self.corr_f32,
                                  identity=self.identity,
                                  gate_w=self.shared_gate if self.gated else None)
        tw, ids = r[0], r[1]
        ident_w, sgate = (r[2], r[3]) if len(r) == 4 else (None, None)
        routed = moe_ops.fused_moe(x, self.w13, self.w2, tw, ids, (0, self.E), act=self.act)
        # (the shared expert's down projection may hand on split-K partials: summed in the
        # block's final launch)
        shared = self.shared(x) if self.shared is not None else None
        return moe_ops.finish_gated(routed, x, ident_w, shared, sgate)


class MixtralForCausalLM(LlamaForCausalLM):
    def __init__(self, cfg: ModelConfig, dtype=torch.bfloat16, device=None):
        super().__init__(cfg, dtype, device, layer_factory=lambda i: LlamaDecoderLayer(
            cfg, i, self.rotary, dtype, device, mlp=MixtralMoE(cfg, dtype, device)))

    def map_weight_name(self, name: str):
        n = name.replace("model.", "", 1) if name.startswith("model.") else name
        n = n.replace("block_sparse_moe.", "mlp.")
        if n.endswith(".mlp.experts.gate_up_proj"):      # transformers>=5 stacked [E, 2I, H]
            return n.replace("experts.gate_up_proj", "experts.w13"), "stacked"
        if n.endswith(".mlp.experts.down_proj"):         # stacked [E, H, I]
            return n.replace("experts.down_proj", "experts.w2"), "stacked"
        if ".mlp.experts." in n:
            pre, rest = n.split(".mlp.experts.", 1)
            e, _, w = rest.partition(".")
            which = {"w1": "w1", "w3": "w3", "w2": "w2", "gate_proj": "w1", "up_proj": "w3",
                     "down_proj": "w2"}[w.split(".")[0]]
            tgt = f"{pre}.mlp.experts.{'w2' if which == 'w2' else 'w13'}"
            return tgt, (int(e), which)
        if ".mlp.shared_expert." in n:
            for part, sid in (("gate_proj", 0), ("up_proj", 1)):
                if f".{part}." in n:
                    return n.replace(part, "gate_up_proj"), sid
            return n, None
        return super().map_weight_name(name)

    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]) -> List[str]:
        return _load_with_stacked_experts(self, weights, super().load_weights)


def _load_with_stacked_experts(model, weights, base_load):
    """Route stacked expert tensors ([E, out, in], or [E, in, out] = "fused_t") through the
    FusedMoE loaders (which shard per rank); everything else through ``base_load``."""
    params = dict(model.named_parameters())
    rest, loaded = [], []
    for name, t in weights:
        pname, sid = model.map_weight_name(name)
        if sid in ("stacked", "fused_t"):
            if pname not in params:          # layer of another pipeline stage
                continue
            p = params[pname]
            kind = "w13" if pname.endswith("w13") else "w2"
            for e in range(t.shape[0]):
                te = t[e].t() if sid == "fused_t" else t[e]
                p.weight_loader(p, te.to(p.dtype), (e, kind))
            loaded.append(pname)
        elif pname != "__skip__":
            rest.append((name, t))
    return loaded + base_load(rest)


# ----------------------------------------------------------------------------- Llama-4


class Llama4Attention(LlamaAttention):
    def __init__(self, cfg: ModelConfig, idx: int, rotary, dtype, device):
        super().__init__(cfg, idx, rotary, dtype, device)
        ex = cfg.extra
        nope = ex.get("no_rope_layers")
        self.use_rope = bool(nope[idx]) if nope else True
        if not self.use_rope:
            self.rotary = None
            self.chunk_size = None
        else:
            self.chunk_size = cfg.attention_chunk_size
        self.qk_l2 = bool(ex.get("use_qk_norm", True)) and self.use_rope
        self.temp_tuning = bool(ex.get("attn_temperature_tuning", True)) and not self.use_rope
        self.floor_scale = float(ex.get("floor_scale", 8192))
        self.attn_scale = float(ex.get("attn_scale", 0.1))
        D = cfg.head_dim
        if self.qk_l2:   # weightless L2 norm == RMSNorm with unit weight (rotation-invariant)
            self.register_buffer("ones", torch.ones(D, dtype=dtype, device=device),
                                 persistent=False)

    def forward(self, h, md, kv):
        from ..ops.attention import attention
        from ..ops.rotary import rope_qkv_cache
        from ..ops import gemm

        T = h.shape[0]
        # split-K QKV slabs are summed inside the RoPE / KV-write kernel (no reduce launch)
        qkv = gemm.linear(h, self.qkv_proj.weight, defer_reduce=True)
        q = rope_qkv_cache(qkv, md.positions, self.rotary, md.slot_mapping, kv[0], kv[1],
                           self.num_heads, self.num_kv_heads, self.head_dim,
                           bias=self.qkv_proj.bias,
                           q_norm_w=self.ones if self.qk_l2 else None,
                           k_norm_w=self.ones if self.qk_l2 else None,
                           norm_eps=self.cfg.rms_norm_eps)
        if self.temp_tuning:
            # the per-position temperature is the same for every NoPE layer of the step:
            # computed once per step (cached on the step's metadata), applied in fp32
            key = (self.floor_scale, self.attn_scale)
            cached = getattr(md, "_l4_attn_temp", None)
            if cached is None or cached[0] != key:
                pos = md.positions.float()
                sc = torch.log1p(torch.floor((pos + 1.0) / self.floor_scale)) * self.attn_scale \
                    + 1.0
                cached = (key, sc[:, None, None])
                md._l4_attn_temp = cached
            q = (q * cached[1]).to(q.dtype)
        o = attention(q, kv[0], kv[1], md, self.scale, None, self.chunk_size)
        return self.o_proj(o.view(T, self.num_heads * self.head_dim), defer_reduce=True)


class Llama4MoE(nn.Module):
    def __init__(self, cfg: ModelConfig, dtype, device):
        super().__init__()
        H = cfg.hidden_size
        self.router = ReplicatedLinear(H, cfg.num_local_experts, dtype=dtype, device=device)
        self.experts = FusedMoE(cfg.num_local_experts, cfg.num_experts_per_tok, H,
                                cfg.intermediate_size, renormalize=False, scoring="sigmoid",
                                scale_input=True, dtype=dtype, device=device)
        self.shared_expert = LlamaMLP(H, cfg.intermediate_size, "silu", dtype, device)
        self.shared_expert.down_proj.reduce_results = False   # one all-reduce for the sum

    def forward(self, x):
        if self.router.bias is None and x.dim() == 2:
            # router GEMM + sigmoid top-1 in one kernel (moe.hip route_kernel)
            routed = self.experts(x, None, reduce=False, router_w=self.router.weight)
        else:
            routed = self.experts(x, self.router(x), reduce=False)
        s = self.shared_expert.down_proj(self.shared_expert.gate_up_proj.forward_act_and_mul(x))
        return _deferred_reduce(routed + s)


class Llama4ForCausalLM(LlamaForCausalLM):
    def __init__(self, cfg: ModelConfig, dtype=torch.bfloat16, device=None):
        cfg.extra.setdefault("rope_interleaved", True)
        ml = cfg.extra.get("moe_layers")
        moe_layers = set(range(cfg.num_hidden_layers) if ml is None else ml)
        inter_mlp = cfg.extra.get("intermediate_size_mlp") or cfg.intermediate_size

        def make(i):
            mlp = Llama4MoE(cfg, dtype, device) if i in moe_layers else \
                LlamaMLP(cfg.hidden_size, inter_mlp, "silu", dtype, device)
            layer = LlamaDecoderLayer(cfg, i, self.rotary, dtype, device, mlp=mlp)
            layer.self_attn = Llama4Attention(cfg, i, self.rotary, dtype, device)
            return layer

        super().__init__(cfg, dtype, device, layer_factory=make)
        self.vision = None
        vc = cfg.extra.get("vision_config")
        if vc and os.environ.get("EIA_DISABLE_VISION", "0") != "1" and self.first:
            from .llama4_vision import Llama4VisionTower
            self.vision = Llama4VisionTower(vc, cfg.hidden_size, dtype, device)
            self.image_token_id = int(cfg.extra.get("image_token_id", 200092))

    def encode_images(self, pixel_values: torch.Tensor) -> torch.Tensor:
        """[tiles, 3, S, S] -> [tiles * 144, hidden] placeholder embeddings."""
        if self.vision is None:
            raise ValueError("this model was loaded without its vision tower")
        return self.vision(pixel_values)

    def map_weight_name(self, name: str):
        n = name
        for p in ("language_model.model.", "language_model.", "model."):
            if n.startswith(p):
                n = n[len(p):]
                break
        if n.startswith("vision_model") or n.startswith("multi_modal_projector"):
            return "__skip__", None
        n = n.replace(".feed_forward.", ".mlp.")
        if ".mlp.experts.gate_up_proj" in n:
            return n.replace("experts.gate_up_proj", "experts.w13"), "fused_t"
        if ".mlp.experts.down_proj" in n:
            return n.replace("experts.down_proj", "experts.w2"), "fused_t"
        if ".mlp.shared_expert." in n:
            for part, sid in (("gate_proj", 0), ("up_proj", 1)):
                if f".{part}." in n:
                    return n.replace(part, "gate_up_proj"), sid
            return n, None
        # dense (non-MoE) layers: feed_forward.{gate,up,down}_proj -> mlp.gate_up_proj / down_proj
        return super().map_weight_name(n)

    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]) -> List[str]:
        strip = lambda n: n[len("language_model."):] if n.startswith("language_model.") else n
        vis_loaded: List[str] = []

        def text_only(ws):
            for n, t in ws:
                m = n[len("model."):] if n.startswith("model.vision_model") or \
                    n.startswith("model.multi_modal_projector") else n
                if m.startswith(("vision_model.", "multi_modal_projector.")):
                    if self.vision is not None and self.vision.load_weight(m, t):
                        vis_loaded.append(n)
                    continue
                yield n, t

        loaded = _load_with_stacked_experts(
            self, text_only(weights), lambda rest: super(Llama4ForCausalLM, self).load_weights(
                (strip(n), t) for n, t in rest))
        return list(loaded) + vis_loaded
