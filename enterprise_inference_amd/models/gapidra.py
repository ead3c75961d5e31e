"""Gapidra: a decoder whose config.json lists its layers one by one.  A layer reads ONE RMS norm
of the fp32 residual stream and adds both of its sublayers to it,

    h = norm1(x);   x <- x + mixer(h) + ff(h),

where the mixer is ``latent_attention`` (LatentAttentionMixer: queries straight from h, keys and
values up-projected from one cached RMS-normed latent per token plus one rotated key part shared
by the heads, half-split rotation pairs, sliding window, a per-head sink in the softmax
denominator, element-wise sigmoid output gate) or ``attention`` (SigmoidWindowAttentionMixer:
grouped-query heads, query and key projections RMS-normed as whole vectors, interleaved rotation
pairs with optional frequency interpolation, sliding window, un-normalised sigmoid weights with a
per-head bias), models/mixers.py, and the optional feed-forward is ``W_down xielu(W_up h)``
(models/mixtral.py UngatedMLP).  The embedding is multiplied by ``embedding.scale``; the model's
norm with ``final.norm`` precedes the LM head.

config.json keys: architecture, vocab, width, norm{eps}, embedding{scale} and layers[i] = {type,
mixer{heads, kv_heads, dim, vdim, rot_dim, kv_rank, scale, mask{size}, rot{base, dims,
scaling{factor, original, fast, slow}}}, mlp{kind: dense, ff} | null}.  Checkpoint names: embed,
head, final.norm, l<i>.norm1, l<i>.mix.*, l<i>.mlp.up|down|act.

Residual stream, norms, angles, scores, attention weights and gates are fp32 whatever the
activation dtype; with dtype float32 the matrix products are fp32 too.  Both sublayers read the
same h, so the feed-forward's up-projection rides in the mixer's fused input projection (one
GEMM per layer input), and a layer boundary (both residual adds and the next layer's input
norm) is one launch (ops/norm.py residual_rms_step).
"""

from __future__ import annotations

import re
from typing import Iterable, List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..config import ModelConfig
from ..ops import gemm, norm as norm_ops
from ..ops.attention import AttentionMetadata
from .layers import _param, default_loader
from .mixers import (LatentAttentionMixer, LatentKVCache, PagedKVRows,
                     SigmoidWindowAttentionMixer)
from .mixtral import UngatedMLP


def _norm_weight(width, dtype, device):
    p = _param((width,), dtype, device)
    p.weight_loader = default_loader
    return p


class GapidraLayer(nn.Module):
    def __init__(self, spec: dict, width: int, eps: float, dtype, device):
        super().__init__()
        m = spec["mixer"]
        self.kind = spec["type"]
        mlp = spec.get("mlp")
        if mlp is not None and mlp.get("kind", "dense") != "dense":
            raise ValueError(f"unknown Gapidra feed-forward kind {mlp.get('kind')!r}")
        # both sublayers read the same h: the feed-forward's up-projection rides in the mixer's
        # fused input projection (one GEMM per layer input)
        ff = int(mlp["ff"]) if mlp is not None else 0
        window = int((m.get("mask") or {}).get("size", 0))
        rot = m.get("rot") or {}
        if self.kind == "latent_attention":
            rd = int(m.get("rot_dim", 0))
            self.mix = LatentAttentionMixer(
                width, m["heads"], m["dim"], rd, m.get("vdim", m["dim"]), m["kv_rank"], 0,
                m["scale"], int(rot.get("dims", rd)), float(rot.get("base", 10000.0)), eps,
                own_kv=True, dtype=dtype, device=device, gate="element", window=window, sink=True,
                rot_half=True, rot_scaling=rot.get("scaling"), defer_out=True, extra_rows=ff)
        elif self.kind == "attention":
            self.mix = SigmoidWindowAttentionMixer(
                width, m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"]),
                m["scale"], window, int(rot.get("dims", m["dim"] if rot else 0)),
                float(rot.get("base", 10000.0)),
                rot.get("scaling"), eps, dtype, device, extra_rows=ff)
        else:
            raise ValueError(f"unknown Gapidra layer type {self.kind!r}")
        self.norm1 = _norm_weight(width, dtype, device)
        self.eps = eps
        self.mlp = None
        if mlp is not None:
            self.mlp = UngatedMLP(width, ff, dtype, device, act="xielu", defer=True, own_up=False)

    def forward(self, x: torch.Tensor, h: torch.Tensor, md: AttentionMetadata, cache,
                w_next: Optional[torch.Tensor]):
        """x: fp32 residual [T, width], updated in place; h = norm1(x) in the activation dtype.
        Returns the next layer's input norm of the new x, or None when ``w_next`` is None."""
        if self.mlp is None:
            return norm_ops.residual_rms_step(x, self.eps, (self.mix(h, md, cache),), w_next)
        y, up = self.mix(h, md, cache, want_extra=True)
        return norm_ops.residual_rms_step(x, self.eps, (y, self.mlp(None, pre=up)), w_next)


class GapidraForCausalLM(nn.Module):
    supports_pp = False
    supports_float32 = True        # every kernel of this model has an fp32 form
    needs_state_slots = False
    supports_graphs = True         # no step reads anything back to the host

    def __init__(self, cfg: ModelConfig, dtype=torch.bfloat16, device=None):
        super().__init__()
        self.cfg = cfg
        self.dtype = dtype
        device = torch.device(device) if device is not None else torch.device("cpu")
        specs = cfg.extra["layers"]
        W = cfg.hidden_size
        self.eps = float((cfg.extra.get("norm") or {}).get("eps", cfg.rms_norm_eps))
        self.embed_scale = float((cfg.extra.get("embedding") or {}).get("scale", 1.0))
        self.embed = _param((cfg.vocab_size, W), dtype, device)
        self.embed.weight_loader = default_loader
        self.layers = nn.ModuleList([GapidraLayer(s, W, self.eps, dtype, device) for s in specs])
        self.final_norm = _norm_weight(W, dtype, device)
        self.head = _param((cfg.vocab_size, W), dtype, device)
        self.head.weight_loader = default_loader

    # ------------------------------------------------------------------ cache geometry
    def kv_heads_per_rank(self) -> int:
        return 1

    def _row_widths(self, L: GapidraLayer) -> int:
        if L.kind == "latent_attention":
            return L.mix.kv_rank + L.mix.rot_dim
        return sum(L.mix.cache_widths())

    def cache_block_bytes(self, block_size: int, dtype: torch.dtype) -> int:
        e = torch.tensor([], dtype=dtype).element_size()
        return sum(block_size * self._row_widths(L) * e for L in self.layers) or 1

    def state_slot_bytes(self) -> int:
        return 0

    def allocate_cache(self, num_blocks: int, block_size: int, num_slots: int,
                       dtype: torch.dtype, device) -> list:
        """One cache object per layer, all indexed by the same block tables: latent rows for a
        latent-attention layer, key rows + page-transposed values for an attention layer.  Zero
        filled: never-written rows stay finite under a zero weight."""
        out: list = []
        for L in self.layers:
            if L.kind == "latent_attention":
                out.append(LatentKVCache(torch.zeros(num_blocks, block_size, self._row_widths(L),
                                                     dtype=dtype, device=device)))
            else:
                kw, vw = L.mix.cache_widths()
                out.append(PagedKVRows.allocate(num_blocks, block_size, kw, vw, dtype, device))
        return out

    def prefill_query_block(self, block_size: int) -> int:
        """The step's work list is built for the first layer's query block; layers with another
        one get theirs from AttentionMetadata.prefill_work_for."""
        for L in self.layers:
            return L.mix.qblock if L.kind == "latent_attention" else L.mix.query_block(block_size)
        return 16

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids: torch.Tensor, md: AttentionMetadata, caches: list,
                intermediate=None, collect: Optional[list] = None):
        """Returns the fp32 residual stream [T, width].  ``collect`` (a list) receives a copy of
        the stream after every layer."""
        x = F.embedding(input_ids, self.embed).float()
        if self.embed_scale != 1.0:
            x *= self.embed_scale
        n = len(self.layers)
        if n == 0:
            return x
        h = norm_ops.residual_rms_step(x, self.eps, (), self.layers[0].norm1)
        for i, L in enumerate(self.layers):
            h = L(x, h, md, caches[i], self.layers[i + 1].norm1 if i + 1 < n else None)
            if collect is not None:
                collect.append(x.clone())
        return x

    def compute_logits(self, x: torch.Tensor) -> torch.Tensor:
        """x: rows of the fp32 residual stream -> fp32 logits."""
        h = norm_ops.residual_rms_step(x.contiguous(), self.eps, (), self.final_norm)
        out = gemm.linear_f32(h, self.head) if h.dtype == torch.bfloat16 and h.is_cuda else None
        return out if out is not None else gemm.linear(h, self.head).float()

    # ------------------------------------------------------------------ weights
    _LAYER = re.compile(r"^l(\d+)\.(.+)$")
    _LATENT = {"q": ("down", "q"), "dkv": ("down", "dkv"), "g": ("down", "g"),
               "dkv.norm": ("kv_norm", None)}
    _ATTN = {"q": ("proj", "q"), "k": ("proj", "k"), "v": ("proj", "v"),
             "q.norm": ("q_norm", None), "k.norm": ("k_norm", None)}
    _MLP = {"down": "down.weight", "act": "act"}

    def _target(self, name: str):
        """checkpoint name -> (parameter name, shard id)."""
        if name in ("embed", "head"):
            return name, None
        if name == "final.norm":
            return "final_norm", None
        m = self._LAYER.match(name)
        if not m or int(m.group(1)) >= len(self.layers):
            return None, None
        i, rest = int(m.group(1)), m.group(2)
        pre = f"layers.{i}."
        if rest == "norm1":
            return pre + rest, None
        if rest.startswith("mix."):
            table = self._LATENT if self.layers[i].kind == "latent_attention" else self._ATTN
            p, sid = table.get(rest[4:], (rest[4:], None))
            return pre + "mix." + p, sid
        if rest == "mlp.up":              # rows of the mixer's fused input projection
            fused = "down" if self.layers[i].kind == "latent_attention" else "proj"
            return pre + "mix." + fused, "x"
        if rest.startswith("mlp.") and rest[4:] in self._MLP:
            return pre + "mlp." + self._MLP[rest[4:]], None
        return None, None

    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]) -> List[str]:
        params = dict(self.named_parameters())
        loaded = []
        for name, t in weights:
            pname, sid = self._target(name)
            if pname is None or pname not in params:
                raise ValueError(f"unexpected tensor {name!r} for this Gapidra configuration")
            p = params[pname]
            t = t.to(p.dtype)
            if sid is None:
                p.weight_loader(p, t)
            else:
                p.weight_loader(p, t, sid)
            loaded.append(pname)
        return loaded

    def init_random(self, seed: int = 0) -> None:
        """Random weights of a plausible scale (no checkpoint): unit norm weights, matrices
        N(0, 1/fan_in), small sinks and activation numbers, score biases that keep the sigmoid
        weights of a window's keys small."""
        import zlib
        for name, p in self.named_parameters():
            g = torch.Generator(device=p.device)
            g.manual_seed(seed * 1000003 + zlib.crc32(name.encode()))
            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("norm1", "final_norm", "q_norm", "k_norm", "kv_norm"):
                p.data.fill_(1.0)
            elif leaf == "pb":
                p.data.fill_(-3.0)
            elif leaf in ("sink", "act"):
                p.data.copy_(torch.randn(p.shape, generator=g, device=p.device) * 0.3)
            elif leaf in ("proj", "down") and name.endswith(("mix.proj", "mix.down")):
                mix = self.get_submodule(name.rsplit(".", 1)[0])
                spans = (list(mix.offsets.values()) if leaf == "proj" else
                         [(0, mix.q_rows + mix.kv_rows + mix.gate_rows),
                          (mix.extra_off, mix.extra_rows)])
                p.data.zero_()                      # pad rows stay zero
                for off, rows in spans:
                    p.data[off:off + rows].copy_(
                        torch.randn((rows, p.shape[1]), generator=g, device=p.device,
                                    dtype=torch.float32) * p.shape[-1] ** -0.5)
            else:
                p.data.copy_(torch.randn(p.shape, generator=g, device=p.device,
                                         dtype=torch.float32) * p.shape[-1] ** -0.5)

    def post_load(self) -> None:
        for L in self.layers:
            L.mix.refresh()
