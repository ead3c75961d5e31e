"""Daburax: a decoder whose config.json lists its layers one by one.  The token embedding is
scaled and joined by a row of a hashed bigram table (ops/embedding.py); the residual is kept as
``streams`` fp32 copies joined by hyper-connections -- every sublayer q of a layer reads
u = sum_s in_q[s] x_s through an RMS norm whose weight is stored around zero, and all streams
are rewritten at once,

    x_t <- sum_s mix_q[s, t] x_s + residual_mult * out_q[t] * sublayer(norm_q(u)),

(ops/norm.py hyper_step: one launch per sublayer boundary; without ``streams`` it is the plain
pre-norm residual sum).  Mixers (models/mixers.py): ``retention`` (RetentionMixer: rotated q / k,
a fixed decay per head, matrix state on state slots, head RMS norm, SiLU gate) and ``parallel``
(ParallelMixer: a grouped-query softmax attention with biases, partial interleaved rotation with
position interpolation and a per-head sink in the denominator, beside a gated matrix memory with
a stabilised exponential input gate; one fused input projection, one output projection).  The
optional feed-forward is a mixture of SiLU-gated experts behind a group-limited softmax router
with a selection-only correction, identity experts and a sigmoid-gated shared expert
(models/mixtral.py GroupLimitedMoE).  The model's norm with ``final.norm`` on the sum of the
streams precedes the LM head.

config.json keys: architecture, vocab, width, norm{eps}, residual_mult, streams,
embedding{scale, bigram{buckets, mul_prev, mul_cur}} and layers[i] = {type, mixer{...},
mlp{kind: moe, expert{ff}, router{experts, top, identity, groups{count, keep}}, shared{ff}} |
null}.  Checkpoint names: embed, bigram, head, final.norm, l<i>.norm1|norm2, l<i>.hc1|hc2.in|
out|mix, l<i>.mix.*, l<i>.mlp.*.

Residual streams, norms, angles, scores and softmax weights, routing, gates, decays and the
recurrent states are fp32 whatever the activation dtype; with dtype float32 the matrix products
are fp32 too.
"""

from __future__ import annotations

import re
from typing import Iterable, List, Optional, Tuple

import torch
import torch.nn as nn

from ..config import ModelConfig
from ..ops import embedding as emb_ops
from ..ops import gemm, norm as norm_ops
from ..ops.attention import AttentionMetadata
from .layers import _param, default_loader
from .mixers import FusedProjection, PagedKVRows, ParallelMixer, RetentionMixer
from .mixtral import GroupLimitedMoE


def _plain(shape, dtype, device):
    p = _param(shape, dtype, device)
    p.weight_loader = default_loader
    return p


class HyperConnection(nn.Module):
    """The three learned pieces of one sublayer's hyper-connection over ``streams`` residual
    streams: read weights ``inw`` [s], write weights ``outw`` [s] and the stream-mixing matrix
    ``mix`` [s, s] (from, to), with fp32 copies for the boundary launches (refreshed IN PLACE
    after a weight load: captured decode graphs hold their addresses).  ``streams`` 0: the plain
    residual sum, one stream with unit constants and no parameters."""

    def __init__(self, streams: int, dtype, device):
        super().__init__()
        self.learned = streams > 0
        n = max(1, streams)
        if self.learned:
            self.inw = _plain((n,), dtype, device)
            self.outw = _plain((n,), dtype, device)
            self.mix = _plain((n, n), dtype, device)
        self.in_f32 = torch.ones(n, dtype=torch.float32, device=device)
        self.out_f32 = torch.ones(n, dtype=torch.float32, device=device)
        self.mix_f32 = torch.eye(n, dtype=torch.float32, device=device)

    def refresh(self) -> None:
        if self.learned:
            self.in_f32.copy_(self.inw.float())
            self.out_f32.copy_(self.outw.float())
            self.mix_f32.copy_(self.mix.float())


class DaburaxLayer(nn.Module):
    def __init__(self, spec: dict, width: int, eps: float, streams: int, dtype, device):
        super().__init__()
        m = spec["mixer"]
        self.kind = spec["type"]
        if self.kind == "retention":
            rot = m.get("rot") or {}
            # (a rot entry without dims rotates the whole head)
            self.mix = RetentionMixer(width, m["heads"], m["dim"], m.get("vdim", m["dim"]),
                                      m["decay"], int(rot.get("dims", m["dim"] if rot else 0)),
                                      float(rot.get("base", 10000.0)), rot.get("scaling"), eps,
                                      dtype, device)
        elif self.kind == "parallel":
            left, right = dict(m["left"]), dict(m["right"])
            left.setdefault("kv_heads", left["heads"])
            left.setdefault("vdim", left["dim"])
            left.setdefault("scale", float(left["dim"]) ** -0.5)
            right.setdefault("gate_cap", 0.0)           # (no cap)
            right.setdefault("vdim", right["dim"])
            self.mix = ParallelMixer(width, left, right, float(m.get("left_scale", 1.0)),
                                     float(m.get("right_scale", 1.0)), eps, dtype, device)
        else:
            raise ValueError(f"unknown Daburax layer type {self.kind!r}")
        self.norm1 = _plain((width,), dtype, device)
        self.hc1 = HyperConnection(streams, dtype, device)
        self.eps = eps
        mlp = spec.get("mlp")
        self.mlp = None
        if mlp is not None:
            if mlp.get("kind", "moe") != "moe":
                raise ValueError(f"unknown Daburax feed-forward kind {mlp.get('kind')!r}")
            r = mlp["router"]
            g = r.get("groups") or {"count": 1, "keep": 1}
            self.mlp = GroupLimitedMoE(width, int(mlp["expert"]["ff"]), int(r["experts"]),
                                       int(r["top"]), int(g.get("count", 1)), int(g.get("keep", 1)),
                                       int(r.get("identity", 0)),
                                       int((mlp.get("shared") or {}).get("ff", 0)),
                                       dtype=dtype, device=device)
            self.norm2 = _plain((width,), dtype, device)
            self.hc2 = HyperConnection(streams, dtype, device)

    def boundaries(self):
        """(hyper-connection, norm weight) of this layer's sublayers, in order."""
        out = [(self.hc1, self.norm1)]
        if self.mlp is not None:
            out.append((self.hc2, self.norm2))
        return out


class DaburaxForCausalLM(nn.Module):
    supports_pp = False
    supports_float32 = True        # every kernel of this model has an fp32 form
    needs_state_slots = True       # recurrent layers and the previous token of the bigram term

    def __init__(self, cfg: ModelConfig, dtype=torch.bfloat16, device=None):
        super().__init__()
        self.cfg = cfg
        self.dtype = dtype
        device = torch.device(device) if device is not None else torch.device("cpu")
        ex = cfg.extra
        specs = ex["layers"]
        W = cfg.hidden_size
        self.eps = float((ex.get("norm") or {}).get("eps", cfg.rms_norm_eps))
        emb = ex.get("embedding") or {}
        self.embed_scale = float(emb.get("scale", 1.0))
        self.bigram_cfg = dict(emb["bigram"]) if emb.get("bigram") else None
        self.mult = float(ex.get("residual_mult", 1.0) if ex.get("residual_mult") is not None
                          else 1.0)
        self.streams = int(ex.get("streams") or 0)      # 0: plain residual (one stream)
        self.embed = _plain((cfg.vocab_size, W), dtype, device)
        self.bigram = None
        if self.bigram_cfg:
            self.bigram = _plain((int(self.bigram_cfg["buckets"]) + 1, W), dtype, device)
        self.layers = nn.ModuleList([DaburaxLayer(s, W, self.eps, self.streams, dtype, device)
                                     for s in specs])
        self.final_norm = _plain((W,), dtype, device)
        self.head = _plain((cfg.vocab_size, W), dtype, device)
        self.ones = torch.ones(max(1, self.streams), dtype=torch.float32, device=device)
        # decode steps replay HIP graphs when every expert block has a device-side grouped form
        # (bf16, width a multiple of 128 and expert ff a multiple of 64); else they read row
        # offsets back per layer
        self.supports_graphs = dtype == torch.bfloat16 and all(
            L.mlp is None or (W % 128 == 0 and L.mlp.I % 64 == 0) for L in self.layers)
        # the sublayer boundaries in order: (layer, hyper-connection, norm weight)
        self.steps = [(i, hc, w) for i, L in enumerate(self.layers) for hc, w in L.boundaries()]

    # ------------------------------------------------------------------ cache geometry
    def kv_heads_per_rank(self) -> int:
        return 1

    def cache_block_bytes(self, block_size: int, dtype: torch.dtype) -> int:
        e = torch.tensor([], dtype=dtype).element_size()
        return sum(block_size * sum(L.mix.left.cache_widths()) * e for L in self.layers
                   if L.kind == "parallel") or 1

    def state_slot_bytes(self) -> int:
        return 4 + sum((L.mix if L.kind == "retention" else L.mix.right).state_bytes()
                       for L in self.layers)

    def allocate_cache(self, num_blocks: int, block_size: int, num_slots: int,
                       dtype: torch.dtype, device) -> list:
        """Per-layer cache objects, then one more entry for the embedding: state slots for a
        retention layer; (paged K / V rows, state slots) for a parallel layer; the previous
        token per slot (int32) for the bigram term.  Zero filled: never-written rows stay finite
        under a zero softmax weight."""
        out: list = []
        for L in self.layers:
            if L.kind == "retention":
                out.append(L.mix.allocate_state(num_slots, device))
            else:
                kw, vw = L.mix.left.cache_widths()
                out.append((PagedKVRows.allocate(num_blocks, block_size, kw, vw, dtype, device),
                            L.mix.right.allocate_state(num_slots, device)))
        out.append(torch.zeros(max(1, num_slots), dtype=torch.int32, device=device))
        return out

    def prefill_query_block(self, block_size: int) -> int:
        """The step's work list is built for the first attention layer's query block; layers
        with another one get theirs from AttentionMetadata.prefill_work_for."""
        for L in self.layers:
            if L.kind == "parallel":
                return L.mix.left.query_block(block_size)
        return 16

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids: torch.Tensor, md: AttentionMetadata, caches: list,
                intermediate=None, collect: Optional[list] = None):
        """Returns the fp32 residual streams [T, streams, width].  ``collect`` (a list) receives
        the sum of the streams after every layer."""
        bg = self.bigram_cfg or {}
        T = input_ids.shape[0]
        nseq = md.num_seqs if md.num_seqs else T
        X = emb_ops.bigram_embed(input_ids, self.embed, self.embed_scale, self.bigram,
                                 int(bg.get("buckets", 1)), int(bg.get("mul_prev", 0)),
                                 int(bg.get("mul_cur", 0)), caches[len(self.layers)],
                                 md.seq_slots, md.seq_cu, nseq, md.positions,
                                 max(1, self.streams))
        steps = self.steps
        if not steps:
            return X
        h = norm_ops.hyper_step(X, self.eps, None, in_next=steps[0][1].in_f32,
                                w_next=steps[0][2], w_offset=1.0)
        for n, (i, hc, _) in enumerate(steps):
            L = self.layers[i]
            y = L.mix(h, md, caches[i]) if hc is L.hc1 else L.mlp(h, md)
            nxt = steps[n + 1] if n + 1 < len(steps) else None
            h = norm_ops.hyper_step(X, self.eps, y, hc.mix_f32, hc.out_f32, self.mult,
                                    nxt[1].in_f32 if nxt else None, nxt[2] if nxt else None, 1.0)
            if collect is not None and (nxt is None or nxt[0] != i):
                collect.append(X.sum(1))
        return X

    def compute_logits(self, X: torch.Tensor) -> torch.Tensor:
        """X: rows of the fp32 residual streams [n, streams, width] -> fp32 logits."""
        h = norm_ops.hyper_step(X.contiguous(), self.eps, None, in_next=self.ones,
                                w_next=self.final_norm, w_offset=1.0)
        out = gemm.linear_f32(h, self.head) if h.dtype == torch.bfloat16 and h.is_cuda else None
        return out if out is not None else gemm.linear(h, self.head).float()

    # ------------------------------------------------------------------ weights
    _LAYER = re.compile(r"^l(\d+)\.(.+)$")
    _HC = {"in": "inw", "out": "outw", "mix": "mix"}

    def _target(self, name: str):
        """checkpoint name -> (parameter name, shard id)."""
        if name in ("embed", "head", "bigram"):
            return name, None
        if name == "final.norm":
            return "final_norm", None
        m = self._LAYER.match(name)
        if not m or int(m.group(1)) >= len(self.layers):
            return None, None
        i, rest = int(m.group(1)), m.group(2)
        pre = f"layers.{i}."
        L = self.layers[i]
        if rest in ("norm1", "norm2"):
            return pre + rest, None
        hc = re.match(r"^(hc[12])\.(in|out|mix)$", rest)
        if hc:
            return pre + hc.group(1) + "." + self._HC[hc.group(2)], None
        if rest.startswith("mix."):
            k = rest[4:]
            if L.kind == "retention":
                if k in ("q", "k", "v", "g"):
                    return pre + "mix.proj.weight", k
                return pre + "mix." + k, None
            side, _, leaf = k.partition(".")
            if side not in ("left", "right"):
                return None, None
            if leaf == "o":
                return pre + "mix.o", side
            if leaf.endswith(".b") and leaf[:-2] in ("q", "k", "v", "i", "f"):
                return pre + "mix.proj.bias", side + "." + leaf[:-2]
            if leaf in ("q", "k", "v", "g", "i", "f") and not (side == "left" and leaf in ("g", "i", "f")):
                return pre + "mix.proj.weight", side + "." + leaf
            return pre + f"mix.{side}.{leaf}", None
        if rest.startswith("mlp.") and L.mlp is not None:
            k = rest[4:]
            e = re.match(r"^e(\d+)\.(gate|up|down)$", k)
            if e:
                if e.group(2) == "down":
                    return pre + "mlp.w2", int(e.group(1))
                return pre + "mlp.w13", (int(e.group(1)), e.group(2))
            table = {"router": ("router", None), "correction": ("correction", None),
                     "shared.gate": ("shared.gate_up_proj.weight", 0),
                     "shared.up": ("shared.gate_up_proj.weight", 1),
                     "shared.down": ("shared.down_proj.weight", None),
                     "shared.sg": ("shared_gate", None)}
            if k in table:
                return pre + "mlp." + table[k][0], table[k][1]
        return None, None

    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]) -> List[str]:
        params = dict(self.named_parameters())
        loaded = []
        for name, t in weights:
            pname, sid = self._target(name)
            if pname is None or pname not in params:
                raise ValueError(f"unexpected tensor {name!r} for this Daburax configuration")
            p = params[pname]
            t = t.to(p.dtype)
            if sid is None:
                p.weight_loader(p, t)
            else:
                p.weight_loader(p, t, sid)
            loaded.append(pname)
        return loaded

    def init_random(self, seed: int = 0) -> None:
        """Random weights of a plausible scale (no checkpoint): norm weights and corrections
        around zero, matrices N(0, 1/fan_in), stream constants near the plain residual sum,
        small sinks and gate biases."""
        import zlib
        for mname, mod in self.named_modules():
            if isinstance(mod, FusedProjection):
                g = torch.Generator(device=mod.weight.device)
                g.manual_seed(seed * 1000003 + zlib.crc32(mname.encode()))
                mod.init_random(g)
        for name, p in self.named_parameters():
            if name.endswith(("proj.weight", "proj.bias")) and ".mix." in name:
                continue
            g = torch.Generator(device=p.device)
            g.manual_seed(seed * 1000003 + zlib.crc32(name.encode()))
            leaf = name.rsplit(".", 1)[-1]
            rnd = lambda s: torch.randn(p.shape, generator=g, device=p.device,
                                        dtype=torch.float32) * s
            if leaf in ("norm1", "norm2", "final_norm", "correction"):
                p.data.copy_(rnd(0.02))
            elif leaf == "norm":
                p.data.copy_(1.0 + rnd(0.05))
            elif leaf in ("inw", "outw"):
                n = p.shape[0]
                p.data.copy_((1.0 / n if leaf == "inw" else 1.0) + rnd(0.05))
            elif leaf == "mix" and name.count("hc"):
                p.data.copy_(torch.eye(p.shape[0], device=p.device) + rnd(0.05))
            elif leaf == "sink":
                p.data.copy_(rnd(0.3))
            elif leaf == "bigram":
                p.data.copy_(rnd(0.5))
            elif leaf == "o" and p.dim() == 2 and name.endswith("mix.o"):
                p.data.copy_(rnd(p.shape[-1] ** -0.5))
                mix = self.get_submodule(name.rsplit(".", 1)[0])
                if isinstance(mix, ParallelMixer):
                    p.data[:, mix.lw:mix.lw_pad].zero_()
                    p.data[:, mix.lw_pad + mix.rw:].zero_()
            else:
                p.data.copy_(rnd(p.shape[-1] ** -0.5))

    def post_load(self) -> None:
        for L in self.layers:
            L.mix.refresh()
            L.hc1.refresh()
            if L.mlp is not None:
                L.mlp.refresh()
                L.hc2.refresh()
