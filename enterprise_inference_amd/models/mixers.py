"""Token mixers beyond multi-head softmax attention over a K/V cache, and the cache layouts
they need.  Each mixer owns its parameters under the checkpoint's names, reads the layer input
in the model's activation dtype (plus the fp32 residual where the mechanism needs it) and
returns the mixer output in the activation dtype.

* ``LatentAttentionMixer`` -- attention through low-rank latents: queries and keys/values are
  up-projected from RMS-normed latents, a rotated key part is shared by all heads, and only the
  KV latent and that key part are cached (one row per token, shared by every head; a layer may
  read another layer's rows).  Runs in the absorbed form (ops/latent_attention.py).  Options:
  queries straight from the layer input (``q_rank`` 0), a sliding window, a per-head sink in
  the softmax denominator, either pair layout of the rotation, and an output gate per head or
  per element.
* ``WKVMixer`` -- token-shift mixing and a per-head matrix-state recurrence with data-dependent
  per-channel decay on per-sequence state slots (ops/wkv.py).
* ``TalkingWindowAttentionMixer`` -- sliding-window softmax attention without rotation: RMS-normed
  queries and keys, the un-normed keys as values, a per-head temperature, a linear distance
  penalty, mixing of the heads' scores before the softmax and a sigmoid output gate.
* ``DifferentialAttentionMixer`` -- two softmax maps per head over the same values, combined as
  ``a1 - lambda * a2`` and RMS-normed per head; sliding window plus always-visible first tokens.
* ``SigmoidWindowAttentionMixer`` -- grouped-query sliding-window attention whose weights are
  ``sigmoid(score + bias_h)``, not normalised over the keys; queries and keys are RMS-normed as
  whole projections and then rotated.
* ``SinkAttentionMixer`` -- grouped-query causal softmax attention with projection biases, a
  partial rotation with optional position interpolation and a learned per-head sink in the
  softmax denominator (optionally windowed).
  All four run on token-major paged K / V rows (``PagedKVRows``, ops/window_attention.py).
* ``RetentionMixer`` -- linear attention with a fixed decay per head: rotated q / k, a matrix
  state per head on per-sequence state slots, head RMS norm, SiLU gate.
* ``MatrixMemoryMixer`` -- a gated matrix memory: exponential input gate and sigmoid forget gate
  per head with soft-capped pre-activations, stabilised by a running maximum, a normaliser
  state, head RMS norm with a weight, sigmoid gate.  Both run ops/linear_scan.py.
* ``ParallelMixer`` -- an attention mixer and a recurrent mixer side by side on the same input:
  one fused input projection, one output projection over the concatenated heads, the two
  outputs added with fixed factors.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from ..ops import activation as act_ops
from ..ops import gemm
from ..ops import latent_attention as lat_ops
from ..ops import linear_scan as scan_ops
from ..ops import rotary as rot_ops
from ..ops import window_attention as win_ops
from ..ops import wkv as wkv_ops
from ..ops.attention import AttentionMetadata
from ..parallel import state as pstate
from .layers import _param, default_loader


def _plain(shape, dtype, device) -> nn.Parameter:
    p = _param(shape, dtype, device)
    p.weight_loader = default_loader
    return p


class LatentKVCache:
    """Paged latent cache of one layer: rows [c | k_rot], tensor [blocks, block, kv_rank +
    rot_dim] in the activation dtype."""

    __slots__ = ("rows",)

    def __init__(self, rows: torch.Tensor):
        self.rows = rows


class RecurrentState:
    """Per-sequence slots of one recurrent layer: S fp32 [slots, heads, dk, dv] and the previous
    token's layer input, fp32 [slots, width]."""

    __slots__ = ("S", "prev")

    def __init__(self, S: torch.Tensor, prev: torch.Tensor):
        self.S, self.prev = S, prev


class LatentAttentionMixer(nn.Module):
    """Keys and values of every head are up-projections (``uk``, ``uv``) of one RMS-normed
    latent per token; a rotated key part is shared by the heads; only both are cached.

    ``q_rank`` > 0: queries are up-projected (``uq``) from an RMS-normed query latent; 0: they
    come straight from the layer input (``q`` rows in the fused projection).  ``gate``: "head"
    (one sigmoid per head, applied to the attended latent), "element" (sigmoid(W_g x) on the
    concatenated heads, after the value up-projection) or None.  ``window`` > 0: sliding window.
    ``sink``: a learned per-head term exp(sink_h) in the softmax denominator.  ``rot_half``:
    rotation pairs (i, i + dims/2) instead of (2i, 2i+1); ``rot_scaling``: frequency
    interpolation (ops/rotary.py rotary_frequencies).  ``defer_out``: hand the output
    projection's split-K partials to the caller's boundary step.  ``extra_rows``: that many more
    rows ride in the fused input projection (shard "x": another consumer of the same layer
    input, e.g. a feed-forward that runs beside the mixer); ``forward(..., want_extra=True)``
    then returns (output, their columns)."""

    def __init__(self, width: int, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int,
                 q_rank: int, scale: float, rot_dims: int, rot_base: float, eps: float,
                 own_kv: bool, dtype, device, *, gate: str = "head", window: int = 0,
                 sink: bool = False, rot_half: bool = False, rot_scaling=None,
                 defer_out: bool = False, extra_rows: int = 0):
        super().__init__()
        if pstate.tp_size() != 1:
            raise NotImplementedError("latent attention runs on one rank (no head sharding yet)")
        if gate not in ("head", "element", None):
            raise ValueError(f"latent attention gate {gate!r}")
        if rot_dims > rot_dim or rot_dims % 2:
            raise ValueError("rot.dims must be even and at most rot_dim")
        self.width, self.heads, self.dim, self.rot_dim, self.vdim = width, heads, dim, rot_dim, vdim
        self.kv_rank, self.q_rank, self.scale, self.eps = kv_rank, q_rank, float(scale), float(eps)
        self.rot_dims = rot_dims
        self.own_kv = own_kv
        self.gate, self.window, self.rot_half, self.defer_out = gate, int(window), rot_half, defer_out
        # one fused projection of the layer input: [query latent or queries | KV latent | shared
        # rotary key | gates]; a layer reading another layer's cache has no KV rows
        self.kv_rows = kv_rank + rot_dim if own_kv else 0
        self.q_rows = q_rank if q_rank else heads * (dim + rot_dim)
        self.gate_rows = {"head": heads, "element": heads * vdim, None: 0}[gate]
        # (rows padded with zeros to a multiple of 64: decode-sized batches then run the
        # weight-streaming GEMM, whose row tiles need it; the pad columns are never read)
        n = self.q_rows + self.kv_rows + self.gate_rows
        self.extra_rows = int(extra_rows)
        self.extra_off = -(-n // 8) * 8 if extra_rows else n      # (16-byte aligned columns)
        n = self.extra_off + self.extra_rows
        self.down = _param((-(-n // 64) * 64, width), dtype, device)
        self.down.data.zero_()
        self.down.weight_loader = self._load_down
        self.q_norm = _plain((q_rank,), dtype, device) if q_rank else None
        self.kv_norm = _plain((kv_rank,), dtype, device) if own_kv else None
        self.uq = _plain((heads * (dim + rot_dim), q_rank), dtype, device) if q_rank else None
        self.uk = _plain((heads * dim, kv_rank), dtype, device)
        self.uv = _plain((heads * vdim, kv_rank), dtype, device)
        self.o = _plain((width, heads * vdim), dtype, device)
        self.sink = _plain((heads,), dtype, device) if sink else None
        # fp32 copy of the sinks for the attention launch, refreshed IN PLACE after a weight
        # load (captured decode graphs hold its address)
        self.sink_f32 = torch.zeros(heads, dtype=torch.float32, device=device) if sink else None
        self.inv_freq, self.rot_amp = rot_ops.rotary_frequencies(rot_dims, rot_base, rot_scaling,
                                                                 device)
        self.qblock = lat_ops.query_block(heads, kv_rank, rot_dim,
                                          dtype if torch.device(device).type == "cuda"
                                          else torch.float32)

    def refresh(self) -> None:
        if self.sink is not None:
            self.sink_f32.copy_(self.sink.float())

    def _load_down(self, param, loaded, shard_id=None):
        off = {"dq": 0, "q": 0, "dkv": self.q_rows, "g": self.q_rows + self.kv_rows,
               "x": self.extra_off}[shard_id]
        rows = {"dq": self.q_rows, "q": self.q_rows, "dkv": self.kv_rows, "g": self.gate_rows,
                "x": self.extra_rows}[shard_id]
        if loaded.shape[0] != rows or param.data[off:off + rows].shape != loaded.shape:
            raise ValueError(f"latent attention {shard_id}: shape {tuple(loaded.shape)}")
        param.data[off:off + rows].copy_(loaded)

    def forward(self, xb: torch.Tensor, md: AttentionMetadata, cache: LatentKVCache,
                want_extra: bool = False):
        T = xb.shape[0]
        H, D, rd, R = self.heads, self.dim, self.rot_dim, self.kv_rank
        fused = gemm.linear(xb, self.down)
        cq = lat_ops.latent_prep(fused, 0, self.q_rank, self.q_norm, self.q_rows, R, self.kv_norm,
                                 self.q_rows + R, rd, self.rot_dims, self.inv_freq, md.positions,
                                 md.slot_mapping, cache.rows if self.own_kv else None, self.eps,
                                 self.rot_half, self.rot_amp)
        if self.q_rank:
            q = gemm.linear(cq, self.uq).view(T, H, D + rd)
        else:
            q = fused[:, :self.q_rows].view(T, H, D + rd)
        # key up-projection folded into the query: q_abs[t, h] = W_uk[h]^T q_nope[t, h]
        q_abs = torch.bmm(q[:, :, :D].transpose(0, 1), self.uk.view(H, D, R)).transpose(0, 1)
        g0 = self.q_rows + self.kv_rows
        lat = lat_ops.latent_attention(q_abs, q[:, :, D:], self.inv_freq, self.rot_dims,
                                       cache.rows, md,
                                       fused[:, g0:g0 + H] if self.gate == "head" else None,
                                       self.scale, self.window, self.sink_f32, self.rot_half,
                                       self.rot_amp)
        # value up-projection of the attended latent, heads concatenated
        o = torch.bmm(lat.transpose(0, 1), self.uv.view(H, self.vdim, R).transpose(1, 2))
        if self.gate == "element":      # [H, T, vdim] -> gated [T, H * vdim] in one pass
            o = act_ops.sigmoid_gate(o, fused[:, g0:g0 + self.gate_rows])
        else:
            o = o.transpose(0, 1).reshape(T, H * self.vdim)
        y = gemm.linear(o, self.o, defer_reduce=self.defer_out)
        if want_extra:
            return y, fused[:, self.extra_off:self.extra_off + self.extra_rows]
        return y


class WKVMixer(nn.Module):
    STREAMS = ("r", "k", "v", "g", "w")

    def __init__(self, width: int, heads: int, dim: int, decay_rank: int, eps: float, dtype,
                 device):
        super().__init__()
        if pstate.tp_size() != 1:
            raise NotImplementedError("the wkv mixer runs on one rank (no head sharding yet)")
        self.width, self.heads, self.dim, self.eps = width, heads, dim, float(eps)
        hd = heads * dim
        self.mu = _param((5, width), dtype, device)              # r, k, v, g, w
        self.mu.weight_loader = self._load_stream
        self.rkvg = _param((4, hd, width), dtype, device)        # W_r, W_k, W_v, W_g
        self.rkvg.weight_loader = self._load_stream
        self.w1 = _plain((decay_rank, width), dtype, device)
        self.w2 = _plain((hd, decay_rank), dtype, device)
        self.w0 = _plain((hd,), dtype, device)
        self.u = _plain((heads, dim), dtype, device)
        self.norm = _plain((hd,), dtype, device)
        self.o = _plain((width, hd), dtype, device)
        # fp32 copy of W_w2 for the decay branch's last product; refreshed IN PLACE after a
        # weight load (captured decode graphs hold its address)
        self.w2_f32 = torch.zeros(hd, decay_rank, dtype=torch.float32, device=device)
        self._w2_ready = False

    def refresh(self) -> None:
        self.w2_f32.copy_(self.w2)
        self._w2_ready = True

    def _load_stream(self, param, loaded, shard_id=None):
        param.data[self.STREAMS.index(shard_id)].copy_(loaded)

    def forward(self, x: torch.Tensor, md: AttentionMetadata, state: RecurrentState) -> torch.Tensor:
        """x: the fp32 residual stream [T, width] (the mixes are formed in fp32)."""
        T = x.shape[0]
        dt = self.o.dtype
        mix = wkv_ops.token_shift_mix(x, self.mu, state.prev, md.seq_slots, md.seq_cu,
                                      md.num_seqs, md.positions, dt)
        rkvg = torch.bmm(mix[:4], self.rkvg.transpose(1, 2))     # [4, T, H*D]
        # decay pre-activation: the low-rank branch ends in an fp32 product (what follows it --
        # bias, both exponentials -- is fp32 inside the scan)
        lo = torch.tanh(gemm.linear(mix[4], self.w1).float())
        if not self._w2_ready:
            self.refresh()
        dec = lo @ self.w2_f32.t()
        y = wkv_ops.wkv_scan(rkvg[0], rkvg[1], rkvg[2], rkvg[3], dec, self.w0, self.u.view(-1),
                             self.norm, state.S, state.prev, x, md.seq_slots, md.seq_cu,
                             md.num_seqs, md.positions,
                             md.decode_seq_lens if md.seq_cu is None else None, self.eps,
                             self.heads)
        return gemm.linear(y, self.o)


class PagedKVRows:
    """Paged cache of one attention layer: token-major key rows [blocks, block, G*P*D] (normed
    when written) and values transposed inside a page, [blocks, G*Dv, block], both in the
    activation dtype."""

    __slots__ = ("k", "v")

    def __init__(self, k: torch.Tensor, v: torch.Tensor):
        self.k, self.v = k, v

    @classmethod
    def allocate(cls, num_blocks: int, block_size: int, k_width: int, v_width: int, dtype, device):
        # zero filled: never-written rows stay finite under a zero softmax weight
        return cls(torch.zeros(num_blocks, block_size, k_width, dtype=dtype, device=device),
                   torch.zeros(num_blocks, v_width, block_size, dtype=dtype, device=device))


def _pad64(n: int) -> int:
    # fused projections are padded with zero rows to a multiple of 64: decode-sized batches then
    # run the weight-streaming GEMM, whose row tiles need it; the pad columns are never read
    return -(-n // 64) * 64


class _WindowMixerBase(nn.Module):
    """Shared parts of the mixers over ``PagedKVRows``: one fused input projection whose named
    slices load separately, per-map RMS norm of queries and keys at cache-write time, the
    attention launch and the output projection."""

    maps = 1

    def _setup(self, width, heads, kv_heads, dim, vdim, scale, window, keep, eps, parts, bias,
               dtype, device, norm_sizes=None, norms=True, own_out=True):
        if pstate.tp_size() != 1:
            raise NotImplementedError("window attention mixers run on one rank (no head sharding yet)")
        if heads % kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        self.width, self.heads, self.kv_heads, self.dim, self.vdim = width, heads, kv_heads, dim, vdim
        self.scale, self.window, self.keep, self.eps = float(scale), int(window), int(keep), float(eps)
        self.offsets, n = {}, 0
        for name, rows in parts:
            if name == "x":                  # another consumer's rows: 16-byte aligned columns
                n = -(-n // 8) * 8
            self.offsets[name] = (n, rows)
            n += rows
        self.proj = _param((_pad64(n), width), dtype, device)
        self.proj.data.zero_()
        self.proj.weight_loader = self._load_part
        self.proj_bias = None
        if bias:
            self.proj_bias = _param((_pad64(n),), dtype, device)
            self.proj_bias.data.zero_()
            self.proj_bias.weight_loader = self._load_part
        # norm weights: one per map entry (shared by the maps), or ``norm_sizes`` = (query, key)
        qn, kn = norm_sizes or (dim, dim)
        self.q_norm = _plain((qn,), dtype, device) if norms else None
        self.k_norm = _plain((kn,), dtype, device) if norms else None
        self.o = _plain((width, heads * vdim), dtype, device) if own_out else None
        M = heads * self.maps
        # fp32 constants of the attention launch, refreshed IN PLACE after a weight load
        # (captured decode graphs hold their addresses)
        self.mult = torch.full((M,), self.scale, dtype=torch.float32, device=device)
        self.spec = win_ops.WindowSpec(heads, kv_heads, self.maps, dim, vdim, self.window,
                                       self.keep, self.mult, eps=self.eps)
        self._qdtype = dtype if torch.device(device).type == "cuda" else torch.float32

    def _load_part(self, param, loaded, shard_id=None):
        off, rows = self.offsets[shard_id]
        if loaded.shape[0] != rows or param.data[off:off + rows].shape != loaded.shape:
            raise ValueError(f"{type(self).__name__} {shard_id}: shape {tuple(loaded.shape)}")
        param.data[off:off + rows].copy_(loaded)

    def query_block(self, block_size: int) -> int:
        """Queries per prefill work item of this layer's attention kernel."""
        return win_ops.query_block(self.spec, self._qdtype, block_size)

    def cache_widths(self):
        """(key row width, value row width) of this layer's PagedKVRows."""
        return self.kv_heads * self.maps * self.dim, self.kv_heads * self.vdim

    def refresh(self) -> None:
        pass

    def _attend(self, xb, md, cache: PagedKVRows, v_part: str, gate_part=None):
        # decode-sized batches: the projection's split-K partials go straight to the cache-write
        # kernel, which sums them (no separate reduce launch, no bf16 round trip)
        fused = gemm.linear(xb, self.proj, self.proj_bias, defer_reduce=True)
        P = self.maps
        g0, gn = self.offsets[gate_part] if gate_part is not None else (0, 0)
        q, gate = win_ops.qk_norm_cache(fused, self.offsets["q"][0], self.offsets["k"][0],
                                        self.offsets[v_part][0], self.heads * P, self.kv_heads * P,
                                        self.dim, self.kv_heads * self.vdim, self.q_norm,
                                        self.k_norm, cache.k, cache.v, md.slot_mapping, self.eps,
                                        g0, gn)
        return win_ops.window_attention(q, cache.k, cache.v, md, self.spec, gate)


class TalkingWindowAttentionMixer(_WindowMixerBase):
    """score_h(i, j) = sum_g talk[h, g] ((q_g . k_j) scale temp_g - slope_g (i - j)) over the
    window 0 <= i - j < window, slope_g = 2^(-slope_bits (g + 1) / H); values are the keys as
    projected (before their norm); the heads are gated by sigmoid(W_g x) before W_o.  q, k and
    the output projection carry biases."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float,
                 window: int, eps: float, dtype, device, slope_bits: float = 8.0):
        super().__init__()
        if vdim != dim:
            raise ValueError("values are the projected keys: vdim must equal dim")
        self._setup(width, heads, kv_heads, dim, vdim, scale, window, 0, eps,
                    [("q", heads * dim), ("k", kv_heads * dim), ("g", heads * vdim)], True,
                    dtype, device)
        self.temp = _plain((heads,), dtype, device)
        self.talk = _plain((heads, heads), dtype, device)
        self.o_bias = _plain((width,), dtype, device)
        h = torch.arange(1, heads + 1, dtype=torch.float64)
        self.spec.slope = torch.pow(2.0, -float(slope_bits) * h / heads).to(torch.float32).to(device)
        self.spec.talk = torch.zeros(heads, heads, dtype=torch.float32, device=device)

    def refresh(self) -> None:
        self.mult.copy_(self.temp.float() * self.scale)
        self.spec.talk.copy_(self.talk.float())

    def forward(self, xb: torch.Tensor, md: AttentionMetadata, cache: PagedKVRows) -> torch.Tensor:
        # may return gemm.SplitK: the output norm step reduces it
        return gemm.linear(self._attend(xb, md, cache, "k", "g"), self.o, self.o_bias,
                           defer_reduce=True)


class DifferentialAttentionMixer(_WindowMixerBase):
    """Each head has two query / key maps (rows laid out head by head as [map 1 | map 2]) that
    attend the same values; lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff is one number for
    the layer; out_h = rms(a1_h - lambda a2_h) (1 - diff).  Position i sees j <= i with
    i - j < window or j < keep."""

    maps = 2

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float,
                 window: int, keep: int, diff: float, eps: float, dtype, device):
        super().__init__()
        self._setup(width, heads, kv_heads, dim, vdim, scale, window, keep, eps,
                    [("q", heads * 2 * dim), ("k", kv_heads * 2 * dim), ("v", kv_heads * vdim)],
                    False, dtype, device)
        self.diff = float(diff)
        self.lq1, self.lk1 = _plain((dim,), dtype, device), _plain((dim,), dtype, device)
        self.lq2, self.lk2 = _plain((dim,), dtype, device), _plain((dim,), dtype, device)
        self.spec.epilogue = 1
        self.spec.post = 1.0 - self.diff
        self.spec.lam = torch.full((1,), self.diff, dtype=torch.float32, device=device)

    def refresh(self) -> None:
        a = torch.exp((self.lq1.float() * self.lk1.float()).sum())
        b = torch.exp((self.lq2.float() * self.lk2.float()).sum())
        self.spec.lam.copy_((a - b + self.diff).reshape(1))

    def forward(self, xb: torch.Tensor, md: AttentionMetadata, cache: PagedKVRows) -> torch.Tensor:
        return gemm.linear(self._attend(xb, md, cache, "v"), self.o, defer_reduce=True)


class SigmoidWindowAttentionMixer(_WindowMixerBase):
    """Grouped-query sliding-window attention with un-normalised weights: a visible key j weighs
    sigmoid((q_h . k_j) scale + pb_h) for head h; out_h = sum_j weight_j v_j.  The query and the
    key projection are each RMS-normed as ONE vector (weights of their full size) before the
    first ``rot_dims`` entries of every head turn by the position (pairs (2i, 2i+1), or
    (i, i + rot_dims/2) with ``rot_half``; ``rot_scaling`` as in ops/rotary.py
    rotary_frequencies).  No biases, no gate.  ``extra_rows``: that many more rows ride in the
    fused input projection (part "x": another consumer of the same layer input);
    ``forward(..., want_extra=True)`` then returns (output, their columns)."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float,
                 window: int, rot_dims: int, rot_base: float, rot_scaling, eps: float, dtype,
                 device, rot_half: bool = False, extra_rows: int = 0):
        super().__init__()
        if rot_dims > dim or rot_dims % 2:
            raise ValueError("rot.dims must be even and at most dim")
        parts = [("q", heads * dim), ("k", kv_heads * dim), ("v", kv_heads * vdim)]
        if extra_rows:
            parts.append(("x", int(extra_rows)))
        self._setup(width, heads, kv_heads, dim, vdim, scale, window, 0, eps, parts, False,
                    dtype, device, norm_sizes=(heads * dim, kv_heads * dim))
        self.rot_dims, self.rot_half = int(rot_dims), rot_half
        self.inv_freq, self.rot_amp = rot_ops.rotary_frequencies(rot_dims, rot_base, rot_scaling,
                                                                 device)
        self.pb = _plain((heads,), dtype, device)
        self.spec.weights = 1
        self.spec.bias = torch.zeros(heads, dtype=torch.float32, device=device)

    def refresh(self) -> None:
        self.spec.bias.copy_(self.pb.float())

    def forward(self, xb: torch.Tensor, md: AttentionMetadata, cache: PagedKVRows,
                want_extra: bool = False):
        fused = gemm.linear(xb, self.proj, None, defer_reduce=True)
        q = win_ops.qk_rope_cache(fused, self.offsets["q"][0], self.offsets["k"][0],
                                  self.offsets["v"][0], self.heads, self.kv_heads, self.dim,
                                  self.kv_heads * self.vdim, self.q_norm, self.k_norm,
                                  self.inv_freq, self.rot_dims, self.rot_half, self.rot_amp,
                                  md.positions, cache.k, cache.v, md.slot_mapping, self.eps)
        a = win_ops.window_attention(q, cache.k, cache.v, md, self.spec, None)
        # may return gemm.SplitK: the layer's boundary step reduces it
        y = gemm.linear(a, self.o, defer_reduce=True)
        if want_extra:
            return y, gemm.columns(fused, *self.offsets["x"])
        return y


class FusedProjection(nn.Module):
    """One input projection shared by several consumers of the same layer input: named parts
    (rows each) stacked into one weight, zero-padded to a multiple of 64 rows, with an optional
    bias over the parts that have one.  ``offsets[name] = (first column, columns)`` of the
    output row."""

    def __init__(self, width: int, parts, dtype, device, bias_parts=()):
        super().__init__()
        self.offsets, n = {}, 0
        for name, rows in parts:
            n = -(-n // 8) * 8                       # 16-byte aligned column ranges
            self.offsets[name] = (n, int(rows))
            n += int(rows)
        self.weight = _param((_pad64(n), width), dtype, device)
        self.weight.data.zero_()
        self.weight.weight_loader = self._load_part
        self.bias = None
        self.bias_parts = tuple(bias_parts)
        if self.bias_parts:
            self.bias = _param((_pad64(n),), dtype, device)
            self.bias.data.zero_()
            self.bias.weight_loader = self._load_part

    def _load_part(self, param, loaded, shard_id=None):
        off, rows = self.offsets[shard_id]
        if loaded.shape[0] != rows or param.data[off:off + rows].shape != loaded.shape:
            raise ValueError(f"fused projection part {shard_id!r}: shape {tuple(loaded.shape)}")
        param.data[off:off + rows].copy_(loaded)

    def init_random(self, gen) -> None:
        """N(0, 1/width) rows for every part, small biases; pad rows stay zero."""
        w = self.weight
        w.data.zero_()
        for name, (off, rows) in self.offsets.items():
            w.data[off:off + rows].copy_(torch.randn((rows, w.shape[1]), generator=gen,
                                                     device=w.device, dtype=torch.float32)
                                         * w.shape[1] ** -0.5)
            if name in self.bias_parts:
                self.bias.data[off:off + rows].copy_(
                    torch.randn((rows,), generator=gen, device=w.device, dtype=torch.float32) * 0.1)

    def forward(self, xb: torch.Tensor, defer_reduce: bool = False):
        return gemm.linear(xb, self.weight, self.bias, defer_reduce=defer_reduce)


class SinkAttentionMixer(_WindowMixerBase):
    """Grouped-query causal softmax attention: q, k and v carry biases; the first ``rot_dims``
    entries of every query / key head turn by the position (pairs (2i, 2i+1), or (i, i +
    rot_dims/2) with ``rot_half``; ``rot_scaling`` as in ops/rotary.py rotary_frequencies, a
    lone ``factor`` divides every frequency); score = (q . k) * scale; the softmax denominator
    of head h also holds exp(sink_h), a learned term without key or value; ``window`` 0 sees
    every earlier token.  The concatenated heads are multiplied by ``out_scale``.
    ``proj`` / ``prefix``: the q, k, v parts live in a caller's FusedProjection under
    ``prefix + "q"`` ...; the caller then also owns the output projection, and ``attend`` writes
    the heads into the caller's buffer."""

    PARTS = ("q", "k", "v")

    @staticmethod
    def parts(heads, kv_heads, dim, vdim):
        return [("q", heads * dim), ("k", kv_heads * dim), ("v", kv_heads * vdim)]

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float,
                 rot_dims: int, rot_base: float, rot_scaling, eps: float, dtype, device,
                 window: int = 0, rot_half: bool = False, out_scale: float = 1.0,
                 proj: "FusedProjection" = None, prefix: str = ""):
        super().__init__()
        if rot_dims > dim or rot_dims % 2:
            raise ValueError("rot.dims must be even and at most dim")
        own = proj is None
        self._setup(width, heads, kv_heads, dim, vdim, scale, window, 0, eps,
                    self.parts(heads, kv_heads, dim, vdim) if own else [], own, dtype, device,
                    norms=False, own_out=own)
        if not own:
            self.proj = self.proj_bias = None
            self.offsets = {n: proj.offsets[prefix + n] for n in self.PARTS}
        self.rot_dims, self.rot_half = int(rot_dims), rot_half
        self.inv_freq, self.rot_amp = rot_ops.rotary_frequencies(rot_dims, rot_base, rot_scaling,
                                                                 device)
        self.sink = _plain((heads,), dtype, device)
        self.spec.sink = torch.zeros(heads, dtype=torch.float32, device=device)
        self.spec.post = float(out_scale)

    def refresh(self) -> None:
        self.spec.sink.copy_(self.sink.float())

    def attend(self, fused, md: AttentionMetadata, cache: PagedKVRows, out=None):
        q = win_ops.qk_rope_cache(fused, self.offsets["q"][0], self.offsets["k"][0],
                                  self.offsets["v"][0], self.heads, self.kv_heads, self.dim,
                                  self.kv_heads * self.vdim, None, None, self.inv_freq,
                                  self.rot_dims, self.rot_half, self.rot_amp, md.positions,
                                  cache.k, cache.v, md.slot_mapping, self.eps)
        return win_ops.window_attention(q, cache.k, cache.v, md, self.spec, None, out=out)

    def forward(self, xb: torch.Tensor, md: AttentionMetadata, cache: PagedKVRows):
        fused = gemm.linear(xb, self.proj, self.proj_bias, defer_reduce=True)
        # may return gemm.SplitK: the layer's boundary step reduces it
        return gemm.linear(self.attend(fused, md, cache), self.o, defer_reduce=True)


class _ScanMixerBase(nn.Module):
    """Shared parts of the mixers over ``ScanState`` slots: the fused input projection (their own
    or a caller's), the scan launch and the output projection."""

    def _setup(self, width, parts, bias_parts, dtype, device, proj, prefix):
        if pstate.tp_size() != 1:
            raise NotImplementedError("recurrent mixers run on one rank (no head sharding yet)")
        self.width = width
        self.own = proj is None
        if self.own:
            self.proj = FusedProjection(width, parts, dtype, device, bias_parts)
            self.offsets = dict(self.proj.offsets)
            self.o = _plain((width, self.spec.heads * self.spec.vdim), dtype, device)
        else:
            self.proj = self.o = None
            self.offsets = {n: proj.offsets[prefix + n] for n, _ in parts}

    def state_bytes(self) -> int:
        return scan_ops.ScanState.slot_bytes(self.spec)

    def allocate_state(self, num_slots: int, device) -> scan_ops.ScanState:
        return scan_ops.ScanState.allocate(num_slots, self.spec, device)

    def refresh(self) -> None:
        pass

    def _scan(self, fused, md, state, norm_w, out):
        from ..ops.gemm import SplitK
        if isinstance(fused, SplitK):
            fused = fused.materialize() if fused.part.is_cuda else \
                fused.part.sum(0) + (fused.bias.float() if fused.bias is not None else 0.0)
        o = self.offsets
        # prompt portions: the step's chunk list, built once per step and shared by its layers
        plan = None
        if fused.is_cuda and md.seq_cu is not None:
            if "scan_chunks" not in md.work_cache:
                lens = [1] * md.num_decode + list(md.prefill_q_lens or [])
                md.work_cache["scan_chunks"] = scan_ops.chunk_plan(
                    lens if len(lens) == md.num_seqs else None, fused.device)
            plan = md.work_cache["scan_chunks"]
        return scan_ops.linear_scan(
            fused, o["q"][0], o["k"][0], o["v"][0], o["g"][0], self.spec, state, md.seq_slots,
            md.seq_cu, md.num_seqs, md.positions,
            md.decode_seq_lens if md.seq_cu is None else None, norm_w,
            o["i"][0] if "i" in o else 0, o["f"][0] if "f" in o else 0, out, plan)

    def forward(self, xb: torch.Tensor, md: AttentionMetadata, state):
        # may return gemm.SplitK: the layer's boundary step reduces it
        return gemm.linear(self.attend(self.proj(xb), md, state), self.o, defer_reduce=True)


class RetentionMixer(_ScanMixerBase):
    """Linear attention with a fixed decay per head and neither softmax nor denominator:
    q, k [heads, dim] and v [heads, vdim] without biases; the first ``rot_dims`` entries of q and
    k turn by the position (pairs (i, i + rot_dims/2), or (2i, 2i+1) with ``rot_half`` False); k
    is then multiplied by dim^(-1/2);  S_t = decay_h S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t;
    every head's o is divided by its root mean square; the concatenated heads are multiplied by
    silu(W_g x) and ``out_scale``."""

    @staticmethod
    def parts(heads, dim, vdim):
        return [("q", heads * dim), ("k", heads * dim), ("v", heads * vdim), ("g", heads * vdim)]

    def __init__(self, width: int, heads: int, dim: int, vdim: int, decay, rot_dims: int,
                 rot_base: float, rot_scaling, eps: float, dtype, device, rot_half: bool = True,
                 out_scale: float = 1.0, proj: "FusedProjection" = None, prefix: str = ""):
        super().__init__()
        if len(decay) != heads:
            raise ValueError("retention: one decay per head")
        if rot_dims > dim or rot_dims % 2:
            raise ValueError("rot.dims must be even and at most dim")
        inv_freq, _ = rot_ops.rotary_frequencies(rot_dims, rot_base, rot_scaling, device)
        self.spec = scan_ops.ScanSpec(
            heads, dim, vdim, "decay",
            decay=torch.tensor([float(d) for d in decay], dtype=torch.float32, device=device),
            inv_freq=inv_freq, rot_dims=int(rot_dims), rot_half=rot_half, qscale=1.0,
            kscale=float(dim) ** -0.5, gate_act="silu", out_scale=float(out_scale), eps=float(eps))
        self._setup(width, self.parts(heads, dim, vdim), (), dtype, device, proj, prefix)

    def attend(self, fused, md: AttentionMetadata, state, out=None):
        return self._scan(fused, md, state, None, out)


class MatrixMemoryMixer(_ScanMixerBase):
    """Gated matrix memory: q = W_q x * dim^(-1/2), k [heads, dim], v [heads, vdim]; per head a
    log input gate i = cap tanh((W_i x + b_i) / cap) and a log forget gate f = logsigmoid(cap
    tanh((W_f x + b_f) / cap)) (``gate_cap`` 0: no cap); with a running maximum m_t = max(f + m_(t-1), i) (from 0):
    S_t = exp(f + m_(t-1) - m_t) S_(t-1) + exp(i - m_t) k v^T, n_t likewise with k alone,
    o = S_t^T q / (max(|n_t . q|, exp(-m_t)) + 1e-6).  Every head's o is divided by its root mean
    square; the concatenated heads are multiplied by the weight ``norm``, sigmoid(W_g x) and
    ``out_scale``."""

    @staticmethod
    def parts(heads, dim, vdim):
        return [("q", heads * dim), ("k", heads * dim), ("v", heads * vdim), ("g", heads * vdim),
                ("i", heads), ("f", heads)]

    BIAS_PARTS = ("i", "f")

    def __init__(self, width: int, heads: int, dim: int, vdim: int, gate_cap: float, eps: float,
                 dtype, device, out_scale: float = 1.0, proj: "FusedProjection" = None,
                 prefix: str = ""):
        super().__init__()
        self.spec = scan_ops.ScanSpec(heads, dim, vdim, "exp_gates", cap=float(gate_cap),
                                      qscale=float(dim) ** -0.5, kscale=1.0, gate_act="sigmoid",
                                      out_scale=float(out_scale), eps=float(eps))
        self._setup(width, self.parts(heads, dim, vdim), self.BIAS_PARTS, dtype, device, proj,
                    prefix)
        self.norm = _plain((heads * vdim,), dtype, device)

    def attend(self, fused, md: AttentionMetadata, state, out=None):
        return self._scan(fused, md, state, self.norm, out)


class ParallelMixer(nn.Module):
    """Two mixers side by side on the same input, ``left_scale * left(x) + right_scale *
    right(x)``: ``left`` a SinkAttentionMixer on paged K / V rows, ``right`` a MatrixMemoryMixer on
    state slots.  Both read ONE fused input projection and write their (scaled) heads into one
    row, so one output projection over the concatenated heads adds the two in fp32."""

    def __init__(self, width: int, left: dict, right: dict, left_scale: float, right_scale: float,
                 eps: float, dtype, device):
        super().__init__()
        lp = SinkAttentionMixer.parts(left["heads"], left["kv_heads"], left["dim"], left["vdim"])
        rp = MatrixMemoryMixer.parts(right["heads"], right["dim"], right["vdim"])
        self.proj = FusedProjection(
            width, [("left." + n, r) for n, r in lp] + [("right." + n, r) for n, r in rp], dtype,
            device, tuple("left." + n for n, _ in lp) +
            tuple("right." + n for n in MatrixMemoryMixer.BIAS_PARTS))
        rot = left.get("rot") or {}
        self.left = SinkAttentionMixer(
            width, left["heads"], left["kv_heads"], left["dim"], left["vdim"], left["scale"],
            int(rot.get("dims", left["dim"] if rot else 0)), float(rot.get("base", 10000.0)),
            rot.get("scaling"), eps,
            dtype, device, window=int((left.get("mask") or {}).get("size", 0)),
            out_scale=left_scale, proj=self.proj, prefix="left.")
        self.right = MatrixMemoryMixer(width, right["heads"], right["dim"], right["vdim"],
                                       right["gate_cap"], eps, dtype, device,
                                       out_scale=right_scale, proj=self.proj, prefix="right.")
        self.lw = left["heads"] * left["vdim"]
        self.rw = right["heads"] * right["vdim"]
        self.lw_pad = -(-self.lw // 8) * 8           # the right heads start 16-byte aligned
        self.row = -(-(self.lw_pad + self.rw) // 8) * 8     # ... and so does every row
        # output projection over [left heads | pad | right heads | pad]; the checkpoint's two
        # output matrices load into its column ranges (pad columns stay zero)
        self.o = _param((width, self.row), dtype, device)
        self.o.data.zero_()
        self.o.weight_loader = self._load_o

    def _load_o(self, param, loaded, shard_id=None):
        off, n = (0, self.lw) if shard_id == "left" else (self.lw_pad, self.rw)
        if loaded.shape != (param.shape[0], n):
            raise ValueError(f"parallel mixer {shard_id}.o: shape {tuple(loaded.shape)}")
        param.data[:, off:off + n].copy_(loaded)

    def refresh(self) -> None:
        self.left.refresh()
        self.right.refresh()

    def forward(self, xb: torch.Tensor, md: AttentionMetadata, cache):
        """cache: (PagedKVRows of the left mixer, ScanState of the right one)."""
        kv, state = cache
        fused = self.proj(xb)
        T = xb.shape[0]
        heads = torch.empty(T, self.row, dtype=xb.dtype, device=xb.device)
        if self.lw_pad != self.lw:
            heads[:, self.lw:self.lw_pad].zero_()
        if self.row != self.lw_pad + self.rw:
            heads[:, self.lw_pad + self.rw:].zero_()
        self.left.attend(fused, md, kv, out=heads[:, :self.lw])
        self.right.attend(fused, md, state, out=heads[:, self.lw_pad:self.lw_pad + self.rw])
        # may return gemm.SplitK: the layer's boundary step reduces it
        return gemm.linear(heads, self.o, defer_reduce=True)
