"""Windowed multi-map attention ops -> csrc/kernels/window_attention.hip.

The paged cache of a layer holds token-major key rows ``[blocks, block, G*P*D]`` (RMS-normed
at write time) and values transposed inside a page, ``[blocks, G*Dv, block]`` (eight consecutive
keys of a value column are one 16-byte load).  A query row carries
``M = H*P`` score maps (P = 1: ordinary heads; P = 2: the two maps of a differential head);
map ``h*P + c`` reads key map ``(h // (H//G))*P + c`` and value head ``h // (H//G)``.  Per map
the score of (query position i, key j) is ``(q.k) * mult[m] - slope[m]*(i-j)``, optionally mixed
across maps by a matrix (``talk``), masked to ``j <= i and (i-j < window or j < keep)`` and
soft-maxed -- or, with ``spec.weights`` 1, every visible key simply weighs
``sigmoid(score + bias[m])`` and nothing is normalised over the keys.  With ``spec.sink`` the
softmax denominator of map m also holds ``exp(sink[m])``, a term without key or value.
``spec.epilogue`` 0 multiplies the heads by ``sigmoid(gate)`` and by ``spec.post``; 1 combines
a head's two maps as ``a1 - lam*a2``, divides by the root mean square over the head and scales.

A step's rows are [decode rows (1 per sequence) | prefill chunks]; both parts read the cache
after ``qk_norm_cache`` wrote this step's rows, so chunked prompts need no special path.
"""

from __future__ import annotations

import dataclasses
import os
from typing import List, Optional

import torch

from ._dispatch import check, lib, ptr, require, stream, use_hip

SCALAR_QB = 4            # queries per prefill work item of the scalar-FMA kernel
MFMA_QB = 16             # ... and of the MFMA kernel (one 16-row tile)
_MFMA_ENV = os.environ.get("EIA_WINDOW_MFMA", "1") != "0"


@dataclasses.dataclass
class WindowSpec:
    """Constants of one attention layer (device tensors are fp32)."""
    heads: int
    kv_heads: int
    maps: int                       # P: score maps per head
    dim: int
    vdim: int
    window: int                     # 0: no window (every earlier key)
    keep: int                       # first tokens that stay visible
    mult: torch.Tensor              # [H*P]
    slope: Optional[torch.Tensor] = None    # [H*P]
    talk: Optional[torch.Tensor] = None     # [H*P, H*P]
    epilogue: int = 0
    lam: Optional[torch.Tensor] = None      # [1], the differential weight (epilogue 1)
    eps: float = 0.0
    post: float = 1.0
    weights: int = 0                # 0: softmax over the visible keys; 1: sigmoid(score + bias)
    bias: Optional[torch.Tensor] = None     # [H*P], added to the score inside the sigmoid
    sink: Optional[torch.Tensor] = None     # [H*P], exp(sink) joins the softmax denominator


def build_work(q_lens: List[int], qblock: int) -> List[int]:
    """[seq, first query] pairs; a windowed row's work does not grow with its position, so the
    order is the batch's own."""
    out: List[int] = []
    for s, n in enumerate(q_lens):
        for q0 in range(0, n, qblock):
            out += [s, q0]
    return out


def mfma_ok(spec: WindowSpec, dtype: torch.dtype, block_size: int) -> bool:
    """The MFMA kernel takes bf16 rows with D % 8 == 0, Dv % 16 == 0, both <= 128, pages of a
    multiple of 32 tokens and, with head mixing, at most 16 heads (one workgroup of up to eight
    waves holds them all, one or two heads per wave); everything else (fp32 models too) runs
    the scalar-FMA kernel."""
    if dtype != torch.bfloat16 or not _MFMA_ENV or not torch.cuda.is_available():
        return False
    return bool(lib().eia_window_attn_mfma_ok(spec.heads, spec.kv_heads, spec.maps, spec.dim,
                                              spec.vdim,
                                              block_size, 1 if spec.talk is not None else 0))


def decode_partitions(batch: int, spec: WindowSpec, cus: int = 256) -> int:
    """Key partitions (grid.z) of a decode launch of the MFMA form: a decode row is one
    workgroup (per four heads without head mixing), so small batches split every row's 32-key
    blocks until about two workgroups per CU exist (a power of two, at most 16, and at least
    two blocks of a full window per partition); a second kernel merges the partials.  A row
    with fewer blocks uses fewer partitions (decided in the kernel).  Depends on the
    batch and the layer's constants only, so a captured decode graph keeps its grid."""
    forced = int(os.environ.get("EIA_WINDOW_DECODE_P", "0"))
    if forced > 0:
        return min(forced, 64)
    # (sigmoid weights: a wave takes two heads where they share a kv head)
    per_wave = 2 if (spec.weights == 1 and (spec.heads // spec.kv_heads) % 2 == 0) else 1
    wgs = max(1, batch) * (1 if spec.talk is not None else -(-(spec.heads // per_wave) // 4))
    limit = 16
    if spec.window > 0:
        limit = max(1, min(16, ((spec.window + 31) // 32 + 1 + (spec.keep + 31) // 32) // 2))
    p = 1
    while p * 2 <= limit and wgs * p * 2 <= 2 * cus:
        p *= 2
    return p


def query_block(spec: WindowSpec, dtype: torch.dtype, block_size: int) -> int:
    return MFMA_QB if mfma_ok(spec, dtype, block_size) else SCALAR_QB


def _rms(v: torch.Tensor, eps: float) -> torch.Tensor:
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def qk_norm_cache(fused, q_off: int, k_off: int, v_off: int, mq: int, mk: int,
                  dim: int, v_width: int, q_w: torch.Tensor, k_w: torch.Tensor,
                  k_cache: torch.Tensor, v_cache: torch.Tensor, slot_mapping: torch.Tensor,
                  eps: float, gate_off: int = 0, gate_width: int = 0):
    """One pass over fused projection rows [T, *]: the ``mq`` query maps at ``q_off`` are
    RMS-normed (weight ``q_w`` [dim]) and returned [T, mq*dim]; the ``mk`` key maps at ``k_off``
    are RMS-normed (``k_w``) into the token's key row and the ``v_width`` value columns at
    ``v_off`` (which may be the un-normed key columns) are copied into its value columns.  Rows
    with a slot < 0 write no cache.  Returns (q, gate): gate is the ``gate_width`` columns at
    ``gate_off`` (None when the width is 0).  ``fused`` may be a ``gemm.SplitK``: the projection's
    fp32 partial sums (+ bias) are then reduced here and the gate columns written out."""
    from .gemm import SplitK
    split = isinstance(fused, SplitK)
    if split and not fused.part.is_cuda:            # CPU path: the plain fp32 sum
        fused = fused.part.sum(0) + (fused.bias.float() if fused.bias is not None else 0.0)
        split = False
    elif split and fused.N % 4:                     # the kernel sums partials in 16-byte units
        fused = (fused.part.sum(0) + (fused.bias.float() if fused.bias is not None else 0.0)
                 ).to(k_cache.dtype)
        split = False
    if not split:
        T = fused.shape[0]
        gate = fused[:, gate_off:gate_off + gate_width] if gate_width else None
    if not split and not use_hip(fused):
        f = fused.float()
        q = _rms(f[:, q_off:q_off + mq * dim].reshape(T, mq, dim), eps) * q_w.float()
        k = _rms(f[:, k_off:k_off + mk * dim].reshape(T, mk, dim), eps) * k_w.float()
        sm = slot_mapping[:T].long()
        ok = sm >= 0
        k_cache.view(-1, k_cache.shape[-1])[sm[ok]] = k.reshape(T, -1)[ok].to(k_cache.dtype)
        bs = v_cache.shape[2]
        v_cache[sm[ok] // bs, :, sm[ok] % bs] = fused[:, v_off:v_off + v_width][ok].to(v_cache.dtype)
        return q.reshape(T, mq * dim).to(fused.dtype), gate
    dt = k_cache.dtype
    bf = dt == torch.bfloat16
    require(bf or dt == torch.float32, "qk_norm_cache: bf16 or fp32")
    if split:
        T, width = fused.M, fused.N
        require(fused.part.dtype == torch.float32 and fused.part.is_contiguous() and
                (fused.bias is None or fused.bias.dtype == dt), "qk_norm_cache: partials")
    else:
        width = fused.shape[1]
        require(fused.stride(1) == 1 and fused.dtype == dt, "qk_norm_cache: fused row layout")
    require(max(q_off + mq * dim, k_off + mk * dim, v_off + v_width, gate_off + gate_width)
            <= width, "qk_norm_cache: columns outside the row")
    require(v_cache.dtype == dt and k_cache.is_contiguous() and v_cache.is_contiguous() and
            k_cache.shape[-1] == mk * dim and v_cache.shape[1] == v_width and
            v_cache.shape[2] == k_cache.shape[1], "qk_norm_cache: cache layout")
    require(q_w.dtype == dt and k_w.dtype == dt and q_w.numel() == dim and k_w.numel() == dim,
            "qk_norm_cache: norm weights")
    require(slot_mapping.dtype == torch.int32 and slot_mapping.numel() >= T, "int32 slots")
    q = torch.empty(T, mq * dim, dtype=dt, device=k_cache.device)
    if split:
        gate = torch.empty(T, gate_width, dtype=dt, device=q.device) if gate_width else None
        check(lib().eia_qk_norm_cache(
            None, width, ptr(fused.part), fused.sk, ptr(fused.bias), q_off, k_off, v_off, gate_off,
            mq, mk, dim, v_width, gate_width, ptr(q_w), ptr(k_w), ptr(q), q.stride(0),
            ptr(k_cache), ptr(v_cache), ptr(gate), gate_width, ptr(slot_mapping),
            k_cache.shape[1], float(eps), T, 1 if bf else 0, stream(q)), "qk_norm_cache")
        return q, gate
    check(lib().eia_qk_norm_cache(
        ptr(fused), fused.stride(0), None, 0, None, q_off, k_off, v_off, 0, mq, mk, dim, v_width,
        0, ptr(q_w), ptr(k_w), ptr(q), q.stride(0), ptr(k_cache), ptr(v_cache), None, 0,
        ptr(slot_mapping), k_cache.shape[1], float(eps), T, 1 if bf else 0, stream(q)),
        "qk_norm_cache")
    return q, gate


def qk_rope_cache(fused, q_off: int, k_off: int, v_off: int, mq: int, mk: int, dim: int,
                  v_width: int, q_w: torch.Tensor, k_w: torch.Tensor, inv_freq: torch.Tensor,
                  rot_dims: int, rot_half: bool, rot_amp: float, positions: torch.Tensor,
                  k_cache: torch.Tensor, v_cache: torch.Tensor, slot_mapping: torch.Tensor,
                  eps: float) -> torch.Tensor:
    """One pass over fused projection rows [T, *] for heads that are normed as ONE vector and
    then rotated: the ``mq * dim`` query columns at ``q_off`` are divided by their common root
    mean square and multiplied by ``q_w`` [mq*dim] (``q_w`` None: no norm), then the first
    ``rot_dims`` entries of every head turn by the token's position (pairs (2i, 2i+1), or
    (i, i + rot_dims/2) with ``rot_half``; angle position * inv_freq[i]; cos and sin times
    ``rot_amp``) and the row is returned [T, mq*dim]; the ``mk * dim`` key columns at ``k_off``
    get the same with ``k_w`` and land in the token's key row, the ``v_width`` value columns at
    ``v_off`` in its value columns.  Rows with a slot < 0 write no cache.  ``fused`` may be a
    ``gemm.SplitK`` (fp32 partial sums of the projection, summed here)."""
    from .gemm import SplitK
    from .latent_attention import _rotate_pairs
    split = isinstance(fused, SplitK)
    if split and (not fused.part.is_cuda or fused.N % 4):
        fused = fused.part.sum(0) + (fused.bias.float() if fused.bias is not None else 0.0)
        fused = fused if not fused.is_cuda else fused.to(k_cache.dtype)
        split = False
    if not split and not use_hip(fused):
        T = fused.shape[0]
        f = fused.float()

        def side(off, m, w):
            x = f[:, off:off + m * dim]
            if w is not None:
                x = _rms(x, eps) * w.float()
            x = _rotate_pairs(x.reshape(T, m, dim), positions[:T, None], inv_freq, rot_dims,
                              rot_half, rot_amp)
            return x.reshape(T, m * dim)

        q, k = side(q_off, mq, q_w), side(k_off, mk, k_w)
        sm = slot_mapping[:T].long()
        ok = sm >= 0
        k_cache.view(-1, k_cache.shape[-1])[sm[ok]] = k[ok].to(k_cache.dtype)
        bs = v_cache.shape[2]
        v_cache[sm[ok] // bs, :, sm[ok] % bs] = f[:, v_off:v_off + v_width][ok].to(v_cache.dtype)
        return q.to(k_cache.dtype)
    dt = k_cache.dtype
    bf = dt == torch.bfloat16
    require(bf or dt == torch.float32, "qk_rope_cache: bf16 or fp32")
    if split:
        T, width = fused.M, fused.N
        require(fused.part.dtype == torch.float32 and fused.part.is_contiguous() and
                (fused.bias is None or fused.bias.dtype == dt), "qk_rope_cache: partials")
    else:
        T, width = fused.shape
        require(fused.stride(1) == 1 and fused.dtype == dt, "qk_rope_cache: fused row layout")
    require(max(q_off + mq * dim, k_off + mk * dim, v_off + v_width) <= width,
            "qk_rope_cache: columns outside the row")
    require(v_cache.dtype == dt and k_cache.is_contiguous() and v_cache.is_contiguous() and
            k_cache.shape[-1] == mk * dim and v_cache.shape[1] == v_width and
            v_cache.shape[2] == k_cache.shape[1], "qk_rope_cache: cache layout")
    require((q_w is None or (q_w.dtype == dt and q_w.numel() == mq * dim)) and
            (k_w is None or (k_w.dtype == dt and k_w.numel() == mk * dim)),
            "qk_rope_cache: norm weights")
    require(0 <= rot_dims <= dim and rot_dims % 2 == 0 and inv_freq.dtype == torch.float32 and
            inv_freq.numel() >= rot_dims // 2, "qk_rope_cache: rotation")
    require(slot_mapping.dtype == torch.int32 and slot_mapping.numel() >= T and
            positions.dtype == torch.int32 and positions.numel() >= T, "int32 slots and positions")
    q = torch.empty(T, mq * dim, dtype=dt, device=k_cache.device)
    check(lib().eia_qk_rope_cache(
        None if split else ptr(fused), width if split else fused.stride(0),
        ptr(fused.part) if split else None, fused.sk if split else 0,
        ptr(fused.bias) if split else None, q_off, k_off, v_off, mq, mk, dim, v_width, ptr(q_w),
        ptr(k_w), ptr(inv_freq), rot_dims, 1 if rot_half else 0, float(rot_amp), ptr(positions),
        ptr(q), q.stride(0), ptr(k_cache), ptr(v_cache), ptr(slot_mapping), k_cache.shape[1],
        float(eps), T, 1 if bf else 0, stream(q)), "qk_rope_cache")
    return q


def _ref_rows(q, k_cache, v_cache, block_table, positions, gate, spec: WindowSpec, seq_of_row):
    """Plain per-row attention over the paged rows (CPU path)."""
    H, G, P, D, Dv = spec.heads, spec.kv_heads, spec.maps, spec.dim, spec.vdim
    rep = H // G
    bs = k_cache.shape[1]
    kf = k_cache.view(-1, G, P, D).float()
    vf = v_cache.permute(0, 2, 1).reshape(-1, G, Dv).float()
    out = torch.zeros(q.shape[0], H * Dv, dtype=torch.float32)
    for row, s in enumerate(seq_of_row):
        i = int(positions[row])
        lo = max(0, i - spec.window + 1) if spec.window > 0 else 0
        js = torch.tensor(list(range(min(spec.keep, lo))) + list(range(lo, i + 1)))
        slots = block_table[s].long()[js // bs] * bs + js % bs
        keys = kf[slots].repeat_interleave(rep, 1).reshape(len(js), H * P, D)      # [n, M, D]
        vals = vf[slots].repeat_interleave(rep, 1)                                 # [n, H, Dv]
        sc = torch.einsum("md,nmd->mn", q[row].float().view(H * P, D), keys) * spec.mult[:, None]
        if spec.slope is not None:
            sc = sc - spec.slope[:, None] * (i - js).float()[None, :]
        if spec.talk is not None:
            sc = spec.talk @ sc
        if spec.weights == 1:
            w = torch.sigmoid(sc + (spec.bias[:, None] if spec.bias is not None else 0.0))
        elif spec.sink is not None:
            w = torch.softmax(torch.cat([sc, spec.sink[:, None]], -1), -1)[:, :-1]
        else:
            w = torch.softmax(sc, -1)
        w = w.view(H, P, len(js))
        a = torch.einsum("hpn,nhd->hpd", w, vals)
        if spec.epilogue == 0:
            o = a[:, 0].reshape(H * Dv) * spec.post
            if gate is not None:
                o = o * torch.sigmoid(gate[row].float())
        else:
            o = a[:, 0] - float(spec.lam[0]) * a[:, 1]
            o = (_rms(o, spec.eps) * spec.post).reshape(H * Dv)
        out[row] = o
    return out


def window_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, md,
                     spec: WindowSpec, gate: Optional[torch.Tensor] = None,
                     out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q [T, H*P*D] (normed; contiguous last dim), gate [T, H*Dv] before the sigmoid or None ->
    [T, H*Dv] in q's dtype.  ``md`` is the step's AttentionMetadata.  ``out``: a [T, H*Dv] view
    (contiguous last dim; the columns of a wider row that another mixer shares) to write into."""
    T = q.shape[0]
    H, P, D, Dv = spec.heads, spec.maps, spec.dim, spec.vdim
    nd = md.num_decode
    if out is None:
        out = torch.empty(T, H * Dv, dtype=q.dtype, device=q.device)
    require(out.shape == (T, H * Dv) and out.dtype == q.dtype and out.stride(1) == 1,
            "window_attention: out layout")
    if not use_hip(q, k_cache):
        if nd:
            out[:nd] = _ref_rows(q[:nd], k_cache, v_cache, md.decode_block_tables,
                                 md.positions[:nd], None if gate is None else gate[:nd], spec,
                                 list(range(nd))).to(out.dtype)
        if md.num_prefill_tokens:
            cu = md.prefill_cu_q.tolist()
            seqs = [s for s in range(len(cu) - 1) for _ in range(cu[s + 1] - cu[s])]
            out[nd:] = _ref_rows(q[nd:], k_cache, v_cache, md.prefill_block_tables,
                                 md.positions[nd:], None if gate is None else gate[nd:], spec,
                                 seqs).to(out.dtype)
        return out
    bf = q.dtype == torch.bfloat16
    require(bf or q.dtype == torch.float32, "window_attention: bf16 or fp32")
    require(q.stride(1) == 1 and q.shape[1] == H * P * D and k_cache.dtype == q.dtype and
            v_cache.dtype == q.dtype and k_cache.is_contiguous() and v_cache.is_contiguous() and
            k_cache.shape[-1] == spec.kv_heads * P * D and v_cache.shape[1] == spec.kv_heads * Dv
            and v_cache.shape[2] == k_cache.shape[1],
            "window_attention: layout")
    require(gate is None or (gate.dtype == q.dtype and gate.stride(1) == 1 and
                             gate.shape[1] >= H * Dv), "window_attention: gate layout")
    require(md.positions.dtype == torch.int32, "positions int32")
    require(spec.weights in (0, 1) and (spec.weights == 0 or (spec.talk is None and P == 1)),
            "window_attention: sigmoid weights come without head mixing or map pairs")
    require(spec.sink is None or spec.weights == 0, "window_attention: a sink needs softmax weights")
    for t in (spec.mult, spec.slope, spec.talk, spec.lam, spec.bias, spec.sink):
        require(t is None or (t.dtype == torch.float32 and t.is_cuda and t.is_contiguous()),
                "window_attention: fp32 device constants")
    bs = k_cache.shape[1]

    mfma = mfma_ok(spec, q.dtype, bs)
    if mfma:
        require(q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0, "window_attention: q alignment")

    def launch(lo, n_items, bt, lens, cu, work, qb):
        require(bt.dtype == torch.int32 and bt.stride(1) == 1, "block tables int32")
        qa, o = q[lo:], out[lo:]
        g = None if gate is None else gate[lo:]
        if mfma:
            NP = decode_partitions(n_items, spec) if cu is None else 1
            pa = pm = None
            if NP > 1:
                pa = torch.empty(n_items * H * P * NP * Dv, dtype=torch.float32, device=q.device)
                pm = torch.empty(n_items * H * P * NP * 2, dtype=torch.float32, device=q.device)
            check(lib().eia_window_attn_mfma(
                ptr(qa), qa.stride(0), ptr(k_cache), ptr(v_cache), ptr(bt), bt.stride(0),
                ptr(md.positions[lo:]), ptr(cu), ptr(work), ptr(lens), n_items, ptr(spec.mult),
                ptr(spec.slope), ptr(spec.talk), ptr(g), g.stride(0) if g is not None else 0,
                ptr(o), o.stride(0), H, spec.kv_heads, P, D, Dv, bs, spec.window, spec.keep,
                spec.epilogue, ptr(spec.lam), float(spec.eps), float(spec.post), spec.weights,
                ptr(spec.bias), NP, ptr(pa), ptr(pm), ptr(spec.sink), stream(q)), "window_attn_mfma")
            return
        check(lib().eia_window_attn(
            ptr(qa), qa.stride(0), ptr(k_cache), ptr(v_cache), ptr(bt), bt.stride(0),
            ptr(md.positions[lo:]), ptr(cu), ptr(work), ptr(lens), n_items, ptr(spec.mult),
            ptr(spec.slope), ptr(spec.talk), ptr(g), g.stride(0) if g is not None else 0, ptr(o),
            o.stride(0), H, spec.kv_heads, P, D, Dv, bs, spec.window, spec.keep, qb,
            spec.epilogue, ptr(spec.lam), float(spec.eps), float(spec.post), spec.weights,
            ptr(spec.bias), ptr(spec.sink), 1 if bf else 0, stream(q)), "window_attn")

    if nd:
        launch(0, nd, md.decode_block_tables, md.decode_seq_lens, None, None, 1)
    if md.num_prefill_tokens:
        qb = query_block(spec, q.dtype, bs)
        work, n_work = md.prefill_work_for(qb, build_work)
        launch(nd, n_work, md.prefill_block_tables, None, md.prefill_cu_q, work, qb)
    return out
