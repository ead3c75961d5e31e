"""Latent (low-rank KV) attention ops -> csrc/kernels/latent_attention.hip.

The paged cache holds one row per token, ``[c | k_rot]``: the RMS-normed KV latent ``c``
(``kv_rank`` wide) and the rotated key part shared by all heads (``rot_dim`` wide).  Attention
runs in the absorbed form: the caller folds the key up-projection into the query
(``q_abs[h] = W_uk[h]^T q_nope[h]``) and applies the value up-projection to the kernel's latent
output, so every head reads the same cache rows and K / V are never materialised.

A step's rows are laid out [decode rows (1 per sequence) | prefill chunks]; both parts read the
cache after ``latent_prep`` wrote this step's rows, so chunked prompts need no special path.
"""

from __future__ import annotations

import os
from typing import List, Optional

import torch

from ._dispatch import check, lib, ptr, require, stream, use_hip

ACC_ROWS = 256 * 32        # csrc/kernels/latent_attention.hip: QB * HB * R <= 256 * LAT_ACC_MAX


def inv_frequencies(dims: int, base: float, device) -> torch.Tensor:
    """f_i = base^(-2i/dims), i < dims/2, evaluated in float64 and rounded once to fp32."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    return torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims).to(
        torch.float32).to(device)


def mfma_ok(kv_rank: int, rot_dim: int, dtype: torch.dtype) -> bool:
    """The MFMA kernel takes bf16 rows whose latent and total widths are multiples of 8 (its
    16-byte chunks) up to 512 / 640; everything else runs the scalar-FMA kernel (fp32 too)."""
    return (dtype == torch.bfloat16 and kv_rank % 8 == 0 and (kv_rank + rot_dim) % 8 == 0
            and kv_rank <= 512 and kv_rank + rot_dim <= 640 and _MFMA_ENV)


_MFMA_ENV = os.environ.get("EIA_LATENT_MFMA", "1") != "0"


def query_block(num_heads: int, kv_rank: int, rot_dim: int = 0,
                dtype: torch.dtype = torch.float32) -> int:
    """Queries per prefill work item.  MFMA form: 64 (query, head) rows per workgroup in slices
    of min(heads, 16) heads.  Scalar form: as many queries as the per-thread accumulators and
    48 KiB of LDS for the staged queries allow for a 16-head slice."""
    hb = min(num_heads, 16)
    if mfma_ok(kv_rank, rot_dim, dtype):
        return 64 // hb
    return max(1, min(16, ACC_ROWS // (hb * kv_rank), 12288 // (hb * (kv_rank + rot_dim))))


def decode_partitions(batch: int, num_heads: int, cus: int = 256, window: int = 0) -> int:
    """Key partitions (grid.z) of a decode launch of the MFMA form: a decode row is one
    single-wave workgroup per 16-head slice, so small batches split every row's keys until about
    four workgroups per CU exist (a power of two, at most 32, and no more than the 32-key units
    a sliding window can hold); the partials are merged by a second kernel.  Depends on the
    batch and the layer's constants only, so a captured decode graph keeps its grid."""
    forced = int(os.environ.get("EIA_LATENT_DECODE_P", "0"))
    if forced > 0:
        return min(forced, 64)
    wgs = max(1, batch * ((num_heads + 15) // 16))
    limit = 32 if window <= 0 else max(1, min(32, (window + 31) // 32 + 1))
    p = 1
    while p * 2 <= limit and wgs * p * 2 <= 4 * cus:
        p *= 2
    return p


def build_work(q_lens: List[int], qblock: int) -> List[int]:
    """[seq, first query] pairs, latest query blocks first (longest causal rows first)."""
    items = [(q0, s) for s, n in enumerate(q_lens) for q0 in range(0, n, qblock)]
    items.sort(key=lambda it: -it[0])
    out: List[int] = []
    for q0, s in items:
        out += [s, q0]
    return out


def _rotate_pairs(v: torch.Tensor, pos: torch.Tensor, inv_freq: torch.Tensor,
                  rot_dims: int, half: bool = False, amp: float = 1.0) -> torch.Tensor:
    """v [..., n] fp32, pos [...] broadcastable: the pairs of the first rot_dims entries turn --
    (2i, 2i+1), or (i, i + rot_dims/2) with ``half``; cos and sin are multiplied by ``amp``."""
    if rot_dims == 0:
        return v
    ang = pos.to(torch.float32)[..., None] * inv_freq[:rot_dims // 2]
    cs, sn = torch.cos(ang) * amp, torch.sin(ang) * amp
    ia = slice(0, rot_dims // 2) if half else slice(0, rot_dims, 2)
    ib = slice(rot_dims // 2, rot_dims) if half else slice(1, rot_dims, 2)
    a, b = v[..., ia], v[..., ib]
    out = v.clone()
    out[..., ia] = a * cs - b * sn
    out[..., ib] = b * cs + a * sn
    return out


def latent_prep(fused: torch.Tensor, q_off: int, q_rank: int, q_norm_w: Optional[torch.Tensor],
                c_off: int, kv_rank: int, kv_norm_w: Optional[torch.Tensor], kr_off: int,
                rot_dim: int, rot_dims: int, inv_freq: torch.Tensor, positions: torch.Tensor,
                slot_mapping: torch.Tensor, cache: Optional[torch.Tensor],
                eps: float, rot_half: bool = False, rot_amp: float = 1.0) -> Optional[torch.Tensor]:
    """One pass over a fused down-projection row [T, *]: RMS-norm of the query latent (returned,
    [T, q_rank]; None when q_rank == 0) and, when ``cache`` is given ([blocks, block, kv_rank +
    rot_dim]), RMS-norm of the KV latent + rotation of the shared key part written to the
    token's cache slot (slots < 0 are skipped).  ``rot_half`` pairs entry i with i + rot_dims/2
    instead of 2i with 2i+1; ``rot_amp`` multiplies cos and sin."""
    T = fused.shape[0]
    cq = None
    if not use_hip(fused):
        f = fused.float()
        if q_rank:
            x = f[:, q_off:q_off + q_rank]
            cq = (x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * q_norm_w.float()).to(fused.dtype)
        if cache is not None:
            x = f[:, c_off:c_off + kv_rank]
            c = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * kv_norm_w.float()
            kr = _rotate_pairs(f[:, kr_off:kr_off + rot_dim], positions[:T], inv_freq, rot_dims,
                               rot_half, rot_amp)
            rows = torch.cat([c, kr], -1).to(cache.dtype)
            sm = slot_mapping[:T].long()
            ok = sm >= 0
            cache.view(-1, cache.shape[-1])[sm[ok]] = rows[ok]
        return cq
    require(fused.stride(1) == 1, "latent_prep: fused rows must be contiguous")
    bf = fused.dtype == torch.bfloat16
    require(bf or fused.dtype == torch.float32, "latent_prep: bf16 or fp32")
    if q_rank:
        cq = torch.empty(T, q_rank, dtype=fused.dtype, device=fused.device)
    if cache is not None:
        require(cache.dtype == fused.dtype and cache.is_contiguous() and
                cache.shape[-1] == kv_rank + rot_dim, "latent_prep: cache layout")
        require(slot_mapping.dtype == torch.int32 and positions.dtype == torch.int32 and
                slot_mapping.numel() >= T and positions.numel() >= T, "latent_prep: int32 metadata")
        require(inv_freq.dtype == torch.float32 and inv_freq.numel() >= rot_dims // 2, "inv_freq")
    check(lib().eia_latent_prep(
        ptr(fused), fused.stride(0), q_off, q_rank, ptr(q_norm_w), ptr(cq),
        cq.stride(0) if cq is not None else 0, c_off, kv_rank, ptr(kv_norm_w), kr_off, rot_dim,
        rot_dims, ptr(inv_freq), ptr(positions), ptr(slot_mapping), ptr(cache),
        cache.shape[-1] if cache is not None else 0, float(eps), 1 if rot_half else 0,
        float(rot_amp), T, 1 if bf else 0, stream(fused)), "latent_prep")
    return cq


def _ref_rows(q_abs, q_rot, inv_freq, rot_dims, cache, block_table, positions, gate, scale,
              rows, seq_of_row, window=0, sink=None, rot_half=False, rot_amp=1.0):
    """Plain per-row attention over the paged latent cache (CPU path)."""
    R = q_abs.shape[-1]
    bs = cache.shape[1]
    flat = cache.view(-1, cache.shape[-1]).float()
    out = torch.zeros(q_abs.shape[0], q_abs.shape[1], R, dtype=torch.float32)
    for row, s in zip(rows, seq_of_row):
        p = int(positions[row])
        n = p + 1
        blocks = block_table[s, : (n + bs - 1) // bs].long()
        slots = (blocks[:, None] * bs + torch.arange(bs)[None, :]).reshape(-1)[:n]
        keys = flat[slots]                                               # [n, R + rd]
        if window > 0:
            keys = keys[max(0, n - window):]
        qr = _rotate_pairs(q_rot[row].float(), positions[row], inv_freq, rot_dims, rot_half,
                           rot_amp)
        q = torch.cat([q_abs[row].float(), qr], -1) * scale              # [H, R + rd]
        sc = q @ keys.t()                                                # [H, n]
        if sink is not None:     # one more term in the denominator, without a key or a value
            sc = torch.cat([sc, sink.float()[:, None]], -1)
        w = torch.softmax(sc, -1)[:, :keys.shape[0]]
        o = w @ keys[:, :R]
        if gate is not None:
            o = o * torch.sigmoid(gate[row].float())[:, None]
        out[row] = o
    return out


def latent_attention(q_abs: torch.Tensor, q_rot: torch.Tensor, inv_freq: torch.Tensor,
                     rot_dims: int, cache: torch.Tensor, md, gate: Optional[torch.Tensor],
                     scale: float, window: int = 0, sink: Optional[torch.Tensor] = None,
                     rot_half: bool = False, rot_amp: float = 1.0) -> torch.Tensor:
    """q_abs [T, H, R] and q_rot [T, H, rd] (any strides with a contiguous last dim; q_rot not
    yet rotated), gate [T, H] pre-sigmoid or None -> latent output [T, H, R] (contiguous):
    softmax((q_abs . c + rot(q_rot) . k_rot) * scale) weighted sum of c, times sigmoid(gate).
    ``window`` > 0: position i sees j with 0 <= i - j < window.  ``sink`` (fp32 [H]): the softmax
    denominator of head h also holds exp(sink[h]) (unscaled, no key, no value).  ``rot_half`` /
    ``rot_amp``: pair layout and cos / sin factor of the rotation, as in ``latent_prep``.
    ``md`` is the step's AttentionMetadata (decode rows first, then prefill chunks; the work
    list comes from ``md.prefill_work_for(query_block(...), build_work)``)."""
    T, H, R = q_abs.shape
    rd = q_rot.shape[-1]
    nd = md.num_decode
    out = torch.empty(T, H, R, dtype=q_abs.dtype, device=q_abs.device)
    if not use_hip(q_abs, cache):
        rows, seqs = list(range(nd)), list(range(nd))
        if nd:
            out[:nd] = _ref_rows(q_abs[:nd], q_rot[:nd], inv_freq, rot_dims, cache,
                                 md.decode_block_tables, md.positions[:nd],
                                 None if gate is None else gate[:nd], scale, rows, seqs, window,
                                 sink, rot_half, rot_amp).to(out.dtype)
        if md.num_prefill_tokens:
            cu = md.prefill_cu_q.tolist()
            rows = list(range(cu[-1]))
            seqs = [s for s in range(len(cu) - 1) for _ in range(cu[s + 1] - cu[s])]
            out[nd:] = _ref_rows(q_abs[nd:], q_rot[nd:], inv_freq, rot_dims, cache,
                                 md.prefill_block_tables, md.positions[nd:],
                                 None if gate is None else gate[nd:], scale, rows, seqs, window,
                                 sink, rot_half, rot_amp).to(out.dtype)
        return out
    bf = q_abs.dtype == torch.bfloat16
    require(bf or q_abs.dtype == torch.float32, "latent_attention: bf16 or fp32")
    require(q_abs.stride(2) == 1 and q_rot.stride(2) == 1 and q_rot.dtype == q_abs.dtype and
            cache.dtype == q_abs.dtype and cache.is_contiguous(), "latent_attention: layout")
    require(gate is None or (gate.dtype == q_abs.dtype and gate.stride(1) == 1), "gate layout")
    require(md.positions.dtype == torch.int32, "positions int32")
    require(sink is None or (sink.dtype == torch.float32 and sink.is_cuda and sink.numel() == H
                             and sink.is_contiguous()), "latent_attention: fp32 sink per head")
    bs = cache.shape[1]
    window = max(0, int(window))
    rh, amp = 1 if rot_half else 0, float(rot_amp)

    mfma = mfma_ok(R, rd, q_abs.dtype)

    def launch(lo, n_items, bt, lens, cu, work, qb):
        qa, qr, o = q_abs[lo:], q_rot[lo:], out[lo:]
        g = None if gate is None else gate[lo:]
        require(bt.dtype == torch.int32 and bt.stride(1) == 1, "block tables int32")
        if mfma:
            P = decode_partitions(n_items, H, window=window) if cu is None else 1
            pa = pm = None
            if P > 1:
                pa = torch.empty(n_items * H * P * R, dtype=torch.float32, device=q_abs.device)
                pm = torch.empty(n_items * H * P * 2, dtype=torch.float32, device=q_abs.device)
            check(lib().eia_latent_attn_mfma(
                ptr(qa), qa.stride(0), qa.stride(1), ptr(qr), qr.stride(0), qr.stride(1),
                ptr(inv_freq), rot_dims, ptr(cache), cache.shape[-1], ptr(bt), bt.stride(0),
                ptr(lens), ptr(cu), ptr(work), n_items, ptr(md.positions[lo:]), ptr(g),
                g.stride(0) if g is not None else 0, ptr(o), o.stride(0), o.stride(1),
                float(scale), H, R, rd, bs, qb, window, ptr(sink), rh, amp, P, ptr(pa), ptr(pm),
                stream(q_abs)), "latent_attn_mfma")
            return
        check(lib().eia_latent_attn(
            ptr(qa), qa.stride(0), qa.stride(1), ptr(qr), qr.stride(0), qr.stride(1),
            ptr(inv_freq), rot_dims, ptr(cache), cache.shape[-1], ptr(bt), bt.stride(0), ptr(lens),
            ptr(cu), ptr(work), n_items, ptr(md.positions[lo:]), ptr(g),
            g.stride(0) if g is not None else 0, ptr(o), o.stride(0), o.stride(1), float(scale),
            H, R, rd, bs, qb, window, ptr(sink), rh, amp, 1 if bf else 0, stream(q_abs)),
            "latent_attn")

    if nd:
        launch(0, nd, md.decode_block_tables, md.decode_seq_lens, None, None, 1)
    if md.num_prefill_tokens:
        qb = query_block(H, R, rd, q_abs.dtype)
        work, n_work = md.prefill_work_for(qb, build_work)
        launch(nd, n_work, md.prefill_block_tables, None, md.prefill_cu_q, work, qb)
    return out
