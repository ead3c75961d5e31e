"""Gapidra test bodies, parametrised by device and dtype: the CPU file runs them on the
framework's PyTorch ops in fp32, the GPU file on the HIP kernels in fp32 and bf16."""

from __future__ import annotations

import math

import numpy as np
import torch

import gapidra_common as C
from oracles import gapidra_oracle as O


def tol(dtype):
    # fp32 is the sharp check; bf16 activations round at every product of these tiny models
    return 2e-4 if dtype == torch.float32 else 0.12


def ktol(dtype):
    """Kernel-level checks: inputs are already rounded to the dtype, so only the kernel's own
    roundings (bf16 outputs) remain."""
    return 2e-4 if dtype == torch.float32 else 1.5e-2


def _tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def _check(got, want, dtype, what):
    e = C.rel_err(got, want)
    assert e < tol(dtype), (what, e)


def _np(t):
    return t.double().cpu().numpy()


# ------------------------------------------------------------------ mechanisms alone
def case_residual_rms_step(device, dtype):
    """The layer boundary: zero, one or two sublayer outputs join the stream un-normed -- stored
    rows or the split-K partial sums of their GEMMs (with and without a bias) -- and the next
    input norm follows or not; widths that are and are not multiples of four."""
    from enterprise_inference_amd.ops import norm
    from enterprise_inference_amd.ops.gemm import SplitK
    g = torch.Generator().manual_seed(1)
    for W in (46, 40, 256, 1024, 130):
        for kinds, use_next in (((), 1), ((1,), 1), ((1, 1), 1), ((2,), 1), ((2, 1), 1), ((1, 2), 0),
                                ((2, 3), 1), ((1, 1), 0)):
            x = torch.randn(5, W, generator=g) * 2
            want = _np(x).copy()
            ys = []
            for kind in kinds:
                if kind == 1:
                    y = (torch.randn(5, W, generator=g) * 3 + 0.5).to(dtype)
                    want += _np(y)
                    ys.append(y.to(device))
                else:
                    part = torch.randn(3, 5, W, generator=g) * 2
                    bias = torch.randn(W, generator=g).to(dtype) if kind == 3 else None
                    want += _np(part).sum(0) + (_np(bias) if bias is not None else 0.0)
                    ys.append(SplitK(part.to(device), 3, 5, W,
                                     bias.to(device) if bias is not None else None))
            w = torch.randn(W, generator=g).to(dtype)
            xd = x.clone().to(device)
            h = norm.residual_rms_step(xd, 1e-5, ys, w.to(device) if use_next else None)
            assert np.allclose(_np(xd), want, atol=3e-5, rtol=1e-5), (W, kinds)
            if use_next:
                assert h.dtype == dtype
                hw = np.stack([O.rms_norm(want[r], _np(w), 1e-5) for r in range(5)])
                assert np.allclose(_np(h), hw, atol=ktol(dtype), rtol=ktol(dtype)), (W, kinds)
            else:
                assert h is None


def case_xielu(device, dtype):
    """Both branches of the activation, its two numbers of either sign, large arguments, and
    the input as a stored row or as split-K partial sums."""
    from enterprise_inference_amd.ops import activation
    from enterprise_inference_amd.ops.gemm import SplitK
    g = torch.Generator().manual_seed(2)
    for F, (p, q) in ((24, (0.3, -0.7)), (130, (-2.0, 1.5)), (64, (4.0, 0.0)), (7, (0.0, -5.0))):
        pq = torch.tensor([p, q]).to(dtype)
        z = (torch.randn(6, F, generator=g) * 3).to(dtype)
        z[0, :3] = torch.tensor([0.0, -30.0, 9.0]).to(dtype)
        want = np.stack([O.xielu(_np(z[r]), float(pq[0]), float(pq[1])) for r in range(6)])
        got = activation.xielu(z.to(device), pq.to(device))
        assert got.dtype == dtype
        assert np.allclose(_np(got), want, atol=ktol(dtype), rtol=ktol(dtype)), (F, p, q)
        part = torch.randn(3, 6, F, generator=g) * 2
        zs = _np(part).sum(0)
        want = np.stack([O.xielu(zs[r], float(pq[0]), float(pq[1])) for r in range(6)])
        got = activation.xielu(SplitK(part.to(device), 3, 6, F), pq.to(device))
        # (a width the kernel does not sum itself is rounded to the dtype before the activation)
        loose = 6e-2 if (dtype != torch.float32 and F % 4) else ktol(dtype)
        assert np.allclose(_np(got), want, atol=loose, rtol=loose), (F, p, q, "partials")
        # the same columns inside the wider row of a fused projection's partial sums
        from enterprise_inference_amd.ops.gemm import columns
        off = 8
        wide = torch.randn(3, 6, off + F + 5 + (-(off + F + 5)) % 4, generator=g)
        wide[:, :, off:off + F] = part
        got = activation.xielu(columns(SplitK(wide.to(device), 3, 6, wide.shape[2]), off, F),
                               pq.to(device))
        assert np.allclose(_np(got), want, atol=loose, rtol=loose), (F, p, q, "partial columns")


def case_sigmoid_gate(device, dtype):
    """a * sigmoid(g) on column slices of wider rows."""
    from enterprise_inference_amd.ops import activation
    g = torch.Generator().manual_seed(3)
    a = (torch.randn(5, 77, generator=g) * 2).to(dtype).to(device)
    gate = (torch.randn(5, 130, generator=g) * 4).to(dtype).to(device)
    for n, a0, g0 in ((30, 0, 3), (77, 0, 53), (1, 5, 129)):
        got = activation.sigmoid_gate(a[:, a0:a0 + n], gate[:, g0:g0 + n])
        want = _np(a[:, a0:a0 + n]) * O.sigmoid(_np(gate[:, g0:g0 + n]))
        assert got.shape == (5, n) and got.is_contiguous()
        assert np.allclose(_np(got), want, atol=ktol(dtype), rtol=ktol(dtype))
    # heads laid out [H, T, V] (a batched product's output) are concatenated on the way
    for H, V in ((3, 10), (4, 16), (1, 7)):
        a3 = (torch.randn(H, 5, V, generator=g) * 2).to(dtype).to(device)
        got = activation.sigmoid_gate(a3, gate[:, 2:2 + H * V])
        want = _np(a3).transpose(1, 0, 2).reshape(5, H * V) * O.sigmoid(_np(gate[:, 2:2 + H * V]))
        assert got.shape == (5, H * V) and got.is_contiguous()
        assert np.allclose(_np(got), want, atol=ktol(dtype), rtol=ktol(dtype))
        got = activation.sigmoid_gate(a3, gate[:, 4:4 + H * V].contiguous())
        want = _np(a3).transpose(1, 0, 2).reshape(5, H * V) * O.sigmoid(_np(gate[:, 4:4 + H * V]))
        assert np.allclose(_np(got), want, atol=ktol(dtype), rtol=ktol(dtype))


def case_frequencies():
    """Rotation frequencies with and without interpolation, also where the blend's ends are
    clamped to the first and the last pair."""
    from enterprise_inference_amd.ops.rotary import rotary_frequencies
    for rot in ({"dims": 8, "base": 1000.0}, {"dims": 6, "base": 5000.0, "scaling": C.YARN},
                {"dims": 32, "base": 250.0, "scaling": {"factor": 16.0, "original": 4096,
                                                        "fast": 64.0, "slow": 2.0}},
                {"dims": 4, "base": 10.0, "scaling": {"factor": 3.0, "original": 8, "fast": 1e-3,
                                                      "slow": 1e-6}},
                {"dims": 16, "base": 1e6, "scaling": {"factor": 2.0, "original": 16, "fast": 1e3,
                                                      "slow": 1e2}}):
        f, amp = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        wf, wamp = O.frequencies(rot)
        assert f.dtype == torch.float32 and f.shape == (rot["dims"] // 2,)
        assert np.allclose(_np(f), np.array(wf), rtol=1e-6, atol=0) and abs(amp - wamp) < 1e-12


def case_qk_rope_cache(device, dtype):
    """Whole-projection RMS norm, rotation of part of every head in either pair layout, values
    copied as projected, rows without a slot skipped, other slots untouched; the row stored or as
    split-K partial sums."""
    from enterprise_inference_amd.ops import window_attention as wa
    from enterprise_inference_amd.ops.gemm import SplitK
    from enterprise_inference_amd.ops.rotary import rotary_frequencies
    g = torch.Generator().manual_seed(4)
    for mq, mk, D, vw, rdims, half, scaling, split in (
            (4, 2, 16, 24, 8, False, C.YARN, 0), (6, 2, 10, 14, 10, True, None, 0),
            (2, 2, 80, 40, 20, False, None, 0), (1, 1, 6, 5, 0, False, None, 0),
            (4, 2, 16, 24, 16, False, C.YARN, 3), (3, 1, 24, 20, 6, True, C.YARN, 2)):
        T, bs, nb = 7, 4, 5
        k_off, v_off = 3, 3 + mk * D
        q_off = v_off + vw + 1
        width = -(-(q_off + mq * D + 2) // 4) * 4
        fused = (torch.randn(T, width, generator=g) * 2).to(dtype)
        part = torch.randn(max(split, 1), T, width, generator=g)
        qw = (1 + 0.3 * torch.randn(mq * D, generator=g)).to(dtype)
        kw = (1 + 0.3 * torch.randn(mk * D, generator=g)).to(dtype)
        inv_freq, amp = rotary_frequencies(rdims, 300.0, scaling if rdims else None)
        pos = torch.tensor([0, 1, 5, 37, 64, 511, 1000], dtype=torch.int32)
        slots = torch.tensor([9, 2, -1, 17, 0, 5, 19], dtype=torch.int32)
        kd = torch.full((nb, bs, mk * D), 7.0, dtype=dtype).to(device)
        vd = torch.full((nb, vw, bs), 7.0, dtype=dtype).to(device)
        src = SplitK(part.to(device), split, T, width) if split else fused.to(device)
        q = wa.qk_rope_cache(src, q_off, k_off, v_off, mq, mk, D, vw, qw.to(device),
                             kw.to(device), inv_freq.to(device), rdims, half, amp,
                             pos.to(device), kd, vd, slots.to(device), 1e-5)
        f = _np(part).sum(0) if split else _np(fused)
        fr = [float(v) for v in inv_freq]
        kflat = _np(kd).reshape(nb * bs, -1)
        vflat = _np(vd.permute(0, 2, 1)).reshape(nb * bs, -1)
        used = set()
        for t in range(T):
            def side(off, m, w):
                x = O.rms_norm(f[t, off:off + m * D], _np(w), 1e-5).reshape(m, D)
                return np.stack([O.rotate(x[a], int(pos[t]), fr, amp, rdims, not half)
                                 for a in range(m)]).reshape(-1)
            assert np.allclose(_np(q[t]), side(q_off, mq, qw), atol=ktol(dtype) * 3, rtol=ktol(dtype))
            s = int(slots[t])
            if s < 0:
                continue
            used.add(s)
            assert np.allclose(kflat[s], side(k_off, mk, kw), atol=ktol(dtype) * 3, rtol=ktol(dtype))
            assert np.allclose(vflat[s], f[t, v_off:v_off + vw], atol=ktol(dtype) if split else 0,
                               rtol=ktol(dtype) if split else 0)
        for s in range(nb * bs):
            if s not in used:
                assert (kflat[s] == 7.0).all() and (vflat[s] == 7.0).all()


def _paged(n, bs, seed):
    """A shuffled block table for n tokens and the slot of every position."""
    nblk = -(-n // bs)
    g = torch.Generator().manual_seed(seed)
    table = (torch.randperm(nblk + 3, generator=g)[:nblk]).to(torch.int32)
    slots = torch.tensor([int(table[j // bs]) * bs + j % bs for j in range(n)])
    return table, slots, nblk + 3


def _metadata(device, table, decode_pos, chunk, slot_of=None):
    """One sequence seen as decode rows (one per position in decode_pos, every row its own copy
    of the sequence) followed by one prefill chunk (start, n).  ``slot_of``: write this step's
    rows into the cache (position -> slot); default: rows write nothing."""
    from enterprise_inference_amd.ops.attention import AttentionMetadata
    nd = len(decode_pos)
    start, n = chunk
    plist = list(decode_pos) + list(range(start, start + n))
    pos = torch.tensor(plist, dtype=torch.int32)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    sm = torch.full((nd + n,), -1, dtype=torch.int32)
    if slot_of is not None:
        sm = torch.tensor([int(slot_of[p]) for p in plist], dtype=torch.int32)
    return AttentionMetadata(
        num_decode=nd, num_prefill_tokens=n, slot_mapping=sm.to(device), positions=pos.to(device),
        decode_block_tables=table[None, :].repeat(max(nd, 1), 1).contiguous().to(device),
        decode_seq_lens=i32([p + 1 for p in decode_pos]) if nd else None,
        prefill_block_tables=table[None, :].contiguous().to(device) if n else None,
        prefill_seq_lens=i32([start + n]) if n else None,
        prefill_cu_q=i32([0, n]) if n else None, prefill_q_lens=[n] if n else None)


def _needle_positions(i, size, n, bs):
    edge = i - size + 1 if size else 0
    cand = {edge, edge - 1, edge + 1, i, i - 1, 0, 1, n // 3, edge - 40,
            (edge // bs) * bs, (edge // bs) * bs - 1, (i // bs) * bs, (i // bs) * bs - 1}
    return sorted(c for c in cand if 0 <= c <= i)


def case_sigmoid_needle(device, dtype, H=4, G=2, D=16, Dv=8, size=40, n=150, bs=16):
    """One key made to stand out under a strongly negative score bias: the query at position i and
    the key at position j share a large component, so head outputs are about that key's value
    when j is visible and about nothing when not.  j runs over the window's inside and outside
    edge, page borders, the first tokens and far keys; i is read as a prefill row and as a
    decode row."""
    from enterprise_inference_amd.ops import window_attention as wa
    g = torch.Generator().manual_seed(5)
    table, slots, nblk = _paged(n, bs, 6)
    i = n - 7
    pb = -6.0 + torch.randn(H, generator=g)
    pb[0] = 0.4                                # one head whose ordinary keys all count
    spec = wa.WindowSpec(H, G, 1, D, Dv, size, 0, mult=torch.full((H,), 0.3).to(device),
                         weights=1, bias=pb.float().to(device))
    for j in _needle_positions(i, size, n, bs):
        q = torch.randn(n, H, D, generator=g) * 0.5
        k = torch.randn(n, G, D, generator=g) * 0.5
        v = torch.randn(n, G, Dv, generator=g)
        u = torch.zeros(D)
        u[j % D] = 1.0
        q[i] += 8.0 * u
        k[j] += 8.0 * u
        q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
        kc = torch.zeros(nblk, bs, G * D, dtype=dtype)
        vc = torch.zeros(nblk, G * Dv, bs, dtype=dtype)
        kc.view(-1, G * D)[slots] = k.reshape(n, -1)
        vc[slots // bs, :, slots % bs] = v.reshape(n, -1)
        rows = [i, min(i + 3, n - 1), j]
        chunk = (i - 5, 9)
        md = _metadata(device, table, rows, chunk)
        pos = rows + list(range(chunk[0], chunk[0] + chunk[1]))
        qs = torch.stack([q[p].reshape(-1) for p in pos])
        got = wa.window_attention(qs.to(device), kc.to(device), vc.to(device), md, spec, None)
        kn, vals = [_np(k[t]) for t in range(n)], [_np(v[t]) for t in range(n)]
        for r, p in enumerate(pos):
            want = O.sigmoid_core(_np(q[p]), kn, vals, p, H, G, size, 0.3, _np(pb)).reshape(-1)
            d = np.abs(_np(got[r]) - want).max()
            # head 0 sums up to ``size`` weights near 0.6, so its output is that much larger
            assert d < (2e-4 if dtype == torch.float32 else 4e-2 * max(1.0, np.abs(want).max())), \
                (j, p, d)


def case_latent_needle(device, dtype, H=3, D=10, rd=6, rdims=4, Dv=14, R=20, size=40, n=150,
                       bs=16, scaling=None):
    """The latent attention kernel with one key made to stand out (through the latent part or
    through the shared rotated part), sinks large enough to matter, both at window edges, page
    borders, first tokens and far away, read as prefill rows and as decode rows; the step's own
    rows are written by the cache-write kernel, the rest of the cache is prepared."""
    from enterprise_inference_amd.ops import latent_attention as la
    from enterprise_inference_amd.ops.rotary import rotary_frequencies
    g = torch.Generator().manual_seed(7)
    table, slots, nblk = _paged(n, bs, 8)
    i = n - 7
    inv_freq, amp = rotary_frequencies(rdims, 200.0, scaling)
    fr = [float(f) for f in inv_freq]
    sink = torch.tensor([3.0, -2.0, 0.5, 1.0] * 8)[:H]
    uk = torch.randn(H, D, R, generator=g) * R ** -0.5
    uv = torch.randn(H, Dv, R, generator=g) * R ** -0.5
    cw = (1 + 0.2 * torch.randn(R, generator=g)).to(dtype)
    scale = 0.3
    for jn, j in enumerate(_needle_positions(i, size, n, bs)):
        via_rot = bool(jn & 1) and rd > rdims         # the stand-out component's place
        raw = (torch.randn(n, R + rd, generator=g)).to(dtype)        # [latent | key part], raw
        qn = torch.randn(n, H, D, generator=g) * 0.5
        qr = torch.randn(n, H, rd, generator=g) * 0.5
        if via_rot:
            raw[j, R + rd - 1] += 9.0                 # an unrotated entry of the shared part
            qr[i, :, rd - 1] += 9.0
        # the cache as earlier steps left it: float64 norm + rotation, rounded once
        lat64 = [O.rms_norm(_np(raw[t, :R]), _np(cw), 1e-5) for t in range(n)]
        if not via_rot:
            lat64[j] = lat64[j] * 1.0
            lat64[j][j % R] += 6.0
        kr64 = [O.rotate(_np(raw[t, R:]), t, fr, amp, rdims, False) for t in range(n)]
        cache = torch.zeros(nblk, bs, R + rd, dtype=dtype)
        rows64 = torch.tensor(np.concatenate([np.stack(lat64), np.stack(kr64)], 1)).to(dtype)
        cache.view(-1, R + rd)[slots] = rows64
        latn = [_np(rows64[t, :R]) for t in range(n)]
        krn = [_np(rows64[t, R:]) for t in range(n)]
        if not via_rot:                               # the query meets the needle through W_uk
            for a in range(H):
                want_dir = _np(uk[a]) @ latn[j]
                qn[i, a] += torch.tensor(4.0 * want_dir / max(np.linalg.norm(want_dir), 1e-6)).float()
        qn, qr = qn.to(dtype), qr.to(dtype)
        rows = [i, min(i + 3, n - 1), j]
        chunk = (i - 5, 9)
        md = _metadata(device, table, rows, chunk)
        pos = rows + list(range(chunk[0], chunk[0] + chunk[1]))
        q_abs = torch.stack([torch.einsum("hd,hdr->hr", qn[p].double(), uk.double()) for p in pos]
                            ).to(dtype)
        q_rot = torch.stack([qr[p] for p in pos])
        got = la.latent_attention(q_abs.to(device), q_rot.to(device), inv_freq.to(device), rdims,
                                  cache.to(device), md, None, scale, size,
                                  sink.float().to(device), True, amp)
        uk_abs = np.broadcast_to(np.eye(R), (H, R, R))        # the queries are already absorbed
        for r, p in enumerate(pos):
            qrp = np.stack([O.rotate(_np(q_rot[r, a]), p, fr, amp, rdims, False) for a in range(H)])
            want = O.latent_core(_np(q_abs[r]), qrp, latn, krn, uk_abs, _np(uv), p, size, scale,
                                 _np(sink))
            have = np.einsum("hr,hvr->hv", _np(got[r]), _np(uv))
            d = np.abs(have - want).max()
            assert d < (2e-4 if dtype == torch.float32 else 5e-2), (j, p, via_rot, d)


def case_latent_prep(device, dtype):
    """Cache write of the latent mixers: norm of the latent, rotation of the shared key part in
    the half-split layout with a factor on cos and sin, on part of its entries."""
    from enterprise_inference_amd.ops import latent_attention as la
    from enterprise_inference_amd.ops.rotary import rotary_frequencies
    g = torch.Generator().manual_seed(9)
    for R, rd, rdims, scaling in ((20, 6, 4, None), (64, 16, 16, C.YARN), (8, 2, 2, None)):
        T, bs, nb = 6, 4, 4
        c_off = 5
        fused = (torch.randn(T, c_off + R + rd + 3, generator=g) * 2).to(dtype)
        cw = (1 + 0.3 * torch.randn(R, generator=g)).to(dtype)
        inv_freq, amp = rotary_frequencies(rdims, 777.0, scaling)
        pos = torch.tensor([0, 3, 64, 65, 900, 17], dtype=torch.int32)
        slots = torch.tensor([3, -1, 8, 0, 15, 6], dtype=torch.int32)
        cache = torch.full((nb, bs, R + rd), 7.0, dtype=dtype).to(device)
        la.latent_prep(fused.to(device), 0, 0, None, c_off, R, cw.to(device), c_off + R, rd, rdims,
                       inv_freq.to(device), pos.to(device), slots.to(device), cache, 1e-5, True, amp)
        flat = _np(cache).reshape(nb * bs, -1)
        fr = [float(f) for f in inv_freq]
        for t, s in enumerate(slots.tolist()):
            if s < 0:
                continue
            f = _np(fused[t])
            want = np.concatenate([O.rms_norm(f[c_off:c_off + R], _np(cw), 1e-5),
                                   O.rotate(f[c_off + R:c_off + R + rd], int(pos[t]), fr, amp,
                                            rdims, False)])
            assert np.allclose(flat[s], want, atol=ktol(dtype) * 3, rtol=ktol(dtype)), (R, t)
        assert sum(int((flat[s] == 7.0).all()) for s in range(nb * bs)) == nb * bs - 5


# ------------------------------------------------------------------ whole models
def case_layers(device, dtype, cfg_fn=C.config_a):
    """The residual stream after every layer."""
    cfg = cfg_fn()
    W = C.random_weights(cfg, 9, dtype)
    t = _tokens(21, cfg["vocab"], 5)
    want = []
    C.oracle_logits(cfg, W, t, want)
    sess = C.make_session(cfg, W, device, dtype, max_tokens=64, block_size=16, max_live=1)
    try:
        from enterprise_inference_amd.engine.sequence import Sequence
        seq = Sequence("s", list(t), sess._params)
        plan = sess.scheduler.plan_given([(seq, len(t))])
        r = sess.runner
        r._flip_staging()
        sp = r._prepare_eager(sess.scheduler.bm, plan, logit_rows=[])
        r.d_e_buf[:sp["off"]].copy_(r.e_buf[:sp["off"]])
        ids, md, _ = r._eager_inputs(sp)
        got = []
        with torch.no_grad():
            r.model(ids, md, r.kv_caches, collect=got)
        r.finish_step()
        assert len(got) == len(want) == len(cfg["layers"])
        for k, (a, b) in enumerate(zip(got, want)):
            e = np.abs(_np(a) - b).max() / np.abs(b).max()
            assert e < (1e-4 if dtype == torch.float32 else 0.08), (k, e)
    finally:
        sess.close()


def case_schedules(device, dtype, cfg_fn=C.config_a, seed=0, block_size=16):
    """Whole prompts, prompt + one-by-one decoding, portions of several sizes down to two tokens
    and mixed batches with reuse of pages all give the oracle's logits."""
    cfg = cfg_fn()
    W = C.random_weights(cfg, seed, dtype)
    V = cfg["vocab"]
    reqs = {"a": _tokens(70, V, 11), "b": _tokens(37, V, 12), "c": _tokens(5, V, 13),
            "d": _tokens(1, V, 14), "e": _tokens(49, V, 15)}
    want = {k: C.oracle_logits(cfg, W, t) for k, t in reqs.items()}
    # pool of 8 pages (of 16 tokens: "a" alone needs 5), so pages must be used again
    sess = C.make_session(cfg, W, device, dtype, max_tokens=8 * block_size, block_size=block_size,
                          max_live=2)
    try:
        for k, t in reqs.items():
            got = sess.step([{"id": k, "tokens": t, "want": list(range(len(t)))}], end=[k])
            _check(got, want[k], dtype, ("whole", k))
        # a prompt portion, then token by token: the windows pass over decoded tokens
        for k in ("a", "b"):
            t = reqs[k]
            n0 = len(t) - 34
            got = [sess.step([{"id": k, "tokens": t[:n0], "want": [n0 - 1]}])]
            for i in range(n0, len(t)):
                got.append(sess.step([{"id": k, "tokens": [t[i]], "want": [0]}],
                                     end=[k] if i == len(t) - 1 else []))
            _check(torch.cat(got), want[k][n0 - 1:], dtype, ("decode", k))
        # portions: sizes cross page borders (16) and window edges and go down to two tokens
        t, at, got = reqs["a"], 0, []
        for n in (2, 13, 2, 16, 1, 17, 2, 15, 2):
            got.append(sess.step([{"id": "a", "tokens": t[at:at + n], "want": list(range(n))}],
                                 end=["a"] if at + n == len(t) else []))
            at += n
        assert at == len(t)
        _check(torch.cat(got), want["a"], dtype, "portions")
    finally:
        sess.close()
    # mixed batches on 4 sequences / 10 pages: unequal requests side by side, decode rows beside
    # prompt portions, requests that pause, pages freed and taken again
    sess = C.make_session(cfg, W, device, dtype, max_tokens=10 * block_size, block_size=block_size,
                          max_live=4)
    try:
        got = {k: [] for k in reqs}
        at = {k: 0 for k in reqs}

        def run(plan, end=()):
            entries = []
            for k, n in plan:
                entries.append({"id": k, "tokens": reqs[k][at[k]:at[k] + n], "want": list(range(n))})
            out = sess.step(entries, end)
            r = 0
            for k, n in plan:
                got[k].append(out[r:r + n])
                r += n
                at[k] += n
        run([("d", 1), ("b", 3), ("c", 2)], end=["d"])
        run([("b", 1), ("c", 3), ("a", 20)], end=["c"])           # c finishes: its page is free
        run([("a", 1), ("e", 30), ("b", 17)])                     # e takes the freed pages
        run([("e", 1), ("b", 16), ("a", 2)], end=["b"])
        run([("a", 47)], end=["a"])                               # e pauses
        run([("e", 18)], end=["e"])
        for k in reqs:
            assert at[k] == len(reqs[k])
            _check(torch.cat(got[k]), want[k], dtype, ("mixed", k))
        # a second life for a finished request's name, on reused pages
        got2 = sess.step([{"id": "b", "tokens": reqs["b"], "want": list(range(len(reqs["b"])))},
                          {"id": "c", "tokens": reqs["c"], "want": [4]}], end=["b", "c"])
        _check(got2[:-1], want["b"], dtype, "again b")
        _check(got2[-1:], want["c"][4:], dtype, "again c")
        bm = sess.scheduler.bm
        assert bm.num_free_blocks() == bm.num_blocks
    finally:
        sess.close()


def case_long_decode(device, dtype, cfg_fn=C.config_b):
    """140 tokens decoded one by one after a 3-token prompt, over many page borders and far past
    every window."""
    cfg = cfg_fn()
    W = C.random_weights(cfg, 3, dtype)
    t = _tokens(143, cfg["vocab"], 21)
    want = C.oracle_logits(cfg, W, t)
    sess = C.make_session(cfg, W, device, dtype, max_tokens=160, block_size=16, max_live=1)
    try:
        got = [sess.step([{"id": "x", "tokens": t[:3], "want": [0, 1, 2]}])]
        for i in range(3, len(t)):
            got.append(sess.step([{"id": "x", "tokens": [t[i]], "want": [0]}]))
        _check(torch.cat(got), want, dtype, "long decode")
    finally:
        sess.close()


def case_generate(device, dtype, cfg_fn=C.config_a, expect_graphs=None):
    """Greedy generation through LLMEngine (its scheduler, batching and sampler): every emitted
    token is the oracle's argmax given the tokens before it, for unequal prompts in one batch."""
    import copy

    from enterprise_inference_amd.config import (CacheConfig, EngineConfig, ModelConfig,
                                                 SchedulerConfig)
    from enterprise_inference_amd.engine.llm_engine import LLMEngine
    from enterprise_inference_amd.engine.sampling_params import SamplingParams
    cfg = cfg_fn()
    W = C.random_weights(cfg, 5, dtype)
    ec = EngineConfig(model=ModelConfig.from_hf_dict(copy.deepcopy(cfg)), dtype=dtype, device=device,
                      load_format="dummy",
                      cache=CacheConfig(block_size=16, num_gpu_blocks=24),
                      scheduler=SchedulerConfig(max_num_seqs=3, max_num_batched_tokens=32,
                                                max_model_len=128))
    eng = LLMEngine(ec)
    model = eng.executor.runner.model
    model.load_weights(W.items())
    model.post_load()
    if expect_graphs is not None:
        assert bool(eng.executor.runner.graphs) == expect_graphs
    prompts = [_tokens(n, cfg["vocab"], 30 + n) for n in (40, 7, 1, 19)]     # 4 prompts, 3 seats
    outs = eng.generate(prompt_token_ids=prompts,
                        params=SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    for p, o in zip(prompts, outs):
        toks = list(o.outputs[0].token_ids)
        assert len(toks) == 12
        lg = C.oracle_logits(cfg, W, p + toks[:-1])
        for i, tk in enumerate(toks):
            row = lg[len(p) - 1 + i]
            # the chosen token is the oracle's best, or within rounding of it
            assert float(row.max() - row[tk]) <= (1e-3 if dtype == torch.float32 else 0.15), (i, tk)
    eng.shutdown()
