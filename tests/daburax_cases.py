"""Daburax test bodies, parametrised by device and dtype: the CPU file runs them on the
framework's PyTorch ops in fp32, the GPU file on the HIP kernels in fp32 and bf16."""

from __future__ import annotations

import math

import numpy as np
import torch

import daburax_common as C
from gapidra_cases import _metadata, _paged
from oracles import daburax_oracle as O


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


def _i32(v, device):
    return torch.tensor(v, dtype=torch.int32, device=device)


def _weights(cfg, seed, dtype):
    """16-bit whole-model runs use weights whose discrete decisions and output signs do not rest
    on close calls (see daburax_common.random_weights); those are checked in fp32."""
    soft = dtype != torch.float32
    return C.random_weights(cfg, seed, dtype, decisive=soft, tie_qk=soft)


# ------------------------------------------------------------------ mechanisms alone
def case_hyper_step(device, dtype):
    """The sublayer boundary over 1 .. 5 streams: no output (only the next input), a stored
    output, split-K partial sums with and without a bias; with and without a next norm; widths
    that are and are not multiples of four; norm weights stored around zero."""
    from enterprise_inference_amd.ops import norm
    from enterprise_inference_amd.ops.gemm import SplitK
    g = torch.Generator().manual_seed(1)
    for W in (46, 40, 256, 1030):
        for NS in (1, 2, 3, 5):
            for kind, use_next in ((0, 1), (1, 1), (1, 0), (2, 1), (3, 1), (3, 0)):
                T = 5
                X = torch.randn(T, NS, W, generator=g) * 2
                mix = torch.eye(NS) + torch.randn(NS, NS, generator=g) * 0.3
                outw, inw = torch.randn(NS, generator=g), torch.randn(NS, generator=g)
                wn = (torch.randn(W, generator=g) * 0.2).to(dtype)
                want = _np(X).copy()
                y = yd = None
                if kind == 1:
                    y = (torch.randn(T, W, generator=g) * 3 + 0.5).to(dtype)
                    yd, y = _np(y), y.to(device)
                elif kind >= 2:
                    part = torch.randn(3, T, W, generator=g) * 2
                    bias = (torch.randn(W, generator=g)).to(dtype) if kind == 3 else None
                    yd = _np(part).sum(0) + (_np(bias) if bias is not None else 0.0)
                    y = SplitK(part.to(device), 3, T, W, bias.to(device) if bias is not None
                               else None)
                if yd is not None:
                    want = np.einsum("sj,tsw->tjw", _np(mix), want) \
                        + 0.7 * _np(outw)[None, :, None] * yd[:, None, :]
                Xd = X.to(device)
                h = norm.hyper_step(Xd, 1e-5, y, mix.to(device), outw.to(device), 0.7,
                                    inw.to(device) if use_next else None,
                                    wn.to(device) if use_next else None, 1.0)
                assert np.allclose(_np(Xd), want, atol=1e-4, rtol=1e-5), (W, NS, kind)
                if use_next:
                    u = np.einsum("j,tjw->tw", _np(inw), want)
                    hw = np.stack([O.norm(u[t], _np(wn), 1e-5) for t in range(T)])
                    assert np.allclose(_np(h), hw, atol=ktol(dtype) * 3, rtol=ktol(dtype)), \
                        (W, NS, kind)
                else:
                    assert h is None


def case_bigram_embed(device, dtype):
    """Embedding rows: first tokens take the table's last row, a chunk's first row takes the
    previous token from the sequence's slot, later rows from the row before; slots are handed
    from one sequence to the next; a padding row stores nothing; the table-free form."""
    from enterprise_inference_amd.ops.embedding import bigram_embed
    g = torch.Generator().manual_seed(2)
    V, W, B = 50, 24, 11
    emb = torch.randn(V, W, generator=g).to(dtype)
    big = torch.randn(B + 1, W, generator=g).to(dtype)
    bg = {"buckets": B, "mul_prev": 7, "mul_cur": 3}
    seqs = {0: _tokens(9, V, 3), 1: _tokens(4, V, 4), 2: _tokens(6, V, 5)}
    last = torch.full((4,), 49, dtype=torch.int32).to(device)          # stale slot contents

    def want_rows(toks, lo, hi):
        out = []
        for t in range(lo, hi):
            r = O.bigram_row(toks[t - 1] if t else None, toks[t], bg)
            out.append(_np(emb[toks[t]]) * 1.5 + _np(big[r]))
        return np.stack(out)

    def step(chunks, streams=2):
        """chunks: (sequence, slot, lo, hi); decode rows (one token, lo > 0) first."""
        ids, pos, cu, slots = [], [], [0], []
        for s, sl, lo, hi in chunks:
            ids += seqs[s][lo:hi]
            pos += list(range(lo, hi))
            cu.append(len(ids))
            slots.append(sl)
        X = bigram_embed(_i32(ids, device), emb.to(device), 1.5, big.to(device), B, 7, 3, last,
                         _i32(slots, device), _i32(cu, device), len(chunks), _i32(pos, device),
                         streams)
        assert X.shape == (len(ids), streams, W) and X.dtype == torch.float32
        r = 0
        for s, sl, lo, hi in chunks:
            for j in range(streams):
                assert np.allclose(_np(X[r:r + hi - lo, j]), want_rows(seqs[s], lo, hi),
                                   atol=1e-5), (s, lo, hi)
            r += hi - lo

    step([(0, 2, 0, 4), (1, 0, 0, 1)])
    step([(0, 2, 4, 5), (1, 0, 1, 4)])                 # a decode row and a portion
    step([(0, 2, 5, 6), (2, 0, 0, 3)])                 # sequence 2 takes sequence 1's slot
    step([(0, 2, 6, 7), (2, 0, 3, 4)], streams=1)
    step([(2, 0, 4, 6), (0, 2, 7, 9)], streams=3)
    assert last.tolist()[0] == seqs[2][5] and last.tolist()[2] == seqs[0][8]
    keep = last.clone()
    X = bigram_embed(_i32([5, 6], device), emb.to(device), 1.0, None, 1, 0, 0, last,
                     _i32([-1, -1], device), None, 2, _i32([0, 0], device), 1)
    assert np.allclose(_np(X[:, 0]), _np(emb[[5, 6]]), atol=1e-6) and torch.equal(keep, last)


def case_route(device, dtype):
    """The router against the plain rule, token by token: softmax scores, a correction that
    decides the choice but not the weights (also one that makes every choice score negative),
    groups scored by their best member, identity outputs, the shared expert's gate; up to 64
    outputs (lane-parallel ranking) and above."""
    from enterprise_inference_amd.ops import moe
    g = torch.Generator().manual_seed(3)
    for E, ident, k, cnt, keep, cmean in ((8, 2, 2, 2, 1, 0.0), (8, 2, 3, 4, 2, -3.0),
                                          (5, 0, 2, 1, 1, 0.0), (8, 4, 4, 4, 2, 0.5),
                                          (72, 8, 6, 8, 3, -1.0), (4, 1, 1, 2, 1, 0.0)):
        Hd, T = 40, 33
        x = torch.randn(T, Hd, generator=g).to(dtype)
        wr = (torch.randn(E, Hd, generator=g) * 0.4).to(dtype)
        wsg = (torch.randn(1, Hd, generator=g) * 0.3).to(dtype)
        corr = cmean + torch.randn(E, generator=g) * 0.2
        w, ids, iw, sg = moe.route_grouped(x.to(device), wr.to(device), k, cnt, keep, 1.0,
                                           scoring="softmax", group_score="max",
                                           correction=corr.to(device), identity=ident,
                                           gate_w=wsg.to(device))
        groups = {"count": cnt, "keep": keep} if cnt > 1 else None
        checked = 0
        for t in range(T):
            z = _np(wr) @ _np(x[t])
            s = np.exp(z - z.max()) / np.exp(z - z.max()).sum()
            c = np.sort(s + _np(corr))
            if np.min(np.diff(c)) < 1e-4:            # no verdict on a close call
                continue
            want = O.route(z, _np(corr), k, groups, E)
            assert [e for e, _ in want] == ids[t].tolist(), (E, t)
            assert np.allclose([v for _, v in want], _np(w[t]), atol=2e-6), (E, t)
            if ident:
                assert abs(sum(v for e, v in want if e >= E - ident) - float(iw[t])) < 2e-6
            assert abs(float(O.sigmoid(_np(wsg[0]) @ _np(x[t]))) - float(sg[t])) < 1e-5
            checked += 1
        assert checked > T // 2
        if not ident:
            assert iw is None


def _force_chunked(on):
    """Tests that hand a chunk list over want the chunk-parallel form whatever the cost rule says."""
    from enterprise_inference_amd.ops import linear_scan as ls
    ls.FORCE_CHUNKED = bool(on)


def _scan_inputs(g, T, H, D, Dv, dtype, gates):
    width = 2 * H * D + 2 * H * Dv + (2 * H if gates else 0) + 3
    fused = torch.randn(T, width, generator=g)
    if gates:
        fused[:, -2 * H - 3:-3] *= 6.0                 # pre-activations that reach the soft cap
    return fused.to(dtype)


def _scan_offsets(H, D, Dv):
    return 0, H * D, 2 * H * D, 2 * H * D + H * Dv, 2 * H * D + 2 * H * Dv, \
        2 * H * D + 2 * H * Dv + H


def case_retention_scan(device, dtype, H=3, D=10, Dv=6, dims=4, half=True, T=75, chunked=False):
    """The fixed-decay recurrence alone: a sequence run whole, and run in portions (down to one
    token) beside another sequence on slots that held something else before; one early token is
    made to stand out so that a slow head still shows it 70 tokens later.  ``chunked``: long
    portions take the chunk-parallel form (their chunk list is handed over), short ones the
    token-by-token form, on the same slots."""
    from enterprise_inference_amd.ops import linear_scan as ls
    from enterprise_inference_amd.ops.rotary import rotary_frequencies
    g = torch.Generator().manual_seed(11)
    decay = [0.999, 0.9, 0.5, 0.97][:H] + [0.8] * max(0, H - 4)
    inv_freq, _ = rotary_frequencies(dims, 300.0, None)
    rot = {"base": 300.0, "dims": dims} if dims else None
    spec = ls.ScanSpec(H, D, Dv, "decay", decay=torch.tensor(decay).to(device),
                       inv_freq=inv_freq.to(device), rot_dims=dims, rot_half=half,
                       kscale=D ** -0.5, gate_act="silu", out_scale=1.3, eps=1e-5)
    fused = _scan_inputs(g, T, H, D, Dv, torch.float32, False)
    qo, ko, vo, go, _, _ = _scan_offsets(H, D, Dv)
    fused[3, ko:ko + D] *= 30.0                        # head 0's key at position 3 stands out
    fused[3, vo:vo + Dv] += 4.0
    fused = fused.to(dtype)
    f64 = _np(fused)
    want = np.zeros((T, H * Dv))
    S = [np.zeros((D, Dv)) for _ in range(H)]
    for t in range(T):
        for a in range(H):
            q = O.rotate(f64[t, qo + a * D:qo + (a + 1) * D], t, rot, not half)
            k = O.rotate(f64[t, ko + a * D:ko + (a + 1) * D], t, rot, not half) * D ** -0.5
            o, S[a] = O.retention_core(q, k, f64[t, vo + a * Dv:vo + (a + 1) * Dv], decay[a], S[a])
            want[t, a * Dv:(a + 1) * Dv] = O.rms(o, 1e-5)
        want[t] *= O.silu(f64[t, go:go + H * Dv]) * 1.3
    state = ls.ScanState.allocate(3, spec, device)
    state.S.fill_(5.0)                                 # stale slots
    fd = fused.to(device)
    _force_chunked(chunked)

    def run(chunks):
        """chunks: (slot, lo, hi) of the one sequence, each as its own step."""
        out = []
        for sl, lo, hi in chunks:
            other = fd[:2] * 0.5                       # a second sequence beside it, slot 0
            rows = torch.cat([other, fd[lo:hi]])
            pos = _i32([0, 1] + list(range(lo, hi)), device)
            plan = ls.chunk_plan([2, hi - lo], device) if chunked else None
            y = ls.linear_scan(rows, qo, ko, vo, go, spec, state, _i32([0, sl], device),
                               _i32([0, 2, 2 + hi - lo], device), 2, pos, plan=plan)
            out.append(y[2:])
        return torch.cat(out)

    tk = ktol(dtype) * 4
    got = run([(1, 0, T)])
    assert np.allclose(_np(got), want, atol=tk, rtol=tk), np.abs(_np(got) - want).max()
    cuts = [c for c in (0, 2, 3, 19, 20, 36, 37, 39, 70) if c < T] + [T]
    got = run([(2, a, b) for a, b in zip(cuts[:-1], cuts[1:])])
    assert np.allclose(_np(got), want, atol=tk, rtol=tk), np.abs(_np(got) - want).max()
    if chunked and T > 130:                            # long portions that start from a held state
        got = run([(2, 0, 65), (2, 65, 66), (2, 66, T)])
        assert np.allclose(_np(got), want, atol=tk, rtol=tk), np.abs(_np(got) - want).max()
    _force_chunked(False)
    # pure decode rows (no row ranges): slot 1 still holds the state after T tokens
    y = ls.linear_scan(fd[T - 1:T], qo, ko, vo, go, spec, state, _i32([1], device), None, 1,
                       _i32([T], device), _i32([T + 1], device))
    assert y.shape == (1, H * Dv) and bool(torch.isfinite(y.float()).all())


def case_memory_scan(device, dtype, H=2, D=6, Dv=10, T=70, cap=8.0, chunked=False):
    """The gated matrix memory alone: whole against portions on stale slots; gate
    pre-activations large enough to reach the soft cap, so the running maximum moves and the
    normaliser's two branches (|n . q| and exp(-m)) are both taken."""
    from enterprise_inference_amd.ops import linear_scan as ls
    g = torch.Generator().manual_seed(12)
    spec = ls.ScanSpec(H, D, Dv, "exp_gates", cap=cap, qscale=D ** -0.5, gate_act="sigmoid",
                       out_scale=0.9, eps=1e-5)
    fused = _scan_inputs(g, T, H, D, Dv, dtype, True)
    qo, ko, vo, go, io, fo = _scan_offsets(H, D, Dv)
    nw = (1 + 0.2 * torch.randn(H * Dv, generator=g)).to(dtype)
    f64 = _np(fused)
    want = np.zeros((T, H * Dv))
    st = [(np.zeros((D, Dv)), np.zeros(D), 0.0) for _ in range(H)]
    branch = [0, 0]
    for t in range(T):
        for a in range(H):
            gi = cap * math.tanh(f64[t, io + a] / cap)
            gf = O.logsigmoid(cap * math.tanh(f64[t, fo + a] / cap))
            q = f64[t, qo + a * D:qo + (a + 1) * D] * D ** -0.5
            o, st[a] = O.matrix_memory_core(q, f64[t, ko + a * D:ko + (a + 1) * D],
                                            f64[t, vo + a * Dv:vo + (a + 1) * Dv], gi, gf, st[a])
            branch[int(abs(st[a][1] @ q) > math.exp(-st[a][2]))] += 1
            want[t, a * Dv:(a + 1) * Dv] = O.rms(o, 1e-5)
        want[t] *= _np(nw) * O.sigmoid(f64[t, go:go + H * Dv]) * 0.9
    assert min(branch) > 0
    state = ls.ScanState.allocate(2, spec, device)
    state.S.fill_(3.0)
    state.n.fill_(-2.0)
    state.m.fill_(4.0)
    fd = fused.to(device)
    _force_chunked(chunked)

    def run(slot, cuts):
        out = []
        for lo, hi in zip(cuts[:-1], cuts[1:]):
            plan = ls.chunk_plan([hi - lo], device) if chunked else None
            out.append(ls.linear_scan(fd[lo:hi], qo, ko, vo, go, spec, state, _i32([slot], device),
                                      _i32([0, hi - lo], device), 1,
                                      _i32(list(range(lo, hi)), device), None, nw.to(device),
                                      io, fo, plan=plan))
        return torch.cat(out)

    tk = ktol(dtype) * 4
    got = run(0, [0, T])
    assert np.allclose(_np(got), want, atol=tk, rtol=tk), np.abs(_np(got) - want).max()
    got = run(1, [c for c in (0, 1, 3, 18, 19, 35, 52, 53) if c < T] + [T])
    assert np.allclose(_np(got), want, atol=tk, rtol=tk), np.abs(_np(got) - want).max()
    if chunked and T > 130:
        got = run(0, [0, 65, 66, T])
        assert np.allclose(_np(got), want, atol=tk, rtol=tk), np.abs(_np(got) - want).max()
    _force_chunked(False)


def case_sink_needle(device, dtype, H=4, G=2, D=16, Dv=8, n=150, bs=16, size=0):
    """Softmax attention with a sink and one key made to stand out: the query at position i and
    the key at position j share a large component.  j runs over far keys, page borders, the first
    tokens and the query itself (and a window's edges when there is one); i is read as a prefill
    row and as a decode row; sinks of +3 and -2 (one large enough to take most of the weight)."""
    from enterprise_inference_amd.ops import window_attention as wa
    g = torch.Generator().manual_seed(5)
    table, slots, nblk = _paged(n, bs, 6)
    i = n - 7
    sink = torch.tensor([3.0, -2.0, 0.5, 6.0] * 8)[:H]
    spec = wa.WindowSpec(H, G, 1, D, Dv, size, 0, mult=torch.full((H,), 0.3).to(device),
                         sink=sink.float().to(device), post=1.2)
    edge = i - size + 1 if size else 0
    cand = {0, 1, 2, n // 3, i, i - 1, (i // bs) * bs, (i // bs) * bs - 1, bs - 1, bs,
            edge, edge - 1, edge + 1}
    for j in sorted(c for c in cand if 0 <= c <= i):
        q = torch.randn(n, H, D, generator=g) * 0.5
        k = torch.randn(n, G, D, generator=g) * 0.5
        v = torch.randn(n, G, Dv, generator=g)
        u = torch.zeros(D)
        u[j % D] = 1.0
        q[i] += 6.0 * u
        k[j] += 6.0 * u
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
        for r, p in enumerate(pos):
            lo = max(0, p - size + 1) if size else 0
            for a in range(H):
                kv = a // (H // G)
                want = 1.2 * O.sink_attention_core(
                    _np(q[p, a]), [_np(k[t, kv]) for t in range(lo, p + 1)],
                    [_np(v[t, kv]) for t in range(lo, p + 1)], 0.3, float(sink[a]))
                d = np.abs(_np(got[r, a * Dv:(a + 1) * Dv]) - want).max()
                assert d < (2e-4 if dtype == torch.float32 else 4e-2), (j, p, a, d)


def case_expert_block(device, dtype, W=46, ff=20, E=6, ident=2, top=3, cnt=4, keep=2, shared=12,
                      T=21):
    """The whole expert block (router, gated experts, identity outputs, gated shared expert,
    final sum) against the plain rule, at sizes that take the per-expert, the grouped
    weight-streaming and the grouped matrix-core forms; corrections 1.5 apart so that no choice
    rests on a close call."""
    from enterprise_inference_amd.models.mixtral import GroupLimitedMoE
    g = torch.Generator().manual_seed(17)
    mlp = {"expert": {"ff": ff}, "router": {"experts": E, "identity": ident, "top": top,
                                            "groups": {"count": cnt, "keep": keep}}}
    if shared:
        mlp["shared"] = {"ff": shared}
    Wt = {}
    mat = lambda n, k, s=1.0: (torch.randn(n, k, generator=g) * (s / k ** 0.5)).to(dtype).float()
    Wt["router"] = mat(E + ident, W, 1.5)
    Wt["correction"] = (torch.randperm(E + ident, generator=g).float() * 1.5).to(dtype).float()
    for e in range(E):
        Wt[f"e{e}.gate"], Wt[f"e{e}.up"], Wt[f"e{e}.down"] = mat(ff, W, 1.5), mat(ff, W, 1.5), \
            mat(W, ff, 0.7)
    if shared:
        Wt["shared.gate"], Wt["shared.up"] = mat(shared, W, 1.5), mat(shared, W, 1.5)
        Wt["shared.down"], Wt["shared.sg"] = mat(W, shared, 0.7), mat(1, W, 2.0)
    mod = GroupLimitedMoE(W, ff, E, top, cnt, keep, ident, shared, dtype=dtype,
                          device=torch.device(device))
    with torch.no_grad():
        mod.router.copy_(Wt["router"])
        mod.correction.copy_(Wt["correction"])
        for e in range(E):
            mod.w13[e, :ff].copy_(Wt[f"e{e}.gate"])
            mod.w13[e, ff:].copy_(Wt[f"e{e}.up"])
            mod.w2[e].copy_(Wt[f"e{e}.down"])
        if shared:
            mod.shared.gate_up_proj.weight[:shared].copy_(Wt["shared.gate"])
            mod.shared.gate_up_proj.weight[shared:].copy_(Wt["shared.up"])
            mod.shared.down_proj.weight.copy_(Wt["shared.down"])
            mod.shared_gate.copy_(Wt["shared.sg"].reshape(-1))
    mod.refresh()
    x = torch.randn(T, W, generator=g).to(dtype)
    with torch.no_grad():
        got = mod(x.to(device))
    W64 = {k: _np(v) for k, v in Wt.items()}
    want = np.stack([O.moe(_np(x[t]), W64, "", mlp) for t in range(T)])
    err = np.abs(_np(got) - want).max() / np.abs(want).max()
    assert err < (1e-4 if dtype == torch.float32 else 3e-2), (W, ff, T, err)


def case_frequencies():
    """Position interpolation with a lone factor divides every frequency."""
    from enterprise_inference_amd.ops.rotary import rotary_frequencies
    for dims, base, factor in ((6, 5000.0, 4.0), (32, 1e6, 2.0), (2, 10.0, 1.0)):
        rot = {"base": base, "dims": dims, "scaling": {"factor": factor}}
        f, amp = rotary_frequencies(dims, base, rot["scaling"])
        assert amp == 1.0 and np.allclose(_np(f), O.frequencies(rot), rtol=1e-6)
    f, _ = rotary_frequencies(8, 100.0, None)
    assert np.allclose(_np(f), O.frequencies({"base": 100.0, "dims": 8}), rtol=1e-6)


# ------------------------------------------------------------------ whole models
def case_layers(device, dtype, cfg_fn=C.config_a):
    """The sum of the residual streams after every layer."""
    cfg = cfg_fn()
    W = _weights(cfg, 9, dtype)
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
    and mixed batches with reuse of pages and state slots all give the oracle's logits."""
    cfg = cfg_fn()
    W = _weights(cfg, seed, dtype)
    V = cfg["vocab"]
    reqs = {"a": _tokens(70, V, 11), "b": _tokens(37, V, 12), "c": _tokens(5, V, 13),
            "d": _tokens(1, V, 14), "e": _tokens(49, V, 15)}
    want = {k: C.oracle_logits(cfg, W, t) for k, t in reqs.items()}
    # pool of 8 pages (of 16 tokens: "a" alone needs 5) and two slots: both are used again
    sess = C.make_session(cfg, W, device, dtype, max_tokens=8 * block_size, block_size=block_size,
                          max_live=2)
    try:
        for k, t in reqs.items():
            got = sess.step([{"id": k, "tokens": t, "want": list(range(len(t)))}], end=[k])
            _check(got, want[k], dtype, ("whole", k))
        # a prompt portion, then token by token
        for k in ("a", "b"):
            t = reqs[k]
            n0 = len(t) - 34
            got = [sess.step([{"id": k, "tokens": t[:n0], "want": [n0 - 1]}])]
            for i in range(n0, len(t)):
                got.append(sess.step([{"id": k, "tokens": [t[i]], "want": [0]}],
                                     end=[k] if i == len(t) - 1 else []))
            _check(torch.cat(got), want[k][n0 - 1:], dtype, ("decode", k))
        # portions: sizes cross page borders (16) and scan chunks and go down to two tokens
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
    # prompt portions, requests that pause, pages and slots freed and taken again
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
        run([("b", 1), ("c", 3), ("a", 20)], end=["c"])           # c finishes: page and slot free
        run([("a", 1), ("e", 30), ("b", 17)])                     # e takes them
        run([("e", 1), ("b", 16), ("a", 2)], end=["b"])
        run([("a", 47)], end=["a"])                               # e pauses
        run([("e", 18)], end=["e"])
        for k in reqs:
            assert at[k] == len(reqs[k])
            _check(torch.cat(got[k]), want[k], dtype, ("mixed", k))
        # a second life for a finished request's name, on reused pages and slots
        got2 = sess.step([{"id": "b", "tokens": reqs["b"], "want": list(range(len(reqs["b"])))},
                          {"id": "c", "tokens": reqs["c"], "want": [4]}], end=["b", "c"])
        _check(got2[:-1], want["b"], dtype, "again b")
        _check(got2[-1:], want["c"][4:], dtype, "again c")
        bm = sess.scheduler.bm
        assert bm.num_free_blocks() == bm.num_blocks and bm.slots.num_free() == 4
    finally:
        sess.close()


def case_long_decode(device, dtype, cfg_fn=C.config_b):
    """140 tokens decoded one by one after a 3-token prompt, over many page borders."""
    cfg = cfg_fn()
    W = _weights(cfg, 3, dtype)
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
    W = _weights(cfg, 5, dtype)
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
