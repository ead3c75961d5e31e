"""Plain float64 implementation of the Daburax design, written from its equations: loops over
tokens, heads and keys, one function per mechanism, no code shared with the framework.

Embedding: ``embed[tok] * scale`` plus a row of a bigram table chosen by a hash of (previous
token, token).  The residual is kept as several streams joined by hyper-connections (read
weights, a stream-mixing matrix, write weights per sublayer).  Mixers: ``retention`` (rotated
q / k, a fixed decay per head, matrix state, head RMS norm, SiLU gate) and ``parallel`` (a
grouped-query softmax attention with biases, partial interleaved rotation with linearly scaled
frequencies and a sink in the denominator, beside a gated matrix memory with a stabilised
exponential input gate; the two outputs are added with fixed factors).  Feed-forward: a mixture
of SiLU-gated experts behind a softmax router with a selection-only correction, a group limit,
identity experts and a sigmoid-gated shared expert.  ``W`` maps the checkpoint's tensor names to
float64 arrays.
"""

from __future__ import annotations

import math

import numpy as np


def rms(x, eps):
    return x / math.sqrt(float(np.mean(x * x)) + eps)


def norm(x, w, eps):
    """Weights are stored around zero."""
    return rms(x, eps) * (1.0 + w)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def logsigmoid(z):
    return -(math.log1p(math.exp(-abs(z))) + max(-z, 0.0))


def bigram_row(prev, tok, bg):
    """Row of the bigram table for a token and its predecessor (None: the sequence starts)."""
    n = int(bg["buckets"])
    if prev is None:
        return n
    return (int(prev) * int(bg["mul_prev"]) + int(tok) * int(bg["mul_cur"])) % n


def embed_tokens(cfg, W, tokens):
    e = cfg.get("embedding") or {}
    scale = float(e.get("scale", 1.0))
    out = []
    for t, tok in enumerate(tokens):
        x = W["embed"][tok] * scale
        if e.get("bigram"):
            x = x + W["bigram"][bigram_row(tokens[t - 1] if t else None, tok, e["bigram"])]
        out.append(x)
    return out


def frequencies(rot):
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if sc:
        f = [v / float(sc["factor"]) for v in f]
    return f


def rotate(v, pos, rot, interleaved):
    """Turns the first rot.dims entries of one head by the position; pairs are (2i, 2i+1) when
    interleaved, else (i, i + dims/2)."""
    if not rot or not int(rot.get("dims", 0)):
        return v
    dims = int(rot["dims"])
    out = v.copy()
    for i, f in enumerate(frequencies(rot)):
        a, b = (2 * i, 2 * i + 1) if interleaved else (i, i + dims // 2)
        c, s = math.cos(pos * f), math.sin(pos * f)
        out[a] = v[a] * c - v[b] * s
        out[b] = v[b] * c + v[a] * s
    return out


# ------------------------------------------------------------------ retention

def retention_core(q, k, v, decay, S):
    """One token of one head: S <- decay S + k v^T; returns (S^T q, S)."""
    S = decay * S + np.outer(k, v)
    return S.T @ q, S


def retention_mixer(hs, W, pre, m, eps):
    """hs: the mixer inputs of one sequence, token by token -> outputs."""
    H, D, Dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    S = [np.zeros((D, Dv)) for _ in range(H)]
    out = []
    for t, h in enumerate(hs):
        q = (W[pre + "q"] @ h).reshape(H, D)
        k = (W[pre + "k"] @ h).reshape(H, D)
        v = (W[pre + "v"] @ h).reshape(H, Dv)
        o = np.zeros((H, Dv))
        for a in range(H):
            qa = rotate(q[a], t, m.get("rot"), False)
            ka = rotate(k[a], t, m.get("rot"), False) * D ** -0.5
            oa, S[a] = retention_core(qa, ka, v[a], float(m["decay"][a]), S[a])
            o[a] = rms(oa, eps)
        out.append(W[pre + "o"] @ (o.reshape(-1) * silu(W[pre + "g"] @ h)))
    return out


# ------------------------------------------------------------------ attention with a sink

def sink_attention_core(q, keys, vals, scale, sink):
    """One query of one head over its visible keys; exp(sink) joins the denominator only."""
    s = np.array([float(q @ k) * scale for k in keys])
    mx = max(float(s.max()), sink)
    p = np.exp(s - mx)
    den = float(p.sum()) + math.exp(sink - mx)
    return sum(pj * vj for pj, vj in zip(p, vals)) / den


def sink_attention_mixer(hs, W, pre, m):
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    keys, vals, out = [], [], []
    for t, h in enumerate(hs):
        q = (W[pre + "q"] @ h + W[pre + "q.b"]).reshape(H, D)
        k = (W[pre + "k"] @ h + W[pre + "k.b"]).reshape(G, D)
        v = (W[pre + "v"] @ h + W[pre + "v.b"]).reshape(G, Dv)
        keys.append([rotate(k[g], t, m.get("rot"), True) for g in range(G)])
        vals.append(v)
        o = np.zeros((H, Dv))
        for a in range(H):
            g = a // (H // G)
            o[a] = sink_attention_core(rotate(q[a], t, m.get("rot"), True),
                                       [kk[g] for kk in keys], [vv[g] for vv in vals],
                                       float(m["scale"]), float(W[pre + "sink"][a]))
        out.append(W[pre + "o"] @ o.reshape(-1))
    return out


# ------------------------------------------------------------------ gated matrix memory

def matrix_memory_core(q, k, v, i_log, f_log, state):
    """One token of one head.  state = (S, n, m); m is the running maximum of the log gates
    (starts at 0)."""
    S, n, m = state
    m_new = max(f_log + m, i_log)
    a, b = math.exp(f_log + m - m_new), math.exp(i_log - m_new)
    S = a * S + b * np.outer(k, v)
    n = a * n + b * k
    den = max(abs(float(n @ q)), math.exp(-m_new)) + 1e-6
    return S.T @ q / den, (S, n, m_new)


def matrix_memory_mixer(hs, W, pre, m, eps):
    H, D, Dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    cap = float(m["gate_cap"])
    st = [(np.zeros((D, Dv)), np.zeros(D), 0.0) for _ in range(H)]
    out = []
    for h in hs:
        q = (W[pre + "q"] @ h).reshape(H, D) * D ** -0.5
        k = (W[pre + "k"] @ h).reshape(H, D)
        v = (W[pre + "v"] @ h).reshape(H, Dv)
        gi = cap * np.tanh((W[pre + "i"] @ h + W[pre + "i.b"]) / cap)
        gf = cap * np.tanh((W[pre + "f"] @ h + W[pre + "f.b"]) / cap)
        o = np.zeros((H, Dv))
        for a in range(H):
            oa, st[a] = matrix_memory_core(q[a], k[a], v[a], float(gi[a]),
                                           logsigmoid(float(gf[a])), st[a])
            o[a] = rms(oa, eps)
        out.append(W[pre + "o"] @ (o.reshape(-1) * W[pre + "norm"] * sigmoid(W[pre + "g"] @ h)))
    return out


def parallel_mixer(hs, W, pre, m, eps):
    left = sink_attention_mixer(hs, W, pre + "left.", m["left"])
    right = matrix_memory_mixer(hs, W, pre + "right.", m["right"], eps)
    return [float(m["left_scale"]) * a + float(m["right_scale"]) * b for a, b in zip(left, right)]


# ------------------------------------------------------------------ feed-forward

def route(z, correction, top, groups, n_out):
    """Softmax scores; selection by score + correction inside the best groups (a group's score
    is its largest corrected score).  -> [(output index, weight)]."""
    z = z - z.max()
    s = np.exp(z) / np.exp(z).sum()
    c = s + correction
    ok = np.ones(n_out, dtype=bool)
    if groups and int(groups.get("count", 1)) > 1:
        cnt, keep = int(groups["count"]), int(groups["keep"])
        per = n_out // cnt
        gs = [max(c[g * per:(g + 1) * per]) for g in range(cnt)]
        best = sorted(range(cnt), key=lambda g: -gs[g])[:keep]
        ok[:] = False
        for g in best:
            ok[g * per:(g + 1) * per] = True
    order = sorted([e for e in range(n_out) if ok[e]], key=lambda e: -c[e])[:top]
    return [(e, float(s[e])) for e in order]


def gated_expert(h, W, pre):
    return W[pre + "down"] @ (silu(W[pre + "gate"] @ h) * (W[pre + "up"] @ h))


def moe(h, W, pre, mlp):
    r = mlp["router"]
    E, ident = int(r["experts"]), int(r.get("identity", 0))
    corr = W.get(pre + "correction")
    if corr is None:
        corr = np.zeros(E + ident)
    y = np.zeros_like(h)
    for e, w in route(W[pre + "router"] @ h, corr, int(r["top"]), r.get("groups"), E + ident):
        y += w * (h if e >= E else gated_expert(h, W, f"{pre}e{e}."))
    if mlp.get("shared"):
        y += float(sigmoid(W[pre + "shared.sg"] @ h)[0]) * gated_expert(h, W, pre + "shared.")
    return y


# ------------------------------------------------------------------ layers

def mixer(hs, W, pre, L, eps):
    if L["type"] == "retention":
        return retention_mixer(hs, W, pre, L["mixer"], eps)
    if L["type"] == "parallel":
        return parallel_mixer(hs, W, pre, L["mixer"], eps)
    raise ValueError(L["type"])


def forward(cfg, W, tokens, collect=None):
    """Logits [tokens, vocab] of one sequence.  ``collect`` receives the residual (the sum of
    the streams) after every layer, [tokens, width] each."""
    eps = float(cfg["norm"]["eps"])
    mult = float(cfg.get("residual_mult", 1.0))
    ns = cfg.get("streams")
    T = len(tokens)
    x0 = embed_tokens(cfg, W, tokens)
    X = [[x.copy() for _ in range(int(ns))] for x in x0] if ns else [[x] for x in x0]

    def sublayer(q, p, fn):
        if ns:
            hin = [sum(W[f"{p}hc{q}.in"][s] * X[t][s] for s in range(ns)) for t in range(T)]
        else:
            hin = [X[t][0] for t in range(T)]
        ys = fn([norm(u, W[f"{p}norm{q}"], eps) for u in hin])
        for t in range(T):
            if ns:
                mixm, outw = W[f"{p}hc{q}.mix"], W[f"{p}hc{q}.out"]
                X[t] = [sum(mixm[s, j] * X[t][s] for s in range(ns)) + mult * outw[j] * ys[t]
                        for j in range(ns)]
            else:
                X[t] = [X[t][0] + mult * ys[t]]

    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        sublayer(1, p, lambda hs: mixer(hs, W, p + "mix.", L, eps))
        if L.get("mlp"):
            sublayer(2, p, lambda hs: [moe(h, W, p + "mlp.", L["mlp"]) for h in hs])
        if collect is not None:
            collect.append(np.stack([sum(X[t]) for t in range(T)]))
    return np.stack([W["head"] @ norm(sum(X[t]), W["final.norm"], eps) for t in range(T)])
