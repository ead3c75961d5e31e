"""Plain float64 implementation of the Gapidra design, written from its equations: loops over
tokens, heads and keys, one function per mechanism, no code shared with the framework.

A layer reads one RMS norm of the stream and adds both sublayers' outputs to it,
``x <- x + mixer(norm1(x)) + ff(norm1(x))``.  Mixers: ``latent_attention`` (keys and values
up-projected from one cached, RMS-normed latent per token plus one rotated key part shared by
the heads; sliding window; a per-head sink in the softmax denominator; element-wise sigmoid
output gate) and ``attention`` (grouped-query heads, RMS norm over the whole query / key
projection, rotation of interleaved pairs with optional frequency interpolation, sliding
window, un-normalised sigmoid weights with a per-head bias).  Feed-forward: ``W_down
xielu(W_up h)``.  ``W`` maps the checkpoint's tensor names to float64 arrays.
"""

from __future__ import annotations

import math

import numpy as np


def rms_norm(x, w, eps):
    return x / math.sqrt(float(np.mean(x * x)) + eps) * w


def softplus(z):
    return math.log1p(math.exp(-abs(z))) + max(z, 0.0)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def xielu(z, p, q):
    """z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2."""
    ap, aq = softplus(p), 0.5 + softplus(q)
    out = np.empty_like(z)
    for i, v in enumerate(z):
        out[i] = ap * v * v + 0.5 * v if v > 0 else aq * (math.exp(v) - 1.0 - v) + 0.5 * v
    return out


def feed_forward(h, W, pre):
    p, q = W[pre + "act"]
    return W[pre + "down"] @ xielu(W[pre + "up"] @ h, float(p), float(q))


def frequencies(rot):
    """(f_i for i < dims/2, factor on cos and sin) of a ``rot`` entry {base, dims, scaling?}."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def turn_dim(t):
        return dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate(v, pos, freqs, amp, dims, interleaved):
    """Turns the first ``dims`` entries of v: pairs (2i, 2i+1) when interleaved, else
    (i, i + dims/2); the rest passes unchanged."""
    out = np.array(v, dtype=np.float64)
    for i in range(dims // 2):
        a, b = (2 * i, 2 * i + 1) if interleaved else (i, i + dims // 2)
        ang = pos * freqs[i]
        c, s = math.cos(ang) * amp, math.sin(ang) * amp
        out[a] = v[a] * c - v[b] * s
        out[b] = v[b] * c + v[a] * s
    return out


def visible(i, window):
    lo = max(0, i - window + 1) if window and window > 0 else 0
    return range(lo, i + 1)


def latent_core(q_plain, q_rot, lat, krot, uk, uv, i, window, scale, sink):
    """Heads [H, Dv] of position i.  q_plain [H, D], q_rot [H, rd] (already rotated); lat[j] the
    normed latent and krot[j] the rotated shared key part of position j; uk [H, D, R], uv
    [H, Dv, R]; sink [H]: one more term exp(sink_h) in head h's denominator."""
    H, Dv = uv.shape[0], uv.shape[1]
    heads = np.zeros((H, Dv))
    js = list(visible(i, window))
    for a in range(H):
        sc = np.array([(q_plain[a] @ (uk[a] @ lat[j]) + q_rot[a] @ krot[j]) * scale for j in js])
        top = max(sc.max(), float(sink[a]))
        e = np.exp(sc - top)
        den = e.sum() + math.exp(float(sink[a]) - top)
        for wgt, j in zip(e / den, js):
            heads[a] += wgt * (uv[a] @ lat[j])
    return heads


def latent_attention(hs, W, pre, m, eps):
    """hs: list of mixer inputs (one per position) -> list of mixer outputs."""
    H, D, rd, R = m["heads"], m["dim"], m["rot_dim"], m["kv_rank"]
    Dv = m.get("vdim", D)
    rot = m.get("rot") or {"dims": rd, "base": 10000.0}
    freqs, amp = frequencies(rot)
    window = (m.get("mask") or {}).get("size", 0)
    lat, krot, qs = [], [], []
    for p, h in enumerate(hs):
        d = W[pre + "dkv"] @ h
        lat.append(rms_norm(d[:R], W[pre + "dkv.norm"], eps))
        krot.append(rotate(d[R:], p, freqs, amp, rot["dims"], False))
        qs.append((W[pre + "q"] @ h).reshape(H, D + rd))
    uk, uv = W[pre + "uk"].reshape(H, D, R), W[pre + "uv"].reshape(H, Dv, R)
    out = []
    for i, h in enumerate(hs):
        qr = np.stack([rotate(qs[i][a, D:], i, freqs, amp, rot["dims"], False) for a in range(H)])
        heads = latent_core(qs[i][:, :D], qr, lat, krot, uk, uv, i, window, m["scale"],
                            W[pre + "sink"])
        gated = heads.reshape(-1) * sigmoid(W[pre + "g"] @ h)
        out.append(W[pre + "o"] @ gated)
    return out


def sigmoid_core(q, ks, vs, i, H, G, window, scale, pb):
    """Heads [H, Dv] of position i: every visible key j weighs sigmoid(q_h . k_j scale + pb_h).
    q [H, D]; ks[j] [G, D]; vs[j] [G, Dv]."""
    heads = np.zeros((H, vs[0].shape[1]))
    for a in range(H):
        b = a // (H // G)
        for j in visible(i, window):
            heads[a] += sigmoid(float(q[a] @ ks[j][b]) * scale + float(pb[a])) * vs[j][b]
    return heads


def sigmoid_attention(hs, W, pre, m, eps):
    H, G, D = m["heads"], m.get("kv_heads", m["heads"]), m["dim"]
    Dv = m.get("vdim", D)
    rot = m.get("rot")
    freqs, amp = frequencies(rot) if rot else ([], 1.0)
    rdims = int(rot["dims"]) if rot else 0
    window = (m.get("mask") or {}).get("size", 0)
    qs, ks, vs = [], [], []
    for p, h in enumerate(hs):
        q = rms_norm(W[pre + "q"] @ h, W[pre + "q.norm"], eps).reshape(H, D)
        k = rms_norm(W[pre + "k"] @ h, W[pre + "k.norm"], eps).reshape(G, D)
        qs.append(np.stack([rotate(q[a], p, freqs, amp, rdims, True) for a in range(H)]))
        ks.append(np.stack([rotate(k[b], p, freqs, amp, rdims, True) for b in range(G)]))
        vs.append((W[pre + "v"] @ h).reshape(G, Dv))
    out = []
    for i in range(len(hs)):
        heads = sigmoid_core(qs[i], ks, vs, i, H, G, window, m["scale"], W[pre + "pb"])
        out.append(W[pre + "o"] @ heads.reshape(-1))
    return out


MIXERS = {"latent_attention": latent_attention, "attention": sigmoid_attention}


def forward(cfg, W, tokens, collect=None):
    """Logits [len(tokens), vocab]; ``collect`` (a list) receives the stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    scale = float((cfg.get("embedding") or {}).get("scale", 1.0))
    xs = [W["embed"][t] * scale for t in tokens]
    for li, L in enumerate(cfg["layers"]):
        pre = f"l{li}."
        hs = [rms_norm(x, W[pre + "norm1"], eps) for x in xs]
        ys = MIXERS[L["type"]](hs, W, pre + "mix.", L["mixer"], eps)
        if L.get("mlp"):
            ys = [y + feed_forward(h, W, pre + "mlp.") for y, h in zip(ys, hs)]
        xs = [x + y for x, y in zip(xs, ys)]
        if collect is not None:
            collect.append(np.stack(xs))
    return np.stack([W["head"] @ rms_norm(x, W["final.norm"], eps) for x in xs])
