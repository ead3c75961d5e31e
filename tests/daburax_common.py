"""Shared pieces of the Daburax tests: small configurations, random checkpoints under the design's
tensor names and a session that drives the engine (scheduler bookkeeping, model runner, kernels)
step by step.  The expected values come from tests/oracles/daburax_oracle.py only."""

from __future__ import annotations

import copy

import torch

from oracles import daburax_oracle as O


def ret(heads=3, dim=10, vdim=6, decay=(0.9, 0.97, 0.5), dims=4, base=1000.0):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}
    if dims:
        m["rot"] = {"base": base, "dims": dims}
    return {"type": "retention", "mixer": m}


def par(lh=4, lg=2, ld=12, lv=8, ldims=6, lbase=5000.0, factor=4.0, lscale=0.3,
        rh=2, rd=6, rv=10, cap=8.0, ls=0.8, rs=1.3):
    left = {"heads": lh, "kv_heads": lg, "dim": ld, "vdim": lv, "scale": lscale}
    if ldims:
        left["rot"] = {"base": lbase, "dims": ldims}
        if factor:
            left["rot"]["scaling"] = {"factor": factor}
    right = {"heads": rh, "dim": rd, "vdim": rv, "gate_cap": cap}
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": ls,
                                          "right_scale": rs}}


def moe(layer, experts=6, top=3, identity=2, count=4, keep=2, ff=20, shared=12):
    layer = dict(layer)
    if not experts:
        layer["mlp"] = None
        return layer
    r = {"experts": experts, "top": top}
    if identity:
        r["identity"] = identity
    if count:
        r["groups"] = {"count": count, "keep": keep}
    layer["mlp"] = {"kind": "moe", "expert": {"ff": ff}, "router": r}
    if shared:
        layer["mlp"]["shared"] = {"ff": shared}
    return layer


def config_a():
    """Odd sizes: two streams, a width that is no multiple of four, rotation on part of a head,
    key / value sizes that differ, three heads with three decays, two of four groups kept, two
    identity experts among eight outputs, a layer without feed-forward, a feed-forward without
    groups, identity or shared expert."""
    return {"architecture": "Daburax", "vocab": 90, "width": 46, "norm": {"eps": 1e-5},
            "residual_mult": 0.7, "streams": 2,
            "embedding": {"scale": 2.5, "bigram": {"buckets": 37, "mul_prev": 5, "mul_cur": 3}},
            "layers": [moe(ret()),
                       moe(par(), experts=0),
                       moe(ret(heads=1, dim=8, vdim=8, decay=(0.8,), dims=8), experts=5, top=2,
                           identity=0, count=0, shared=0),
                       moe(par(lh=3, lg=3, ld=8, lv=10, ldims=8, factor=0, rh=3, rd=10, rv=4,
                               cap=5.0, ls=1.1, rs=0.6), experts=3, top=2, identity=1, count=2,
                           keep=1, ff=16, shared=24)]}


def config_b():
    """The plain residual sum (no streams), no bigram term, no embedding scale, no residual
    factor; a parallel layer first; one attention head, no rotation in one left mixer, one
    recurrent head; a retention layer without rotation; one group (no limit); top 1."""
    return {"architecture": "Daburax", "vocab": 70, "width": 40, "norm": {"eps": 1e-6},
            "layers": [moe(par(lh=1, lg=1, ld=16, lv=16, ldims=16, factor=2.0, lscale=0.2, rh=1,
                               rd=12, rv=12, cap=15.0, ls=1.0, rs=1.0), experts=4, top=1,
                           identity=0, count=1, keep=1, ff=24, shared=8),
                       moe(ret(heads=2, dim=6, vdim=12, decay=(0.99, 0.6), dims=0), experts=0),
                       moe(par(lh=6, lg=2, ld=8, lv=6, ldims=0, rh=2, rd=4, rv=6, cap=3.0,
                               ls=0.5, rs=2.0), experts=2, top=2, identity=2, count=2, keep=2,
                           ff=12, shared=0)]}


def config_c():
    """Sizes in multiples of the matrix-core tiles, four streams, heads of 32 .. 64 with value
    sizes that differ from the key sizes, expert sizes that take the grouped expert kernels."""
    return {"architecture": "Daburax", "vocab": 160, "width": 128, "norm": {"eps": 1e-5},
            "residual_mult": 0.6, "streams": 4,
            "embedding": {"scale": 4.0, "bigram": {"buckets": 101, "mul_prev": 13, "mul_cur": 29}},
            "layers": [moe(par(lh=4, lg=2, ld=32, lv=64, ldims=16, lbase=20000.0, factor=2.0,
                               lscale=0.15, rh=2, rd=64, rv=32, cap=10.0, ls=1.2, rs=0.9),
                           experts=6, top=2, identity=2, count=2, keep=1, ff=128, shared=64),
                       moe(ret(heads=2, dim=32, vdim=64, decay=(0.95, 0.999), dims=32,
                               base=100000.0), experts=4, top=2, identity=0, count=2, keep=2,
                           ff=64, shared=128),
                       moe(par(lh=8, lg=1, ld=64, lv=16, ldims=64, factor=0, lscale=0.1, rh=4,
                               rd=32, rv=32, cap=11.0, ls=0.7, rs=1.4), experts=0)]}


def config_d():
    """One learned stream; an attention side whose sizes take the matrix-core form beside a
    recurrent side of odd width (3 heads of 5), so the shared row of the two needs padding; a
    retention layer whose rotation covers part of a 24-wide head."""
    return {"architecture": "Daburax", "vocab": 80, "width": 64, "norm": {"eps": 1e-5},
            "residual_mult": 1.5, "streams": 1, "embedding": {"scale": 0.5},
            "layers": [moe(par(lh=2, lg=1, ld=16, lv=16, ldims=8, lbase=300.0, factor=3.0,
                               lscale=0.25, rh=3, rd=8, rv=5, cap=6.0, ls=0.9, rs=1.1),
                           experts=4, top=2, identity=0, count=2, keep=2, ff=16, shared=16),
                       moe(ret(heads=2, dim=24, vdim=16, decay=(0.9, 0.99), dims=10), experts=0)]}


def random_weights(cfg: dict, seed: int = 0, dtype=torch.float32, decisive: bool = False,
                   tie_qk: bool = False) -> dict:
    """A checkpoint for ``cfg`` under the design's tensor names (values rounded to ``dtype``).
    ``decisive``: router corrections 1.5 apart, so no expert choice rests on a close call of the
    scores (which lie in [0, 1]); ``tie_qk``: W_k = W_q in the recurrent mixers, so a first
    token's q . k is a square and the sign of its output survives 16-bit rounding."""
    g = torch.Generator().manual_seed(seed)
    W = {}

    def mat(n, k, s=1.0):
        return torch.randn(n, k, generator=g) * (s / k ** 0.5)

    def vec(n, mean=0.0, s=0.2):
        return mean + torch.randn(n, generator=g) * s

    Wd, V = cfg["width"], cfg["vocab"]
    W["embed"] = torch.randn(V, Wd, generator=g)
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        W["bigram"] = torch.randn(bg["buckets"] + 1, Wd, generator=g) * 0.7
    W["head"] = mat(V, Wd)
    W["final.norm"] = vec(Wd)
    ns = cfg.get("streams")
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        W[p + "norm1"] = vec(Wd)
        subs = [1] + ([2] if L.get("mlp") else [])
        if ns:
            for q in subs:
                W[f"{p}hc{q}.in"] = vec(ns, 1.0 / ns, 0.3)
                W[f"{p}hc{q}.out"] = vec(ns, 1.0, 0.3)
                W[f"{p}hc{q}.mix"] = torch.eye(ns) + torch.randn(ns, ns, generator=g) * 0.2
        if L["type"] == "retention":
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            W[p + "mix.q"], W[p + "mix.k"] = mat(H * D, Wd, 1.5), mat(H * D, Wd, 1.5)
            if tie_qk:
                W[p + "mix.k"] = W[p + "mix.q"].clone()
            W[p + "mix.v"], W[p + "mix.g"] = mat(H * Dv, Wd), mat(H * Dv, Wd, 2.0)
            W[p + "mix.o"] = mat(Wd, H * Dv, 0.7)
        else:
            l, r = m["left"], m["right"]
            H, G, D, Dv = l["heads"], l["kv_heads"], l["dim"], l["vdim"]
            q = p + "mix.left."
            W[q + "q"], W[q + "k"], W[q + "v"] = mat(H * D, Wd, 1.5), mat(G * D, Wd, 1.5), \
                mat(G * Dv, Wd)
            W[q + "q.b"], W[q + "k.b"], W[q + "v.b"] = vec(H * D, 0, 0.3), vec(G * D, 0, 0.3), \
                vec(G * Dv, 0, 0.3)
            W[q + "sink"] = vec(H, 0.5, 1.0)
            W[q + "o"] = mat(Wd, H * Dv, 0.7)
            H, D, Dv = r["heads"], r["dim"], r["vdim"]
            q = p + "mix.right."
            W[q + "q"], W[q + "k"] = mat(H * D, Wd, 1.5), mat(H * D, Wd, 1.5)
            if tie_qk:
                W[q + "k"] = W[q + "q"].clone()
            W[q + "v"], W[q + "g"] = mat(H * Dv, Wd), mat(H * Dv, Wd, 2.0)
            W[q + "i"], W[q + "f"] = mat(H, Wd, 2.0), mat(H, Wd, 2.0)
            W[q + "i.b"], W[q + "f.b"] = vec(H, 0.0, 1.0), vec(H, 2.0, 1.0)
            W[q + "norm"] = vec(H * Dv, 1.0, 0.2)
            W[q + "o"] = mat(Wd, H * Dv, 0.7)
        if L.get("mlp"):
            mlp = L["mlp"]
            r = mlp["router"]
            E, ident, ff = r["experts"], r.get("identity", 0), mlp["expert"]["ff"]
            W[p + "norm2"] = vec(Wd)
            W[p + "mlp.router"] = mat(E + ident, Wd, 1.5)
            if decisive:
                W[p + "mlp.correction"] = torch.randperm(E + ident, generator=g).float() * 1.5
            else:
                W[p + "mlp.correction"] = vec(E + ident, 0.0, 0.15)
            for e in range(E):
                W[f"{p}mlp.e{e}.gate"], W[f"{p}mlp.e{e}.up"] = mat(ff, Wd, 1.5), mat(ff, Wd, 1.5)
                W[f"{p}mlp.e{e}.down"] = mat(Wd, ff, 0.7)
            if mlp.get("shared"):
                sf = mlp["shared"]["ff"]
                W[p + "mlp.shared.gate"], W[p + "mlp.shared.up"] = mat(sf, Wd, 1.5), mat(sf, Wd, 1.5)
                W[p + "mlp.shared.down"] = mat(Wd, sf, 0.7)
                W[p + "mlp.shared.sg"] = mat(1, Wd, 2.0)
    return {k: v.to(dtype).float() for k, v in W.items()}


def as_numpy(W: dict) -> dict:
    return {k: v.double().numpy() for k, v in W.items()}


def oracle_logits(cfg, W, tokens, collect=None):
    return torch.from_numpy(O.forward(cfg, as_numpy(W), list(tokens), collect)).float()


def make_session(cfg: dict, W: dict, device: str, dtype=torch.float32, max_tokens: int = 512,
                 block_size: int = 16, max_live: int = 4):
    """A replay session of the engine holding the checkpoint W."""
    from enterprise_inference_amd.config import ModelConfig
    from enterprise_inference_amd.entrypoints.trace_run import TraceSession, replay_config

    mc = ModelConfig.from_hf_dict(copy.deepcopy(cfg))
    ec = replay_config(mc, None, dtype, device, max_tokens, block_size, max_live,
                       load_format="dummy")
    sess = TraceSession(ec)
    model = sess.runner.model
    model.load_weights(W.items())
    model.post_load()
    return sess


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """Row-wise error as the mean-free RMS difference over the RMS of the expected logits."""
    d = got.double().cpu() - want.double()
    d = d - d.mean(-1, keepdim=True)
    w = want.double() - want.double().mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-9)).max())
