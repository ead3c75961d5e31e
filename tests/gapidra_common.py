"""Shared pieces of the Gapidra tests: small configurations, random checkpoints under the design's
tensor names and a session that drives the engine (scheduler bookkeeping, model runner, kernels)
step by step.  The expected values come from tests/oracles/gapidra_oracle.py only."""

from __future__ import annotations

import copy

import torch

from oracles import gapidra_oracle as O


def lat(heads=3, dim=10, rot_dim=6, vdim=14, kv_rank=20, size=9, scale=0.3, base=1000.0,
        dims=None, scaling=None):
    rot = {"base": base, "dims": rot_dim if dims is None else dims}
    if scaling:
        rot["scaling"] = scaling
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
         "scale": scale, "rot": rot}
    if size:
        m["mask"] = {"size": size}
    return {"type": "latent_attention", "mixer": m}


def att(heads=4, kv_heads=2, dim=12, vdim=8, size=7, scale=0.3, base=5000.0, dims=6, scaling=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if dims:
        m["rot"] = {"base": base, "dims": dims}
        if scaling:
            m["rot"]["scaling"] = scaling
    if size:
        m["mask"] = {"size": size}
    return {"type": "attention", "mixer": m}


def with_ff(layer, ff):
    layer = dict(layer)
    layer["mlp"] = {"kind": "dense", "ff": ff} if ff else None
    return layer


YARN = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}


def config_a():
    """Odd sizes: windows shorter than a 16-token page, rotation on part of the rotary entries,
    frequency interpolation in one attention layer, a layer without a feed-forward, one layer
    with a window of one token, a width that is no multiple of four."""
    return {"architecture": "Gapidra", "vocab": 90, "width": 46, "norm": {"eps": 1e-5},
            "embedding": {"scale": 3.0},
            "layers": [with_ff(lat(dims=4), 40),
                       with_ff(att(scaling=YARN), 36),
                       with_ff(att(heads=2, kv_heads=2, dim=8, vdim=10, size=1, dims=8), 0),
                       with_ff(lat(heads=1, dim=6, rot_dim=4, vdim=5, kv_rank=12, size=20,
                                   scale=0.4), 24)]}


def config_b():
    """No embedding scale, no windows at all in two layers (every earlier token is seen), no
    rotation in one attention layer, as many key / value heads as heads, one head, frequency
    interpolation in a latent layer, the attention layers in the middle."""
    return {"architecture": "Gapidra", "vocab": 70, "width": 40, "norm": {"eps": 1e-6},
            "layers": [with_ff(lat(heads=2, dim=8, rot_dim=8, vdim=8, kv_rank=16, size=0,
                                   scaling={"factor": 2.0, "original": 32, "fast": 4.0,
                                            "slow": 0.5}), 0),
                       with_ff(att(heads=3, kv_heads=3, dim=10, vdim=6, size=0, dims=0), 32),
                       with_ff(att(heads=1, kv_heads=1, dim=16, vdim=16, size=400, dims=16,
                                   scale=0.2), 24),
                       with_ff(lat(heads=5, dim=4, rot_dim=2, vdim=6, kv_rank=8, size=3), 16)]}


def config_c():
    """Sizes in multiples of the matrix-core tiles (heads of 32 .. 96, windows that cross several
    pages), value heads wider and narrower than the key heads, an attention layer first."""
    return {"architecture": "Gapidra", "vocab": 160, "width": 128, "norm": {"eps": 1e-5},
            "embedding": {"scale": 0.5},
            "layers": [with_ff(att(heads=4, kv_heads=2, dim=64, vdim=32, size=40, scale=0.12,
                                   dims=32, scaling=YARN), 128),
                       with_ff(lat(heads=4, dim=32, rot_dim=16, vdim=48, kv_rank=64, size=33,
                                   scale=0.15), 128),
                       with_ff(att(heads=8, kv_heads=1, dim=32, vdim=80, size=70, scale=0.18,
                                   dims=8), 0),
                       with_ff(lat(heads=16, dim=16, rot_dim=32, vdim=16, kv_rank=128, size=50,
                                   scale=0.2, dims=16), 256)]}


def random_weights(cfg: dict, seed: int = 0, dtype=torch.float32) -> dict:
    """A checkpoint for ``cfg`` under the design's tensor names (values rounded to ``dtype``)."""
    g = torch.Generator().manual_seed(seed)
    W = {}

    def mat(n, k, s=1.0):
        return torch.randn(n, k, generator=g) * (s / k ** 0.5)

    def vec(n, mean=1.0, s=0.2):
        return mean + torch.randn(n, generator=g) * s

    Wd, V = cfg["width"], cfg["vocab"]
    W["embed"] = torch.randn(V, Wd, generator=g)
    W["head"] = mat(V, Wd)
    W["final.norm"] = vec(Wd)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, D = m["heads"], m["dim"]
        Dv = m.get("vdim", D)
        W[p + "norm1"] = vec(Wd)
        if L["type"] == "latent_attention":
            rd, R = m["rot_dim"], m["kv_rank"]
            W[p + "mix.q"] = mat(H * (D + rd), Wd, 1.5)
            W[p + "mix.dkv"] = mat(R + rd, Wd, 1.5)
            W[p + "mix.dkv.norm"] = vec(R)
            W[p + "mix.uk"], W[p + "mix.uv"] = mat(H * D, R, 1.5), mat(H * Dv, R)
            W[p + "mix.sink"] = vec(H, 0.5, 1.0)
            W[p + "mix.g"] = mat(H * Dv, Wd, 2.0)
        else:
            G = m.get("kv_heads", H)
            W[p + "mix.q"], W[p + "mix.k"] = mat(H * D, Wd, 1.5), mat(G * D, Wd, 1.5)
            W[p + "mix.v"] = mat(G * Dv, Wd)
            W[p + "mix.q.norm"], W[p + "mix.k.norm"] = vec(H * D), vec(G * D)
            W[p + "mix.pb"] = vec(H, -1.0, 0.7)
        W[p + "mix.o"] = mat(Wd, H * Dv, 0.7)
        if L.get("mlp"):
            ff = L["mlp"]["ff"]
            W[p + "mlp.up"], W[p + "mlp.down"] = mat(ff, Wd, 1.5), mat(Wd, ff, 0.7)
            W[p + "mlp.act"] = torch.randn(2, generator=g) * 0.8
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
