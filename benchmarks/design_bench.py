"""Prefill and decode throughput of one decoder design beside another at equal layer sizes
(random weights, one GPU), through the offline engine: ``python bench.py --mode design``.

For each size the two engines are built one after the other on the same device:
* Sekolorn -- latent attention / wkv / latent attention reading the first layer's cache, each
  with a group-routed ungated MoE and a shared expert;
* the closest existing family, a Mixtral-style decoder (grouped-query attention + SwiGLU MoE)
  with the same width, layer count, head count, head size, expert count, top-k and expert ff.
``--design vedadra`` runs the Vedadra design (windowed attention with head mixing, differential
attention, grouped norms, a looped stack, gated GELU feed-forward) beside a Mistral-style decoder
(sliding-window grouped-query attention + SwiGLU) with the same width, number of layer runs, head
count, head size, window and ff.
``--design gapidra`` runs the Gapidra design (parallel sublayers on one norm; sigmoid window
attention and windowed latent attention with sinks, alternating; ungated xIELU feed-forward)
beside the same Mistral-style decoder at equal width, depth, heads, head size, window and ff.
``--design daburax`` runs the Daburax design (hyper-connected residual streams; retention layers
and parallel layers of sink attention beside a gated matrix memory; a group-limited mixture of
gated experts with identity experts and a gated shared expert) beside Sekolorn, the closest
existing design (recurrent and attention layers on state slots and paged rows, a group-routed
mixture of experts with a shared expert), at equal width, depth, heads, experts and expert ff.
Prefill: ``--design-prompts`` prompts of ``--design-prompt-len`` tokens, one sampled token each.
Decode: ``--design-users`` sequences of 128 prompt tokens generating ``--design-gen`` tokens; the
decode rate is the extra tokens over the extra time against the same run with one token.
Prints one JSON line per (size, model) and a closing summary line.
"""

from __future__ import annotations

import gc
import json
import time

SIZES = {
    # name: width, layers (multiple of 3), heads, head dim, rot dim, kv_rank, q_rank, wkv heads,
    #       experts, top, groups, keep, ff, vocab
    "s": dict(width=1024, layers=3, heads=8, dim=64, rot=32, kv_rank=128, q_rank=256,
              wkv_heads=16, experts=8, top=2, groups=4, keep=2, ff=512, vocab=32000),
    "s6": dict(width=1024, layers=6, heads=8, dim=64, rot=32, kv_rank=128, q_rank=256,
               wkv_heads=16, experts=8, top=2, groups=4, keep=2, ff=512, vocab=32000),
    "m": dict(width=2048, layers=6, heads=16, dim=64, rot=32, kv_rank=256, q_rank=512,
              wkv_heads=32, experts=16, top=2, groups=4, keep=2, ff=1024, vocab=32000),
    "l": dict(width=4096, layers=6, heads=32, dim=128, rot=64, kv_rank=512, q_rank=1536,
              wkv_heads=64, experts=16, top=4, groups=4, keep=2, ff=1536, vocab=32000),
}
# Sizes whose whole-engine run is switched off on the GPU: a profiled run of the two "m"
# engines ended with a GPU fault whose cause was not found (every kernel variant those sizes
# select passes its unit tests, the engines were never seen to fail unprofiled); they raise
# until that cause is shown.
GATED = {"m", "l"}


def sekolorn_config(z: dict) -> dict:
    def lat(kv_from=None):
        m = {"heads": z["heads"], "dim": z["dim"], "rot_dim": z["rot"], "vdim": z["dim"],
             "kv_rank": z["kv_rank"], "q_rank": z["q_rank"],
             "scale": (z["dim"] + z["rot"]) ** -0.5, "rot": {"dims": z["rot"], "base": 10000.0}}
        if kv_from is not None:
            m["kv_from"] = kv_from
        return m

    def mlp():
        return {"kind": "moe", "expert": {"ff": z["ff"]}, "shared": {"ff": z["ff"]},
                "router": {"experts": z["experts"], "top": z["top"], "scale": 1.0,
                           "groups": {"count": z["groups"], "keep": z["keep"]}}}

    layers = []
    for i in range(0, z["layers"], 3):
        layers += [{"type": "latent_attention", "mixer": lat(), "mlp": mlp()},
                   {"type": "wkv", "mixer": {"heads": z["wkv_heads"], "dim": 64, "decay_rank": 64},
                    "mlp": mlp()},
                   {"type": "latent_attention", "mixer": lat(kv_from=i), "mlp": mlp()}]
    return {"architecture": "Sekolorn", "vocab": z["vocab"], "width": z["width"],
            "norm": {"eps": 1e-6}, "layers": layers}


def mixtral_config(z: dict) -> dict:
    return {"architectures": ["MixtralForCausalLM"], "hidden_size": z["width"],
            "num_hidden_layers": z["layers"], "num_attention_heads": z["heads"],
            "num_key_value_heads": max(1, z["heads"] // 4), "head_dim": 128,
            "vocab_size": z["vocab"], "intermediate_size": z["ff"],
            "num_local_experts": z["experts"], "num_experts_per_tok": z["top"],
            "max_position_embeddings": 32768, "rms_norm_eps": 1e-6, "rope_theta": 1e6}


VSIZES = {
    # name: width, layer runs (3 layers looped twice), heads, kv heads, head dim, window, ff, vocab
    "vs": dict(width=1024, heads=8, kv_heads=2, dim=128, window=1024, ff=4096, vocab=32000),
    "vm": dict(width=2048, heads=16, kv_heads=4, dim=128, window=1024, ff=8192, vocab=32000),
}


def vedadra_config(z: dict) -> dict:
    H, G, D = z["heads"], z["kv_heads"], z["dim"]
    mlp = {"kind": "dense", "ff": z["ff"]}
    att = {"type": "attention", "mlp": mlp,
           "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": D ** -0.5,
                     "mask": {"size": z["window"]}}}
    att2 = {"type": "attention_2", "mlp": mlp,
            "mixer": {"heads": H, "kv_heads": G, "dim": D // 2, "vdim": D, "scale": (D // 2) ** -0.5,
                      "diff": 0.3, "mask": {"size": z["window"], "keep_first": 4}}}
    return {"architecture": "Vedadra", "vocab": z["vocab"], "width": z["width"],
            "norm": {"eps": 1e-5, "groups": 4}, "loop": {"start": 0, "stop": 3, "times": 2},
            "layers": [att, att2, att]}


def mistral_config(z: dict) -> dict:
    return {"architectures": ["MistralForCausalLM"], "hidden_size": z["width"],
            "num_hidden_layers": 6, "num_attention_heads": z["heads"],
            "num_key_value_heads": z["kv_heads"], "head_dim": z["dim"], "vocab_size": z["vocab"],
            "intermediate_size": z["ff"], "sliding_window": z["window"],
            "max_position_embeddings": 32768, "rms_norm_eps": 1e-5, "rope_theta": 1e6}


GSIZES = {
    # name: width, heads, kv heads, head dim, latent rank, rotary part, window, ff, vocab
    "gs": dict(width=1024, heads=8, kv_heads=2, dim=128, kv_rank=256, rot=64, window=1024, ff=4096,
               vocab=32000),
    "gm": dict(width=2048, heads=16, kv_heads=4, dim=128, kv_rank=512, rot=64, window=1024,
               ff=8192, vocab=32000),
}


def gapidra_config(z: dict) -> dict:
    H, G, D = z["heads"], z["kv_heads"], z["dim"]
    mlp = {"kind": "dense", "ff": z["ff"]}
    att = {"type": "attention", "mlp": mlp,
           "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": D ** -0.5,
                     "mask": {"size": z["window"]},
                     "rot": {"base": 1e6, "dims": D // 2,
                             "scaling": {"factor": 4.0, "original": 8192, "fast": 32.0,
                                         "slow": 1.0}}}}
    lat = {"type": "latent_attention", "mlp": mlp,
           "mixer": {"heads": H, "dim": D - z["rot"], "rot_dim": z["rot"], "vdim": D,
                     "kv_rank": z["kv_rank"], "scale": D ** -0.5, "mask": {"size": z["window"]},
                     "rot": {"base": 1e6, "dims": z["rot"]}}}
    return {"architecture": "Gapidra", "vocab": z["vocab"], "width": z["width"],
            "norm": {"eps": 1e-5}, "embedding": {"scale": z["width"] ** 0.5},
            "layers": [att, lat, lat, att, lat, att]}


DSIZES = {
    # name: width, heads, head dim, experts (+ 2 identity outputs), expert ff, streams, vocab
    "ds": dict(width=1024, layers=6, heads=8, dim=128, experts=8, top=2, ff=512, streams=4,
               vocab=32000),
    "dm": dict(width=2048, layers=6, heads=16, dim=128, experts=16, top=2, ff=1024, streams=4,
               vocab=32000),
}


def daburax_config(z: dict) -> dict:
    H, D = z["heads"], z["dim"]
    mlp = {"kind": "moe", "expert": {"ff": z["ff"]}, "shared": {"ff": z["ff"]},
           "router": {"experts": z["experts"] - 2, "identity": 2, "top": z["top"],
                      "groups": {"count": 4, "keep": 2}}}
    ret = {"type": "retention", "mlp": mlp,
           "mixer": {"heads": H, "dim": D, "vdim": D, "rot": {"base": 1e4, "dims": D},
                     "decay": [1.0 - 2.0 ** (-4 - 6 * i / H) for i in range(H)]}}
    par = {"type": "parallel", "mlp": mlp,
           "mixer": {"left": {"heads": H, "kv_heads": max(1, H // 4), "dim": D, "vdim": D,
                              "scale": D ** -0.5,
                              "rot": {"base": 5e5, "dims": D // 2, "scaling": {"factor": 4.0}}},
                     "right": {"heads": H // 2, "dim": D, "vdim": D, "gate_cap": 15.0},
                     "left_scale": 1.0, "right_scale": 1.0}}
    return {"architecture": "Daburax", "vocab": z["vocab"], "width": z["width"],
            "norm": {"eps": 1e-5}, "residual_mult": 0.7, "streams": z["streams"],
            "embedding": {"scale": z["width"] ** 0.5,
                          "bigram": {"buckets": 65521, "mul_prev": 1009, "mul_cur": 8191}},
            "layers": [ret, ret, par] * (z["layers"] // 3)}


def sekolorn_like(z: dict) -> dict:
    """Sekolorn at a Daburax size: same width, depth, heads, experts, top-k and expert ff."""
    return sekolorn_config(dict(width=z["width"], layers=z["layers"], heads=z["heads"], dim=64,
                                rot=32, kv_rank=z["width"] // 8, q_rank=z["width"] // 4,
                                wkv_heads=z["width"] // 64, experts=z["experts"], top=z["top"],
                                groups=4, keep=2, ff=z["ff"], vocab=z["vocab"]))


def _measure(cfg_dict: dict, a) -> dict:
    import torch

    from enterprise_inference_amd.config import (CacheConfig, EngineConfig, ModelConfig,
                                                 SchedulerConfig)
    from enterprise_inference_amd.engine.llm_engine import LLMEngine
    from enterprise_inference_amd.engine.sampling_params import SamplingParams

    P, NP, B, G = a.design_prompt_len, a.design_prompts, a.design_users, a.design_gen
    ec = EngineConfig(model=ModelConfig.from_hf_dict(cfg_dict), device="cuda", load_format="dummy",
                      cache=CacheConfig(block_size=128, num_gpu_blocks=max(
                          NP * (P // 128 + 2), B * 4) + 8, swap_space_gb=0.0),
                      scheduler=SchedulerConfig(max_num_seqs=max(B, NP),
                                                max_num_batched_tokens=max(P, 2048),
                                                max_model_len=P + 256),
                      seed=a.seed)
    eng = LLMEngine(ec)
    V = cfg_dict.get("vocab", cfg_dict.get("vocab_size"))
    g = torch.Generator().manual_seed(a.seed)

    def prompts(n, length):
        return torch.randint(1, V, (n, length), generator=g).tolist()

    def run(pr, max_tokens):
        torch.cuda.synchronize()
        t0 = time.time()
        eng.generate(prompt_token_ids=pr, params=SamplingParams(max_tokens=max_tokens,
                                                                temperature=0.0, ignore_eos=True))
        torch.cuda.synchronize()
        return time.time() - t0

    run(prompts(2, P), 2)                                     # warm-up (library heuristics)
    tp = min(run(prompts(NP, P), 1) for _ in range(a.steps))
    dp = prompts(B, 128)
    run(dp, 4)
    t1 = min(run(dp, 1) for _ in range(a.steps))
    t2 = min(run(dp, 1 + G) for _ in range(a.steps))
    out = {"prefill_tok_s": NP * P / tp, "decode_tok_s": B * G / max(1e-9, t2 - t1),
           "decode_ms_per_step": 1e3 * (t2 - t1) / G,
           "graphs": bool(eng.executor.runner.graphs)}
    eng.shutdown()
    del eng
    gc.collect()
    torch.cuda.empty_cache()
    return out


def run(a) -> int:
    rows = []
    design = getattr(a, "design", "sekolorn")
    vedadra = design == "vedadra"
    default = {"vedadra": "vs,vm", "gapidra": "gs,gm", "daburax": "ds,dm"}.get(design, "s,s6")
    for name in (a.design_sizes or default).split(","):
        if name in GATED:
            raise SystemExit(f"design size {name!r} is switched off (see GATED in "
                             "benchmarks/design_bench.py); run s or s6")
        if design == "daburax":
            z = DSIZES[name]
            # (Sekolorn's engines at width 2048 are switched off, see GATED: the larger size
            # runs beside the Mixtral-style decoder instead)
            other = ("Sekolorn", sekolorn_like(z)) if name == "ds" else \
                ("Mixtral-style", mixtral_config(z))
            pair = (("Daburax", daburax_config(z)), other)
        elif design == "gapidra":
            z = dict(GSIZES[name], layers=6)
            pair = (("Gapidra", gapidra_config(z)), ("Mistral-style", mistral_config(z)))
        elif vedadra:
            z = dict(VSIZES[name], layers=6)
            pair = (("Vedadra", vedadra_config(z)), ("Mistral-style", mistral_config(z)))
        else:
            z = SIZES[name]
            pair = (("Sekolorn", sekolorn_config(z)), ("Mixtral-style", mixtral_config(z)))
        for label, cfg in pair:
            if label.split("-")[0].lower() not in a.design_models.lower():
                continue
            r = _measure(cfg, a)
            r.update(size=name, model=label, width=z["width"], layers=z["layers"],
                     prompt_len=a.design_prompt_len, users=a.design_users)
            rows.append(r)
            print(json.dumps(r), flush=True)
    print(json.dumps({"metric": "design_comparison", "rows": rows, "dtype": "bf16",
                      "data": "synthetic", "n_gpus": 1}), flush=True)
    return 0


# ---------------------------------------------------------------------------------- kernel rates
def _time(fn, iters: int = 5) -> float:
    import torch
    fn()
    torch.cuda.synchronize()
    best = 1e9
    for _ in range(iters):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        torch.cuda.synchronize()
        best = min(best, a.elapsed_time(b) * 1e-3)
    return best


def kernel_rates(a) -> int:
    """Achieved rates of the new design's kernels beside the like kernels of the Llama / Mixtral
    path at equal head counts and lengths (``--design-kernels``): causal prefill attention
    (useful TFLOP/s: 2 (Dqk + Dv) per query-key pair and head, the hi/lo second product of the
    latent kernel not counted), decode attention (cache bytes read per second) and the wkv scan
    (tokens/s and state bytes/s).  One JSON line per kernel."""
    import torch

    if getattr(a, "design", "sekolorn") == "vedadra":
        return window_kernel_rates(a)
    if getattr(a, "design", "sekolorn") == "gapidra":
        return gapidra_kernel_rates(a)
    if getattr(a, "design", "sekolorn") == "daburax":
        return daburax_kernel_rates(a)
    from enterprise_inference_amd.ops import attention as A
    from enterprise_inference_amd.ops import latent_attention as LA
    from enterprise_inference_amd.ops import wkv as WK

    dev, bf = "cuda", torch.bfloat16
    bs = 128
    rows = []
    for (H, R, rd, T) in ((8, 128, 32, 4096), (16, 512, 64, 4096)):
        nb = T // bs
        cache = torch.randn(nb, bs, R + rd, device=dev).to(bf)
        qa = torch.randn(T, H, R, device=dev).to(bf) * 0.1
        qr = torch.randn(T, H, rd, device=dev).to(bf) * 0.1
        inv = LA.inv_frequencies(rd, 10000.0, dev)
        bt = torch.arange(nb, dtype=torch.int32, device=dev)[None]
        pos = torch.arange(T, dtype=torch.int32, device=dev)
        qb = LA.query_block(H, R, rd, bf)
        work = LA.build_work([T], qb)
        md = A.AttentionMetadata(
            num_decode=0, num_prefill_tokens=T, slot_mapping=pos, positions=pos,
            prefill_block_tables=bt, prefill_seq_lens=torch.tensor([T], dtype=torch.int32, device=dev),
            prefill_cu_q=torch.tensor([0, T], dtype=torch.int32, device=dev),
            prefill_work=torch.tensor(work, dtype=torch.int32, device=dev),
            prefill_n_work=len(work) // 2, prefill_qblock=qb)
        t = _time(lambda: LA.latent_attention(qa, qr, inv, rd, cache, md, None, 0.1))
        fl = 2.0 * (2 * R + rd) * H * T * (T + 1) / 2
        rows.append({"kernel": "latent_attn_mfma prefill", "heads": H, "kv_rank": R, "rot": rd,
                     "tokens": T, "ms": t * 1e3, "tflops": fl / t / 1e12})
        # the like kernel: paged flash prefill, same heads, D = 128, GQA group 4
        D, Hkv = 128, max(1, H // 4)
        kc = torch.randn(nb, Hkv, bs, D, device=dev).to(bf)
        vc = torch.randn(nb, Hkv, D, bs, device=dev).to(bf)
        q = torch.randn(T, H, D, device=dev).to(bf) * 0.1
        qb2 = A.prefill_query_block(H, Hkv, D, block_size=bs)
        w2 = A.build_prefill_work([T], qb2)
        t2 = _time(lambda: A.paged_prefill(q, kc, vc, bt, md.prefill_seq_lens, md.prefill_cu_q,
                                           torch.tensor(w2, dtype=torch.int32, device=dev),
                                           len(w2) // 2, 0.1))
        rows.append({"kernel": "paged_prefill (flash)", "heads": H, "head_dim": D, "tokens": T,
                     "ms": t2 * 1e3, "tflops": 2.0 * 2 * D * H * T * (T + 1) / 2 / t2 / 1e12})
        # decode: B sequences of context L
        B, L = 64, 4096
        nbd = B * L // bs
        cache_d = torch.randn(nbd, bs, R + rd, device=dev).to(bf)
        btd = torch.arange(nbd, dtype=torch.int32, device=dev).view(B, L // bs)
        posd = torch.full((B,), L - 1, dtype=torch.int32, device=dev)
        lens = torch.full((B,), L, dtype=torch.int32, device=dev)
        mdd = A.AttentionMetadata(num_decode=B, num_prefill_tokens=0, slot_mapping=posd,
                                  positions=posd, decode_block_tables=btd, decode_seq_lens=lens)
        qad, qrd = qa[:B].contiguous(), qr[:B].contiguous()
        t3 = _time(lambda: LA.latent_attention(qad, qrd, inv, rd, cache_d, mdd, None, 0.1))
        rows.append({"kernel": "latent_attn_mfma decode", "heads": H, "kv_rank": R, "batch": B,
                     "context": L, "ms": t3 * 1e3,
                     "cache_GBps": B * L * (R + rd) * 2 / t3 / 1e9})
        kcd = torch.randn(nbd, Hkv, bs, D, device=dev).to(bf)
        vcd = torch.randn(nbd, Hkv, D, bs, device=dev).to(bf)
        qd = q[:B].contiguous()
        t4 = _time(lambda: A.paged_decode(qd, kcd, vcd, btd, lens, 0.1))
        rows.append({"kernel": "paged_decode", "heads": H, "kv_heads": Hkv, "batch": B,
                     "context": L, "ms": t4 * 1e3,
                     "cache_GBps": B * L * Hkv * D * 2 * 2 / t4 / 1e9})
    # wkv: one long prompt (sequential scan) and a decode batch (state traffic)
    Hh, D, W = 32, 64, 2048
    for (nseq, per) in ((1, 4096), (64, 1)):
        T = nseq * per
        HD = Hh * D
        r, k, v, g = (torch.randn(T, HD, device=dev).to(bf) * 0.3 for _ in range(4))
        dec = torch.randn(T, HD, device=dev) * 0.3
        w0 = torch.full((HD,), -1.0, device=dev).to(bf)
        u = (torch.randn(HD, device=dev) * 0.3).to(bf)
        nw = torch.ones(HD, device=dev).to(bf)
        S = torch.zeros(nseq, Hh, D, D, device=dev)
        prev = torch.zeros(nseq, W, device=dev)
        x = torch.randn(T, W, device=dev)
        slots = torch.arange(nseq, dtype=torch.int32, device=dev)
        cu = torch.arange(0, T + 1, per, dtype=torch.int32, device=dev)
        pos = (torch.arange(T, dtype=torch.int32, device=dev) % per) + (5 if per == 1 else 0)
        t5 = _time(lambda: WK.wkv_scan(r, k, v, g, dec, w0, u, nw, S, prev, x, slots, cu, nseq,
                                       pos, None, 1e-5, Hh))
        rows.append({"kernel": "wkv_scan", "heads": Hh, "dim": D, "seqs": nseq, "tokens_per_seq": per,
                     "ms": t5 * 1e3, "tokens_per_s": T / t5,
                     "state_GBps": nseq * Hh * D * D * 4 * 2 / t5 / 1e9})
    for r_ in rows:
        print(json.dumps(r_), flush=True)
    print(json.dumps({"metric": "design_kernel_rates", "rows": rows}), flush=True)
    return 0


def window_kernel_rates(a) -> int:
    """Achieved rates of the window attention kernels (head-mixing and differential forms) beside
    the sliding-window paged kernels of the Llama path at equal heads, head size, window and
    lengths: prefill in useful TFLOP/s (2 P (D + Dv) per visible query-key pair and head; the
    second product's remainder pass and the head mixing are not counted), decode in cache bytes
    of the visible keys per second, and the grouped-norm boundary step beside the fused add +
    RMS norm in bytes moved per second.  One JSON line per kernel."""
    import torch

    from enterprise_inference_amd.ops import attention as A
    from enterprise_inference_amd.ops import norm as N
    from enterprise_inference_amd.ops import window_attention as WA

    dev, bf = "cuda", torch.bfloat16
    bs, win, T = 128, 1024, 4096
    rows = []
    pairs = T * win - win * (win - 1) // 2                     # visible (query, key) pairs
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    for H, G in ((8, 2), (16, 4)):
        for kind in ("talking", "differential"):
            P, D, Dv = (1, 128, 128) if kind == "talking" else (2, 64, 128)
            M = H * P
            spec = WA.WindowSpec(H, G, P, D, Dv, win, 0 if P == 1 else 4,
                                 mult=torch.full((M,), D ** -0.5, device=dev))
            if P == 1:
                hh = torch.arange(1, H + 1, dtype=torch.float64)
                spec.slope = torch.pow(2.0, -8.0 * hh / H).float().to(dev)
                spec.talk = (torch.eye(H) + 0.05 * torch.randn(H, H)).to(dev)
            else:
                spec.epilogue, spec.eps, spec.post = 1, 1e-5, 0.7
                spec.lam = torch.tensor([0.4], device=dev)
            nb = T // bs
            kc = torch.randn(nb, bs, G * P * D, device=dev).to(bf)
            vc = torch.randn(nb, G * Dv, bs, device=dev).to(bf)
            q = torch.randn(T, M * D, device=dev).to(bf)
            gate = torch.randn(T, H * Dv, device=dev).to(bf) if P == 1 else None
            pos = torch.arange(T, dtype=torch.int32, device=dev)
            bt = torch.arange(nb, dtype=torch.int32, device=dev)[None]
            md = A.AttentionMetadata(
                num_decode=0, num_prefill_tokens=T, slot_mapping=pos, positions=pos,
                prefill_block_tables=bt, prefill_seq_lens=i32([T]), prefill_cu_q=i32([0, T]),
                prefill_q_lens=[T])
            t = _time(lambda: WA.window_attention(q, kc, vc, md, spec, gate))
            rows.append({"kernel": f"window_attn prefill ({kind})", "heads": H, "kv_heads": G,
                         "dim": D, "vdim": Dv, "window": win, "tokens": T, "ms": t * 1e3,
                         "mfma": WA.mfma_ok(spec, bf, bs),
                         "tflops": 2.0 * P * (D + Dv) * H * pairs / t / 1e12})
            # decode: B sequences of context L, the last `win` keys visible
            B, L = 64, 4096
            nbd = B * L // bs
            kcd = torch.randn(nbd, bs, G * P * D, device=dev).to(bf)
            vcd = torch.randn(nbd, G * Dv, bs, device=dev).to(bf)
            btd = torch.arange(nbd, dtype=torch.int32, device=dev).view(B, L // bs)
            posd = torch.full((B,), L - 1, dtype=torch.int32, device=dev)
            mdd = A.AttentionMetadata(num_decode=B, num_prefill_tokens=0, slot_mapping=posd,
                                      positions=posd, decode_block_tables=btd,
                                      decode_seq_lens=i32([L] * B))
            qd = q[:B].contiguous()
            gd = gate[:B].contiguous() if gate is not None else None
            t3 = _time(lambda: WA.window_attention(qd, kcd, vcd, mdd, spec, gd))
            rows.append({"kernel": f"window_attn decode ({kind})", "heads": H, "kv_heads": G,
                         "batch": B, "context": L, "window": win, "ms": t3 * 1e3,
                         "cache_GBps": B * win * G * (P * D + Dv) * 2 / t3 / 1e9})
        # the like kernels: sliding-window paged prefill (flash form) and decode, D = 128
        D = 128
        nb = T // bs
        kc = torch.randn(nb, G, bs, D, device=dev).to(bf)
        vc = torch.randn(nb, G, D, bs, device=dev).to(bf)
        q = torch.randn(T, H, D, device=dev).to(bf) * 0.1
        bt = torch.arange(nb, dtype=torch.int32, device=dev)[None]
        qb2 = A.prefill_query_block(H, G, D, block_size=bs)
        w2 = A.build_prefill_work([T], qb2)
        wt = i32(w2)
        t2 = _time(lambda: A.paged_prefill(q, kc, vc, bt, i32([T]), i32([0, T]), wt, len(w2) // 2,
                                           0.1, sliding_window=win))
        rows.append({"kernel": "paged_prefill (flash, sliding window)", "heads": H, "kv_heads": G,
                     "head_dim": D, "window": win, "tokens": T, "ms": t2 * 1e3,
                     "tflops": 2.0 * 2 * D * H * pairs / t2 / 1e12})
        B, L = 64, 4096
        nbd = B * L // bs
        kcd = torch.randn(nbd, G, bs, D, device=dev).to(bf)
        vcd = torch.randn(nbd, G, D, bs, device=dev).to(bf)
        btd = torch.arange(nbd, dtype=torch.int32, device=dev).view(B, L // bs)
        lens = i32([L] * B)
        qd = q[:B].contiguous()
        t4 = _time(lambda: A.paged_decode(qd, kcd, vcd, btd, lens, 0.1, sliding_window=win))
        rows.append({"kernel": "paged_decode (sliding window)", "heads": H, "kv_heads": G,
                     "batch": B, "context": L, "window": win, "ms": t4 * 1e3,
                     "cache_GBps": B * win * G * D * 2 * 2 / t4 / 1e9})
    # sublayer boundary: output norm + residual + next input norm (fp32 stream) beside the
    # bf16 fused add + RMS norm
    for W in (2048, 4096):
        Tn = 8192
        x = torch.randn(Tn, W, device=dev)
        y = torch.randn(Tn, W, device=dev).to(bf)
        w1, w2_ = torch.ones(W, device=dev).to(bf), torch.ones(W, device=dev).to(bf)
        t5 = _time(lambda: N.group_norm_step(x, 4, 1e-5, y, w1, None, w2_))
        rows.append({"kernel": "group_norm_step", "width": W, "rows": Tn, "ms": t5 * 1e3,
                     "GBps": Tn * W * (2 + 4 + 4 + 2) / t5 / 1e9})
        res = torch.randn(Tn, W, device=dev).to(bf)
        t6 = _time(lambda: N.fused_add_rms_norm(y, res, w1, 1e-5))
        rows.append({"kernel": "fused_add_rms_norm", "width": W, "rows": Tn, "ms": t6 * 1e3,
                     "GBps": Tn * W * (2 + 2 + 2 + 2) / t6 / 1e9})
    for r_ in rows:
        print(json.dumps(r_), flush=True)
    print(json.dumps({"metric": "design_kernel_rates", "design": "vedadra", "rows": rows}),
          flush=True)
    return 0


def gapidra_kernel_rates(a) -> int:
    """Achieved rates of the Gapidra kernels beside the sliding-window paged kernels of the Llama
    path at equal heads, head size, window and lengths: sigmoid window attention and windowed
    latent attention with sinks -- prefill in useful TFLOP/s (2 (Dqk + Dv) per visible query-key
    pair and head; the second product's remainder pass is not counted), decode in cache bytes of
    the visible keys per second -- and the layer boundary (two sublayer outputs + residual + next
    norm on an fp32 stream) beside the bf16 fused add + RMS norm in bytes moved per second.  One
    JSON line per kernel."""
    import torch

    from enterprise_inference_amd.ops import attention as A
    from enterprise_inference_amd.ops import latent_attention as LA
    from enterprise_inference_amd.ops import norm as N
    from enterprise_inference_amd.ops import window_attention as WA
    from enterprise_inference_amd.ops.rotary import rotary_frequencies

    dev, bf = "cuda", torch.bfloat16
    bs, win, T = 128, 1024, 4096
    rows = []
    pairs = T * win - win * (win - 1) // 2                     # visible (query, key) pairs
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    B, L = 64, 4096
    nb, nbd = T // bs, B * L // bs
    pos = torch.arange(T, dtype=torch.int32, device=dev)
    bt = torch.arange(nb, dtype=torch.int32, device=dev)[None]
    md = A.AttentionMetadata(
        num_decode=0, num_prefill_tokens=T, slot_mapping=pos, positions=pos,
        prefill_block_tables=bt, prefill_seq_lens=i32([T]), prefill_cu_q=i32([0, T]),
        prefill_q_lens=[T])
    btd = torch.arange(nbd, dtype=torch.int32, device=dev).view(B, L // bs)
    posd = torch.full((B,), L - 1, dtype=torch.int32, device=dev)
    mdd = A.AttentionMetadata(num_decode=B, num_prefill_tokens=0, slot_mapping=posd,
                              positions=posd, decode_block_tables=btd,
                              decode_seq_lens=i32([L] * B))
    for H, G, R, rd in ((8, 2, 256, 64), (16, 4, 512, 64)):
        D = Dv = 128
        # sigmoid window attention
        spec = WA.WindowSpec(H, G, 1, D, Dv, win, 0, mult=torch.full((H,), D ** -0.5, device=dev),
                             weights=1, bias=torch.full((H,), -4.0, device=dev))
        kc = torch.randn(nb, bs, G * D, device=dev).to(bf)
        vc = torch.randn(nb, G * Dv, bs, device=dev).to(bf)
        q = torch.randn(T, H * D, device=dev).to(bf)
        t = _time(lambda: WA.window_attention(q, kc, vc, md, spec, None))
        rows.append({"kernel": "window_attn prefill (sigmoid)", "heads": H, "kv_heads": G,
                     "dim": D, "vdim": Dv, "window": win, "tokens": T, "ms": t * 1e3,
                     "mfma": WA.mfma_ok(spec, bf, bs),
                     "tflops": 2.0 * (D + Dv) * H * pairs / t / 1e12})
        kcd = torch.randn(nbd, bs, G * D, device=dev).to(bf)
        vcd = torch.randn(nbd, G * Dv, bs, device=dev).to(bf)
        qd = q[:B].contiguous()
        t = _time(lambda: WA.window_attention(qd, kcd, vcd, mdd, spec, None))
        rows.append({"kernel": "window_attn decode (sigmoid)", "heads": H, "kv_heads": G,
                     "batch": B, "context": L, "window": win, "ms": t * 1e3,
                     "cache_GBps": B * win * G * (D + Dv) * 2 / t / 1e9})
        del kcd, vcd
        # windowed latent attention with sinks (absorbed form: Dqk = R + rd, Dv = R)
        inv, amp = rotary_frequencies(rd, 1e6, None, dev)
        sink = torch.zeros(H, device=dev)
        cache = torch.randn(nb, bs, R + rd, device=dev).to(bf)
        qa = torch.randn(T, H, R, device=dev).to(bf) * 0.1
        qr = torch.randn(T, H, rd, device=dev).to(bf) * 0.1
        qb = LA.query_block(H, R, rd, bf)
        work = LA.build_work([T], qb)
        mdl = A.AttentionMetadata(
            num_decode=0, num_prefill_tokens=T, slot_mapping=pos, positions=pos,
            prefill_block_tables=bt, prefill_seq_lens=i32([T]), prefill_cu_q=i32([0, T]),
            prefill_work=i32(work), prefill_n_work=len(work) // 2, prefill_qblock=qb)
        t = _time(lambda: LA.latent_attention(qa, qr, inv, rd, cache, mdl, None, 0.1, win, sink,
                                              True, amp))
        rows.append({"kernel": "latent_attn prefill (window, sink)", "heads": H, "kv_rank": R,
                     "rot": rd, "window": win, "tokens": T, "ms": t * 1e3,
                     "tflops": 2.0 * (2 * R + rd) * H * pairs / t / 1e12})
        cache_d = torch.randn(nbd, bs, R + rd, device=dev).to(bf)
        qad, qrd = qa[:B].contiguous(), qr[:B].contiguous()
        t = _time(lambda: LA.latent_attention(qad, qrd, inv, rd, cache_d, mdd, None, 0.1, win, sink,
                                              True, amp))
        rows.append({"kernel": "latent_attn decode (window, sink)", "heads": H, "kv_rank": R,
                     "batch": B, "context": L, "window": win, "ms": t * 1e3,
                     "cache_GBps": B * win * (R + rd) * 2 / t / 1e9})
        del cache_d
        # the like kernels: sliding-window paged prefill (flash form) and decode, D = 128
        kc = torch.randn(nb, G, bs, D, device=dev).to(bf)
        vc = torch.randn(nb, G, D, bs, device=dev).to(bf)
        q3 = torch.randn(T, H, D, device=dev).to(bf) * 0.1
        qb2 = A.prefill_query_block(H, G, D, block_size=bs)
        w2 = A.build_prefill_work([T], qb2)
        wt = i32(w2)
        t = _time(lambda: A.paged_prefill(q3, kc, vc, bt, i32([T]), i32([0, T]), wt, len(w2) // 2,
                                          0.1, sliding_window=win))
        rows.append({"kernel": "paged_prefill (flash, sliding window)", "heads": H, "kv_heads": G,
                     "head_dim": D, "window": win, "tokens": T, "ms": t * 1e3,
                     "tflops": 2.0 * 2 * D * H * pairs / t / 1e12})
        kcd = torch.randn(nbd, G, bs, D, device=dev).to(bf)
        vcd = torch.randn(nbd, G, D, bs, device=dev).to(bf)
        lens = i32([L] * B)
        qd3 = q3[:B].contiguous()
        t = _time(lambda: A.paged_decode(qd3, kcd, vcd, btd, lens, 0.1, sliding_window=win))
        rows.append({"kernel": "paged_decode (sliding window)", "heads": H, "kv_heads": G,
                     "batch": B, "context": L, "window": win, "ms": t * 1e3,
                     "cache_GBps": B * win * G * D * 2 * 2 / t / 1e9})
        del kcd, vcd
    for W in (2048, 4096):
        Tn = 8192
        x = torch.randn(Tn, W, device=dev)
        y1 = torch.randn(Tn, W, device=dev).to(bf)
        y2 = torch.randn(Tn, W, device=dev).to(bf)
        w1 = torch.ones(W, device=dev).to(bf)
        t = _time(lambda: N.residual_rms_step(x, 1e-5, (y1, y2), w1))
        rows.append({"kernel": "residual_rms_step (2 outputs)", "width": W, "rows": Tn,
                     "ms": t * 1e3, "GBps": Tn * W * (2 + 2 + 4 + 4 + 2) / t / 1e9})
        res = torch.randn(Tn, W, device=dev).to(bf)
        t = _time(lambda: N.fused_add_rms_norm(y1, res, w1, 1e-5))
        rows.append({"kernel": "fused_add_rms_norm", "width": W, "rows": Tn, "ms": t * 1e3,
                     "GBps": Tn * W * (2 + 2 + 2 + 2) / t / 1e9})
    for r_ in rows:
        print(json.dumps(r_), flush=True)
    print(json.dumps({"metric": "design_kernel_rates", "design": "gapidra", "rows": rows}),
          flush=True)
    return 0


def daburax_kernel_rates(a) -> int:
    """Achieved rates of the Daburax kernels beside their like kernels: the fixed-decay and the
    gated linear scans beside the wkv scan at equal heads and head size (one 4096-token prompt:
    tokens/s; a 64-row decode batch: state bytes/s); sink attention beside the paged flash
    prefill and paged decode kernels of the Llama path at equal heads and lengths (prefill in
    useful TFLOP/s, decode in cache bytes/s); the hyper-connection step over four streams beside
    the fused add + RMS norm (bytes moved per second); the router.  One JSON line per kernel."""
    import torch

    from enterprise_inference_amd.ops import attention as A
    from enterprise_inference_amd.ops import linear_scan as LS
    from enterprise_inference_amd.ops import moe as M
    from enterprise_inference_amd.ops import norm as N
    from enterprise_inference_amd.ops import window_attention as WA
    from enterprise_inference_amd.ops import wkv as WK
    from enterprise_inference_amd.ops.rotary import rotary_frequencies

    dev, bf = "cuda", torch.bfloat16
    rows = []
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    # ---- scans: Hh heads of 64 x 64 (the wkv kernel's shape) and of 128 x 128
    for Hh, D in ((32, 64), (16, 128)):
        for (nseq, per) in ((1, 4096), (4, 2048), (64, 1)):
            T = nseq * per
            slots = torch.arange(nseq, dtype=torch.int32, device=dev)
            cu = torch.arange(0, T + 1, per, dtype=torch.int32, device=dev)
            pos = (torch.arange(T, dtype=torch.int32, device=dev) % per) + (5 if per == 1 else 0)
            fused = (torch.randn(T, 4 * Hh * D + 2 * Hh, device=dev) * 0.3).to(bf)
            inv, _ = rotary_frequencies(D, 1e4, None, dev)
            for mode in ("decay", "exp_gates"):
                spec = LS.ScanSpec(Hh, D, D, mode,
                                   decay=torch.full((Hh,), 0.97, device=dev), cap=15.0,
                                   inv_freq=inv if mode == "decay" else None,
                                   rot_dims=D if mode == "decay" else 0, kscale=D ** -0.5,
                                   gate_act="silu" if mode == "decay" else "sigmoid", eps=1e-5)
                st = LS.ScanState.allocate(nseq, spec, dev)
                forms = [("token by token", None)]
                if per > 1:
                    forms.append(("chunk-parallel", LS.chunk_plan([per] * nseq, dev)))
                for form, plan in forms:
                    LS.FORCE_CHUNKED = plan is not None
                    t = _time(lambda: LS.linear_scan(fused, 0, Hh * D, 2 * Hh * D, 3 * Hh * D,
                                                     spec, st, slots, cu, nseq, pos, None, None,
                                                     4 * Hh * D, 4 * Hh * D + Hh, plan=plan))
                    rows.append({"kernel": f"linear_scan ({mode}, {form})", "heads": Hh, "dim": D,
                                 "seqs": nseq, "tokens_per_seq": per, "ms": t * 1e3,
                                 "tokens_per_s": T / t,
                                 "state_GBps": nseq * Hh * D * D * 4 * 2 / t / 1e9})
            if D == 64:
                HD, W = Hh * D, 2048
                r, k, v, g = (torch.randn(T, HD, device=dev).to(bf) * 0.3 for _ in range(4))
                dec = torch.randn(T, HD, device=dev) * 0.3
                w0 = torch.full((HD,), -1.0, device=dev).to(bf)
                u = (torch.randn(HD, device=dev) * 0.3).to(bf)
                nw = torch.ones(HD, device=dev).to(bf)
                S = torch.zeros(nseq, Hh, D, D, device=dev)
                prev = torch.zeros(nseq, W, device=dev)
                x = torch.randn(T, W, device=dev)
                t = _time(lambda: WK.wkv_scan(r, k, v, g, dec, w0, u, nw, S, prev, x, slots, cu,
                                              nseq, pos, None, 1e-5, Hh))
                rows.append({"kernel": "wkv_scan", "heads": Hh, "dim": D, "seqs": nseq,
                             "tokens_per_seq": per, "ms": t * 1e3, "tokens_per_s": T / t,
                             "state_GBps": nseq * Hh * D * D * 4 * 2 / t / 1e9})
    # ---- sink attention beside the paged kernels
    bs, T = 128, 4096
    pairs = T * (T + 1) // 2
    B, L = 64, 4096
    nb, nbd = T // bs, B * L // bs
    pos = torch.arange(T, dtype=torch.int32, device=dev)
    bt = torch.arange(nb, dtype=torch.int32, device=dev)[None]
    # (the step's work list as the model runner builds it: latest query blocks first)
    wl = A.build_prefill_work([T], WA.MFMA_QB)
    md = A.AttentionMetadata(
        num_decode=0, num_prefill_tokens=T, slot_mapping=pos, positions=pos,
        prefill_block_tables=bt, prefill_seq_lens=i32([T]), prefill_cu_q=i32([0, T]),
        prefill_q_lens=[T], prefill_work=i32(wl), prefill_n_work=len(wl) // 2,
        prefill_qblock=WA.MFMA_QB)
    btd = torch.arange(nbd, dtype=torch.int32, device=dev).view(B, L // bs)
    posd = torch.full((B,), L - 1, dtype=torch.int32, device=dev)
    mdd = A.AttentionMetadata(num_decode=B, num_prefill_tokens=0, slot_mapping=posd,
                              positions=posd, decode_block_tables=btd,
                              decode_seq_lens=i32([L] * B))
    for H, G in ((8, 2), (16, 4)):
        D = Dv = 128
        spec = WA.WindowSpec(H, G, 1, D, Dv, 0, 0, mult=torch.full((H,), D ** -0.5, device=dev),
                             sink=torch.zeros(H, device=dev))
        kc = torch.randn(nb, bs, G * D, device=dev).to(bf)
        vc = torch.randn(nb, G * Dv, bs, device=dev).to(bf)
        q = torch.randn(T, H * D, device=dev).to(bf)
        t = _time(lambda: WA.window_attention(q, kc, vc, md, spec, None))
        rows.append({"kernel": "window_attn prefill (causal, sink)", "heads": H, "kv_heads": G,
                     "dim": D, "vdim": Dv, "tokens": T, "ms": t * 1e3,
                     "mfma": WA.mfma_ok(spec, bf, bs),
                     "tflops": 2.0 * (D + Dv) * H * pairs / t / 1e12})
        kcd = torch.randn(nbd, bs, G * D, device=dev).to(bf)
        vcd = torch.randn(nbd, G * Dv, bs, device=dev).to(bf)
        qd = q[:B].contiguous()
        t = _time(lambda: WA.window_attention(qd, kcd, vcd, mdd, spec, None))
        rows.append({"kernel": "window_attn decode (causal, sink)", "heads": H, "kv_heads": G,
                     "batch": B, "context": L, "ms": t * 1e3,
                     "cache_GBps": B * L * G * (D + Dv) * 2 / t / 1e9})
        del kcd, vcd
        kc = torch.randn(nb, G, bs, D, device=dev).to(bf)
        vc = torch.randn(nb, G, D, bs, device=dev).to(bf)
        q3 = torch.randn(T, H, D, device=dev).to(bf) * 0.1
        qb2 = A.prefill_query_block(H, G, D, block_size=bs)
        w2 = A.build_prefill_work([T], qb2)
        wt = i32(w2)
        t = _time(lambda: A.paged_prefill(q3, kc, vc, bt, i32([T]), i32([0, T]), wt, len(w2) // 2,
                                          0.1))
        rows.append({"kernel": "paged_prefill (flash)", "heads": H, "kv_heads": G,
                     "head_dim": D, "tokens": T, "ms": t * 1e3,
                     "tflops": 2.0 * 2 * D * H * pairs / t / 1e12})
        kcd = torch.randn(nbd, G, bs, D, device=dev).to(bf)
        vcd = torch.randn(nbd, G, D, bs, device=dev).to(bf)
        lens = i32([L] * B)
        qd3 = q3[:B].contiguous()
        t = _time(lambda: A.paged_decode(qd3, kcd, vcd, btd, lens, 0.1))
        rows.append({"kernel": "paged_decode", "heads": H, "kv_heads": G, "batch": B,
                     "context": L, "ms": t * 1e3,
                     "cache_GBps": B * L * G * D * 2 * 2 / t / 1e9})
        del kcd, vcd
    # ---- sublayer boundary over four streams beside the fused add + RMS norm
    for W in (2048, 4096):
        Tn, NS = 8192, 4
        X = torch.randn(Tn, NS, W, device=dev)
        y = torch.randn(Tn, W, device=dev).to(bf)
        w1 = torch.zeros(W, device=dev).to(bf)
        mix = torch.eye(NS, device=dev)
        ones = torch.ones(NS, device=dev)
        t = _time(lambda: N.hyper_step(X, 1e-5, y, mix, ones, 0.5, ones, w1, 1.0))
        rows.append({"kernel": "hyper_step (4 streams)", "width": W, "rows": Tn, "ms": t * 1e3,
                     "GBps": Tn * W * (2 * 4 * NS + 2 + 2) / t / 1e9})
        res = torch.randn(Tn, W, device=dev).to(bf)
        t = _time(lambda: N.fused_add_rms_norm(y, res, w1, 1e-5))
        rows.append({"kernel": "fused_add_rms_norm", "width": W, "rows": Tn, "ms": t * 1e3,
                     "GBps": Tn * W * (2 + 2 + 2 + 2) / t / 1e9})
    # ---- router: softmax, correction, groups by their best member, identity outputs, gate
    for E, W in ((10, 1024), (18, 2048)):
        Tn = 8192
        x = torch.randn(Tn, W, device=dev).to(bf)
        wr = (torch.randn(E, W, device=dev) * 0.05).to(bf)
        wsg = (torch.randn(W, device=dev) * 0.05).to(bf)
        corr = torch.zeros(E, device=dev)
        t = _time(lambda: M.route_grouped(x, wr, 2, 2, 1, 1.0, scoring="softmax",
                                          group_score="max", correction=corr, identity=2,
                                          gate_w=wsg))
        rows.append({"kernel": "route_grouped (softmax, correction, identity, gate)",
                     "outputs": E, "width": W, "rows": Tn, "ms": t * 1e3,
                     "GBps": Tn * W * 2 / t / 1e9})
        t = _time(lambda: M.route_grouped(x, wr, 2, 2, 1, 1.0))
        rows.append({"kernel": "route_grouped (sigmoid)", "outputs": E, "width": W, "rows": Tn,
                     "ms": t * 1e3, "GBps": Tn * W * 2 / t / 1e9})
    for r_ in rows:
        print(json.dumps(r_), flush=True)
    print(json.dumps({"metric": "design_kernel_rates", "rows": rows}), flush=True)
    return 0
