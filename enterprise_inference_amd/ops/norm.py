"""RMSNorm / LayerNorm ops (K5, K5b) -> csrc/kernels/norm.hip on the GPU."""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import reference as ref
from ._dispatch import check, lib, ptr, require, stream, use_hip


def _rows(x: torch.Tensor) -> torch.Tensor:
    return x.reshape(-1, x.shape[-1])


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float,
             out: Optional[torch.Tensor] = None) -> torch.Tensor:
    if not (use_hip(x) and x.dtype == torch.bfloat16):
        r = ref.rms_norm(x, weight, eps)
        if out is not None:
            out.copy_(r)
            return out
        return r
    x2 = _rows(x)
    require(x2.stride(-1) == 1, "rms_norm: last dim must be contiguous")
    o = torch.empty(x.shape, dtype=x.dtype, device=x.device) if out is None else out
    o2 = _rows(o)
    T, H = x2.shape
    check(lib().eia_rms_norm(ptr(o2), ptr(x2), None, ptr(weight), float(eps), T, H,
                             x2.stride(0), o2.stride(0), stream(x)), "rms_norm")
    return o


def fused_add_rms_norm(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor,
                       eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """residual <- x + residual (in place); returns (rms_norm(residual), residual)."""
    if not (use_hip(x, residual) and x.dtype == torch.bfloat16):
        out, r = ref.fused_add_rms_norm(x, residual, weight, eps)
        residual.copy_(r)
        return out, residual
    x2, r2 = _rows(x), _rows(residual)
    require(r2.is_contiguous() and x2.stride(-1) == 1, "fused_add_rms_norm: layout")
    T, H = x2.shape
    o = torch.empty_like(r2)
    check(lib().eia_rms_norm(ptr(o), ptr(x2), ptr(r2), ptr(weight), float(eps), T, H,
                             x2.stride(0), o.stride(0), stream(x)), "fused_add_rms_norm")
    return o.view(residual.shape), residual


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], eps: float,
               residual: Optional[torch.Tensor] = None) -> torch.Tensor:
    """LayerNorm; with ``residual`` computes residual <- x + residual first (in place)."""
    if not (use_hip(x) and x.dtype == torch.bfloat16):
        if residual is not None:
            out, r = ref.fused_add_layer_norm(x, residual, weight, bias, eps)
            residual.copy_(r)
            return out
        return ref.layer_norm(x, weight, bias, eps)
    x2 = _rows(x).contiguous()
    T, H = x2.shape
    o = torch.empty_like(x2)
    r2 = None if residual is None else _rows(residual)
    check(lib().eia_layer_norm(ptr(o), ptr(x2), ptr(r2), ptr(weight), ptr(bias), float(eps), T, H,
                               stream(x)), "layer_norm")
    return o.view(x.shape)


def post_norm_residual(y: torch.Tensor, weight: torch.Tensor, eps: float, x: torch.Tensor,
                       copy: bool = True) -> Optional[torch.Tensor]:
    """Sublayer-output norm with an fp32 residual stream: x += layernorm(y) * weight in place
    (no bias, variance = mean of squared deviations, all fp32); returns the new x in y's dtype
    for the next GEMMs (``copy``; an fp32 model reads x itself)."""
    if not use_hip(y, x):
        yf = y.float()
        d = yf - yf.mean(-1, keepdim=True)
        x += d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * weight.float()
        return x.to(y.dtype) if copy and y.dtype != torch.float32 else (x if copy else None)
    require(x.dtype == torch.float32 and x.is_contiguous() and y.stride(-1) == 1 and
            y.shape == x.shape and weight.dtype == y.dtype, "post_norm_residual: layout")
    bf = y.dtype == torch.bfloat16
    require(bf or y.dtype == torch.float32, "post_norm_residual: bf16 or fp32")
    T, W = x.shape
    xb = torch.empty(T, W, dtype=y.dtype, device=y.device) if (copy and bf) else None
    check(lib().eia_ln_residual(ptr(y), y.stride(0), ptr(weight), ptr(x), ptr(xb),
                                W, float(eps), T, W, 1 if bf else 0, stream(y)), "ln_residual")
    return xb if bf else (x if copy else None)


def layer_norm_f32(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """layernorm(x fp32 [T, W]) * weight (no bias) -> [T, W] in the weight's dtype."""
    if not use_hip(x):
        d = x - x.mean(-1, keepdim=True)
        return (d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * weight.float()).to(weight.dtype)
    require(x.dtype == torch.float32 and x.stride(-1) == 1, "layer_norm_f32: fp32 rows")
    bf = weight.dtype == torch.bfloat16
    require(bf or weight.dtype == torch.float32, "layer_norm_f32: bf16 or fp32 weight")
    T, W = x.shape
    out = torch.empty(T, W, dtype=weight.dtype, device=x.device)
    check(lib().eia_ln_f32in(ptr(x), x.stride(0), ptr(weight), ptr(out), W, float(eps), T, W,
                             1 if bf else 0, stream(x)), "ln_f32in")
    return out


def _group_rms(v: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    p = v.reshape(*v.shape[:-1], groups, v.shape[-1] // groups)
    return (p / torch.sqrt((p * p).mean(-1, keepdim=True) + eps)).reshape(v.shape)


def group_norm_step(x: torch.Tensor, groups: int, eps: float, y=None,
                    w_post: Optional[torch.Tensor] = None, add: Optional[torch.Tensor] = None,
                    w_next: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """One sublayer boundary of a model whose norms are RMS norms in ``groups`` equal consecutive
    parts (each part divided by its own root mean square, the row times a weight) around an fp32
    residual stream x [T, W], in one pass over the row:

        x += gnorm(y) * w_post      (y given: a sublayer's output joins the stream, in place)
        x += add                    (add given: fp32 rows, in place)
        h  = gnorm(x) * w_next      (w_next given: returned in the weights' dtype)

    All arithmetic is fp32; y and the weights are in the activation dtype.  y may also be a
    ``gemm.SplitK`` (the fp32 partial sums of the GEMM that produced it, plus its bias): the
    reduction then happens here, on fp32 values that were never rounded."""
    from .gemm import SplitK
    T, W = x.shape
    require(W % groups == 0, "group_norm_step: width not divisible by the group count")
    split = isinstance(y, SplitK)
    if split and use_hip(x) and W % 4:
        # the kernel sums partials in 16-byte units: other widths (no GEMM of the framework
        # produces them) take the unfused fp32 sum
        ys = y.part.sum(0) + (y.bias.float() if y.bias is not None else 0.0)
        x += _group_rms(ys, groups, eps) * w_post.float()
        y, split = None, False
        if add is None and w_next is None:
            return None
    if not use_hip(x):
        if split:
            y = y.part.sum(0) + (y.bias.float() if y.bias is not None else 0.0)
        if y is not None:
            x += _group_rms(y.float(), groups, eps) * w_post.float()
        if add is not None:
            x += add
        if w_next is None:
            return None
        return (_group_rms(x, groups, eps) * w_next.float()).to(w_next.dtype)
    ref_w = w_next if w_next is not None else w_post
    require(x.dtype == torch.float32 and x.is_contiguous(), "group_norm_step: fp32 stream")
    require(ref_w is not None and ref_w.dtype in (torch.bfloat16, torch.float32),
            "group_norm_step: bf16 or fp32 weights")
    bf = ref_w.dtype == torch.bfloat16
    part = ybias = yt = None
    sk = 0
    if split:
        require(y.M == T and y.N == W and y.part.is_contiguous() and y.part.dtype == torch.float32
                and w_post is not None and w_post.dtype == ref_w.dtype and w_post.numel() == W
                and (y.bias is None or y.bias.dtype == ref_w.dtype), "group_norm_step: partials")
        part, sk, ybias = y.part, y.sk, y.bias
    elif y is not None:
        require(y.shape == x.shape and y.stride(-1) == 1 and y.dtype == ref_w.dtype and
                w_post.dtype == ref_w.dtype and w_post.numel() == W, "group_norm_step: y layout")
        yt = y
    if add is not None:
        require(add.dtype == torch.float32 and add.is_contiguous() and add.shape == x.shape,
                "group_norm_step: add layout")
    h = None
    if w_next is not None:
        require(w_next.numel() == W, "group_norm_step: weight size")
        h = torch.empty(T, W, dtype=w_next.dtype, device=x.device)
    check(lib().eia_gnorm(ptr(yt), yt.stride(0) if yt is not None else 0, ptr(part), sk,
                          ptr(ybias), ptr(w_post), ptr(x), ptr(add), ptr(w_next), ptr(h), W,
                          float(eps), T, W, groups, 1 if bf else 0, stream(x)), "gnorm")
    return h


def residual_rms_step(x: torch.Tensor, eps: float, ys=(), w_next: Optional[torch.Tensor] = None
                      ) -> Optional[torch.Tensor]:
    """Boundary of a layer whose sublayers run side by side on one normed input, around an fp32
    residual stream x [T, W], in one pass over the row:

        x += y            for every y in ``ys`` (at most two sublayer outputs, un-normed, in place)
        h  = x / sqrt(mean(x^2) + eps) * w_next      (w_next given: returned in its dtype)

    All arithmetic is fp32.  A y is a tensor in the activation dtype or a ``gemm.SplitK`` (the
    fp32 partial sums of the GEMM that produced it, plus its bias), reduced here."""
    from .gemm import SplitK
    T, W = x.shape
    ys = [y for y in ys if y is not None]
    require(len(ys) <= 2, "residual_rms_step: at most two sublayer outputs")

    def dense(y):
        if isinstance(y, SplitK):
            return y.part.sum(0) + (y.bias.float() if y.bias is not None else 0.0)
        return y.float()

    if use_hip(x) and W % 4:
        # the kernel sums partials in 16-byte units; other widths (no GEMM of the framework
        # produces them) join the stream through the unfused fp32 sum
        for y in ys:
            if isinstance(y, SplitK):
                x += dense(y)
        ys = [y for y in ys if not isinstance(y, SplitK)]
    if not use_hip(x):
        for y in ys:
            x += dense(y)
        if w_next is None:
            return None
        return (x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w_next.float()).to(w_next.dtype)
    require(x.dtype == torch.float32 and x.is_contiguous(), "residual_rms_step: fp32 stream")
    dt = w_next.dtype if w_next is not None else None
    args = []
    for y in ys:
        if isinstance(y, SplitK):
            require(y.M == T and y.N == W and y.part.is_contiguous() and
                    y.part.dtype == torch.float32, "residual_rms_step: partials")
            dt = dt or (y.bias.dtype if y.bias is not None else None)
            args.append((None, 0, y.part, y.sk, y.bias))
        else:
            require(y.shape == x.shape and y.stride(-1) == 1, "residual_rms_step: y layout")
            dt = dt or y.dtype
            require(y.dtype == dt, "residual_rms_step: one activation dtype")
            args.append((y, y.stride(0), None, 0, None))
    for a in args:
        require(a[4] is None or a[4].dtype == dt, "residual_rms_step: bias dtype")
    dt = dt or torch.float32
    require(dt in (torch.bfloat16, torch.float32), "residual_rms_step: bf16 or fp32")
    while len(args) < 2:
        args.append((None, 0, None, 0, None))
    h = None
    if w_next is not None:
        require(w_next.numel() == W, "residual_rms_step: weight size")
        h = torch.empty(T, W, dtype=w_next.dtype, device=x.device)
    (y1, l1, p1, s1, b1), (y2, l2, p2, s2, b2) = args
    check(lib().eia_add_rms(ptr(y1), l1, ptr(p1), s1, ptr(b1), ptr(y2), l2, ptr(p2), s2, ptr(b2),
                            ptr(x), ptr(w_next), ptr(h), W, float(eps), T, W,
                            1 if dt == torch.bfloat16 else 0, stream(x)), "add_rms")
    return h


def hyper_step(X: torch.Tensor, eps: float, y=None, mix: Optional[torch.Tensor] = None,
               outw: Optional[torch.Tensor] = None, ymult: float = 1.0,
               in_next: Optional[torch.Tensor] = None, w_next: Optional[torch.Tensor] = None,
               w_offset: float = 0.0) -> Optional[torch.Tensor]:
    """Boundary of a sublayer whose residual is kept as several streams joined by
    hyper-connections, X fp32 [T, NS, W] updated in place, in one pass over the row:

        X_j <- sum_s mix[s, j] X_s + ymult * outw[j] * y        (y given; all streams at once)
        u    = sum_j in_next[j] X_j
        h    = u / sqrt(mean(u^2) + eps) * (w_offset + w_next)   (w_next given: returned)

    ``mix`` [NS, NS] (from, to), ``outw`` [NS] and ``in_next`` [NS] are fp32.  y is a tensor in the
    activation dtype or a ``gemm.SplitK`` (fp32 partial sums of the GEMM that produced it, plus
    its bias), reduced here.  NS = 1 with unit constants is the plain residual sum."""
    from .gemm import SplitK
    T, NS, W = X.shape
    split = isinstance(y, SplitK)
    if split and (not use_hip(X)):
        y = y.part.sum(0) + (y.bias.float() if y.bias is not None else 0.0)
        split = False
    if not use_hip(X):
        if y is not None:
            X.copy_(torch.einsum("sj,tsw->tjw", mix.float(), X)
                    + ymult * outw.float()[None, :, None] * y.float()[:, None, :])
        if w_next is None:
            return None
        u = torch.einsum("j,tjw->tw", in_next.float(), X)
        return (u / torch.sqrt((u * u).mean(-1, keepdim=True) + eps)
                * (w_offset + w_next.float())).to(w_next.dtype)
    require(X.dtype == torch.float32 and X.is_contiguous() and NS <= 8, "hyper_step: fp32 streams")
    dt = w_next.dtype if w_next is not None else (
        (y.bias.dtype if y.bias is not None else torch.bfloat16) if split else
        (y.dtype if y is not None else torch.float32))
    require(dt in (torch.bfloat16, torch.float32), "hyper_step: bf16 or fp32")
    for t in (mix, outw, in_next):
        require(t is None or (t.dtype == torch.float32 and t.is_cuda and t.is_contiguous()),
                "hyper_step: fp32 device constants")
    yt = part = ybias = None
    sk = 0
    if split:
        require(y.M == T and y.N == W and y.part.is_contiguous() and
                y.part.dtype == torch.float32 and (y.bias is None or y.bias.dtype == dt),
                "hyper_step: partials")
        part, sk, ybias = y.part, y.sk, y.bias
    elif y is not None:
        require(y.shape == (T, W) and y.stride(-1) == 1 and y.dtype == dt, "hyper_step: y layout")
        yt = y
    if y is not None:
        require(mix is not None and outw is not None and mix.numel() == NS * NS and
                outw.numel() == NS, "hyper_step: stream constants")
    h = None
    if w_next is not None:
        require(w_next.numel() == W and in_next is not None and in_next.numel() == NS,
                "hyper_step: next norm")
        h = torch.empty(T, W, dtype=dt, device=X.device)
    check(lib().eia_hyper_step(ptr(X), NS, W, ptr(yt), yt.stride(0) if yt is not None else 0,
                               ptr(part), sk, ptr(ybias), ptr(mix), ptr(outw), float(ymult),
                               ptr(in_next), ptr(w_next), float(w_offset), ptr(h),
                               h.stride(0) if h is not None else 0, float(eps), T,
                               1 if dt == torch.bfloat16 else 0, stream(X)), "hyper_step")
    return h
