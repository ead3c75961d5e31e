"""Gated activations (K7 epilogue form) -> csrc/kernels/activation.hip."""

from __future__ import annotations

import torch

from . import reference as ref
from ._dispatch import check, lib, ptr, require, stream, use_hip

_KIND = {"silu": 0, "swiglu": 0, "gelu_tanh": 1, "gelu_pytorch_tanh": 1, "gelu_new": 1,
         "gelu": 2, "gelu_erf": 2}


def act_and_mul(x, act: str = "silu") -> torch.Tensor:
    """act(x[:, :F]) * x[:, F:].  x may be a ``gemm.SplitK`` (fp32 partial sums of the [gate; up]
    GEMM): they are then summed inside the activation kernel."""
    from .gemm import SplitK
    kind = _KIND[act]
    if isinstance(x, SplitK):
        F = x.N // 2
        if x.bias is None and x.part.is_cuda and x.part.is_contiguous() and F % 4 == 0:
            out = torch.empty((x.M, F), dtype=torch.bfloat16, device=x.part.device)
            check(lib().eia_splitk_act_and_mul(ptr(x.part), x.sk, x.M, F, ptr(out), out.stride(0),
                                               kind, stream(out)), "splitk_act_and_mul")
            return out
        x = x.materialize()
    # (the kernel works on 16-byte units: other widths take the unfused form)
    if not (use_hip(x) and x.dtype == torch.bfloat16 and x.shape[-1] % 16 == 0
            and x.stride(-1) == 1):
        return ref.silu_and_mul(x) if kind == 0 else ref.gelu_and_mul(x) if kind == 1 else (
            (torch.nn.functional.gelu(x[..., :x.shape[-1] // 2].float()) *
             x[..., x.shape[-1] // 2:].float()).to(x.dtype))
    x2 = x.reshape(-1, x.shape[-1])
    T, F2 = x2.shape
    F = F2 // 2
    out = torch.empty((T, F), dtype=x.dtype, device=x.device)
    check(lib().eia_act_and_mul(ptr(out), ptr(x2), T, F, x2.stride(0), out.stride(0), kind,
                                stream(x)), "act_and_mul")
    return out.view(*x.shape[:-1], F)


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    return act_and_mul(x, "silu")


def activation(x: torch.Tensor, act: str) -> torch.Tensor:
    if act == "relu":
        return torch.relu(x)
    kind = _KIND[act]
    if not (use_hip(x) and x.dtype == torch.bfloat16 and x.is_contiguous() and x.numel() % 8 == 0):
        if kind == 0:
            return torch.nn.functional.silu(x.float()).to(x.dtype)
        return torch.nn.functional.gelu(x.float(), approximate="tanh" if kind == 1 else "none").to(x.dtype)
    out = torch.empty_like(x)
    check(lib().eia_act(ptr(out), ptr(x), x.numel(), kind, stream(x)), "activation")
    return out


def relu2(x: torch.Tensor) -> torch.Tensor:
    """Squared ReLU, max(x, 0)^2 (bf16 or fp32)."""
    if not (use_hip(x) and x.is_contiguous() and x.dtype in (torch.bfloat16, torch.float32)):
        r = torch.relu(x.float())
        return (r * r).to(x.dtype)
    out = torch.empty_like(x)
    check(lib().eia_relu2(ptr(out), ptr(x), x.numel(), 1 if x.dtype == torch.bfloat16 else 0,
                          stream(x)), "relu2")
    return out


def xielu(x, pq: torch.Tensor) -> torch.Tensor:
    """xIELU with the two learned numbers ``pq`` = (p, q) read from device memory:
    z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2, evaluated
    in fp32.  x [T, F] in the activation dtype (rows may be a column slice of a wider row), or a
    ``gemm.SplitK`` / ``gemm.SplitKSlice`` (fp32 partial sums of the up-projection, or of a fused
    projection that holds it, summed here) -> [T, F] in pq's dtype."""
    from .gemm import SplitK, SplitKSlice
    if isinstance(x, SplitKSlice):          # some columns of a fused projection's partials
        src = x.src
        if src.part.is_cuda and src.bias is None and x.n % 4 == 0 and x.off % 4 == 0 and \
                src.N % 4 == 0 and src.part.is_contiguous() and pq.dtype in (torch.bfloat16,
                                                                             torch.float32):
            out = torch.empty(src.M, x.n, dtype=pq.dtype, device=pq.device)
            check(lib().eia_xielu(None, 0, src.part.data_ptr() + 4 * x.off, src.sk, src.N, ptr(pq),
                                  ptr(out), out.stride(0), src.M, x.n,
                                  1 if pq.dtype == torch.bfloat16 else 0, stream(out)), "xielu")
            return out
        x = x.dense(pq.dtype)
    split = isinstance(x, SplitK)
    if split and not (x.part.is_cuda and x.bias is None and x.N % 4 == 0 and x.part.is_contiguous()):
        x = (x.part.sum(0) + (x.bias.float() if x.bias is not None else 0.0)).to(pq.dtype)
        split = False
    if not split and not use_hip(x):
        z = x.float()
        ap = torch.nn.functional.softplus(pq[0].float())
        aq = 0.5 + torch.nn.functional.softplus(pq[1].float())
        pos = ap * z * z + 0.5 * z
        neg = aq * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z
        return torch.where(z > 0, pos, neg).to(x.dtype)
    dt = pq.dtype
    require(dt in (torch.bfloat16, torch.float32) and pq.numel() == 2 and pq.is_contiguous(),
            "xielu: two numbers, bf16 or fp32")
    if split:
        T, F = x.M, x.N
        out = torch.empty(T, F, dtype=dt, device=pq.device)
        check(lib().eia_xielu(None, 0, ptr(x.part), x.sk, F, ptr(pq), ptr(out), out.stride(0), T, F,
                              1 if dt == torch.bfloat16 else 0, stream(out)), "xielu")
        return out
    require(x.dim() == 2 and x.stride(1) == 1 and x.dtype == dt, "xielu: row layout")
    T, F = x.shape
    out = torch.empty(T, F, dtype=dt, device=x.device)
    check(lib().eia_xielu(ptr(x), x.stride(0), None, 0, 0, ptr(pq), ptr(out), out.stride(0), T, F,
                          1 if dt == torch.bfloat16 else 0, stream(out)), "xielu")
    return out


def sigmoid_gate(a: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    """a * sigmoid(gate), element by element (fp32 inside) -> [T, N] contiguous.  gate [T, N]
    rows with a contiguous last dim (may be a column slice of a wider row); a is [T, N] likewise,
    or [H, T, V] with H * V == N -- the output of a batched product over heads -- whose heads are
    concatenated here (no transposing copy)."""
    if a.dim() == 3:
        H, T, V = a.shape
        if not use_hip(a, gate):
            return (a.transpose(0, 1).reshape(T, H * V).float()
                    * torch.sigmoid(gate.float())).to(a.dtype)
        require(a.stride(2) == 1 and gate.shape == (T, H * V), "sigmoid_gate: head layout")
        lda, a_sh, N = a.stride(1), a.stride(0), H * V
    else:
        if not use_hip(a, gate):
            return (a.float() * torch.sigmoid(gate.float())).to(a.dtype)
        require(a.dim() == 2 and a.shape == gate.shape and a.stride(1) == 1, "sigmoid_gate: layout")
        T, N = a.shape
        V, lda, a_sh = N, a.stride(0), 0
    require(gate.stride(1) == 1 and a.dtype == gate.dtype and
            a.dtype in (torch.bfloat16, torch.float32), "sigmoid_gate: layout")
    out = torch.empty(T, N, dtype=a.dtype, device=a.device)
    check(lib().eia_sigmoid_gate(ptr(a), lda, a_sh, V, ptr(gate), gate.stride(0), ptr(out),
                                 out.stride(0), T, N, 1 if a.dtype == torch.bfloat16 else 0,
                                 stream(a)), "sigmoid_gate")
    return out
