"""Linear-attention recurrences with one decay number per head and token, on per-sequence state
slots -> csrc/kernels/linear_scan.hip.

Per head a matrix state S [dk, dv] (fp32, slot-resident) that every token scales and adds an
outer product to; the token's output reads the updated state:

    S_t = a_t S_(t-1) + b_t k_t v_t^T,        o_t = S_t^T q_t

* ``mode="decay"`` (retention): a_t = decay[h], b_t = 1.
* ``mode="exp_gates"`` (matrix memory with exponential gating): per head two gate
  pre-activations x_i, x_f per token; i = cap tanh(x_i / cap), f = logsigmoid(cap tanh(x_f /
  cap)) (cap 0: i = x_i, f = logsigmoid(x_f)); a running maximum m_t = max(f + m_(t-1), i) (m starts at 0) keeps the exponentials
  bounded: a_t = exp(f + m_(t-1) - m_t), b_t = exp(i - m_t); a normaliser n_t = a_t n_(t-1) +
  b_t k_t divides the output, o_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6).

q and k may be rotated by the token's position on their first ``rot_dims`` entries and are then
scaled; every head's output is divided by its root mean square, multiplied by an optional weight,
by silu or sigmoid of the gate columns and by ``out_scale``.

A sequence whose first row of the step is position 0 starts from the initial state whatever its
slot held, so freed slots are reused without clearing.  Batch layout: sequence ``s`` owns rows
``[cu[s], cu[s+1])`` of the step (``cu`` None: row ``s``, a pure decode step); ``slots[s]`` is its
state slot (< 0: padding row, skipped).

Prompt portions run a chunk-parallel form on the GPU (``chunk_plan``): the step's rows are cut
into chunks of 32 tokens, every chunk's own contribution to the state is formed in parallel, a
short scan over a sequence's chunks yields the state before each chunk, and the outputs of all
chunks are formed in parallel from that state and the chunk's own tokens.  The token-by-token
kernel serves decode steps (also inside captured graphs) and heads wider than 128.
"""

from __future__ import annotations

import dataclasses
import math
import os
from typing import Optional

import torch

from ._dispatch import check, lib, ptr, require, stream, use_hip


@dataclasses.dataclass
class ScanSpec:
    """Constants of one recurrent layer (device tensors are fp32)."""
    heads: int
    dim: int                        # dk
    vdim: int                       # dv
    mode: str                       # "decay" | "exp_gates"
    decay: Optional[torch.Tensor] = None        # [H] fp32 ("decay")
    cap: float = 0.0                            # gate soft cap ("exp_gates")
    inv_freq: Optional[torch.Tensor] = None     # [rot_dims / 2] fp32
    rot_dims: int = 0
    rot_half: bool = True
    qscale: float = 1.0
    kscale: float = 1.0
    gate_act: str = "silu"          # "silu" | "sigmoid"
    out_scale: float = 1.0
    eps: float = 0.0


class ScanState:
    """Per-sequence slots of one recurrent layer: S fp32 [slots, H, dk, dv]; with exponential
    gates also the normaliser n [slots, H, dk] and the running maximum m [slots, H]."""

    __slots__ = ("S", "n", "m")

    def __init__(self, S: torch.Tensor, n: Optional[torch.Tensor] = None,
                 m: Optional[torch.Tensor] = None):
        self.S, self.n, self.m = S, n, m

    @classmethod
    def allocate(cls, num_slots: int, spec: ScanSpec, device):
        z = lambda *shape: torch.zeros(*shape, dtype=torch.float32, device=device)
        n = max(1, num_slots)
        if spec.mode == "exp_gates":
            return cls(z(n, spec.heads, spec.dim, spec.vdim), z(n, spec.heads, spec.dim),
                       z(n, spec.heads))
        return cls(z(n, spec.heads, spec.dim, spec.vdim))

    @staticmethod
    def slot_bytes(spec: ScanSpec) -> int:
        per = spec.heads * spec.dim * spec.vdim
        if spec.mode == "exp_gates":
            per += spec.heads * (spec.dim + 1)
        return 4 * per


CHUNK = 32                 # tokens per chunk of the chunk-parallel form (linear_scan.hip LC)
CHUNK_MAX_DIM = 128        # ... and its largest dk / dv
CHUNK_MIN_ROWS = 48        # a sequence with at least this many rows in the step selects it
# tests and measurements: take the chunk-parallel form whenever a plan is handed over
FORCE_CHUNKED = os.environ.get("EIA_SCAN_FORCE_CHUNKED", "0") == "1"


class ChunkPlan:
    """A step's rows cut into chunks for the chunk-parallel form: ``chunks`` int32 [n, 4]
    (sequence, first row, tokens, 0), ``seq_first`` int32 [nseq + 1] (first chunk of every
    sequence), both on the device; ``rows`` the step's row count."""

    __slots__ = ("chunks", "seq_first", "n", "rows", "nseq", "longest")

    def __init__(self, chunks, seq_first, n, rows, nseq=1, longest=0):
        self.chunks, self.seq_first, self.n, self.rows = chunks, seq_first, n, rows
        self.nseq, self.longest = nseq, longest

    def pays(self, heads: int, dim: int, cus: int = 256) -> bool:
        """Whether the chunk-parallel form beats the token-by-token one for a layer of ``heads``
        heads up to ``dim`` wide: the latter walks the longest sequence with one workgroup per
        (sequence, head) at about 0.5 us a token (0.85 us above 64), the former costs about 5 ns
        (7 ns) per token and head over all rows (MI355X, measured on 4096-token prompts)."""
        wide = dim > 64
        serial = self.longest * (0.85 if wide else 0.5) * -(-self.nseq * heads // cus)
        return self.rows * heads * (0.0072 if wide else 0.0052) < serial


def chunk_plan(host_lens, device) -> Optional["ChunkPlan"]:
    """The chunk list of a step whose sequences own ``host_lens`` rows each (batch order), or
    None when no sequence is long enough for the chunk-parallel form to pay."""
    if not host_lens or max(host_lens) < CHUNK_MIN_ROWS:
        return None
    chunks, first, row = [], [0], 0
    for s, n in enumerate(host_lens):
        for lo in range(0, n, CHUNK):
            chunks += [s, row + lo, min(CHUNK, n - lo), 0]
        row += n
        first.append(len(chunks) // 4)
    return ChunkPlan(torch.tensor(chunks, dtype=torch.int32, device=device).view(-1, 4),
                     torch.tensor(first, dtype=torch.int32, device=device), len(chunks) // 4, row,
                     len(host_lens), max(host_lens))


def _seq_bounds(cu: Optional[torch.Tensor], nseq: int):
    if cu is None:
        return [(s, s + 1) for s in range(nseq)]
    c = cu.tolist()
    return [(c[s], c[s + 1]) for s in range(nseq)]


def _rotate(v: torch.Tensor, pos: torch.Tensor, spec: ScanSpec) -> torch.Tensor:
    """v fp32 [T, H, D]; pos [T]."""
    rd = spec.rot_dims
    if not rd:
        return v
    ang = pos.float()[:, None] * spec.inv_freq.float()[None, :rd // 2]       # [T, rd/2]
    cs, sn = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = v.clone()
    if spec.rot_half:
        a, b = v[..., :rd // 2], v[..., rd // 2:rd]
        out[..., :rd // 2], out[..., rd // 2:rd] = a * cs - b * sn, b * cs + a * sn
    else:
        a, b = v[..., 0:rd:2], v[..., 1:rd:2]
        out[..., 0:rd:2], out[..., 1:rd:2] = a * cs - b * sn, b * cs + a * sn
    return out


def linear_scan(fused: torch.Tensor, q_off: int, k_off: int, v_off: int, g_off: int,
                spec: ScanSpec, state: ScanState, slots: torch.Tensor,
                cu: Optional[torch.Tensor], nseq: int, positions: torch.Tensor,
                seq_lens: Optional[torch.Tensor] = None, norm_w: Optional[torch.Tensor] = None,
                i_off: int = 0, f_off: int = 0, out: Optional[torch.Tensor] = None,
                plan: Optional[ChunkPlan] = None) -> torch.Tensor:
    """fused [T, *]: rows of one fused projection holding q [H*dk], k [H*dk], v [H*dv], the gate
    [H*dv] (and, with exponential gates, the H input-gate and H forget-gate pre-activations) at
    the given column offsets -> y [T, H*dv] in fused's dtype (``out``: a view to write into).
    ``norm_w`` [H*dv]: weight after the head RMS norm.  Updates the sequences' slots.
    ``plan``: the step's ``chunk_plan`` -- the GPU then runs the chunk-parallel form (heads up to
    128 wide, outside graph capture)."""
    T = fused.shape[0]
    H, D, Dv = spec.heads, spec.dim, spec.vdim
    exp_gates = spec.mode == "exp_gates"
    if out is None:
        out = torch.empty(T, H * Dv, dtype=fused.dtype, device=fused.device)
    require(out.shape == (T, H * Dv) and out.dtype == fused.dtype and out.stride(1) == 1,
            "linear_scan: out layout")
    if not use_hip(fused):
        f = fused.float()
        q = _rotate(f[:, q_off:q_off + H * D].reshape(T, H, D), positions[:T], spec) * spec.qscale
        k = _rotate(f[:, k_off:k_off + H * D].reshape(T, H, D), positions[:T], spec) * spec.kscale
        v = f[:, v_off:v_off + H * Dv].reshape(T, H, Dv)
        g = f[:, g_off:g_off + H * Dv]
        y = torch.zeros(T, H, Dv)
        if exp_gates:
            soft = (lambda z: spec.cap * torch.tanh(z / spec.cap)) if spec.cap > 0 else \
                (lambda z: z)
            gi = soft(f[:, i_off:i_off + H])
            gf = torch.nn.functional.logsigmoid(soft(f[:, f_off:f_off + H]))
        for s, (lo, hi) in enumerate(_seq_bounds(cu, nseq)):
            sl = int(slots[s])
            if hi <= lo or sl < 0:
                continue
            fresh = int(positions[lo]) == 0
            S = torch.zeros(H, D, Dv) if fresh else state.S[sl].clone()
            if exp_gates:
                n = torch.zeros(H, D) if fresh else state.n[sl].clone()
                m = torch.zeros(H) if fresh else state.m[sl].clone()
            for t in range(lo, hi):
                kv = k[t][:, :, None] * v[t][:, None, :]
                if exp_gates:
                    m_new = torch.maximum(gf[t] + m, gi[t])
                    a, b = torch.exp(gf[t] + m - m_new), torch.exp(gi[t] - m_new)
                    S = a[:, None, None] * S + b[:, None, None] * kv
                    n = a[:, None] * n + b[:, None] * k[t]
                    m = m_new
                    den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
                    o = torch.einsum("hi,hij->hj", q[t], S) / den[:, None]
                else:
                    S = spec.decay.float()[:, None, None] * S + kv
                    o = torch.einsum("hi,hij->hj", q[t], S)
                y[t] = o / torch.sqrt((o * o).mean(-1, keepdim=True) + spec.eps)
            state.S[sl] = S
            if exp_gates:
                state.n[sl], state.m[sl] = n, m
        y = y.reshape(T, H * Dv)
        if norm_w is not None:
            y = y * norm_w.float()
        y = y * (torch.nn.functional.silu(g) if spec.gate_act == "silu" else torch.sigmoid(g))
        out.copy_((y * spec.out_scale).to(out.dtype))
        return out
    bf = fused.dtype == torch.bfloat16
    require(bf or fused.dtype == torch.float32, "linear_scan: bf16 or fp32")
    require(fused.stride(1) == 1 and max(q_off + H * D, k_off + H * D, v_off + H * Dv,
                                         g_off + H * Dv) <= fused.shape[1],
            "linear_scan: columns outside the row")
    require(spec.mode in ("decay", "exp_gates") and spec.gate_act in ("silu", "sigmoid"),
            "linear_scan: mode")
    require(state.S.dtype == torch.float32 and state.S.is_contiguous() and
            state.S.shape[1:] == (H, D, Dv), "linear_scan: state layout")
    if exp_gates:
        require(max(i_off, f_off) + H <= fused.shape[1] and state.n is not None and
                state.m is not None and state.n.is_contiguous() and state.m.is_contiguous() and
                spec.cap >= 0, "linear_scan: gates")
    else:
        require(spec.decay is not None and spec.decay.dtype == torch.float32 and
                spec.decay.is_cuda and spec.decay.numel() == H, "linear_scan: decay per head")
    require(spec.rot_dims == 0 or (spec.inv_freq is not None and spec.inv_freq.is_cuda and
                                   spec.inv_freq.dtype == torch.float32 and
                                   spec.inv_freq.numel() >= spec.rot_dims // 2 and
                                   spec.rot_dims <= D and spec.rot_dims % 2 == 0),
            "linear_scan: rotation")
    require(slots.dtype == torch.int32 and positions.dtype == torch.int32 and
            (cu is None or cu.dtype == torch.int32), "linear_scan: int32 metadata")
    require(norm_w is None or (norm_w.dtype == fused.dtype and norm_w.is_contiguous() and
                               norm_w.numel() == H * Dv), "linear_scan: norm weight")
    if (plan is not None and plan.n and max(D, Dv) <= CHUNK_MAX_DIM and cu is not None
            and plan.rows == T and (FORCE_CHUNKED or plan.pays(H, max(D, Dv)))
            and not torch.cuda.is_current_stream_capturing()):
        dev = fused.device
        f32 = lambda *shape: torch.empty(*shape, dtype=torch.float32, device=dev)
        wsS, wsG = f32(plan.n, H, D, Dv), f32(plan.n, H)
        wsN = f32(plan.n, H, D) if exp_gates else None
        la, lb, nm = (f32(T, H), f32(T, H), f32(T, H)) if exp_gates else (None, None, None)
        check(lib().eia_linear_scan_chunked(
            ptr(fused), fused.stride(0), q_off, k_off, v_off, g_off, i_off, f_off,
            ptr(spec.decay), ptr(spec.inv_freq), spec.rot_dims, 1 if spec.rot_half else 0,
            float(spec.qscale), float(spec.kscale), float(spec.cap), float(spec.out_scale),
            ptr(norm_w), ptr(state.S), ptr(state.n), ptr(state.m), ptr(slots), ptr(cu),
            ptr(positions), ptr(out), out.stride(0), float(spec.eps), nseq, H, D, Dv,
            1 if exp_gates else 0, 0 if spec.gate_act == "silu" else 1, 1 if bf else 0,
            ptr(plan.chunks), ptr(plan.seq_first), plan.n, ptr(wsS), ptr(wsN), ptr(wsG), ptr(la),
            ptr(lb), ptr(nm), stream(fused)), "linear_scan_chunked")
        return out
    check(lib().eia_linear_scan(
        ptr(fused), fused.stride(0), q_off, k_off, v_off, g_off, i_off, f_off, ptr(spec.decay),
        ptr(spec.inv_freq), spec.rot_dims, 1 if spec.rot_half else 0, float(spec.qscale),
        float(spec.kscale), float(spec.cap), float(spec.out_scale), ptr(norm_w), ptr(state.S),
        ptr(state.n), ptr(state.m), ptr(slots), ptr(cu), ptr(positions), ptr(seq_lens), ptr(out),
        out.stride(0), float(spec.eps), nseq, H, D, Dv, 1 if exp_gates else 0,
        0 if spec.gate_act == "silu" else 1, 1 if bf else 0, stream(fused)), "linear_scan")
    return out
