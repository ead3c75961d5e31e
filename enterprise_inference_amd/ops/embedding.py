"""Token embedding with a hashed bigram term -> csrc/kernels/embed.hip.

    x = embed[tok] * scale + bigram[(prev * mul_prev + tok * mul_cur) mod buckets]

and the table's last row (index ``buckets``) for the first token of a sequence.  The output is
the fp32 residual of a decoder that keeps ``streams`` equal copies of it, [T, streams, W].  The
previous token of a step's first row lives in the sequence's state slot (``last_tok`` int32
[slots]), which also receives the step's last token -- the host need not know a decode row's
input token (it may still be in flight from the previous step's sampler).

Batch layout: sequence ``s`` owns rows ``[cu[s], cu[s+1])`` (``cu`` None: row ``s``);
``slots[s]`` < 0 is a padding row.
"""

from __future__ import annotations

from typing import Optional

import torch

from ._dispatch import check, lib, ptr, require, stream, use_hip


def bigram_embed(ids: torch.Tensor, embed: torch.Tensor, scale: float,
                 bigram: Optional[torch.Tensor], buckets: int, mul_prev: int, mul_cur: int,
                 last_tok: Optional[torch.Tensor], slots: Optional[torch.Tensor],
                 cu: Optional[torch.Tensor], nseq: int, positions: torch.Tensor,
                 streams: int = 1) -> torch.Tensor:
    """-> fp32 [T, streams, W]; updates ``last_tok`` at the sequences' slots.  ``bigram`` None:
    the plain scaled embedding."""
    T = ids.shape[0]
    V, W = embed.shape
    if not use_hip(embed):
        tok = ids[:T].long().clamp(0, V - 1)
        x = embed[tok].float() * scale
        if bigram is not None:
            prev = torch.full((T,), -1, dtype=torch.long)
            c = cu.tolist() if cu is not None else list(range(nseq + 1))
            for s in range(nseq):
                lo, hi = c[s], c[s + 1]
                sl = int(slots[s]) if slots is not None else -1
                if hi <= lo:
                    continue
                prev[lo + 1:hi] = ids[lo:hi - 1].long()
                if int(positions[lo]) > 0 and sl >= 0 and last_tok is not None:
                    prev[lo] = int(last_tok[sl])
                if sl >= 0 and last_tok is not None:
                    last_tok[sl] = int(ids[hi - 1])
            row = torch.where(prev < 0, torch.full_like(prev, buckets),
                              (prev * mul_prev + tok * mul_cur) % buckets)
            x = x + bigram[row].float()
        return x[:, None, :].repeat(1, streams, 1).contiguous()
    bf = embed.dtype == torch.bfloat16
    require((bf or embed.dtype == torch.float32) and embed.is_contiguous(), "bigram_embed: table")
    require(bigram is None or (bigram.dtype == embed.dtype and bigram.is_contiguous() and
                               bigram.shape == (buckets + 1, W)), "bigram_embed: bigram table")
    require(ids.dtype == torch.int32 and positions.dtype == torch.int32 and
            (slots is None or slots.dtype == torch.int32) and
            (cu is None or cu.dtype == torch.int32) and
            (last_tok is None or (last_tok.dtype == torch.int32 and last_tok.is_contiguous())),
            "bigram_embed: int32 metadata")
    X = torch.empty(T, streams, W, dtype=torch.float32, device=embed.device)
    check(lib().eia_bigram_embed(ptr(ids), ptr(embed), float(scale), ptr(bigram), int(buckets),
                                 int(mul_prev), int(mul_cur), ptr(last_tok), ptr(slots), ptr(cu),
                                 nseq, ptr(positions), ptr(X), streams, W, V, T, 1 if bf else 0,
                                 stream(embed)), "bigram_embed")
    return X
