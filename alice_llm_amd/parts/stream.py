"""The residual stream of a step: a float32 [tokens, width] tensor and one pending branch.

Blocks push a branch output (with the norm that applies to it before the add, if any) and ask
for the normed stream that feeds their next part.  The add of the pending branch and the next
norm run as one kernel when both norms can be fused; otherwise the same result is computed in
separate kernels.  The stream itself is only ever added to, in 32-bit
(llama3.rs:14468-14470, 14555-14557).
"""
from __future__ import annotations

from typing import Optional

import torch

from ..hip import ops
from .base import FragmentActs, Precision


class ResidualStream:
    def __init__(self, x: torch.Tensor, precision: Precision):
        assert x.dtype == torch.float32 and x.dim() == 2
        self.x = x
        self.precision = precision
        self._branch: Optional[torch.Tensor] = None
        self._post = None

    def push(self, branch: torch.Tensor, post_norm=None) -> None:
        """Queue `x += post_norm(branch)`.  branch: float32 [T, H], or [S, T, H] partial sums."""
        if self._branch is not None:
            self.flush()
        self._branch = branch
        self._post = post_norm

    def _partials(self):
        b = self._branch
        return (b.shape[0], b) if b.dim() == 3 else (1, b)

    def flush(self) -> None:
        if self._branch is None:
            return
        n, b = self._partials()
        post = self._post
        fused = post.fused() if post is not None and hasattr(post, "fused") else None
        if post is None or fused is not None:
            w, eps, off = fused if fused is not None else (None, 0.0, 0.0)
            ops.add_norm(self.x, b, w, None, None, eps_post=eps, off_post=off, n_partials=n,
                         full_precision=self.precision.full)
        else:
            if n > 1:
                b = b.sum(dim=0)
            normed = post.forward(b.contiguous(), torch.float32)
            ops.add_norm(self.x, normed, None, None, None, full_precision=self.precision.full)
        self._branch = None
        self._post = None

    def normed(self, norm, out_dtype: Optional[torch.dtype] = None, fragments: bool = False):
        """Apply the pending add, then return norm(x) in the activation dtype (x itself if norm is None).
        fragments: the consumer reads fragment order; given where possible (see FragmentActs), else a tensor."""
        out_dtype = out_dtype or self.precision.act
        T, H = self.x.shape
        pre = norm.fused() if norm is not None and hasattr(norm, "fused") else None
        if fragments and pre is not None and out_dtype == torch.bfloat16 and FragmentActs.possible(self.precision, T, H):
            post = self._post
            pf = post.fused() if post is not None and hasattr(post, "fused") else None
            if self._branch is not None and not ((post is None or pf is not None) and (pf is None or pf[0].dtype == pre[0].dtype)):
                self.flush()
            n, b = self._partials() if self._branch is not None else (1, None)
            w_post, eps_post, off_post = pf if (pf is not None and b is not None) else (None, 0.0, 0.0)
            out = FragmentActs.empty(T, H, self.x.device)
            ops.add_norm(self.x, b, w_post, pre[0], out.data, eps_post=eps_post, eps_pre=pre[1], off_post=off_post,
                         off_pre=pre[2], n_partials=n, full_precision=self.precision.full, out_layout=ops.LAYOUT_FRAG16)
            self._branch = None
            self._post = None
            return out
        if self._branch is not None and (norm is None or pre is not None):
            post = self._post
            pf = post.fused() if post is not None and hasattr(post, "fused") else None
            same = pf is None or pre is None or pf[0].dtype == pre[0].dtype
            if (post is None or pf is not None) and same:
                n, b = self._partials()
                out = torch.empty((T, H), dtype=out_dtype, device=self.x.device)
                w_post, eps_post, off_post = pf if pf is not None else (None, 0.0, 0.0)
                w_pre, eps_pre, off_pre = pre if pre is not None else (None, 0.0, 0.0)
                ops.add_norm(self.x, b, w_post, w_pre, out, eps_post=eps_post, eps_pre=eps_pre,
                             off_post=off_post, off_pre=off_pre, n_partials=n,
                             full_precision=self.precision.full)
                self._branch = None
                self._post = None
                return out
        self.flush()
        if norm is None:
            return self.x.to(out_dtype)
        return norm.forward(self.x, out_dtype)

    def rows_normed(self, norm, rows: torch.Tensor, out_dtype: Optional[torch.dtype] = None, fragments: bool = False):
        """norm(x[rows]) after all pending adds: what the output head reads."""
        self.flush()
        out_dtype = out_dtype or self.precision.act
        pre = norm.fused() if norm is not None and hasattr(norm, "fused") else None
        if fragments and pre is not None and out_dtype == torch.bfloat16 and \
                FragmentActs.possible(self.precision, rows.numel(), self.x.shape[1]):
            out = FragmentActs.empty(rows.numel(), self.x.shape[1], self.x.device)
            ops.add_norm(self.x, None, None, pre[0], out.data, eps_pre=pre[1], off_pre=pre[2], rows=rows,
                         full_precision=self.precision.full, out_layout=ops.LAYOUT_FRAG16)
            return out
        if norm is None:
            return self.x.index_select(0, rows.long()).to(out_dtype)
        return norm.forward(self.x, out_dtype, rows=rows)
