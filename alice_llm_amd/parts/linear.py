"""A dense projection y = x W^T: the building brick of mixers, feed-forwards and the head.

Orientation as in the reference: W is [out, in] row-major and y[r] = sum_c W[r, c] x[c]
(gguf.rs:4063-4074).  The bfloat16 path rounds a weight stored in 32-bit to bfloat16 and rearranges
it once, at load, into the fragment layout that the MFMA kernels read (llama3.rs:12889-12890 converts
once at load as well); only when the run was asked to keep stored dtypes does such a weight stay
row-major 32-bit and run on the plain kernel.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..hip import ops
from .base import FragmentActs, Precision

# Whether the bfloat16 path rearranges its weights for the MFMA kernels.  The kernels refuse
# nothing: shapes they do not cover are padded inside the layout.
USE_FRAGMENT_LAYOUT = True


class Linear:
    def __init__(self, in_features: int, out_features: int, precision: Precision, *,
                 epilogue: int = ops.EPI_NONE, epi_param: float = 0.0):
        self.k = in_features
        self.n = out_features               # columns of y (half of W's rows for GeGLU)
        self.precision = precision
        self.epilogue = epilogue
        self.epi_param = epi_param
        self.weight: Optional[torch.Tensor] = None
        self.layout = ops.LAYOUT_ROW

    @property
    def weight_rows(self) -> int:
        return self.n * (2 if self.epilogue == ops.EPI_GEGLU else 1)

    def load(self, w: torch.Tensor) -> None:
        """Takes a row-major [rows, in] device tensor in its stored dtype."""
        if tuple(w.shape) != (self.weight_rows, self.k):
            raise ValueError(f"weight must be {(self.weight_rows, self.k)}, found {tuple(w.shape)}")
        w = self.precision.matrix(w)
        if (USE_FRAGMENT_LAYOUT and self.precision.name == "bfloat16" and w.dtype == torch.bfloat16
                and ops.fragment_layout_supported(self.weight_rows, self.k, self.epilogue)):
            self.weight = ops.to_frag16(w.contiguous())
            self.layout = ops.LAYOUT_FRAG16
        else:
            self.weight = w.contiguous()
            self.layout = ops.LAYOUT_ROW

    def nbytes(self) -> int:
        return self.weight.numel() * self.weight.element_size()

    @property
    def accepts_fragment_input(self) -> bool:
        """Whether activations in fragment order can be fed in (the MFMA kernels, inner width a multiple of 32)."""
        return self.layout == ops.LAYOUT_FRAG16 and self.k % 32 == 0

    def can_write_fragments(self, rows: int) -> bool:
        return (self.layout == ops.LAYOUT_FRAG16 and rows >= 1 and self.n % 32 == 0
                and self.epilogue != ops.EPI_SOFTCAP and self.precision.act == torch.bfloat16)

    def __call__(self, x, out_dtype: torch.dtype, *, allow_partials: bool = False,
                 variant: int = ops.LINEAR_AUTO, out_fragments: bool = False):
        """x: [M, k] tensor or FragmentActs.  Returns [M, n], or [S, M, n] float32 partial sums when the
        kernel prefers to split the inner dimension and the caller can add them up (allow_partials), or a
        FragmentActs when out_fragments is asked for (bfloat16)."""
        M = x.shape[0]
        frag_in = isinstance(x, FragmentActs)
        if frag_in and not self.accepts_fragment_input:
            raise ValueError("this projection cannot read activations in fragment order")
        split = 1
        if allow_partials and self.epilogue == ops.EPI_NONE and out_dtype == torch.float32:
            split = ops.linear_split_hint(M, self.n, self.k, self.layout)
        if out_fragments:
            if not self.can_write_fragments(M) or out_dtype != torch.bfloat16:
                raise ValueError("this projection cannot write activations in fragment order here")
            out = FragmentActs.empty(M, self.n, x.device)
            y = out.data
        else:
            shape = (split, M, self.n) if split > 1 else (M, self.n)
            out = y = torch.empty(shape, dtype=out_dtype, device=x.device)
        ops.linear(x.data if frag_in else x, self.weight, y, n_out=self.n, k_in=self.k, layout=self.layout,
                   epilogue=self.epilogue, epi_param=self.epi_param, split_k=split, variant=variant,
                   full_precision=self.precision.full, rows=M,
                   x_layout=ops.LAYOUT_FRAG16 if frag_in else ops.LAYOUT_ROW,
                   y_layout=ops.LAYOUT_FRAG16 if out_fragments else ops.LAYOUT_ROW)
        return out
