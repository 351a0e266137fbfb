"""`torch.library` registration of the operator, so that it can stand in for `nn.Linear`-style call sites.

    torch.ops.hipkittensp.mxfp6_gemm(A, B, A_scale, B_scale, fmt_a, fmt_b, layout_a, layout_b, out_f32,
                                     bias, row_scale, col_scale, activation) -> C

is `tk_kernel.dispatch_micro` with the output allocated for the caller (bf16, or fp32 accumulators when out_f32):
C[..., N] = act(dq(A)[..., K] . dq(B)[N, K]^T * row_scale * col_scale + bias), everything after the product optional
and fused into the GEMM's epilogue.  A fake (meta) implementation gives shapes and dtypes to tracing tools
without touching the GPU.  `MXFP6Linear` keeps a weight quantised once, tile-major, and quantises its input on
the fly with the library's own kernel.  The reference has no counterpart: its harness calls the pybind module
directly (kernels/gemm/bf16fp32/bench.py:34).
"""
from __future__ import annotations

import torch

from . import tk_kernel


def _k_of(packed_width: int) -> int:
    if packed_width % 24:
        raise RuntimeError(f"packed width {packed_width} is not a whole number of 32-element blocks (24 bytes each)")
    return packed_width // 3 * 4


@torch.library.custom_op("hipkittensp::mxfp6_gemm", mutates_args=())
def mxfp6_gemm(A: torch.Tensor, B: torch.Tensor, A_scale: torch.Tensor, B_scale: torch.Tensor, fmt_a: int = 2, fmt_b: int = 2,
               layout_a: int = 0, layout_b: int = 0, out_f32: bool = False, bias: torch.Tensor | None = None,
               row_scale: torch.Tensor | None = None, col_scale: torch.Tensor | None = None, activation: str = "none") -> torch.Tensor:
    if B.dim() != 2:
        raise RuntimeError("B: expected a 2-D packed weight [N, 3K/4]")
    C = torch.empty(*A.shape[:-1], B.shape[0], dtype=torch.float32 if out_f32 else torch.bfloat16, device=A.device)
    tk_kernel.dispatch_micro(A, B, A_scale, B_scale, C, fmt_a, fmt_b, layout_a, layout_b, bias=bias, row_scale=row_scale,
                             col_scale=col_scale, activation=activation)
    return C


@mxfp6_gemm.register_fake
def _(A, B, A_scale, B_scale, fmt_a=2, fmt_b=2, layout_a=0, layout_b=0, out_f32=False, bias=None, row_scale=None, col_scale=None,
      activation="none"):
    K = _k_of(A.shape[-1])
    if B.dim() != 2 or B.shape[-1] != A.shape[-1]:
        raise RuntimeError("A and B disagree on K")
    if A_scale.shape[-1] != tk_kernel.scale_width(K, layout_a) or B_scale.shape[-1] != tk_kernel.scale_width(K, layout_b):
        raise RuntimeError("scale tensors do not match K and the layouts")
    return A.new_empty(*A.shape[:-1], B.shape[0], dtype=torch.float32 if out_f32 else torch.bfloat16)


class MXFP6Linear(torch.nn.Module):
    """y = act(x . W^T + bias) with W quantised once to MXFP6 (tile-major when its shape allows), x quantised per call,
    bias (float32 or bfloat16) and activation (None / "relu" / "gelu" / "silu") fused into the GEMM."""

    def __init__(self, weight: torch.Tensor, fmt_w: int = tk_kernel.E2M3, fmt_x: int = tk_kernel.E2M3, bias: torch.Tensor | None = None,
                 activation: str | None = None):
        super().__init__()
        self.activation = activation or "none"
        if bias is not None and (bias.dim() != 1 or bias.shape[0] != weight.shape[0]):
            raise RuntimeError("bias: expected [out_features]")
        self.register_buffer("bias", None if bias is None else bias.detach().to(torch.float32 if bias.dtype != torch.bfloat16 else torch.bfloat16).contiguous())
        if weight.dim() != 2 or weight.shape[1] % 32:
            raise RuntimeError("weight: expected [out_features, in_features] with in_features % 32 == 0")
        self.out_features, self.in_features = weight.shape
        self.fmt_w, self.fmt_x = fmt_w, fmt_x
        self.layout_w = tk_kernel.LAYOUT_TILE if (weight.shape[0] % 32 == 0 and weight.shape[1] % 128 == 0) else tk_kernel.LAYOUT_ROW
        packed, scales = tk_kernel.quantize(weight.detach().to(torch.float32).contiguous(), fmt_w, self.layout_w)
        self.register_buffer("weight_packed", packed)
        self.register_buffer("weight_scale", scales)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        # the input tile-major too from 64 rows on (a whole number of 32-row tiles): the tiled and block kernels then need
        # no re-layout and load whole cache lines; fewer rows stay row-major for the skinny kernel
        rows = x.numel() // x.shape[-1]
        layout_x = tk_kernel.LAYOUT_TILE if (rows >= 64 and rows % 32 == 0 and self.in_features % 128 == 0) else tk_kernel.LAYOUT_ROW
        xp, xs = tk_kernel.quantize((x if x.dtype == torch.bfloat16 else x.to(torch.float32)).contiguous(), self.fmt_x, layout_x)
        return mxfp6_gemm(xp, self.weight_packed, xs, self.weight_scale, self.fmt_x, self.fmt_w, layout_x, self.layout_w,
                          bias=self.bias, activation=self.activation)
