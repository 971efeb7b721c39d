"""y = x @ W^T for the projections of a step.

float32: hand-written kernels with true 32-bit multiply-add and one summation order
(tiled, or weight-streaming for up to 64 rows; row-wise deterministic, equal bits).  bfloat16: hand-written MFMA kernels for up to 64 rows, else
the library product that torch binds (as the reference's nn.Linear does).

Decode steps of few rows (bfloat16, up to 16) can do without the kernels between the
products: a part's last product adds its result into the float32 residual stream itself
(``linear(..., add_into=StreamSink)`` -> ``Added``), leaving bf16(stream * gamma) for the
norm that reads the stream next and the rows' sums of squares; that norm then hands both on
as a ``DeferredNorm``, and the product after it applies the rows' scale to its own result
(an RMSNorm is a row scale times a column scale, and a product is linear in the row scale).
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from tokamak_amd.kernels import ops


# A product adds into the stream itself (one block walking the whole of K for 16 columns)
# only if K is short: up to one chunk of 256 for each of a block's sixteen waves.  With a
# longer K the split product and the norm kernel after it are as fast (measured: the o
# projection of an 8B-shaped layer gains 2 us, its down projection nothing).
ADD_INTO_MAX_K = 16 * 256
GATED_WHOLEK_MAX_BYTES = 32 << 20   # gate and up together, up to which the whole-K form takes the gated product


@dataclass
class StreamSink:
    """Offered to a part whose last product may add its result into the residual stream
    itself: the float32 stream [M, H], and the weight [H] of the RMSNorm that reads the
    stream next (None if what follows is not one)."""

    resid: torch.Tensor
    gamma: torch.Tensor | None


@dataclass
class Added:
    """What ``linear(..., add_into=sink)`` returns in place of its result when the product
    has added it into the stream: ``sumsq`` [slabs, M], the sums of squares of every row of
    the new stream over slabs of columns, and, if the sink named a norm weight ``gamma``,
    ``scaled`` = bf16(stream * gamma)."""

    sumsq: torch.Tensor
    scaled: torch.Tensor | None
    gamma: torch.Tensor | None


@dataclass
class DeferredNorm:
    """An RMSNorm of the stream that is not finished: ``scaled`` = bf16(resid * weight) and
    the rows' sums of squares are at hand, the rows' scale rsqrt(mean(resid^2) + eps) is still
    to be applied.  ``linear`` and ``gated_linear`` take it in place of a tensor and apply the
    scale to their result; ``materialize()`` runs the norm kernel on the stream instead.  It
    must be used before the stream is written again."""

    resid: torch.Tensor
    weight: torch.Tensor
    eps: float
    dtype: torch.dtype
    scaled: torch.Tensor
    sumsq: torch.Tensor

    @property
    def shape(self):
        return self.resid.shape

    @property
    def device(self):
        return self.resid.device

    def materialize(self) -> torch.Tensor:
        out = torch.empty(self.resid.shape, dtype=self.dtype, device=self.resid.device)
        ops.add_rmsnorm(self.resid, None, self.weight, self.eps, out)
        return out


def _few_rows_fit(m: int, x: torch.Tensor, weight: torch.Tensor, rows: int) -> bool:
    """Whether the fused forms for few rows take these operands."""
    from tokamak_amd.kernels import gemm_bf16

    return (0 < m <= rows and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
            and x.dim() == 2 and x.stride(1) == 1 and weight.stride(1) == 1 and gemm_bf16.skinny_fits(x, weight))


def linear(x: torch.Tensor | DeferredNorm, weight: torch.Tensor, out_dtype: torch.dtype | None = None,
           allow_partials: bool = False, add_into: StreamSink | None = None) -> torch.Tensor | Added:
    """``x`` [M, K], ``weight`` [N, K] -> [M, N] in ``out_dtype`` (default: x's).

    With ``allow_partials`` the result may instead be float32 partial sums
    [P, M, N] that the consumer adds (the norm kernel and the q/k norm kernel do).
    With ``add_into`` the product may add its result into the sink's stream itself and
    return ``Added`` (bfloat16 steps of up to 16 rows do).
    """
    from tokamak_amd.kernels import gemm_bf16

    out_dtype = out_dtype or x.dtype
    m, n = x.shape[0], weight.shape[0]
    if isinstance(x, DeferredNorm):
        if (_few_rows_fit(m, x.scaled, weight, ops.ROW_SCALE_MAX_ROWS) and n >= gemm_bf16.STREAM_MIN_ROWS_OUT
                and x.sumsq.shape[0] <= ops.ROW_SCALE_MAX_SLABS):
            splits = gemm_bf16.stream_splits(n, weight.shape[1], m) if allow_partials else 1
            if splits > 1:
                out = torch.empty((splits, m, n), dtype=torch.float32, device=x.device)
                return out[:ops.gemm_stream(x.scaled, weight, out, splits=splits, sumsq=x.sumsq, eps=x.eps)]
            out = torch.empty((m, n), dtype=out_dtype, device=x.device)
            ops.gemm_stream(x.scaled, weight, out, sumsq=x.sumsq, eps=x.eps)
            return out
        x = x.materialize()
    if m == 0:
        return torch.empty((0, n), dtype=out_dtype, device=x.device)
    if x.dtype == torch.float32:
        out = torch.empty((m, n), dtype=out_dtype, device=x.device)
        ops.gemm_tiled(x, weight, out)
        return out
    if (add_into is not None and weight.shape[1] <= ADD_INTO_MAX_K and _few_rows_fit(m, x, weight, ops.WHOLEK_MAX_ROWS)
            and _sink_fits(add_into, m, n)):
        sumsq, scaled = ops.gemm_wholek_add(x, weight, add_into.resid, add_into.gamma)
        return Added(sumsq, scaled, add_into.gamma)
    return gemm_bf16.gemm(x, weight, out_dtype, allow_partials)


def _sink_fits(sink: StreamSink, m: int, n: int) -> bool:
    r, g = sink.resid, sink.gamma
    return (r.dtype == torch.float32 and r.shape == (m, n) and r.stride(1) == 1 and r.stride(0) % 4 == 0
            and r.data_ptr() % 16 == 0 and n % 4 == 0
            and (g is None or (g.dtype == torch.float32 and g.numel() == n and g.is_contiguous() and g.data_ptr() % 16 == 0)))


def gated_linear(x: torch.Tensor | DeferredNorm, gate_up: torch.Tensor) -> torch.Tensor:
    """silu(x @ gate^T) * (x @ up^T) for ``gate_up`` = [gate; up] ([2I, K]) -> [M, I].

    bfloat16 with up to 64 rows: one fused weight-streaming kernel.  Otherwise
    the product, then the SiLU-gate kernel.
    """
    m = x.shape[0]
    inter = gate_up.shape[0] // 2
    # A very small pair of matrices (0.6B-shaped: 13 MB) goes to the whole-K form, whose blocks of 16
    # columns let their waves split K, which the streaming kernel cannot do under the gate: in a
    # decode step 6.6 us against 8.6 with blocks of four waves and 7.8 with blocks of two (whose start
    # costs more than their size saves there); from 50 MB on the streaming kernel is ahead.
    small = 2 * gate_up.numel() <= GATED_WHOLEK_MAX_BYTES
    if isinstance(x, DeferredNorm):
        if _few_rows_fit(m, x.scaled, gate_up, ops.ROW_SCALE_MAX_ROWS) and x.sumsq.shape[0] <= ops.ROW_SCALE_MAX_SLABS:
            out = torch.empty((m, inter), dtype=x.dtype, device=x.device)
            if small and m <= ops.WHOLEK_MAX_ROWS:
                ops.gemm_wholek(x.scaled, gate_up, out, gated=True, sumsq=x.sumsq, eps=x.eps)
            else:
                ops.gemm_stream_swiglu(x.scaled, gate_up, out, sumsq=x.sumsq, eps=x.eps)
            return out
        x = x.materialize()
    out = torch.empty((m, inter), dtype=x.dtype, device=x.device)
    if m == 0:
        return out
    if x.dtype == torch.bfloat16 and m <= 64:
        from tokamak_amd.kernels import gemm_bf16

        if gemm_bf16.skinny_fits(x, gate_up):
            if small and _few_rows_fit(m, x, gate_up, ops.WHOLEK_MAX_ROWS):
                ops.gemm_wholek(x, gate_up, out, gated=True)
            else:
                ops.gemm_stream_swiglu(x, gate_up, out)
            return out
    ops.silu_mul(linear(x, gate_up), out)
    return out
