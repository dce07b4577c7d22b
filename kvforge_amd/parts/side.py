"""Per-layer token input: every layer owns a few columns of a second embedding table and feeds
the token's entries there into the residual stream, gated by the stream itself."""

from __future__ import annotations

import torch

from kvforge_amd.kernels import ops
from kvforge_amd.parts.base import Part, WeightSpec


class TokenSideInput(Part):
    """With ``e = table[token, first_col : first_col + dim]`` and the fp32 stream row ``x``:
    ``y = proj @ (gelu_tanh(gate @ x) * e)`` and ``x += y * rsqrt(mean(y^2) + eps) * weight`` (an RMS
    norm with a weight per coordinate).  Few rows take one kernel with fp32 sums throughout; many
    rows send the two products to the matrix kernels (in the engine's type, fp32 sums) with
    three row-wise kernels around them.

    ``table_name``: checkpoint name of the table ``[vocab, table_cols]`` that the layers share;
    ``gate [dim, hidden]``, ``proj [hidden, dim]`` and ``norm [hidden]`` live under the prefix.
    What the stream is still owed when this part runs (a bias, a product) is added by the same
    kernel."""

    replayable = True

    def __init__(self, prefix: str, hidden: int, dim: int, vocab: int, table_name: str,
                 table_cols: int, first_col: int, eps: float) -> None:
        if not 0 <= first_col <= table_cols - dim:
            raise ValueError(f"columns {first_col}..{first_col + dim} lie outside a table of {table_cols}")
        self.prefix, self.hidden, self.dim, self.vocab = prefix, int(hidden), int(dim), int(vocab)
        self.table_name, self.table_cols, self.first_col = table_name, int(table_cols), int(first_col)
        self.eps = float(eps)
        self.table = self.gate = self.proj = self.proj_t = self.weight = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {self.table_name: WeightSpec((self.vocab, self.table_cols)),
                self._name("gate"): WeightSpec((self.dim, self.hidden)),
                self._name("proj"): WeightSpec((self.hidden, self.dim)),
                self._name("norm"): WeightSpec((self.hidden,), init="norm", std=0.1)}

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        self.table = tensors[self.table_name]
        self.gate, self.proj = tensors[self._name("gate")], tensors[self._name("proj")]
        if not (self.table.dtype == self.gate.dtype == self.proj.dtype):
            self.table, self.gate, self.proj = self.table.float(), self.gate.float(), self.proj.float()
        self.weight = tensors[self._name("norm")].float().contiguous()
        # the projection once more, transposed: what the kernel for few rows reads side by side
        self.proj_t = self.proj.t().contiguous()

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        return {"elementwise", "gemm_generic"} | ({"gemm_bf16"} if dtype == torch.bfloat16 else set())

    def num_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.gate, self.proj, self.weight) if t is not None)

    def held_tensors(self) -> list[torch.Tensor]:
        return [t for t in (self.table, self.gate, self.proj, self.proj_t, self.weight) if t is not None]

    # rows up to which one kernel does everything, a workgroup per row with the two small
    # matrices read through the caches; beyond, the two products go to the matrix kernels
    FUSED_MAX_ROWS = 32

    def forward(self, residual: torch.Tensor, step, bias: torch.Tensor | None = None) -> None:
        """``bias`` (fp32 ``[hidden]``): a bias the stream is still owed, besides ``step.owed``."""
        n = residual.shape[0]
        owed = step.take_owed(residual)
        if n <= self.FUSED_MAX_ROWS:
            ops.token_side(residual, step.token_ids, self.table, self.first_col, self.gate, self.proj,
                           self.weight, self.eps, bias=bias, owed=owed, proj_t=self.proj_t)
            return
        ws, dt = step.ws, self.gate.dtype
        x = residual
        if dt != torch.float32:
            x = ws.buf("side_rows", (n, self.hidden), dt)
        ops.settle_cast(residual, bias, owed, x if x is not residual else None)
        a = ws.buf("side_a", (n, self.dim), dt)
        ops.gemm(x, self.gate, a)
        g = ws.buf("side_g", (n, self.dim), dt)
        ops.side_gate(a, step.token_ids, self.table, self.first_col, g)
        y = ws.buf("side_y", (n, self.hidden), torch.float32)
        ops.gemm(g, self.proj, y)
        ops.rms_add(residual, y, self.weight, self.eps)
