"""Matrix-memory recurrence (the mLSTM of xLSTM) as a mixer with per-request state.

Per head a matrix ``S [key_dim, value_dim]``, a normaliser ``n [key_dim]`` and a running maximum
``m``, all zero before a sequence's first token.  For a token with projections ``q`` (times
``key_dim^-1/2``), ``k``, ``v`` and log gates ``li = cap(W_i x + b_i)``,
``lf = logsigmoid(cap(W_f x + b_f))`` with ``cap(z) = gate_cap * tanh(z / gate_cap)``::

    a = lf + m;   m' = max(a, li)
    S' = exp(a - m') S + exp(li - m') k v^T;   n' = exp(a - m') n + exp(li - m') k
    o  = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)

Every head's ``o`` is divided by its root mean square, the heads side by side are multiplied by
a weight vector and by ``sigmoid(W_g x)``, and projected out.  Gates, state and everything that
enters the recurrence besides the projected q, k, v rows are fp32 in every mode; the gates'
pre-activations come from a product with fp32 sums stored in fp32.
"""

from __future__ import annotations

import torch

from kvforge_amd.kernels import ops
from kvforge_amd.parts.base import LayerState, Mixer, StateSpec, WeightSpec, add_product
from kvforge_amd.registry import register_mixer


@register_mixer("mlstm")
class MatrixLSTM(Mixer):
    """``names``: checkpoint names under the prefix, by ``q k v g o norm i f``; a gate's bias is
    ``<name><bias_suffix>``.  The state of a request is one slot of
    ``heads * (key_dim * value_dim + key_dim + 1)`` fp32 numbers per call of the layer."""

    NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "i": "i", "f": "f"}

    replayable = True
    cache_spec = None

    def __init__(self, prefix: str, hidden: int, heads: int, key_dim: int, value_dim: int,
                 gate_cap: float, norm_eps: float, names: dict[str, str] | None = None,
                 bias_suffix: str = ".b") -> None:
        self.prefix, self.hidden = prefix, int(hidden)
        self.H, self.dk, self.dv = int(heads), int(key_dim), int(value_dim)
        if min(self.H, self.dk, self.dv) <= 0 or self.dk > 256:
            raise ValueError(f"mlstm kernels take key sizes up to 256, got heads {heads}, sizes {key_dim} / {value_dim}")
        self.gate_cap, self.norm_eps = float(gate_cap), float(norm_eps)
        if not self.gate_cap > 0.0:
            raise ValueError(f"gate_cap must be positive, got {gate_cap}")
        self.names, self.bias_suffix = dict(self.NAMES, **(names or {})), bias_suffix
        self.state_spec = StateSpec((ops.mlstm_state_floats(self.H, self.dk, self.dv),), torch.float32)
        self.w_rows = self.w_gates = self.gate_bias = self.head_weight = self.w_o = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        h, H, dk, dv = self.hidden, self.H, self.dk, self.dv
        n = lambda key: self._name(self.names[key])  # noqa: E731
        return {n("q"): WeightSpec((H * dk, h)), n("k"): WeightSpec((H * dk, h)),
                n("v"): WeightSpec((H * dv, h)), n("g"): WeightSpec((H * dv, h)),
                n("o"): WeightSpec((h, H * dv)), n("norm"): WeightSpec((H * dv,), init="norm", std=0.1),
                n("i"): WeightSpec((H, h)), n("i") + self.bias_suffix: WeightSpec((H,), std=1.0),
                n("f"): WeightSpec((H, h)), n("f") + self.bias_suffix: WeightSpec((H,), std=1.0)}

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        t = lambda key, tail="": tensors[self._name(self.names[key]) + tail]  # noqa: E731
        mats = [t("q"), t("k"), t("v"), t("g")]
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        # one product for q, k, v and the output gate: their heads side by side in that order
        self.w_rows = torch.cat(mats, dim=0).contiguous()
        # the gates' product: input gates' rows, then forget gates', padded with zero rows to a
        # multiple of 16 (which every product kernel takes); its 32-bit sums are stored in fp32
        gi, gf = t("i"), t("f")
        if gi.dtype != gf.dtype:
            gi, gf = gi.float(), gf.float()
        self.G_pad = -(-2 * self.H // 16) * 16
        self.w_gates = torch.cat([gi, gf, gi.new_zeros(self.G_pad - 2 * self.H, self.hidden)], dim=0).contiguous()
        self.gate_bias = torch.cat([t("i", self.bias_suffix), t("f", self.bias_suffix)], dim=0).float().contiguous()
        self.head_weight = t("norm").float().contiguous()
        self.w_o = t("o")

    def seal(self) -> None:
        self.w_rows, self.w_o = ops.streamed(ops.plain_of(self.w_rows)), ops.streamed(ops.plain_of(self.w_o))
        self.w_gates = ops.streamed(ops.plain_of(self.w_gates))

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        return {"mlstm", "gemm_generic"} | ({"gemm_bf16"} if dtype == torch.bfloat16 else set())

    def _small(self) -> list[torch.Tensor]:
        return [x for x in (ops.plain_of(self.w_gates), self.gate_bias, self.head_weight) if x is not None]

    def num_bytes(self) -> int:
        return sum(x.numel() * x.element_size()
                   for x in (*map(ops.plain_of, (self.w_rows, self.w_o)), *self._small()) if x is not None)

    def held_tensors(self) -> list[torch.Tensor]:
        return (ops.copies_of(self.w_rows) + ops.copies_of(self.w_o) + ops.copies_of(self.w_gates)
                + [x for x in (self.gate_bias, self.head_weight) if x is not None])

    def _longest_runs(self, step, n: int) -> dict | None:
        """What the passes over all chunks at once need for the step's longest runs: the chunk
        and run tables (made once a step for all layers of this key size, sent along with the
        batch) and scratch from the step's workspace.  ``None`` when no run is that long."""
        key = ("mlstm.longest_runs", ops.mlstm_chunk_len(self.dk))
        plan = step.scratch.get(key)
        if plan is None:
            chunks, runs = ops.mlstm_multi_plan(step.q_lens, self.dk)
            plan = (step.upload_ints(chunks).view(-1, 4), step.upload_ints(runs).view(-1, 3)) if chunks else ()
            step.scratch[key] = plan
        if not plan:
            return None
        out = {"chunks": plan[0], "runs": plan[1]}
        for name, (shape, dtype) in ops.mlstm_multi_scratch(n, plan[0].shape[0], self.H, self.dk, self.dv).items():
            out[name] = step.ws.buf("mlstm_multi_" + name, shape, dtype)
        return out

    def forward(self, x, step, layer: LayerState, residual) -> None:
        """``x``: normalised activations."""
        if layer.state is None:
            raise RuntimeError("the matrix-memory mixer needs a state slot per request")
        n = x.shape[0]
        H, dk, dv = self.H, self.dk, self.dv
        ws, act = step.ws, step.act_dtype
        step.settle()
        rows = ws.buf("mlstm_rows", (n, 2 * H * dk + 2 * H * dv), act)
        ops.gemm(x, self.w_rows, rows)
        gates = ws.buf("mlstm_gates", (n, self.G_pad), torch.float32)
        ops.gemm(x, self.w_gates, gates)
        raw = ws.buf("mlstm_raw", (n, H * dv), torch.float32)
        # which of the two kernels have work is known from the runs' lengths (all ones in a
        # captured step of single tokens, so a replay launches what the capture launched)
        long_runs = any(ops.MLSTM_CHUNK_FROM <= q < ops.MLSTM_MULTI_FROM for q in step.q_lens)
        short_runs = any(q < ops.MLSTM_CHUNK_FROM for q in step.q_lens)
        ops.mlstm_scan(rows, gates, self.gate_bias, step.cu_q, step.positions, step.slot_ids,
                       layer.state, raw, step.n_seqs, H, dk, dv, 0, H * dk, 2 * H * dk,
                       self.gate_cap, float(dk) ** -0.5, short_runs=short_runs, long_runs=long_runs,
                       multi=self._longest_runs(step, n))
        heads = ws.buf("mlstm_heads", (n, H * dv), act)
        g0 = 2 * H * dk + H * dv
        ops.mlstm_out(raw, rows[:, g0:g0 + H * dv], self.head_weight, self.norm_eps, heads, H, dv)
        add_product(step, heads, self.w_o, residual)
