"""Mixers that keep a matrix per head and request in the request's state slot instead of keys and values in pages, and the
mixer that runs two others side by side.

``MatrixMemoryMixer`` (the mLSTM of xLSTM): q = W_q h / sqrt(dim), k = W_k h, v = W_v h; per head a log input gate i = cap
tanh((W_i h + b_i) / cap) and a log forget gate f = logsigmoid(cap tanh((W_f h + b_f) / cap)); with a running maximum m that
starts at 0, m_t = max(f_t + m_(t-1), i_t), S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T, n_t likewise with k_t
alone, o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6); every head's o divided by its root mean square, the heads laid
behind each other, times a gain vector, times sigmoid(W_g h), then W_o.

``DecayedLinearAttention``: q, k, v = silu of their projections; S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t with one fixed
decay per head; the heads laid behind each other are RMS-normed together with a gain vector, times sigmoid(W_g h), then W_o.

Both: one product makes everything that reads h (32-bit sums), ``kernels.recurrence`` walks each request's rows of the step from
the state its slot holds (zero at admission), ``kernels.gated_norm`` norms and gates. State, gates and sums are 32-bit in every
precision.

``ParallelMixer``: left_scale * left(h) + right_scale * right(h), two mixers of the framework reading the same rows. Each folds
its scale into its last elementwise kernel, and the second one's output product adds the first one's result, so the sum costs no
kernel of its own."""

from __future__ import annotations

from dataclasses import replace

import torch

from ..ops import kernels
from ..weights.spec import TABLE, VECTOR, Normal, TensorSpec
from .base import LayerContext, Mixer, StateNeed, register_part
from .linear import BranchProduct, fuse_rows


def _whole_batch(batch) -> None:
    if getattr(batch, "first_row", 0):
        raise ValueError("a mixer that keeps state per request takes a step's batch whole")


class MatrixMemoryMixer(Mixer):
    graph_safe = True
    folds_out_scale = True

    def __init__(self, width: int, n_heads: int, dim: int, vdim: int, eps: float, gate_cap: float | None = None, out_scale: float = 1.0):
        self.width, self.n_heads, self.dim, self.vdim = width, n_heads, dim, vdim
        self.eps, self.gate_cap, self.out_scale = float(eps), gate_cap, float(out_scale)
        self.w_in = self.b_in = self.o = self.norm = None
        self._out_product = BranchProduct()

    def tensor_specs(self):
        H, std = self.n_heads, self.width ** -0.5
        return {"q": TensorSpec((H * self.dim, self.width), TABLE, Normal(std)),
                "k": TensorSpec((H * self.dim, self.width), TABLE, Normal(std)),
                "v": TensorSpec((H * self.vdim, self.width), TABLE, Normal(std)),
                "g": TensorSpec((H * self.vdim, self.width), TABLE, Normal(std)),
                "i": TensorSpec((H, self.width), TABLE, Normal(std)),
                "f": TensorSpec((H, self.width), TABLE, Normal(std)),
                "i.b": TensorSpec((H,), VECTOR, Normal(0.5)),
                "f.b": TensorSpec((H,), VECTOR, Normal(0.5, mean=3.0)),
                "norm": TensorSpec((H * self.vdim,), VECTOR, Normal(0.1, mean=1.0)),
                "o": TensorSpec((self.width, H * self.vdim), TABLE, Normal((H * self.vdim) ** -0.5))}

    def bind(self, tensors):
        H = self.n_heads
        fused = fuse_rows([tensors[name] for name in ("q", "k", "v", "g", "i", "f")])
        on_gpu = fused.is_cuda
        self.w_in = kernels.pack_matrix(fused) if on_gpu else fused
        self.b_in = torch.zeros((fused.shape[0],), dtype=torch.float32, device=fused.device)
        at = 2 * H * self.dim + 2 * H * self.vdim
        self.b_in[at : at + H] = tensors["i.b"]
        self.b_in[at + H : at + 2 * H] = tensors["f.b"]
        self.o = kernels.pack_matrix(tensors["o"].contiguous()) if on_gpu else tensors["o"]
        self.norm = tensors["norm"]

    def state_need(self):
        H = self.n_heads
        return StateNeed((H * self.dim * self.vdim + H * self.dim + H,), torch.float32)

    def forward(self, x, residual, ctx: LayerContext):
        """The branch alone (float32) when ``residual`` is None, else residual + branch."""
        batch, H = ctx.batch, self.n_heads
        _whole_batch(batch)
        fused = kernels.linear(x, self.w_in, self.b_in, out_dtype=torch.float32)
        qw, vw = H * self.dim, H * self.vdim
        q, k, v, gate = fused[:, :qw], fused[:, qw : 2 * qw], fused[:, 2 * qw : 2 * qw + vw], fused[:, 2 * qw + vw : 2 * qw + 2 * vw]
        at = 2 * qw + 2 * vw
        summed = kernels.recurrence(q, k, v, ctx.state, batch.q_starts, batch.state_slots, H, self.dim, self.vdim,
                                    gate_in=fused[:, at : at + H], gate_forget=fused[:, at + H : at + 2 * H], cap=self.gate_cap or 0.0,
                                    q_scale=self.dim ** -0.5, max_q_len=batch.max_q_len)
        mixed = torch.empty((x.shape[0], vw), dtype=x.dtype, device=x.device)
        kernels.gated_norm(summed, self.norm, gate, self.eps, mixed, group=self.vdim, scale=self.out_scale)
        return self._out_product(mixed, self.o, residual)


class DecayedLinearAttention(Mixer):
    graph_safe = True
    folds_out_scale = True

    def __init__(self, width: int, n_heads: int, dim: int, vdim: int, decay, eps: float, out_scale: float = 1.0):
        decay = [float(d) for d in decay]
        if len(decay) != n_heads:
            raise ValueError(f"{len(decay)} decays for {n_heads} heads")
        self.width, self.n_heads, self.dim, self.vdim, self.decay_values = width, n_heads, dim, vdim, decay
        self.eps, self.out_scale = float(eps), float(out_scale)
        self.w_in = self.o = self.norm = self.decay = None
        self._out_product = BranchProduct()

    def tensor_specs(self):
        H, std = self.n_heads, self.width ** -0.5
        return {"q": TensorSpec((H * self.dim, self.width), TABLE, Normal(std)),
                "k": TensorSpec((H * self.dim, self.width), TABLE, Normal(std)),
                "v": TensorSpec((H * self.vdim, self.width), TABLE, Normal(std)),
                "g": TensorSpec((H * self.vdim, self.width), TABLE, Normal(std)),
                "norm": TensorSpec((H * self.vdim,), VECTOR, Normal(0.1, mean=1.0)),
                "o": TensorSpec((self.width, H * self.vdim), TABLE, Normal((H * self.vdim) ** -0.5))}

    def bind(self, tensors):
        fused = fuse_rows([tensors[name] for name in ("q", "k", "v", "g")])
        on_gpu = fused.is_cuda
        self.w_in = kernels.pack_matrix(fused) if on_gpu else fused
        self.o = kernels.pack_matrix(tensors["o"].contiguous()) if on_gpu else tensors["o"]
        self.norm = tensors["norm"]
        self.decay = torch.tensor(self.decay_values, dtype=torch.float64).to(torch.float32).to(fused.device)

    def state_need(self):
        return StateNeed((self.n_heads * self.dim * self.vdim,), torch.float32)

    def forward(self, x, residual, ctx: LayerContext):
        """The branch alone (float32) when ``residual`` is None, else residual + branch."""
        batch, H = ctx.batch, self.n_heads
        _whole_batch(batch)
        fused = kernels.linear(x, self.w_in, out_dtype=torch.float32)
        qw, vw = H * self.dim, H * self.vdim
        q, k, v, gate = fused[:, :qw], fused[:, qw : 2 * qw], fused[:, 2 * qw : 2 * qw + vw], fused[:, 2 * qw + vw : 2 * qw + 2 * vw]
        summed = kernels.recurrence(q, k, v, ctx.state, batch.q_starts, batch.state_slots, H, self.dim, self.vdim, decay=self.decay,
                                    max_q_len=batch.max_q_len, positive_decay=min(self.decay_values) > 0)
        mixed = torch.empty((x.shape[0], vw), dtype=x.dtype, device=x.device)
        kernels.gated_norm(summed, self.norm, gate, self.eps, mixed, scale=self.out_scale)
        return self._out_product(mixed, self.o, residual)


class ParallelMixer(Mixer):
    """``left`` and ``right`` are built with their share of the sum as their ``out_scale``. At most one of them keeps keys and
    values in pages; the state slots of both lie behind each other in one slot."""

    graph_safe = True

    def __init__(self, left: Mixer, right: Mixer, names=("left.", "right.")):
        for part in (left, right):
            if not getattr(part, "folds_out_scale", False):
                raise ValueError(f"{type(part).__name__} cannot scale its own output, which a mixer beside another has to")
        if left.kv_need() is not None and right.kv_need() is not None:
            raise ValueError("two mixers side by side share one cache layer: only one of them may keep keys and values")
        for need in (left.state_need(), right.state_need()):
            if need is not None and (len(need.shape) != 1 or need.dtype != torch.float32):
                raise ValueError("mixers side by side keep their state as a row of 32-bit numbers")
        self.left, self.right = left, right
        self._names = names
        self.short_portion = left.short_portion if left.short_portion is not None else right.short_portion
        self.decode_reaches = tuple(sorted(set(left.decode_reaches) | set(right.decode_reaches)))

    def children(self):
        return dict(zip(self._names, (self.left, self.right)))

    def kv_need(self):
        return self.left.kv_need() or self.right.kv_need()

    def _state_sizes(self):
        return [0 if need is None else need.shape[0] for need in (self.left.state_need(), self.right.state_need())]

    def state_need(self):
        total = sum(self._state_sizes())
        return StateNeed((total,), torch.float32) if total else None

    def forward(self, x, residual, ctx: LayerContext):
        n_left, n_right = self._state_sizes()
        left_ctx = replace(ctx, state=ctx.state[:, :n_left] if n_left else None)
        right_ctx = replace(ctx, state=ctx.state[:, n_left : n_left + n_right] if n_right else None)
        out = self.left.forward(x, residual, left_ctx)
        if out.dim() == 3:   # a product cut along K: its parts added up before another product adds to them
            out = kernels.settle(kernels.PendingRows(out[0], out[1:], None)) if out.shape[0] > 1 else out[0]
        return self.right.forward(x, out, right_ctx)


register_part("mixer", "matrix_memory", MatrixMemoryMixer)
register_part("mixer", "decayed_linear_attention", DecayedLinearAttention)
register_part("mixer", "parallel", ParallelMixer)
