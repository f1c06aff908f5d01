"""Attention over a window of the paged cache whose queries and keys are normed over the whole projection and rotated in
neighbouring pairs, with the options its users pick from.

With h the layer's input, H query heads of ``dim`` elements and G key/value heads: q = W_q h, k = W_k h (+ biases); a short causal
convolution over time on every channel of q and k (``conv_taps``; the last taps - 1 inputs of a sequence are kept in its state
slot); an RMS norm over ALL H dim elements of q at once, and over all G dim of k, each with a gain vector of that length; the
rotation; score = scale q . k, then ``softcap`` tanh(score / softcap); keys p - window + 1 .. p; a softmax whose denominator may
hold exp(sink_h), a learned number per head; every head's output times sigmoid((W_g h)_h), one gate a head; W_o (+ bias).

The values are either a projection of their own (``values`` "own": v = W_v h, ``vdim`` elements a head) or the keys as they leave
the convolution, before norm and rotation (``values`` "keys"). ``value_mix`` names a group of layers that blend their values: the
first layer of the group (``value_mix_first``) leaves its values of the step's rows in the batch's ``carry``; every later one
stores (1 - m) v + m v_first, m its learned number ``vmix``, and attends over those.

One product makes everything that reads h ([q | k | v | g], 32-bit sums); ``kernels.projection_rows`` norms, rotates, blends and
writes the pages; the framework's paged attention kernels do the rest. Heads of different key and value sizes are kept in pages of
the larger size (rounded to 16) with zeros behind, and the output matrix gets zero columns to match."""

from __future__ import annotations

import torch

from ..ops import kernels
from ..weights.spec import TABLE, VECTOR, Normal, TensorSpec
from .attention import MAX_HEAD_SIZE
from .base import KVNeed, LayerContext, Mixer, StateNeed, register_part
from .linear import BranchProduct, fuse_rows
from .positions import RotaryEncoding


class ProjectionNormAttention(Mixer):
    graph_safe = True
    short_portion = kernels.DECODE_MAX_Q_LEN
    folds_out_scale = True   # with a gate per head: ``out_scale`` multiplies the gated heads (and the output bias)

    def __init__(self, width: int, n_heads: int, n_kv_heads: int, dim: int, vdim: int | None, scale: float, eps: float, *,
                 rotary: RotaryEncoding | None = None, window: int | None = None, softcap: float | None = None, sink: bool = False,
                 qk_norm: bool = True, values: str = "own", biases: bool = False, conv_taps: int | None = None, head_gate: bool = False,
                 value_mix: str | None = None, value_mix_first: bool = False, out_scale: float = 1.0):
        if n_heads < 1 or n_kv_heads < 1 or n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} heads do not divide into {n_kv_heads} key/value heads")
        if values not in ("own", "keys"):
            raise ValueError(f"values are a projection of their 'own' or the 'keys', not {values!r}")
        vdim = dim if values == "keys" else int(vdim)
        self.head_size = -(-max(dim, vdim) // 16) * 16
        if not 1 <= self.head_size <= MAX_HEAD_SIZE:
            raise ValueError(f"heads of {max(dim, vdim)} are wider than the attention kernels take ({MAX_HEAD_SIZE})")
        if rotary is not None and (rotary.pairing != "neighbours" or rotary.dims > dim or rotary.magnitude != 1.0):
            raise ValueError("this mixer rotates neighbouring pairs of a head's first elements, at their own size")
        if out_scale != 1.0 and not head_gate:
            raise ValueError("an output scale is folded into the heads' gates, and this mixer has none")
        if value_mix is not None and values != "own":
            raise ValueError("only values of their own are mixed between layers")
        self.width, self.n_heads, self.n_kv_heads, self.dim, self.vdim = width, n_heads, n_kv_heads, dim, vdim
        self.scale, self.eps, self.rotary, self.window, self.softcap = float(scale), float(eps), rotary, window, softcap
        self.has_sink, self.qk_norm, self.values, self.biases, self.head_gate = sink, qk_norm, values, biases, head_gate
        self.conv_taps = int(conv_taps) if conv_taps else None
        self.value_mix, self.value_mix_first, self.out_scale = value_mix, value_mix_first, float(out_scale)
        self.q_width, self.k_width, self.v_width = n_heads * dim, n_kv_heads * dim, n_kv_heads * vdim
        self.w_in = self.b_in = self.o = self.o_bias = self.q_norm = self.k_norm = self.sink = self.vmix = self.conv = None
        self._out_product = BranchProduct()

    def tensor_specs(self):
        std = self.width ** -0.5
        specs = {"q": TensorSpec((self.q_width, self.width), TABLE, Normal(std)),
                 "k": TensorSpec((self.k_width, self.width), TABLE, Normal(std)),
                 "o": TensorSpec((self.width, self.n_heads * self.vdim), TABLE, Normal((self.n_heads * self.vdim) ** -0.5))}
        if self.values == "own":
            specs["v"] = TensorSpec((self.v_width, self.width), TABLE, Normal(std))
        if self.biases:
            specs["q.b"] = TensorSpec((self.q_width,), VECTOR, Normal(0.1))
            specs["k.b"] = TensorSpec((self.k_width,), VECTOR, Normal(0.1))
            specs["o.b"] = TensorSpec((self.width,), VECTOR, Normal(0.1))
        if self.conv_taps:
            specs["q.conv"] = TensorSpec((self.q_width, self.conv_taps), VECTOR, Normal(self.conv_taps ** -0.5))
            specs["k.conv"] = TensorSpec((self.k_width, self.conv_taps), VECTOR, Normal(self.conv_taps ** -0.5))
        if self.qk_norm:
            specs["q.norm"] = TensorSpec((self.q_width,), VECTOR, Normal(0.1, mean=1.0))
            specs["k.norm"] = TensorSpec((self.k_width,), VECTOR, Normal(0.1, mean=1.0))
        if self.has_sink:
            specs["sink"] = TensorSpec((self.n_heads,), VECTOR, Normal(1.0))
        if self.head_gate:
            specs["g"] = TensorSpec((self.n_heads, self.width), TABLE, Normal(std))
        if self.value_mix is not None:   # the group's first layer has the number too, and does not use it
            specs["vmix"] = TensorSpec((), VECTOR, Normal(0.1, mean=0.5))
        return specs

    def bind(self, tensors):
        fused = fuse_rows([tensors[name] for name in ("q", "k", "v", "g") if name in tensors])
        o = tensors["o"]
        if self.head_size != self.vdim:   # the attention leaves heads of head_size: the columns beyond a head's vdim meet zeros
            wide = torch.zeros((self.width, self.n_heads, self.head_size), dtype=o.dtype, device=o.device)
            wide[:, :, : self.vdim] = o.view(self.width, self.n_heads, self.vdim)
            o = wide.view(self.width, self.n_heads * self.head_size)
        on_gpu = fused.is_cuda
        self.w_in, self.o = (kernels.pack_matrix(fused), kernels.pack_matrix(o.contiguous())) if on_gpu else (fused, o)
        if self.biases:
            self.b_in = torch.zeros((fused.shape[0],), dtype=torch.float32, device=fused.device)
            self.b_in[: self.q_width] = tensors["q.b"]
            self.b_in[self.q_width : self.q_width + self.k_width] = tensors["k.b"]
            self.o_bias = (tensors["o.b"] * self.out_scale).contiguous()
        if self.conv_taps:
            self.conv = torch.cat([tensors["q.conv"], tensors["k.conv"]], dim=0).contiguous()
        self.q_norm, self.k_norm, self.sink = tensors.get("q.norm"), tensors.get("k.norm"), tensors.get("sink")
        if self.value_mix is not None:
            self.vmix = tensors["vmix"].reshape(1).contiguous()

    def kv_need(self):
        return KVNeed(self.n_kv_heads, self.head_size, self.window)

    def state_need(self):
        if self.conv_taps and self.conv_taps > 1:
            return StateNeed(((self.conv_taps - 1) * (self.q_width + self.k_width),), torch.float32)
        return None

    def forward(self, x, residual, ctx: LayerContext):
        """The branch alone (float32) when ``residual`` is None, else residual + branch."""
        batch = ctx.batch
        fused = kernels.linear(x, self.w_in, self.b_in, out_dtype=torch.float32)
        qk_width = self.q_width + self.k_width
        qk = fused[:, :qk_width]
        if self.conv_taps:
            if getattr(batch, "first_row", 0):
                raise ValueError("a mixer that keeps state per request takes a step's batch whole")
            qk = kernels.short_conv(qk, self.conv, ctx.state, batch.token_request, batch.q_starts, batch.state_slots, keep=ctx.write_cache)
        q, k = qk[:, : self.q_width], qk[:, self.q_width :]
        at = qk_width
        if self.values == "own":
            v, at = fused[:, at : at + self.v_width], at + self.v_width
        else:
            v = k
        gate = fused[:, at : at + self.n_heads] if self.head_gate else None
        v_other = None
        if self.value_mix is not None:
            if self.value_mix_first:
                batch.carry[self.value_mix] = v
            else:
                v_other = batch.carry.get(self.value_mix)
                if v_other is None:
                    raise ValueError(f"no earlier layer of this step has left the values of group {self.value_mix!r}")
        rotary = self.rotary
        q = kernels.projection_rows(q, k, v, self.q_norm, self.k_norm, self.eps, None if rotary is None else rotary.frequencies64(x.device),
                                    0 if rotary is None else rotary.dims, batch.positions, ctx.group.slots, ctx.k_pages, ctx.v_pages,
                                    self.n_heads, self.n_kv_heads, self.dim, self.vdim, v_other=v_other, mix=self.vmix, write_cache=ctx.write_cache)
        mixed = kernels.paged_attention(
            q, ctx.k_pages, ctx.v_pages, batch.token_request, batch.positions, ctx.group.block_tables,
            self.n_heads, self.n_kv_heads, self.head_size, self.scale, window=self.window or 0,
            max_q_len=batch.max_q_len, max_len=batch.max_total_len, q_starts=batch.q_starts, context_lens=batch.context_lens,
            first_row=getattr(batch, "first_row", 0), softcap=self.softcap or 0.0, sinks=self.sink,
            **({"short_rows": batch.short_rows, "short_requests": batch.short_requests} if batch.short_portion <= kernels.DECODE_MAX_Q_LEN else {}),
        )
        if self.head_gate:
            kernels.head_gate(mixed, gate, mixed, self.n_heads, self.head_size, scale=self.out_scale)
        return self._out_product(mixed, self.o, residual, bias=self.o_bias)


register_part("mixer", "projection_norm_attention", ProjectionNormAttention)
