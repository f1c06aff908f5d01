"""Attention over a shared latent: per token the layer keeps one normed vector c of ``kv_rank`` elements and one rotated key
part of ``rot_dim`` elements, shared by all heads, instead of keys and values per head.

In formulas (h the layer's input, H heads): q = W_q h, per head [dim plain | rot_dim rotated]; [c' | k_r'] = W_dkv h, c =
rmsnorm(c') * g, k_r = rotate(k_r'); head i's key is [W_uk,i c | k_r] and its value W_uv,i c; score = scale * (q_plain . k_plain
+ rotate(q_rot) . k_r); causal softmax whose denominator also holds exp(sink_i); the heads' outputs, laid behind each other,
are multiplied by sigmoid(W_g h) and go through W_o. A layer built with ``own_latent=False`` has no W_dkv: it reads the rows that
the layer whose cache it is given has stored, with its own W_uk, W_uv and queries.

Keys and values are never expanded: W_uk is folded into the query (q'_i = W_uk,i^T q_plain,i, so that a score is a dot product
with the cached row as it lies) and W_uv is applied once to the weighted sum of the latents (ops.kernels.latent_attention)."""

from __future__ import annotations

import torch

from ..ops import kernels
from ..weights.spec import TABLE, VECTOR, Normal, TensorSpec
from .base import KVNeed, LayerContext, Mixer, register_part
from .linear import BranchProduct
from .positions import RotaryEncoding


class LatentAttention(Mixer):
    graph_safe = True

    def __init__(self, width: int, n_heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int, scale: float, eps: float,
                 rotary: RotaryEncoding, sink: bool = True, gated: bool = True, own_latent: bool = True):
        if rotary.dims > rot_dim:
            raise ValueError(f"{rotary.dims} rotated elements do not fit a rotated part of {rot_dim}")
        self.width, self.n_heads, self.dim, self.rot_dim, self.vdim, self.kv_rank = width, n_heads, dim, rot_dim, vdim, kv_rank
        self.scale, self.eps, self.rotary = float(scale), float(eps), rotary
        self.has_sink, self.gated, self.own_latent = sink, gated, own_latent
        # a cached row: [latent | rotated key part | zeros up to a size the attention kernels take]
        self.row_size = kernels.latent_row_size(kv_rank + rot_dim)
        self.w_in = self.uk_t = self.uv = self.o = self.sink = self.dkv_norm = None
        self._out_product = BranchProduct()

    def tensor_specs(self):
        H, std = self.n_heads, self.width ** -0.5
        specs = {"q": TensorSpec((H * (self.dim + self.rot_dim), self.width), TABLE, Normal(std)),
                 "uk": TensorSpec((H * self.dim, self.kv_rank), TABLE, Normal(self.kv_rank ** -0.5)),
                 "uv": TensorSpec((H * self.vdim, self.kv_rank), TABLE, Normal(self.kv_rank ** -0.5)),
                 "o": TensorSpec((self.width, H * self.vdim), TABLE, Normal((H * self.vdim) ** -0.5))}
        if self.own_latent:
            specs["dkv"] = TensorSpec((self.kv_rank + self.rot_dim, self.width), TABLE, Normal(std))
            specs["dkv.norm"] = TensorSpec((self.kv_rank,), VECTOR, Normal(0.1, mean=1.0))
        if self.has_sink:
            specs["sink"] = TensorSpec((H,), VECTOR, Normal(1.0))
        if self.gated:
            specs["g"] = TensorSpec((H * self.vdim, self.width), TABLE, Normal(std))
        return specs

    def bind(self, tensors):
        H = self.n_heads
        # one product for everything that reads the layer's input: [q | dkv | g]
        fused = torch.cat([tensors[name] for name in ("q", "dkv", "g") if name in tensors], dim=0).contiguous()
        on_gpu = fused.is_cuda
        self.w_in = kernels.pack_matrix(fused) if on_gpu else fused
        self.uk_t = tensors["uk"].view(H, self.dim, self.kv_rank).transpose(1, 2).contiguous()   # [H, rank, dim]: q' = uk_t q
        self.uv = tensors["uv"].view(H, self.vdim, self.kv_rank).contiguous()
        self.o = kernels.pack_matrix(tensors["o"].contiguous()) if on_gpu else tensors["o"]
        self.sink, self.dkv_norm = tensors.get("sink"), tensors.get("dkv.norm")

    def kv_need(self):
        return KVNeed(1, self.row_size, None, planes=1)

    def forward(self, x, residual, ctx: LayerContext):
        """The branch alone (float32) when ``residual`` is None, else residual + branch."""
        if ctx.write_cache != self.own_latent:
            raise ValueError("a latent layer writes the cache it is given exactly when it has a latent of its own")
        batch, H, rows = ctx.batch, self.n_heads, x.shape[0]
        q_width, kept = H * (self.dim + self.rot_dim), self.kv_rank + self.rot_dim
        fused = kernels.linear(x, self.w_in)
        q = fused[:, :q_width]
        at = q_width
        dkv = None
        if self.own_latent:
            dkv, at = fused[:, at : at + kept], at + kept
        gate = fused[:, at:] if self.gated else None
        q_full = kernels.latent_rows(q, dkv, self.dkv_norm, self.eps, self.rotary.frequencies(x.device), self.rotary.magnitude, self.rotary.dims,
                                     batch.positions, ctx.group.slots, ctx.k_pages, H, self.dim, self.rot_dim, self.kv_rank)
        kernels.heads_linear(q, self.uk_t, q_full, n_heads=H, k=self.dim, x_head_stride=self.dim + self.rot_dim)
        whole = getattr(batch, "first_row", 0) == 0   # a part of a batch numbers its rows from the whole batch's top
        summed = kernels.latent_attention(q_full, ctx.k_pages, self.sink, batch.token_request, batch.positions, ctx.group.block_tables,
                                          self.kv_rank, self.scale, max_len=batch.max_total_len, q_starts=batch.q_starts if whole else None,
                                          context_lens=batch.context_lens, max_q_len=batch.max_q_len)
        mixed = torch.empty((rows, H, self.vdim), dtype=x.dtype, device=x.device)
        kernels.heads_linear(summed, self.uv, mixed, n_heads=H, k=self.kv_rank, x_head_stride=self.kv_rank, gate=gate)
        return self._out_product(mixed.view(rows, H * self.vdim), self.o, residual)


register_part("mixer", "latent_attention", LatentAttention)
