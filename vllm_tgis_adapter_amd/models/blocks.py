"""Building blocks for models that keep an f32 residual stream.

Each block is one mechanism with its constants as constructor parameters, so
that another design can assemble them differently:

- ``StreamRMSNorm``     RMS norm of the f32 stream, weight applied as (offset + w)
- ``ShortConv``         depthwise causal convolution over time whose last
                        taps-1 inputs are per-sequence state
- ``LatentAttention``   multi-head attention whose keys and values are
                        up-projections of one cached latent row per token, with
                        a rotated key part shared by all heads, an optional
                        sliding window and a per-head sink in the softmax
- ``DenseMLP``          down(act(up(h))) with the tanh-form GELU
- ``TokenSideInput``    gated per-layer token embedding added to the stream
                        through its own RMS norm

The stream itself, norms, rotation angles, attention scores and softmax are
f32 whatever the compute dtype is; projections run in the compute dtype.
"""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from .. import ops
from ..engine.metadata import AttnMetadata
from ..parallel import divide, get_tp_rank, get_tp_world_size
from ..parallel.layers import ColumnParallelLinear, RowParallelLinear


def _f32_param(*shape, fill: float = 0.0) -> nn.Parameter:
    return nn.Parameter(torch.full(shape, fill, dtype=torch.float32), requires_grad=False)


class StreamRMSNorm(nn.Module):
    """f32 stream -> compute dtype: x / sqrt(mean(x^2) + eps) * (offset + w)."""

    def __init__(self, width: int, eps: float, weight_offset: float, dtype: torch.dtype):
        super().__init__()
        self.eps = eps
        self.weight_offset = weight_offset
        self.dtype = dtype
        self.weight = _f32_param(width, fill=1.0 - weight_offset)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.rms_norm_stream(x, self.weight, self.eps, self.weight_offset, self.dtype)


class ShortConv(nn.Module):
    """h + conv(h): per-channel causal convolution over time, ``taps`` taps,
    no bias.  The last taps-1 inputs of a sequence are carried in a state
    slot so that a sequence can be fed in portions of any size."""

    def __init__(self, width: int, taps: int):
        super().__init__()
        self.width = width
        self.taps = taps
        w = torch.empty(width, taps, dtype=torch.float32).normal_(0.0, 0.1)
        self.weight = nn.Parameter(w, requires_grad=False)

    def state_shape(self) -> tuple:
        return (max(self.taps - 1, 0), self.width)

    def forward(self, h: torch.Tensor, state: torch.Tensor, meta: AttnMetadata) -> torch.Tensor:
        return ops.causal_conv_state(
            h, self.weight, state, meta.seq_start_loc, meta.seq_lens,
            meta.state_slots, add_input=True)


class LatentAttention(nn.Module):
    """Attention over a cached latent.

    Per token the cache holds one row [rank + rot]: the RMS-normed latent c
    and a rotated key part shared by all heads.  Head h's key is
    [W_uk[h] c ; k_rot] and its value W_uv[h] c.  The kernels work in latent
    space: the unrotated query is folded through W_uk[h] first
    (q_lat = W_uk[h]^T q), scores are (q_lat . c + q_rot . k_rot) * scale, the
    weighted sum of c is unfolded through W_uv[h] afterwards — every head
    reads the same single row per token.

    ``kv_owner`` False: the layer has no down-projection of its own and reads
    the rows another layer wrote this step (its cache tensor is that layer's).
    """

    def __init__(self, width: int, *, heads: int, dim: int, rot_dim: int, vdim: int,
                 rank: int, scale: float, window: int, rot_base: float,
                 rot_dims: int, eps: float, kv_owner: bool, has_sink: bool,
                 dtype: torch.dtype):
        super().__init__()
        tp = get_tp_world_size()
        self.heads = divide(heads, tp)
        self.dim, self.rot_dim, self.vdim, self.rank = dim, rot_dim, vdim, rank
        self.scale, self.window, self.eps = scale, window, eps
        self.rot_dims = rot_dims
        self.kv_owner = kv_owner
        self.dtype = dtype
        self.q_proj = ColumnParallelLinear(width, heads * (dim + rot_dim), dtype=dtype)
        self.o_proj = RowParallelLinear(heads * vdim, width, dtype=dtype)
        if kv_owner:
            # replicated on every rank: the latent is shared by all heads
            self.dkv_weight = nn.Parameter(
                torch.empty(rank + rot_dim, width, dtype=dtype).normal_(0.0, 0.02),
                requires_grad=False)
            self.dkv_norm = _f32_param(rank, fill=1.0)
        # [H, dim, rank] and [H, rank, vdim] for the batched fold / unfold
        self.uk = nn.Parameter(
            torch.empty(self.heads, dim, rank, dtype=dtype).normal_(0.0, 0.02),
            requires_grad=False)
        self.uv_t = nn.Parameter(
            torch.empty(self.heads, rank, vdim, dtype=dtype).normal_(0.0, 0.02),
            requires_grad=False)
        self.sink = _f32_param(self.heads) if has_sink else None
        half = rot_dims // 2
        inv_freq = torch.tensor(
            [float(rot_base) ** (-2.0 * i / rot_dims) for i in range(half)],
            dtype=torch.float64).to(torch.float32)
        self.register_buffer("inv_freq", inv_freq, persistent=False)

    # -- weights -----------------------------------------------------------
    def load(self, q, dkv, dkv_norm, uk, uv, sink, o) -> None:
        r, h = get_tp_rank(), self.heads
        self.q_proj.load_full_weight(q)
        self.o_proj.load_full_weight(o)
        if self.kv_owner:
            self.dkv_weight.data.copy_(dkv.to(self.dtype))
            self.dkv_norm.data.copy_(dkv_norm.float())
        uk = uk.view(-1, self.dim, self.rank)[r * h:(r + 1) * h]
        uv = uv.view(-1, self.vdim, self.rank)[r * h:(r + 1) * h]
        self.uk.data.copy_(uk.to(self.dtype))
        self.uv_t.data.copy_(uv.transpose(1, 2).to(self.dtype))
        if self.sink is not None:
            self.sink.data.copy_(sink.float()[r * h:(r + 1) * h])

    # -- forward -----------------------------------------------------------
    def forward(self, h: torch.Tensor, positions: torch.Tensor,
                cache: torch.Tensor, meta: AttnMetadata) -> torch.Tensor:
        t = h.shape[0]
        nh, d, r, rank = self.heads, self.dim, self.rot_dim, self.rank
        q = self.q_proj(h).view(t, nh, d + r)
        ops.rope_partial(q, positions, self.inv_freq, d, self.rot_dims)
        if self.kv_owner:
            dkv = ops.linear(h, self.dkv_weight)
            ops.latent_kv_write(dkv, self.dkv_norm, self.eps, positions,
                                self.inv_freq, self.rot_dims, cache,
                                meta.slot_mapping)
        # fold the unrotated query into latent space: [H, T, rank]
        q_lat = torch.bmm(q[:, :, :d].transpose(0, 1), self.uk).transpose(0, 1)
        q_rot = q[:, :, d:]
        o_lat = torch.empty((nh, t, rank), dtype=h.dtype, device=h.device)
        o_view = o_lat.transpose(0, 1)   # [T, H, rank]
        npt = meta.num_prefill_tokens
        if npt:
            ops.latent_attention_prefill(
                q_lat[:npt], q_rot[:npt], cache, meta.prefill_block_tables,
                meta.prefill_query_start_loc, meta.prefill_seq_lens, self.scale,
                self.window, self.sink, meta.max_prefill_query_len,
                out=o_view[:npt])
        if meta.num_decode_seqs:
            ops.latent_attention_decode(
                q_lat[npt:], q_rot[npt:], cache, meta.decode_block_tables,
                meta.decode_seq_lens, self.scale, self.window, self.sink,
                out=o_view[npt:])
        o = torch.bmm(o_lat, self.uv_t)                    # [H, T, vdim]
        return self.o_proj(o.transpose(0, 1).reshape(t, nh * self.vdim))


class DenseMLP(nn.Module):
    def __init__(self, width: int, ff: int, dtype: torch.dtype):
        super().__init__()
        self.up = ColumnParallelLinear(width, ff, dtype=dtype)
        self.down = RowParallelLinear(ff, width, dtype=dtype)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.down(ops.gelu_tanh(self.up(h)))


class TokenSideInput(nn.Module):
    """x <- x + mult * rmsnorm(proj(gelu_tanh(gate x) * e)) * w, e being this
    layer's slice of a per-token side embedding."""

    def __init__(self, width: int, side_dim: int, eps: float, mult: float,
                 dtype: torch.dtype):
        super().__init__()
        self.eps, self.mult = eps, mult
        self.gate = nn.Parameter(
            torch.empty(side_dim, width, dtype=dtype).normal_(0.0, 0.02), requires_grad=False)
        self.proj = nn.Parameter(
            torch.empty(width, side_dim, dtype=dtype).normal_(0.0, 0.02), requires_grad=False)
        self.norm = _f32_param(width, fill=1.0)

    def forward(self, x: torch.Tensor, x_cast: torch.Tensor, e: torch.Tensor,
                next_norm: "StreamRMSNorm | None" = None):
        """Updates x in place; with ``next_norm`` the norm that reads the
        updated stream next is computed in the same kernel and returned."""
        g = ops.gelu_tanh(ops.linear(x_cast, self.gate), mul=e)
        y = ops.linear(g, self.proj)
        nn_ = None
        if next_norm is not None:
            nn_ = (next_norm.weight, next_norm.eps, next_norm.weight_offset, next_norm.dtype)
        return ops.stream_add_rms_norm(x, y, self.norm, self.eps, self.mult, nn_)
