"""Plain-PyTorch reference implementations of every custom op.

These are the CPU execution path (protocol tests run the full engine on CPU,
like the reference's CPU-build CI — SURVEY.md §4) and the numerics oracle the
GPU kernels are tested against (fp32 upcast).
"""

from __future__ import annotations

import torch


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    out = xf * torch.rsqrt(var + eps)
    return (out * weight.float()).to(x.dtype)


def fused_add_rms_norm(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float
) -> tuple[torch.Tensor, torch.Tensor]:
    """Returns (normed, new_residual) where new_residual = x + residual."""
    summed = (x.float() + residual.float()).to(x.dtype)
    return rms_norm(summed, weight, eps), summed


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    d = x.shape[-1] // 2
    a, b = x[..., :d], x[..., d:]
    return (torch.nn.functional.silu(a.float()) * b.float()).to(x.dtype)


def make_cos_sin_cache(
    head_dim: int, max_len: int, theta: float, dtype: torch.dtype,
    scaling: dict | None = None,
) -> torch.Tensor:
    """[max_len, head_dim] cache: first half cos, second half sin (f32)."""
    rot = head_dim
    inv_freq = 1.0 / (theta ** (torch.arange(0, rot, 2, dtype=torch.float64) / rot))
    if scaling and scaling.get("rope_type") == "llama3":
        # llama-3.1-style frequency rescaling
        factor = scaling["factor"]
        lo = scaling.get("low_freq_factor", 1.0)
        hi = scaling.get("high_freq_factor", 4.0)
        orig = scaling.get("original_max_position_embeddings", 8192)
        wavelen = 2 * torch.pi / inv_freq
        ratio = orig / wavelen
        smooth = ((ratio - lo) / (hi - lo)).clamp(0, 1)
        inv_freq = torch.where(
            wavelen > orig / lo,
            torch.where(wavelen < orig / hi, inv_freq, inv_freq / factor),
            inv_freq * ((1 - smooth) / factor + smooth),
        )
    t = torch.arange(max_len, dtype=torch.float64)
    freqs = torch.outer(t, inv_freq)
    return torch.cat([freqs.cos(), freqs.sin()], dim=-1).float()


def rotary_embedding(
    positions: torch.Tensor,  # [T]
    q: torch.Tensor,          # [T, num_heads * head_dim]
    k: torch.Tensor,          # [T, num_kv_heads * head_dim]
    head_dim: int,
    cos_sin_cache: torch.Tensor,  # [max_len, head_dim] f32
) -> tuple[torch.Tensor, torch.Tensor]:
    """NeoX-style (rotate halves) rotary embedding, out-of-place reference."""
    half = head_dim // 2
    cs = cos_sin_cache[positions]          # [T, head_dim]
    cos = cs[:, :half].unsqueeze(1)        # [T, 1, half]
    sin = cs[:, half:].unsqueeze(1)

    def rot(x: torch.Tensor) -> torch.Tensor:
        t = x.shape[0]
        xs = x.view(t, -1, head_dim).float()
        x1, x2 = xs[..., :half], xs[..., half:]
        o1 = x1 * cos - x2 * sin
        o2 = x2 * cos + x1 * sin
        return torch.cat([o1, o2], dim=-1).to(x.dtype).view(t, -1)

    return rot(q), rot(k)


def reshape_and_cache(
    k: torch.Tensor,  # [T, num_kv_heads, head_dim]
    v: torch.Tensor,
    k_cache: torch.Tensor,  # [num_blocks, block_size, num_kv_heads, head_dim]
    v_cache: torch.Tensor,
    slot_mapping: torch.Tensor,  # [T] int64 (flat slot = block*block_size + off)
) -> None:
    bs = k_cache.shape[1]
    blocks = torch.div(slot_mapping, bs, rounding_mode="floor")
    offs = slot_mapping % bs
    k_cache[blocks, offs] = k.to(k_cache.dtype)
    v_cache[blocks, offs] = v.to(v_cache.dtype)


def _gather_kv(
    k_cache: torch.Tensor, v_cache: torch.Tensor,
    block_table: torch.Tensor, seq_len: int,
) -> tuple[torch.Tensor, torch.Tensor]:
    bs = k_cache.shape[1]
    nb = (seq_len + bs - 1) // bs
    k = k_cache[block_table[:nb]].reshape(-1, *k_cache.shape[2:])[:seq_len]
    v = v_cache[block_table[:nb]].reshape(-1, *v_cache.shape[2:])[:seq_len]
    return k, v


def paged_attention(
    q: torch.Tensor,            # [T, num_heads, head_dim]
    k_cache: torch.Tensor,      # [num_blocks, block_size, num_kv_heads, head_dim]
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,  # [num_seqs, max_blocks]
    query_start_loc: torch.Tensor,  # [num_seqs + 1] (cpu)
    seq_lens: torch.Tensor,         # [num_seqs] total context per seq (cpu)
    scale: float,
) -> torch.Tensor:
    """Causal paged attention over queries that are the *tail* of each
    sequence (covers prefill chunks and single-token decode uniformly)."""
    num_heads = q.shape[1]
    num_kv_heads = k_cache.shape[2]
    group = num_heads // num_kv_heads
    out = torch.empty_like(q)
    qs = query_start_loc.tolist()
    lens = seq_lens.tolist()
    for i in range(len(lens)):
        s, e = qs[i], qs[i + 1]
        q_len = e - s
        seq_len = lens[i]
        k, v = _gather_kv(k_cache, v_cache, block_tables[i], seq_len)
        qf = q[s:e].float()                       # [q, H, d]
        kf = k.float().repeat_interleave(group, dim=1)  # [S, H, d]
        vf = v.float().repeat_interleave(group, dim=1)
        scores = torch.einsum("qhd,shd->hqs", qf, kf) * scale
        # causal: query position j (global seq_len - q_len + j) sees keys <= it
        kpos = torch.arange(seq_len, device=q.device)
        qpos = torch.arange(seq_len - q_len, seq_len, device=q.device)
        mask = kpos[None, :] > qpos[:, None]
        scores.masked_fill_(mask.unsqueeze(0), float("-inf"))
        probs = torch.softmax(scores, dim=-1)
        out[s:e] = torch.einsum("hqs,shd->qhd", probs, vf).to(q.dtype)
    return out


def topk_softmax(gate_logits: torch.Tensor, top_k: int) -> tuple[torch.Tensor, torch.Tensor]:
    """MoE router: softmax over experts then top-k, renormalized."""
    probs = torch.softmax(gate_logits.float(), dim=-1)
    weights, ids = torch.topk(probs, top_k, dim=-1)
    weights = weights / weights.sum(dim=-1, keepdim=True)
    return weights, ids


# ---------------------------------------------------------------------------
# f32 residual-stream ops, short causal convolution with per-sequence state,
# windowed latent attention with sinks (the `_C_seq` kernel set)
# ---------------------------------------------------------------------------


def gelu_tanh(x: torch.Tensor, mul: torch.Tensor | None = None) -> torch.Tensor:
    z = x.float()
    y = 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z * z * z)))
    if mul is not None:
        y = y * mul.float()
    return y.to(x.dtype)


def embedding_scaled(ids: torch.Tensor, table: torch.Tensor, scale: float) -> torch.Tensor:
    return table[ids].float() * scale


def rms_norm_stream(x: torch.Tensor, weight: torch.Tensor, eps: float,
                    weight_offset: float, out_dtype: torch.dtype) -> torch.Tensor:
    xf = x.float()
    r = torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps)
    return (xf * r * (weight.float() + weight_offset)).to(out_dtype)


def stream_add(x: torch.Tensor, a: torch.Tensor, b: torch.Tensor | None,
               mult: float, cast_dtype: torch.dtype | None) -> torch.Tensor | None:
    s = a.float() if b is None else a.float() + b.float()
    x.add_(s, alpha=mult)
    return x.to(cast_dtype) if cast_dtype is not None else None


def stream_add_rms_norm(x: torch.Tensor, y: torch.Tensor, weight: torch.Tensor,
                        eps: float, mult: float) -> None:
    yf = y.float()
    r = torch.rsqrt(yf.pow(2).mean(dim=-1, keepdim=True) + eps)
    x.add_(yf * r * weight.float(), alpha=mult)


def softcap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    lf = logits.float()
    return cap * torch.tanh(lf / cap)


def causal_conv_state(
    h: torch.Tensor,            # [T, W]
    weight: torch.Tensor,       # [W, taps]
    state: torch.Tensor,        # [slots, taps-1, W]
    seq_start_loc: torch.Tensor,  # [S+1] rows of each sequence's new tokens
    seq_lens: torch.Tensor,       # [S] tokens of the sequence incl. the new ones
    state_slots: torch.Tensor,    # [S]
    add_input: bool,
) -> torch.Tensor:
    """out_t = (h_t if add_input) + sum_j w[:, j] * h_(t - taps + 1 + j) per
    sequence, inputs before the step's rows come from ``state`` (the last
    taps-1 inputs of the sequence), inputs before the sequence are zero;
    ``state`` is then advanced past the new rows."""
    taps = weight.shape[1]
    out = torch.empty_like(h)
    loc = seq_start_loc.tolist()
    lens = seq_lens.tolist()
    slots = state_slots.tolist()
    wf = weight.float()
    for i in range(len(lens)):
        a, b = loc[i], loc[i + 1]
        n = b - a
        if n == 0:
            continue
        start = lens[i] - n
        hist = state[slots[i]].float() if taps > 1 else h.new_zeros((0, h.shape[1]), dtype=torch.float32)
        if taps > 1:
            # state row j is position start - (taps-1) + j; negative => zero
            valid = (torch.arange(taps - 1) + start - (taps - 1)) >= 0
            hist = hist * valid.to(hist.dtype).unsqueeze(1).to(hist.device)
        ext = torch.cat([hist, h[a:b].float()], dim=0)     # [taps-1+n, W]
        acc = h[a:b].float().clone() if add_input else torch.zeros_like(ext[taps - 1:])
        for j in range(taps):
            acc = acc + wf[:, j] * ext[j:j + n]
        out[a:b] = acc.to(h.dtype)
        if taps > 1:
            state[slots[i]] = ext[n:].to(state.dtype)
    return out


def rope_partial(x: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor,
                 offset: int, rot_dims: int) -> None:
    """In place: dims [offset, offset+rot_dims) of the last axis of x [T, H, D]
    are rotated, dim i paired with i + rot_dims/2, angle = position * inv_freq[i]
    in f32."""
    half = rot_dims // 2
    ang = positions.to(torch.float32).unsqueeze(1) * inv_freq.float().unsqueeze(0)
    cos, sin = ang.cos().unsqueeze(1), ang.sin().unsqueeze(1)
    u = x[..., offset:offset + half].float()
    v = x[..., offset + half:offset + rot_dims].float()
    a = (u * cos - v * sin).to(x.dtype)   # both halves before either store:
    b = (v * cos + u * sin).to(x.dtype)   # for f32 x, u and v alias x
    x[..., offset:offset + half] = a
    x[..., offset + half:offset + rot_dims] = b


def latent_kv_write(
    dkv: torch.Tensor,          # [T, rank + rot]
    norm_weight: torch.Tensor,  # [rank]
    eps: float,
    positions: torch.Tensor,
    inv_freq: torch.Tensor,     # [rot_dims/2] f32
    rot_dims: int,
    cache: torch.Tensor,        # [blocks, block_size, rank + rot]
    slot_mapping: torch.Tensor,
) -> None:
    rank = norm_weight.shape[0]
    c = dkv[:, :rank].float()
    c = c * torch.rsqrt(c.pow(2).mean(dim=-1, keepdim=True) + eps) * norm_weight.float()
    kr = dkv[:, rank:].float().unsqueeze(1).clone()
    rope_partial(kr, positions, inv_freq, 0, rot_dims)
    row = torch.cat([c, kr.squeeze(1)], dim=-1).to(cache.dtype)
    bs = cache.shape[1]
    ok = slot_mapping >= 0
    sm = slot_mapping[ok]
    cache[torch.div(sm, bs, rounding_mode="floor"), sm % bs] = row[ok]


def latent_attention(
    q_lat: torch.Tensor,        # [T, H, rank]  (queries folded into latent space)
    q_rot: torch.Tensor,        # [T, H, rot]
    cache: torch.Tensor,        # [blocks, block_size, rank + rot]
    block_tables: torch.Tensor,
    query_start_loc: torch.Tensor,
    seq_lens: torch.Tensor,
    scale: float,
    window: int,                # 0 = unbounded causal
    sinks: torch.Tensor | None,  # [H] f32
) -> torch.Tensor:
    """Multi-query attention of every head over one shared latent row per
    token: score = (q_lat . c + q_rot . k_rot) * scale, softmax whose
    denominator also holds exp(sink_h), value = c.  Queries are the tail of
    each sequence."""
    t, nh, rank = q_lat.shape
    out = torch.zeros((t, nh, rank), dtype=q_lat.dtype, device=q_lat.device)
    qs = query_start_loc.tolist()
    lens = seq_lens.tolist()
    bs = cache.shape[1]
    for i in range(len(lens)):
        s, e = qs[i], qs[i + 1]
        n, sl = e - s, lens[i]
        if n == 0 or sl == 0:
            continue
        nb = (sl + bs - 1) // bs
        kv = cache[block_tables[i, :nb].long()].reshape(-1, cache.shape[-1])[:sl].float()
        q = torch.cat([q_lat[s:e].float(), q_rot[s:e].float()], dim=-1)
        sc = torch.einsum("qhd,sd->hqs", q, kv) * scale
        kpos = torch.arange(sl)
        qpos = torch.arange(sl - n, sl)
        dist = qpos[:, None] - kpos[None, :]
        bad = dist < 0
        if window > 0:
            bad = bad | (dist >= window)
        sc = sc.masked_fill(bad.unsqueeze(0).to(sc.device), float("-inf"))
        m = sc.max(dim=-1).values
        if sinks is not None:
            m = torch.maximum(m, sinks.float().view(-1, 1))
        p = torch.exp(sc - m.unsqueeze(-1))
        den = p.sum(dim=-1)
        if sinks is not None:
            den = den + torch.exp(sinks.float().view(-1, 1) - m)
        p = p / den.unsqueeze(-1)
        out[s:e] = torch.einsum("hqs,sd->qhd", p, kv[:, :rank]).to(out.dtype)
    return out
