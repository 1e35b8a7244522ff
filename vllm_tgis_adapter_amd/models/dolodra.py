"""Dolodra: a decoder-only model with an f32 residual stream.

Every layer is a *parallel* block: one RMS norm (weight stored around zero)
feeds both the mixer and the feed-forward, and x <- x + m * (mixer + ff).
The mixer reads h + conv(h), a short causal convolution whose last inputs are
per-sequence state.  The mixer is latent attention (sliding window, softmax
sink); a layer may borrow the latent rows of an earlier layer instead of
projecting its own.  After the feed-forward a gated slice of a per-token side
embedding is added through its own norm.  Logits are soft-capped with tanh.

Sizes and constants all come from config.json:

  vocab, width, residual_mult, logit_softcap, norm.eps, embedding.scale,
  canon.taps, token_side.dim, layers[i] = {type, mixer{heads, dim, rot_dim,
  vdim, kv_rank, scale, mask.size, rot.base, rot.dims, kv_from?}, mlp{kind,
  ff} | null}

Tensors: embed, side.embed, l<i>.norm1, l<i>.canon1, l<i>.mix.{q, dkv,
dkv.norm, uk, uv, sink, o}, l<i>.mlp.{up, down}, l<i>.side.{gate, proj,
norm}, final.norm, head.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops
from ..engine.config import ModelConfig
from ..engine.metadata import AttnMetadata
from ..parallel import get_tp_world_size
from ..parallel.layers import ParallelLMHead
from .blocks import DenseMLP, LatentAttention, ShortConv, StreamRMSNorm, TokenSideInput

# positions are unbounded in this design (rotary only); the default bounds
# block tables and capture buffers and can be raised with --max-model-len
_DEFAULT_MAX_LEN = 32768


@dataclass
class LatentMixerSpec:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    rank: int
    scale: float
    window: int          # 0 = plain causal
    rot_base: float
    rot_dims: int
    kv_from: Optional[int]

    @staticmethod
    def from_json(m: dict) -> "LatentMixerSpec":
        rot = m.get("rot") or {}
        rot_dim = int(m["rot_dim"])
        dim = int(m["dim"])
        mask = m.get("mask") or {}
        return LatentMixerSpec(
            heads=int(m["heads"]), dim=dim, rot_dim=rot_dim, vdim=int(m["vdim"]),
            rank=int(m["kv_rank"]),
            scale=float(m.get("scale", (dim + rot_dim) ** -0.5)),
            window=int(mask.get("size") or 0),
            rot_base=float(rot.get("base", 10000.0)),
            rot_dims=int(rot.get("dims", rot_dim)),
            kv_from=(int(m["kv_from"]) if m.get("kv_from") is not None else None),
        )


@dataclass
class LayerSpec:
    mixer: LatentMixerSpec
    ff: int              # 0 = no feed-forward


def parse_layers(hf: dict) -> list[LayerSpec]:
    out = []
    for i, entry in enumerate(hf["layers"]):
        if entry.get("type") != "latent_attention":
            raise ValueError(f"layer {i}: unknown mixer type {entry.get('type')!r}")
        mlp = entry.get("mlp")
        ff = 0
        if mlp is not None:
            if mlp.get("kind", "dense") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            ff = int(mlp["ff"])
        out.append(LayerSpec(LatentMixerSpec.from_json(entry["mixer"]), ff))
    for i, spec in enumerate(out):
        j = spec.mixer.kv_from
        if j is None:
            continue
        if not (0 <= j < i) or out[j].mixer.kv_from is not None:
            raise ValueError(f"layer {i}: kv_from must name an earlier layer with a latent of its own")
        a, b = spec.mixer, out[j].mixer
        if (a.rank, a.rot_dim, a.rot_dims, a.rot_base) != (b.rank, b.rot_dim, b.rot_dims, b.rot_base):
            raise ValueError(f"layer {i}: latent sizes and rotation must equal layer {j}'s")
    return out


def model_config_from_json(model: str, hf: dict) -> ModelConfig:
    layers = parse_layers(hf)
    widest = max(layers, key=lambda s: s.mixer.rank + s.mixer.rot_dim).mixer
    return ModelConfig(
        model=model,
        architecture="dolodra",
        vocab_size=int(hf["vocab"]),
        hidden_size=int(hf["width"]),
        intermediate_size=max((s.ff for s in layers), default=0),
        num_layers=len(layers),
        num_heads=max(s.mixer.heads for s in layers),
        num_kv_heads=1,
        head_dim=widest.rank + widest.rot_dim,
        rope_theta=widest.rot_base,
        rms_norm_eps=float((hf.get("norm") or {}).get("eps", 1e-6)),
        max_model_len=int(hf.get("max_len", _DEFAULT_MAX_LEN)),
        tie_word_embeddings=False,
        dtype=torch.bfloat16,
        hf_config=hf,
    )


class DolodraLayer(nn.Module):
    def __init__(self, idx: int, spec: LayerSpec, width: int, eps: float, mult: float,
                 taps: int, side_dim: int, dtype: torch.dtype):
        super().__init__()
        self.idx = idx
        self.mult = mult
        self.dtype = dtype
        self.norm1 = StreamRMSNorm(width, eps, 1.0, dtype)
        self.canon = ShortConv(width, taps) if taps > 0 else None
        m = spec.mixer
        self.mix = LatentAttention(
            width, heads=m.heads, dim=m.dim, rot_dim=m.rot_dim, vdim=m.vdim,
            rank=m.rank, scale=m.scale, window=m.window, rot_base=m.rot_base,
            rot_dims=m.rot_dims, eps=eps, kv_owner=m.kv_from is None,
            has_sink=True, dtype=dtype)
        self.mlp = DenseMLP(width, spec.ff, dtype) if spec.ff else None
        self.side = TokenSideInput(width, side_dim, eps, mult, dtype) if side_dim else None

    def forward(self, x, positions, cache, meta, side_e, h=None, next_norm=None):
        """x: f32 stream (updated in place).  h: this layer's norm1 output when
        the previous layer already produced it.  Returns (x, h_next): h_next is
        next_norm(x) computed inside the side-input kernel, or None."""
        latent, conv_state = cache
        if h is None:
            h = self.norm1(x)
        hm = self.canon(h, conv_state, meta) if self.canon is not None else h
        mix = self.mix(hm, positions, latent, meta)
        ff = self.mlp(h) if self.mlp is not None else None
        xc = ops.stream_add(x, mix, ff, self.mult,
                            cast_dtype=self.dtype if self.side is not None else None)
        h_next = None
        if self.side is not None:
            h_next = self.side(x, xc, side_e, next_norm)
        return x, h_next


class DolodraForCausalLM(nn.Module):
    uses_seq_state = True

    def __init__(self, cfg: ModelConfig):
        super().__init__()
        hf = cfg.hf_config
        self.cfg = cfg
        dtype = cfg.dtype
        self.specs = parse_layers(hf)
        tp = get_tp_world_size()
        for s in self.specs:
            if s.mixer.heads % tp or (s.ff and s.ff % tp):
                raise ValueError("heads and ff of every layer must divide by the TP degree")
        width = cfg.hidden_size
        eps = cfg.rms_norm_eps
        self.mult = float(hf.get("residual_mult", 1.0))
        self.embed_scale = float((hf.get("embedding") or {}).get("scale", 1.0))
        self.softcap = float(hf.get("logit_softcap") or 0.0)
        self.taps = int((hf.get("canon") or {}).get("taps", 0))
        self.side_dim = int((hf.get("token_side") or {}).get("dim", 0))
        nl = len(self.specs)

        self.embed = nn.Parameter(
            torch.empty(cfg.vocab_size, width, dtype=dtype).normal_(0.0, 0.02),
            requires_grad=False)
        self.side_embed = (
            nn.Parameter(torch.empty(cfg.vocab_size, nl * self.side_dim,
                                     dtype=dtype).normal_(0.0, 0.02), requires_grad=False)
            if self.side_dim else None)
        self.layers = nn.ModuleList([
            DolodraLayer(i, s, width, eps, self.mult, self.taps, self.side_dim, dtype)
            for i, s in enumerate(self.specs)
        ])
        self.final_norm = StreamRMSNorm(width, eps, 1.0, dtype)
        self.lm_head = ParallelLMHead(cfg.vocab_size, width, dtype=dtype)

    # -- cache layout (asked for by the worker) ----------------------------
    def _elt(self) -> int:
        return torch.tensor([], dtype=self.cfg.dtype).element_size()

    def cache_bytes_per_block(self, block_size: int) -> int:
        rows = sum(s.mixer.rank + s.mixer.rot_dim for s in self.specs
                   if s.mixer.kv_from is None)
        return rows * block_size * self._elt()

    def state_bytes_per_slot(self) -> int:
        return len(self.specs) * max(self.taps - 1, 0) * self.cfg.hidden_size * self._elt()

    def allocate_caches(self, num_blocks: int, block_size: int, num_slots: int,
                        device) -> list:
        """Per layer (latent rows [blocks, block_size, rank + rot], conv state
        [slots, taps-1, width]); a borrowing layer gets its owner's tensor."""
        dtype = self.cfg.dtype
        latents: dict[int, torch.Tensor] = {}
        out = []
        for i, s in enumerate(self.specs):
            m = s.mixer
            if m.kv_from is None:
                latents[i] = torch.zeros(
                    (num_blocks, block_size, m.rank + m.rot_dim), dtype=dtype, device=device)
                lat = latents[i]
            else:
                lat = latents[m.kv_from]
            state = torch.zeros(
                (max(num_slots, 1), max(self.taps - 1, 0), self.cfg.hidden_size),
                dtype=dtype, device=device)
            out.append((lat, state))
        return out

    # -- forward -----------------------------------------------------------
    def forward(self, input_ids, positions, kv_caches, meta: AttnMetadata) -> torch.Tensor:
        x = ops.embedding_scaled(input_ids, self.embed, self.embed_scale)   # f32 [T, W]
        side = F.embedding(input_ids, self.side_embed) if self.side_dim else None
        sd = self.side_dim
        h = None
        last = len(self.layers) - 1
        for i, layer in enumerate(self.layers):
            e = side[:, i * sd:(i + 1) * sd] if sd else None
            nxt = self.layers[i + 1].norm1 if i < last else self.final_norm
            x, h = layer(x, positions, kv_caches[i], meta, e, h, nxt)
        return h if h is not None else self.final_norm(x)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        logits = self.lm_head(hidden)
        if self.softcap:
            return ops.softcap(logits, self.softcap)
        return logits.float()

    # -- weights -----------------------------------------------------------
    def load_weights(self, weights: dict[str, torch.Tensor]) -> None:
        dtype = self.cfg.dtype
        self.embed.data.copy_(weights["embed"].to(dtype))
        if self.side_embed is not None:
            self.side_embed.data.copy_(weights["side.embed"].to(dtype))
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            layer.norm1.weight.data.copy_(weights[p + "norm1"].float())
            if layer.canon is not None:
                layer.canon.weight.data.copy_(weights[p + "canon1"].float())
            owner = layer.mix.kv_owner
            layer.mix.load(
                weights[p + "mix.q"],
                weights[p + "mix.dkv"] if owner else None,
                weights[p + "mix.dkv.norm"] if owner else None,
                weights[p + "mix.uk"], weights[p + "mix.uv"],
                weights[p + "mix.sink"], weights[p + "mix.o"])
            if layer.mlp is not None:
                layer.mlp.up.load_full_weight(weights[p + "mlp.up"])
                layer.mlp.down.load_full_weight(weights[p + "mlp.down"])
            if layer.side is not None:
                layer.side.gate.data.copy_(weights[p + "side.gate"].to(dtype))
                layer.side.proj.data.copy_(weights[p + "side.proj"].to(dtype))
                layer.side.norm.data.copy_(weights[p + "side.norm"].float())
        self.final_norm.weight.data.copy_(weights["final.norm"].float())
        self.lm_head.load_full_weight(weights["head"])
