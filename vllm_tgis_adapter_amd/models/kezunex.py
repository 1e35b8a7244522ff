"""Kezunex: a decoder-only model with an f32 residual stream whose layers mix
tokens in different ways, and whose first layers may be run several times.

A layer is x <- x + ls1 * LN1b(mixer(LN1(x))), then (if it has a feed-forward)
x <- x + ls2 * LN2b(ff(LN2(x))); every norm is a bias-free layer norm and ls*
are per-channel layer scales.  The mixer is one of

  parallel   grouped-query softmax attention (per-head query/key RMS norm, no
             rotation, a query temperature that grows with the position) and a
             state-space-duality recurrence fed the same normed input, their
             outputs mixed with fixed scales
  rglru      a recurrent block with a real-gated linear recurrent unit
  mlstm      a matrix memory with exponential gating

``loop`` = {start, stop, times} repeats the layer range [start, stop) ``times``
times with shared weights; cache and recurrent state are kept per pass.  A pass
after the first begins by adding the embedding output back into the stream, and
every pass (the first included) then adds its own row of ``loop.step``.  The
head is the final layer norm followed by the embedding table, unscaled.

Sizes and constants all come from config.json:

  vocab, width, norm.eps, embedding.scale, loop{start, stop, times},
  layers[i] = {type, mixer{...}, mlp{kind, ff} | null}

Tensors: embed, loop.step, final.norm, l<i>.{norm1, norm1b, norm2, norm2b, ls1,
ls2}, l<i>.mix.* (per mixer, see models/blocks.py), l<i>.mlp.{gate, up, down}.
"""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from .. import ops
from ..engine.config import ModelConfig
from ..engine.metadata import AttnMetadata
from ..parallel import get_tp_world_size
from .blocks import (
    GatedDenseMLP,
    MLSTMMixer,
    ParallelMixer,
    QKNormAttention,
    RGLRUMixer,
    SSDMixer,
    StreamLayerNorm,
    _f32_param,
)

# positions are unbounded in this design; the default bounds block tables and
# capture buffers and can be raised with --max-model-len
_DEFAULT_MAX_LEN = 32768

# log a = -RGLRU_C * r * softplus(lam) in the gated linear recurrent unit
RGLRU_C = 8.0


def build_mixer(kind: str, m: dict, width: int, eps: float, dtype: torch.dtype):
    if kind == "parallel":
        l, r = m["left"], m["right"]
        qt = l.get("q_temp") or {}
        left = QKNormAttention(
            width, heads=int(l["heads"]), kv_heads=int(l["kv_heads"]), dim=int(l["dim"]),
            vdim=int(l["vdim"]), scale=float(l["scale"]), eps=eps,
            temp_coef=float(qt.get("coef", 0.0)), temp_every=int(qt.get("every", 0)),
            own_in=False, dtype=dtype)
        right = SSDMixer(
            width, heads=int(r["heads"]), vdim=int(r["vdim"]), state=int(r["state"]),
            groups=int(r["groups"]), taps=int(r["conv"]),
            norm_groups=int(r["norm_groups"]), eps=eps, own_in=False, dtype=dtype)
        return ParallelMixer(width, left, right, float(m["left_scale"]),
                             float(m["right_scale"]), dtype)
    if kind == "rglru":
        return RGLRUMixer(width, rec_width=int(m["width"]), blocks=int(m["blocks"]),
                          taps=int(m["conv"]), gate_c=RGLRU_C, dtype=dtype)
    if kind == "mlstm":
        return MLSTMMixer(width, heads=int(m["heads"]), dim=int(m["dim"]),
                          vdim=int(m["vdim"]), gate_cap=float(m["gate_cap"]), eps=eps,
                          dtype=dtype)
    raise ValueError(f"unknown mixer type {kind!r}")


def layer_runs(hf: dict) -> list[tuple[int, Optional[int]]]:
    """(layer index, pass number at the first layer of a pass, else None) in
    the order the layers run."""
    n = len(hf["layers"])
    loop = hf.get("loop")
    if not loop or int(loop.get("times", 1)) < 1:
        return [(i, None) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    if not (0 <= a < b <= n):
        raise ValueError("loop: need 0 <= start < stop <= number of layers")
    runs: list[tuple[int, Optional[int]]] = [(i, None) for i in range(a)]
    for t in range(times):
        runs += [(i, t if i == a else None) for i in range(a, b)]
    runs += [(i, None) for i in range(b, n)]
    return runs


def model_config_from_json(model: str, hf: dict) -> ModelConfig:
    layers = hf["layers"]
    att = [e["mixer"]["left"] for e in layers if e.get("type") == "parallel"]
    return ModelConfig(
        model=model,
        architecture="kezunex",
        vocab_size=int(hf["vocab"]),
        hidden_size=int(hf["width"]),
        intermediate_size=max((int(e["mlp"]["ff"]) for e in layers if e.get("mlp")), default=0),
        num_layers=len(layer_runs(hf)),
        num_heads=max((int(a["heads"]) for a in att), default=1),
        num_kv_heads=max((int(a["kv_heads"]) for a in att), default=1),
        head_dim=max((int(a["dim"]) for a in att), default=1),
        rope_theta=0.0,
        rms_norm_eps=float((hf.get("norm") or {}).get("eps", 1e-5)),
        max_model_len=int(hf.get("max_len", _DEFAULT_MAX_LEN)),
        tie_word_embeddings=True,
        dtype=torch.bfloat16,
        hf_config=hf,
    )


def native_extensions(cfg: ModelConfig) -> list[str]:
    """The stream / recurrence / any-shape attention kernels always; the
    llama-class MFMA attention kernels (alone, without the rest of that
    extension) when an attention mixer has a shape they take."""
    need = ["_C_seq"]
    for e in cfg.hf_config["layers"]:
        if e.get("type") != "parallel":
            continue
        a = e["mixer"]["left"]
        if ops.attention_uses_matrix_cores(cfg.dtype, int(a["heads"]), int(a["kv_heads"]),
                                           int(a["dim"]), int(a["vdim"])):
            return need + ["_C_attn"]
    return need


class KezunexLayer(nn.Module):
    def __init__(self, idx: int, entry: dict, width: int, eps: float, dtype: torch.dtype):
        super().__init__()
        self.idx = idx
        self.kind = entry["type"]
        self.dtype = dtype
        self.eps = eps
        self.norm1 = StreamLayerNorm(width, eps, dtype)
        self.norm1b = _f32_param(width, fill=1.0)
        self.ls1 = _f32_param(width, fill=1.0)
        self.mix = build_mixer(self.kind, entry["mixer"], width, eps, dtype)
        mlp = entry.get("mlp")
        self.mlp = None
        if mlp is not None:
            if mlp.get("kind", "dense") != "dense":
                raise ValueError(f"layer {idx}: unknown feed-forward kind {mlp.get('kind')!r}")
            self.mlp = GatedDenseMLP(width, int(mlp["ff"]), dtype)
            self.norm2 = StreamLayerNorm(width, eps, dtype)
            self.norm2b = _f32_param(width, fill=1.0)
            self.ls2 = _f32_param(width, fill=1.0)

    def forward(self, x, positions, cache, meta, h=None, next_norm=None):
        """x: f32 stream, updated in place.  h: this layer's first norm when the
        kernel that last wrote the stream already produced it.  Returns what
        ``next_norm`` makes of the stream this layer leaves (or None)."""
        if h is None:
            h = self.norm1(x)
        after = self.norm2.as_next() if self.mlp is not None else next_norm
        if isinstance(self.mix, ParallelMixer):
            a, b = self.mix(h, positions, cache, meta)
            h = ops.stream_add_layer_norm(x, a, b, self.mix.left_scale, self.mix.right_scale,
                                          self.norm1b, self.ls1, self.eps, after)
        else:
            y = self.mix(h, positions, cache, meta)
            h = ops.stream_add_layer_norm(x, y, None, 1.0, 0.0, self.norm1b, self.ls1,
                                          self.eps, after)
        if self.mlp is not None:
            y = self.mlp(h)
            h = ops.stream_add_layer_norm(x, y, None, 1.0, 0.0, self.norm2b, self.ls2,
                                          self.eps, next_norm)
        return h


class KezunexForCausalLM(nn.Module):
    uses_seq_state = True

    def __init__(self, cfg: ModelConfig):
        super().__init__()
        if get_tp_world_size() != 1:
            raise ValueError("Kezunex is not sharded yet; run it with tensor_parallel_size 1")
        hf = cfg.hf_config
        self.cfg = cfg
        dtype = cfg.dtype
        width = cfg.hidden_size
        eps = cfg.rms_norm_eps
        self.embed_scale = float((hf.get("embedding") or {}).get("scale", 1.0))
        self.runs = layer_runs(hf)
        loop = hf.get("loop") or {}
        self.loop_times = int(loop.get("times", 0)) if loop else 0
        self.embed = nn.Parameter(
            torch.empty(cfg.vocab_size, width, dtype=dtype).normal_(0.0, 0.02),
            requires_grad=False)
        self.loop_step = _f32_param(max(self.loop_times, 1), width)
        self.layers = nn.ModuleList([
            KezunexLayer(i, e, width, eps, dtype) for i, e in enumerate(hf["layers"])])
        self.final_norm = StreamLayerNorm(width, eps, dtype)
        # set by the test harness to collect the stream after every layer run
        self.stream_probe: Optional[list] = None

    # -- cache layout (asked for by the worker) ----------------------------
    def _run_shapes(self, block_size: int):
        for li, _ in self.runs:
            yield self.layers[li].mix.cache_shapes(block_size)

    @staticmethod
    def _bytes(shape, dtype) -> int:
        n = 1
        for s in shape:
            n *= s
        return n * torch.tensor([], dtype=dtype).element_size()

    def cache_bytes_per_block(self, block_size: int) -> int:
        return max(1, sum(self._bytes(shape, dt) for shapes in self._run_shapes(block_size)
                          for kind, shape, dt in shapes if kind == "paged"))

    def state_bytes_per_slot(self) -> int:
        return sum(self._bytes(shape, dt) for shapes in self._run_shapes(1)
                   for kind, shape, dt in shapes if kind == "slot")

    def allocate_caches(self, num_blocks: int, block_size: int, num_slots: int,
                        device) -> list:
        """One entry per layer run (a looped layer has one per pass): the
        tensors its mixer names, paged ones [blocks, ...] and per-sequence ones
        [slots, ...]."""
        out = []
        for shapes in self._run_shapes(block_size):
            entry = []
            for kind, shape, dt in shapes:
                lead = num_blocks if kind == "paged" else max(num_slots, 1)
                entry.append(torch.zeros((lead,) + tuple(shape), dtype=dt, device=device))
            out.append(tuple(entry))
        return out

    # -- forward -----------------------------------------------------------
    def forward(self, input_ids, positions, kv_caches, meta: AttnMetadata) -> torch.Tensor:
        x = ops.embedding_scaled(input_ids, self.embed, self.embed_scale)   # f32 [T, W]
        x0 = x.clone() if self.loop_times > 1 else None
        h = None
        last = len(self.runs) - 1
        for r, (li, t) in enumerate(self.runs):
            layer = self.layers[li]
            if t is not None:
                ops.stream_add_vec(x, x0 if t > 0 else None, self.loop_step[t])
                h = None
            nxt = None
            if r == last:
                nxt = self.final_norm.as_next()
            elif self.runs[r + 1][1] is None:
                nxt = self.layers[self.runs[r + 1][0]].norm1.as_next()
            h = layer(x, positions, kv_caches[r], meta, h, nxt)
            if self.stream_probe is not None:
                self.stream_probe.append(x.clone())
        return h if h is not None else self.final_norm(x)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return ops.linear(hidden, self.embed).float()

    # -- weights -----------------------------------------------------------
    @staticmethod
    def _sub(weights: dict, prefix: str) -> dict:
        return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}

    def load_weights(self, weights: dict[str, torch.Tensor]) -> None:
        dtype = self.cfg.dtype
        self.embed.data.copy_(weights["embed"].to(dtype))
        if self.loop_times:
            self.loop_step.data.copy_(weights["loop.step"].float())
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            layer.norm1.weight.data.copy_(weights[p + "norm1"].float())
            layer.norm1b.data.copy_(weights[p + "norm1b"].float())
            layer.ls1.data.copy_(weights[p + "ls1"].float())
            if isinstance(layer.mix, ParallelMixer):
                layer.mix.load(self._sub(weights, p + "mix.left."),
                               self._sub(weights, p + "mix.right."))
            else:
                layer.mix.load(self._sub(weights, p + "mix."))
            if layer.mlp is not None:
                layer.mlp.load(weights[p + "mlp.gate"], weights[p + "mlp.up"],
                               weights[p + "mlp.down"])
                layer.norm2.weight.data.copy_(weights[p + "norm2"].float())
                layer.norm2b.data.copy_(weights[p + "norm2b"].float())
                layer.ls2.data.copy_(weights[p + "ls2"].float())
        self.final_norm.weight.data.copy_(weights["final.norm"].float())
