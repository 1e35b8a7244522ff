"""A plain, slow implementation of the Dolodra design, one function per
mechanism, written from the design's equations in float64.  It shares no code
with the package: tests compare the engine against it.

Notation: x is the residual stream [n, width] of ONE sequence, processed whole.
Attention is computed in the expanded form (per-head keys and values are
materialised from the latent), not in the folded form the kernels use.
"""

from __future__ import annotations

import json
import math
import os

import torch

F64 = torch.float64


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm_around_zero(x, w, eps):
    return unit_rms(x, eps) * (1.0 + w)


def short_conv(h, w):
    """h + causal depthwise conv; w [width, taps], zeros before the start."""
    n, taps = h.shape[0], w.shape[1]
    out = h.clone()
    for t in range(n):
        for j in range(taps):
            src = t - taps + 1 + j
            if src >= 0:
                out[t] += w[:, j] * h[src]
    return out


def rotate_half(v, pos, base, dims):
    """v [..., dims'] with dims' >= dims: first `dims` dims rotated, dim i paired
    with i + dims/2; pos a scalar position."""
    out = v.clone()
    half = dims // 2
    for i in range(half):
        a = pos * float(base) ** (-2.0 * i / dims)
        c, s = math.cos(a), math.sin(a)
        u, w = v[..., i], v[..., i + half]
        out[..., i] = u * c - w * s
        out[..., i + half] = w * c + u * s
    return out


def latent_and_key(h, w_dkv, w_norm, eps, rank, base, dims):
    """Per token: normed latent c [n, rank] and the shared rotated key part."""
    dkv = h @ w_dkv.T
    c = unit_rms(dkv[:, :rank], eps) * w_norm
    kr = torch.stack([rotate_half(dkv[t, rank:], t, base, dims) for t in range(h.shape[0])])
    return c, kr


def latent_attention(h, c, kr, w_q, w_uk, w_uv, sink, w_o, *, heads, dim, rot_dim,
                     vdim, scale, window, base, dims):
    n = h.shape[0]
    q = (h @ w_q.T).view(n, heads, dim + rot_dim)
    out = torch.zeros(n, heads * vdim, dtype=h.dtype)
    for hh in range(heads):
        k_h = c @ w_uk[hh * dim:(hh + 1) * dim].T          # [n, dim]
        v_h = c @ w_uv[hh * vdim:(hh + 1) * vdim].T        # [n, vdim]
        for i in range(n):
            q_plain = q[i, hh, :dim]
            q_rot = rotate_half(q[i, hh, dim:], i, base, dims)
            lo = 0 if not window else max(0, i - window + 1)
            scores = torch.stack([
                (q_plain @ k_h[j] + q_rot @ kr[j]) * scale for j in range(lo, i + 1)])
            m = max(float(scores.max()), float(sink[hh]))
            e = torch.exp(scores - m)
            den = e.sum() + math.exp(float(sink[hh]) - m)
            p = e / den
            out[i, hh * vdim:(hh + 1) * vdim] = p @ v_h[lo:i + 1]
    return out @ w_o.T


def dense_ff(h, w_up, w_down):
    return gelu_tanh(h @ w_up.T) @ w_down.T


def token_side(x, e, w_gate, w_proj, w_norm, eps, mult):
    g = gelu_tanh(x @ w_gate.T) * e
    y = g @ w_proj.T
    return x + mult * unit_rms(y, eps) * w_norm


def softcap(z, cap):
    return cap * torch.tanh(z / cap)


def forward(cfg: dict, w: dict, tokens: list[int], layers_out: list | None = None):
    """Logits [n, vocab] of one whole sequence."""
    w = {k: v.to(F64) for k, v in w.items()}
    eps = cfg["norm"]["eps"]
    m = cfg.get("residual_mult", 1.0)
    tok = torch.tensor(tokens)
    x = w["embed"][tok] * cfg["embedding"]["scale"]
    sd = (cfg.get("token_side") or {}).get("dim", 0)
    kept: dict[int, tuple] = {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        mx = layer["mixer"]
        h = norm_around_zero(x, w[p + "norm1"], eps)
        hm = short_conv(h, w[p + "canon1"]) if cfg.get("canon") else h
        base, dims = mx["rot"]["base"], mx["rot"]["dims"]
        if mx.get("kv_from") is None:
            kept[i] = latent_and_key(hm, w[p + "mix.dkv"], w[p + "mix.dkv.norm"], eps,
                                     mx["kv_rank"], base, dims)
            c, kr = kept[i]
        else:
            c, kr = kept[mx["kv_from"]]
        mix = latent_attention(
            hm, c, kr, w[p + "mix.q"], w[p + "mix.uk"], w[p + "mix.uv"], w[p + "mix.sink"],
            w[p + "mix.o"], heads=mx["heads"], dim=mx["dim"], rot_dim=mx["rot_dim"],
            vdim=mx["vdim"], scale=mx["scale"], window=(mx.get("mask") or {}).get("size", 0),
            base=base, dims=dims)
        ff = dense_ff(h, w[p + "mlp.up"], w[p + "mlp.down"]) if layer.get("mlp") else 0.0
        x = x + m * (mix + ff)
        if sd:
            e = w["side.embed"][tok][:, i * sd:(i + 1) * sd]
            x = token_side(x, e, w[p + "side.gate"], w[p + "side.proj"], w[p + "side.norm"],
                           eps, m)
        if layers_out is not None:
            layers_out.append(x.clone())
    z = norm_around_zero(x, w["final.norm"], eps) @ w["head"].T
    cap = cfg.get("logit_softcap")
    return softcap(z, cap) if cap else z


# ---------------------------------------------------------------------------
# small random models on disk
# ---------------------------------------------------------------------------


def make_config(*, vocab=97, width=48, layers=None, taps=3, side_dim=6, mult=0.8,
                softcap_=12.0, eps=1e-5, embed_scale=2.5) -> dict:
    if layers is None:
        layers = [
            dict(heads=3, dim=8, rot_dim=4, vdim=10, kv_rank=20, window=5, ff=40),
            dict(heads=2, dim=6, rot_dim=4, vdim=8, kv_rank=20, window=9, ff=0, kv_from=0),
            dict(heads=1, dim=10, rot_dim=8, vdim=6, kv_rank=12, window=3, ff=24,
                 base=500.0),
        ]
    out = []
    for sp in layers:
        mixer = {
            "heads": sp["heads"], "dim": sp["dim"], "rot_dim": sp["rot_dim"],
            "vdim": sp["vdim"], "kv_rank": sp["kv_rank"],
            "scale": sp.get("scale", 1.7 / math.sqrt(sp["dim"] + sp["rot_dim"])),
            "mask": {"size": sp["window"]},
            "rot": {"base": sp.get("base", 10000.0), "dims": sp["rot_dim"]},
        }
        if sp.get("kv_from") is not None:
            mixer["kv_from"] = sp["kv_from"]
        out.append({
            "type": "latent_attention", "mixer": mixer,
            "mlp": {"kind": "dense", "ff": sp["ff"]} if sp.get("ff") else None,
        })
    cfg = {
        "architecture": "Dolodra", "vocab": vocab, "width": width, "layers": out,
        "norm": {"eps": eps}, "residual_mult": mult, "logit_softcap": softcap_,
        "embedding": {"scale": embed_scale},
    }
    if taps:
        cfg["canon"] = {"taps": taps}
    if side_dim:
        cfg["token_side"] = {"dim": side_dim}
    return cfg


def make_weights(cfg: dict, seed: int = 0, gain: float = 1.0) -> dict:
    """Random bf16 weights (stored values are exact in f32 and f64)."""
    g = torch.Generator().manual_seed(seed)
    width, vocab = cfg["width"], cfg["vocab"]
    nl = len(cfg["layers"])

    def r(*shape, std):
        return (torch.randn(*shape, generator=g) * std * gain).to(torch.bfloat16)

    w = {"embed": r(vocab, width, std=1.0), "head": r(vocab, width, std=0.3),
         "final.norm": r(width, std=0.2)}
    sd = (cfg.get("token_side") or {}).get("dim", 0)
    if sd:
        w["side.embed"] = r(vocab, nl * sd, std=1.0)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        mx = layer["mixer"]
        hq = mx["heads"] * (mx["dim"] + mx["rot_dim"])
        w[p + "norm1"] = r(width, std=0.2)
        w[p + "mix.q"] = r(hq, width, std=width ** -0.5)
        if mx.get("kv_from") is None:
            w[p + "mix.dkv"] = r(mx["kv_rank"] + mx["rot_dim"], width, std=width ** -0.5)
            w[p + "mix.dkv.norm"] = (1.0 + r(mx["kv_rank"], std=0.2).float()).to(torch.bfloat16)
        w[p + "mix.uk"] = r(mx["heads"] * mx["dim"], mx["kv_rank"], std=mx["kv_rank"] ** -0.5)
        w[p + "mix.uv"] = r(mx["heads"] * mx["vdim"], mx["kv_rank"], std=mx["kv_rank"] ** -0.5)
        w[p + "mix.sink"] = r(mx["heads"], std=1.0)
        w[p + "mix.o"] = r(width, mx["heads"] * mx["vdim"], std=(mx["heads"] * mx["vdim"]) ** -0.5)
        if layer.get("mlp"):
            ff = layer["mlp"]["ff"]
            w[p + "mlp.up"] = r(ff, width, std=width ** -0.5)
            w[p + "mlp.down"] = r(width, ff, std=ff ** -0.5)
        if cfg.get("canon"):
            w[p + "canon1"] = r(width, cfg["canon"]["taps"], std=0.4)
        if sd:
            w[p + "side.gate"] = r(sd, width, std=width ** -0.5)
            w[p + "side.proj"] = r(width, sd, std=sd ** -0.5)
            w[p + "side.norm"] = r(width, std=0.5)
    return w


def save_model(path, cfg: dict, w: dict) -> str:
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in w.items()}, os.path.join(path, "model.safetensors"))
    return str(path)
