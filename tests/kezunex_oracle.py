"""Plain, slow float64 implementation of the Kezunex design, written from its
equations: one function per mechanism, whole sequences only, no cache, no
batching, token-by-token recurrences.  It shares no code with the package and
is the yardstick for tests/test_kezunex.py.

Notation: h is a sublayer's input [T, width]; weights are stored [out, in]
and applied as W h; positions count from 0.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def _w(weights, name):
    return weights[name].to(F64)


def lin(w, x, b=None):
    y = x @ w.T
    return y if b is None else y + b


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def layer_norm(x, w, eps):
    mu = x.mean(dim=-1, keepdim=True)
    d = x - mu
    var = (d * d).mean(dim=-1, keepdim=True)
    return d / torch.sqrt(var + eps) * w


def causal_conv(u, w, b):
    """u [T, C]; column j of w [C, taps] weighs the input taps-1-j steps back;
    inputs before position 0 count as zero."""
    t, c = u.shape
    taps = w.shape[1]
    out = torch.zeros_like(u)
    for j in range(taps):
        shift = taps - 1 - j
        if shift >= t:
            continue
        out[shift:] += u[: t - shift] * w[:, j]
    return out + b


# ---------------------------------------------------------------------------
# mixers
# ---------------------------------------------------------------------------

def softmax_attention(h, weights, p, m, eps):
    """Grouped-query softmax attention, per-head RMS norm on q and k, no
    rotation, a position-dependent query temperature, causal."""
    t = h.shape[0]
    nh, ng, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = lin(_w(weights, p + "q"), h).view(t, nh, d)
    k = lin(_w(weights, p + "k"), h).view(t, ng, d)
    v = lin(_w(weights, p + "v"), h).view(t, ng, dv)
    q = rms_unit(q, eps) * _w(weights, p + "q.norm")
    k = rms_unit(k, eps) * _w(weights, p + "k.norm")
    qt = m.get("q_temp")
    if qt:
        pos = torch.arange(t, dtype=F64)
        temp = 1.0 + qt["coef"] * torch.log(torch.floor((pos + 1.0) / qt["every"]) + 1.0)
        q = q * temp.view(t, 1, 1)
    out = torch.zeros(t, nh, dv, dtype=F64)
    per = nh // ng
    for hd in range(nh):
        g = hd // per
        s = (q[:, hd] @ k[:, g].T) * m["scale"]
        mask = torch.ones(t, t, dtype=torch.bool).tril()
        s = s.masked_fill(~mask, float("-inf"))
        out[:, hd] = torch.softmax(s, dim=-1) @ v[:, g]
    return lin(_w(weights, p + "o"), out.reshape(t, nh * dv))


def ssd(h, weights, p, m, eps):
    """State-space-duality recurrence with a short convolution in front and a
    gated grouped RMS norm behind."""
    t = h.shape[0]
    nh, dv, n, g = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = nh * dv
    zxbcdt = lin(_w(weights, p + "in"), h)
    z = zxbcdt[:, :inner]
    xbc = zxbcdt[:, inner:2 * inner + 2 * g * n]
    dt = zxbcdt[:, 2 * inner + 2 * g * n:]
    xbc = silu(causal_conv(xbc, _w(weights, p + "conv"), _w(weights, p + "conv.b")))
    x = xbc[:, :inner].view(t, nh, dv)
    bmat = xbc[:, inner:inner + g * n].view(t, g, n)
    cmat = xbc[:, inner + g * n:].view(t, g, n)
    dt = softplus(dt + _w(weights, p + "dt_bias"))
    a = torch.exp(_w(weights, p + "A_log"))
    dskip = _w(weights, p + "D")
    per = nh // g
    y = torch.zeros(t, nh, dv, dtype=F64)
    for hd in range(nh):
        grp = hd // per
        s = torch.zeros(n, dv, dtype=F64)
        for i in range(t):
            s = math.exp(-a[hd].item() * dt[i, hd].item()) * s \
                + dt[i, hd] * torch.outer(bmat[i, grp], x[i, hd])
            y[i, hd] = s.T @ cmat[i, grp] + dskip[hd] * x[i, hd]
    y = y.reshape(t, inner) * silu(z)
    ng = m["norm_groups"]
    y = rms_unit(y.view(t, ng, inner // ng), eps).reshape(t, inner) * _w(weights, p + "norm")
    return lin(_w(weights, p + "o"), y)


def parallel_mixer(h, weights, p, m, eps):
    left = softmax_attention(h, weights, p + "left.", m["left"], eps)
    right = ssd(h, weights, p + "right.", m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


def rglru(h, weights, p, m, eps):
    """Recurrent block with a real-gated linear recurrent unit."""
    t = h.shape[0]
    width, nb = m["width"], m["blocks"]
    y = gelu_tanh(lin(_w(weights, p + "y"), h, _w(weights, p + "y.b")))
    u = causal_conv(lin(_w(weights, p + "x"), h, _w(weights, p + "x.b")),
                    _w(weights, p + "conv"), _w(weights, p + "conv.b"))
    ub = u.view(t, nb, width // nb)
    ra, rab = _w(weights, p + "ra"), _w(weights, p + "ra.b")
    ri, rib = _w(weights, p + "ri"), _w(weights, p + "ri.b")
    r = torch.sigmoid(torch.einsum("boi,tbi->tbo", ra, ub) + rab).reshape(t, width)
    gate = torch.sigmoid(torch.einsum("boi,tbi->tbo", ri, ub) + rib).reshape(t, width)
    log_a = -8.0 * r * softplus(_w(weights, p + "lam"))
    a = torch.exp(log_a)
    s = torch.zeros(width, dtype=F64)
    out = torch.zeros(t, width, dtype=F64)
    for i in range(t):
        s = a[i] * s + torch.sqrt(1.0 - a[i] ** 2) * gate[i] * u[i]
        out[i] = s
    return lin(_w(weights, p + "o"), out * y)


def mlstm(h, weights, p, m, eps):
    """Matrix memory with exponential gating, stabilised by a running maximum
    initialised to 0."""
    t = h.shape[0]
    nh, d, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (lin(_w(weights, p + "q"), h) * d ** -0.5).view(t, nh, d)
    k = lin(_w(weights, p + "k"), h).view(t, nh, d)
    v = lin(_w(weights, p + "v"), h).view(t, nh, dv)
    ig = cap * torch.tanh(lin(_w(weights, p + "i"), h, _w(weights, p + "i.b")) / cap)
    fg = torch.nn.functional.logsigmoid(
        cap * torch.tanh(lin(_w(weights, p + "f"), h, _w(weights, p + "f.b")) / cap))
    o = torch.zeros(t, nh, dv, dtype=F64)
    for hd in range(nh):
        s = torch.zeros(d, dv, dtype=F64)
        n = torch.zeros(d, dtype=F64)
        mx = 0.0
        for i in range(t):
            f, g = fg[i, hd].item(), ig[i, hd].item()
            m_new = max(f + mx, g)
            s = math.exp(f + mx - m_new) * s + math.exp(g - m_new) * torch.outer(k[i, hd], v[i, hd])
            n = math.exp(f + mx - m_new) * n + math.exp(g - m_new) * k[i, hd]
            mx = m_new
            den = max(abs(float(n @ q[i, hd])), math.exp(-mx)) + 1e-6
            o[i, hd] = (s.T @ q[i, hd]) / den
    o = rms_unit(o, eps).reshape(t, nh * dv) * _w(weights, p + "norm")
    o = o * torch.sigmoid(lin(_w(weights, p + "g"), h))
    return lin(_w(weights, p + "o"), o)


MIXERS = {"parallel": parallel_mixer, "rglru": rglru, "mlstm": mlstm}


def dense_ff(h, weights, p):
    return lin(_w(weights, p + "down"),
               gelu_tanh(lin(_w(weights, p + "gate"), h)) * lin(_w(weights, p + "up"), h))


# ---------------------------------------------------------------------------
# whole model
# ---------------------------------------------------------------------------

def layer_schedule(cfg):
    """[(layer index, pass number or None, first of its pass)] in run order."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    runs = [(i, None, False) for i in range(a)]
    for t in range(times):
        runs += [(i, t, i == a) for i in range(a, b)]
    runs += [(i, None, False) for i in range(b, n)]
    return runs


def forward(cfg, weights, tokens, return_layers=False):
    """Logits [T, vocab] (f64) for one whole sequence; optionally also the
    residual stream after every layer run."""
    eps = cfg["norm"]["eps"]
    ids = torch.as_tensor(tokens, dtype=torch.long)
    emb = _w(weights, "embed")
    x0 = emb[ids] * cfg["embedding"]["scale"]
    x = x0.clone()
    streams = []
    for i, t, first in layer_schedule(cfg):
        if first:
            if t > 0:
                x = x + x0
            x = x + _w(weights, "loop.step")[t]
        spec = cfg["layers"][i]
        p = f"l{i}."
        h = layer_norm(x, _w(weights, p + "norm1"), eps)
        y = MIXERS[spec["type"]](h, weights, p + "mix.", spec["mixer"], eps)
        x = x + layer_norm(y, _w(weights, p + "norm1b"), eps) * _w(weights, p + "ls1")
        if spec.get("mlp") is not None:
            h = layer_norm(x, _w(weights, p + "norm2"), eps)
            y = dense_ff(h, weights, p + "mlp.")
            x = x + layer_norm(y, _w(weights, p + "norm2b"), eps) * _w(weights, p + "ls2")
        streams.append(x.clone())
    x = layer_norm(x, _w(weights, "final.norm"), eps)
    logits = x @ emb.T
    if return_layers:
        return logits, torch.stack(streams)
    return logits


# ---------------------------------------------------------------------------
# small configurations and random weights for the tests
# ---------------------------------------------------------------------------

def attn_spec(heads=4, kv_heads=2, dim=8, vdim=6, scale=0.3, coef=0.4, every=5):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if every:
        m["q_temp"] = {"coef": coef, "every": every}
    return m


def ssd_spec(heads=4, vdim=6, state=5, groups=2, conv=3, norm_groups=2):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
            "norm_groups": norm_groups}


def layer(kind, ff=0, **kw):
    if kind == "parallel":
        mixer = {"left": kw.get("left") or attn_spec(), "right": kw.get("right") or ssd_spec(),
                 "left_scale": kw.get("left_scale", 0.7), "right_scale": kw.get("right_scale", 0.4)}
    elif kind == "rglru":
        mixer = {"width": kw.get("width", 24), "blocks": kw.get("blocks", 3),
                 "conv": kw.get("conv", 4)}
    elif kind == "mlstm":
        mixer = {"heads": kw.get("heads", 3), "dim": kw.get("dim", 4), "vdim": kw.get("vdim", 6),
                 "gate_cap": kw.get("gate_cap", 9.0)}
    else:
        raise ValueError(kind)
    return {"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def make_config(*, vocab=101, width=40, layers=None, loop=(1, 3, 2), eps=1e-5,
                embed_scale=2.0) -> dict:
    if layers is None:
        layers = [layer("rglru"), layer("parallel", ff=48), layer("mlstm"),
                  layer("parallel", ff=0, left=attn_spec(3, 3, 6, 10, 0.25, 0.3, 3),
                        right=ssd_spec(2, 8, 7, 1, 2, 1))]
    cfg = {"architecture": "Kezunex", "vocab": vocab, "width": width, "layers": layers,
           "norm": {"eps": eps}, "embedding": {"scale": embed_scale}}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def make_weights(cfg: dict, seed: int = 0) -> dict:
    """Random bf16 weights (their values are exact in f32 and f64)."""
    g = torch.Generator().manual_seed(seed)
    width, vocab = cfg["width"], cfg["vocab"]

    def r(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).to(torch.bfloat16)

    w = {"embed": r(vocab, width, std=0.7), "final.norm": r(width, std=0.2, mean=1.0)}
    if cfg.get("loop"):
        w["loop.step"] = r(cfg["loop"]["times"], width, std=0.5)
    for i, e in enumerate(cfg["layers"]):
        p = f"l{i}."
        for nm in ("norm1", "norm1b"):
            w[p + nm] = r(width, std=0.2, mean=1.0)
        w[p + "ls1"] = r(width, std=0.3, mean=0.6)
        m = e["mixer"]
        q = p + "mix."
        fan = width ** -0.5
        if e["type"] == "parallel":
            a, s = m["left"], m["right"]
            w[q + "left.q"] = r(a["heads"] * a["dim"], width, std=fan)
            w[q + "left.k"] = r(a["kv_heads"] * a["dim"], width, std=fan)
            w[q + "left.v"] = r(a["kv_heads"] * a["vdim"], width, std=fan)
            w[q + "left.q.norm"] = r(a["dim"], std=0.3, mean=1.0)
            w[q + "left.k.norm"] = r(a["dim"], std=0.3, mean=1.0)
            w[q + "left.o"] = r(width, a["heads"] * a["vdim"], std=(a["heads"] * a["vdim"]) ** -0.5)
            inner = s["heads"] * s["vdim"]
            ch = inner + 2 * s["groups"] * s["state"]
            w[q + "right.in"] = r(inner + ch + s["heads"], width, std=fan)
            w[q + "right.conv"] = r(ch, s["conv"], std=0.5)
            w[q + "right.conv.b"] = r(ch, std=0.2)
            w[q + "right.dt_bias"] = r(s["heads"], std=1.0, mean=-1.0)
            w[q + "right.A_log"] = r(s["heads"], std=0.7)
            w[q + "right.D"] = r(s["heads"], std=0.5, mean=1.0)
            w[q + "right.norm"] = r(inner, std=0.2, mean=1.0)
            w[q + "right.o"] = r(width, inner, std=inner ** -0.5)
        elif e["type"] == "rglru":
            rw, nb = m["width"], m["blocks"]
            bw = rw // nb
            for nm in ("y", "x"):
                w[q + nm] = r(rw, width, std=fan)
                w[q + nm + ".b"] = r(rw, std=0.2)
            w[q + "conv"] = r(rw, m["conv"], std=0.5)
            w[q + "conv.b"] = r(rw, std=0.2)
            for nm in ("ra", "ri"):
                w[q + nm] = r(nb, bw, bw, std=bw ** -0.5)
                w[q + nm + ".b"] = r(nb, bw, std=0.5)
            w[q + "lam"] = r(rw, std=1.0, mean=-2.0)
            w[q + "o"] = r(width, rw, std=rw ** -0.5)
        else:
            nh, d, dv = m["heads"], m["dim"], m["vdim"]
            w[q + "q"] = r(nh * d, width, std=fan)
            w[q + "k"] = r(nh * d, width, std=fan)
            w[q + "v"] = r(nh * dv, width, std=fan)
            w[q + "g"] = r(nh * dv, width, std=fan)
            w[q + "i"] = r(nh, width, std=fan * 2)
            w[q + "i.b"] = r(nh, std=1.0)
            w[q + "f"] = r(nh, width, std=fan * 2)
            w[q + "f.b"] = r(nh, std=1.0, mean=2.0)
            w[q + "norm"] = r(nh * dv, std=0.2, mean=1.0)
            w[q + "o"] = r(width, nh * dv, std=(nh * dv) ** -0.5)
        if e.get("mlp"):
            ff = e["mlp"]["ff"]
            for nm in ("norm2", "norm2b"):
                w[p + nm] = r(width, std=0.2, mean=1.0)
            w[p + "ls2"] = r(width, std=0.3, mean=0.6)
            w[p + "mlp.gate"] = r(ff, width, std=fan)
            w[p + "mlp.up"] = r(ff, width, std=fan)
            w[p + "mlp.down"] = r(width, ff, std=ff ** -0.5)
    return w


def save_model(path, cfg: dict, w: dict) -> str:
    import json
    import os

    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in w.items()}, os.path.join(path, "model.safetensors"))
    return str(path)
