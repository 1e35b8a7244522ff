"""HIP kernels of the `_C_seq` extension against the plain PyTorch reference of
the same op (f32 and bf16 storage; odd sizes included)."""

from __future__ import annotations

import pytest
import torch

from vllm_tgis_adapter_amd import ops
from vllm_tgis_adapter_amd.ops import reference as ref

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def _tol(dtype):
    return dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


@pytest.fixture(autouse=True)
def _need_ext():
    assert torch.cuda.is_available()
    assert ops.has_native_seq(), "_C_seq must be built"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("t,w", [(37, 200), (5, 199)])   # rows of 4-groups / odd rows
def test_elementwise_and_norms(dtype, t, w):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(t, w, generator=g) * 3
    a = torch.randn(t, w, generator=g).to(dtype)
    b = torch.randn(t, w, generator=g).to(dtype)
    wt = torch.randn(w, generator=g) * 0.2
    xd, ad, bd, wd = x.cuda(), a.cuda(), b.cuda(), wt.cuda()

    torch.testing.assert_close(
        ops.rms_norm_stream(xd, wd, 1e-6, 1.0, dtype).cpu().float(),
        ref.rms_norm_stream(x, wt, 1e-6, 1.0, dtype).float(), **_tol(dtype))
    torch.testing.assert_close(
        ops.gelu_tanh(ad).cpu().float(), ref.gelu_tanh(a).float(), **_tol(dtype))
    mul = torch.randn(t, 3 * w, generator=g).to(dtype)
    torch.testing.assert_close(
        ops.gelu_tanh(ad, mul.cuda()[:, w:2 * w]).cpu().float(),
        ref.gelu_tanh(a, mul[:, w:2 * w]).float(), **_tol(dtype))

    x1, x2 = x.clone(), xd.clone()
    c1 = ref.stream_add(x1, a, b, 0.6, dtype)
    c2 = ops.stream_add(x2, ad, bd, 0.6, dtype)
    torch.testing.assert_close(x2.cpu(), x1, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(c2.cpu().float(), c1.float(), **_tol(dtype))
    assert ops.stream_add(x2, ad, None, 0.5) is None
    ref.stream_add(x1, a, None, 0.5, None)
    torch.testing.assert_close(x2.cpu(), x1, atol=1e-5, rtol=1e-5)

    ref.stream_add_rms_norm(x1, a, wt, 1e-6, 0.6)
    ops.stream_add_rms_norm(x2, ad, wd, 1e-6, 0.6)
    torch.testing.assert_close(x2.cpu(), x1, atol=2e-5, rtol=1e-5)
    # the same with the following norm fused in
    ref.stream_add_rms_norm(x1, b, wt, 1e-6, 0.3)
    h2 = ops.stream_add_rms_norm(x2, bd, wd, 1e-6, 0.3, (wd, 1e-5, 1.0, dtype))
    torch.testing.assert_close(x2.cpu(), x1, atol=2e-5, rtol=1e-5)
    torch.testing.assert_close(h2.cpu().float(),
                               ref.rms_norm_stream(x1, wt, 1e-5, 1.0, dtype).float(), **_tol(dtype))

    torch.testing.assert_close(
        ops.softcap(ad * 10, 15.0).cpu(), ref.softcap(a * 10, 15.0), atol=1e-5, rtol=1e-5)
    ids = torch.randint(0, t, (50,), generator=g)
    torch.testing.assert_close(
        ops.embedding_scaled(ids.cuda(), ad, 3.5).cpu(), ref.embedding_scaled(ids, a, 3.5))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps", [1, 2, 3, 4, 5])
def test_causal_conv_state(dtype, taps):
    g = torch.Generator().manual_seed(taps)
    w = 72
    wt = torch.randn(w, taps, generator=g) * 0.5
    state = torch.randn(6, taps - 1, w, generator=g).to(dtype)  # stale garbage
    # sequences: fresh start (3 rows), continuing (1 row), continuing (7 rows),
    # a start shorter than the taps, a padding row (slot -1)
    loc = torch.tensor([0, 3, 4, 11, 12, 13], dtype=torch.int32)
    lens = torch.tensor([3, 9, 20, 1, 0], dtype=torch.int32)
    slots = torch.tensor([4, 0, 2, 5, -1], dtype=torch.int32)
    h = torch.randn(13, w, generator=g).to(dtype)
    s1, s2 = state.clone(), state.cuda()
    o1 = ref.causal_conv_state(h[:12], wt, s1, loc[:5], lens[:4], slots[:4], True)
    o2 = ops.causal_conv_state(h.cuda(), wt.cuda(), s2, loc.cuda(), lens.cuda(),
                               slots.cuda(), True)
    torch.testing.assert_close(o2.cpu()[:12].float(), o1.float(), **_tol(dtype))
    assert float(o2[12].abs().max()) == 0.0
    for sl, ln in zip(slots[:4].tolist(), lens[:4].tolist()):
        keep = min(ln, taps - 1)   # rows before the sequence's start are free
        if keep:
            torch.testing.assert_close(s2.cpu()[sl, taps - 1 - keep:].float(),
                                       s1[sl, taps - 1 - keep:].float(), **_tol(dtype))
    torch.testing.assert_close(s2.cpu()[1], state[1])   # untouched slot


@pytest.mark.parametrize("dtype", DTYPES)
def test_rope_and_latent_write(dtype):
    g = torch.Generator().manual_seed(3)
    t, nh, d, r, rank = 19, 3, 24, 16, 40
    q = torch.randn(t, nh, d + r, generator=g).to(dtype)
    pos = torch.randint(0, 5000, (t,), generator=g)
    inv = torch.tensor([10000.0 ** (-2 * i / 12) for i in range(6)])
    q1, q2 = q.clone(), q.cuda()
    ref.rope_partial(q1, pos, inv, d, 12)
    ops.rope_partial(q2, pos.cuda(), inv.cuda(), d, 12)
    torch.testing.assert_close(q2.cpu().float(), q1.float(), **_tol(dtype))

    dkv = torch.randn(t, rank + r, generator=g).to(dtype)
    nw = torch.randn(rank, generator=g)
    c1 = torch.zeros(8, 4, rank + r, dtype=dtype)
    c2 = c1.cuda()
    slots = torch.randperm(32, generator=g)[:t]
    slots[5] = -1
    ref.latent_kv_write(dkv, nw, 1e-6, pos, inv, 12, c1, slots)
    ops.latent_kv_write(dkv.cuda(), nw.cuda(), 1e-6, pos.cuda(), inv.cuda(), 12, c2,
                        slots.cuda())
    torch.testing.assert_close(c2.cpu().float(), c1.float(), **_tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rank,rot,window", [(40, 16, 7), (96, 64, 24), (130, 6, 0),
                                             (300, 20, 300)])
def test_latent_attention(dtype, rank, rot, window):
    g = torch.Generator().manual_seed(rank)
    nh, bs, nb = 3, 8, 80
    cache = torch.randn(nb, bs, rank + rot, generator=g).to(dtype)
    # portions: (context incl. portion, portion length)
    seqs = [(5, 5), (300, 17), (41, 2), (290, 290 if window == 0 else 9)]
    perm = torch.randperm(nb, generator=g).tolist()
    tables = torch.zeros(len(seqs), nb, dtype=torch.int32)
    k = 0
    for i, (ctx, _) in enumerate(seqs):
        n = (ctx + bs - 1) // bs
        tables[i, :n] = torch.tensor(perm[k:k + n] if k + n <= nb else perm[:n])
        k = (k + n) % nb if k + n <= nb else n
    qsl = torch.tensor([0] + list(torch.tensor([n for _, n in seqs]).cumsum(0)), dtype=torch.int32)
    lens = torch.tensor([c for c, _ in seqs], dtype=torch.int32)
    t = int(qsl[-1])
    scale = 0.3 / (rank + rot) ** 0.5
    q_lat = torch.randn(nh, t, rank, generator=g).to(dtype).transpose(0, 1)  # strided
    q_full = torch.randn(t, nh, 8 + rot, generator=g).to(dtype)
    q_rot = q_full[:, :, 8:]
    sinks = torch.randn(nh, generator=g)
    want = ref.latent_attention(q_lat, q_rot, cache, tables, qsl, lens, scale, window, sinks)
    out = torch.empty(nh, t, rank, dtype=dtype, device="cuda").transpose(0, 1)
    ops.latent_attention_prefill(
        q_lat.cuda(), q_rot.cuda(), cache.cuda(), tables.cuda(), qsl.cuda(), lens.cuda(),
        scale, window, sinks.cuda(), max(n for _, n in seqs), out=out)
    torch.testing.assert_close(out.cpu().float(), want.float(), **_tol(dtype))

    # decode: the last row of every sequence alone
    rows = (qsl[1:] - 1).long()
    out_d = torch.empty(len(seqs), nh, rank, dtype=dtype, device="cuda")
    ops.latent_attention_decode(
        q_lat[rows].cuda(), q_rot[rows].cuda(), cache.cuda(), tables.cuda(), lens.cuda(),
        scale, window, None, out=out_d)
    want_d = ref.latent_attention(
        q_lat[rows], q_rot[rows], cache, tables,
        torch.arange(len(seqs) + 1, dtype=torch.int32), lens, scale, window, None)
    torch.testing.assert_close(out_d.cpu().float(), want_d.float(), **_tol(dtype))


@pytest.mark.parametrize("rank,rot,heads,window,bs", [
    (32, 32, 3, 5, 4), (64, 32, 4, 40, 16), (96, 32, 6, 21, 8), (96, 64, 16, 0, 16),
    (128, 64, 70, 33, 8), (256, 32, 16, 100, 16), (512, 64, 16, 64, 16), (512, 32, 5, 0, 32),
])
def test_latent_attention_mfma(rank, rot, heads, window, bs):
    """The bf16 MFMA kernel (prompt portions and single queries) against the
    f32 reference and against the general kernel."""
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(rank + heads)
    nb = 40 * 16 // bs + 8
    cache = torch.randn(nb, bs, rank + rot, generator=g).to(dtype)
    seqs = [(3, 3), (200, 70), (65, 1), (33, 2), (130, 130 if window == 0 else 45)]
    tables = torch.zeros(len(seqs), nb, dtype=torch.int32)
    for i, (ctx, _) in enumerate(seqs):
        n = (ctx + bs - 1) // bs
        tables[i, :n] = torch.randperm(nb, generator=g)[:n].to(torch.int32)
    qsl = torch.tensor([0] + list(torch.tensor([n for _, n in seqs]).cumsum(0)), dtype=torch.int32)
    lens = torch.tensor([c for c, _ in seqs], dtype=torch.int32)
    t = int(qsl[-1])
    scale = 2.0 / (rank + rot) ** 0.5
    q_lat = torch.randn(heads, t, rank, generator=g).to(dtype).transpose(0, 1)
    q_full = torch.randn(t, heads, 8 + rot, generator=g).to(dtype)
    q_rot = q_full[:, :, 8:]
    sinks = torch.randn(heads, generator=g)
    want = ref.latent_attention(q_lat.float(), q_rot.float(), cache.float(), tables, qsl, lens,
                                scale, window, sinks)
    args = (q_lat.cuda(), q_rot.cuda(), cache.cuda(), tables.cuda(), qsl.cuda(), lens.cuda(),
            scale, window, sinks.cuda(), max(n for _, n in seqs))
    out = torch.full((heads, t, rank), float("nan"), dtype=dtype, device="cuda").transpose(0, 1)
    ops.latent_attention_prefill(*args, out=out)
    gen = torch.empty(heads, t, rank, dtype=dtype, device="cuda").transpose(0, 1)
    ops.latent_attention_prefill(*args, out=gen, general=True)
    torch.testing.assert_close(out.cpu().float(), want, atol=3e-2, rtol=3e-2)
    torch.testing.assert_close(out.cpu().float(), gen.cpu().float(), atol=3e-2, rtol=3e-2)

    rows = (qsl[1:] - 1).long()
    out_d = torch.full((len(seqs), heads, rank), float("nan"), dtype=dtype, device="cuda")
    ops.latent_attention_decode(
        q_lat[rows].contiguous().cuda(), q_rot[rows].cuda(), cache.cuda(), tables.cuda(),
        lens.cuda(), scale, window, sinks.cuda(), out=out_d)
    want_d = ref.latent_attention(
        q_lat[rows].float(), q_rot[rows].float(), cache.float(), tables,
        torch.arange(len(seqs) + 1, dtype=torch.int32), lens, scale, window, sinks)
    torch.testing.assert_close(out_d.cpu().float(), want_d, atol=3e-2, rtol=3e-2)


@pytest.mark.parametrize("window", [0, 100, 700])
def test_latent_decode_key_slices_and_padding_rows(window):
    """Single-query steps slice long key ranges over workgroups and merge;
    rows of length zero (padding of a captured bucket) come out as zeros."""
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(window)
    rank, rot, heads, bs = 128, 64, 8, 16
    lens = torch.tensor([900, 0, 1, 33, 0, 640], dtype=torch.int32)
    nb = 64
    cache = torch.randn(nb * len(lens), bs, rank + rot, generator=g).to(dtype)
    tables = torch.arange(nb * len(lens), dtype=torch.int32).view(len(lens), nb)
    q_lat = torch.randn(len(lens), heads, rank, generator=g).to(dtype)
    q_rot = torch.randn(len(lens), heads, rot, generator=g).to(dtype)
    sinks = torch.randn(heads, generator=g)
    out = torch.full((len(lens), heads, rank), float("nan"), dtype=dtype, device="cuda")
    ops.latent_attention_decode(q_lat.cuda(), q_rot.cuda(), cache.cuda(), tables.cuda(),
                                lens.cuda(), 0.1, window, sinks.cuda(), out=out)
    want = ref.latent_attention(
        q_lat.float(), q_rot.float(), cache.float(), tables,
        torch.arange(len(lens) + 1, dtype=torch.int32), lens, 0.1, window, sinks)
    torch.testing.assert_close(out.cpu().float(), want, atol=3e-2, rtol=3e-2)
    assert float(out[1].abs().max()) == 0.0 and float(out[4].abs().max()) == 0.0
