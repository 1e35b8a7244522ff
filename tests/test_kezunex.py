"""Kezunex through the engine against the plain oracle (tests/kezunex_oracle.py).

Every test builds its own small configuration with random weights.  CPU runs
use the reference ops, GPU runs (marked) the HIP kernels; both go through the
engine's request, cache-block and state-slot bookkeeping.
"""

from __future__ import annotations

import pytest
import torch

import kezunex_oracle as oracle
from vllm_tgis_adapter_amd import ops
from vllm_tgis_adapter_amd.engine import EngineConfig, LLMEngine, ModelConfig, SamplingParams
from vllm_tgis_adapter_amd.engine.config import CacheConfig, SchedulerConfig
from vllm_tgis_adapter_amd.models import blocks

CPU = pytest.param("cpu", id="cpu")
GPU = pytest.param("cuda", id="gpu", marks=pytest.mark.gpu)
DEVICES = [CPU, GPU]
F64 = torch.float64


def _engine(path, device, dtype="float32", blocks=64, slots=4, block_size=4, eager=True):
    mc = ModelConfig.from_model_arg(path, dtype=dtype)
    return LLMEngine(EngineConfig(
        model_config=mc,
        cache_config=CacheConfig(block_size=block_size, num_gpu_blocks=blocks),
        scheduler_config=SchedulerConfig(max_num_seqs=slots, max_num_batched_tokens=1 << 20),
        device=device, enforce_eager=eager))


def _tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def _feed(engine, rid, tokens, cuts):
    """Feed one request in portions; logits of every position."""
    rows, at = [], 0
    for n in cuts:
        last = at + n == len(tokens)
        rows.append(engine.replay_step([(rid, tokens[at:at + n], list(range(n)))],
                                       [rid] if last else []))
        at += n
    assert at == len(tokens)
    return torch.cat(rows).double().cpu()


def _close(got, want, dtype="float32", what=""):
    # bf16: a few percent of the largest logit
    tol = 3e-4 if dtype == "float32" else 0.04 * max(1.0, float(want.abs().max()))
    err = float((got - want).abs().max())
    assert err < tol, f"{what} {err}"


@pytest.fixture
def model(tmp_path):
    cfg = oracle.make_config()
    w = oracle.make_weights(cfg, seed=1)
    return cfg, w, oracle.save_model(tmp_path / "m", cfg, w)


# -- each mechanism alone, as the framework's block, in portions --------------


class _Meta:
    """What a mixer reads of the step metadata, for one sequence fed in
    portions through block tables of its own."""

    def __init__(self, dev, bs, nblocks, slot):
        self.dev, self.bs, self.slot = dev, bs, slot
        self.blocks = list(range(nblocks - 1, -1, -1))   # scattered on purpose
        self.at = 0

    def step(self, n):
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=self.dev)
        s, e = self.at, self.at + n
        self.at = e
        nb = (e + self.bs - 1) // self.bs
        m = type("M", (), {})()
        m.slot_mapping = torch.tensor(
            [self.blocks[p // self.bs] * self.bs + p % self.bs for p in range(s, e)],
            dtype=torch.long, device=self.dev)
        m.seq_start_loc, m.seq_lens, m.state_slots = i32([0, n]), i32([e]), i32([self.slot])
        table = i32([self.blocks[:nb]])
        empty_t, empty = torch.empty((0, 0), dtype=torch.int32, device=self.dev), i32([])
        if n > 1:
            m.num_prefill_tokens, m.num_decode_seqs = n, 0
            m.prefill_block_tables, m.prefill_query_start_loc = table, i32([0, n])
            m.prefill_seq_lens, m.max_prefill_query_len = i32([e]), n
            m.decode_block_tables, m.decode_seq_lens = empty_t, empty
        else:
            m.num_prefill_tokens, m.num_decode_seqs = 0, 1
            m.prefill_block_tables, m.prefill_query_start_loc = empty_t, i32([0])
            m.prefill_seq_lens, m.max_prefill_query_len = empty, 0
            m.decode_block_tables, m.decode_seq_lens = table, i32([e])
        return m, torch.arange(s, e, device=self.dev)


def _run_mixer(mod, h, dev, cuts, bs=4):
    """The block's forward over h [T, W] fed in portions; caches start dirty."""
    mod = mod.to(dev)
    nblocks = (h.shape[0] + bs - 1) // bs + 2
    cache = []
    for kind, shape, dt in mod.cache_shapes(bs):
        lead = nblocks if kind == "paged" else 3
        cache.append(torch.full((lead,) + tuple(shape), 3.0, dtype=dt, device=dev))
    meta = _Meta(dev, bs, nblocks, slot=2)
    outs, at = [], 0
    for n in cuts:
        m, pos = meta.step(n)
        y = mod(h[at:at + n].to(dev), pos, tuple(cache), m)
        if isinstance(y, tuple):
            y = mod.left_scale * y[0].double() + mod.right_scale * y[1].double()
        outs.append(y.double().cpu())
        at += n
    return torch.cat(outs)


CUTS = [[19], [1] * 19, [2] * 9 + [1], [7, 1, 1, 3, 2, 5], [17, 2]]


def _sub(w, prefix):
    return {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("spec", [oracle.attn_spec(), oracle.attn_spec(3, 1, 5, 9, 0.4, 0.0, 0),
                                  oracle.attn_spec(2, 2, 16, 16, 0.2, 1.0, 1)])
def test_attention_alone(device, spec):
    cfg = oracle.make_config(layers=[oracle.layer("parallel", left=spec)], loop=None)
    w = oracle.make_weights(cfg, seed=3)
    g = torch.Generator().manual_seed(4)
    h = torch.randn(19, cfg["width"], generator=g)
    want = oracle.softmax_attention(h.double(), w, "l0.mix.left.", spec, 1e-5)
    qt = spec.get("q_temp") or {}
    mod = blocks.QKNormAttention(cfg["width"], heads=spec["heads"], kv_heads=spec["kv_heads"],
                                 dim=spec["dim"], vdim=spec["vdim"], scale=spec["scale"], eps=1e-5,
                                 temp_coef=qt.get("coef", 0.0), temp_every=qt.get("every", 0),
                                 dtype=torch.float32)
    mod.load(_sub(w, "l0.mix.left."))
    for cuts in CUTS:
        _close(_run_mixer(mod, h, device, cuts), want, what=str(cuts))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("spec", [oracle.ssd_spec(), oracle.ssd_spec(1, 16, 16, 1, 1, 1),
                                  oracle.ssd_spec(6, 3, 20, 3, 4, 6)])
def test_ssd_alone(device, spec):
    cfg = oracle.make_config(layers=[oracle.layer("parallel", right=spec)], loop=None)
    w = oracle.make_weights(cfg, seed=5)
    g = torch.Generator().manual_seed(6)
    h = torch.randn(19, cfg["width"], generator=g)
    want = oracle.ssd(h.double(), w, "l0.mix.right.", spec, 1e-5)
    mod = blocks.SSDMixer(cfg["width"], heads=spec["heads"], vdim=spec["vdim"], state=spec["state"],
                          groups=spec["groups"], taps=spec["conv"], norm_groups=spec["norm_groups"],
                          eps=1e-5, dtype=torch.float32)
    mod.load(_sub(w, "l0.mix.right."))
    for cuts in CUTS:
        _close(_run_mixer(mod, h, device, cuts), want, what=str(cuts))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kw", [dict(), dict(width=16, blocks=1, conv=1), dict(width=30, blocks=5, conv=2)])
def test_rglru_alone(device, kw):
    cfg = oracle.make_config(layers=[oracle.layer("rglru", **kw)], loop=None)
    m = cfg["layers"][0]["mixer"]
    w = oracle.make_weights(cfg, seed=7)
    g = torch.Generator().manual_seed(8)
    h = torch.randn(19, cfg["width"], generator=g)
    want = oracle.rglru(h.double(), w, "l0.mix.", m, 1e-5)
    mod = blocks.RGLRUMixer(cfg["width"], rec_width=m["width"], blocks=m["blocks"], taps=m["conv"],
                            dtype=torch.float32)
    mod.load(_sub(w, "l0.mix."))
    for cuts in CUTS:
        _close(_run_mixer(mod, h, device, cuts), want, what=str(cuts))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kw", [dict(), dict(heads=1, dim=16, vdim=16, gate_cap=3.0),
                                dict(heads=2, dim=20, vdim=5, gate_cap=30.0)])
def test_mlstm_alone(device, kw):
    cfg = oracle.make_config(layers=[oracle.layer("mlstm", **kw)], loop=None)
    m = cfg["layers"][0]["mixer"]
    w = oracle.make_weights(cfg, seed=9)
    g = torch.Generator().manual_seed(10)
    h = torch.randn(19, cfg["width"], generator=g) * 2
    want = oracle.mlstm(h.double(), w, "l0.mix.", m, 1e-5)
    mod = blocks.MLSTMMixer(cfg["width"], heads=m["heads"], dim=m["dim"], vdim=m["vdim"],
                            gate_cap=m["gate_cap"], eps=1e-5, dtype=torch.float32)
    mod.load(_sub(w, "l0.mix."))
    for cuts in CUTS:
        _close(_run_mixer(mod, h, device, cuts), want, what=str(cuts))


@pytest.mark.parametrize("device", DEVICES)
def test_norms_and_feed_forward_alone(device):
    g = torch.Generator().manual_seed(11)
    n, width, ff = 9, 40, 24
    dev = torch.device(device)
    x = torch.randn(n, width, generator=g) * 2 + 0.5
    wn = torch.randn(width, generator=g)
    got = ops.layer_norm_stream(x.to(dev), wn.to(dev), 1e-5, torch.float32).cpu().double()
    _close(got, oracle.layer_norm(x.double(), wn.double(), 1e-5))
    wts = {"l0.mlp.gate": torch.randn(ff, width, generator=g) * 0.2,
           "l0.mlp.up": torch.randn(ff, width, generator=g) * 0.2,
           "l0.mlp.down": torch.randn(width, ff, generator=g) * 0.2}
    mlp = blocks.GatedDenseMLP(width, ff, torch.float32)
    mlp.load(wts["l0.mlp.gate"], wts["l0.mlp.up"], wts["l0.mlp.down"])
    got = mlp.to(dev)(x.to(dev)).cpu().double()
    _close(got, oracle.dense_ff(x.double(), wts, "l0.mlp."))


# -- a key that must be seen --------------------------------------------------


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("ctx,spike_at", [(9, 0), (300, 1), (300, 255), (300, 256), (517, 3), (16, 15)])
def test_far_keys_and_page_borders(device, ctx, spike_at):
    """One key among hundreds carries almost all the weight of the last
    query: dropping it (a page or tile border, the first token) shows."""
    spec = oracle.attn_spec(2, 1, 8, 4, 1.0, 0.0, 0)
    cfg = oracle.make_config(layers=[oracle.layer("parallel", left=spec)], loop=None, width=16)
    w = oracle.make_weights(cfg, seed=12)
    eye = torch.zeros(8, 16)
    eye[:, :8] = torch.eye(8)
    w["l0.mix.left.q"] = torch.cat([eye, eye]).to(torch.bfloat16)
    w["l0.mix.left.k"] = eye.to(torch.bfloat16)
    w["l0.mix.left.q.norm"] = torch.full((8,), 3.0).to(torch.bfloat16)
    w["l0.mix.left.k.norm"] = torch.full((8,), 3.0).to(torch.bfloat16)
    g = torch.Generator().manual_seed(13)
    h = torch.randn(ctx, 16, generator=g)
    h[:, :8] = torch.randn(ctx, 8, generator=g) * 0.05 + torch.tensor([0, 1.0, 0, 0, 0, 0, 0, 0])
    h[spike_at, :8] = torch.tensor([2.0, 0, 0, 0, 0, 0, 0, 0])
    h[-1, :8] = torch.tensor([2.0, 0, 0, 0, 0, 0, 0, 0])
    want = oracle.softmax_attention(h.double(), w, "l0.mix.left.", spec, 1e-5)
    mod = blocks.QKNormAttention(16, heads=2, kv_heads=1, dim=8, vdim=4, scale=1.0, eps=1e-5,
                                 dtype=torch.float32)
    mod.load(_sub(w, "l0.mix.left."))
    for cuts in ([ctx], [ctx - 1, 1], [max(ctx - 5, 1)] + [1] * min(5, ctx - 1)):
        _close(_run_mixer(mod, h, device, cuts, bs=16)[-1], want[-1], what=str(cuts))


# -- the whole model ---------------------------------------------------------


@pytest.mark.parametrize("device", DEVICES)
def test_whole_prompt_and_layers_match_oracle(model, device):
    cfg, w, path = model
    toks = _tokens(21, cfg["vocab"], 3)
    e = _engine(path, device)
    probe = []
    e.worker.model.stream_probe = probe
    got = _feed(e, "a", toks, [21])
    want, streams = oracle.forward(cfg, w, toks, return_layers=True)
    assert len(probe) == streams.shape[0] == 6      # 1 + 2 * 2 + 1 layer runs
    for r, x in enumerate(probe):
        _close(x.double().cpu(), streams[r], what=f"layer run {r}")
    _close(got, want)


@pytest.mark.parametrize("device", DEVICES)
def test_decode_and_portions_equal_whole(model, device):
    cfg, w, path = model
    n = 31
    toks = _tokens(n, cfg["vocab"], 6)
    want = oracle.forward(cfg, w, toks)
    e = _engine(path, device)
    for cuts in ([1] * n, [2] * 15 + [1], [7, 2, 3, 11, 2, 2, 4], [20] + [1] * 11, [3, 28]):
        _close(_feed(e, "r", toks, cuts), want, what=str(cuts))


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode(model, device):
    cfg, w, path = model
    n = 90    # the query temperature steps many times, states decay to nothing
    toks = _tokens(n, cfg["vocab"], 7)
    e = _engine(path, device)
    _close(_feed(e, "r", toks, [4] + [1] * (n - 4)), oracle.forward(cfg, w, toks))


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batch_and_reuse_of_blocks_and_slots(model, device):
    """Unequal requests side by side equal each alone; the pool has room for
    only part of them, so blocks and the two state slots are used again."""
    cfg, w, path = model
    vocab = cfg["vocab"]
    reqs = {f"r{k}": _tokens(n, vocab, 20 + k) for k, n in enumerate([23, 9, 1, 14, 30, 2])}
    want = {k: oracle.forward(cfg, w, t) for k, t in reqs.items()}
    e = _engine(path, device, blocks=14, slots=2, block_size=4)
    plans = {
        "r0": [5, 1, 1, 9, 2, 5], "r1": [2, 2, 1, 1, 3], "r2": [1],
        "r3": [14], "r4": [1, 1, 2, 26], "r5": [2],
    }
    for pair in [("r0", "r1"), ("r2", "r3"), ("r4", "r5")]:
        at = {k: 0 for k in pair}
        got = {k: [] for k in pair}
        left = {k: list(plans[k]) for k in pair}
        while any(left.values()):
            entries, done = [], []
            for k in pair:
                if left[k]:
                    c = left[k].pop(0)
                    entries.append((k, reqs[k][at[k]:at[k] + c], list(range(c))))
                    at[k] += c
                    if not left[k]:
                        done.append(k)
            lg = e.replay_step(entries, done).double().cpu()
            o = 0
            for k, t, _ in entries:
                got[k].append(lg[o:o + len(t)])
                o += len(t)
        for k in pair:
            _close(torch.cat(got[k]), want[k], what=k)
    assert e.block_manager.num_free_blocks == 14
    assert e.state_manager.num_free_slots == 2


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("variant", ["no_loop", "loop_all_once", "loop_tail", "ones", "wide"])
def test_other_shapes(tmp_path, device, variant):
    L = oracle.layer
    if variant == "no_loop":
        cfg = oracle.make_config(layers=[L("mlstm", ff=16), L("rglru", ff=16)], loop=None)
    elif variant == "loop_all_once":
        cfg = oracle.make_config(layers=[L("parallel"), L("rglru")], loop=(0, 2, 1))
    elif variant == "loop_tail":
        cfg = oracle.make_config(
            layers=[L("mlstm"), L("parallel", ff=8), L("rglru", width=8, blocks=2, conv=3)],
            loop=(2, 3, 4))
    elif variant == "ones":
        cfg = oracle.make_config(
            vocab=37, width=8, embed_scale=1.0,
            layers=[L("parallel", ff=8, left=oracle.attn_spec(1, 1, 1, 1, 1.0, 1.0, 1),
                      right=oracle.ssd_spec(1, 1, 1, 1, 1, 1), left_scale=1.0, right_scale=1.0),
                    L("mlstm", heads=1, dim=1, vdim=1, gate_cap=1.0),
                    L("rglru", width=1, blocks=1, conv=1)],
            loop=(0, 1, 3))
    else:
        cfg = oracle.make_config(
            width=136, vocab=300,
            layers=[L("parallel", ff=200, left=oracle.attn_spec(6, 2, 24, 40, 0.2, 0.5, 16),
                      right=oracle.ssd_spec(4, 40, 48, 2, 4, 2)),
                    L("mlstm", heads=2, dim=48, vdim=72),
                    L("rglru", width=272, blocks=4, conv=4, ff=0)],
            loop=(0, 2, 2))
    w = oracle.make_weights(cfg, seed=11)
    path = oracle.save_model(tmp_path / variant, cfg, w)
    n = 38
    toks = _tokens(n, cfg["vocab"], 12)
    want = oracle.forward(cfg, w, toks)
    e = _engine(path, device, block_size=8, blocks=24)
    _close(_feed(e, "a", toks, [n]), want)
    _close(_feed(e, "b", toks, [5, 2, 1, 1, 16, 2] + [1] * 11), want)


@pytest.mark.parametrize("device", DEVICES)
def test_bf16_stays_near_oracle(model, device):
    cfg, w, path = model
    toks = _tokens(33, cfg["vocab"], 9)
    want = oracle.forward(cfg, w, toks)
    e = _engine(path, device, dtype="bfloat16")
    a = _feed(e, "a", toks, [33])
    b = _feed(e, "b", toks, [6, 2, 9] + [1] * 16)
    _close(a, want, "bfloat16")
    _close(b, want, "bfloat16")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("attn", [(4, 2, 64), (6, 2, 128), (8, 1, 64), (3, 3, 128)])
def test_matrix_core_shapes(tmp_path, device, dtype, attn):
    """Head sizes the MFMA attention kernels take (bf16, key size = value size
    of 64 or 128, one to eight query heads per key head) and vector-width
    state sizes."""
    L = oracle.layer
    nh, ng, hd = attn
    cfg = oracle.make_config(
        width=128, vocab=211,
        layers=[L("parallel", ff=128, left=oracle.attn_spec(nh, ng, hd, hd, 0.1, 0.3, 32),
                  right=oracle.ssd_spec(4, 32, 64, 1, 4, 1)),
                L("mlstm", heads=2, dim=32, vdim=64)],
        loop=(0, 1, 2))
    w = oracle.make_weights(cfg, seed=21)
    path = oracle.save_model(tmp_path / "mc", cfg, w)
    toks = _tokens(150, cfg["vocab"], 22)
    want = oracle.forward(cfg, w, toks)
    e = _engine(path, device, dtype=dtype, block_size=16, blocks=24)
    _close(_feed(e, "a", toks, [150]), want, dtype)
    _close(_feed(e, "b", toks, [100, 17, 2] + [1] * 31), want, dtype)


@pytest.mark.gpu
def test_captured_decode_steps_match_eager(model):
    """Decode-only steps replay captured graphs; replays interleaved with eager
    prompt portions and with slot / block reuse equal the eager engine."""
    cfg, w, path = model
    toks = {k: _tokens(n, cfg["vocab"], 50 + i) for i, (k, n) in
            enumerate([("a", 25), ("b", 17), ("c", 22)])}
    outs = []
    for eager in (True, False):
        e = _engine(path, "cuda", blocks=24, slots=2, eager=eager)
        if not eager:
            assert e.worker.graph_runner is not None and e.worker.graph_runner.graphs
        got = {k: [] for k in toks}
        at = {k: 0 for k in toks}

        def step(parts, done=()):
            entries = [(k, toks[k][at[k]:at[k] + n], list(range(n))) for k, n in parts]
            lg = e.replay_step(entries, list(done)).double().cpu()
            o = 0
            for k, n in parts:
                got[k].append(lg[o:o + n])
                at[k] += n
                o += n

        step([("a", 9), ("b", 5)])
        for _ in range(6):
            step([("a", 1), ("b", 1)])             # graph bucket 2
        step([("a", 1), ("b", 6)], done=["b"])     # eager, mixed
        for _ in range(4):
            step([("a", 1)])                       # graph bucket 1
        step([("c", 20), ("a", 1)])                # c takes b's slot and blocks
        for _ in range(2):
            step([("a", 1), ("c", 1)])
        step([("a", 2)], done=["a"])
        outs.append({k: torch.cat(v) for k, v in got.items()})
    for k in ("a", "b"):
        want = oracle.forward(cfg, w, toks[k])
        _close(outs[1][k], want)
        _close(outs[0][k], outs[1][k])
    _close(outs[1]["c"], oracle.forward(cfg, w, toks["c"])[:22])


@pytest.mark.gpu
def test_captured_decode_with_padding_rows(model):
    """Three sequences decode together in the four-row captured bucket: the
    padding row (slot -1, length 0) must leave every state slot alone."""
    cfg, w, path = model
    toks = {k: _tokens(n, cfg["vocab"], 70 + i) for i, (k, n) in
            enumerate([("a", 14), ("b", 11), ("c", 12), ("d", 9)])}
    e = _engine(path, "cuda", blocks=32, slots=4, eager=False)
    assert 4 in e.worker.graph_runner.graphs
    got = {k: [] for k in toks}
    at = {k: 0 for k in toks}

    def step(parts, done=()):
        entries = [(k, toks[k][at[k]:at[k] + n], list(range(n))) for k, n in parts]
        lg = e.replay_step(entries, list(done)).double().cpu()
        o = 0
        for k, n in parts:
            got[k].append(lg[o:o + n])
            at[k] += n
            o += n

    step([("a", 5), ("b", 3), ("c", 4), ("d", 9)], done=["d"])   # d's slot is dirty now
    for _ in range(6):
        step([("a", 1), ("b", 1), ("c", 1)])                     # bucket 4, one padding row
    step([("a", 3), ("b", 2), ("c", 2)], done=["a", "b", "c"])
    for k in ("a", "b", "c", "d"):
        _close(torch.cat(got[k]), oracle.forward(cfg, w, toks[k]), what=k)


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_matches_oracle(model, device):
    cfg, w, path = model
    e = _engine(path, device, blocks=40, slots=3, eager=False)
    prompts = {"a": _tokens(11, cfg["vocab"], 31), "b": _tokens(3, cfg["vocab"], 32),
               "c": _tokens(18, cfg["vocab"], 33), "d": _tokens(6, cfg["vocab"], 34)}
    new = 7
    for rid, p in prompts.items():    # four requests for three slots: one waits
        e.add_request(rid, None, p, SamplingParams(temperature=0.0, max_tokens=new))
    done = {}
    steps = 0
    while e.has_unfinished():
        for o in e.step():
            if o.finished:
                done[o.request_id] = list(o.outputs[0].token_ids)
        steps += 1
        assert steps < 200
    for rid, p in prompts.items():
        seq = list(p)
        for _ in range(new):
            seq.append(int(oracle.forward(cfg, w, seq)[-1].argmax()))
            if seq[-1] == e.eos_token_id:
                break
        assert done[rid] == seq[len(p):], rid
    assert e.state_manager.num_free_slots == 3


def test_served_from_command_line_flags(tmp_path):
    """A Kezunex directory given as --model goes through the server's flag
    parsing into the async engine and streams greedy tokens equal to the
    oracle's, concurrent requests included."""
    import asyncio

    from vllm_tgis_adapter_amd.__main__ import parse_args
    from vllm_tgis_adapter_amd.engine.async_engine import AsyncLLMEngine
    from vllm_tgis_adapter_amd.tgis_utils.args import engine_config_from_args

    cfg = oracle.make_config(vocab=300)    # room for the byte-level test tokenizer
    w = oracle.make_weights(cfg, seed=5)
    path = oracle.save_model(tmp_path / "served", cfg, w)
    args = parse_args(["--model", path, "--dtype", "float32", "--max-num-seqs", "2",
                       "--num-gpu-blocks", "64", "--block-size", "8", "--device", "cpu"])
    engine = AsyncLLMEngine(engine_config_from_args(args))
    prompts = {"x": _tokens(12, 300, 61), "y": _tokens(5, 300, 62), "z": _tokens(9, 300, 63)}

    async def one(rid):
        last = None
        async for out in engine.generate(
                {"prompt_token_ids": prompts[rid]},
                SamplingParams(temperature=0.0, max_tokens=5), request_id=rid):
            last = out
        return rid, list(last.outputs[0].token_ids)

    async def main():
        return dict(await asyncio.gather(*[one(r) for r in prompts]))

    try:
        got = asyncio.run(main())
    finally:
        engine.shutdown()
    eos = engine.engine.eos_token_id
    for rid, p in prompts.items():
        seq = list(p)
        for _ in range(5):
            seq.append(int(oracle.forward(cfg, w, seq)[-1].argmax()))
            if seq[-1] == eos:
                break
        assert got[rid] == seq[len(p):], rid


def test_refuses_what_it_cannot_run(tmp_path):
    cfg = oracle.make_config(layers=[oracle.layer("rglru")], loop=None)
    cfg["layers"][0]["type"] = "retention"
    path = oracle.save_model(tmp_path / "bad", cfg, {})
    with pytest.raises(ValueError):
        _engine(path, "cpu")


def test_trace_replay_program(tmp_path):
    """bin/trace_run as a user runs it: JSON steps on stdin, 'done <step>' lines
    on stdout, little-endian f32 logits files for the steps that want some;
    two requests in portions side by side, one leaving early."""
    import json
    import os
    import subprocess
    import sys

    import numpy as np

    cfg = oracle.make_config()
    w = oracle.make_weights(cfg, seed=8)
    path = oracle.save_model(tmp_path / "m", cfg, w)
    a, b = _tokens(70, cfg["vocab"], 41), _tokens(9, cfg["vocab"], 42)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:66], "want": [0, 65]}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b[:2], "want": []}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": a[66:67], "want": [0]},
                                {"id": "b", "tokens": b[2:], "want": [6, 2]}], "end": ["b"]},
        {"step": 3, "entries": [{"id": "a", "tokens": a[67:], "want": [2, 0]}], "end": ["a"]},
    ]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    proc = subprocess.run(
        [sys.executable, os.path.join(root, "bin", "trace_run"), "--model", path, "--dtype",
         "float32", "--out", str(out), "--max-tokens", "192", "--device", "cpu"],
        input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True,
        timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    done = [ln for ln in proc.stdout.splitlines() if ln.startswith("done ")]
    assert done == ["done 0", "done 1", "done 2", "done 3"]
    assert not (out / "1.f32").exists()
    wa, wb = oracle.forward(cfg, w, a), oracle.forward(cfg, w, b)
    want = {0: torch.stack([wa[0], wa[65]]), 2: torch.stack([wa[66], wb[8], wb[4]]),
            3: torch.stack([wa[69], wa[67]])}
    for n, rows in want.items():
        got = np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, cfg["vocab"])
        _close(torch.from_numpy(got).double(), rows, what=f"step {n}")
