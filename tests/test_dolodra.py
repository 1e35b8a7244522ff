"""Dolodra through the engine against the plain oracle (tests/dolodra_oracle.py).

Every test builds its own small configuration with random weights.  CPU runs
use the reference ops, GPU runs (marked) the HIP kernels; both go through the
engine's request, cache-block and state-slot bookkeeping.
"""

from __future__ import annotations

import math

import pytest
import torch

import dolodra_oracle as oracle
from vllm_tgis_adapter_amd.engine import EngineConfig, LLMEngine, ModelConfig, SamplingParams
from vllm_tgis_adapter_amd.engine.config import CacheConfig, SchedulerConfig

CPU = pytest.param("cpu", id="cpu")
GPU = pytest.param("cuda", id="gpu", marks=pytest.mark.gpu)
DEVICES = [CPU, GPU]


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
    for k, n in enumerate(cuts):
        last = at + n == len(tokens)
        rows.append(engine.replay_step([(rid, tokens[at:at + n], list(range(n)))],
                                       [rid] if last else []))
        at += n
    assert at == len(tokens)
    return torch.cat(rows).double().cpu()


def _close(got, want, dtype="float32"):
    tol = 2e-4 if dtype == "float32" else 0.12
    err = float((got - want).abs().max())
    assert err < tol, err


@pytest.fixture
def model(tmp_path):
    cfg = oracle.make_config()
    w = oracle.make_weights(cfg, seed=1)
    return cfg, w, oracle.save_model(tmp_path / "m", cfg, w)


# -- each mechanism alone ---------------------------------------------------


@pytest.mark.parametrize("device", DEVICES)
def test_mechanisms_alone(device):
    from vllm_tgis_adapter_amd import ops

    g = torch.Generator().manual_seed(5)
    n, width = 11, 40
    x = torch.randn(n, width, generator=g)
    w = torch.randn(width, generator=g) * 0.3
    dev = torch.device(device)
    got = ops.rms_norm_stream(x.to(dev), w.to(dev), 1e-5, 1.0, torch.float32).cpu()
    _close(got.double(), oracle.norm_around_zero(x.double(), w.double(), 1e-5))

    got = ops.gelu_tanh(x.to(dev)).cpu()
    _close(got.double(), oracle.gelu_tanh(x.double()))

    got = ops.softcap((x * 9).to(dev), 7.0).cpu()
    _close(got.double(), oracle.softcap(x.double() * 9, 7.0))

    # side input: gate, slice of the side embedding, projection, own norm
    sd = 5
    e = torch.randn(n, 3 * sd, generator=g)
    wg, wp = torch.randn(sd, width, generator=g) * 0.2, torch.randn(width, sd, generator=g)
    wn = torch.randn(width, generator=g)
    xs = x.clone().to(dev)
    gg = ops.gelu_tanh(torch.nn.functional.linear(xs, wg.to(dev)), mul=e.to(dev)[:, sd:2 * sd])
    ops.stream_add_rms_norm(xs, torch.nn.functional.linear(gg, wp.to(dev)), wn.to(dev), 1e-5, 0.6)
    _close(xs.cpu().double(), oracle.token_side(
        x.double(), e.double()[:, sd:2 * sd], wg.double(), wp.double(), wn.double(), 1e-5, 0.6))

    # rotation at large positions, on a slice of each head
    q = torch.randn(n, 2, 14, generator=g)
    pos = torch.tensor([0, 1, 2, 3, 100, 1000, 4095, 4096, 20000, 7, 8])
    inv = torch.tensor([777.0 ** (-2.0 * i / 8) for i in range(4)], dtype=torch.float64).float()
    qd = q.clone().to(dev)
    ops.rope_partial(qd, pos.to(dev), inv.to(dev), 6, 8)
    want = q.double().clone()
    for t in range(n):
        want[t, :, 6:] = oracle.rotate_half(q[t, :, 6:].double(), int(pos[t]), 777.0, 8)
    _close(qd.cpu().double(), want, "float32")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("taps", [1, 2, 4])
def test_short_conv_in_portions(device, taps):
    from vllm_tgis_adapter_amd import ops

    g = torch.Generator().manual_seed(taps)
    n, width = 17, 24
    h = torch.randn(n, width, generator=g)
    w = torch.randn(width, taps, generator=g)
    want = oracle.short_conv(h.double(), w.double())
    dev = torch.device(device)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    for cuts in ([17], [1] * 17, [2, 1, 5, 2, 7], [3, 14]):
        state = torch.full((3, taps - 1, width), 9.0, device=dev)   # a used slot
        outs, at = [], 0
        for c in cuts:
            outs.append(ops.causal_conv_state(
                h[at:at + c].to(dev), w.to(dev), state, i32([0, c]), i32([at + c]), i32([1])))
            at += c
        _close(torch.cat(outs).cpu().double(), want)


# -- the whole model ---------------------------------------------------------


@pytest.mark.parametrize("device", DEVICES)
def test_whole_prompt_matches_oracle(model, device):
    cfg, w, path = model
    toks = _tokens(29, cfg["vocab"], 3)
    e = _engine(path, device)
    _close(_feed(e, "a", toks, [29]), oracle.forward(cfg, w, toks))


@pytest.mark.parametrize("device", DEVICES)
def test_layer_by_layer(model, device):
    cfg, w, path = model
    toks = _tokens(13, cfg["vocab"], 4)
    e = _engine(path, device)
    caps = []
    for layer in e.worker.model.layers:
        layer.register_forward_hook(lambda m, i, o: caps.append(o[0].detach().double().cpu().clone()))
    _feed(e, "a", toks, [13])
    want = []
    oracle.forward(cfg, w, toks, want)
    assert len(caps) == len(want)
    for a, b in zip(caps, want):
        _close(a, b)


@pytest.mark.parametrize("device", DEVICES)
def test_decode_and_portions_equal_whole(model, device):
    cfg, w, path = model
    n = 31
    toks = _tokens(n, cfg["vocab"], 6)
    want = oracle.forward(cfg, w, toks)
    e = _engine(path, device)
    for cuts in ([1] * n, [2] * 15 + [1], [7, 2, 3, 11, 2, 2, 4], [20] + [1] * 11, [3, 28]):
        _close(_feed(e, "r", toks, cuts), want)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode_past_every_window(model, device):
    cfg, w, path = model
    n = 40   # windows are 5, 9 and 3: all pass over decoded tokens many times
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
    order = [("r0", "r1"), ("r2", "r3"), ("r4", "r5")]
    for pair in order:
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
            _close(torch.cat(got[k]), want[k])
    assert e.block_manager.num_free_blocks == 14
    assert e.state_manager.num_free_slots == 2


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("variant", ["no_ff_no_side", "taps1_one_head", "plain_causal", "wide"])
def test_other_shapes(tmp_path, device, variant):
    if variant == "no_ff_no_side":
        cfg = oracle.make_config(
            side_dim=0, taps=2, mult=1.0, softcap_=None,
            layers=[dict(heads=2, dim=4, rot_dim=2, vdim=4, kv_rank=6, window=1, ff=0),
                    dict(heads=4, dim=4, rot_dim=2, vdim=2, kv_rank=6, window=2, ff=0, kv_from=0),
                    dict(heads=1, dim=2, rot_dim=2, vdim=3, kv_rank=6, window=50, ff=0, kv_from=0)])
    elif variant == "taps1_one_head":
        cfg = oracle.make_config(
            taps=1, width=20, vocab=31,
            layers=[dict(heads=1, dim=16, rot_dim=16, vdim=16, kv_rank=16, window=4, ff=20)])
    elif variant == "plain_causal":
        cfg = oracle.make_config(
            taps=0, side_dim=3,
            layers=[dict(heads=2, dim=6, rot_dim=6, vdim=5, kv_rank=9, window=0, ff=12),
                    dict(heads=2, dim=6, rot_dim=6, vdim=5, kv_rank=9, window=0, ff=12)])
        for layer in cfg["layers"]:
            del layer["mixer"]["mask"]
    else:
        cfg = oracle.make_config(
            width=136, vocab=300, taps=5, side_dim=10,
            layers=[dict(heads=5, dim=24, rot_dim=16, vdim=40, kv_rank=136, window=33, ff=272),
                    dict(heads=2, dim=40, rot_dim=16, vdim=24, kv_rank=136, window=17, ff=0,
                         kv_from=0)])
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


# -- a key that must / must not be seen ---------------------------------------


def _spiky_case(window, ctx, spike_at, rank=12, rot=4, bs=4):
    """Cache rows with tiny latents except one row whose latent matches the
    query strongly: if that row is seen the output is (almost) its latent."""
    g = torch.Generator().manual_seed(ctx * 131 + spike_at)
    cache = torch.randn(64, bs, rank + rot, generator=g) * 0.01
    q_lat = torch.randn(1, 2, rank, generator=g)
    q_lat = q_lat / q_lat.norm(dim=-1, keepdim=True)
    perm = torch.randperm(64, generator=g)[: (ctx + bs - 1) // bs].to(torch.int32)
    blk, off = int(perm[spike_at // bs]), spike_at % bs
    cache[blk, off, :rank] = q_lat[0, 0] * 30.0
    return cache, q_lat, torch.zeros(1, 2, rot), perm.view(1, -1)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("window,ctx", [(6, 6), (6, 30), (8, 8), (8, 9), (16, 200), (0, 200)])
def test_window_edge_and_far_keys(device, window, ctx):
    """A dominant key just inside the window is seen, just outside it is not,
    at page borders and far back, for a single query and inside a portion."""
    from vllm_tgis_adapter_amd import ops

    dev = torch.device(device)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    qpos = ctx - 1
    inside = qpos - (window - 1) if window else 0       # oldest visible key
    cases = [(inside, True), (qpos, True)]
    if window and inside > 0:
        cases.append((inside - 1, False))
    for spike_at, seen in cases:
        if spike_at < 0:
            continue
        cache, q_lat, q_rot, table = _spiky_case(window, ctx, spike_at)
        out = torch.empty(1, 2, 12, device=dev)
        ops.latent_attention_decode(q_lat.to(dev), q_rot.to(dev), cache.to(dev), table.to(dev),
                                    i32([ctx]), 1.0, window, torch.zeros(2, device=dev), out=out)
        # as the last row of a 3-row portion too
        if ctx >= 3:
            out3 = torch.empty(3, 2, 12, device=dev)
            q3 = torch.cat([torch.zeros(2, 2, 12), q_lat]).to(dev)
            ops.latent_attention_prefill(
                q3, torch.zeros(3, 2, 4, device=dev), cache.to(dev), table.to(dev),
                i32([0, 3]), i32([ctx]), 1.0, window, torch.zeros(2, device=dev), 3, out=out3)
            assert torch.allclose(out3[2], out[0], atol=1e-5)
        strength = float((out[0, 0].cpu() @ q_lat[0, 0]))
        if seen:
            assert strength > 25.0, (spike_at, strength)
        else:
            assert abs(strength) < 1.0, (spike_at, strength)


@pytest.mark.parametrize("device", DEVICES)
def test_sink_takes_weight_without_value(device):
    from vllm_tgis_adapter_amd import ops

    dev = torch.device(device)
    cache = torch.zeros(2, 4, 6, device=dev)
    cache[0, 0, :4] = torch.tensor([1.0, 2.0, 3.0, 4.0])
    q = torch.zeros(1, 2, 4, device=dev)          # all scores 0
    sinks = torch.tensor([0.0, math.log(3.0)], device=dev)
    out = torch.empty(1, 2, 4, device=dev)
    ops.latent_attention_decode(
        q, torch.zeros(1, 2, 2, device=dev), cache, torch.zeros(1, 2, dtype=torch.int32, device=dev),
        torch.tensor([1], dtype=torch.int32, device=dev), 0.5, 4, sinks, out=out)
    # one key with exp(0) against a sink of exp(0) / exp(log 3)
    torch.testing.assert_close(out[0, 0].cpu(), torch.tensor([1.0, 2.0, 3.0, 4.0]) / 2)
    torch.testing.assert_close(out[0, 1].cpu(), torch.tensor([1.0, 2.0, 3.0, 4.0]) / 4)


# -- generation through the engine's own entry point --------------------------


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


# -- tensor parallel (gloo, two ranks on the CPU) ------------------------------


def _tp_worker(rank, world, port, q):
    import os

    try:
        os.environ.update(MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port), RANK=str(rank),
                          WORLD_SIZE=str(world))
        from vllm_tgis_adapter_amd.parallel import init_distributed

        init_distributed(world, rank=rank, device="cpu", backend="gloo")
        from vllm_tgis_adapter_amd.engine.worker import Worker

        mc = ModelConfig.from_model_arg(os.environ["DOLODRA_TP_MODEL"], dtype="float32")
        cfg = EngineConfig(
            model_config=mc,
            cache_config=CacheConfig(block_size=4, num_gpu_blocks=48),
            scheduler_config=SchedulerConfig(max_num_seqs=3, max_num_batched_tokens=1 << 20),
            device="cpu", tensor_parallel_size=world, enforce_eager=True)
        if rank == 0:
            e = LLMEngine(cfg)
            a, b = _tokens(21, mc.vocab_size, 41), _tokens(9, mc.vocab_size, 42)
            got_a = [e.replay_step([("a", a[:8], list(range(8))), ("b", b[:2], [0, 1])])]
            got_a.append(e.replay_step([("a", a[8:9], [0]), ("b", b[2:], list(range(7)))], ["b"]))
            got_a.append(e.replay_step([("a", a[9:], list(range(12)))], ["a"]))
            e.worker.stop_workers()
            rows_a = torch.cat([got_a[0][:8], got_a[1][:1], got_a[2]]).double()
            rows_b = torch.cat([got_a[0][8:], got_a[1][1:]]).double()
            q.put((rank, (rows_a, rows_b)))
        else:
            w = Worker(cfg)
            w.init_kv_cache()
            w.worker_loop()
            q.put((rank, None))
    except Exception:
        import traceback

        q.put((rank, "ERROR " + traceback.format_exc()))
    finally:
        import torch.distributed as dist

        if dist.is_initialized():
            dist.destroy_process_group()


def test_tensor_parallel_two_ranks(tmp_path, monkeypatch):
    """Heads, feed-forward and vocabulary sharded over two ranks (latent rows
    and conv state replicated) reproduce the oracle."""
    from test_distributed import _run_spawn

    cfg = oracle.make_config(layers=[
        dict(heads=4, dim=8, rot_dim=4, vdim=6, kv_rank=20, window=5, ff=40),
        dict(heads=2, dim=6, rot_dim=4, vdim=8, kv_rank=20, window=9, ff=0, kv_from=0),
        dict(heads=2, dim=10, rot_dim=8, vdim=6, kv_rank=12, window=3, ff=24)], vocab=98)
    w = oracle.make_weights(cfg, seed=2)
    path = oracle.save_model(tmp_path / "tp", cfg, w)
    monkeypatch.setenv("DOLODRA_TP_MODEL", path)
    res = _run_spawn(_tp_worker, 2, timeout=300)
    rows_a, rows_b = res[0]
    _close(rows_a, oracle.forward(cfg, w, _tokens(21, 98, 41)))
    _close(rows_b, oracle.forward(cfg, w, _tokens(9, 98, 42)))


# -- the serving entry: command-line flags -> async engine ---------------------


def test_served_from_command_line_flags(tmp_path):
    """A Dolodra directory given as --model goes through the server's flag
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


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_matrix_core_shapes(tmp_path, device, dtype):
    """Latent sizes on the bf16 matrix-core kernel's list (64+32, 32+32 with more
    than 16 heads, 128+64) through the engine: whole, portions, decode, batch."""
    cfg = oracle.make_config(
        width=64, vocab=211, taps=4, side_dim=8,
        layers=[dict(heads=4, dim=16, rot_dim=32, vdim=16, kv_rank=64, window=11, ff=96),
                dict(heads=20, dim=8, rot_dim=32, vdim=8, kv_rank=64, window=37, ff=0, kv_from=0),
                dict(heads=20, dim=8, rot_dim=32, vdim=8, kv_rank=32, window=6, ff=64),
                dict(heads=2, dim=32, rot_dim=64, vdim=32, kv_rank=128, window=70, ff=0)])
    w = oracle.make_weights(cfg, seed=21)
    path = oracle.save_model(tmp_path / "mc", cfg, w)
    a, b = _tokens(45, 211, 71), _tokens(19, 211, 72)
    want_a, want_b = oracle.forward(cfg, w, a), oracle.forward(cfg, w, b)
    e = _engine(path, device, dtype=dtype, block_size=16, blocks=12, slots=2, eager=False)
    _close(_feed(e, "w", a, [45]), want_a, dtype)
    got_a, got_b = [], []
    lg = e.replay_step([("a", a[:30], list(range(30))), ("b", b[:2], [0, 1])])
    got_a.append(lg[:30]); got_b.append(lg[30:])
    for i in range(15):
        lg = e.replay_step([("b", b[2 + i:3 + i], [0]), ("a", a[30 + i:31 + i], [0])],
                           ["a"] if i == 14 else [])
        got_b.append(lg[:1]); got_a.append(lg[1:])
    lg = e.replay_step([("b", b[17:], [0, 1])], ["b"])
    got_b.append(lg)
    _close(torch.cat(got_a).double().cpu(), want_a, dtype)
    _close(torch.cat(got_b).double().cpu(), want_b, dtype)
