"""1P1D through the production KV data plane in ONE process
(disagg/loopback.py): prefill engine -> layer-streamed WRITE -> decode
engine, plus one prefix READ in the reverse direction, over LoopbackLinks.

* CPU: tiny model, tokens equal to the aggregated engine, transferred blocks
  byte-identical, staging reservations all returned.
* GPU (`-m gpu`): Llama-3-8B shape, 8 ISL-3000 prompts + one decode-side
  prefix hit pulled by READ, device staging (no host staging), every
  data-plane call and both engines' steps under
  `torch.cuda.set_sync_debug_mode("error")` -- any host synchronisation
  inside the transfer path raises.
"""
import contextlib
import os

import pytest
import torch

from dynamo_exp_amd.disagg.loopback import Loopback1P1D
from dynamo_exp_amd.engine.engine import EngineConfig, LLMEngine
from dynamo_exp_amd.engine.request import SamplingParams



# Two processes sharing the decode engine's KV cache over dma-buf (kv_transport
# "ipc" across processes): on the GPU boxes in use the import in the peer process
# does not return (seen with the unchanged transfer code of the previous
# release as well), so the children sit until their timeout.  The in-process
# ipc loopback tests above the bench tests cover the one-sided transfer logic.
# DX_RUN_XPROC_IPC=1 runs them.
xproc_ipc = pytest.mark.skipif(os.environ.get("DX_RUN_XPROC_IPC") != "1",
                               reason="cross-process dma-buf import of the KV cache hangs on these GPU boxes "
                                      "(DX_RUN_XPROC_IPC=1 to run)")

def _generate(eng_like, prompts, n, add):
    out = {}
    for rid, p in prompts.items():
        add(rid, p, SamplingParams(max_tokens=n, ignore_eos=True),
            lambda r, t, lp, fin: out.setdefault(r.request_id, []).extend(zip(t, lp)))
    return out


def _agg(eng, prompts, n):
    out = _generate(eng, prompts, n, lambda rid, p, sp, cb: eng.add_request(rid, p, sp, on_output=cb))
    while eng.has_unfinished():
        eng.step()
    return out


def _watch_blocks(lb):
    """Record each remote request's prefill-side and decode-side block ids."""
    seen = {"p": {}, "d": {}}
    on_prefilled = lb.pa.on_prefilled

    def pre(req):
        seen["p"][req.request_id] = (list(req.block_ids), req.remote_meta.get("skip", 0))
        on_prefilled(req)

    lb.p.engine.prefill_done_hook = pre
    finish = lb.d.handlers["kv_finish"]

    def fin(m):
        r = lb.d.engine.scheduler.remote.get(m["rid"])
        if r is not None:
            seen["d"][m["rid"]] = list(r.block_ids)
        finish(m)

    lb.d.handlers["kv_finish"] = fin
    return seen


def _check_bytes(lb, seen, prompts, bs):
    """Full prompt blocks on the decode side == the prefill side's bytes."""
    kp, kd = lb.p.engine.runner.kv_cache, lb.d.engine.runner.kv_cache
    n = 0
    for rid, (pblocks, skip) in seen["p"].items():
        full = len(prompts[rid]) // bs
        dblocks = seen["d"][rid]
        a = kp[:, :, pblocks[skip:full]].view(torch.uint8)
        b = kd[:, :, dblocks[skip:full]].view(torch.uint8)
        assert torch.equal(a, b), rid
        n += full - skip
    return n


def _compare(got, want, tol=0.1):
    """identical, or a near-tie swap (first differing token's logprob within
    tol nats in both runs: different batch shapes pick different GEMM
    kernels, so random-weight logits can tie-break differently)."""
    same = near = 0
    for rid, w in want.items():
        g = got[rid]
        assert len(g) == len(w), rid
        if [t for t, _ in g] == [t for t, _ in w]:
            same += 1
            continue
        j = next(i for i, (a, b) in enumerate(zip(g, w)) if a[0] != b[0])
        assert abs(g[j][1] - w[j][1]) < tol, (rid, j, g[j], w[j])
        near += 1
    return same, near


def test_loopback_1p1d_cpu():
    kw = dict(model="tiny", device="cpu", block_size=16, max_model_len=512, num_gpu_blocks=300, max_num_seqs=8,
              seed=5, use_cuda_graph=False)
    agg = LLMEngine(EngineConfig(**kw))
    prompts = {f"r{i}": [(7 * i + 3 * j) % 500 + 1 for j in range(150 + 9 * i)] for i in range(4)}
    shared = list(range(40, 40 + 64))
    prompts["pre"] = shared + [11] * 90  # its first 4 blocks are cached on the decode side -> READ
    want = _agg(agg, prompts, 8)
    pe = LLMEngine(EngineConfig(chunked_prefill=False, **kw), model=agg.model)
    de = LLMEngine(EngineConfig(**kw), model=agg.model)
    lb = Loopback1P1D(pe, de, pool_cap_bytes=64 << 20, layer_group_count=2)
    seen = _watch_blocks(lb)
    # the decode engine caches the shared prefix (a locally prefilled request)
    _generate(lb, {"warm": shared + [9] * 10}, 2, lambda rid, p, sp, cb: lb.add(rid, p, sp, cb, remote=False))
    lb.run_until_idle(120)
    got = _generate(lb, prompts, 8, lambda rid, p, sp, cb: lb.add(rid, p, sp, cb, remote=True))
    lb.run_until_idle(120)
    assert {k: [t for t, _ in v] for k, v in got.items()} == {k: [t for t, _ in v] for k, v in want.items()}
    assert lb.pa.stats["reads"] == 1 and lb.da.stats["served"] == 1
    assert lb.pa.stats["sent"] == 5 and lb.da.stats["recv"] == 5
    assert _check_bytes(lb, seen, prompts, 16) > 0
    assert lb.pa.pool.reserved == 0 and lb.da.pool.reserved == 0 and not lb.pa.reservations
    assert lb.hub.stats["copies"] > 0


def test_prefill_prefix_hit_releases_read_reservation_cpu():
    """the prefill engine already caches the prefix the
    decode side offered to serve, so the READ is skipped -- its staging
    reservation must still come back (pool.reserved == 0), or admission
    eventually defers forever."""
    kw = dict(model="tiny", device="cpu", block_size=16, max_model_len=512, num_gpu_blocks=300, max_num_seqs=8,
              seed=5, use_cuda_graph=False)
    pe = LLMEngine(EngineConfig(chunked_prefill=False, **kw))
    de = LLMEngine(EngineConfig(**kw), model=pe.model)
    lb = Loopback1P1D(pe, de, pool_cap_bytes=64 << 20)
    shared = list(range(40, 40 + 64))
    for eng in (pe, de):  # both sides cache the prefix
        eng.add_request("w", shared + [9] * 10, SamplingParams(max_tokens=1, ignore_eos=True))
        while eng.has_unfinished():
            eng.step()
    _generate(lb, {"x": shared + [5] * 70}, 4, lambda rid, p, sp, cb: lb.add(rid, p, sp, cb, remote=True))
    lb.run_until_idle(60)
    assert lb.pa.stats["reads"] == 0  # the local cache covered it
    assert lb.pa.pool.reserved == 0 and not lb.pa.reservations
    assert lb.pa.stats["sent"] == 1


@contextlib.contextmanager
def _sync_error():
    torch.cuda.set_sync_debug_mode("error")
    try:
        yield
    finally:
        torch.cuda.set_sync_debug_mode(0)


def _no_sync(fn):
    def wrapped(*a, **kw):
        with _sync_error():
            return fn(*a, **kw)
    return wrapped


@pytest.mark.gpu
def test_loopback_1p1d_device_path_gpu(cuda):
    """the non-host-staged data plane on a GPU, 8 x ISL
    3000 + one prefix READ, Llama-3-8B shape, 4 layer groups; the prefill
    forward (with its layer hooks), serve_read, and every other data-plane
    call run with host syncs turned into errors."""
    kw = dict(model="llama3-8b", device=str(cuda), block_size=64, max_model_len=4096, num_gpu_blocks=640, seed=3)
    agg = LLMEngine(EngineConfig(max_num_seqs=16, use_cuda_graph=False, chunked_prefill=False,
                                 max_num_batched_tokens=16384, **kw))
    pe = LLMEngine(EngineConfig(max_num_seqs=16, use_cuda_graph=False, chunked_prefill=False,
                                max_num_batched_tokens=16384, **kw), model=agg.model)
    de = LLMEngine(EngineConfig(max_num_seqs=16, graph_sizes=(1, 2, 4, 8, 16), max_num_batched_tokens=8192, **kw),
                   model=agg.model)
    agg.warmup()
    pe.warmup()
    de.warmup()
    g = torch.Generator().manual_seed(11)
    prompts = {f"r{i}": torch.randint(1, 120000, (3000,), generator=g).tolist() for i in range(8)}
    shared = torch.randint(1, 120000, (1024,), generator=g).tolist()
    prompts["pre"] = shared + torch.randint(1, 120000, (1976,), generator=g).tolist()
    want = _agg(agg, prompts, 12)

    lb = Loopback1P1D(pe, de, pool_cap_bytes=8 << 30, layer_group_count=4)
    assert len(lb.pa.dp.groups) == 4 and not lb.pa.dp.host_staging
    seen = _watch_blocks(lb)
    _generate(lb, {"warm": shared + [5] * 40}, 2, lambda rid, p, sp, cb: lb.add(rid, p, sp, cb, remote=False))
    lb.run_until_idle(300)
    # from here on: the data plane and both engines' steps must not synchronise the host
    for dp in (lb.pa.dp, lb.da.dp):
        for name in ("on_layer", "begin_send", "end_forward", "post_recv_batch", "finish_recv", "serve_read",
                     "post_read", "finish_read", "poll_sends", "poll_recvs", "poll_served", "poll_reads"):
            setattr(dp, name, _no_sync(getattr(dp, name)))
    pe.model.layer_hook = lb.pa.dp.on_layer
    lb.p.step = _no_sync(lb.p.step)
    lb.d.step = _no_sync(lb.d.step)
    got = _generate(lb, prompts, 12, lambda rid, p, sp, cb: lb.add(rid, p, sp, cb, remote=True))
    lb.run_until_idle(600)
    torch.cuda.synchronize()
    # the transfer itself is checked byte for byte; the token comparison with
    # the aggregated engine (different prefill batch shapes -> different GEMM
    # kernels on random weights) allows near-tie swaps, never a divergence
    nblk = _check_bytes(lb, seen, prompts, 64)
    same, near = _compare(got, want)
    assert same + near == len(prompts) and same >= len(prompts) // 2, (same, near)
    assert lb.pa.stats["reads"] == 1 and lb.da.stats["served"] == 1  # the 16 shared blocks came by READ
    assert lb.pa.stats["sent"] == 9 and lb.da.stats["recv"] == 9
    assert nblk >= 8 * 46
    assert lb.pa.pool.reserved == 0 and lb.da.pool.reserved == 0
    assert lb.hub.stats["bytes"] >= nblk * 32 * 2 * 8 * 64 * 128 * 2


def _run_bench_child(cmd, env, root, timeout, name):
    """Run a bench.py child with its stderr streamed to gpurun_out/<name>.err:
    the multi-rank one-GPU rehearsals take minutes, and pytest prints nothing
    until a test ends, so the file is what shows a long run is alive.  The
    warm-up GEMM tuners are off (they time kernels these tests do not check)."""
    import os
    import subprocess

    env = dict(env, DX_PREFILL_TUNE="0", DX_SKINNY="0", PYTHONUNBUFFERED="1")
    os.makedirs(os.path.join(root, "gpurun_out"), exist_ok=True)
    errp = os.path.join(root, "gpurun_out", name + ".err")
    with open(errp, "w") as err:
        p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=err, text=True, timeout=timeout, env=env, cwd=root)
    with open(errp) as f:
        tail = f.read()[-3000:]
    return p, tail


@pytest.mark.gpu
def test_bench_two_ranks_one_gpu_host_staged_self_validating_gpu(cuda):
    """the N > 1 bench path on one MI355X -- 1P1D, both
    ranks on the one GPU, KV host-staged over gloo (RCCL needs one device per
    rank) -- with the preflight and --verify-tokens 2 on; short window."""
    import json
    import os
    import socket
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    s = socket.socket()
    s.bind(("127.0.0.1", 0))
    port = s.getsockname()[1]
    s.close()
    env = dict(os.environ, MASTER_PORT=str(port), DX_DUMP_AFTER="170")
    for k in ("WORLD_SIZE", "RANK", "LOCAL_RANK"):
        env.pop(k, None)
    cmd = [sys.executable, os.path.join(root, "bench.py"), "--gpus", "2", "--p2p-backend", "gloo",
           "--model", "llama3-8b@8", "--concurrency", "8", "--steps", "2", "--warmup", "1", "--iters-per-step", "10",
           "--num-gpu-blocks", "1200", "--qps-segment", "0", "--verify-tokens", "2", "--no-graph"]
    p, tail = _run_bench_child(cmd, env, root, 240, "test_bench_two_ranks")
    assert p.returncode == 0, tail
    res = json.loads([line for line in p.stdout.splitlines() if line.startswith("{")][-1])
    cfg = res["config"]
    assert cfg["kv_transport"] == "gloo-host" and cfg["parallelism"] == "disagg-1P(tp1)1D(tp1)"
    assert cfg["preflight"]["ok"] and cfg["preflight"]["kv_pairs_checked"] == 1
    assert cfg["verify"]["requests"] == 2 and cfg["verify"]["diverged"] == 0
    assert res["value"] > 0 and cfg["remote_prefills"] > 0


@pytest.mark.gpu
def test_bench_tp2_layout_host_staged_preflight_gpu(cuda):
    """1P(tp2)1D(tp2), all 4 ranks on one GPU (host-staged gloo KV, gloo TP
    collectives): the pre-flight checks every TP group's all-reduce paths and
    the all-gather, and one WRITE + READ per rank pair, then tokens are
    verified.  Round 4 hung here once in five runs: the TP groups used the
    custom IPC all-reduce, whose spin barrier needs the peer process's kernel
    resident at the same time, and four processes on one GPU are time-sliced
    by the hardware scheduler (profiles/r4_tp2_rehearsal_test_hang.log: the
    prefill follower blocked in a host sync behind its own compute stream,
    the leader in the next collective waiting for it).  Ranks sharing a
    device now skip the custom all-reduce (parallel/custom_ar.py; the
    cross-process custom AR + graph path keeps its 2-rank tests in
    test_tp_gpu.py), and a failed barrier fails every later launch at once."""
    import json
    import os
    import socket
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    s = socket.socket()
    s.bind(("127.0.0.1", 0))
    port = s.getsockname()[1]
    s.close()
    env = dict(os.environ, MASTER_PORT=str(port), DX_DUMP_AFTER="240")
    for k in ("WORLD_SIZE", "RANK", "LOCAL_RANK"):
        env.pop(k, None)
    cmd = [sys.executable, os.path.join(root, "bench.py"), "--gpus", "4", "--p2p-backend", "gloo",
           "--prefill-tp", "2", "--decode-tp", "2", "--model", "llama3-8b@8", "--concurrency", "4", "--steps", "2",
           "--warmup", "1", "--iters-per-step", "10", "--num-gpu-blocks", "1200", "--qps-segment", "0",
           "--verify-tokens", "2"]
    p, tail = _run_bench_child(cmd, env, root, 280, "test_bench_tp2_layout")
    assert p.returncode == 0, tail
    res = json.loads([line for line in p.stdout.splitlines() if line.startswith("{")][-1])
    cfg = res["config"]
    assert cfg["parallelism"] == "disagg-1P(tp2)1D(tp2)"
    assert cfg["preflight"]["ok"] and cfg["preflight"]["tp_groups_checked"] == 2
    assert set(cfg["preflight"]["tp_paths"]) == {"gloo"}, cfg["preflight"]
    assert cfg["verify"]["diverged"] == 0


# ------------------------------------------------------------ one-sided (ipc)
def _ipc_pair(**extra):
    kw = dict(model="tiny", device="cpu", block_size=16, max_model_len=512, num_gpu_blocks=300, max_num_seqs=8,
              seed=5, use_cuda_graph=False)
    agg = LLMEngine(EngineConfig(**kw))
    pe = LLMEngine(EngineConfig(chunked_prefill=False, **kw), model=agg.model)
    de = LLMEngine(EngineConfig(**kw), model=agg.model)
    lb = Loopback1P1D(pe, de, layer_group_count=2, kv_transport="ipc", **extra)
    return agg, lb


def test_loopback_one_sided_write_cpu():
    """kv_transport "ipc": the prefill engine writes each layer group straight
    into the decode engine's blocks (no staging, no receive) and copies a
    prefix the decode engine caches straight out of its blocks (one-sided
    READ: pin -> copy -> unpin); tokens equal the aggregated engine's, the
    blocks byte-identical, "done" is only published after the writes."""
    agg, lb = _ipc_pair()
    try:
        prompts = {f"r{i}": [(7 * i + 3 * j) % 500 + 1 for j in range(150 + 9 * i)] for i in range(4)}
        shared = list(range(40, 40 + 64))
        prompts["pre"] = shared + [11] * 90  # decode-side prefix hit: READ, and those blocks are not written
        want = _agg(agg, prompts, 8)
        seen = _watch_blocks(lb)
        _generate(lb, {"warm": shared + [9] * 10}, 2, lambda rid, p, sp, cb: lb.add(rid, p, sp, cb, remote=False))
        lb.run_until_idle(120)
        got = _generate(lb, prompts, 8, lambda rid, p, sp, cb: lb.add(rid, p, sp, cb, remote=True))
        lb.run_until_idle(120)
        assert {k: [t for t, _ in v] for k, v in got.items()} == {k: [t for t, _ in v] for k, v in want.items()}
        assert lb.pa.transport == "ipc" and lb.pa.dp.one_sided
        assert lb.pa.stats["reads"] == 1 and lb.da.stats["served"] == 1  # the shared prefix came by one-sided READ
        assert not lb.d.engine.scheduler.read_pinned and not lb.pa._read1
        assert lb.pa.stats["sent"] == 5 and lb.da.stats["recv"] == 5
        assert _check_bytes(lb, seen, prompts, 16) > 0
        assert lb.hub.stats["copies"] == 0  # nothing went through the send / recv links
        assert lb.pa.pool.in_use == 0 and lb.da.pool.in_use == 0 and not lb.pa.reservations
        assert not lb.d.engine.scheduler.write_pending and not lb.d.engine.scheduler.write_zombies
    finally:
        lb.pa.close()
        lb.da.close()


def test_one_sided_abort_holds_blocks_until_write_done_cpu():
    """A decode request aborted while the prefill worker may be writing into
    its blocks keeps them (write_zombies) until the write is over ("done"
    arrives), then frees them -- never handed to another request mid-write."""
    agg, lb = _ipc_pair()
    try:
        de = lb.d.engine
        sched = de.scheduler
        free0 = de.kv.num_free()
        _generate(lb, {"a": [(5 * j) % 400 + 1 for j in range(200)]}, 4,
                  lambda rid, p, sp, cb: lb.add(rid, p, sp, cb, remote=True))
        # run until the prefill announced the write (decode side marks it pending)
        for _ in range(50):
            lb.step()
            if "a" in sched.write_pending:
                break
        assert "a" in sched.write_pending
        held = len(sched.remote["a"].block_ids)
        lb.d.abort("a")
        lb.d.step()  # apply the abort on the decode engine
        assert "a" in sched.write_zombies and de.kv.num_free() == free0 - held
        lb.run_until_idle(60)  # "done" arrives: the write is over, the blocks come back
        assert not sched.write_zombies and not sched.write_pending
        assert de.kv.num_free() == free0
    finally:
        lb.pa.close()
        lb.da.close()


def test_one_sided_bounds_checked_cpu():
    """A destination block id outside the decode cache is refused on the
    host, before any copy is launched."""
    agg, lb = _ipc_pair()
    try:
        dp = lb.pa.dp
        nb = lb.da.dp.lay.num_blocks
        dp.begin_send("x", [1, 2], "d0", 1, dst_block_ids=[3, nb])
        with pytest.raises(RuntimeError, match="outside"):
            dp.end_forward()  # the group writes are launched here (no forward ran): refused first
        with pytest.raises(ValueError):
            dp.begin_send("y", [1, 2], "d0", 1, dst_block_ids=[3])
    finally:
        lb.pa.close()
        lb.da.close()


@pytest.mark.gpu
def test_loopback_one_sided_write_gpu(cuda):
    """The one-sided WRITE on a GPU, in one process: kv_copy_blocks writes each
    layer group of 4 ISL-1000 prompts into the decode engine's blocks from the
    copy stream, and a fifth prompt's 512-token prefix cached on the decode
    side comes by one-sided READ; blocks byte-identical, tokens equal to the
    aggregated engine (near-tie swaps allowed), no staging used."""
    kw = dict(model="llama3-8b@4", device=str(cuda), block_size=64, max_model_len=2048, num_gpu_blocks=256, seed=3)
    agg = LLMEngine(EngineConfig(max_num_seqs=8, use_cuda_graph=False, chunked_prefill=False, **kw))
    pe = LLMEngine(EngineConfig(max_num_seqs=8, use_cuda_graph=False, chunked_prefill=False, **kw), model=agg.model)
    de = LLMEngine(EngineConfig(max_num_seqs=8, use_cuda_graph=False, **kw), model=agg.model)
    g = torch.Generator().manual_seed(5)
    prompts = {f"r{i}": torch.randint(1, 120000, (1000 + 37 * i,), generator=g).tolist() for i in range(4)}
    shared = torch.randint(1, 120000, (512,), generator=g).tolist()
    prompts["pre"] = shared + torch.randint(1, 120000, (700,), generator=g).tolist()
    want = _agg(agg, prompts, 8)
    lb = Loopback1P1D(pe, de, layer_group_count=2, kv_transport="ipc")
    try:
        seen = _watch_blocks(lb)
        _generate(lb, {"warm": shared + [5] * 40}, 2, lambda rid, p, sp, cb: lb.add(rid, p, sp, cb, remote=False))
        lb.run_until_idle(300)
        got = _generate(lb, prompts, 8, lambda rid, p, sp, cb: lb.add(rid, p, sp, cb, remote=True))
        lb.run_until_idle(300)
        torch.cuda.synchronize()
        assert _check_bytes(lb, seen, prompts, 64) >= 4 * 15
        same, near = _compare(got, want)
        assert same + near == len(prompts), (same, near)
        assert lb.pa.stats["sent"] == 5 and lb.da.stats["recv"] == 5
        assert lb.pa.stats["reads"] == 1 and lb.da.stats["served"] == 1  # the 8 shared blocks came by one-sided READ
        assert not lb.d.engine.scheduler.read_pinned
        assert lb.pa.pool.in_use == 0 and lb.da.pool.in_use == 0
    finally:
        lb.pa.close()
        lb.da.close()


@xproc_ipc
@pytest.mark.gpu
def test_bench_two_ranks_one_gpu_ipc_self_validating_gpu(cuda):
    """The one-sided WRITE between two PROCESSES: 1P1D bench, both ranks on the
    one GPU, the prefill rank maps the decode rank's KV cache through its IPC
    handle and writes into it; the one-sided preflight checks the bytes and
    --verify-tokens 2 compares remote- and local-prefilled decodes."""
    import json
    import os
    import socket
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    s = socket.socket()
    s.bind(("127.0.0.1", 0))
    port = s.getsockname()[1]
    s.close()
    env = dict(os.environ, MASTER_PORT=str(port), DX_DUMP_AFTER="170")
    for k in ("WORLD_SIZE", "RANK", "LOCAL_RANK"):
        env.pop(k, None)
    cmd = [sys.executable, os.path.join(root, "bench.py"), "--gpus", "2", "--p2p-backend", "ipc",
           "--model", "llama3-8b@8", "--concurrency", "8", "--steps", "2", "--warmup", "1", "--iters-per-step", "10",
           "--num-gpu-blocks", "1200", "--qps-segment", "0", "--verify-tokens", "2", "--no-graph"]
    p, tail = _run_bench_child(cmd, env, root, 240, "test_bench_two_ranks_ipc")
    assert p.returncode == 0, tail
    res = json.loads([line for line in p.stdout.splitlines() if line.startswith("{")][-1])
    cfg = res["config"]
    assert cfg["kv_transport"] == "ipc" and cfg["parallelism"] == "disagg-1P(tp1)1D(tp1)"
    assert cfg["preflight"]["ok"] and cfg["preflight"]["kv_pairs_checked"] == 1
    assert cfg["verify"]["requests"] == 2 and cfg["verify"]["diverged"] == 0
    assert res["value"] > 0 and cfg["remote_prefills"] > 0


def test_one_sided_write_timeout_prefills_locally_cpu():
    """A write announced but never done (the prefill worker died mid-write:
    its "done" is dropped here) -> after the write timeout the decode engine
    prefills the request itself and decodes the aggregated engine's tokens;
    the blocks stay held (write_pending) until the late "done" releases them."""
    from dynamo_exp_amd.disagg.agent import decode_leader_hook

    agg, lb = _ipc_pair()
    try:
        lb.dhook = decode_leader_hook(lb.d, lb.da, write_timeout=0.3)
        held = []
        pub = lb.pa._publish

        def drop_done(engine_id, msg):
            if msg.get("t") == "done" and msg["rid"] == "lost":
                held.append((engine_id, msg))
                return
            pub(engine_id, msg)

        lb.pa._publish = drop_done
        prompt = [(7 * j) % 450 + 1 for j in range(120)]
        want = _agg(agg, {"lost": prompt}, 6)
        got = _generate(lb, {"lost": prompt}, 6, lambda rid, p, sp, cb: lb.add(rid, p, sp, cb, remote=True))
        lb.run_until_idle(60)
        assert [t for t, _ in got["lost"]] == [t for t, _ in want["lost"]]
        assert lb.da.stats.get("write_timeouts") == 1 and held
        sched = lb.d.engine.scheduler
        assert "lost" in sched.write_zombies  # finished, blocks still held for the writer
        free = lb.d.engine.kv.num_free()
        pub(*held[0])  # the late "done"
        lb.step()
        lb.step()
        assert not sched.write_zombies and not sched.write_pending
        assert lb.d.engine.kv.num_free() > free
    finally:
        lb.pa.close()
        lb.da.close()


def test_one_sided_unmaps_departed_decode_engines_cpu():
    """gc_peers: a mapped decode cache whose engine's metadata is gone (lease
    expired) is unmapped once no write to it is in flight."""
    agg, lb = _ipc_pair()
    try:
        closed = []

        class _Map:
            def close(self):
                closed.append(True)

        m = _Map()
        key = ("d0", 0)
        lb.pa._ipc_by_key[key] = m
        lb.pa._ipc_owned.append(m)
        assert lb.pa.gc_peers() == 0  # d0's metadata is still published
        del lb.cp.kv[f"{lb.pa.ns}/kv_transfer/d0/0"]
        assert lb.pa.gc_peers() == 1 and closed and key not in lb.pa._ipc_by_key
    finally:
        lb.pa.close()
        lb.da.close()


@xproc_ipc
@pytest.mark.gpu
def test_bench_1p_tp1_to_1d_tp2_one_gpu_ipc_gpu(cuda):
    """The reference benchmark's layout shape at small scale (prefill TP 1 ->
    decode TP 2), three processes on the one GPU over the one-sided transport:
    the prefill rank writes each decode rank's KV-head piece into that rank's
    shared cache; one-sided preflight per (prefill, decode rank) pair and
    --verify-tokens 2 against a local prefill."""
    import json
    import os
    import socket
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    s = socket.socket()
    s.bind(("127.0.0.1", 0))
    port = s.getsockname()[1]
    s.close()
    env = dict(os.environ, MASTER_PORT=str(port), DX_DUMP_AFTER="230", GPU_MAX_HW_QUEUES="2")
    for k in ("WORLD_SIZE", "RANK", "LOCAL_RANK"):
        env.pop(k, None)
    cmd = [sys.executable, os.path.join(root, "bench.py"), "--gpus", "3", "--p2p-backend", "ipc",
           "--prefill-tp", "1", "--decode-tp", "2", "--prefill-ranks", "1", "--model", "llama3-8b@8",
           "--concurrency", "4", "--steps", "2", "--warmup", "1", "--iters-per-step", "10", "--num-gpu-blocks", "1200",
           "--qps-segment", "0", "--verify-tokens", "2"]
    p, tail = _run_bench_child(cmd, env, root, 280, "test_bench_1p1d_tp2_ipc")
    assert p.returncode == 0, tail
    res = json.loads([line for line in p.stdout.splitlines() if line.startswith("{")][-1])
    cfg = res["config"]
    assert cfg["kv_transport"] == "ipc" and cfg["parallelism"] == "disagg-1P(tp1)1D(tp2)"
    assert cfg["preflight"]["ok"] and cfg["preflight"]["tp_groups_checked"] == 1
    assert cfg["verify"]["diverged"] == 0 and cfg["remote_prefills"] > 0


def test_one_sided_read_refused_recomputes_cpu():
    """One-sided READ whose blocks the decode engine no longer holds (its
    verdict is false): nothing is copied, nothing stays pinned or held, and
    the prefill engine computes the whole prompt -- same tokens."""
    agg, lb = _ipc_pair()
    try:
        shared = list(range(40, 40 + 64))
        prompt = shared + [13] * 70
        want = _agg(agg, {"p": prompt}, 5)
        _generate(lb, {"warm": shared + [9] * 10}, 2, lambda rid, p, sp, cb: lb.add(rid, p, sp, cb, remote=False))
        lb.run_until_idle(60)
        lb.da.read_blocks_of = lambda rid, first, last: None  # the decode engine gave the blocks up
        got = _generate(lb, {"p": prompt}, 5, lambda rid, p, sp, cb: lb.add(rid, p, sp, cb, remote=True))
        lb.run_until_idle(60)
        assert [t for t, _ in got["p"]] == [t for t, _ in want["p"]]
        assert lb.pa.stats["reads"] == 1 and lb.da.stats.get("reads_refused") == 1
        assert not lb.pa._read1 and not lb.p.engine.scheduler.write_pending
        assert not lb.d.engine.scheduler.read_pinned and not lb.d.engine.scheduler.write_zombies
    finally:
        lb.pa.close()
        lb.da.close()


def test_one_sided_preflight_write_and_read_round_trip_cpu():
    """kv_check_one_sided over the in-process pair: the prefill rank's WRITE
    lands byte-exact in the decode cache and its one-sided READ brings the
    same bytes back into fresh blocks (barriers are no-ops in one process)."""
    from dynamo_exp_amd.disagg.preflight import kv_check_one_sided

    agg, lb = _ipc_pair()
    try:
        tps = {"p0": 1, "d0": 1}
        rp = kv_check_one_sided(lb.pa.dp, "p0", True, ["p0"], ["d0"], tps, lambda: None)
        rd = kv_check_one_sided(lb.da.dp, "d0", False, ["p0"], ["d0"], tps, lambda: None)
        assert rp["ok"] and rp["read_ok"] == 1, rp
        assert rd["ok"] and rd["write_ok"] == 1, rd
    finally:
        lb.pa.close()
        lb.da.close()


def test_one_sided_read_timeout_recomputes_cpu(monkeypatch):
    """A one-sided READ the decode engine never answers (its "read1" lost):
    after DX_REMOTE_READ_TIMEOUT_S the prefill engine recomputes the prefix
    -- same tokens, nothing left held."""
    monkeypatch.setenv("DX_REMOTE_READ_TIMEOUT_S", "0.2")
    agg, lb = _ipc_pair()
    try:
        shared = list(range(40, 40 + 64))
        prompt = shared + [17] * 70
        want = _agg(agg, {"p": prompt}, 5)
        _generate(lb, {"warm": shared + [9] * 10}, 2, lambda rid, p, sp, cb: lb.add(rid, p, sp, cb, remote=False))
        lb.run_until_idle(60)
        pub = lb.pa._publish
        lb.pa._publish = lambda e, m: None if m.get("t") == "read1" else pub(e, m)
        got = _generate(lb, {"p": prompt}, 5, lambda rid, p, sp, cb: lb.add(rid, p, sp, cb, remote=True))
        lb.run_until_idle(60)
        assert [t for t, _ in got["p"]] == [t for t, _ in want["p"]]
        assert lb.pa.stats["reads"] == 1 and lb.da.stats["served"] == 0
        assert not lb.pa._read1 and not lb.pa._read1_t0 and not lb.p.engine.scheduler.write_pending
    finally:
        lb.pa.close()
        lb.da.close()


@xproc_ipc
@pytest.mark.gpu
def test_bench_two_sided_preflight_failure_falls_back_to_one_sided_gpu(cuda):
    """A two-sided KV path that fails its preflight (a corrupted piece,
    DX_FAULTS) makes every rank switch to the one-sided transport together
    (the decode caches are allocated shareable up front), re-check, and run:
    the result names the transport it measured and the failure it left."""
    import json
    import os
    import socket
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    s = socket.socket()
    s.bind(("127.0.0.1", 0))
    port = s.getsockname()[1]
    s.close()
    env = dict(os.environ, MASTER_PORT=str(port), DX_DUMP_AFTER="170", DX_FAULTS="kv_transfer.corrupt_pieces=1")
    for k in ("WORLD_SIZE", "RANK", "LOCAL_RANK"):
        env.pop(k, None)
    cmd = [sys.executable, os.path.join(root, "bench.py"), "--gpus", "2", "--p2p-backend", "gloo",
           "--model", "llama3-8b@8", "--concurrency", "8", "--steps", "2", "--warmup", "1", "--iters-per-step", "10",
           "--num-gpu-blocks", "1200", "--qps-segment", "0", "--verify-tokens", "2", "--no-graph"]
    p, tail = _run_bench_child(cmd, env, root, 240, "test_bench_fallback")
    assert p.returncode == 0, tail
    res = json.loads([line for line in p.stdout.splitlines() if line.startswith("{")][-1])
    cfg = res["config"]
    assert cfg["kv_transport"] == "ipc" and cfg["preflight"]["ok"]
    assert cfg["preflight"]["fallback_from"]["transport"] == "gloo-host"
    assert cfg["verify"]["diverged"] == 0 and cfg["remote_prefills"] > 0


def test_one_sided_dead_writer_releases_blocks_cpu(monkeypatch):
    """A decode request that was written into by a prefill engine that then
    vanished (its lease and metadata gone, no "done" ever) is not left holding
    its blocks: the decode hook notices the writer is gone and releases them
    (prefilling locally whatever still waits)."""
    import time as _time

    from dynamo_exp_amd.disagg.agent import decode_leader_hook

    agg, lb = _ipc_pair()
    try:
        lb.dhook = decode_leader_hook(lb.d, lb.da, write_timeout=0.2)
        pub = lb.pa._publish
        lb.pa._publish = lambda e, m: None if m.get("t") == "done" else pub(e, m)
        prompt = [(11 * j) % 450 + 1 for j in range(100)]
        want = _agg(agg, {"x": prompt}, 4)
        got = _generate(lb, {"x": prompt}, 4, lambda rid, p, sp, cb: lb.add(rid, p, sp, cb, remote=True))
        lb.run_until_idle(60)  # the write times out, the request is prefilled locally, finishes: zombie
        sched = lb.d.engine.scheduler
        assert [t for t, _ in got["x"]] == [t for t, _ in want["x"]]
        assert "x" in sched.write_zombies
        del lb.cp.kv[f"{lb.pa.ns}/kv_transfer/p0/0"]  # the prefill engine's lease expired
        t0 = _time.time()
        while sched.write_zombies and _time.time() - t0 < 30:
            lb.step()
            _time.sleep(0.05)
        assert not sched.write_zombies and not sched.write_pending
    finally:
        lb.pa.close()
        lb.da.close()
