"""Bekulix in the engine against the plain oracle (tests/bekulix_oracle.py).

Every test builds its own small configuration and random (or crafted) weights
in the checkpoint's naming, runs the engine -- scheduler, page manager, model
runner, the model's ops -- and compares with the oracle's dense, whole-sequence
float64 arithmetic.  On `cpu` the ops run their PyTorch forms, on `cuda` (gpu
marker) the gfx950 kernels, in float32 and bfloat16.
"""
from __future__ import annotations

import math

import pytest
import torch

import bekulix_oracle as O
from dynamo_exp_amd.engine.engine import EngineConfig, LLMEngine
from dynamo_exp_amd.engine.request import SamplingParams
from dynamo_exp_amd.models.bekulix import BekulixForCausalLM
from dynamo_exp_amd.models.config import LayeredConfig
from dynamo_exp_amd.ops import mixers as mx

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
CASES = [("cpu", "float32"), pytest.param("cuda", "float32", marks=pytest.mark.gpu),
         pytest.param("cuda", "bfloat16", marks=pytest.mark.gpu)]
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


# ----------------------------------------------------------------- configurations
def att(H=6, G=3, d=20, coef=0.5, every=4, mlp=56):
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": d, "scale": d ** -0.5}
    if coef:
        m["q_temp"] = {"coef": coef, "every": every}
    return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": mlp} if mlp else None}


def lat(H=5, d=12, dv=28, r=36, window=5, mlp=40):
    return {"type": "latent_attention",
            "mixer": {"heads": H, "dim": d, "vdim": dv, "kv_rank": r, "scale": d ** -0.5, "mask": {"size": window}},
            "mlp": {"kind": "dense", "ff": mlp} if mlp else None}


def dif(H=4, G=2, d=12, dv=40, chunk=7, diff=0.3, mlp=48):
    return {"type": "attention_2",
            "mixer": {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": d ** -0.5, "diff": diff,
                      "mask": {"size": chunk}},
            "mlp": {"kind": "dense", "ff": mlp} if mlp else None}


def config(layers, width=72, vocab=97, streams=3, loop=None, eps=1e-5):
    return LayeredConfig(name="t", vocab_size=vocab, hidden_size=width, layers=layers, loop=loop, rms_norm_eps=eps,
                         streams=streams)


def cfg_dict(cfg: LayeredConfig) -> dict:
    d = {"layers": cfg.layers, "norm": {"eps": cfg.rms_norm_eps}, "vocab": cfg.vocab_size, "width": cfg.hidden_size}
    if cfg.loop:
        d["loop"] = cfg.loop
    if cfg.streams:
        d["streams"] = cfg.streams
    return d


CONFIGS = {
    # all three mixers, a loop, three streams, widths that are no multiples of 8
    "mixed": lambda: config([lat(), att(), dif(), att(H=4, G=4, d=16, coef=0.0, mlp=None)],
                            loop={"start": 0, "stop": 2, "times": 2}),
    # values a model may happen to make equal or one: one KV head, one stream with
    # its own weights, a loop that runs once, a window and a chunk of one token
    "ones": lambda: config([att(H=4, G=1, d=8, every=1), lat(H=2, d=8, dv=8, r=8, window=1),
                            dif(H=2, G=1, d=8, dv=8, chunk=1, diff=0.0)], width=32, streams=1,
                           loop={"start": 1, "stop": 2, "times": 1}),
    # nothing divides by 4 or 8: width, vocabulary, feed-forward and head widths on the scalar paths, five streams
    "odd": lambda: config([att(H=3, G=1, d=18, mlp=50), lat(H=3, d=10, dv=14, r=38, window=7, mlp=34),
                           dif(H=2, G=2, d=6, dv=22, chunk=5, mlp=None)], width=102, vocab=101, streams=5),
    # head widths the matrix-core prefill kernel serves (bf16 on the GPU)
    "tiles": lambda: config([att(H=4, G=2, d=32, every=16), lat(H=2, d=16, dv=32, r=48, window=20),
                             dif(H=2, G=1, d=64, dv=128, chunk=24), att(H=2, G=1, d=64, coef=0.0)], width=64,
                            streams=2, loop={"start": 1, "stop": 3, "times": 2}),
    # no streams at all (plain residual), heads == kv heads, wide value heads (> 64 columns)
    "plain": lambda: config([dif(H=2, G=2, d=24, dv=136, chunk=9), lat(H=3, d=8, dv=72, r=80, window=11),
                             att(H=2, G=2, d=72, every=3)], width=64, streams=None),
}


def weights(cfg, seed=0):
    return BekulixForCausalLM(cfg, "cpu", torch.float32).random_state(seed)


def engine(cfg, sd, device, dtype, blocks=48, bs=8, graphs=False, seqs=4):
    model = BekulixForCausalLM(cfg, device, DT[dtype]).load_state(sd)
    return LLMEngine(EngineConfig(model="t", device=device, dtype=dtype, block_size=bs, num_gpu_blocks=blocks,
                                  max_model_len=blocks * bs, max_num_seqs=seqs, enable_prefix_caching=False,
                                  use_cuda_graph=graphs, graph_sizes=(1, 2, 4), async_schedule=False),
                     model_cfg=cfg, model=model)


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def close(got, want, dtype, what=""):
    """Logit rows agree: error relative to the rows' spread, after the mean is taken off."""
    got = got.detach().double().cpu()
    want = want.double()
    a, b = got - got.mean(-1, keepdim=True), want - want.mean(-1, keepdim=True)
    err = ((a - b) ** 2).mean(-1).sqrt() / b.pow(2).mean().sqrt()
    lim = 2e-4 if dtype == "float32" else 4e-2
    assert float(err.max()) < lim, f"{what}: error {float(err.max()):.3g} at row {int(err.argmax())} (limit {lim})"


def run_cut(eng, rid, toks, cuts, want=None):
    """Feed `toks` in portions of the given sizes (the rest one by one); logits of all positions."""
    out, at = [], 0
    sizes = list(cuts) + [1] * (len(toks) - sum(cuts))
    for n in sizes:
        part = toks[at:at + n]
        last = at + n == len(toks)
        got = eng.forced_step([(rid, part, list(range(n)))], [rid] if last else [])
        out.append(got[rid])
        at += n
    return torch.cat(out, 0)


# ----------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("S", [1, 3, 8])
def test_stream_step_alone(device, S):
    torch.manual_seed(S)
    T, W = 5, 70
    X = torch.randn(T, S, W)
    y = torch.randn(T, W)
    mix, gain, rin, nw = torch.randn(S, S), torch.randn(S), torch.randn(S), torch.randn(W)
    want_x = torch.einsum("st,nsw->ntw", mix.double(), X.double()) + gain.double()[None, :, None] * y.double()[:, None]
    u = torch.einsum("s,nsw->nw", rin.double(), want_x)
    want = O.rms(u, 1e-5) * nw.double()
    Xd = X.to(device).clone()
    got = mx.stream_step(Xd, y.to(device), mix.to(device), gain.to(device), rin.to(device), nw.to(device), 1e-5,
                         torch.float32)
    assert torch.allclose(Xd.cpu().double(), want_x, atol=1e-5)
    assert torch.allclose(got.cpu().double(), want, atol=1e-5)
    # read-in only (no pending output), plain sum
    got = mx.stream_step(Xd, None, None, None, torch.ones(S, device=device), None, 1e-5, torch.float32)
    assert torch.allclose(got.cpu().double(), want_x.sum(1), atol=1e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("act", ["relu", "silu", "gelu_tanh"])
def test_glu_act_alone(device, act):
    torch.manual_seed(1)
    gu = torch.randn(7, 2 * 37)
    g, u = gu.double().split(37, 1)
    f = {"relu": torch.relu(g), "silu": g * torch.sigmoid(g),
         "gelu_tanh": 0.5 * g * (1 + torch.tanh(math.sqrt(2 / math.pi) * (g + 0.044715 * g ** 3)))}[act]
    assert torch.allclose(mx.glu_act(gu.to(device), act).cpu().double(), f * u, atol=1e-5)


def paged(T, bs, n_blocks, width, device, dtype=torch.float32, seed=0):
    """A shuffled block table for one sequence of T tokens, and empty caches."""
    g = torch.Generator().manual_seed(seed)
    nb = -(-T // bs)
    table = torch.randperm(n_blocks, generator=g)[:nb].to(torch.int32)
    j = torch.arange(T)
    slots = table.long()[j // bs] * bs + j % bs
    return table[None].to(device), slots.to(device), torch.zeros(n_blocks * bs, width, dtype=dtype, device=device)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("mask,size", [("causal", 0), ("window", 6), ("window", 1), ("chunk", 5), ("chunk", 64)])
@pytest.mark.parametrize("dims", [(4, 2, 1, 20, 20), (4, 1, 2, 12, 72), (3, 3, 1, 8, 136)])
def test_row_attention_alone(device, mask, size, dims):
    """Prompt rows over a shuffled page table against dense masked softmax; then the
    same rows as decode rows (row i = its own sequence), split into key parts."""
    H, G, maps, d, dv = dims
    T, bs = 70, 8
    torch.manual_seed(7)
    q = torch.randn(T, H, maps, d)
    k = torch.randn(T, G, maps, d)
    v = torch.randn(T, G, dv)
    vis = O.visible(T, mask, size)
    want = torch.stack([O.softmax_attend(q[:, :, m].double(), O.expand_heads(k[:, :, m].double(), H),
                                         O.expand_heads(v.double(), H), 0.3, vis) for m in range(maps)], 2)
    table, slots, kc = paged(T, bs, 12, G * maps * d, device)
    vc = torch.zeros(12 * bs, G * dv, device=device)
    kc[slots] = k.reshape(T, -1).to(device)
    vc[slots] = v.reshape(T, -1).to(device)
    pos = torch.arange(T, device=device)
    seq = torch.zeros(T, dtype=torch.int32, device=device)
    qd = q.reshape(T, -1).to(device)
    got = mx.row_attention(qd, kc, vc, pos, seq, table, bs, H * maps, maps, H // G, d, dv, 0.3, mask, size)
    assert torch.allclose(got.cpu().double().view(T, H, maps, dv), want, atol=2e-5)
    rows = torch.tensor([0, 1, 7, 8, 33, 69], device=device)
    got = mx.row_attention(qd[rows], kc, vc, pos[rows], None, table.expand(len(rows), -1).contiguous(), bs, H * maps,
                           maps, H // G, d, dv, 0.3, mask, size, parts=2)
    assert torch.allclose(got.cpu().double().view(-1, H, maps, dv), want[rows.cpu()], atol=2e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("mask,size", [("causal", 0), ("window", 70), ("window", 3), ("chunk", 50), ("chunk", 200)])
@pytest.mark.parametrize("dims", [(4, 2, 1, 32, 32), (2, 1, 2, 64, 128), (3, 3, 1, 128, 128), (2, 2, 1, 48, 48),
                                  (2, 1, 1, 256, 256), (2, 1, 2, 128, 256), (2, 2, 2, 48, 96), (40, 1, 1, 64, 64),
                                  (20, 1, 1, 32, 32)])
def test_tile_attention_alone(mask, size, dims):
    """The matrix-core prefill kernel: a 263-row portion that starts at position
    37 of a cached prefix (three tiles, the last ragged, cut inside pages,
    windows and chunks) beside two decode rows of another sequence, against
    dense masked softmax over the bf16 values; fp32 output, so the weights'
    precision shows."""
    H, G, maps, d, dv = dims
    T, bs, start = 300, 16, 37
    torch.manual_seed(5)
    q = torch.randn(T, H, maps, d).bfloat16()
    k = (torch.randn(T, G, maps, d) * 0.5).bfloat16()
    v = torch.randn(T, G, dv).bfloat16()
    vis = O.visible(T, mask, size)
    want = torch.stack([O.softmax_attend(q[:, :, m].double(), O.expand_heads(k[:, :, m].double(), H),
                                         O.expand_heads(v.double(), H), 0.2, vis) for m in range(maps)], 2)
    perm = torch.randperm(40, generator=torch.Generator().manual_seed(3)).to(torch.int32)
    table = torch.stack([perm[:19], perm[19:38]]).contiguous().cuda()  # two sequences, the same tokens on other pages
    j = torch.arange(T, device="cuda")
    slots, s2 = (table[i].long()[j // bs] * bs + j % bs for i in (0, 1))
    kc = torch.zeros(40 * bs, G * maps * d, device="cuda", dtype=torch.bfloat16)
    vc = torch.zeros(40 * bs, G * dv, device="cuda", dtype=torch.bfloat16)
    for sl in (slots, s2):
        kc[sl] = k.reshape(T, -1).cuda()
        vc[sl] = v.reshape(T, -1).cuda()
    rows = list(range(start, T)) + [5, 290]
    n_pre = T - start
    pos = torch.tensor(rows, device="cuda")
    seq = torch.tensor([0] * n_pre + [1, 1], dtype=torch.int32, device="cuda")
    tiles = torch.tensor(mx.tile_list(0, n_pre), dtype=torch.int32, device="cuda")
    qd = q.reshape(T, -1).cuda()[pos]
    assert mx.tile_attention_ok(qd, d, dv)
    got = mx.attention(qd, kc, vc, pos, seq, table, bs, H * maps, maps, H // G, d, dv, 0.2, mask, size, 1, True, tiles,
                       n_pre)
    err = (got.cpu().double().view(-1, H, maps, dv) - want[rows]).abs().max()
    assert float(err) < 3e-4, float(err)
    got = mx.attention(qd, kc, vc, pos, seq, table, bs, H * maps, maps, H // G, d, dv, 0.2, mask, size, 3, False,
                       tiles, n_pre)
    assert float((got.cpu().double().view(-1, H, maps, dv) - want[rows]).abs().max()) < 3e-2
    # decode rows alone (row i = sequence i), keys split into parts
    dr = torch.tensor([0, 1, 63, 64, 65, 255, 299], device="cuda")
    got = mx.attention(q.reshape(T, -1).cuda()[dr], kc, vc, dr, None, table[:1].expand(len(dr), -1).contiguous(), bs,
                       H * maps, maps, H // G, d, dv, 0.2, mask, size, 2, True)
    assert float((got.cpu().double().view(-1, H, maps, dv) - want[dr.cpu()]).abs().max()) < 3e-4


@pytest.mark.parametrize("device", DEVICES)
def test_headprep_and_diff_combine_alone(device):
    torch.manual_seed(3)
    T, H, G, d, eps = 9, 3, 2, 10, 1e-5
    x = torch.randn(T, (H + G) * d + 5)
    qw, kw = torch.randn(d), torch.randn(d)
    pos = torch.arange(100, 100 + T)
    table, slots, kc = paged(T, 4, 6, G * d, device)
    vc = torch.zeros_like(kc)
    xd = x.to(device).clone()
    mx.headprep_cache(xd, pos.to(device), slots, H, G, d, H * d, qw.to(device), kw.to(device), eps, (0.5, 8), kc, vc,
                      v_mode=1)
    q = O.norm_plain(x[:, :H * d].double().view(T, H, d), qw.double(), eps)
    q = q * (1 + 0.5 * torch.log(torch.floor((pos.double() + 1) / 8) + 1))[:, None, None]
    k = x[:, H * d:(H + G) * d].double().view(T, G, d)
    assert torch.allclose(xd[:, :H * d].cpu().double(), q.reshape(T, -1), atol=1e-5)
    assert torch.allclose(kc[slots].cpu().double(), O.norm_plain(k, kw.double(), eps).reshape(T, -1), atol=1e-5)
    assert torch.equal(vc[slots].cpu(), x[:, H * d:(H + G) * d])
    assert torch.equal(xd[:, (H + G) * d:].cpu(), x[:, (H + G) * d:])
    a = torch.randn(T, H, 2, 44)
    o = O.rms(a[:, :, 0].double() - 0.7 * a[:, :, 1].double(), eps) * 0.4
    got = mx.diff_combine(a.to(device), 0.7, 0.4, eps, torch.float32)
    assert torch.allclose(got.cpu().double(), o.reshape(T, -1), atol=1e-5)


# ----------------------------------------------------------------- crafted keys
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("decode", [False, True])
def test_one_key_stands_out(device, decode):
    """A query that matches exactly one key by a wide margin returns that key's
    value if and only if the mask lets it through: far keys among hundreds, keys
    at page borders, and keys just inside / just outside a window or chunk."""
    T, d, dv, bs = 300, 16, 24, 16
    torch.manual_seed(11)
    k = torch.randn(T, d) * 0.1
    v = torch.randn(T, dv)
    table, slots, kc = paged(T, bs, 24, d, device)
    vc = torch.zeros(24 * bs, dv, device=device)
    vc[slots] = v.to(device)
    p = T - 1
    cases = [("causal", 0, 3, True), ("causal", 0, 0, True), ("causal", 0, bs - 1, True), ("causal", 0, bs, True),
             ("window", 40, p - 39, True), ("window", 40, p - 40, False), ("window", 40, p, True),
             ("chunk", 50, 250, True), ("chunk", 50, 249, False), ("chunk", 149, 298, True), ("chunk", 149, 297, False)]
    for mask, size, j, seen in cases:
        kk = k.clone()
        kk[j] = 0
        kk[j, 0] = 40.0
        kc[slots] = kk.to(device)
        q = torch.zeros(1, d)
        q[0, 0] = 1.0
        pos = torch.tensor([p], device=device)
        seq = None if decode else torch.zeros(1, dtype=torch.int32, device=device)
        got = mx.row_attention(q.to(device), kc, vc, pos, seq, table, bs, 1, 1, 1, d, dv, 1.0, mask, size,
                               parts=3 if decode else 1).cpu()[0, 0]
        hit = torch.allclose(got, v[j], atol=1e-4)
        assert hit == seen, f"{mask} {size}: key {j} from position {p} seen={hit}, expected {seen}"


# ----------------------------------------------------------------- the model in the engine
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_and_layers(device, dtype, name):
    cfg = CONFIGS[name]()
    sd = weights(cfg, 1)
    toks = tokens(45, cfg.vocab_size, 2)
    want, layers = O.forward(cfg_dict(cfg), sd, toks, return_layers=True)
    eng = engine(cfg, sd, device, dtype)
    eng.model.trace_layers = []
    got = eng.forced_step([("a", toks, list(range(len(toks))))], ["a"])["a"]
    close(got, want, dtype, name)
    assert len(eng.model.trace_layers) == len(cfg.layer_runs()) == layers.shape[0]
    tol = 1e-3 if dtype == "float32" else 0.25
    for i, x in enumerate(eng.model.trace_layers):
        assert float((x.cpu().double() - layers[i]).abs().max()) < tol * max(1.0, float(layers[i].abs().max())), i
    assert eng.kv.num_free() == eng.kv.num_blocks


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_token_by_token_and_portions(device, dtype, name):
    """Prefill against one-token steps and against portions of several sizes
    (down to two tokens, cut inside pages, windows and chunks), long enough that
    every window and chunk passes over decoded tokens."""
    cfg = CONFIGS[name]()
    sd = weights(cfg, 3)
    toks = tokens(52, cfg.vocab_size, 4)
    want = O.forward(cfg_dict(cfg), sd, toks)
    eng = engine(cfg, sd, device, dtype)
    close(run_cut(eng, "one", toks, []), want, dtype, "token by token")
    close(run_cut(eng, "cut", toks, [2, 3, 2, 11, 7, 2, 9]), want, dtype, "portions")
    close(run_cut(eng, "pre", toks, [17]), want, dtype, "prefill then decode")
    assert eng.kv.num_free() == eng.kv.num_blocks


@pytest.mark.parametrize("device,dtype", CASES)
def test_mixed_batches_and_reused_pages(device, dtype):
    """Four unequal requests interleaved (portions beside single tokens, a request
    left out of steps) in a pool that only fits them because finished requests
    give their pages back; every request equals itself alone."""
    cfg = CONFIGS["mixed"]()
    sd = weights(cfg, 5)
    lens = {"a": 37, "b": 9, "c": 23, "d": 1, "e": 30, "f": 18}
    toks = {k: tokens(n, cfg.vocab_size, 10 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: O.forward(cfg_dict(cfg), sd, t) for k, t in toks.items()}
    eng = engine(cfg, sd, device, dtype, blocks=14, bs=8)  # 112 token slots < 118 tokens in all
    at = {k: 0 for k in toks}
    got = {k: [] for k in toks}
    plan = [[("a", 20), ("b", 2)], [("a", 1), ("b", 5), ("c", 23)], [("a", 1), ("b", 1), ("d", 1)],
            [("a", 15), ("b", 1)], [("e", 2), ("f", 17)], [("e", 1), ("f", 1)], [("e", 27)]]
    for step in plan:
        entries, end = [], []
        for k, n in step:
            entries.append((k, toks[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == lens[k]:
                end.append(k)
        out = eng.forced_step(entries, end)
        for k, _ in step:
            got[k].append(out[k])
    for k in toks:
        close(torch.cat(got[k], 0), want[k], dtype, f"request {k}")
    assert eng.kv.num_free() == eng.kv.num_blocks
    with pytest.raises(RuntimeError):  # a fifth live request
        for i in range(5):
            eng.forced_step([(f"x{i}", [1, 2], [])], [])


@pytest.mark.parametrize("device,dtype", CASES)
def test_first_tokens_and_long_decoding(device, dtype):
    cfg = config([att(H=2, G=1, d=8, every=16), lat(H=2, d=8, dv=8, r=16, window=24), dif(H=2, G=1, d=8, dv=16, chunk=32)],
                 width=32, streams=2)
    sd = weights(cfg, 6)
    toks = tokens(150, cfg.vocab_size, 7)
    want = O.forward(cfg_dict(cfg), sd, toks)
    eng = engine(cfg, sd, device, dtype, blocks=40, bs=4)
    got = run_cut(eng, "r", toks, [1, 1, 2])  # positions 0, 1, then a portion, then 146 decode steps
    close(got, want, dtype, "long decoding")


@pytest.mark.parametrize("device,dtype", CASES)
def test_temperature_window_edge_shows_in_logits(device, dtype):
    """Weights made so that faults cannot hide: the query gain steps at `every`,
    and one strong token just outside / inside the window moves the logits."""
    cfg = config([lat(H=2, d=8, dv=8, r=16, window=6, mlp=None), att(H=2, G=1, d=8, coef=2.0, every=5, mlp=None)],
                 width=32, streams=None)
    sd = weights(cfg, 8)
    sd["l0.mix.o"] = sd["l0.mix.o"] * 4
    sd["l1.mix.o"] = sd["l1.mix.o"] * 4
    toks = tokens(30, cfg.vocab_size, 9)
    want = O.forward(cfg_dict(cfg), sd, toks)
    # the oracle itself is sensitive: a window one token off changes the logits visibly
    off = cfg_dict(cfg)
    off["layers"] = [dict(off["layers"][0], mixer=dict(off["layers"][0]["mixer"], mask={"size": 7})), off["layers"][1]]
    assert float((O.forward(off, sd, toks) - want).abs().max()) > 1e-2
    eng = engine(cfg, sd, device, dtype)
    close(run_cut(eng, "r", toks, [13, 2]), want, dtype)


# ----------------------------------------------------------------- generation through the engine's entry point
@pytest.mark.parametrize("device,dtype,graphs", [("cpu", "float32", False),
                                                 pytest.param("cuda", "float32", False, marks=pytest.mark.gpu),
                                                 pytest.param("cuda", "float32", True, marks=pytest.mark.gpu),
                                                 pytest.param("cuda", "bfloat16", True, marks=pytest.mark.gpu)])
def test_greedy_generation(device, dtype, graphs):
    """add_request + step(): the scheduler batches three prompts of unequal
    length, chunked prefill, decode (HIP graphs when asked), greedy sampling.
    Each request's tokens equal the oracle's greedy continuation (fp32), or the
    engine's own forced replay of what it generated (bf16)."""
    cfg = CONFIGS["mixed"]()
    sd = weights(cfg, 12)
    eng = engine(cfg, sd, device, dtype, blocks=64, bs=8, graphs=graphs)
    eng.cfg.max_num_batched_tokens = eng.scheduler.cfg.max_num_batched_tokens = 16  # prompts are split
    if graphs:
        eng.warmup()
    prompts = {f"g{i}": tokens(n, cfg.vocab_size, 20 + i) for i, n in enumerate((5, 21, 12))}
    outs = {k: [] for k in prompts}
    for k, p in prompts.items():
        eng.add_request(k, p, SamplingParams(max_tokens=12, ignore_eos=True),
                        on_output=lambda r, t, lp, fin: outs[r.request_id].extend(t))
    while eng.has_unfinished():
        eng.step()
    for k, p in prompts.items():
        assert len(outs[k]) == 12
        seq = p + outs[k]
        if dtype == "float32":
            lg = O.forward(cfg_dict(cfg), sd, seq[:-1])
        else:
            lg = eng.forced_step([(k + "r", seq[:-1], list(range(len(seq) - 1)))], [k + "r"])[k + "r"].cpu().double()
        top2 = lg[len(p) - 1:].topk(2, -1).values
        sure = (top2[:, 0] - top2[:, 1]) > (1e-3 if dtype == "float32" else 0.1)  # skip near-ties
        pick = lg[len(p) - 1:].argmax(-1)
        assert torch.equal(pick[sure], torch.tensor(outs[k])[sure]), k
        assert int(sure.sum()) >= 6
    assert eng.kv.num_free() == eng.kv.num_blocks


def test_registry_and_config_roundtrip(tmp_path):
    from dynamo_exp_amd.models.config import get_config
    from dynamo_exp_amd.models.registry import MODEL_REGISTRY, build_model, supports_dtype

    cfg = CONFIGS["mixed"]()
    cfg.write_hf_config(str(tmp_path))
    back = get_config(str(tmp_path))
    assert isinstance(back, LayeredConfig) and back.layers == cfg.layers and back.loop == cfg.loop
    assert back.layer_runs() == [0, 1, 0, 1, 2, 3] and back.streams == 3
    assert "Bekulix" in MODEL_REGISTRY and supports_dtype("Bekulix", "float32")
    assert not supports_dtype("LlamaForCausalLM", "float32")
    m = build_model(back, "cpu", dtype="float32")
    assert isinstance(m, BekulixForCausalLM)
    from safetensors.torch import save_file

    sd = weights(cfg, 1)
    save_file({k: v.contiguous() for k, v in sd.items()}, str(tmp_path / "model.safetensors"))
    m.load_safetensors(str(tmp_path))
    assert len(m.layers) == 4 and len(m.cache_widths()) == 6
