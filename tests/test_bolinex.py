"""Bolinex in the engine against the plain oracle (tests/bolinex_oracle.py).

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

import bolinex_oracle as O
from dynamo_exp_amd.engine.engine import EngineConfig, LLMEngine
from dynamo_exp_amd.engine.request import SamplingParams
from dynamo_exp_amd.models.bolinex import BolinexForCausalLM
from dynamo_exp_amd.models.config import LayeredConfig
from dynamo_exp_amd.ops import mixers as mx
from dynamo_exp_amd.ops import moe

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
CASES = [("cpu", "float32"), pytest.param("cuda", "float32", marks=pytest.mark.gpu),
         pytest.param("cuda", "bfloat16", marks=pytest.mark.gpu)]
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
F64 = torch.float64


# ----------------------------------------------------------------- configurations
def mixer(H=6, G=3, d=20, dv=12, window=9, cap=5.0, v_mix=True):
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": d ** -0.5, "v_mix": v_mix}
    if window:
        m["mask"] = {"size": window}
    if cap:
        m["softcap"] = cap
    return m


def dense(ff=56):
    return {"kind": "dense", "ff": ff}


def experts(E=8, top=2, ff=24, groups=(4, 2), shared=40):
    r = {"experts": E, "top": top}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": r, "shared": {"ff": shared} if shared else None}


def layer(m, mlp):
    return {"type": "attention", "mixer": m, "mlp": mlp}


def config(layers, width=72, vocab=97, side=6, maxpos=256, eps=1e-5):
    return LayeredConfig(name="t", architecture="Bolinex", vocab_size=vocab, hidden_size=width, layers=layers,
                         rms_norm_eps=eps, token_side={"dim": side} if side else None, learned_positions=True,
                         max_position_embeddings=maxpos)


def cfg_dict(cfg: LayeredConfig) -> dict:
    d = {"layers": cfg.layers, "norm": {"eps": cfg.rms_norm_eps}, "vocab": cfg.vocab_size, "width": cfg.hidden_size}
    if cfg.token_side:
        d["token_side"] = cfg.token_side
    return d


CONFIGS = {
    # dense and routed feed-forwards, a layer without one; the first layer takes no part in value
    # mixing, so the values mixed in are layer 1's; windows differ per layer; q/k width != value width
    "mixed": lambda: config([layer(mixer(v_mix=False, window=5), dense()),
                             layer(mixer(H=6, G=2, d=12, dv=18, window=9), experts()),
                             layer(mixer(H=4, G=2, d=8, dv=18, window=30, cap=0), None),
                             layer(mixer(H=4, G=2, d=16, dv=18, window=17), experts(E=6, top=3, groups=(2, 1), ff=20))]),
    # values a model may happen to make equal or one: one head, one expert per group, every group
    # kept, one choice, a window of one token, no shared expert, a side input one column wide
    "ones": lambda: config([layer(mixer(H=1, G=1, d=8, dv=8, window=1), experts(E=4, top=1, groups=(4, 4), shared=0)),
                            layer(mixer(H=2, G=2, d=8, dv=4, window=2, v_mix=False), experts(E=3, top=1, groups=None, ff=8)),
                            layer(mixer(H=2, G=1, d=8, dv=8, window=64), dense(8))], width=32, side=1),
    # nothing divides by 4 or 8 (scalar paths), no window in one layer (plain causal), no side input
    "odd": lambda: config([layer(mixer(H=4, G=2, d=18, dv=7, window=0), dense(50)),
                           layer(mixer(H=2, G=2, d=6, dv=7, window=7, cap=2.0), experts(E=5, top=2, groups=None, ff=10,
                                                                                       shared=6))],
                          width=102, vocab=101, side=0),
    # head widths the matrix-core kernels serve (bf16 on the GPU)
    "tiles": lambda: config([layer(mixer(H=4, G=2, d=32, dv=32, window=20, v_mix=False), dense(64)),
                             layer(mixer(H=2, G=1, d=64, dv=64, window=70), experts(E=8, top=2, ff=32, shared=32)),
                             layer(mixer(H=4, G=2, d=48, dv=96, window=33, v_mix=False), dense(64)),
                             layer(mixer(H=2, G=1, d=64, dv=64, window=0, cap=0), None)], width=64, side=8),
    # expert shapes the 256-tile grouped GEMM serves in bf16 on the GPU (fused SwiGLU epilogue)
    "wide": lambda: config([layer(mixer(H=4, G=2, d=32, dv=32, window=40), experts(E=4, top=2, groups=(2, 1), ff=128,
                                                                                   shared=64)),
                            layer(mixer(H=4, G=2, d=32, dv=32, window=12), dense(96))], width=256, side=0),
}


def weights(cfg, seed=0):
    return BolinexForCausalLM(cfg, "cpu", torch.float32).random_state(seed)


def engine(cfg, sd, device, dtype, blocks=48, bs=8, graphs=False, seqs=4):
    model = BolinexForCausalLM(cfg, device, DT[dtype]).load_state(sd)
    return LLMEngine(EngineConfig(model="t", device=device, dtype=dtype, block_size=bs, num_gpu_blocks=blocks,
                                  max_model_len=blocks * bs, max_num_seqs=seqs, enable_prefix_caching=False,
                                  use_cuda_graph=graphs, graph_sizes=(1, 2, 4), async_schedule=False),
                     model_cfg=cfg, model=model)


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def oracle(cfg, sd, toks):
    """(logits, sure): the oracle's logits, and per position whether every expert choice there is
    clear of a close call (bf16 rounding of the router's input may decide a closer one otherwise)."""
    gaps = []
    lg = O.forward(cfg_dict(cfg), sd, toks, margin=gaps)
    sure = torch.stack(gaps).min(0).values > 0.03 if gaps else torch.ones(len(toks), dtype=torch.bool)
    return lg, sure


def close(got, want, dtype, what="", sure=None):
    """Logit rows agree: error relative to the rows' spread, after the mean is taken off.  In
    bfloat16, rows of a close expert choice (`sure` false) are left out; they stay a minority."""
    got = got.detach().double().cpu()
    want = want.double()
    a, b = got - got.mean(-1, keepdim=True), want - want.mean(-1, keepdim=True)
    err = ((a - b) ** 2).mean(-1).sqrt() / b.pow(2).mean().sqrt()
    lim = 2e-4 if dtype == "float32" else 5e-2
    if dtype != "float32" and sure is not None:
        assert float(sure.float().mean()) > 0.6 or len(sure) < 8, f"{what}: too few rows with a clear expert choice"
        err = torch.where(sure, err, torch.zeros_like(err))
    assert float(err.max()) < lim, f"{what}: error {float(err.max()):.3g} at row {int(err.argmax())} (limit {lim})"


def run_cut(eng, rid, toks, cuts):
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
@pytest.mark.parametrize("W", [70, 72, 2052, 8200])
def test_residual_step_alone(device, W):
    torch.manual_seed(W)
    T, eps = 5, 1e-5
    X = torch.randn(T, W) * 2 + 0.5
    a, b, c = torch.randn(T, W), torch.randn(T, W), torch.randn(T, W) * 3
    cw, nw, nb = torch.randn(W), torch.randn(W), torch.randn(W)
    want_x = X.double() + a.double() + b.double() + O.unit_rms(c.double(), eps) * cw.double()
    d = lambda t: t.to(device)  # noqa: E731
    Xd = d(X).clone()
    h, xc = mx.residual_step(Xd, d(a), d(b), d(c), d(cw), eps, "layer", d(nw), d(nb), torch.float32, want_cast=True)
    assert torch.allclose(Xd.cpu().double(), want_x, atol=2e-5)
    assert torch.allclose(xc.cpu().double(), want_x, atol=2e-5)
    assert torch.allclose(h.cpu().double(), O.layer_norm(want_x, nw.double(), nb.double(), eps), atol=5e-5)
    # one addend, RMS norm; then no addend (the norm alone), then the update alone
    Xd = d(X).clone()
    h, xc = mx.residual_step(Xd, None, d(b), eps=eps, norm="rms", norm_w=d(nw), out_dtype=torch.float32)
    assert xc is None
    assert torch.allclose(h.cpu().double(), O.unit_rms(X.double() + b.double(), eps) * nw.double(), atol=5e-5)
    h2, _ = mx.residual_step(Xd, eps=eps, norm="rms", norm_w=d(nw), out_dtype=torch.float32)
    assert torch.allclose(h2, h, atol=1e-6)
    h3, _ = mx.residual_step(Xd, c=d(c), c_w=d(cw), eps=eps, out_dtype=torch.float32)
    assert h3 is None
    assert torch.allclose(Xd.cpu().double(), X.double() + b.double() + O.unit_rms(c.double(), eps) * cw.double(),
                          atol=2e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("act", ["relu", "silu", "gelu_tanh", "sigmoid", "relu2"])
def test_act_mul_alone(device, act):
    torch.manual_seed(1)
    x = torch.randn(7, 120)
    g = x[:, 3:40].double()
    f = {"relu": torch.relu(g), "silu": g * torch.sigmoid(g), "gelu_tanh": O.gelu_tanh(g), "sigmoid": torch.sigmoid(g),
         "relu2": torch.relu(g) ** 2}[act]
    xd = x.to(device)
    # sections of a wider row, not aligned to 16 bytes; then aligned ones; then no multiplier
    assert torch.allclose(mx.act_mul(xd[:, 3:40], xd[:, 50:87], act).cpu().double(), f * x[:, 50:87].double(), atol=1e-5)
    g2 = x[:, 8:48].double()
    f2 = mx._act(g2, act)
    assert torch.allclose(mx.act_mul(xd[:, 8:48], xd[:, 64:104], act).cpu().double(), f2 * x[:, 64:104].double(), atol=1e-5)
    assert torch.allclose(mx.act_mul(xd[:, 3:40], None, act).cpu().double(), f, atol=1e-5)
    assert torch.allclose(mx.glu_act(xd, act).cpu().double(), mx._act(x[:, :60].double(), act) * x[:, 60:].double(),
                          atol=1e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_embed_positions_and_gather(device):
    torch.manual_seed(2)
    table, ptab = torch.randn(11, 30), torch.randn(40, 30)
    ids = torch.tensor([3, 0, 10, 3, 7])
    pos = torch.tensor([0, 39, 5, 6, 1])
    X = mx.embed_streams(ids.to(device), table.to(device), 1, ptab.to(device), pos.to(device))
    assert torch.allclose(X.cpu()[:, 0], table[ids] + ptab[pos], atol=1e-6)
    X = mx.embed_streams(ids.to(device), table.to(device), 2)
    assert torch.equal(X.cpu()[:, 1], table[ids])
    assert torch.equal(mx.gather_rows(table.to(device), ids.to(device)).cpu(), table[ids])


def paged(T, bs, n_blocks, width, device, dtype=torch.float32, seed=0):
    """A shuffled block table for one sequence of T tokens, and empty caches."""
    g = torch.Generator().manual_seed(seed)
    nb = -(-T // bs)
    table = torch.randperm(n_blocks, generator=g)[:nb].to(torch.int32)
    j = torch.arange(T)
    slots = table.long()[j // bs] * bs + j % bs
    return table[None].to(device), slots.to(device), torch.zeros(n_blocks * bs, width, dtype=dtype, device=device)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("G,d,dv", [(2, 10, 7), (2, 8, 12)])
def test_value_mix_into_cache(device, G, d, dv):
    torch.manual_seed(3)
    T, H = 9, 4
    x = torch.randn(T, (H + G) * d + G * dv + 5)
    first = torch.randn(T, 3 + G * dv)
    table, slots, kc = paged(T, 4, 6, G * d, device)
    vc = torch.zeros(6 * 4, G * dv, device=device)
    slots[4] = -1  # a row that caches nothing
    xd = x.to(device).clone()
    v_off = (H + G) * d
    mx.headprep_cache(xd, torch.arange(T, device=device), slots, 0, G, d, H * d, None, None, 1e-5, None, kc, vc,
                      v_mode=2, v_off=v_off, v_w=G * dv, v_first=first.to(device)[:, 3:], v_lambda=0.3)
    ok = slots.cpu() >= 0
    want = O.value_mix(x[:, v_off:v_off + G * dv].double(), first[:, 3:].double(), 0.3)
    assert torch.allclose(vc[slots[ok.to(device)]].cpu().double(), want[ok], atol=1e-6)
    assert torch.equal(kc[slots[ok.to(device)]].cpu(), x[ok, H * d:(H + G) * d])
    assert torch.equal(xd.cpu(), x)  # queries, keys and values as projected stay in place
    assert float(vc.abs().sum(1).ne(0).sum()) == T - 1


def dense_attention(q, k, v, scale, cap, r1, r2, size):
    """Oracle attention of one sequence: q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv]."""
    T, H = q.shape[:2]
    rep = H // k.shape[1]
    s = O.scores(q.double(), k.double().repeat_interleave(rep, 1), scale, cap,
                 None if r1 is None else r1.double(), None if r2 is None else r2.double())
    return O.attend(s, v.double().repeat_interleave(rep, 1), O.window_mask(T, size or None))


TERMS = [(0.0, False, 0), (4.0, False, 6), (0.0, True, 70), (3.0, True, 9), (50.0, True, 1), (3.0, True, 0)]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cap,bias,size", TERMS)
@pytest.mark.parametrize("dims", [(4, 2, 20, 12), (3, 3, 8, 136), (4, 1, 12, 72)])
def test_row_attention_score_terms(device, cap, bias, size, dims):
    """Prompt rows over a shuffled page table against the dense oracle with the tanh
    cap and the distance penalty; then rows as decode rows, keys split in parts."""
    H, G, d, dv = dims
    T, bs = 70, 8
    torch.manual_seed(7)
    q, k, v = torch.randn(T, H, d) * 2, torch.randn(T, G, d) * 2, torch.randn(T, G, dv)
    r1 = torch.rand(H) * 2 if bias else None
    r2 = torch.rand(H) + 0.01 if bias else None
    want = dense_attention(q, k, v, 0.4, cap, r1, r2, size)
    table, slots, kc = paged(T, bs, 12, G * d, device)
    vc = torch.zeros(12 * bs, G * dv, device=device)
    kc[slots] = k.reshape(T, -1).to(device)
    vc[slots] = v.reshape(T, -1).to(device)
    pos = torch.arange(T, device=device)
    seq = torch.zeros(T, dtype=torch.int32, device=device)
    qd = q.reshape(T, -1).to(device)
    db = (r1.to(device), r2.to(device)) if bias else None
    mask = "window" if size else "causal"
    got = mx.row_attention(qd, kc, vc, pos, seq, table, bs, H, 1, H // G, d, dv, 0.4, mask, size, 1, False, cap, db)
    assert torch.allclose(got.cpu().double(), want, atol=3e-5)
    rows = torch.tensor([0, 1, 7, 8, 33, 69], device=device)
    got = mx.row_attention(qd[rows], kc, vc, pos[rows], None, table.expand(len(rows), -1).contiguous(), bs, H, 1,
                           H // G, d, dv, 0.4, mask, size, 2, False, cap, db)
    assert torch.allclose(got.cpu().double(), want[rows.cpu()], atol=3e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("cap,bias,size", TERMS)
@pytest.mark.parametrize("dims", [(4, 2, 32, 32), (6, 2, 48, 48), (2, 2, 48, 96), (3, 1, 64, 64), (4, 4, 128, 128),
                                  (20, 1, 64, 64)])
def test_matrix_core_attention_score_terms(cap, bias, size, dims):
    """The matrix-core kernels with score terms: a 263-row portion that starts at
    position 37 of a cached prefix (three tiles, the last ragged, cut inside pages
    and windows) beside two decode rows of another sequence, then decode rows
    alone, against the dense oracle over the bf16 values."""
    H, G, d, dv = dims
    T, bs, start = 300, 16, 37
    torch.manual_seed(5)
    q = torch.randn(T, H, d).bfloat16()
    k = (torch.randn(T, G, d) * 0.7).bfloat16()
    v = torch.randn(T, G, dv).bfloat16()
    r1 = torch.rand(H) * 2 if bias else None
    r2 = torch.rand(H) + 0.01 if bias else None
    want = dense_attention(q, k, v, 0.2, cap, r1, r2, size)
    perm = torch.randperm(40, generator=torch.Generator().manual_seed(3)).to(torch.int32)
    table = torch.stack([perm[:19], perm[19:38]]).contiguous().cuda()
    j = torch.arange(T, device="cuda")
    kc = torch.zeros(40 * bs, G * d, device="cuda", dtype=torch.bfloat16)
    vc = torch.zeros(40 * bs, G * dv, device="cuda", dtype=torch.bfloat16)
    for i in (0, 1):
        sl = table[i].long()[j // bs] * bs + j % bs
        kc[sl] = k.reshape(T, -1).cuda()
        vc[sl] = v.reshape(T, -1).cuda()
    rows = list(range(start, T)) + [5, 290]
    n_pre = T - start
    pos = torch.tensor(rows, device="cuda")
    seq = torch.tensor([0] * n_pre + [1, 1], dtype=torch.int32, device="cuda")
    tiles = torch.tensor(mx.tile_list(0, n_pre), dtype=torch.int32, device="cuda")
    qd = q.reshape(T, -1).cuda()[pos]
    db = (r1.cuda(), r2.cuda()) if bias else None
    mask = "window" if size else "causal"
    assert mx.tile_attention_ok(qd, d, dv)
    got = mx.attention(qd, kc, vc, pos, seq, table, bs, H, 1, H // G, d, dv, 0.2, mask, size, 1, True, tiles, n_pre,
                       softcap=cap, dist_bias=db)
    assert float((got.cpu().double() - want[rows]).abs().max()) < 4e-4
    got = mx.attention(qd, kc, vc, pos, seq, table, bs, H, 1, H // G, d, dv, 0.2, mask, size, 3, False, tiles, n_pre,
                       softcap=cap, dist_bias=db)
    assert float((got.cpu().double() - want[rows]).abs().max()) < 3e-2
    dr = torch.tensor([0, 1, 63, 64, 65, 255, 299], device="cuda")
    got = mx.attention(q.reshape(T, -1).cuda()[dr], kc, vc, dr, None, table[:1].expand(len(dr), -1).contiguous(), bs,
                       H, 1, H // G, d, dv, 0.2, mask, size, 2, True, softcap=cap, dist_bias=db)
    assert float((got.cpu().double() - want[dr.cpu()]).abs().max()) < 4e-4


# ----------------------------------------------------------------- crafted keys
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("decode", [False, True])
def test_one_key_stands_out(device, dtype, decode):
    """A query that matches exactly one key by a wide margin -- also after the cap
    and the distance penalty -- returns that key's value if and only if the window
    lets it through: far keys among hundreds, page borders, one position inside
    and outside the window."""
    T, d, dv, bs = 300, 16, 48 if dtype == "bfloat16" else 24, 16
    dt = DT[dtype]
    torch.manual_seed(11)
    k = torch.randn(T, d) * 0.1
    v = torch.randn(T, dv).to(dt)
    table, slots, kc = paged(T, bs, 24, d, device, dt)
    vc = torch.zeros(24 * bs, dv, device=device, dtype=dt)
    vc[slots] = v.to(device)
    p = T - 1
    r1 = torch.tensor([0.5], device=device)
    r2 = torch.tensor([1.0], device=device)
    cases = [(0, 3, True), (0, 0, True), (0, bs - 1, True), (0, bs, True), (40, p - 39, True), (40, p - 40, False),
             (40, p, True), (1, p, True), (1, p - 1, False), (299, 1, True), (299, 0, False), (300, 0, True)]
    for size, j, seen in cases:
        kk = k.clone()
        kk[j] = 0
        kk[j, 0] = 40.0
        kc[slots] = kk.to(device, dt)
        q = torch.zeros(1, d)
        q[0, 0] = 1.0
        pos = torch.tensor([p], device=device)
        seq = None if decode else torch.zeros(1, dtype=torch.int32, device=device)
        tiles = None if decode else torch.tensor([[0, 1]], dtype=torch.int32, device=device)
        got = mx.attention(q.to(device, dt), kc, vc, pos, seq, table, bs, 1, 1, 1, d, dv, 1.0,
                           "window" if size else "causal", size, 3 if decode else 1, True, tiles, 0 if decode else 1,
                           softcap=30.0, dist_bias=(r1, r2)).cpu()[0, 0]
        hit = torch.allclose(got, v[j].float(), atol=2e-3)
        assert hit == seen, f"window {size}: key {j} from position {p} seen={hit}, expected {seen}"


# ----------------------------------------------------------------- routed experts
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,top,groups", [(8, 2, (4, 2)), (12, 3, (3, 1)), (6, 1, (6, 6)), (5, 2, None), (64, 6, (8, 3)),
                                          (130, 4, (2, 2)), (4, 4, (2, 2))])
def test_route_alone(device, E, top, groups):
    """Choice by corrected scores inside the best groups, weights without the
    correction.  Corrections reach below -1, so choice scores are negative and a
    dropped group must count as minus infinity, not as zero."""
    torch.manual_seed(E)
    T = 37
    z = (torch.randperm(T * E).float() / (T * E) * 8 - 4).view(T, E)  # no two scores within rounding of each other
    corr = torch.randn(E) * 0.5 - 1.2
    gd = {"count": groups[0], "keep": groups[1]} if groups else None
    idx, w = O.route(z.double(), corr.double(), top, gd)
    n, keep = groups or (1, 1)
    gi, gw = moe.route(z.to(device), corr.to(device), top, n, keep)
    assert torch.equal(gi.cpu().long(), idx)
    assert torch.allclose(gw.cpu().double(), w, atol=1e-6)
    gi, gw = moe.route(z.to(device), None, top, n, keep)
    idx, w = O.route(z.double(), torch.zeros(E, dtype=F64), top, gd)
    assert torch.equal(gi.cpu().long(), idx)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("T,E,top", [(26000, 5, 2), (50, 300, 3), (8192, 8, 2), (1, 1, 1)])
def test_plan_sizes(device, T, E, top):
    """More slots than the kernel stages in LDS, more experts than a byte counts, a usual prompt step."""
    g = torch.Generator().manual_seed(T)
    idx = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(min(T, 64))]).to(torch.int32)
    idx = idx.repeat(-(-T // idx.shape[0]), 1)[:T].contiguous()
    idx[::7] = idx[::7].flip(1)
    order, offsets = moe.plan(idx.to(device), E)
    flat = idx.reshape(-1).long()
    assert torch.equal(order.cpu().long(), torch.sort(flat, stable=True).indices)
    assert offsets.cpu().tolist() == [0] + torch.bincount(flat, minlength=E).cumsum(0).tolist()


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("T,E,top,K,N", [(1, 3, 1, 16, 8), (37, 5, 2, 70, 33), (150, 4, 3, 96, 130), (70, 16, 1, 64, 64)])
def test_plan_grouped_gemm_combine(device, dtype, T, E, top, K, N):
    """The plan is a stable sort of the slots by expert; grouped GEMMs (gathered
    token rows in, sorted rows out; sorted rows in, slot rows out) against one
    dense product per slot; the combine against the weighted sum."""
    torch.manual_seed(T + E)
    dt = DT[dtype]
    idx = torch.stack([torch.randperm(E)[:top] for _ in range(T)]).to(torch.int32)
    if T > 40:
        idx[idx == 1] = 0  # an expert without rows (E > 1), another with many
    order, offsets = moe.plan(idx.to(device), E)
    flat = idx.reshape(-1).long()
    assert torch.equal(order.cpu().long(), torch.sort(flat, stable=True).indices)
    assert offsets.cpu().tolist() == [0] + torch.bincount(flat, minlength=E).cumsum(0).tolist()
    a = torch.randn(T, K).to(dt)
    w1 = (torch.randn(E, N, K) * K ** -0.5).to(dt)
    w2 = (torch.randn(E, K, N) * N ** -0.5).to(dt)
    tol = 1e-4 if dtype == "float32" else 3e-2
    y1 = moe.grouped_gemm(a.to(device), w1.to(device), order, offsets, top, gather=True, scatter=False)
    o = order.cpu().long()
    want1 = torch.stack([a[s // top].double() @ w1[flat[s]].double().t() for s in o.tolist()])
    assert float((y1.cpu().double() - want1).abs().max()) < tol
    y2 = moe.grouped_gemm(y1, w2.to(device), order, offsets, top, gather=False, scatter=True)
    want2 = torch.empty(T * top, K, dtype=F64)
    want2[o] = torch.stack([y1.cpu()[r].double() @ w2[flat[s]].double().t() for r, s in enumerate(o.tolist())])
    assert float((y2.cpu().double() - want2).abs().max()) < tol
    wgt = torch.rand(T, top)
    sh = torch.randn(T, K).to(dt)
    got = moe.combine(y2, wgt.to(device), sh.to(device))
    want = (y2.cpu().double().view(T, top, K) * wgt.double()[:, :, None]).sum(1) + sh.double()
    assert float((got.cpu().double() - want).abs().max()) < tol
    got = moe.combine(y2, wgt.to(device), None)
    assert float((got.cpu().double() - (want - sh.double())).abs().max()) < tol


@pytest.mark.gpu
@pytest.mark.parametrize("T,E,top,K,N", [(300, 4, 2, 256, 512), (3, 8, 2, 128, 256), (700, 3, 1, 384, 256)])
def test_grouped_gemm_on_the_256_tile_kernel(T, E, top, K, N):
    """Shapes the 256 x 256-tile GEMM serves in grouped mode (bf16, N % 256 == 0, K % 128 == 0):
    gathered rows in, scattered rows out, experts without rows, row tiles that end inside a
    tile, and the SwiGLU epilogue over interleaved gate / up rows."""
    torch.manual_seed(T)
    idx = torch.stack([torch.randperm(E)[:top] for _ in range(T)]).to(torch.int32)
    if E > 2:
        idx[idx == 1] = 0 if top == 1 else idx[idx == 1]  # top 1: expert 1 gets no rows
    order, offsets = moe.plan(idx.cuda(), E)
    flat, o = idx.reshape(-1).long(), order.cpu().long()
    a = torch.randn(T, K).bfloat16()
    w1 = (torch.randn(E, N, K) * K ** -0.5).bfloat16()
    assert moe.tile_gemm_ok(a.cuda(), w1.cuda())
    y1 = moe.grouped_gemm(a.cuda(), w1.cuda(), order, offsets, top, gather=True, scatter=False)
    want1 = torch.stack([a[s // top].double() @ w1[flat[s]].double().t() for s in o.tolist()])
    assert float((y1.cpu().double() - want1).abs().max()) < 3e-2
    g, u = want1[:, :N // 2], want1[:, N // 2:]
    y1g = moe.grouped_gemm(a.cuda(), moe.interleave_glu(w1.cuda()), order, offsets, top, gather=True, scatter=False,
                           glu=True)
    assert float((y1g.cpu().double() - g * torch.sigmoid(g) * u).abs().max()) < 3e-2
    w2 = (torch.randn(E, N, K) * K ** -0.5).bfloat16()
    b = torch.randn(T * top, K).bfloat16()  # rows already in sorted order
    y2 = moe.grouped_gemm(b.cuda(), w2.cuda(), order, offsets, top, gather=False, scatter=True)
    want2 = torch.empty(T * top, N, dtype=F64)
    want2[o] = torch.stack([b[r].double() @ w2[flat[s]].double().t() for r, s in enumerate(o.tolist())])
    assert float((y2.cpu().double() - want2).abs().max()) < 3e-2


# ----------------------------------------------------------------- the model in the engine
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_and_layers(device, dtype, name):
    cfg = CONFIGS[name]()
    sd = weights(cfg, 1)
    toks = tokens(45, cfg.vocab_size, 2)
    want, layers = O.forward(cfg_dict(cfg), sd, toks, return_layers=True)
    sure = oracle(cfg, sd, toks)[1]
    eng = engine(cfg, sd, device, dtype)
    eng.model.trace_layers = []
    got = eng.forced_step([("a", toks, list(range(len(toks))))], ["a"])["a"]
    close(got, want, dtype, name, sure)
    assert len(eng.model.trace_layers) == len(cfg.layers) == layers.shape[0]
    tol = 1e-3 if dtype == "float32" else 0.25
    rows = sure if dtype != "float32" else torch.ones_like(sure)
    for i, x in enumerate(eng.model.trace_layers):
        assert float((x.cpu().double() - layers[i])[rows].abs().max()) < tol * max(1.0, float(layers[i].abs().max())), i
    assert eng.kv.num_free() == eng.kv.num_blocks
    eng.model.trace_layers = None  # the fused path (norms joined with the residual steps) gives the same
    close(eng.forced_step([("b", toks, list(range(len(toks))))], ["b"])["b"], want, dtype, name + " fused", sure)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_token_by_token_and_portions(device, dtype, name):
    """Prefill against one-token steps and against portions of several sizes
    (down to two tokens, cut inside pages and windows), long enough that every
    window passes over decoded tokens."""
    cfg = CONFIGS[name]()
    sd = weights(cfg, 3)
    toks = tokens(52, cfg.vocab_size, 4)
    want, sure = oracle(cfg, sd, toks)
    eng = engine(cfg, sd, device, dtype)
    close(run_cut(eng, "one", toks, []), want, dtype, "token by token", sure)
    close(run_cut(eng, "cut", toks, [2, 3, 2, 11, 7, 2, 9]), want, dtype, "portions", sure)
    close(run_cut(eng, "pre", toks, [17]), want, dtype, "prefill then decode", sure)
    assert eng.kv.num_free() == eng.kv.num_blocks


@pytest.mark.parametrize("device,dtype", CASES)
def test_mixed_batches_and_reused_pages(device, dtype):
    """Unequal requests interleaved (portions beside single tokens, a request left
    out of steps) in a pool that only fits them because finished requests give
    their pages back; every request equals itself alone."""
    cfg = CONFIGS["mixed"]()
    sd = weights(cfg, 5)
    lens = {"a": 37, "b": 9, "c": 23, "d": 1, "e": 30, "f": 18}
    toks = {k: tokens(n, cfg.vocab_size, 10 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: oracle(cfg, sd, t) for k, t in toks.items()}
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
        close(torch.cat(got[k], 0), want[k][0], dtype, f"request {k}", want[k][1] if lens[k] > 9 else None)
    assert eng.kv.num_free() == eng.kv.num_blocks


@pytest.mark.parametrize("device,dtype", CASES)
def test_first_tokens_and_long_decoding(device, dtype):
    cfg = config([layer(mixer(H=2, G=1, d=8, dv=8, window=24), dense(16)),
                  layer(mixer(H=2, G=1, d=4, dv=8, window=100), experts(E=4, top=2, groups=(2, 1), ff=8, shared=8))],
                 width=32, side=4)
    sd = weights(cfg, 6)
    toks = tokens(150, cfg.vocab_size, 7)
    want, sure = oracle(cfg, sd, toks)
    eng = engine(cfg, sd, device, dtype, blocks=40, bs=4)
    got = run_cut(eng, "r", toks, [1, 1, 2])  # positions 0, 1, then a portion, then 146 decode steps
    close(got, want, dtype, "long decoding", sure)


@pytest.mark.parametrize("device,dtype", CASES)
def test_window_edge_and_far_key_show_in_logits(device, dtype):
    """Weights made so that faults cannot hide: a strong attention output, a window
    whose edge moves the logits (the oracle with a window one token off differs
    visibly), value mixing whose weight matters, and a router without its
    correction would choose other experts."""
    cfg = config([layer(mixer(H=2, G=1, d=8, dv=8, window=6, cap=0), None),
                  layer(mixer(H=2, G=1, d=8, dv=8, window=11), experts(E=6, top=2, groups=(3, 2), ff=8, shared=0))],
                 width=32, side=0)
    sd = weights(cfg, 8)
    for i in (0, 1):
        sd[f"l{i}.mix.o"] = sd[f"l{i}.mix.o"] * 4
        sd[f"l{i}.mix.q"] = sd[f"l{i}.mix.q"] * 3
    sd["l1.mlp.correction"] = sd["l1.mlp.correction"] * 3
    toks = tokens(30, cfg.vocab_size, 9)
    base = cfg_dict(cfg)
    want = O.forward(base, sd, toks)

    def changed(**kw):
        d = dict(base)
        d["layers"] = [dict(L, mixer=dict(L["mixer"])) for L in base["layers"]]
        sd2 = dict(sd)
        if "window" in kw:
            d["layers"][0]["mixer"]["mask"] = {"size": kw["window"]}
        if "lam" in kw:
            sd2["l1.mix.vmix"] = torch.tensor(kw["lam"])
        if "corr" in kw:
            sd2["l1.mlp.correction"] = sd["l1.mlp.correction"] * 0
        return float((O.forward(d, sd2, toks) - want).abs().max())

    assert changed(window=7) > 1e-2 and changed(window=5) > 1e-2
    assert changed(lam=0.0) > 1e-2 and changed(corr=0) > 1e-2
    eng = engine(cfg, sd, device, dtype)
    close(run_cut(eng, "r", toks, [13, 2]), want, dtype, "edges", oracle(cfg, sd, toks)[1])


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


@pytest.mark.parametrize("device,dtype", CASES)
def test_trace_replay_command(tmp_path, monkeypatch, capsys, device, dtype):
    """The replay command on a checkpoint directory: the class follows config.json, the pool holds
    exactly the two live requests' pages, a portion beside a shorter one, a decode token beside a
    portion, a step in which nothing is wanted; logits files against the oracle."""
    import io
    import sys

    import numpy as np
    from safetensors.torch import save_file

    from dynamo_exp_amd.cli import trace_run

    cfg = CONFIGS["mixed"]()
    sd = weights(cfg, 21)
    model_dir, out = tmp_path / "m", tmp_path / "out"
    cfg.write_hf_config(str(model_dir))
    save_file({k: v.contiguous() for k, v in sd.items()}, str(model_dir / "model.safetensors"))
    a, b = tokens(40, cfg.vocab_size, 31), tokens(9, cfg.vocab_size, 32)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:25], "want": [0, 24]},
                                     {"id": "b", "tokens": b[:2], "want": [1]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[25:26], "want": [0]},
                                     {"id": "b", "tokens": b[2:], "want": [0, 6]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[26:], "want": []}], "end": ["a"]},
             {"step": 3, "entries": [{"id": "c", "tokens": b, "want": [8]}], "end": ["c"]}]
    import json

    monkeypatch.setattr(sys, "stdin", io.StringIO("\n".join(json.dumps(st) for st in steps) + "\n"))
    rc = trace_run.main(["--model", str(model_dir), "--dtype", dtype, "--out", str(out), "--max-tokens", "128",
                         "--device", device])
    assert rc == 0
    assert [ln for ln in capsys.readouterr().out.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(4)]
    assert not (out / "2.f32").exists()
    wa, sa = oracle(cfg, sd, a)
    wb, sb = oracle(cfg, sd, b)
    got = {i: torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, cfg.vocab_size)) for i in (0, 1, 3)}
    close(got[0], torch.cat([wa[[0, 24]], wb[[1]]]), dtype, "step 0", torch.cat([sa[[0, 24]], sb[[1]]]))
    close(got[1], torch.cat([wa[[25]], wb[[2, 8]]]), dtype, "step 1", torch.cat([sa[[25]], sb[[2, 8]]]))
    close(got[3], wb[[8]], dtype, "step 3", sb[[8]])


def test_registry_and_config_roundtrip(tmp_path):
    from dynamo_exp_amd.models.config import PRESETS, get_config
    from dynamo_exp_amd.models.registry import MODEL_REGISTRY, build_model, supports_dtype

    cfg = CONFIGS["mixed"]()
    cfg.write_hf_config(str(tmp_path))
    back = get_config(str(tmp_path))
    assert isinstance(back, LayeredConfig) and back.architecture == "Bolinex" and back.layers == cfg.layers
    assert back.token_side == {"dim": 6} and back.learned_positions and back.max_position_embeddings == 256
    assert "Bolinex" in MODEL_REGISTRY and supports_dtype("Bolinex", "float32") and supports_dtype("Bolinex", "bfloat16")
    m = build_model(back, "cpu", dtype="float32")
    assert isinstance(m, BolinexForCausalLM)
    from safetensors.torch import save_file

    sd = weights(cfg, 1)
    save_file({k: v.contiguous() for k, v in sd.items()}, str(tmp_path / "model.safetensors"))
    m.load_safetensors(str(tmp_path))
    assert len(m.layers) == 4 and len(m.cache_widths()) == 4
    assert m.layers[0]["mix_from"] is None and m.layers[1]["mix_from"] is None and m.layers[2]["mix_from"] == 1
    n = sum(v.numel() for v in sd.values())
    assert back.num_params() == n
    assert PRESETS["bolinex-tiny"].architecture == "Bolinex" and PRESETS["bolinex-tiny"].num_params() > 0
    with pytest.raises(ValueError):
        BolinexForCausalLM(config([{"type": "latent_attention", "mixer": mixer(), "mlp": None}]), "cpu", torch.float32)
