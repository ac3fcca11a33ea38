"""Bolinex: a layer-listed decoder with parallel blocks for the MI355X engine.

A Bolinex checkpoint lists its layers.  Every layer is a parallel block: one
layer norm (weight and bias) feeds both a windowed attention mixer and a
feed-forward (dense, a routed mixture of experts, or none), and both outputs
join one fp32 residual.  Token embeddings get a learned vector per position,
and after each block a per-layer token input (a slice of a second embedding,
gated by the residual) is added with unit RMS.  Per layer, T rows of one
engine step (prompt chunks and decode tokens of different sequences):

    p  = h @ [Wq | Wk | Wv | Wg]^T          hipBLASLt, one fused projection
    headprep_cache(p)                       HIP  K to the paged cache; V mixed with the first
                                                 mixing layer's values of the same tokens, then cached
    a  = attention(q, K cache, V cache)     HIP  scores capped by tanh, a log-distance penalty per
                                                 head, sliding window; prompt chunks on the MFMA tile
                                                 kernel, decode rows on the grouped decode kernel
                                                 (fp32, odd head widths: the row kernel)
    ym = act_mul(g, a, sigmoid) @ Wo^T      HIP + hipBLASLt   output gate from the same input h
    yf = relu(h @ Wup^T)^2 @ Wdown^T        dense feed-forward, or
    yf = combine(experts(h), shared(h))     HIP  route -> plan -> grouped GEMMs over each expert's
                                                 tokens -> weighted sum (ops/moe.py)
    X += ym + yf; xa = cast(X)              HIP  residual_step
    y  = (gelu(xa @ Wsg^T) * e_tok) @ Wsp^T per-layer token input
    X += unit_rms(y) * ws; h = LN(X)        HIP  residual_step: the next layer's norm in the same pass

Scores, softmax, norms, router and the residual are fp32; projections and
activations are bf16 (dtype=bfloat16) or everything is fp32 (dtype=float32).
"""
from __future__ import annotations

import glob
import math
import os

import torch

from ..ops import mixers as mx
from ..ops import moe
from .config import LayeredConfig
from .gemm_tuning import planned_mm, tune_small_m
from .llama import AttnMeta, TPGroup

MLP_KINDS = ("dense", "moe")


class BolinexForCausalLM:
    #: the runner builds per-row sequence ids and one block table over all rows of a step
    unified_rows = True

    def __init__(self, cfg: LayeredConfig, device: torch.device | str = "cuda", dtype=torch.bfloat16,
                 tp: TPGroup | None = None):
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.tp = tp or TPGroup()
        if self.tp.size != 1:
            raise ValueError("Bolinex runs on one GPU per engine (tensor parallel size 1)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"unsupported dtype {dtype}")
        if cfg.loop or cfg.streams:
            raise ValueError("Bolinex has neither a layer loop nor parallel residual streams")
        vm = None
        for i, L in enumerate(cfg.layers):
            if L["type"] != "attention":
                raise ValueError(f"unknown mixer type {L['type']!r}")
            if L.get("mlp") and L["mlp"].get("kind") not in MLP_KINDS:
                raise ValueError(f"unknown feed-forward kind {L['mlp'].get('kind')!r}")
            m = L["mixer"]
            if m["heads"] % m["kv_heads"]:
                raise ValueError(f"layer {i}: {m['heads']} heads over {m['kv_heads']} key/value heads")
            if m.get("v_mix"):
                w = m["kv_heads"] * m["vdim"]
                if vm is not None and vm != w:
                    raise ValueError(f"layer {i}: value mixing needs the first mixing layer's value width {vm}, got {w}")
                vm = w
        self.side_dim = int((cfg.token_side or {}).get("dim", 0))
        self.layers: list[dict] = []
        self.embed = self.head = self.pos = self.side_embed = self.final_w = self.final_b = None
        self.fp8 = False
        self.kv_scales = (1.0, 1.0)
        self.kv_amax = None
        self.layer_hook = None
        self.gemm_plan: dict = {}
        self.gemm_tuned: set = set()
        # debugging: when a list, forward() appends the residual after every layer
        self.trace_layers: list | None = None

    # ------------------------------------------------------------------ engine hooks (no-ops here)
    def enable_fused_mlp(self) -> bool:
        return False

    def fold_norms(self) -> bool:
        return False

    #: dense projections of a layer, by the name of their weight
    LINEARS = ("w_in", "w_o", "w_up", "w_down", "w_sgu", "w_sdown", "side_gate", "side_proj")

    def tune_gemms(self, sizes, **kw) -> list:
        """Decode batch sizes: the hand-written small-M GEMMs where they beat the
        library (bf16 on the GPU; models/gemm_tuning.py)."""
        if self.device.type != "cuda" or self.dtype != torch.bfloat16 or not self.layers:
            return []
        groups = [[L[n] for L in self.layers if L.get(n) is not None] for n in self.LINEARS]
        return tune_small_m([g for g in groups if g], sizes, self.gemm_plan, self.gemm_tuned, **kw)

    def _mm(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        return planned_mm(self.gemm_plan, x, w)

    def tune_prefill_gemms(self, max_tokens, **kw) -> list:
        return []

    def quantize_fp8(self):
        raise ValueError("fp8 linears are not available for Bolinex")

    @torch.no_grad()
    def warmup_linears(self, tokens: int) -> None:
        """Run every distinct dense projection shape at M = tokens once (the
        GEMM library loads its kernels for the size before serving)."""
        seen = set()
        for L in self.layers:
            for name in self.LINEARS:
                w = L.get(name)
                if w is None or tuple(w.shape) in seen:
                    continue
                seen.add(tuple(w.shape))
                torch.matmul(torch.zeros(tokens, w.shape[1], device=self.device, dtype=self.dtype), w.t())

    def weight_bytes(self) -> int:
        ts = [t for L in self.layers for t in L.values() if isinstance(t, torch.Tensor)]
        ts += [t for t in (self.embed, self.head, self.pos, self.side_embed) if t is not None]
        return sum(t.numel() * t.element_size() for t in ts)

    # ------------------------------------------------------------------ paged caches
    def cache_widths(self) -> list[tuple[int, int]]:
        """(K row width, V row width) of every layer."""
        return [(L["mixer"]["kv_heads"] * L["mixer"]["dim"], L["mixer"]["kv_heads"] * L["mixer"]["vdim"])
                for L in self.cfg.layers]

    def kv_bytes_per_block(self, block_size: int, dtype: torch.dtype) -> int:
        es = torch.empty((), dtype=dtype).element_size()
        return sum((k + v) * block_size * es for k, v in self.cache_widths())

    def alloc_kv_caches(self, num_blocks: int, block_size: int, dtype: torch.dtype) -> list[tuple]:
        """One (K, V) pair per layer, token-major [num_blocks * block_size,
        width], indexed by the engine's one block table.  Windowed layers keep
        every page of a live sequence; the mask alone bounds what is read."""
        if dtype != self.dtype:
            raise ValueError(f"the cache holds the model's activation dtype {self.dtype}, not {dtype}")
        return [(torch.zeros((num_blocks * block_size, wk), dtype=dtype, device=self.device),
                 torch.zeros((num_blocks * block_size, wv), dtype=dtype, device=self.device))
                for wk, wv in self.cache_widths()]

    # ------------------------------------------------------------------ weights
    def random_state(self, seed: int = 0) -> dict[str, torch.Tensor]:
        """Random weights in the checkpoint's naming and dtypes (bf16), scaled
        so activations stay O(1)."""
        cfg = self.cfg
        g = torch.Generator().manual_seed(seed)
        W, nl, sdim = cfg.hidden_size, max(1, len(cfg.layers)), self.side_dim

        def rnd(*shape, std):
            return (torch.randn(*shape, generator=g) * std).to(torch.bfloat16)

        def gated(p, F, out_std):
            return {p + "gate": rnd(F, W, std=W ** -0.5), p + "up": rnd(F, W, std=W ** -0.5),
                    p + "down": rnd(W, F, std=out_std)}

        sd = {"embed": rnd(cfg.vocab_size, W, std=1.0), "final.norm": 1 + rnd(W, std=0.1),
              "final.norm.b": rnd(W, std=0.1), "head": rnd(cfg.vocab_size, W, std=W ** -0.5)}
        if cfg.learned_positions:
            sd["pos"] = rnd(cfg.max_position_embeddings, W, std=0.5)
        if sdim:
            sd["side.embed"] = rnd(cfg.vocab_size, sdim * len(cfg.layers), std=1.0)
        for i, L in enumerate(cfg.layers):
            m, p = L["mixer"], f"l{i}.mix."
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            sd[f"l{i}.norm1"], sd[f"l{i}.norm1.b"] = 1 + rnd(W, std=0.1), rnd(W, std=0.1)
            sd[p + "q"], sd[p + "k"] = rnd(H * d, W, std=W ** -0.5), rnd(G * d, W, std=W ** -0.5)
            sd[p + "v"], sd[p + "g"] = rnd(G * dv, W, std=W ** -0.5), rnd(H * dv, W, std=W ** -0.5)
            sd[p + "o"] = rnd(W, H * dv, std=(H * dv) ** -0.5 / math.sqrt(nl))
            sd[p + "r1"] = (torch.rand(H, generator=g) * 1.5).to(torch.bfloat16)
            sd[p + "r2"] = (0.05 + torch.rand(H, generator=g)).to(torch.bfloat16)
            sd[p + "vmix"] = (0.2 + 0.6 * torch.rand((), generator=g)).to(torch.bfloat16)
            mlp = L.get("mlp")
            q = f"l{i}.mlp."
            if mlp and mlp["kind"] == "dense":
                F = mlp["ff"]
                sd[q + "up"], sd[q + "down"] = rnd(F, W, std=W ** -0.5), rnd(W, F, std=F ** -0.5 / math.sqrt(nl))
            elif mlp:
                E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
                for e in range(E):
                    sd.update(gated(f"{q}e{e}.", F, 2.0 * F ** -0.5 / math.sqrt(nl)))
                sd[q + "router"] = rnd(E, W, std=2.0 * W ** -0.5)
                sd[q + "correction"] = rnd(E, std=0.3)
                if mlp.get("shared"):
                    Fs = mlp["shared"]["ff"]
                    sd.update(gated(q + "shared.", Fs, Fs ** -0.5 / math.sqrt(nl)))
            if sdim:
                sd[f"l{i}.side.gate"] = rnd(sdim, W, std=W ** -0.5)
                sd[f"l{i}.side.proj"] = rnd(W, sdim, std=sdim ** -0.5)
                sd[f"l{i}.side.norm"] = rnd(W, std=0.3 / math.sqrt(nl))
        return sd

    def random_init(self, seed: int = 0) -> "BolinexForCausalLM":
        return self.load_state(self.random_state(seed))

    def load_safetensors(self, path: str) -> "BolinexForCausalLM":
        from safetensors import safe_open

        files = sorted(glob.glob(os.path.join(path, "*.safetensors")))
        if not files:
            raise FileNotFoundError(f"no safetensors in {path}")
        tensors = {}
        for f in files:
            with safe_open(f, framework="pt", device="cpu") as sf:
                for k in sf.keys():
                    tensors[k] = sf.get_tensor(k)
        return self.load_state(tensors)

    def load_state(self, sd: dict[str, torch.Tensor]) -> "BolinexForCausalLM":
        """Build the run-time weights from a checkpoint-named state dict:
        fused projection matrices in the activation dtype; norms, the router,
        the distance-penalty numbers and every scalar in fp32."""
        cfg, dev, dt = self.cfg, self.device, self.dtype

        def act(*names):  # (fused) projection weight
            t = torch.cat([sd[n] for n in names], 0) if len(names) > 1 else sd[names[0]]
            return t.to(dev, dt).contiguous()

        def f32(t):
            return t.to(dev, torch.float32).contiguous()

        self.layers = []
        first_vmix = None
        for i, L in enumerate(cfg.layers):
            m, p = L["mixer"], f"l{i}.mix."
            out = dict(m=m, norm_w=f32(sd[f"l{i}.norm1"]), norm_b=f32(sd[f"l{i}.norm1.b"]),
                       w_in=act(p + "q", p + "k", p + "v", p + "g"), w_o=act(p + "o"),
                       bias=(f32(sd[p + "r1"]), f32(sd[p + "r2"])) if p + "r1" in sd else None,
                       mix_from=None, mix_source=False, lam=0.0)
            if m.get("v_mix"):
                if first_vmix is None:
                    first_vmix = i
                    out["mix_source"] = True
                else:
                    out.update(mix_from=first_vmix, lam=float(sd[p + "vmix"].float()))
            mlp, q = L.get("mlp"), f"l{i}.mlp."
            out["mlp"] = mlp
            if mlp and mlp["kind"] == "dense":
                out.update(w_up=act(q + "up"), w_down=act(q + "down"))
            elif mlp:
                E = mlp["router"]["experts"]
                w_egu = torch.stack([torch.cat([sd[f"{q}e{e}.gate"], sd[f"{q}e{e}.up"]], 0)
                                     for e in range(E)]).to(dev, dt).contiguous()
                # where the 256-tile GEMM serves the shape, gate and up rows are interleaved
                # for its SwiGLU epilogue and the [rows, 2 ff] intermediate is never written
                probe = torch.empty((1, w_egu.shape[2]), device=dev, dtype=dt)
                fused = moe.tile_gemm_ok(probe, w_egu) and (w_egu.shape[1] // 2) % moe.GLU_BLOCK == 0
                out.update(router=f32(sd[q + "router"]),
                           correction=f32(sd[q + "correction"]) if q + "correction" in sd else None,
                           w_egu=moe.interleave_glu(w_egu) if fused else w_egu, egu_fused=fused,
                           w_edown=torch.stack([sd[f"{q}e{e}.down"] for e in range(E)]).to(dev, dt).contiguous())
                if mlp.get("shared"):
                    out.update(w_sgu=act(q + "shared.gate", q + "shared.up"), w_sdown=act(q + "shared.down"))
            if self.side_dim:
                out.update(side_gate=act(f"l{i}.side.gate"), side_proj=act(f"l{i}.side.proj"),
                           side_w=f32(sd[f"l{i}.side.norm"]))
            self.layers.append(out)
        self.embed = act("embed")
        self.head = act("head")
        self.pos = act("pos") if "pos" in sd else None
        self.side_embed = act("side.embed") if self.side_dim else None
        self.final_w, self.final_b = f32(sd["final.norm"]), f32(sd["final.norm.b"])
        return self

    # ------------------------------------------------------------------ forward
    def _parts(self, rows: int, H: int, group: int, size: int, meta: AttnMeta) -> int:
        """Key partitions of the step's decode rows (rows that are no prompt-chunk tiles)."""
        vis = meta.max_ctx if meta.max_ctx else self.cfg.max_position_embeddings
        if size:
            vis = min(vis, size)
        if meta.is_prefill:
            rows -= meta.num_prefill_tokens if self.dtype == torch.bfloat16 and self.device.type == "cuda" else 0
        units = H if self.dtype != torch.bfloat16 else max(1, H // group) * (-(-group // 32))
        grouped = self.dtype == torch.bfloat16 and self.device.type == "cuda"
        return mx.row_attention_parts(max(rows, 1), units, vis,
                                      mx.GROUP_TARGET_WAVES if grouped else mx.ROW_TARGET_WAVES)

    def _mix(self, L: dict, h: torch.Tensor, meta: AttnMeta, kc, vc, seq, tables, bs: int, firsts: dict, i: int):
        m, T = L["m"], h.shape[0]
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        p = self._mm(h, L["w_in"])
        k_off, v_off, g_off = H * d, (H + G) * d, (H + G) * d + G * dv
        if L["mix_source"]:  # the values as projected stay alive for the layers that mix them in
            firsts[i] = p[:, v_off:v_off + G * dv]
        vf = firsts[L["mix_from"]] if L["mix_from"] is not None else None
        mx.headprep_cache(p, meta.positions, meta.slot_mapping, 0, G, d, k_off, None, None, self.cfg.rms_norm_eps,
                          None, kc, vc, v_mode=2, v_off=v_off, v_w=G * dv, v_first=vf, v_lambda=L["lam"])
        size = int((m.get("mask") or {}).get("size") or 0)
        tl = (meta.row_tiles, meta.num_prefill_tokens) if meta.is_prefill else (None, 0)
        a = mx.attention(p, kc, vc, meta.positions, seq, tables, bs, H, 1, H // G, d, dv, m["scale"],
                         "window" if size else "causal", size, self._parts(T, H, H // G, size, meta), False, *tl,
                         softcap=float(m.get("softcap") or 0.0), dist_bias=L["bias"])
        a = mx.act_mul(p[:, g_off:g_off + H * dv], a.view(T, H * dv), "sigmoid")
        return self._mm(a, L["w_o"])

    def _ff(self, L: dict, h: torch.Tensor) -> torch.Tensor | None:
        mlp = L["mlp"]
        if not mlp:
            return None
        if mlp["kind"] == "dense":
            return self._mm(mx.act_mul(self._mm(h, L["w_up"]), None, "relu2"), L["w_down"])
        r = mlp["router"]
        gr = r.get("groups") or {"count": 1, "keep": 1}
        z = torch.matmul(h.float(), L["router"].t())
        idx, w = moe.route(z, L["correction"], r["top"], gr["count"], gr["keep"])
        order, offsets = moe.plan(idx, r["experts"])
        if L["egu_fused"]:
            act = moe.grouped_gemm(h, L["w_egu"], order, offsets, r["top"], gather=True, scatter=False, glu=True)
        else:
            act = mx.glu_act(moe.grouped_gemm(h, L["w_egu"], order, offsets, r["top"], gather=True, scatter=False),
                             "silu")
        y = moe.grouped_gemm(act, L["w_edown"], order, offsets, r["top"], gather=False, scatter=True)
        shared = None
        if "w_sgu" in L:
            shared = self._mm(mx.glu_act(self._mm(h, L["w_sgu"]), "silu"), L["w_sdown"])
        return moe.combine(y, w, shared)

    def forward(self, input_ids: torch.Tensor, meta: AttnMeta, kv_caches: list[tuple]) -> torch.Tensor:
        """Final-normed hidden rows at meta.logits_idx (or all rows)."""
        cfg, eps, dt = self.cfg, self.cfg.rms_norm_eps, self.dtype
        X = mx.embed_streams(input_ids, self.embed, 1, self.pos, meta.positions if self.pos is not None else None)
        X = X.view(X.shape[0], X.shape[2])
        if meta.is_prefill:  # rows of several sequences: per-row sequence ids + one table
            seq, tables = meta.row_seq, meta.row_tables
        else:  # decode: row i is sequence i
            seq, tables = None, meta.block_tables
        bs = meta.block_size
        side = mx.gather_rows(self.side_embed, input_ids) if self.side_dim else None
        firsts: dict = {}
        n = len(self.layers)
        L0 = self.layers[0]
        h, _ = mx.residual_step(X, eps=eps, norm="layer", norm_w=L0["norm_w"], norm_b=L0["norm_b"], out_dtype=dt)
        ysel = None
        for i, L in enumerate(self.layers):
            kc, vc = kv_caches[i]
            ym = self._mix(L, h, meta, kc, vc, seq, tables, bs, firsts, i)
            if self.layer_hook is not None and meta.is_prefill:
                self.layer_hook(i)
            yf = self._ff(L, h)
            last = i + 1 == n
            nxt = None if last else self.layers[i + 1]
            # the norm that follows: the next layer's, or (on the chosen rows) the final one
            fuse = dict(norm="layer", norm_w=nxt["norm_w"], norm_b=nxt["norm_b"]) if nxt and self.trace_layers is None \
                else dict(norm=None)
            if self.side_dim:
                _, xa = mx.residual_step(X, ym, yf, eps=eps, out_dtype=dt, want_cast=dt != torch.float32)
                xa = X if xa is None else xa
                sd_ = self.side_dim
                g = mx.act_mul(self._mm(xa, L["side_gate"]), side[:, i * sd_:(i + 1) * sd_], "gelu_tanh")
                y = self._mm(g, L["side_proj"])
                if last and self.trace_layers is None:
                    ysel = y  # joins the residual with the final norm, on the chosen rows only
                else:
                    h, _ = mx.residual_step(X, c=y, c_w=L["side_w"], eps=eps, out_dtype=dt, **fuse)
            elif not last or self.trace_layers is not None:
                h, _ = mx.residual_step(X, ym, yf, eps=eps, out_dtype=dt, **fuse)
            else:
                ysel = (ym, yf)
            if self.trace_layers is not None:
                self.trace_layers.append(X.clone())
                if nxt:
                    h, _ = mx.residual_step(X, eps=eps, norm="layer", norm_w=nxt["norm_w"], norm_b=nxt["norm_b"],
                                            out_dtype=dt)
        pick = meta.logits_idx
        if pick is not None:
            if pick.numel() == 0:
                return torch.empty((0, cfg.hidden_size), device=X.device, dtype=dt)
            X = X.index_select(0, pick)
        sel = (lambda t: t if t is None or pick is None else t.index_select(0, pick))
        fin = dict(eps=eps, norm="layer", norm_w=self.final_w, norm_b=self.final_b, out_dtype=dt)
        if isinstance(ysel, tuple):
            return mx.residual_step(X, sel(ysel[0]), sel(ysel[1]), **fin)[0]
        if ysel is not None:
            return mx.residual_step(X, c=sel(ysel), c_w=self.layers[-1]["side_w"], **fin)[0]
        return mx.residual_step(X, **fin)[0]

    def compute_logits(self, hidden: torch.Tensor, fp32: bool = False) -> torch.Tensor:
        """Logits of final-normed rows; fp32: the products of the bf16 operands
        accumulated and returned in fp32 (scoring), in vocabulary slices so no
        fp32 copy of the head persists."""
        if not fp32 or hidden.dtype == torch.float32:
            return torch.matmul(hidden, self.head.t())
        hf = hidden.float()
        V = self.head.shape[0]
        out = torch.empty((hidden.shape[0], V), dtype=torch.float32, device=hidden.device)
        for v0 in range(0, V, 16384):
            torch.matmul(hf, self.head[v0:v0 + 16384].float().t(), out=out[:, v0:v0 + 16384])
        return out

    def sample_sharded(self, *a, **kw):
        raise RuntimeError("vocab-sharded sampling needs tensor parallelism, which Bolinex does not use")
