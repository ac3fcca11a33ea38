"""Bekulix: a layer-listed decoder for the MI355X engine.

A Bekulix checkpoint lists its layers; each has one of three attention mixers
and an optional gated feed-forward, all under a pre-norm residual that may run
over several parallel streams (hyper-connections), and a span of layers may
loop with shared weights.  Per layer run (T rows of one engine step, prompt
chunks and decode tokens of different sequences side by side):

    h  = stream_step(X, y_prev)             HIP  apply the previous sublayer's output to the
                                                 fp32 streams, read in, RMS norm (1 + w)
    p  = h @ Wfused^T (+ b)                 hipBLASLt, one fused projection per mixer
    headprep_cache(p)                       HIP  q/k head norms, position gain, paged cache write
    a  = attention(q, K cache, V cache)     HIP  causal / sliding-window / chunked masks; prompt
                                                 chunks on the MFMA tile kernel, decode rows (and
                                                 fp32, odd head widths) on the row kernel
    [a = diff_combine(a)]                   HIP  two-map (differential) layers
    y  = a @ Wo^T                           hipBLASLt
    h  = stream_step(X, y)                  HIP
    y  = glu_act(h @ Wgu^T) @ Wd^T          hipBLASLt + HIP

The mixers:
  * `attention`: grouped-query attention whose values are the key projection
    itself (one projection, cached twice: normed as K, raw as V), per-head
    q/k RMS norms, and a query gain that grows with log position;
  * `latent_attention`: keys and values are up-projections of one normed
    low-rank latent per token.  Only the latent is cached: W_uk is folded
    into the query (q' = q W_uk) and W_uv applied after the weighted sum, so
    attention runs over the latent cache as one shared key/value head of width
    kv_rank -- the same arithmetic for prompt chunks and decode rows;
  * `attention_2`: differential attention, two score maps per head over the
    same values, combined as unit_rms(a1 - lambda a2) (1 - diff).

Scores, softmax, norms and the residual streams are fp32; projections and
activations are bf16 (dtype=bfloat16) or everything is fp32 (dtype=float32).
"""
from __future__ import annotations

import glob
import math
import os

import torch

from ..ops import mixers as mx
from .config import LayeredConfig
from .llama import AttnMeta, TPGroup

MIXER_TYPES = ("attention", "latent_attention", "attention_2")


def _mask_of(m: dict, kind: str) -> tuple[str, int]:
    """(mask kind, size) of a mixer whose mask is of `kind` when it gives a size, plain causal otherwise."""
    size = (m.get("mask") or {}).get("size")
    return (kind, int(size)) if size else ("causal", 0)


class BekulixForCausalLM:
    #: the runner builds per-row sequence ids and one block table over all rows of a step
    unified_rows = True

    def __init__(self, cfg: LayeredConfig, device: torch.device | str = "cuda", dtype=torch.bfloat16,
                 tp: TPGroup | None = None):
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.tp = tp or TPGroup()
        if self.tp.size != 1:
            raise ValueError("Bekulix runs on one GPU per engine (tensor parallel size 1)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"unsupported dtype {dtype}")
        for L in cfg.layers:
            if L["type"] not in MIXER_TYPES:
                raise ValueError(f"unknown mixer type {L['type']!r}")
            if L.get("mlp") and L["mlp"].get("kind") != "dense":
                raise ValueError(f"unknown feed-forward kind {L['mlp'].get('kind')!r}")
        self.S = int(cfg.streams) if cfg.streams else 1
        if self.S > mx.MAX_STREAMS:
            raise ValueError(f"{self.S} residual streams (limit {mx.MAX_STREAMS})")
        self.runs = cfg.layer_runs()
        self.layers: list[dict] = []
        self.embed = self.head = self.final_w = None
        self.fp8 = False
        self.kv_scales = (1.0, 1.0)
        self.kv_amax = None
        self.layer_hook = None
        self.gemm_plan: dict = {}
        # debugging: when a list, forward() appends the summed residual streams after every layer run
        self.trace_layers: list | None = None

    # ------------------------------------------------------------------ engine hooks (no-ops here)
    def enable_fused_mlp(self) -> bool:
        return False

    def fold_norms(self) -> bool:
        return False

    def tune_gemms(self, sizes, **kw) -> list:
        return []

    def tune_prefill_gemms(self, max_tokens, **kw) -> list:
        return []

    def quantize_fp8(self):
        raise ValueError("fp8 linears are not available for Bekulix")

    @torch.no_grad()
    def warmup_linears(self, tokens: int) -> None:
        """Run every distinct projection shape at M = tokens once (the GEMM
        library loads its kernels for the size before serving)."""
        x = torch.zeros(tokens, self.cfg.hidden_size, device=self.device, dtype=self.dtype)
        seen = set()
        for L in self.layers:
            for name in ("w_in", "w_o", "w_gu", "w_down"):
                w = L.get(name)
                if w is None or tuple(w.shape) in seen:
                    continue
                seen.add(tuple(w.shape))
                torch.matmul(x if w.shape[1] == x.shape[1] else
                             torch.zeros(tokens, w.shape[1], device=self.device, dtype=self.dtype), w.t())

    def weight_bytes(self) -> int:
        n = sum(t.numel() * t.element_size() for L in self.layers for t in L.values() if isinstance(t, torch.Tensor))
        return n + self.embed.numel() * self.embed.element_size() + self.head.numel() * self.head.element_size()

    # ------------------------------------------------------------------ paged caches
    def cache_widths(self) -> list[tuple[int, int]]:
        """(K row width, V row width) of every layer run; V width 0: the V
        cache is the K cache (latent layers)."""
        out = []
        for li in self.runs:
            L = self.cfg.layers[li]
            m = L["mixer"]
            if L["type"] == "latent_attention":
                out.append((m["kv_rank"], 0))
            elif L["type"] == "attention":
                out.append((m["kv_heads"] * m["dim"], m["kv_heads"] * m["dim"]))
            else:
                out.append((m["kv_heads"] * 2 * m["dim"], m["kv_heads"] * m["vdim"]))
        return out

    def kv_bytes_per_block(self, block_size: int, dtype: torch.dtype) -> int:
        es = torch.empty((), dtype=dtype).element_size()
        return sum((k + v) * block_size * es for k, v in self.cache_widths())

    def alloc_kv_caches(self, num_blocks: int, block_size: int, dtype: torch.dtype) -> list[tuple]:
        """One (K, V) pair per layer run (a looped layer has a cache per pass),
        token-major [num_blocks * block_size, width], indexed by the engine's
        one block table."""
        if dtype != self.dtype:
            raise ValueError(f"the cache holds the model's activation dtype {self.dtype}, not {dtype}")
        caches = []
        for wk, wv in self.cache_widths():
            k = torch.zeros((num_blocks * block_size, wk), dtype=dtype, device=self.device)
            v = torch.zeros((num_blocks * block_size, wv), dtype=dtype, device=self.device) if wv else k
            caches.append((k, v))
        return caches

    # ------------------------------------------------------------------ weights
    def random_state(self, seed: int = 0) -> dict[str, torch.Tensor]:
        """Random weights in the checkpoint's naming and dtypes (bf16), scaled
        so activations stay O(1)."""
        cfg = self.cfg
        g = torch.Generator().manual_seed(seed)
        W = cfg.hidden_size
        S = self.S

        def rnd(*shape, std):
            return (torch.randn(*shape, generator=g) * std).to(torch.bfloat16)

        sd = {"embed": rnd(cfg.vocab_size, W, std=1.0), "final.norm": rnd(W, std=0.1),
              "head": rnd(cfg.vocab_size, W, std=W ** -0.5)}
        nl = max(1, len(self.runs))
        for i, L in enumerate(cfg.layers):
            m, p = L["mixer"], f"l{i}.mix."
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            sd[f"l{i}.norm1"] = rnd(W, std=0.1)
            if L["type"] == "attention":
                G = m["kv_heads"]
                sd[p + "q"], sd[p + "k"] = rnd(H * d, W, std=W ** -0.5), rnd(G * d, W, std=W ** -0.5)
                sd[p + "q.norm"], sd[p + "k.norm"] = 1 + rnd(d, std=0.1), 1 + rnd(d, std=0.1)
                sd[p + "o"] = rnd(W, H * d, std=(H * d) ** -0.5 / math.sqrt(nl))
            elif L["type"] == "latent_attention":
                r = m["kv_rank"]
                sd[p + "q"], sd[p + "dkv"] = rnd(H * d, W, std=W ** -0.5), rnd(r, W, std=W ** -0.5)
                sd[p + "dkv.norm"] = 1 + rnd(r, std=0.1)
                sd[p + "uk"], sd[p + "uv"] = rnd(H * d, r, std=r ** -0.5), rnd(H * dv, r, std=r ** -0.5)
                sd[p + "o"] = rnd(W, H * dv, std=(H * dv) ** -0.5 / math.sqrt(nl))
            else:
                G = m["kv_heads"]
                for n, rows in (("q", H * 2 * d), ("k", G * 2 * d), ("v", G * dv)):
                    sd[p + n] = rnd(rows, W, std=W ** -0.5)
                    sd[p + n + ".b"] = rnd(rows, std=0.1)
                for n in ("lq1", "lk1", "lq2", "lk2"):
                    sd[p + n] = rnd(d, std=0.1)
                sd[p + "o"] = rnd(W, H * dv, std=(H * dv) ** -0.5 / math.sqrt(nl))
            if L.get("mlp"):
                F = L["mlp"]["ff"]
                sd[f"l{i}.norm2"] = rnd(W, std=0.1)
                sd[f"l{i}.mlp.gate"], sd[f"l{i}.mlp.up"] = rnd(F, W, std=W ** -0.5), rnd(F, W, std=W ** -0.5)
                sd[f"l{i}.mlp.down"] = rnd(W, F, std=F ** -0.5 / math.sqrt(nl))
            if cfg.streams:
                for q in ("hc1", "hc2") if L.get("mlp") else ("hc1",):
                    sd[f"l{i}.{q}.in"] = (torch.full((S,), 1.0 / S) + torch.randn(S, generator=g) * 0.1).to(torch.bfloat16)
                    sd[f"l{i}.{q}.out"] = (1 + torch.randn(S, generator=g) * 0.1).to(torch.bfloat16)
                    sd[f"l{i}.{q}.mix"] = (torch.eye(S) + torch.randn(S, S, generator=g) * 0.05).to(torch.bfloat16)
        return sd

    def random_init(self, seed: int = 0) -> "BekulixForCausalLM":
        return self.load_state(self.random_state(seed))

    def load_safetensors(self, path: str) -> "BekulixForCausalLM":
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

    def load_state(self, sd: dict[str, torch.Tensor]) -> "BekulixForCausalLM":
        """Build the run-time weights from a checkpoint-named state dict:
        fused projection matrices in the activation dtype, every norm / stream
        / scalar parameter in fp32."""
        cfg, dev, dt = self.cfg, self.device, self.dtype
        S = self.S

        def act(*names):  # (fused) projection weight
            t = torch.cat([sd[n] for n in names], 0) if len(names) > 1 else sd[names[0]]
            return t.to(dev, dt).contiguous()

        def f32(t):
            return t.to(dev, torch.float32).contiguous()

        def hc(i, q):
            if cfg.streams:
                p = f"l{i}.{q}."
                return dict(mix=f32(sd[p + "mix"]), gain=f32(sd[p + "out"]), rin=f32(sd[p + "in"]))
            one = torch.ones(1, device=dev, dtype=torch.float32)
            return dict(mix=one.view(1, 1), gain=one, rin=one)

        self.layers = []
        for i, L in enumerate(cfg.layers):
            m, p = L["mixer"], f"l{i}.mix."
            H, d = m["heads"], m["dim"]
            out = dict(type=L["type"], m=m, norm1=f32(1.0 + sd[f"l{i}.norm1"].float()), hc1=hc(i, "hc1"))
            if L["type"] == "attention":
                out.update(w_in=act(p + "q", p + "k"), qn=f32(sd[p + "q.norm"]), kn=f32(sd[p + "k.norm"]))
            elif L["type"] == "latent_attention":
                r, dv = m["kv_rank"], m["vdim"]
                out.update(w_in=act(p + "q", p + "dkv"), cn=f32(sd[p + "dkv.norm"]),
                           uk=sd[p + "uk"].to(dev, dt).view(H, d, r).contiguous(),
                           uv=sd[p + "uv"].to(dev, dt).view(H, dv, r).transpose(1, 2).contiguous())
            else:
                lam = math.exp(float((sd[p + "lq1"].float() * sd[p + "lk1"].float()).sum())) \
                    - math.exp(float((sd[p + "lq2"].float() * sd[p + "lk2"].float()).sum())) + float(m["diff"])
                out.update(w_in=act(p + "q", p + "k", p + "v"), b_in=act(p + "q.b", p + "k.b", p + "v.b"), lam=lam)
            out["w_o"] = act(p + "o")
            if L.get("mlp"):
                out.update(norm2=f32(1.0 + sd[f"l{i}.norm2"].float()), hc2=hc(i, "hc2"),
                           w_gu=act(f"l{i}.mlp.gate", f"l{i}.mlp.up"), w_down=act(f"l{i}.mlp.down"))
            self.layers.append(out)
        self.embed = act("embed")
        self.head = act("head")
        self.final_w = f32(1.0 + sd["final.norm"].float())
        self.ones_s = torch.ones(S, device=dev, dtype=torch.float32)
        return self

    # ------------------------------------------------------------------ forward
    def _parts(self, rows: int, n_qh: int, mask: str, size: int, meta: AttnMeta, group: int = 1) -> int:
        """Key partitions of the step's decode rows (rows that are no prompt-chunk tiles)."""
        vis = meta.max_ctx if meta.max_ctx else self.cfg.max_position_embeddings
        if mask != "causal":
            vis = min(vis, size)
        if meta.is_prefill:
            rows -= meta.num_prefill_tokens if self.dtype == torch.bfloat16 and self.device.type == "cuda" else 0
        units = n_qh if self.dtype != torch.bfloat16 else max(1, n_qh // group) * (-(-group // 32))
        grouped = self.dtype == torch.bfloat16 and self.device.type == "cuda"
        return mx.row_attention_parts(max(rows, 1), units, vis,
                                      mx.GROUP_TARGET_WAVES if grouped else mx.ROW_TARGET_WAVES)

    def _mix(self, L: dict, h: torch.Tensor, meta: AttnMeta, kc, vc, seq, tables, bs: int) -> torch.Tensor:
        m, T = L["m"], h.shape[0]
        H, d, eps = m["heads"], m["dim"], self.cfg.rms_norm_eps
        pos, slots = meta.positions, meta.slot_mapping
        # prompt-chunk rows (the first num_prefill_tokens) as tiles for the matrix-core kernel
        tl = (meta.row_tiles, meta.num_prefill_tokens) if meta.is_prefill else (None, 0)
        if L["type"] == "attention":
            G = m["kv_heads"]
            p = torch.matmul(h, L["w_in"].t())
            qt = m.get("q_temp")
            mx.headprep_cache(p, pos, slots, H, G, d, H * d, L["qn"], L["kn"], eps,
                              (qt["coef"], qt["every"]) if qt else None, kc, vc, v_mode=1)
            a = mx.attention(p, kc, vc, pos, seq, tables, bs, H, 1, H // G, d, d, m["scale"], "causal", 0,
                             self._parts(T, H, "causal", 0, meta, H // G), False, *tl)
            return torch.matmul(a.view(T, H * d), L["w_o"].t())
        if L["type"] == "latent_attention":
            r, dv = m["kv_rank"], m["vdim"]
            mask, size = _mask_of(m, "window")
            p = torch.matmul(h, L["w_in"].t())
            mx.headprep_cache(p, pos, slots, 0, 1, r, H * d, None, L["cn"], eps, None, kc, None, v_mode=0)
            # fold W_uk into the query: the latent cache is the one key/value head of every query head
            ql = torch.bmm(p[:, : H * d].view(T, H, d).transpose(0, 1), L["uk"]).transpose(0, 1).contiguous()
            a = mx.attention(ql.view(T, H * r), kc, kc, pos, seq, tables, bs, H, 1, H, r, r, m["scale"], mask,
                             size, self._parts(T, H, mask, size, meta, H), False, *tl)
            o = torch.bmm(a.transpose(0, 1), L["uv"]).transpose(0, 1).reshape(T, H * dv)
            return torch.matmul(o, L["w_o"].t())
        G, dv = m["kv_heads"], m["vdim"]
        mask, size = _mask_of(m, "chunk")
        p = torch.addmm(L["b_in"], h, L["w_in"].t())
        qw, kw = H * 2 * d, G * 2 * d
        mx.headprep_cache(p, pos, slots, 0, 2 * G, d, qw, None, None, eps, None, kc, vc, v_mode=2, v_off=qw + kw,
                          v_w=G * dv)
        a = mx.attention(p, kc, vc, pos, seq, tables, bs, 2 * H, 2, H // G, d, dv, m["scale"], mask, size,
                         self._parts(T, 2 * H, mask, size, meta, H // G), True, *tl)
        o = mx.diff_combine(a.view(T, H, 2, dv), L["lam"], 1.0 - float(m["diff"]), eps, self.dtype)
        return torch.matmul(o, L["w_o"].t())

    def forward(self, input_ids: torch.Tensor, meta: AttnMeta, kv_caches: list[tuple]) -> torch.Tensor:
        """Final-normed hidden rows at meta.logits_idx (or all rows)."""
        cfg, eps, dt = self.cfg, self.cfg.rms_norm_eps, self.dtype
        T = input_ids.shape[0]
        X = mx.embed_streams(input_ids, self.embed, self.S)
        if meta.is_prefill:  # rows of several sequences: per-row sequence ids + one table
            seq, tables = meta.row_seq, meta.row_tables
        else:  # decode: row i is sequence i
            seq, tables = None, meta.block_tables
        bs = meta.block_size
        y = hcp = None  # the previous sublayer's output and its stream weights, applied by the next step
        for run, li in enumerate(self.runs):
            L = self.layers[li]
            kc, vc = kv_caches[run]
            h = mx.stream_step(X, y, hcp and hcp["mix"], hcp and hcp["gain"], L["hc1"]["rin"], L["norm1"], eps, dt)
            y, hcp = self._mix(L, h, meta, kc, vc, seq, tables, bs), L["hc1"]
            if self.layer_hook is not None and meta.is_prefill:
                self.layer_hook(run)
            if "w_gu" in L:
                h = mx.stream_step(X, y, hcp["mix"], hcp["gain"], L["hc2"]["rin"], L["norm2"], eps, dt)
                y, hcp = torch.matmul(mx.glu_act(torch.matmul(h, L["w_gu"].t()), "relu"), L["w_down"].t()), L["hc2"]
            if self.trace_layers is not None:
                mx.stream_step(X, y, hcp["mix"], hcp["gain"], None, None, eps, dt)
                y = hcp = None
                self.trace_layers.append(X.sum(1))
        if meta.logits_idx is not None:
            if meta.logits_idx.numel() == 0:
                return torch.empty((0, cfg.hidden_size), device=X.device, dtype=dt)
            X = X.index_select(0, meta.logits_idx)
            y = y.index_select(0, meta.logits_idx) if y is not None else None
        return mx.stream_step(X, y, hcp and hcp["mix"], hcp and hcp["gain"], self.ones_s, self.final_w, eps, dt)

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
        raise RuntimeError("vocab-sharded sampling needs tensor parallelism, which Bekulix does not use")
