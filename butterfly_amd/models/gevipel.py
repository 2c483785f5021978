"""Gevipel: a decoder-only LM whose sublayers sit between two layer norms (ModelConfig.layer_specs,
ModelConfig.layer_runs).

  embedding   : x = table[token] * embed_scale, an f32 residual; this value is the embedding output e
  every layer : x <- x + m * LN_1b(mixer(LN_1(x))), then x <- x + m * LN_2b(ff(LN_2(x))); all four norms
                have weight and bias, m = residual_mult
    mixer "sloped_attention" : GQA without rotation; queries and keys RMS-normed per head with a shared
                        weight; the values are the keys as projected (before their norm); the query
                        scale grows with the logarithm of the position; the scores lose slope_h (i - j)
                        with slope_h = 2^(-8 (h + 1) / H); sliding window; ordinary softmax
    mixer "delta"            : gated delta rule: short causal convolutions + silu on the q, k, v rows,
                        unit-length q and k, S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q
                        with g = exp(-exp(A_log) softplus(a + dt_bias)), beta = sigmoid(b); per-head
                        RMS norm of o with a weight, a silu gate, the output projection. S and the
                        convolutions' last inputs live in the cache's per-sequence state slots
    mixer "latent_attention" : queries projected from the mixer's input, keys and values expanded
                        from one RMS-normed latent plus one rotated key part shared by the heads
                        (only those are cached; the heads attend to the latent itself, see
                        models/zinesun.py), causal, a learned sink logit per head in the softmax
    feed-forward      : softmax router over all experts in f32; the experts with the largest (score +
                        correction) are chosen and weigh in with their plain scores; an expert is
                        W_down relu(W_up h)^2
  layer runs  : a span of layers may run several times in a row with the same weights; every run has its
                own pages and state, and e is added to the residual before every repetition
  output      : layer norm with weight and bias, logits = head x, f32

Every size and constant comes from the config; the residual, norms, softmax, angles, decays, unit
norms and the recurrent state are f32 in the bf16 model too. Unsharded (tp = pp = ep = 1). Prompt
chunks always attend through the paged cache, so one attention op serves fresh prompts,
continuation chunks and decoded tokens.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from .. import ops
from ..config import ModelConfig
from ..engine.batch import ForwardBatch
from ..parallel.comm import Communicator
from .shard import LocalDims, Shard
from .stack import PackedStack, pad128
from .transformer import LogicalParam, _name_seed

SLOPE_EXP = 8.0         # slope of head h: 2^(-SLOPE_EXP (h + 1) / H)
UNIT_EPS = 1e-6         # q / sqrt(sum q^2 + UNIT_EPS) in the delta rule
NO_WINDOW = 1 << 30     # plain causal attention


class GevipelLM(PackedStack):
    attention_types = ("sloped_attention", "latent_attention")

    def __init__(self, cfg: ModelConfig, shard: Shard = Shard(), device="cpu",
                 dtype: torch.dtype = torch.bfloat16, comm: Optional[Communicator] = None):
        if not cfg.layer_specs:
            raise ValueError("Gevipel needs ModelConfig.layer_specs (ModelConfig.from_gevipel)")
        if shard.tp_size != 1 or shard.ep_size != 1 or shard.layer_start != 0 or \
                (shard.layer_end is not None and shard.layer_end != cfg.num_layers):
            raise NotImplementedError("Gevipel runs unsharded (tp = pp = ep = 1)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Gevipel runs in bfloat16 or float32")
        for sp in cfg.layer_specs:
            if sp["type"] not in self.attention_types + ("delta",):
                raise ValueError(f"layer {sp['index']}: Gevipel has no mixer {sp['type']!r}")
            if sp["type"] == "latent_attention" and sp["q_rank"]:
                raise ValueError(f"layer {sp['index']}: Gevipel projects its queries directly (no query latent)")
            if sp["ffn"] and (sp["ffn"]["kind"] != "moe" or sp["ffn"].get("glu", True)):
                raise ValueError(f"layer {sp['index']}: Gevipel's feed-forward is a router over plain experts")
        self.cfg, self.shard = cfg, shard
        self.device, self.dtype = torch.device(device), dtype
        self.comm = comm or Communicator.single()
        self.specs = cfg.layer_specs
        # layer indices in running order; run r owns its own cache pair and state tensors
        self.runs = list(cfg.layer_runs) if cfg.layer_runs is not None else list(range(cfg.num_layers))
        # runs before which the embedding output re-enters: every start of the repeated span but the first
        first = self.runs.index(cfg.loop_start) if cfg.loop_start in self.runs else -1
        self.reentry = {r for r, i in enumerate(self.runs) if i == cfg.loop_start and r != first}
        self.layer_ids = list(range(cfg.num_layers))
        self.first = self.last = True
        self.tp = self.ep = 1
        vpad = pad128(cfg.vocab_size)
        self.dims = LocalDims(hq=cfg.num_heads, hkv=cfg.num_kv_heads, kv_head0=0, q_head0=0,
                              ffn=max(cfg.intermediate_size, 1), ffn0=0, vocab=vpad, vocab0=0, vocab_padded=vpad,
                              experts=max(cfg.num_experts, 1), expert0=0)
        # cached row sizes (keys, values), padded with zeros to sizes the attention's matrix-core form tiles
        self.cache_dims = {}
        for sp in self.specs:
            if sp["type"] == "sloped_attention":
                d = ops.attn_window_pad(sp["dim"], dtype)
                self.cache_dims[sp["index"]] = (d, d)
            elif sp["type"] == "latent_attention":
                self.cache_dims[sp["index"]] = (ops.attn_window_pad(sp["kv_rank"] + sp["rot_dim"], dtype),
                                                ops.attn_window_pad(sp["kv_rank"], dtype))
        # run -> index of its (K, V) pair / of its first state tensor
        self.cache_index, self.state_index = {}, {}
        for r, i in enumerate(self.runs):
            if self.specs[i]["type"] == "delta":
                self.state_index[r] = 2 * len(self.state_index)
            else:
                self.cache_index[r] = len(self.cache_index)
        self.has_state = bool(self.state_index)   # delta-rule matrices and convolution histories
        self.state: list = []                     # set by allocate_state (the cache object owns the pool)
        self.layer_probe = None                   # debug hook: f(run, residual [T, W] f32) after every layer run
        self.p: dict[str, torch.Tensor] = {}
        self.packed: dict = {}
        self._arange: dict = {}
        self._alloc()

    # ------------------------------------------------------------------------------------
    # parameters
    # ------------------------------------------------------------------------------------
    def _wide(self, rows: int, k: int) -> int:
        """Rows of a projection: padded to the tuned GEMMs' 128-row tiling when its K fits them."""
        return pad128(rows) if k % 64 == 0 else rows

    @staticmethod
    def _conv_channels(sp) -> int:
        return 2 * sp["kv_heads"] * sp["dim"] + sp["heads"] * sp["vdim"]

    def _alloc(self):
        c, W = self.cfg, self.cfg.hidden_size
        z = lambda *s: torch.zeros(*s, dtype=self.dtype, device=self.device)                  # noqa: E731
        f = lambda *s: torch.zeros(*s, dtype=torch.float32, device=self.device)               # noqa: E731
        p = self.p
        p["embed"] = z(c.vocab_size, W)
        for sp in self.specs:
            i = sp["index"]
            pre = f"l{i}."
            H, D, Dv = sp["heads"], sp["dim"], sp["vdim"]
            for n in ("norm1", "norm1b") + (("norm2", "norm2b") if sp["ffn"] else ()):
                p[pre + n], p[pre + n + ".b"] = f(W), f(W)
            if sp["type"] == "sloped_attention":
                G = sp["kv_heads"]
                p[pre + "qk"] = z(self._wide(H * D + G * D, W), W)                # q | k (the values are the keys)
                p[pre + "q.norm"], p[pre + "k.norm"] = f(D), f(D)
                h = torch.arange(1, H + 1, dtype=torch.float64)
                p[pre + "slopes"] = torch.pow(2.0, -SLOPE_EXP * h / H).to(torch.float32).to(self.device)
                p[pre + "inv_freq"] = f(0)
                # the attention leaves heads of the padded value size: W_o carries zero columns there
                p[pre + "o"] = z(W, H * self.cache_dims[i][1])
            elif sp["type"] == "delta":
                C = self._conv_channels(sp)
                # one projection of the mixer's input: q | k | v (the convolved rows) | gate | b | a
                p[pre + "in"] = z(self._wide(C + H * Dv + 2 * H, W), W)
                p[pre + "conv"] = f(C, sp["taps"])
                p[pre + "A_log"], p[pre + "dt_bias"], p[pre + "gnorm"] = f(H), f(H), f(Dv)
                p[pre + "o"] = z(W, H * Dv)
            else:
                R, rd = sp["kv_rank"], sp["rot_dim"]
                p[pre + "in"] = z(self._wide(H * (D + rd) + R + rd, W), W)        # queries | latent | rotated key
                p[pre + "dkv.norm"], p[pre + "sink"] = f(R), f(H)
                p[pre + "ukT"] = z(H, R, D)               # W_uk per head, transposed: q_lat = ukT[h] q_plain
                p[pre + "uv"] = z(H, Dv, R)
                p[pre + "o"] = z(W, H * Dv)
                n = torch.arange(sp["rot_dims"] // 2, dtype=torch.float64)
                p[pre + "inv_freq"] = (sp["rot_base"] ** (-2.0 * n / max(sp["rot_dims"], 1))).to(torch.float32).to(self.device)
            fs = sp["ffn"]
            if fs:
                E, F = fs["experts"], fs["ff"]
                p[pre + "router"], p[pre + "correction"] = z(E, W), f(E)
                p[pre + "up"], p[pre + "edown"] = z(E, F, W), z(E, W, F)
        p["final.norm"], p["final.norm.b"] = f(W), f(W)
        p["head"] = z(self.dims.vocab, W)             # rows past the vocabulary stay zero

    @property
    def head_weight(self) -> torch.Tensor:
        return self.p["head"]

    def logical_params(self) -> list[LogicalParam]:
        """Checkpoint tensors by their file names ('l<i>.mix.q', 'l<i>.mlp.e<j>.up', ...), each a view into
        (or a transposition of) the fused local tensors."""
        c, p = self.cfg, self.p
        W = c.hidden_size
        out: list[LogicalParam] = []

        def add(name, t, init="normal", put=None, shape=None, get=None):
            out.append(LogicalParam(name, tuple(shape or t.shape), None, 0, 0, init, get or (lambda t=t: t),
                                    put or (lambda x, t=t: t.copy_(x.reshape(t.shape)))))

        add("embed", p["embed"], "embed")
        for sp in self.specs:
            i = sp["index"]
            L = f"l{i}."
            H, D, Dv = sp["heads"], sp["dim"], sp["vdim"]
            for n in ("norm1", "norm1b") + (("norm2", "norm2b") if sp["ffn"] else ()):
                add(L + n, p[L + n], "ones")
                add(L + n + ".b", p[L + n + ".b"], "small")
            if sp["type"] == "sloped_attention":
                G, w = sp["kv_heads"], p[L + "qk"]
                add(L + "mix.q", w[:H * D])
                add(L + "mix.k", w[H * D:H * D + G * D])
                add(L + "mix.q.norm", p[L + "q.norm"], "ones")
                add(L + "mix.k.norm", p[L + "k.norm"], "ones")
                ov = p[L + "o"].view(W, H, self.cache_dims[i][1])[:, :, :Dv]      # the columns of real values
                add(L + "mix.o", ov, shape=(W, H * Dv), get=lambda t=ov: t.reshape(t.shape[0], -1),
                    put=lambda x, t=ov: t.copy_(x.reshape(t.shape)))
            elif sp["type"] == "delta":
                G, w, cw = sp["kv_heads"], p[L + "in"], p[L + "conv"]
                o1, o2, C = G * D, 2 * G * D, self._conv_channels(sp)
                for n, a, b in (("q", 0, o1), ("k", o1, o2), ("v", o2, C)):
                    add(L + "mix." + n, w[a:b])
                    add(L + "mix." + n + ".conv", cw[a:b], "taps")
                add(L + "mix.g", w[C:C + H * Dv])
                add(L + "mix.b", w[C + H * Dv:C + H * Dv + H])
                add(L + "mix.a", w[C + H * Dv + H:C + H * Dv + 2 * H])
                add(L + "mix.A_log", p[L + "A_log"], "a_log")
                add(L + "mix.dt_bias", p[L + "dt_bias"], "sink")
                add(L + "mix.norm", p[L + "gnorm"], "ones")
                add(L + "mix.o", p[L + "o"])
            else:
                R, rd, w = sp["kv_rank"], sp["rot_dim"], p[L + "in"]
                HQ = H * (D + rd)
                add(L + "mix.q", w[:HQ])
                add(L + "mix.dkv", w[HQ:HQ + R + rd])
                add(L + "mix.dkv.norm", p[L + "dkv.norm"], "ones")
                ukT, uv = p[L + "ukT"], p[L + "uv"]
                add(L + "mix.uk", ukT, shape=(H * D, R), get=lambda t=ukT: t.transpose(1, 2).reshape(-1, t.shape[1]),
                    put=lambda x, t=ukT: t.copy_(x.reshape(t.shape[0], t.shape[2], t.shape[1]).transpose(1, 2)))
                add(L + "mix.uv", uv, shape=(H * Dv, R), get=lambda t=uv: t.reshape(-1, t.shape[2]))
                add(L + "mix.sink", p[L + "sink"], "sink")
                add(L + "mix.o", p[L + "o"])
            fs = sp["ffn"]
            if fs:
                add(L + "mlp.router", p[L + "router"])
                add(L + "mlp.correction", p[L + "correction"], "tiny")
                for e in range(fs["experts"]):
                    add(L + f"mlp.e{e}.up", p[L + "up"][e])
                    add(L + f"mlp.e{e}.down", p[L + "edown"][e])
        add("final.norm", p["final.norm"], "ones")
        add("final.norm.b", p["final.norm.b"], "small")
        add("head", p["head"][:c.vocab_size])
        return out

    @torch.no_grad()
    def init_random(self, seed: int = 0) -> None:
        """Deterministic random weights: each tensor is drawn on the host from a generator keyed on
        (seed, tensor name). Projections are scaled by 1 / sqrt(fan-in), the embedding so that the
        scaled rows have unit entries, norm weights sit around one, decay rates below one."""
        for lp in self.logical_params():
            g = torch.Generator().manual_seed(_name_seed(lp.name, seed))
            shp = lp.global_shape
            r = torch.randn(shp, generator=g)
            if lp.init == "normal":
                t = r / math.sqrt(shp[-1])
            elif lp.init == "embed":
                t = r / max(self.cfg.embed_scale, 1e-6)
            elif lp.init == "ones":
                t = 1.0 + 0.1 * r
            elif lp.init == "small":
                t = 0.1 * r
            elif lp.init == "tiny":
                t = 0.02 * r
            elif lp.init == "taps":
                t = 0.5 * r
            elif lp.init == "sink":
                t = r
            elif lp.init == "a_log":
                t = -1.0 + 0.5 * r
            else:
                raise ValueError(lp.init)
            # weights are bf16 values in every run (an f32 model holds them exactly)
            lp.set(t.to(torch.bfloat16).to(self.device))

    # ------------------------------------------------------------------------------------
    # caches
    # ------------------------------------------------------------------------------------
    def kv_bytes_per_token(self, dtype: Optional[torch.dtype] = None) -> int:
        es = torch.empty((), dtype=dtype or self.dtype).element_size()
        n = 0
        for r in self.cache_index:
            sp = self.specs[self.runs[r]]
            dk, dv = self.cache_dims[sp["index"]]
            n += (dk + dv) * (sp["kv_heads"] if sp["type"] == "sloped_attention" else 1)
        return max(1, n * es)

    def state_bytes_per_slot(self) -> int:
        n = 0
        for r in self.state_index:
            sp = self.specs[self.runs[r]]
            n += sp["heads"] * sp["dim"] * sp["vdim"] + (sp["taps"] - 1) * self._conv_channels(sp)
        return 4 * n

    def allocate_kv_cache(self, num_blocks: int, block_size: int, dtype: Optional[torch.dtype] = None) -> list:
        """One (K [blocks, G, BS, D], V [blocks, G, Dv, BS]) pair per run of an attention layer (a layer
        that runs twice caches twice), V with a page's tokens contiguous, row sizes padded with zeros.
        A sloped layer's V holds the keys as projected; a latent layer has one shared "head" whose K
        rows are [normed latent | rotated key part] and whose V is the latent again."""
        dt = dtype or self.dtype
        if dt != self.dtype:
            raise NotImplementedError("Gevipel caches hold the model's element type")
        caches = []
        for r in sorted(self.cache_index, key=self.cache_index.get):
            sp = self.specs[self.runs[r]]
            dk, dv = self.cache_dims[sp["index"]]
            G = sp["kv_heads"] if sp["type"] == "sloped_attention" else 1
            caches.append((torch.zeros(num_blocks, G, block_size, dk, dtype=dt, device=self.device),
                           torch.zeros(num_blocks, G, dv, block_size, dtype=dt, device=self.device)))
        return caches

    def allocate_state(self, num_slots: int) -> list:
        """Two f32 tensors per run of a delta layer: the last taps - 1 projected q | k | v rows
        [slots, taps - 1, C] (oldest first) and the delta-rule matrices, column by column [slots, H, Dv, D]."""
        self.state = []
        for r in sorted(self.state_index, key=self.state_index.get):
            sp = self.specs[self.runs[r]]
            self.state.append(torch.zeros(num_slots, sp["taps"] - 1, self._conv_channels(sp), dtype=torch.float32,
                                          device=self.device))
            self.state.append(torch.zeros(num_slots, sp["heads"], sp["vdim"], sp["dim"], dtype=torch.float32,
                                          device=self.device))
        return self.state

    # ------------------------------------------------------------------------------------
    # forward
    # ------------------------------------------------------------------------------------
    def forward(self, fb: ForwardBatch, kv_caches: Optional[list] = None,
                hidden_in: Optional[torch.Tensor] = None) -> torch.Tensor:
        """One step over the packed rows of `fb`; returns f32 logits [R, padded vocab] for the rows
        fb.logits_idx names (None: all)."""
        p, c, eps, m = self.p, self.cfg, self.cfg.norm_eps, self.cfg.residual_mult
        meta = self._step_meta(fb)
        T, W = fb.num_tokens, c.hidden_size
        if self.has_state and T and not self.state:
            raise RuntimeError("Gevipel: the delta-rule state pool is not allocated (KVCache state slots)")
        if kv_caches is None and self.cache_index:
            raise RuntimeError("Gevipel attention runs through the paged cache")
        e = ops.embed_scaled(fb.input_ids, p["embed"], c.embed_scale)
        x = e
        if self.reentry:                                  # the residual is updated in place: keep e apart
            x = ops.new_empty(T, W, dtype=torch.float32, device=self.device)
            x.copy_(e)
        # sublayers in running order: (run, layer, 1 = mixer / 2 = feed-forward)
        subs = [(r, i, q) for r, i in enumerate(self.runs) for q in ((1, 2) if self.specs[i]["ffn"] else (1,))]
        h = ops.layer_norm_rows(x, p[f"l{subs[0][1]}.norm1"], p[f"l{subs[0][1]}.norm1.b"], eps, None, self.dtype) \
            if subs else None
        for n, (r, i, q) in enumerate(subs):
            sp, pre = self.specs[i], f"l{i}."
            if q == 2:
                y = self._ffn(sp["ffn"], pre, h)
            elif sp["type"] == "sloped_attention":
                y = self._sloped_attention(sp, pre, h, fb, meta, kv_caches[self.cache_index[r]])
            elif sp["type"] == "delta":
                y = self._delta(sp, pre, h, fb, meta, self.state_index[r])
            else:
                y = self._latent_attention(sp, pre, h, fb, meta, kv_caches[self.cache_index[r]])
            nxt = subs[n + 1] if n + 1 < len(subs) else None
            last_of_run = nxt is None or nxt[0] != r
            extra = e if (nxt is not None and last_of_run and nxt[0] in self.reentry) else None
            nw = nb = None
            if nxt is not None:
                nw, nb = p[f"l{nxt[1]}.norm{nxt[2]}"], p[f"l{nxt[1]}.norm{nxt[2]}.b"]
            if self.layer_probe is not None and last_of_run:
                # the probe sees the residual as the layer leaves it, before the embedding re-enters
                ops.post_norm_add_norm(x, y, p[pre + f"norm{q}b"], p[pre + f"norm{q}b.b"], eps, m, None, None, None, self.dtype)
                self.layer_probe(r, x)
                if extra is not None:
                    x += extra
                h = ops.layer_norm_rows(x, nw, nb, eps, None, self.dtype) if nxt is not None else None
            else:
                # the residual update fused with the next sublayer's norm
                h = ops.post_norm_add_norm(x, y, p[pre + f"norm{q}b"], p[pre + f"norm{q}b.b"], eps, m, extra, nw, nb,
                                           self.dtype)
        xf = ops.layer_norm_rows(x, p["final.norm"], p["final.norm.b"], eps, fb.logits_idx, self.dtype)
        return ops.linear_act(xf, p["head"], out_dtype=torch.float32)

    def _sloped_attention(self, sp, pre, h, fb, meta, cache):
        T = fb.num_tokens
        H, G, D = sp["heads"], sp["kv_heads"], sp["dim"]
        kc, vc = cache
        p = self.p
        z = ops.linear_act(h, p[pre + "qk"])
        q, k = z[:, :H * D].view(T, H, D), z[:, H * D:H * D + G * D].view(T, G, D)
        # normed queries (a copy) and normed keys (to the pages); the keys as projected are the values
        qp = ops.qk_norm_rope_kv(q, k, k, p[pre + "q.norm"], p[pre + "k.norm"], self.cfg.norm_eps, fb.positions,
                                 p[pre + "inv_freq"], fb.slots, kc, vc)
        o = ops.attn_window_paged(qp, kc, vc, meta["tables"], meta["row_cu"], fb.positions, sp["scale"],
                                  min(sp["window"], NO_WINDOW), 0, None, row_map=meta["row_map"],
                                  dist_bias=(p[pre + "slopes"], None),
                                  q_temp=(sp["qt_coef"], sp["qt_every"]) if sp["qt_coef"] else None)
        return ops.linear_act(o.view(T, H * vc.shape[2]), p[pre + "o"])

    def _delta(self, sp, pre, h, fb, meta, si):
        T = fb.num_tokens
        H, G, D, Dv = sp["heads"], sp["kv_heads"], sp["dim"], sp["vdim"]
        p = self.p
        hist, S = self.state[si], self.state[si + 1]
        z = ops.linear_act(h, p[pre + "in"])
        C = self._conv_channels(sp)
        zc = z[:, :C]
        y = ops.short_conv_act(zc, p[pre + "conv"], hist, meta["state_slots"], meta["row_cu"], fb.positions, "silu",
                               torch.float32)
        if sp["taps"] > 1:
            ops.short_conv_state_update_(zc, hist, meta["state_slots"], meta["row_cu"], fb.positions)
        q, k, v = y[:, :G * D].view(T, G, D), y[:, G * D:2 * G * D].view(T, G, D), y[:, 2 * G * D:].view(T, H, Dv)
        o1 = C + H * Dv
        o = ops.delta_scan(q, k, v, z[:, o1:o1 + H], z[:, o1 + H:o1 + 2 * H], p[pre + "A_log"], p[pre + "dt_bias"], S,
                           meta["state_slots"], meta["row_cu"], fb.positions, D ** -0.5, UNIT_EPS)
        g = ops.gla_out(o, z[:, C:o1], p[pre + "gnorm"], self.cfg.norm_eps, self.dtype)
        return ops.linear_act(g, p[pre + "o"])

    def _latent_attention(self, sp, pre, h, fb, meta, cache):
        T = fb.num_tokens
        H, D, Dv, R, rd = sp["heads"], sp["dim"], sp["vdim"], sp["kv_rank"], sp["rot_dim"]
        kc, vc = cache
        p = self.p
        z = ops.linear_act(h, p[pre + "in"])
        HQ = H * (D + rd)
        ops.latent_prep(z[:, HQ:], 0, R, rd, 0, None, p[pre + "dkv.norm"], self.cfg.norm_eps, fb.positions,
                        p[pre + "inv_freq"], fb.slots, kc, vc, self.dtype)
        q = z[:, :HQ].view(T, H, D + rd)
        # queries in the latent space: [W_uk^T q_plain | rotated q_rot] per head
        ql = ops.new_empty(T, H, kc.shape[3], dtype=self.dtype, device=self.device)
        ops.linear_heads(q[:, :, :D], p[pre + "ukT"], ql[:, :, :R])
        ops.rope_heads_copy(q[:, :, D:], ql[:, :, R:], fb.positions, p[pre + "inv_freq"])    # (zero-fills the padding)
        ol = ops.attn_window_paged(ql, kc, vc, meta["tables"], meta["row_cu"], fb.positions, sp["scale"],
                                   min(sp["window"], NO_WINDOW), 0, p[pre + "sink"], row_map=meta["row_map"],
                                   fold_heads=True)
        o = ops.new_empty(T, H, Dv, dtype=self.dtype, device=self.device)
        ops.linear_heads(ol[:, :, :R], p[pre + "uv"], o)
        return ops.linear_act(o.view(T, H * Dv), p[pre + "o"])

    def _ffn(self, fs, pre, h):
        p = self.p
        ids, w = ops.moe_route_scores(h, p[pre + "router"], fs["top"], scoring="softmax", renorm=False,
                                      select_bias=p[pre + "correction"])
        return ops.moe_glu_ffn(h, ids, w, p[pre + "up"], p[pre + "edown"], float("inf"), 1.0, up_offset=0.0,
                               scale_input=False, plain_act="relu2")
