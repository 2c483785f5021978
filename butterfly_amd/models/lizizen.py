"""Lizizen: a decoder-only LM of parallel layers with a token shift (ModelConfig.layer_specs,
ModelConfig.layer_runs).

  embedding   : x = table[token], an f32 residual
  every layer : n = x / rms(x);  h1 = n (1 + w1),  h2 = n (1 + w2)    (weights stored around zero,
                                         both inputs from the same x)
                h1 <- h1 + (h1_prev - h1) * shift    token shift: mixed per channel with the
                                         previous token's unmixed h1 (zeros before the first
                                         token); a sequence's last h1 of every layer run lives in
                                         the cache's per-sequence state slots
                x <- x + (mixer(h1) + ff(h2))
    mixer "biased_attention" : GQA without rotation; the scores lose a per-head distance bias
                        a_h ln(1 + b_h (i - j)); the query is scaled by a temperature that grows with
                        the logarithm of the position; causal over the whole sequence; softmax
                        with a zero-logit sink in the denominator
    mixer "diff_attention"   : two attention maps per head over the same values (query / key rows
                        laid out [head][map][dim]): per-(head, map) RMS norm with a shared
                        weight, rotation of dimension i with i + dims / 2, tanh cap on the scores,
                        keys visible inside the query's chunk of positions, ordinary softmax;
                        o = a1 - lambda a2 with one lambda per layer, unit RMS per head, a constant
                        factor, a sigmoid gate from the mixer's input; then the output projection
    feed-forward      : W_down (g sigmoid(1.702 g) (u + 1)) with g = min(W_gate h, L), u =
                        clamp(W_up h, +-L), all three with biases
  layer runs  : a span of layers may run several times in a row with the same weights; every run has
                its own pages and state
  output      : the offset-weight norm, logits = head x, f32

Every size and constant comes from the config; the residual, norms, the shift state, softmax,
angles and the differential combination run in f32 in the bf16 model too. Unsharded (tp = pp =
ep = 1). Prompt chunks always attend through the paged cache, so one attention op serves fresh
prompts, continuation chunks and decoded tokens.
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

NORM_OFFSET = 1.0       # norm weights are stored around zero
GLU_ALPHA = 1.702       # feed-forward activation g * sigmoid(alpha g)
GLU_UP_OFFSET = 1.0     # ... times (u + 1)
NO_WINDOW = 1 << 30     # plain causal attention


class LizizenLM(PackedStack):
    attention_types = ("biased_attention", "diff_attention")

    def __init__(self, cfg: ModelConfig, shard: Shard = Shard(), device="cpu",
                 dtype: torch.dtype = torch.bfloat16, comm: Optional[Communicator] = None):
        if not cfg.layer_specs:
            raise ValueError("Lizizen needs ModelConfig.layer_specs (ModelConfig.from_lizizen)")
        if shard.tp_size != 1 or shard.ep_size != 1 or shard.layer_start != 0 or \
                (shard.layer_end is not None and shard.layer_end != cfg.num_layers):
            raise NotImplementedError("Lizizen runs unsharded (tp = pp = ep = 1)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Lizizen runs in bfloat16 or float32")
        for sp in cfg.layer_specs:
            if sp["type"] not in self.attention_types:
                raise ValueError(f"layer {sp['index']}: Lizizen has no mixer {sp['type']!r}")
            if sp["ffn"] and sp["ffn"]["kind"] != "glu":
                raise ValueError(f"layer {sp['index']}: Lizizen has no feed-forward {sp['ffn']['kind']!r}")
        self.cfg, self.shard = cfg, shard
        self.device, self.dtype = torch.device(device), dtype
        self.comm = comm or Communicator.single()
        self.specs = cfg.layer_specs
        # layer indices in running order; run r owns cache pair r and state tensor r
        self.runs = list(cfg.layer_runs) if cfg.layer_runs is not None else list(range(cfg.num_layers))
        self.layer_ids = list(range(cfg.num_layers))
        self.first = self.last = True
        self.tp = self.ep = 1
        vpad = pad128(cfg.vocab_size)
        self.dims = LocalDims(hq=cfg.num_heads, hkv=cfg.num_kv_heads, kv_head0=0, q_head0=0,
                              ffn=max(cfg.intermediate_size, 1), ffn0=0, vocab=vpad, vocab0=0, vocab_padded=vpad,
                              experts=1, expert0=0)
        # cached head sizes: padded with zeros to sizes the attention's matrix-core form tiles
        self.cache_dims = {sp["index"]: (ops.attn_window_pad(sp["dim"], dtype), ops.attn_window_pad(sp["vdim"], dtype))
                           for sp in self.specs}
        # feed-forwards whose [gate | up] projection can run on the tuned GEMMs with the fused GLU
        # epilogue keep its rows (and biases) in alternating 16-row gate / up blocks
        self.glu_group = {sp["index"]: (ops.SILU_INTERLEAVE if (sp["ffn"] and dtype == torch.bfloat16
                                                                 and self.device.type == "cuda"
                                                                 and cfg.hidden_size % 64 == 0
                                                                 and sp["ffn"]["ff"] % 128 == 0) else 0)
                          for sp in self.specs}
        self.has_state = bool(self.runs)          # the token shift's previous input, per layer run
        self.state: list = []                     # set by allocate_state (the cache object owns the pool)
        self.layer_probe = None                   # debug hook: f(run, residual [T, W] f32) after every layer run
        self.p: dict[str, torch.Tensor] = {}
        self.packed: dict = {}
        self._arange: dict = {}
        self._lambda: dict = {}                   # layer -> lambda of its differential attention (float)
        self._alloc()

    # ------------------------------------------------------------------------------------
    # parameters
    # ------------------------------------------------------------------------------------
    def _wide(self, rows: int, k: int) -> int:
        """Rows of a projection: padded to the tuned GEMMs' 128-row tiling when its K fits them."""
        return pad128(rows) if k % 64 == 0 else rows

    def _alloc(self):
        c, W = self.cfg, self.cfg.hidden_size
        z = lambda *s: torch.zeros(*s, dtype=self.dtype, device=self.device)                  # noqa: E731
        f = lambda *s: torch.zeros(*s, dtype=torch.float32, device=self.device)               # noqa: E731
        p = self.p
        p["embed"] = z(c.vocab_size, W)
        for sp in self.specs:
            pre = f"l{sp['index']}."
            H, G, D, Dv, M = sp["heads"], sp["kv_heads"], sp["dim"], sp["vdim"], sp["maps"]
            Dvp = self.cache_dims[sp["index"]][1]
            p[pre + "norm1"], p[pre + "shift"] = f(W), f(W)
            if sp["type"] == "biased_attention":
                # one projection of the mixer's input: q | k | v
                p[pre + "qkv"] = z(self._wide(H * D + G * D + G * Dv, W), W)
                p[pre + "r1"], p[pre + "r2"], p[pre + "sink"] = f(H), f(H), f(H)     # the sink's logit is zero
                p[pre + "inv_freq"] = f(0)
                # the attention leaves heads of the padded value size: W_o carries zero columns there
                p[pre + "o"] = z(W, H * Dvp)
            else:
                # q (two maps per head) | k (two maps per head) | v | output gate
                p[pre + "qkvg"] = z(self._wide(M * H * D + M * G * D + G * Dv + H * Dv, W), W)
                p[pre + "q.norm"], p[pre + "k.norm"] = f(D), f(D)
                for n in ("lq1", "lk1", "lq2", "lk2"):
                    p[pre + n] = f(D)
                i = torch.arange(sp["rot_dims"] // 2, dtype=torch.float64)
                p[pre + "inv_freq"] = (sp["rot_base"] ** (-2.0 * i / max(sp["rot_dims"], 1))).to(torch.float32).to(self.device)
                p[pre + "o"] = z(W, H * Dv)
            fs = sp["ffn"]
            if fs:
                F = fs["ff"]
                p[pre + "norm2"] = f(W)
                if self.glu_group[sp["index"]]:
                    p[pre + "gate_up"] = z(2 * F, W)
                    p[pre + "gate_up.b"] = ops.glu_bias_block(z(2 * F), fs["limit"], GLU_ALPHA, GLU_UP_OFFSET)
                else:
                    p[pre + "gate_up"], p[pre + "gate_up.b"] = z(self._wide(2 * F, W), W), z(self._wide(2 * F, W))
                p[pre + "down"], p[pre + "down.b"] = z(self._wide(W, F), F), z(self._wide(W, F))
        p["final.norm"] = f(W)
        p["head"] = z(self.dims.vocab, W)             # rows past the vocabulary stay zero

    @property
    def head_weight(self) -> torch.Tensor:
        return self.p["head"]

    def logical_params(self) -> list[LogicalParam]:
        """Checkpoint tensors by their file names ('l<i>.mix.q', 'l<i>.mlp.gate.b', ...), each a view
        into the fused local tensors."""
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
            H, G, D, Dv, M = sp["heads"], sp["kv_heads"], sp["dim"], sp["vdim"], sp["maps"]
            add(L + "norm1", p[L + "norm1"], "norm")
            if sp["ffn"]:
                add(L + "norm2", p[L + "norm2"], "norm")
            if sp["type"] == "biased_attention":
                w = p[L + "qkv"]
                o1, o2 = H * D, H * D + G * D
                add(L + "mix.q", w[:o1])
                add(L + "mix.k", w[o1:o2])
                add(L + "mix.v", w[o2:o2 + G * Dv])
                add(L + "mix.r1", p[L + "r1"], "dist_a")
                add(L + "mix.r2", p[L + "r2"], "dist_b")
                ov = p[L + "o"].view(W, H, self.cache_dims[i][1])[:, :, :Dv]      # the columns of real values
                add(L + "mix.o", ov, shape=(W, H * Dv), get=lambda t=ov: t.reshape(t.shape[0], -1),
                    put=lambda x, t=ov: t.copy_(x.reshape(t.shape)))
            else:
                w = p[L + "qkvg"]
                o1 = M * H * D
                o2 = o1 + M * G * D
                o3 = o2 + G * Dv
                add(L + "mix.q", w[:o1])
                add(L + "mix.k", w[o1:o2])
                add(L + "mix.v", w[o2:o3])
                add(L + "mix.q.norm", p[L + "q.norm"], "ones")
                add(L + "mix.k.norm", p[L + "k.norm"], "ones")
                for n in ("lq1", "lk1", "lq2", "lk2"):
                    t = p[L + n]
                    add(L + "mix." + n, t, "small",
                        put=lambda x, t=t, i=i: (t.copy_(x.reshape(t.shape)), self._lambda.pop(i, None)))
                add(L + "mix.g", w[o3:o3 + H * Dv])
                add(L + "mix.o", p[L + "o"])
            fs = sp["ffn"]
            if fs:
                F, grp = fs["ff"], self.glu_group[i]
                if grp:        # alternating blocks of `grp` gate and up rows
                    wv, bv = p[L + "gate_up"].view(F // grp, 2, grp, W), p[L + "gate_up.b"][:2 * F].view(F // grp, 2, grp)
                    for j, n in enumerate(("gate", "up")):
                        add(L + "mlp." + n, wv[:, j], shape=(F, W), get=lambda t=wv[:, j]: t.reshape(-1, t.shape[-1]))
                        add(L + "mlp." + n + ".b", bv[:, j], "small", shape=(F,), get=lambda t=bv[:, j]: t.reshape(-1))
                else:
                    add(L + "mlp.gate", p[L + "gate_up"][:F])
                    add(L + "mlp.gate.b", p[L + "gate_up.b"][:F], "small")
                    add(L + "mlp.up", p[L + "gate_up"][F:2 * F])
                    add(L + "mlp.up.b", p[L + "gate_up.b"][F:2 * F], "small")
                add(L + "mlp.down", p[L + "down"][:W])
                add(L + "mlp.down.b", p[L + "down.b"][:W], "small")
            add(L + "shift", p[L + "shift"], "unit")
        add("final.norm", p["final.norm"], "norm")
        add("head", p["head"][:c.vocab_size])
        return out

    @torch.no_grad()
    def init_random(self, seed: int = 0) -> None:
        """Deterministic random weights: each tensor is drawn on the host from a generator keyed on
        (seed, tensor name). Projections are scaled by 1 / sqrt(fan-in), the embedding has unit
        entries, norm weights sit around zero, shifts are uniform in (0, 1), distance-bias numbers
        positive."""
        for lp in self.logical_params():
            g = torch.Generator().manual_seed(_name_seed(lp.name, seed))
            shp = lp.global_shape
            r = torch.randn(shp, generator=g)
            if lp.init == "normal":
                t = r / math.sqrt(shp[-1])
            elif lp.init == "embed":
                t = r
            elif lp.init == "norm":
                t = 0.1 * r
            elif lp.init == "ones":
                t = 1.0 + 0.1 * r
            elif lp.init == "small":
                t = 0.1 * r
            elif lp.init == "unit":
                t = torch.rand(shp, generator=g)
            elif lp.init == "dist_a":
                t = 0.2 + 0.8 * torch.rand(shp, generator=g)
            elif lp.init == "dist_b":
                t = 0.05 + 0.5 * torch.rand(shp, generator=g)
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
        for i in self.runs:
            sp, (Dp, Dvp) = self.specs[i], self.cache_dims[i]
            n += sp["kv_heads"] * (sp["maps"] * Dp + Dvp)
        return max(1, n * es)

    def state_bytes_per_slot(self) -> int:
        return 4 * self.cfg.hidden_size * len(self.runs)

    def allocate_kv_cache(self, num_blocks: int, block_size: int, dtype: Optional[torch.dtype] = None) -> list:
        """One (K [blocks, G * maps, BS, D], V [blocks, G, Dv, BS]) pair per layer run (a layer that
        runs twice caches twice), V with a page's tokens contiguous, head sizes padded with zeros."""
        dt = dtype or self.dtype
        if dt != self.dtype:
            raise NotImplementedError("Lizizen caches hold the model's element type")
        caches = []
        for i in self.runs:
            sp, (Dp, Dvp) = self.specs[i], self.cache_dims[i]
            G = sp["kv_heads"]
            caches.append((torch.zeros(num_blocks, G * sp["maps"], block_size, Dp, dtype=dt, device=self.device),
                           torch.zeros(num_blocks, G, Dvp, block_size, dtype=dt, device=self.device)))
        return caches

    def allocate_state(self, num_slots: int) -> list:
        """The token shift's pool: one [slots, W] f32 tensor per layer run (a sequence's last unmixed
        mixer input)."""
        self.state = [torch.zeros(num_slots, self.cfg.hidden_size, dtype=torch.float32, device=self.device)
                      for _ in self.runs]
        return self.state

    # ------------------------------------------------------------------------------------
    # forward
    # ------------------------------------------------------------------------------------
    def _diff_lambda(self, i: int, pre: str, diff: float) -> float:
        """exp(lq1 . lk1) - exp(lq2 . lk2) + diff of layer i, in f32, read once from the weights (a
        host float, before any graph capture)."""
        lam = self._lambda.get(i)
        if lam is None:
            p = self.p
            e1 = torch.exp((p[pre + "lq1"] * p[pre + "lk1"]).sum())
            e2 = torch.exp((p[pre + "lq2"] * p[pre + "lk2"]).sum())
            lam = self._lambda[i] = float(e1 - e2 + torch.tensor(diff, dtype=torch.float32))
        return lam

    def prepare(self) -> None:
        """Host-side constants derived from weights (read once, outside any graph capture)."""
        for sp in self.specs:
            if sp["type"] == "diff_attention":
                self._diff_lambda(sp["index"], f"l{sp['index']}.", sp["diff"])

    def forward(self, fb: ForwardBatch, kv_caches: Optional[list] = None,
                hidden_in: Optional[torch.Tensor] = None) -> torch.Tensor:
        """One step over the packed rows of `fb`; returns f32 logits [R, padded vocab] for the rows
        fb.logits_idx names (None: all)."""
        p, c, eps = self.p, self.cfg, self.cfg.norm_eps
        meta = self._step_meta(fb)
        meta["rope"] = {}
        T, W = fb.num_tokens, c.hidden_size
        if self.has_state and T and not self.state:
            raise RuntimeError("Lizizen: the token-shift pool is not allocated (KVCache state slots)")
        if kv_caches is None and self.runs:
            raise RuntimeError("Lizizen attention runs through the paged cache")
        # the residual alternates between two buffers: a row's update also reads its neighbour's old row
        bufs = [ops.new_empty(T, W, dtype=torch.float32, device=self.device) for _ in range(2)]
        x = ops.embed_scaled(fb.input_ids, p["embed"], 1.0, out=bufs[0])
        cur = 0
        ya = yb = None
        for r, i in enumerate(self.runs):
            sp = self.specs[i]
            pre = f"l{i}."
            x, ha, hb = ops.par_norm_shift(x, ya, yb, p[pre + "norm1"], p[pre + "norm2"] if sp["ffn"] else None, eps,
                                           NORM_OFFSET, p[pre + "shift"], self.state[r] if self.state else None,
                                           meta["state_slots"], meta["row_cu"], fb.positions, self.dtype,
                                           x_out=bufs[1 - cur], row_map=meta["row_map"])
            if ya is not None or yb is not None:
                cur = 1 - cur
            if self.layer_probe is not None and r > 0:
                self.layer_probe(r - 1, x)
            if sp["type"] == "biased_attention":
                ya = self._biased_attention(sp, pre, ha, fb, meta, kv_caches[r])
            else:
                ya = self._diff_attention(sp, pre, ha, fb, meta, kv_caches[r])
            yb = self._ffn(sp, pre, hb) if sp["ffn"] else None
        if self.layer_probe is not None and self.runs:
            self.layer_probe(len(self.runs) - 1, x + (ya.float() + (yb.float() if yb is not None else 0)))
        xf = ops.par_final(x, ya, yb, p["final.norm"], eps, NORM_OFFSET, fb.logits_idx, self.dtype)
        return ops.linear_act(xf, p["head"], out_dtype=torch.float32)

    def _biased_attention(self, sp, pre, h, fb, meta, cache):
        T = fb.num_tokens
        H, G, D, Dv = sp["heads"], sp["kv_heads"], sp["dim"], sp["vdim"]
        kc, vc = cache
        p = self.p
        z = ops.linear_act(h, p[pre + "qkv"])
        o1, o2 = H * D, H * D + G * D
        q, k, v = z[:, :o1].view(T, H, D), z[:, o1:o2].view(T, G, D), z[:, o2:o2 + G * Dv].view(T, G, Dv)
        qp = ops.qk_norm_rope_kv(q, k, v, None, None, self.cfg.norm_eps, fb.positions, p[pre + "inv_freq"], fb.slots, kc, vc)
        o = ops.attn_window_paged(qp, kc, vc, meta["tables"], meta["row_cu"], fb.positions, sp["scale"], NO_WINDOW, 0,
                                  p[pre + "sink"], row_map=meta["row_map"], dist_bias=(p[pre + "r1"], p[pre + "r2"]),
                                  q_temp=(sp["qt_coef"], sp["qt_every"]) if sp["qt_coef"] else None)
        return ops.linear_act(o.view(T, H * vc.shape[2]), p[pre + "o"])

    def _diff_attention(self, sp, pre, h, fb, meta, cache):
        T = fb.num_tokens
        H, G, D, Dv, M = sp["heads"], sp["kv_heads"], sp["dim"], sp["vdim"], sp["maps"]
        kc, vc = cache
        p, eps = self.p, self.cfg.norm_eps
        z = ops.linear_act(h, p[pre + "qkvg"])
        o1 = M * H * D
        o2 = o1 + M * G * D
        o3 = o2 + G * Dv
        q, k, v = z[:, :o1].view(T, M * H, D), z[:, o1:o2].view(T, M * G, D), z[:, o2:o3].view(T, G, Dv)
        # one rotation table per step for all layer runs that share (base, dims)
        key = (sp["rot_base"], sp["rot_dims"])
        if key not in meta["rope"]:
            meta["rope"][key] = ops.rope_table(fb.positions, p[pre + "inv_freq"])
        qp = ops.qk_norm_rope_kv(q, k, v, p[pre + "q.norm"], p[pre + "k.norm"], eps, fb.positions, p[pre + "inv_freq"],
                                 fb.slots, kc, vc, cs=meta["rope"][key])
        a = ops.attn_window_paged(qp, kc, vc, meta["tables"], meta["row_cu"], fb.positions, sp["scale"], NO_WINDOW, 0,
                                  None, row_map=meta["row_map"], chunk=sp["chunk"] if sp["chunk"] < NO_WINDOW else 0,
                                  softcap=sp["softcap"], maps=M, out_dtype=torch.float32)
        o = ops.diff_combine(a, self._diff_lambda(sp["index"], pre, sp["diff"]), eps, 1.0 - sp["diff"],
                             z[:, o3:o3 + H * Dv], Dv, self.dtype)
        return ops.linear_act(o, p[pre + "o"])

    def _ffn(self, sp, pre, h):
        fs = sp["ffn"]
        p, W, F = self.p, self.cfg.hidden_size, fs["ff"]
        a = ops.linear_glu(h, p[pre + "gate_up"], p[pre + "gate_up.b"], F, fs["limit"], GLU_ALPHA, GLU_UP_OFFSET,
                           self.glu_group[sp["index"]])
        y = ops.linear_act(a, p[pre + "down"], bias=p[pre + "down.b"])
        return y if y.shape[1] == W else y[:, :W].contiguous()
