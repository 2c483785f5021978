"""Lizizen (models/lizizen.py) against the plain float64 implementation in tests/lizizen_oracle.py:
every mechanism alone, then whole models through the engine: prefill vs token-by-token decoding,
prompt portions of many sizes, mixed batches of unequal requests, pages and state slots that are
freed and used again, chunk and page edges, far keys, the sink, the first tokens, long decoding,
looped layer spans, greedy generation through the scheduler. Each case runs on the CPU reference
ops (f32) and, marked gpu, on the HIP kernels in f32 and bf16. Configurations and weights are made
here; nothing is read from disk but what a test wrote itself."""
import json

import pytest
import torch
from safetensors.torch import save_file

from butterfly_amd import ops
from butterfly_amd.ckpt import load_into, model_config
from butterfly_amd.config import EngineConfig, ModelConfig
from butterfly_amd.engine.engine import LLMEngine
from butterfly_amd.engine.sampler import SamplingParams
from butterfly_amd.models import build_model

from . import lizizen_oracle as O

gpu = pytest.mark.gpu
TARGETS = [pytest.param(("cpu", torch.float32), id="cpu-f32"),
           pytest.param(("cuda", torch.float32), id="gpu-f32", marks=gpu),
           pytest.param(("cuda", torch.bfloat16), id="gpu-bf16", marks=gpu)]
F64 = torch.float64


@pytest.fixture(params=TARGETS)
def target(request):
    dev, dt = request.param
    if dev == "cuda":
        if not torch.cuda.is_available():
            pytest.skip("no GPU")
        ops.require_library()
    return torch.device(dev), dt


def rel_err(got, want):
    """Per-row error as a logit comparison sees it: mean removed, RMS over the last dim, relative
    to the RMS of the expected row."""
    got, want = got.detach().cpu().to(F64), want.to(F64)
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / (w.pow(2).mean(-1).sqrt() + 1e-9)


def assert_rows(got, want, dt, what=""):
    e = rel_err(got, want).flatten()
    if dt == torch.float32:
        assert e.max() < 3e-4, f"{what}: worst row {int(e.argmax())} err {e.max():.3g}"
    else:
        # bf16 rounding in models this narrow is a few percent per row; the f32 runs carry the
        # exact comparison, this one checks that the bf16 kernels compute the same thing
        assert e.median() < 0.05 and e.quantile(0.9) < 0.15, \
            f"{what}: median {e.median():.3g}, 90th percentile {e.quantile(0.9):.3g}"


def bf(t):
    """bf16-representable f64 values (every tensor a bf16 run sees exactly)."""
    return t.to(torch.bfloat16).to(F64)


def close(got, want, dt, f32_tol=2e-5, bf16_tol=2e-2):
    want = want.to(F64)
    err = (got.detach().cpu().to(F64) - want).abs().max()
    return err < (f32_tol if dt == torch.float32 else bf16_tol) * (1 + want.abs().max())


def i32(v, dev):
    return torch.tensor(v, dtype=torch.int32, device=dev)


def rnd(*shape, seed=0, scale=1.0):
    return bf(torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F64) * scale)


# ---------------------------------------------------------------------------------------
# mechanisms alone
# ---------------------------------------------------------------------------------------
def packed_step(seqs, dev):
    """seqs: [(first position, rows)] -> row_cu, positions of a packed step."""
    cu, pos = [0], []
    for p0, n in seqs:
        cu.append(cu[-1] + n)
        pos += list(range(p0, p0 + n))
    return i32(cu, dev), i32(pos, dev)


@pytest.mark.parametrize("W", [24, 200, 1030])
def test_layer_step_norms_token_shift_and_state(target, W):
    """x + (ya + yb), both offset-weight norms of the sum, the token shift through packed steps:
    three sequences cut into portions of 1, 2 and more rows, one of them in a slot another sequence
    used before, a sequence that pauses for a step; and the output norm of chosen rows."""
    dev, dt = target
    lens = [13, 6, 9]
    x = [rnd(n, W, seed=10 + s) for s, n in enumerate(lens)]
    ya = [rnd(n, W, seed=20 + s) for s, n in enumerate(lens)]
    yb = [rnd(n, W, seed=30 + s) for s, n in enumerate(lens)]
    wa, wb, sh = rnd(W, seed=1, scale=0.2), rnd(W, seed=2, scale=0.2), bf(torch.rand(W, dtype=F64))
    eps = 1e-5
    want_a, want_b, want_x = [], [], []
    for s in range(3):
        xs = x[s] + (ya[s] + yb[s])
        want_x.append(xs)
        want_a.append(O.token_shift(O.offset_norm(xs, wa, eps), sh))
        want_b.append(O.offset_norm(xs, wb, eps))
    state = torch.full((2, W), 7.0, dtype=torch.float32, device=dev)      # stale values: never read at position 0
    slot = [1, 0, 1]                          # sequence 2 takes the slot sequence 0 leaves
    steps = [[(0, 2), (1, 1)], [(0, 1), (1, 2)], [(0, 7)], [(0, 1), (1, 3)], [(0, 2)],
             [(2, 1)], [(2, 1)], [(2, 5)], [(2, 2)]]
    at = [0, 0, 0]
    got_a = [[] for _ in lens]
    got_b = [[] for _ in lens]
    got_x = [[] for _ in lens]
    g = lambda t: t.to(dt).to(dev)                                    # noqa: E731
    for step in steps:
        cu, pos = packed_step([(at[s], c) for s, c in step], dev)
        rows = lambda src: torch.cat([src[s][at[s]:at[s] + c] for s, c in step])      # noqa: E731
        xn, ha, hb = ops.par_norm_shift(rows(x).float().to(dev), g(rows(ya)), g(rows(yb)), wa.float().to(dev),
                                        wb.float().to(dev), eps, 1.0, sh.float().to(dev), state,
                                        i32([slot[s] for s, _ in step], dev), cu, pos, dt)
        r = 0
        for s, c in step:
            got_a[s].append(ha[r:r + c]), got_b[s].append(hb[r:r + c]), got_x[s].append(xn[r:r + c])
            r += c
            at[s] += c
    assert at == lens
    for s in range(3):
        assert close(torch.cat(got_x[s]), want_x[s], torch.float32), f"sum, sequence {s}"
        assert close(torch.cat(got_a[s]), want_a[s], dt), f"shifted mixer input, sequence {s}"
        assert close(torch.cat(got_b[s]), want_b[s], dt), f"feed-forward input, sequence {s}"
    # no outputs of a previous layer (the first layer), no second norm (a layer without feed-forward)
    cu, pos = packed_step([(0, 5)], dev)
    xn, ha, hb = ops.par_norm_shift(x[1][:5].float().to(dev), None, None, wa.float().to(dev), None, eps, 1.0,
                                    sh.float().to(dev), state, i32([0], dev), cu, pos, dt)
    assert hb is None and close(ha, O.token_shift(O.offset_norm(x[1][:5], wa, eps), sh), dt)
    idx = torch.tensor([0, 4, 12], device=dev)
    out = ops.par_final(x[0].float().to(dev), g(ya[0]), None, wb.float().to(dev), eps, 1.0, idx, dt)
    assert close(out, O.offset_norm(x[0] + ya[0], wb, eps)[idx.cpu()], dt)


@pytest.mark.parametrize("M,F,K,limit", [(5, 7, 13, 1.0), (70, 130, 50, 0.5), (3, 128, 128, 7.0), (300, 192, 64, 1.0),
                                         (16, 256, 256, 1.0), (700, 512, 128, 0.75), (40, 1024, 1024, 1.0)])
def test_clamped_glu_feed_forward(target, M, F, K, limit):
    """min(gate, L) sigmoid(1.702 .) (clamp(up, +-L) + 1) between two biased projections, on shapes
    the tuned matrix-core GEMMs take and on odd ones; inputs large enough that every clamp acts."""
    dev, dt = target
    w = {"gate": rnd(F, K, seed=1, scale=K ** -0.5), "gate.b": rnd(F, seed=2, scale=0.3),
         "up": rnd(F, K, seed=3, scale=K ** -0.5), "up.b": rnd(F, seed=4, scale=0.3),
         "down": rnd(K, F, seed=5, scale=F ** -0.5), "down.b": rnd(K, seed=6, scale=0.3)}
    h = rnd(M, K, seed=7, scale=2.0)
    want = O.glu_ffn(h, w, "", {"limit": limit})
    g = lambda t: t.to(dt).to(dev)                                    # noqa: E731
    pad = (2 * F + 127) // 128 * 128 if K % 64 == 0 else 2 * F
    wgu, bgu = torch.zeros(pad, K, dtype=F64), torch.zeros(pad, dtype=F64)
    wgu[:F], wgu[F:2 * F], bgu[:F], bgu[F:2 * F] = w["gate"], w["up"], w["gate.b"], w["up.b"]
    gu = ops.linear_act(g(h), g(wgu), bias=g(bgu))
    a = ops.glu_clamp(gu[:, :2 * F], limit, 1.702, 1.0)
    y = ops.linear_act(a, g(w["down"]), bias=g(w["down.b"]))
    assert close(y, want, dt, f32_tol=3e-5, bf16_tol=3e-2)
    # the same through linear_glu, and with gate / up rows in alternating 16-row blocks (the layout
    # of the GEMMs' fused epilogue, which bf16 shapes the tuned GEMMs take run as one kernel)
    a2 = ops.linear_glu(g(h), g(wgu), g(bgu), F, limit, 1.702, 1.0, 0)
    assert close(ops.linear_act(a2, g(w["down"]), bias=g(w["down.b"])), want, dt, f32_tol=3e-5, bf16_tol=3e-2)
    if F % 16 == 0:
        wi = ops.interleave_gate_up(w["gate"], w["up"], 16)
        bi = ops.interleave_gate_up(w["gate.b"][:, None], w["up.b"][:, None], 16)[:, 0]
        blk = ops.glu_bias_block(g(bi), limit, 1.702, 1.0)
        if dt == torch.float32:
            blk = blk.float()          # (an f32 run never takes the fused kernel: plain biases)
            blk[2 * F:] = 0
        a3 = ops.linear_glu(g(h), g(wi), blk, F, limit, 1.702, 1.0, 16)
        assert a3.shape == (M, F)
        assert close(ops.linear_act(a3, g(w["down"]), bias=g(w["down.b"])), want, dt, f32_tol=3e-5, bf16_tol=3e-2)


class Paged:
    """A paged cache for a few sequences with shuffled pages, filled step by step through the
    framework's own append (ops.qk_norm_rope_kv)."""

    def __init__(self, lens, Gk, Gv, D, Dv, dev, dt, bs=32, seed=0):
        self.bs, self.dev, self.dt = bs, dev, dt
        self.Dp, self.Dvp = ops.attn_window_pad(D, dt), ops.attn_window_pad(Dv, dt)
        nb = [(n + bs - 1) // bs for n in lens]
        order = torch.randperm(sum(nb) + 2, generator=torch.Generator().manual_seed(seed)).tolist()
        self.tables = torch.zeros(len(lens), max(nb), dtype=torch.int32)
        for s, n in enumerate(nb):
            for b in range(n):
                self.tables[s, b] = order.pop()
        self.kc = torch.zeros(sum(nb) + 2, Gk, bs, self.Dp, dtype=dt, device=dev)
        self.vc = torch.zeros(sum(nb) + 2, Gv, self.Dvp, bs, dtype=dt, device=dev)

    def step(self, step, at, q, k, v, prep, attn):
        """step [(sequence, rows)] from positions at[s]: prepare (prep = norm weights, eps,
        frequencies), append, attend; -> out rows [T, Hq, Dvp]."""
        dev, g = self.dev, (lambda t: t.to(self.dt).to(self.dev))
        cu, pos = packed_step([(at[s], c) for s, c in step], dev)
        slots = [int(self.tables[s, j // self.bs]) * self.bs + j % self.bs for s, c in step for j in range(at[s], at[s] + c)]
        rows = lambda src: g(torch.cat([src[s][at[s]:at[s] + c] for s, c in step]))      # noqa: E731
        qn, kn, eps, inv = prep
        qp = ops.qk_norm_rope_kv(rows(q), rows(k), rows(v), qn, kn, eps, pos, inv, i32(slots, dev), self.kc, self.vc)
        tab = self.tables[[s for s, _ in step]].to(dev)
        return ops.attn_window_paged(qp, self.kc, self.vc, tab, cu, pos, row_map=None, **attn)


def aim(q, k, pairs, scale, heads_per_kv, strength=14.0):
    """Make query row i (all heads) point at key row j: its score there stands out by `strength`."""
    for i, j in pairs:
        for h in range(q.shape[1]):
            kj = k[j, h // heads_per_kv]
            q[i, h] = bf(kj * strength / (scale * kj.pow(2).sum()))
    return q


STEPS = [[(0, 150), (1, 1)], [(0, 2), (1, 1), (2, 40)], [(0, 1), (1, 2)], [(0, 1), (2, 30)], [(0, 33), (1, 3)],
         [(0, 1), (1, 26)], [(0, 64)]] + [[(0, 1), (2, 1)]] * 8


@pytest.mark.parametrize("H,G,D,Dv,coef,every", [(6, 3, 20, 12, 0.5, 7), (8, 2, 64, 64, 0.25, 100), (4, 4, 40, 96, 0.0, 1),
                                                 (2, 1, 128, 32, 1.0, 1)])
def test_distance_biased_attention_with_sink(target, H, G, D, Dv, coef, every):
    """Causal attention over hundreds of cached keys in prompts, portions and decoded rows: queries
    aimed at the first key, at keys far back, at page borders and at themselves; rows whose scores
    are all very low, so that the sink takes nearly all the weight; the temperature steps with the
    position; three sequences share steps and shuffled pages."""
    dev, dt = target
    lens = [260, 33, 78]
    scale = 0.3
    q = [rnd(n, H, D, seed=40 + s) for s, n in enumerate(lens)]
    k = [rnd(n, G, D, seed=50 + s) for s, n in enumerate(lens)]
    v = [rnd(n, G, Dv, seed=60 + s) for s, n in enumerate(lens)]
    aim(q[0], k[0], [(259, 0), (258, 3), (255, 31), (254, 32), (200, 63), (199, 64), (150, 150), (149, 1), (257, 129)],
        scale, H // G)
    aim(q[2], k[2], [(77, 0), (70, 31), (69, 32), (40, 39)], scale, H // G)
    u = rnd(D, seed=9)
    for j in range(lens[1]):
        k[1][j] = bf(k[1][j] * 0.05 + u)              # a common direction in every key of sequence 1 ...
    for i in (5, 20, 32):
        q[1][i] = bf(-u * 12.0 / (scale * u.pow(2).sum())).expand(H, D)    # ... that these queries point away from
    r1, r2 = bf(0.2 + 0.8 * torch.rand(H, dtype=F64)), bf(0.05 + 0.5 * torch.rand(H, dtype=F64))
    want = [O.biased_attend(q[s], k[s], v[s], r1, r2, scale, coef, every) for s in range(3)]
    assert want[1][20].abs().max() < 1e-2 * want[1][19].abs().max()          # the sink has the weight there
    cache = Paged(lens, G, G, D, Dv, dev, dt)
    inv = torch.zeros(0, dtype=torch.float32, device=dev)
    attn = dict(scale=scale, window=1 << 30, keep_first=0, sink=torch.zeros(H, dtype=torch.float32, device=dev),
                dist_bias=(r1.float().to(dev), r2.float().to(dev)), q_temp=(coef, every) if coef else None)
    at, got = [0, 0, 0], [[], [], []]
    for step in STEPS:
        out = cache.step(step, at, q, k, v, (None, None, 1e-5, inv), attn)
        r = 0
        for s, c in step:
            got[s].append(out[r:r + c, :, :Dv])
            r += c
            at[s] += c
    assert at == lens
    for s in range(3):
        assert close(torch.cat(got[s]), want[s], dt, f32_tol=2e-5, bf16_tol=2.5e-2), f"sequence {s}"


@pytest.mark.parametrize("H,G,D,Dv,chunk,cap,dims", [(3, 1, 20, 12, 7, 3.0, 8), (4, 2, 64, 64, 40, 0.0, 64), (2, 2, 40, 96, 64, 30.0, 20),
                                                     (4, 2, 32, 128, 33, 2.0, 0), (2, 1, 16, 16, 1, 0.0, 4)])
def test_chunked_two_map_attention(target, H, G, D, Dv, chunk, cap, dims):
    """Two maps per head over shared values, normed and half-rotated, keys of the query's own chunk
    only: queries aimed at the first key of their chunk (seen) and at the key just before it (not
    seen), in prompts, portions and decoded rows, with chunk borders inside pages, at page borders
    and across steps; scores large enough that the cap acts; f32 outputs."""
    dev, dt = target
    lens = [260, 33, 78]
    scale, eps, base = 14.0 / D, 1e-5, 300.0       # an aimed pair scores about 14
    q = [rnd(n, H, 2, D, seed=70 + s) for s, n in enumerate(lens)]
    k = [rnd(n, G, 2, D, seed=80 + s) for s, n in enumerate(lens)]
    v = [rnd(n, G, Dv, seed=90 + s) for s, n in enumerate(lens)]
    qn, kn = bf(1 + 0.2 * torch.randn(D, dtype=F64)), bf(1 + 0.2 * torch.randn(D, dtype=F64))
    # aimed before norm and rotation: the norm keeps a direction, the rotation turns part of it away
    for s in (0, 2):
        n = lens[s]
        for i in list(range(n - 12, n)) + [150, 151, 185, 186]:
            if i >= n:
                continue
            c0 = i - i % chunk
            j = c0 if (i % 2 == 0 or c0 == 0) else c0 - 1        # first key of the chunk / the key before it
            for h in range(H):
                for m in range(2):
                    q[s][i, h, m] = bf(k[s][j, h // (H // G), m] * 3.0)
    want = []
    for s in range(3):
        qq = O.normed_rotated(q[s], qn, eps, base, dims)
        kk = O.normed_rotated(k[s], kn, eps, base, dims)
        want.append(O.chunk_attend(qq, kk, v[s], scale, cap, chunk).reshape(lens[s], 2 * H, Dv))
    cache = Paged(lens, 2 * G, G, D, Dv, dev, dt, seed=3)
    inv = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64).float().to(dev)
    attn = dict(scale=scale, window=1 << 30, keep_first=0, sink=None, chunk=chunk, softcap=cap, maps=2,
                out_dtype=torch.float32)
    flat = lambda t: [x.reshape(x.shape[0], -1, x.shape[-1]) for x in t]      # noqa: E731
    at, got = [0, 0, 0], [[], [], []]
    for step in STEPS:
        out = cache.step(step, at, flat(q), flat(k), v, (qn.float().to(dev), kn.float().to(dev), eps, inv), attn)
        assert out.dtype == torch.float32
        r = 0
        for s, c in step:
            got[s].append(out[r:r + c, :, :Dv])
            r += c
            at[s] += c
    for s in range(3):
        assert close(torch.cat(got[s]), want[s], dt, f32_tol=3e-5, bf16_tol=4e-2), f"sequence {s}"


@pytest.mark.parametrize("kind", ["biased", "two_map"])
def test_attention_decoding_over_long_contexts(target, kind):
    """Decoded rows over a thousand cached tokens (on the GPU the pages of a row are then split over
    several workgroups and merged), two sequences per step, then a short portion: a far key, the
    first key, the sink's share and a long chunk's first key are all met."""
    dev, dt = target
    lens = [1060, 700]
    steps = [[(0, 1000), (1, 650)]] + [[(0, 1), (1, 1)]] * 30 + [[(0, 30), (1, 20)]]
    if kind == "biased":
        H, G, D, Dv, scale = 4, 2, 64, 64, 0.2
        q = [rnd(n, H, D, seed=140 + s) for s, n in enumerate(lens)]
        k = [rnd(n, G, D, seed=150 + s) for s, n in enumerate(lens)]
        v = [rnd(n, G, Dv, seed=160 + s) for s, n in enumerate(lens)]
        aim(q[0], k[0], [(1005, 0), (1010, 17), (1020, 999), (1029, 512), (1040, 31)], scale, H // G)
        aim(q[1], k[1], [(660, 1), (679, 640), (690, 300)], scale, H // G)
        r1, r2 = bf(0.2 + 0.8 * torch.rand(H, dtype=F64)), bf(0.05 + 0.5 * torch.rand(H, dtype=F64))
        want = [O.biased_attend(q[s], k[s], v[s], r1, r2, scale, 0.5, 300) for s in range(2)]
        cache = Paged(lens, G, G, D, Dv, dev, dt, seed=5)
        prep = (None, None, 1e-5, torch.zeros(0, dtype=torch.float32, device=dev))
        attn = dict(scale=scale, window=1 << 30, keep_first=0, sink=torch.zeros(H, dtype=torch.float32, device=dev),
                    dist_bias=(r1.float().to(dev), r2.float().to(dev)), q_temp=(0.5, 300))
        qs, ks = q, k
    else:
        H, G, D, Dv, chunk, cap, dims, base, eps = 2, 1, 32, 64, 600, 8.0, 16, 1e4, 1e-5
        scale = 14.0 / D
        q = [rnd(n, H, 2, D, seed=170 + s) for s, n in enumerate(lens)]
        k = [rnd(n, G, 2, D, seed=180 + s) for s, n in enumerate(lens)]
        v = [rnd(n, G, Dv, seed=190 + s) for s, n in enumerate(lens)]
        for s, rows in ((0, range(1000, 1060, 7)), (1, range(650, 700, 5))):
            for i in rows:
                j = i - i % chunk if i % 2 else i - i % chunk - 1          # first key of the chunk / the key before it
                q[s][i] = bf(k[s][j, 0] * 3.0).expand(H, 2, D)
        qn, kn = bf(1 + 0.2 * torch.randn(D, dtype=F64)), bf(1 + 0.2 * torch.randn(D, dtype=F64))
        want = [O.chunk_attend(O.normed_rotated(q[s], qn, eps, base, dims), O.normed_rotated(k[s], kn, eps, base, dims),
                               v[s], scale, cap, chunk).reshape(lens[s], 2 * H, Dv) for s in range(2)]
        cache = Paged(lens, 2 * G, G, D, Dv, dev, dt, seed=6)
        inv = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64).float().to(dev)
        prep = (qn.float().to(dev), kn.float().to(dev), eps, inv)
        attn = dict(scale=scale, window=1 << 30, keep_first=0, sink=None, chunk=chunk, softcap=cap, maps=2,
                    out_dtype=torch.float32)
        qs, ks = [x.reshape(x.shape[0], -1, D) for x in q], [x.reshape(x.shape[0], -1, D) for x in k]
    at, got = [0, 0], [[], []]
    for step in steps:
        out = cache.step(step, at, qs, ks, v, prep, attn)
        r = 0
        for s, c in step:
            got[s].append(out[r:r + c, :, :Dv])
            r += c
            at[s] += c
    assert at == lens
    for s in range(2):
        assert close(torch.cat(got[s]), want[s], dt, f32_tol=3e-5, bf16_tol=4e-2), f"sequence {s}"


def test_query_key_preparation_and_cache_append(target):
    """Per-head norm with a shared weight, rotation of dimension i with i + n on the first 2 n
    dimensions only, zero padding of the query, K rows and transposed V rows at their slots (a
    page crossing, a row without a slot)."""
    dev, dt = target
    T, Hq, Gk, Gv, D, Dv, bs, n = 9, 5, 2, 1, 24, 10, 32, 5
    q, k, v = rnd(T, Hq, D, seed=1), rnd(T, Gk, D, seed=2), rnd(T, Gv, Dv, seed=3)
    qn, kn = bf(1 + 0.3 * torch.randn(D, dtype=F64)), bf(1 + 0.3 * torch.randn(D, dtype=F64))
    pos = [28, 29, 30, 31, 32, 33, 0, 1000, 7]
    slots = [3 * bs + 28, 3 * bs + 29, 3 * bs + 30, 3 * bs + 31, 1 * bs + 0, 1 * bs + 1, 0, -1, 2 * bs + 7]
    base = 50.0
    f = torch.tensor([base ** (-2.0 * i / (2 * n)) for i in range(n)], dtype=F64)

    def want(x, w):
        x = O.rms(x, 1e-6) * w
        out = x.clone()
        for t in range(T):
            a = pos[t] * f
            u, z = x[t, :, :n], x[t, :, n:2 * n]
            out[t, :, :n] = u * torch.cos(a) - z * torch.sin(a)
            out[t, :, n:2 * n] = z * torch.cos(a) + u * torch.sin(a)
        return out

    Dp, Dvp = ops.attn_window_pad(D, dt), ops.attn_window_pad(Dv, dt)
    kc = torch.zeros(5, Gk, bs, Dp, dtype=dt, device=dev)
    vc = torch.zeros(5, Gv, Dvp, bs, dtype=dt, device=dev)
    g = lambda t: t.to(dt).to(dev)                                    # noqa: E731
    qp = ops.qk_norm_rope_kv(g(q), g(k), g(v), qn.float().to(dev), kn.float().to(dev), 1e-6, i32(pos, dev),
                             f.float().to(dev), i32(slots, dev), kc, vc)
    assert qp.shape == (T, Hq, Dp) and close(qp[:, :, :D], want(q, qn), dt)
    assert float(qp[:, :, D:].abs().sum()) == 0
    wk = want(k, kn)
    for t, sl in enumerate(slots):
        if sl >= 0:
            assert close(kc[sl // bs, :, sl % bs, :D], wk[t], dt), t
            assert close(vc[sl // bs, :, :Dv, sl % bs], v[t], dt), t
    assert int((kc.float().abs().sum(-1) > 0).sum()) == 8 * Gk           # nothing else was written


@pytest.mark.parametrize("T,H,Dv", [(1, 1, 8), (7, 3, 20), (40, 4, 96), (3, 2, 300)])
def test_map_difference_unit_norm_and_gate(target, T, H, Dv):
    dev, dt = target
    Dvp = ops.attn_window_pad(Dv, dt)
    a = rnd(T, H, 2, Dv, seed=5)
    gate = rnd(T, H * Dv + 16, seed=6)
    lam, diff, eps = 0.83, 0.3, 1e-5
    want = (O.combine_maps(a, lam, diff, eps).reshape(T, H * Dv) * torch.sigmoid(gate[:, :H * Dv]))
    ap = torch.full((T, 2 * H, Dvp), 3.0, dtype=torch.float32)          # padding the op must not read into the norm
    ap[:, :, :Dv] = a.reshape(T, 2 * H, Dv).float()
    out = ops.diff_combine(ap.to(dev), lam, eps, 1.0 - diff, gate.to(dt).to(dev)[:, :H * Dv], Dv, dt)
    assert close(out, want, dt)


# ---------------------------------------------------------------------------------------
# whole models through the engine
# ---------------------------------------------------------------------------------------
def cfg_a():
    """Layers that differ from one another in every size; sizes no MFMA tile divides; chunks
    shorter than a page; a layer without feed-forward; the middle span of layers runs three times."""
    return O.config([
        O.biased_layer(6, 3, 12, 20, 0.3, 0.5, 5, O.dense(56, 1.0)),
        O.diff_layer(3, 1, 10, 6, 0.4, 0.65, 7, 100.0, 4, 3.0, O.dense(24, 0.5)),
        O.biased_layer(2, 2, 8, 8, 0.25, 0.25, 16, None),
        O.diff_layer(4, 2, 6, 14, 0.5, 0.2, 40, 1e4, 6, 20.0, O.dense(40, 2.0)),
    ], width=40, vocab=70, eps=1e-5, loop=(1, 3, 3))


def cfg_b():
    """What another model may make equal or 1 made unequal here, and the other way round: one
    head, as many key heads as query heads, a chunk of one position and one longer than the
    sequences, every dimension rotated and none, no cap, no temperature, a temperature that steps
    at every position, no repeated span, one feed-forward limit that never acts."""
    layers = [
        O.diff_layer(1, 1, 16, 24, 0.25, 0.8, 4096, 500.0, 16, 0.0, O.dense(20, 1e9)),
        O.biased_layer(5, 5, 4, 4, 0.5, 0.0, 1, O.dense(16, 1.0)),
        O.diff_layer(2, 2, 8, 12, 0.3, 0.1, 1, 50.0, 0, 5.0, O.dense(32, 1.0)),
        O.biased_layer(1, 1, 24, 8, 0.2, 1.0, 1, O.dense(32, 0.25)),
    ]
    del layers[2]["mixer"]["rot"]
    del layers[0]["mixer"]["softcap"]
    del layers[1]["mixer"]["q_temp"]
    return O.config(layers, width=48, vocab=50, eps=1e-6)


def cfg_c():
    """Sizes the matrix-core kernels tile (bf16): heads of 64 / 64, 32 / 128 and 128 / 32, chunks
    that end inside a page and on a page border, a width the tuned GEMMs take, the first two layers
    run twice."""
    return O.config([
        O.biased_layer(8, 2, 64, 64, 0.125, 0.5, 48, O.dense(256, 1.0)),
        O.diff_layer(4, 2, 32, 128, 0.18, 0.55, 40, 2e5, 16, 30.0, O.dense(128, 1.0)),
        O.diff_layer(2, 1, 128, 32, 0.09, 0.4, 64, 1e4, 128, 45.0, O.dense(256, 3.0)),
    ], width=128, vocab=256, eps=1e-5, loop=(0, 2, 2))


_ORACLE = {}


def oracle_logits(name, cfg, W, tokens):
    key = (name, tuple(tokens))
    if key not in _ORACLE:
        _ORACLE[key] = O.forward(cfg, W, tokens)
    return _ORACLE[key]


def write_model(tmp_path, cfg, W):
    d = tmp_path / "model"
    d.mkdir(exist_ok=True)
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in W.items()}, str(d / "model.safetensors"))
    return str(d)


def make_engine(tmp_path, cfg, W, dev, dt, max_batch=4, cache_tokens=512, graphs=False, **kw):
    d = write_model(tmp_path, cfg, W)
    mc = model_config(d)
    assert mc.arch == "lizizen"
    m = build_model(mc, device=dev, dtype=dt)
    assert load_into(m, d) == []
    ecfg = EngineConfig(max_batch=max_batch, max_seq_len=cache_tokens, max_prefill_tokens=kw.pop("budget", cache_tokens),
                        kv_cache_tokens=cache_tokens, use_graphs=graphs, dtype="fp32" if dt == torch.float32 else "bf16",
                        async_decode=kw.pop("async_decode", False), graph_batch_sizes=[1, 2, 4], **kw)
    return LLMEngine(mc, engine_cfg=ecfg, model=m, device=dev)


def tokens_of(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def replay(eng, reqs, schedule):
    """Run `schedule` (steps of [(name, count)]) asking for every row; -> {name: logits [len, V]}."""
    at = {n: 0 for n in reqs}
    rid = {n: i for i, n in enumerate(reqs)}
    out = {n: [] for n in reqs}
    for step in schedule:
        entries, end = [], []
        for n, c in step:
            entries.append((rid[n], reqs[n][at[n]:at[n] + c], list(range(c))))
            at[n] += c
            if at[n] == len(reqs[n]):
                end.append(rid[n])
        lg = eng.replay_step(entries, end).cpu()
        r = 0
        for n, c in step:
            out[n].append(lg[r:r + c])
            r += c
    assert all(at[n] == len(reqs[n]) for n in reqs)
    return {n: torch.cat(v) for n, v in out.items()}


def test_weights_round_trip_and_layer_outputs(tmp_path):
    """Loading a folder and reading the tensors back gives the file's tensors (also the fused and
    padded ones), and every layer run hands on what the oracle's layer does."""
    cfg = cfg_a()
    W = O.random_weights(cfg, seed=5)
    eng = make_engine(tmp_path, cfg, W, torch.device("cpu"), torch.float32)
    back = {lp.name: lp.get() for lp in eng.model.logical_params()}
    assert set(back) == set(W)
    for k, v in W.items():
        assert torch.equal(back[k].reshape(v.shape).float(), v.float()), k
    toks = tokens_of(cfg, 20, 1)
    seen, want = [], []
    eng.model.layer_probe = lambda i, x: seen.append(x.clone())
    eng.replay_step([(0, toks, [0])], [0])
    O.forward(cfg, W, toks, want)
    assert O.layer_runs(cfg) == [0, 1, 2, 1, 2, 1, 2, 3] and len(seen) == len(want) == 8
    for a, b in zip(seen, want):
        assert close(a, b, torch.float32, f32_tol=1e-4)


@pytest.mark.gpu
def test_padded_head_sizes_round_trip_on_the_gpu(tmp_path):
    """bf16 caches pad head sizes to what the matrix-core attention tiles; the projections that
    read padded heads carry zero columns, and the file's tensors come back unchanged."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    cfg = cfg_a()
    W = O.random_weights(cfg, seed=5)
    eng = make_engine(tmp_path, cfg, W, torch.device("cuda"), torch.bfloat16)
    assert eng.model.cache_dims[0] == (32, 32) and eng.model.p["l0.o"].shape == (40, 6 * 32)
    for lp in eng.model.logical_params():
        assert torch.equal(lp.get().reshape(W[lp.name].shape).float().cpu(), W[lp.name].float()), lp.name
    # a width and feed-forward sizes the tuned GEMMs take: gate / up rows in alternating 16-row blocks
    cfg = cfg_c()
    W = O.random_weights(cfg, seed=6)
    eng = make_engine(tmp_path, cfg, W, torch.device("cuda"), torch.bfloat16)
    assert eng.model.glu_group == {0: 16, 1: 16, 2: 16}
    assert torch.equal(eng.model.p["l1.gate_up"][16:32].float().cpu(), W["l1.mlp.up"][:16].float())
    for lp in eng.model.logical_params():
        assert torch.equal(lp.get().reshape(W[lp.name].shape).float().cpu(), W[lp.name].float()), lp.name


@pytest.mark.parametrize("name,mk", [("a", cfg_a), ("b", cfg_b), ("c", cfg_c)])
def test_prompt_decode_and_portions(target, tmp_path, name, mk):
    """One request: whole prompt; prompt then token-by-token decoding (long: chunks begin and end
    among decoded tokens); portions of many sizes down to two tokens, ending on single tokens; the
    first tokens one by one. Same logits as the oracle every way."""
    dev, dt = target
    cfg = mk()
    W = O.random_weights(cfg, seed=11)
    toks = tokens_of(cfg, 150, 3)
    want = oracle_logits(name, cfg, W, toks)
    eng = make_engine(tmp_path, cfg, W, dev, dt, cache_tokens=160)    # 5 pages: nothing to spare
    got = replay(eng, {"r": toks}, [[("r", 150)]])["r"]
    assert_rows(got, want, dt, "whole prompt")
    got = replay(eng, {"r": toks}, [[("r", 50)]] + [[("r", 1)]] * 100)["r"]          # pages / slot reused
    assert_rows(got, want, dt, "prompt + 100 decoded tokens")
    cuts = [2, 3, 5, 31, 23, 2, 32, 33, 7, 2] + [1] * 10
    assert sum(cuts) == 150
    got = replay(eng, {"r": toks}, [[("r", c)] for c in cuts])["r"]
    assert_rows(got, want, dt, "portions")
    got = replay(eng, {"r": toks[:4]}, [[("r", 1)]] * 4)["r"]                         # first tokens, one by one
    assert_rows(got, want[:4], dt, "first tokens")


@pytest.mark.parametrize("name,mk", [("a", cfg_a), ("b", cfg_b), ("c", cfg_c)])
def test_mixed_batches_reuse_pages_and_slots(target, tmp_path, name, mk):
    """Six requests of unequal length through three state slots and a cache that holds about
    half of them: portions beside decoded tokens of other requests, requests that pause,
    pages and slots handed from finished requests to new ones. Each equals the request alone."""
    dev, dt = target
    cfg = mk()
    W = O.random_weights(cfg, seed=12)
    lens = {"p": 70, "q": 33, "r": 1, "s": 96, "t": 64, "u": 40}
    reqs = {n: tokens_of(cfg, L, 20 + i) for i, (n, L) in enumerate(lens.items())}
    eng = make_engine(tmp_path, cfg, W, dev, dt, max_batch=3, cache_tokens=224)
    sched = [[("p", 40), ("q", 2)], [("p", 1), ("q", 30), ("r", 1)], [("q", 1), ("p", 20)],
             [("p", 1), ("s", 33)], [("s", 31), ("p", 1)], [("p", 1), ("s", 1)]] + \
            [[("p", 1), ("s", 1), ("t", 3)]] * 6 + [[("s", 24), ("t", 46)], [("u", 2)], [("u", 37), ("s", 1)],
                                                    [("u", 1)]]
    got = replay(eng, reqs, sched)
    for n in reqs:
        assert_rows(got[n], oracle_logits(name, cfg, W, reqs[n]), dt, f"request {n}")
    m = eng.kv.manager
    assert m.num_free == m.num_blocks and m.num_free_state_slots == 3


@pytest.mark.parametrize("graphs", [False, pytest.param(True, marks=gpu)])
def test_greedy_generation_through_the_scheduler(target, tmp_path, graphs):
    """LLMEngine.generate: the scheduler's own admission, chunked prompts (a small token budget),
    mixed steps, decode (hipGraph replays on the GPU) and the sampler; tokens equal the oracle's
    greedy continuation."""
    dev, dt = target
    if graphs and dev.type != "cuda":
        pytest.skip("graphs need a GPU")
    cfg = cfg_a()
    W = O.random_weights(cfg, seed=13)
    prompts = [tokens_of(cfg, n, 40 + n) for n in (37, 5, 64, 18, 2)]
    eng = make_engine(tmp_path, cfg, W, dev, dt, max_batch=3, cache_tokens=512, graphs=graphs, budget=24,
                      async_decode=graphs)
    outs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    for p, o in zip(prompts, outs):
        if dt == torch.float32:
            assert o == O.greedy(cfg, W, p, 12)
        else:       # bf16: every generated token is (nearly) the oracle's best continuation of its prefix
            lg = O.forward(cfg, W, p + o)
            for i, t in enumerate(o):
                row = lg[len(p) + i - 1]
                assert row[t] >= row.max() - 0.15 * (row.max() - row.mean())
    m = eng.kv.manager
    assert m.num_free == m.num_blocks and m.num_free_state_slots == 3


def test_random_init_and_registry():
    """The family is built from a configuration alone (random weights, as the benchmarks do)."""
    mc = ModelConfig.from_lizizen(cfg_b())
    assert mc.arch == "lizizen" and mc.layer_runs == [0, 1, 2, 3] and mc.layer_specs[2]["rot_dims"] == 0
    assert mc.layer_specs[0]["softcap"] == 0.0 and mc.layer_specs[1]["qt_coef"] == 0.0
    assert ModelConfig.from_lizizen(cfg_a()).layer_runs == [0, 1, 2, 1, 2, 1, 2, 3]
    m = build_model(mc, device="cpu", dtype=torch.float32)
    m.init_random(3)
    assert m.has_state and m.state_bytes_per_slot() == 4 * 48 * 4
    assert m.kv_bytes_per_token() == 4 * ((2 * 16 + 24) + 5 * (4 + 4) + 2 * (2 * 8 + 12) + (24 + 8))
    eng = LLMEngine(mc, engine_cfg=EngineConfig(max_batch=2, max_seq_len=64, kv_cache_tokens=128, use_graphs=False,
                                                dtype="fp32", async_decode=False), model=m, device=torch.device("cpu"))
    out = eng.generate([[1, 2, 3], [4]], SamplingParams(max_tokens=3, temperature=0.0, ignore_eos=True))
    assert [len(o) for o in out] == [3, 3]
    with pytest.raises(ValueError):
        ModelConfig.from_lizizen({**cfg_b(), "loop": {"start": 3, "stop": 2, "times": 2}})


def test_llm_entry_point_from_a_model_folder(tmp_path):
    """butterfly_amd.LLM on a folder: family chosen by config.json, a data-parallel-only plan from
    the partitioner, the default (overlapped) engine settings, greedy tokens equal the oracle's."""
    from butterfly_amd.api import LLM

    cfg = cfg_b()
    W = O.random_weights(cfg, seed=21)
    d = write_model(tmp_path, cfg, W)
    llm = LLM(d, engine_config=EngineConfig(max_batch=3, max_seq_len=96, kv_cache_tokens=256, dtype="fp32"))
    assert llm.cfg.arch == "lizizen" and (llm.plan.mesh.tp, llm.plan.mesh.pp) == (1, 1)
    prompts = [tokens_of(cfg, n, 60 + n) for n in (9, 33, 2)]
    outs = llm.generate(prompts, SamplingParams(max_tokens=5, temperature=0.0, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o.token_ids == O.greedy(cfg, W, p, 5)
    llm.close()
