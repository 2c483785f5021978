"""Gevipel (models/gevipel.py) against the plain float64 implementation in tests/gevipel_oracle.py:
every mechanism alone, then whole models through the engine: prefill vs token-by-token decoding,
prompt portions of many sizes, mixed batches of unequal requests, pages and state slots that are
freed and used again, window and page edges, far keys, the sink, the first tokens, long decoding,
looped layer spans with the embedding re-entering, greedy generation through the scheduler. Each
case runs on the CPU reference ops (f32) and, marked gpu, on the HIP kernels in f32 and bf16.
Configurations and weights are made here; nothing is read from disk but what a test wrote itself."""
import json
import math

import pytest
import torch
from safetensors.torch import save_file

from butterfly_amd import ops
from butterfly_amd.ckpt import load_into, model_config
from butterfly_amd.config import EngineConfig, ModelConfig
from butterfly_amd.engine.engine import LLMEngine
from butterfly_amd.engine.sampler import SamplingParams
from butterfly_amd.models import build_model

from . import gevipel_oracle as O

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


def assert_rows(got, want, dt, what="", clear=None):
    """`clear` (bf16 only): the number of leading rows whose expert choices hang on no close call."""
    e = rel_err(got, want).flatten()
    if dt == torch.float32:
        assert e.max() < 3e-4, f"{what}: worst row {int(e.argmax())} err {e.max():.3g}"
    else:
        # bf16 rounding in models this narrow is a few percent per row; the f32 runs carry the
        # exact comparison, this one checks that the bf16 kernels compute the same thing. Where
        # rounding may turn a router's choice, that row and (through caches and state) the rows after
        # it differ by more: those rows are held to the median and the upper quartile only
        assert e.median() < 0.05 and e.quantile(0.75) < 0.2, \
            f"{what}: median {e.median():.3g}, 75th percentile {e.quantile(0.75):.3g}"
        e = e if clear is None else e[:clear]
        if e.numel() >= 8:
            assert e.median() < 0.05 and e.quantile(0.9) < 0.15, \
                f"{what}: median {e.median():.3g}, 90th percentile {e.quantile(0.9):.3g} over {e.numel()} rows"


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


def packed_step(seqs, dev):
    """seqs: [(first position, rows)] -> row_cu, positions of a packed step."""
    cu, pos = [0], []
    for p0, n in seqs:
        cu.append(cu[-1] + n)
        pos += list(range(p0, p0 + n))
    return i32(cu, dev), i32(pos, dev)


# ---------------------------------------------------------------------------------------
# mechanisms alone
# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("W", [24, 200, 1030])
def test_sandwich_step(target, W):
    """x + m LN(y) (+ the re-entering embedding), fused with the next sublayer's norm; alone, and
    without a next norm; rows chosen for the output norm."""
    dev, dt = target
    T, eps, m = 9, 1e-5, 0.7
    x, y, e = rnd(T, W, seed=1, scale=3.0), rnd(T, W, seed=2), rnd(T, W, seed=3)
    w1, b1, w2, b2 = 1 + rnd(W, seed=4, scale=0.2), rnd(W, seed=5, scale=0.2), 1 + rnd(W, seed=6, scale=0.2), rnd(W, seed=7)
    f = lambda t: t.float().to(dev)                                   # noqa: E731
    for extra in (None, e):
        want_x = x + m * O.layer_norm(y, w1, b1, eps) + (0 if extra is None else extra)
        xg = f(x)
        h = ops.post_norm_add_norm(xg, y.to(dt).to(dev), f(w1), f(b1), eps, m, None if extra is None else f(extra),
                                   f(w2), f(b2), dt)
        assert close(xg, want_x, torch.float32) and close(h, O.layer_norm(want_x, w2, b2, eps), dt)
    xg = f(x)
    assert ops.post_norm_add_norm(xg, y.to(dt).to(dev), f(w1), f(b1), eps, 1.0, None, None, None, dt) is None
    assert close(xg, x + O.layer_norm(y, w1, b1, eps), torch.float32)
    idx = torch.tensor([0, 4, 8], device=dev)
    assert close(ops.layer_norm_rows(f(x), f(w2), f(b2), eps, idx, dt), O.layer_norm(x[[0, 4, 8]], w2, b2, eps), dt)


@pytest.mark.parametrize("taps,C", [(1, 24), (2, 40), (4, 300), (7, 65)])
def test_short_convolution_through_packed_steps(target, taps, C):
    """silu(conv) over three sequences cut into portions of 1, 2 and more rows, one of them in a slot
    another sequence used before, a sequence that pauses; the input rows are a view into wider rows."""
    dev, dt = target
    lens = [13, 6, 9]
    z = [rnd(n, C, seed=10 + s) for s, n in enumerate(lens)]
    w = rnd(C, taps, seed=3, scale=0.5)
    want = [O.silu(O.short_conv(z[s], w)) for s in range(3)]
    state = torch.full((2, taps - 1, C), 7.0, dtype=torch.float32, device=dev)      # stale: never read at position 0
    slot = [1, 0, 1]                          # sequence 2 takes the slot sequence 0 leaves
    steps = [[(0, 2), (1, 1)], [(0, 1), (1, 2)], [(0, 7)], [(0, 1), (1, 3)], [(0, 2)],
             [(2, 1)], [(2, 1)], [(2, 5)], [(2, 2)]]
    at = [0, 0, 0]
    got = [[] for _ in lens]
    for step in steps:
        cu, pos = packed_step([(at[s], c) for s, c in step], dev)
        rows = torch.cat([z[s][at[s]:at[s] + c] for s, c in step])
        wide = torch.zeros(rows.shape[0], C + 11, dtype=dt, device=dev)
        wide[:, 3:3 + C] = rows.to(dt)
        zin = wide[:, 3:3 + C]
        sl = i32([slot[s] for s, _ in step], dev)
        y = ops.short_conv_act(zin, w.float().to(dev), state, sl, cu, pos, "silu", torch.float32)
        if taps > 1:
            ops.short_conv_state_update_(zin, state, sl, cu, pos)
        r = 0
        for s, c in step:
            got[s].append(y[r:r + c])
            r += c
            at[s] += c
    assert at == lens
    for s in range(3):
        assert close(torch.cat(got[s]), want[s], dt), f"sequence {s}"
    # no activation, output in the model's type
    cu, pos = packed_step([(0, 5)], dev)
    y = ops.short_conv_act(z[0][:5].to(dt).to(dev), w.float().to(dev), state, i32([0], dev), cu, pos, "none", dt)
    assert y.dtype == dt and close(y, O.short_conv(z[0][:5], w), dt)


@pytest.mark.parametrize("taps,C", [(4, 256), (8, 72), (9, 64), (3, 130)])
def test_short_convolution_in_large_steps(target, taps, C):
    """Steps of hundreds of rows (a thread slides over rows with the history in registers): two prompts
    and a decoded row in one step, then their continuations from the history pool; bf16 output."""
    dev, dt = target
    lens = [260, 150, 40]
    z = [rnd(n, C, seed=20 + s) for s, n in enumerate(lens)]
    w = rnd(C, taps, seed=4, scale=0.5)
    want = [O.silu(O.short_conv(z[s], w)) for s in range(3)]
    state = torch.full((3, taps - 1, C), -3.0, dtype=torch.float32, device=dev)
    at, got = [0, 0, 0], [[] for _ in lens]
    for step in ([(2, 39)], [(2, 1), (0, 200), (1, 97)], [(0, 60), (1, 53)]):
        cu, pos = packed_step([(at[s], c) for s, c in step], dev)
        zin = torch.cat([z[s][at[s]:at[s] + c] for s, c in step]).to(dt).to(dev)
        sl = i32([s for s, _ in step], dev)
        y = ops.short_conv_act(zin, w.float().to(dev), state, sl, cu, pos, "silu", torch.float32)
        y2 = ops.short_conv_act(zin, w.float().to(dev), state, sl, cu, pos, "silu", dt)
        assert close(y2, y.double().cpu(), dt)
        ops.short_conv_state_update_(zin, state, sl, cu, pos)
        r = 0
        for s, c in step:
            got[s].append(y[r:r + c])
            r += c
            at[s] += c
    assert at == lens
    for s in range(3):
        assert close(torch.cat(got[s]), want[s], dt), f"sequence {s}"


def delta_inputs(T, H, G, D, Dv, seed):
    q, k, v = rnd(T, G, D, seed=seed), rnd(T, G, D, seed=seed + 1), rnd(T, H, Dv, seed=seed + 2)
    b, a = rnd(T, H, seed=seed + 3, scale=2.0), rnd(T, H, seed=seed + 4, scale=2.0)
    return q, k, v, b, a


def delta_want(q, k, v, b, a, a_log, dt_bias, D):
    H, G = v.shape[1], q.shape[1]
    qn = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    kn = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    qn, kn = qn.repeat_interleave(H // G, 1), kn.repeat_interleave(H // G, 1)
    decay = torch.exp(-torch.exp(a_log) * torch.nn.functional.softplus(a + dt_bias))
    return O.delta_rule(qn, kn, v, torch.sigmoid(b), decay)


@pytest.mark.parametrize("H,G,D,Dv", [(1, 1, 8, 8), (4, 2, 12, 20), (3, 3, 32, 64), (2, 1, 100, 130), (6, 2, 64, 32),
                                      (2, 2, 200, 16)])
def test_delta_rule_through_packed_steps(target, H, G, D, Dv):
    """The recurrence over three sequences cut into portions (1, 2, more than a staging block of 16),
    interleaved in steps, one in a slot another sequence used before; state handed from step to step."""
    dev, dt = target
    lens = [45, 6, 23]
    ins = [delta_inputs(n, H, G, D, Dv, 100 * s) for s, n in enumerate(lens)]
    a_log, dt_bias = rnd(H, seed=7, scale=0.7) - 1.0, rnd(H, seed=8)
    want = [delta_want(*ins[s], a_log, dt_bias, D) for s in range(3)]
    state = torch.full((2, H, Dv, D), 5.0, dtype=torch.float32, device=dev)       # stale: never read at position 0
    slot = [1, 0, 1]
    steps = [[(0, 2), (1, 1)], [(0, 1), (1, 2)], [(0, 35)], [(0, 1), (1, 3)], [(0, 6)],
             [(2, 1)], [(2, 1)], [(2, 19)], [(2, 2)]]
    at = [0, 0, 0]
    got = [[] for _ in lens]
    for step in steps:
        cu, pos = packed_step([(at[s], c) for s, c in step], dev)
        cat = lambda j, cast: torch.cat([ins[s][j][at[s]:at[s] + c] for s, c in step]).to(cast).to(dev)      # noqa: E731
        o = ops.delta_scan(cat(0, torch.float32), cat(1, torch.float32), cat(2, torch.float32), cat(3, dt), cat(4, dt),
                           a_log.float().to(dev), dt_bias.float().to(dev), state, i32([slot[s] for s, _ in step], dev),
                           cu, pos, D ** -0.5, 1e-6)
        r = 0
        for s, c in step:
            got[s].append(o[r:r + c])
            r += c
            at[s] += c
    assert at == lens
    for s in range(3):
        assert close(torch.cat(got[s]), want[s], torch.float32, f32_tol=1e-4), f"sequence {s}"


def test_delta_rule_recalls_a_far_write(target):
    """Four hundred tokens one by one with decays near one: the value written under one key at the start is
    read back by a query aimed at that key at the end; with a strong decay it is gone."""
    dev, dt = target
    T, H, D, Dv = 400, 2, 16, 24
    q, k, v, b, a = delta_inputs(T, H, H, D, Dv, 5)
    k[:, :, 0], q[:, :, 0] = 0.0, 0.0           # every later key is orthogonal to the first one
    k[0], q[-1] = 0.0, 0.0
    k[0, :, 0], q[-1, :, 0] = 4.0, 4.0
    b[0] = 20.0
    a[:] = -30.0                                # softplus ~ 0: nothing decays
    a_log, dt_bias = torch.zeros(H, dtype=F64), torch.zeros(H, dtype=F64)
    want = delta_want(q, k, v, b, a, a_log, dt_bias, D)
    assert (want[-1] - v[0] * D ** -0.5).abs().max() < 1e-3     # the oracle itself recalls it
    state = torch.zeros(1, H, Dv, D, dtype=torch.float32, device=dev)
    got = []
    for t in range(T):
        cu, pos = packed_step([(t, 1)], dev)
        f = lambda x, cast=torch.float32: x[t:t + 1].to(cast).to(dev)            # noqa: E731
        got.append(ops.delta_scan(f(q), f(k), f(v), f(b, dt), f(a, dt), a_log.float().to(dev), dt_bias.float().to(dev),
                                  state, i32([0], dev), cu, pos, D ** -0.5, 1e-6))
    assert close(torch.cat(got), want, torch.float32, f32_tol=1e-4)
    a[200] = 30.0                               # one step that wipes the state
    want2 = delta_want(q, k, v, b, a, a_log, dt_bias, D)
    assert want2[-1].abs().max() < 1e-3 < want[-1].abs().max()


def sloped_case(dev, dt, H, G, D, window, qt, T, aim, bs=32):
    """Queries and keys of T positions; `aim` lists (query position, key position): that query is
    aimed at that key (a scaled copy of it), so that whether the key is visible decides the output."""
    q, k = rnd(T, H, D, seed=1), rnd(T, G, D, seed=2)
    for i, j in aim:
        for h in range(H):
            q[i, h] = bf(4.0 * k[j, h // (H // G)])
    qn, kn = bf(1 + rnd(D, seed=3, scale=0.2)), bf(1 + rnd(D, seed=4, scale=0.2))
    eps, scale = 1e-5, 1.3 / math.sqrt(D)
    want = O.sloped_window_softmax(O.rms_norm(q, qn, eps), O.rms_norm(k, kn, eps), k, scale, window, qt)
    Dp = ops.attn_window_pad(D, dt)
    nblk = (T + bs - 1) // bs
    kc = torch.zeros(nblk + 1, G, bs, Dp, dtype=dt, device=dev)
    vc = torch.zeros(nblk + 1, G, Dp, bs, dtype=dt, device=dev)
    table = i32([[(b + 1) % (nblk + 1) for b in range(nblk)]], dev)              # pages in a shuffled order
    slopes = torch.pow(2.0, -8.0 * torch.arange(1, H + 1, dtype=F64) / H).float().to(dev)

    def run(p0, n):
        cu, pos = packed_step([(p0, n)], dev)
        slots = i32([int(table[0, p // bs]) * bs + p % bs for p in range(p0, p0 + n)], dev)
        g = lambda t: t[p0:p0 + n].to(dt).to(dev)                                # noqa: E731
        qp = ops.qk_norm_rope_kv(g(q), g(k), g(k), qn.float().to(dev), kn.float().to(dev), eps, pos,
                                 torch.zeros(0, device=dev), slots, kc, vc)
        o = ops.attn_window_paged(qp, kc, vc, table, cu, pos, scale, window if window else 1 << 30, 0, None,
                                  dist_bias=(slopes, None), q_temp=qt)
        return o[:, :, :D]
    return want, run


@pytest.mark.parametrize("H,G,D,window", [(4, 2, 16, 9), (2, 2, 64, 33), (6, 1, 24, 40), (3, 3, 32, 1), (8, 2, 64, 500),
                                          (2, 1, 128, None)])
def test_sloped_window_attention_edges(target, H, G, D, window):
    """Queries aimed at the key just inside and just outside the window, at keys on both sides of a
    page border and at themselves; as a whole prompt, in portions that cut the window, and decoded
    one by one. The values are the keys before their norm; the bias is linear in the distance."""
    dev, dt = target
    T = 150
    wd = window or 10 ** 6
    aim = []
    for i in (40, 64, 95, 96, 120, 149):
        aim += [(i, max(0, i - wd + 1))] if i % 2 == 0 else [(i, max(0, i - wd))]
    aim += [(70, 70), (100, 63), (101, 64)]
    want, run = sloped_case(dev, dt, H, G, D, window, (0.5, 7), T, aim)
    assert close(run(0, T), want, dt), "whole prompt"
    want, run = sloped_case(dev, dt, H, G, D, window, (0.5, 7), T, aim)
    got, at = [], 0
    for c in [2, 3, 31, 5, 23, 32, 2] + [1] * 52:
        got.append(run(at, c))
        at += c
    assert at == T and close(torch.cat(got), want, dt), "portions and decoded rows"


def test_sloped_attention_without_temperature_and_with_long_context(target):
    """No query temperature; a thousand cached tokens with a window of a few hundred (pages before the
    window are skipped; decoding splits the pages over workgroups)."""
    dev, dt = target
    T, window = 1100, 300
    aim = [(1099, 800), (1098, 798), (1050, 751), (1000, 1000)]
    want, run = sloped_case(dev, dt, 4, 2, 64, window, None, T, aim)
    got = [run(0, 1040)] + [run(t, 1) for t in range(1040, T)]
    assert close(torch.cat(got), want, dt)


@pytest.mark.parametrize("H,R,rd,T", [(3, 24, 8, 70), (6, 96, 32, 200), (4, 64, 0, 40), (2, 160, 64, 600)])
def test_shared_latent_attention_with_a_sink(target, H, R, rd, T):
    """All heads attend to one cached row [latent | rotated key part] and read the latent as the value
    (head folding); a learned sink per head joins the denominator. One query is aimed at the first key
    far back, one head's scores are all very low so that its sink takes nearly all the weight. Whole
    prompt (the 64-row tile when large), portions, decoded rows."""
    dev, dt = target
    bs, Dk = 32, R + rd
    ql, kl = rnd(T, H, Dk, seed=1, scale=0.5), rnd(T, Dk, seed=2, scale=0.5)
    ql[T - 1, 0] = bf(6.0 * kl[0])               # the last row's first head looks for the first key
    ql[:, H - 1] = bf(-3.0 * kl.mean(0))        # low scores everywhere: the sink wins
    sink = rnd(H, seed=3)
    sink[H - 1] = 9.0
    scale = 0.9 / math.sqrt(Dk)
    want = torch.zeros(T, H, R, dtype=F64)
    for h in range(H):
        want[:, h] = O.causal_sink_softmax((ql[:, h] @ kl.T) * scale, sink[h]) @ kl[:, :R]
    assert want[:, H - 1].abs().max() < 0.2 * want[:, 0].abs().max()
    Dkp, Dvp = ops.attn_window_pad(Dk, dt), ops.attn_window_pad(R, dt)
    nblk = (T + bs - 1) // bs
    table = i32([[nblk - 1 - b for b in range(nblk)]], dev)

    def run(cuts):
        kc = torch.zeros(nblk, 1, bs, Dkp, dtype=dt, device=dev)
        vc = torch.zeros(nblk, 1, Dvp, bs, dtype=dt, device=dev)
        out, at = [], 0
        for n in cuts:
            cu, pos = packed_step([(at, n)], dev)
            for p in range(at, at + n):          # the cached rows, as latent_prep leaves them
                b, o = int(table[0, p // bs]), p % bs
                kc[b, 0, o, :Dk] = kl[p].to(dt)
                vc[b, 0, :R, o] = kl[p, :R].to(dt)
            qp = torch.zeros(n, H, Dkp, dtype=dt, device=dev)
            qp[:, :, :Dk] = ql[at:at + n].to(dt)
            o = ops.attn_window_paged(qp, kc, vc, table, cu, pos, scale, 1 << 30, 0, sink.float().to(dev), fold_heads=True)
            out.append(o[:, :, :R])
            at += n
        assert at == T
        return torch.cat(out)
    assert close(run([T]), want, dt), "whole prompt"
    assert close(run([2, 15, T - 17 - 20] + [1] * 20), want, dt), "portions and decoded rows"


def test_latent_rows_without_a_query_latent(target):
    """latent_prep with no query latent and no gates: the RMS-normed latent and the rotated shared key
    part reach the pages (a page crossing, a row without a slot); the input is a view into wider rows."""
    dev, dt = target
    T, R, rd, bs, base = 6, 20, 8, 4, 100.0
    z = rnd(T, 13 + R + rd, seed=1)
    nw = bf(1 + rnd(R, seed=2, scale=0.2))
    pos = [2, 3, 4, 5, 9, 0]
    slots = [6, 7, 8, 9, -1, 0]
    inv = torch.tensor([base ** (-2.0 * i / rd) for i in range(rd // 2)], dtype=torch.float32)
    kc = torch.zeros(3, 1, bs, R + rd, dtype=dt, device=dev)
    vc = torch.zeros(3, 1, R, bs, dtype=dt, device=dev)
    cq, gate = ops.latent_prep(z.to(dt).to(dev)[:, 13:], 0, R, rd, 0, None, nw.float().to(dev), 1e-5, i32(pos, dev),
                               inv.to(dev), i32(slots, dev), kc, vc, dt)
    assert cq is None and gate is None
    c = O.rms_norm(z[:, 13:13 + R], nw, 1e-5)
    for t, sl in enumerate(slots):
        if sl < 0:
            continue
        kr = z[t:t + 1, 13 + R:].repeat(pos[t] + 1, 1)          # rotate_pairs turns row i by position i
        want = torch.cat([c[t], O.rotate_pairs(kr, base, rd)[pos[t]]])
        assert close(kc[sl // bs, 0, sl % bs], want, dt), t
        assert close(vc[sl // bs, 0, :, sl % bs], c[t], dt), t
    assert int((kc.float().abs().sum(-1) > 0).sum()) == 5


@pytest.mark.parametrize("E,top", [(4, 1), (16, 2), (70, 3), (5, 5)])
def test_router_choice_with_a_score_correction(target, E, top):
    """Softmax over all experts; the choice is made among score + correction, the weights are the plain
    scores of the chosen experts, not renormalised. The corrections here change most choices."""
    dev, dt = target
    T, W = 33, 48
    x, wr = rnd(T, W, seed=1), rnd(E, W, seed=2, scale=0.3)
    corr = rnd(E, seed=3, scale=0.3)
    s = torch.softmax(x @ wr.T, -1)
    pick = s + corr
    want_ids = pick.topk(top, -1).indices
    ids, w = ops.moe_route_scores(x.to(dt).to(dev), wr.to(dt).to(dev), top, scoring="softmax", renorm=False,
                                  select_bias=corr.float().to(dev))
    # rows whose choice does not hang on a close call
    srt = pick.sort(-1, descending=True).values
    clear = (srt[:, top - 1] - srt[:, top]).abs() > 1e-3 if top < E else torch.ones(T, dtype=torch.bool)
    assert clear.sum() > T // 2
    assert (want_ids != s.topk(top, -1).indices).any() or top == E          # the correction matters
    got = ids.cpu().long().sort(-1).values
    assert torch.equal(got[clear], want_ids.sort(-1).values[clear])
    ws = torch.gather(s, 1, ids.cpu().long())
    assert close(w[clear], ws[clear], torch.float32, f32_tol=1e-5)


@pytest.mark.parametrize("T,W,F,E,top", [(1, 24, 20, 4, 2), (37, 40, 56, 6, 3), (300, 128, 256, 8, 2), (5, 64, 128, 3, 1)])
def test_plain_squared_relu_experts(target, T, W, F, E, top):
    dev, dt = target
    x = rnd(T, W, seed=1)
    up, down = rnd(E, F, W, seed=2, scale=W ** -0.5), rnd(E, W, F, seed=3, scale=F ** -0.5)
    g = torch.Generator().manual_seed(4)
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)])
    wts = bf(torch.rand(T, top, generator=g, dtype=F64))
    want = torch.zeros(T, W, dtype=F64)
    for t in range(T):
        for j in range(top):
            e = int(ids[t, j])
            want[t] += wts[t, j] * (down[e] @ torch.relu(up[e] @ x[t]) ** 2)
    got = ops.moe_glu_ffn(x.to(dt).to(dev), ids.to(torch.int32).to(dev), wts.float().to(dev), up.to(dt).to(dev),
                          down.to(dt).to(dev), float("inf"), 1.0, up_offset=0.0, scale_input=False, plain_act="relu2")
    assert close(got, want, dt, bf16_tol=3e-2)


# ---------------------------------------------------------------------------------------
# whole models through the engine
# ---------------------------------------------------------------------------------------
def cfg_a():
    """Layers that differ from one another in every size; sizes no MFMA tile divides; a window
    shorter than a page; a layer without feed-forward; the middle span of layers runs three times
    (the embedding re-enters twice)."""
    return O.config([
        O.window_layer(6, 3, 12, 0.3, 9, 0.5, 5, O.moe(5, 2, 24)),
        O.delta_layer(4, 2, 10, 6, 3, O.moe(3, 1, 20)),
        O.latent_layer(3, 8, 4, 10, 14, 0.3, 100.0, None),
        O.delta_layer(2, 1, 20, 12, 5, O.moe(7, 3, 12)),
        O.window_layer(2, 2, 8, 0.25, 40, 0.25, 16, O.moe(4, 2, 16)),
    ], width=40, vocab=70, eps=1e-5, embed_scale=2.5, residual_mult=0.6, loop=(1, 3, 3))


def cfg_b():
    """What another model may make equal or 1 made unequal here, and the other way round: one head,
    as many key heads as query heads, a window of one position and one longer than the sequences, a
    single-tap convolution (no history), no temperature and one that steps at every position, no
    rotated part, every expert chosen and only one, factors of one, no repeated span."""
    layers = [
        O.delta_layer(1, 1, 16, 24, 1, O.moe(3, 3, 20)),
        O.window_layer(5, 5, 4, 0.5, 1, 0.0, 1, O.moe(2, 1, 16)),
        O.latent_layer(1, 12, 0, 6, 9, 0.25, 1e4, O.moe(6, 2, 8)),
        O.window_layer(1, 1, 24, 0.2, 4096, 1.0, 1, None),
        O.delta_layer(3, 3, 8, 8, 2, None),
        O.latent_layer(5, 4, 12, 4, 30, 0.4, 50.0, O.moe(4, 1, 32)),
    ]
    del layers[1]["mixer"]["q_temp"]
    del layers[3]["mixer"]["mask"]
    return O.config(layers, width=48, vocab=50, eps=1e-6, embed_scale=1.0, residual_mult=1.0)


def cfg_c():
    """Sizes the matrix-core kernels tile (bf16): window heads of 64, cached latent rows of 96 / 64,
    delta heads of 64 x 32, a width and expert sizes the tuned GEMMs take; the first two layers run
    twice (the embedding re-enters before a window layer)."""
    return O.config([
        O.window_layer(8, 2, 64, 0.125, 48, 0.5, 48, O.moe(8, 2, 128)),
        O.delta_layer(4, 1, 64, 32, 3, O.moe(4, 2, 64)),
        O.latent_layer(4, 32, 32, 64, 64, 0.125, 2e5, O.moe(8, 2, 128)),
    ], width=128, vocab=256, eps=1e-5, embed_scale=4.0, residual_mult=0.5, loop=(0, 2, 2))


_ORACLE = {}


def oracle_logits(name, cfg, W, tokens, with_clear=False):
    """Oracle logits, and on demand the number of leading rows all of whose routers choose with a
    margin that bf16 rounding does not bridge."""
    key = (name, tuple(tokens))
    if key not in _ORACLE:
        picks = []
        lg = O.forward(cfg, W, tokens, choice=picks)
        tops = [L["mlp"]["router"]["top"] for i, _ in O.layer_runs(cfg) for L in [cfg["layers"][i]] if L["mlp"]]
        close_call = torch.zeros(len(tokens), dtype=torch.bool)
        for pick, top in zip(picks, tops):
            if top < pick.shape[1]:
                srt = pick.sort(-1, descending=True).values
                close_call |= (srt[:, top - 1] - srt[:, top]) < 0.03
        first = int(close_call.nonzero()[0]) if close_call.any() else len(tokens)
        _ORACLE[key] = (lg, first)
    return _ORACLE[key] if with_clear else _ORACLE[key][0]


def write_model(tmp_path, cfg, W):
    d = tmp_path / "model"
    d.mkdir(exist_ok=True)
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in W.items()}, str(d / "model.safetensors"))
    return str(d)


def make_engine(tmp_path, cfg, W, dev, dt, max_batch=4, cache_tokens=512, graphs=False, **kw):
    d = write_model(tmp_path, cfg, W)
    mc = model_config(d)
    assert mc.arch == "gevipel"
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
    """Loading a folder and reading the tensors back gives the file's tensors (also the fused ones),
    and every layer run hands on what the oracle's layer does (before the embedding re-enters)."""
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
    probed = eng.replay_step([(0, toks, list(range(20)))], [0])
    O.forward(cfg, W, toks, want)
    assert [i for i, _ in O.layer_runs(cfg)] == [0, 1, 2, 1, 2, 1, 2, 3, 4] and len(seen) == len(want) == 9
    for a, b in zip(seen, want):
        assert close(a, b, torch.float32, f32_tol=1e-4)
    eng.model.layer_probe = None
    fused = eng.replay_step([(1, toks, list(range(20)))], [1])
    assert close(fused, probed.to(F64), torch.float32)


@pytest.mark.gpu
def test_padded_head_sizes_round_trip_on_the_gpu(tmp_path):
    """bf16 caches pad row sizes to what the matrix-core attention tiles; the projection that reads
    padded heads carries zero columns, and the file's tensors come back unchanged."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    cfg = cfg_a()
    W = O.random_weights(cfg, seed=5)
    eng = make_engine(tmp_path, cfg, W, torch.device("cuda"), torch.bfloat16)
    assert eng.model.cache_dims[0] == (32, 32) and eng.model.p["l0.o"].shape == (40, 6 * 32)
    assert eng.model.cache_dims[2] == (32, 32)
    for lp in eng.model.logical_params():
        assert torch.equal(lp.get().reshape(W[lp.name].shape).float().cpu(), W[lp.name].float()), lp.name


@pytest.mark.parametrize("name,mk", [("a", cfg_a), ("b", cfg_b), ("c", cfg_c)])
def test_prompt_decode_and_portions(target, tmp_path, name, mk):
    """One request: whole prompt; prompt then token-by-token decoding (long: the windows pass over
    decoded tokens); portions of many sizes down to two tokens, ending on single tokens; the first
    tokens one by one. Same logits as the oracle every way."""
    dev, dt = target
    cfg = mk()
    W = O.random_weights(cfg, seed=11)
    toks = tokens_of(cfg, 150, 3)
    want, clear = oracle_logits(name, cfg, W, toks, with_clear=True)
    eng = make_engine(tmp_path, cfg, W, dev, dt, cache_tokens=160)    # 5 pages: nothing to spare
    got = replay(eng, {"r": toks}, [[("r", 150)]])["r"]
    assert_rows(got, want, dt, "whole prompt", clear)
    got = replay(eng, {"r": toks}, [[("r", 50)]] + [[("r", 1)]] * 100)["r"]          # pages / slot reused
    assert_rows(got, want, dt, "prompt + 100 decoded tokens", clear)
    cuts = [2, 3, 5, 31, 23, 2, 32, 33, 7, 2] + [1] * 10
    assert sum(cuts) == 150
    got = replay(eng, {"r": toks}, [[("r", c)] for c in cuts])["r"]
    assert_rows(got, want, dt, "portions", clear)
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
        want, clear = oracle_logits(name, cfg, W, reqs[n], with_clear=True)
        assert_rows(got[n], want, dt, f"request {n}", clear)
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
    ref = None
    for p, o in zip(prompts, outs):
        if dt == torch.float32:
            assert o == O.greedy(cfg, W, p, 12)
        else:
            # bf16: a generated token is (nearly) the best continuation of its prefix by the engine's own
            # replayed logits, which the tests above hold against the oracle, and for most tokens by the
            # oracle's too (rounding that turns a router's choice moves a row's logits by more)
            ok = 0
            ref = ref or make_engine(tmp_path, cfg, W, dev, dt, max_batch=3, cache_tokens=512)      # (synchronous)
            own = ref.replay_step([(1000, p + o, list(range(len(p + o))))], [1000]).cpu().double()
            lg = O.forward(cfg, W, p + o)
            for i, t in enumerate(o):
                row = own[len(p) + i - 1]
                assert row[t] >= row.max() - 0.1 * (row.max() - row.mean())
                row = lg[len(p) + i - 1]
                ok += bool(row[t] >= row.max() - 0.15 * (row.max() - row.mean()))
            assert ok >= 0.75 * len(o)
    m = eng.kv.manager
    assert m.num_free == m.num_blocks and m.num_free_state_slots == 3


def test_random_init_and_registry():
    """The family is built from a configuration alone (random weights, as the benchmarks do)."""
    mc = ModelConfig.from_gevipel(cfg_b())
    assert mc.arch == "gevipel" and mc.layer_runs == [0, 1, 2, 3, 4, 5] and mc.loop_start == -1
    assert mc.layer_specs[1]["qt_coef"] == 0.0 and mc.layer_specs[3]["window"] == 1 << 30
    assert mc.layer_specs[2]["q_rank"] == 0 and mc.layer_specs[0]["taps"] == 1
    ma = ModelConfig.from_gevipel(cfg_a())
    assert ma.layer_runs == [0, 1, 2, 1, 2, 1, 2, 3, 4] and ma.loop_start == 1 and ma.residual_mult == 0.6
    m = build_model(mc, device="cpu", dtype=torch.float32)
    m.init_random(3)
    assert m.has_state and m.state_bytes_per_slot() == 4 * (16 * 24 + 3 * 8 * 8 + (2 * 3 * 8 + 3 * 8))
    assert m.kv_bytes_per_token() == 4 * (5 * (4 + 4) + (9 + 9) + (24 + 24) + (42 + 30))
    eng = LLMEngine(mc, engine_cfg=EngineConfig(max_batch=2, max_seq_len=64, kv_cache_tokens=128, use_graphs=False,
                                                dtype="fp32", async_decode=False), model=m, device=torch.device("cpu"))
    out = eng.generate([[1, 2, 3], [4]], SamplingParams(max_tokens=3, temperature=0.0, ignore_eos=True))
    assert [len(o) for o in out] == [3, 3]
    with pytest.raises(ValueError):
        ModelConfig.from_gevipel({**cfg_b(), "loop": {"start": 3, "stop": 2, "times": 2}})
    # a span that runs zero times is left out; one that runs once is the plain order
    assert ModelConfig.from_gevipel({**cfg_b(), "loop": {"start": 1, "stop": 3, "times": 0}}).layer_runs == [0, 3, 4, 5]
    once = ModelConfig.from_gevipel({**cfg_b(), "loop": {"start": 1, "stop": 3, "times": 1}})
    assert once.layer_runs == [0, 1, 2, 3, 4, 5] and build_model(once, device="cpu", dtype=torch.float32).reentry == set()
    bad = cfg_b()
    bad["layers"][1]["mixer"]["vdim"] = 8
    with pytest.raises(ValueError):
        ModelConfig.from_gevipel(bad)


def test_llm_entry_point_from_a_model_folder(tmp_path):
    """butterfly_amd.LLM on a folder: family chosen by config.json, a data-parallel-only plan from
    the partitioner, the default (overlapped) engine settings, greedy tokens equal the oracle's."""
    from butterfly_amd.api import LLM

    cfg = cfg_a()
    W = O.random_weights(cfg, seed=21)
    d = write_model(tmp_path, cfg, W)
    llm = LLM(d, engine_config=EngineConfig(max_batch=3, max_seq_len=96, kv_cache_tokens=256, dtype="fp32"))
    assert llm.cfg.arch == "gevipel" and (llm.plan.mesh.tp, llm.plan.mesh.pp) == (1, 1)
    prompts = [tokens_of(cfg, n, 60 + n) for n in (9, 33, 2)]
    outs = llm.generate(prompts, SamplingParams(max_tokens=5, temperature=0.0, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o.token_ids == O.greedy(cfg, W, p, 5)
    llm.close()
