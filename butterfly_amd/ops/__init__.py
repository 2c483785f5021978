"""butterfly_amd ops: hand-written HIP/CDNA4 kernels bound as torch.ops.bfly.*.

GPU tensors always run the HIP kernels from the in-tree `butterfly_amd/_C.so`; if that
library is missing or fails to load, every GPU call raises (no silent eager fallback).
CPU tensors run `ops.reference` (the CPU/gloo plumbing path and the numerics oracle).

Workspaces (split-K GEMM partials, split-KV decode partials, sampling partials) come from a
per-device arena that the engine sizes before hipGraph capture (`reserve_workspace`), so
captured steps never allocate.
"""
from __future__ import annotations

import os
import threading
from typing import Optional
from pathlib import Path

import torch

from . import reference as ref
from .reference import SILU_INTERLEAVE, glu_bias_block, interleave_gate_up, rope_tables, split_gate_up  # noqa: F401

_LIB_PATH = Path(__file__).resolve().parent.parent / "_C.so"
_loaded = False
_load_error: str | None = None

EPILOGUES = {"none": 0, "bias": 1, "silu": 2, "glu": 4}
DECODE_PART_TOKENS = 0   # 0 = pick the context split per call (attn_decode_part_tokens)


def load_library(path: str | os.PathLike | None = None) -> bool:
    """Load the HIP kernel library (idempotent). Returns True on success."""
    global _loaded, _load_error
    if _loaded:
        return True
    # BFLY_KERNEL_LIB: another build of the kernel library (same-box A/B runs of kernel changes)
    p = Path(path) if path else Path(os.environ.get("BFLY_KERNEL_LIB") or _LIB_PATH)
    if not p.exists():
        _load_error = f"{p} not built (run `python -m butterfly_amd._build`)"
        return False
    try:
        torch.ops.load_library(str(p))
        _loaded = True
        _load_error = None
    except Exception as e:  # pragma: no cover - depends on the environment
        _load_error = f"failed to load {p}: {e}"
    return _loaded


def require_library() -> None:
    """Raise unless the HIP kernel library is loaded (GPU-only features call this)."""
    if not load_library():
        raise RuntimeError(f"butterfly_amd HIP kernels unavailable: {_load_error}")


def native_available() -> bool:
    return load_library()


def library_path() -> str:
    return str(_LIB_PATH)


_FORCE_REF = False


class reference_mode:
    """Route every op to its fp32 PyTorch reference (ops/reference.py) even for GPU tensors:
    tests build an fp32 reference model on the same GPU as the kernel model (full-size layers
    whose CPU reference would take minutes). Not thread-scoped; tests only."""

    def __enter__(self):
        global _FORCE_REF
        self._prev, _FORCE_REF = _FORCE_REF, True
        return self

    def __exit__(self, *exc):
        global _FORCE_REF
        _FORCE_REF = self._prev
        return False


def _gpu(t: torch.Tensor) -> bool:
    if not t.is_cuda or _FORCE_REF:
        return False
    if not load_library():
        raise RuntimeError(f"butterfly_amd HIP kernels unavailable: {_load_error}")
    return True


# ---------------------------------------------------------------------------------------
# Workspace arena
# ---------------------------------------------------------------------------------------
class _Arena:
    """Named scratch buffers reused by every kernel call (split-K slabs, decode-attention
    partials, MoE slot maps and tile lists, sampling pairs). Buffers are shared by the threads
    of a process (an engine built on one thread and stepped on another reuses them) unless a
    thread sets its own scope (`arena_scope`): several ranks driven from threads of ONE process
    (the loopback backend, parallel/fake.py) must never share e.g. a MoE tile list, or one
    rank's moe_align would steer the other's grouped GEMM outside its own activations."""

    def __init__(self):
        self.bufs: dict[tuple, torch.Tensor] = {}
        self.frozen = False
        # buffers replaced by a larger one stay allocated: a hipGraph captured earlier still
        # reads / writes the old address (freeing it would hand that memory to someone else)
        self.retired: list = []

    def get(self, device, name: str, numel: int, dtype, zero: bool = False) -> torch.Tensor:
        key = (str(device), name, dtype, getattr(_scope, "name", None))
        buf = self.bufs.get(key)
        if buf is None or buf.numel() < numel:
            if self.frozen or (torch.cuda.is_available() and torch.cuda.is_current_stream_capturing()):
                raise RuntimeError(
                    f"workspace '{name}' needs {numel} elements but is frozen/capturing; "
                    "call ops.reserve_workspace() before capture")
            if buf is not None:
                self.retired.append(buf)
            buf = torch.empty(max(numel, 1), dtype=dtype, device=device)
            if zero:
                zero_(buf)
            self.bufs[key] = buf
        return buf


def zero_(t: torch.Tensor) -> torch.Tensor:
    """t.zero_() through the runtime's memset on the GPU (keeps torch kernels out of traces)."""
    if t.is_cuda and load_library():
        torch.ops.bfly.zero_(t)
    else:
        t.zero_()
    return t


# Output poisoning (`set_poison`): every op output is allocated filled with NaN
# (floating point) or a negative sentinel (integers) instead of left uninitialised, so an
# element a kernel forgot to write shows up in the comparison against the unpoisoned run.
_POISON = os.environ.get("BFLY_POISON_OUTPUTS", "0").strip().lower() in ("1", "true", "yes", "on")
# MoE prefill expert GEMMs on the 256x256 8-phase tile (BFLY_MOE_BIG_TILE=0: the 64/128-row tile)
_BIG_MOE = os.environ.get("BFLY_MOE_BIG_TILE", "1").strip().lower() not in ("0", "false", "no", "off")
# Host-side index checks of ops whose kernels cannot raise (BFLY_DEBUG_CHECKS; each costs a sync)
_DEBUG_CHECKS = os.environ.get("BFLY_DEBUG_CHECKS", "0").strip().lower() in ("1", "true", "yes", "on")


def set_poison(on: bool) -> None:
    """Allocate op outputs poisoned (debug / tests; costs one fill per output)."""
    global _POISON
    _POISON = bool(on)


def _poisoned(t: torch.Tensor) -> torch.Tensor:
    return t.fill_(float("nan") if t.is_floating_point() else -7777777)


def _empty(*shape, **kw) -> torch.Tensor:
    t = torch.empty(*shape, **kw)
    return _poisoned(t) if _POISON else t


def _empty_like(x: torch.Tensor, **kw) -> torch.Tensor:
    t = torch.empty_like(x, **kw)
    return _poisoned(t) if _POISON else t


_scope = threading.local()
_arena = _Arena()


def arena_scope(name) -> None:
    """Give this host thread its own workspace buffers (None: the process-wide set)."""
    _scope.name = name


def reserve_workspace(device, max_tokens: int, max_n: int, max_k: int, max_batch: int = 0,
                      max_ctx: int = 0, num_kv_heads: int = 0, head_dim: int = 128, shapes=()) -> None:
    """Pre-size every workspace for problems up to the given bounds (call before capture).
    `shapes`: the model's GEMM weight shapes (N, K); the split-K slab need is the max over them
    and every token-count bucket of the plan table (a tuned plan may split a small projection
    more than the largest one is split)."""
    if not load_library():
        return
    ws = 0
    nk = {(int(max_n), int(max_k))} | {(int(n), int(k)) for n, k in shapes}
    for m in sorted({1, 16, 32, 48, 64, 128, 256, 512, max_tokens}):
        if m > max_tokens:
            continue
        for n, k in nk:
            ws = max(ws, torch.ops.bfly.gemm_workspace_size(m, n, k))
    _arena.get(device, "gemm", ws // 4 + 1, torch.float32, zero=True)
    if max_batch and max_ctx:
        ns = max(torch.ops.bfly.attn_decode_splits(max_ctx, torch.ops.bfly.attn_decode_part_tokens(b, num_kv_heads, max_ctx))
                 for b in range(1, max_batch + 1))
        _arena.get(device, "attn_o", max_batch * num_kv_heads * ns * 16 * head_dim, torch.float32)
        _arena.get(device, "attn_ml", max_batch * num_kv_heads * ns * 16 * 2, torch.float32)
    _arena.get(device, "sample", max(max_batch, max_tokens, 1) * 64, torch.int64)
    _arena.get(device, "tkp", max(max_batch, max_tokens, 1) * 521, torch.float32)


# ---------------------------------------------------------------------------------------
# Ops
# ---------------------------------------------------------------------------------------
class Partial:
    """Output of a split-K GEMM whose reduce was deferred to its consumer (`linear(...,
    defer=True)`): `slabs` [sk, M, N] f32 live in the shared GEMM workspace and must be consumed
    (rms_norm / rope_kv fuse the reduce) or `materialize()`d before the next GEMM runs.
    `out` is the bf16 [M, N] buffer the result belongs in."""

    __slots__ = ("slabs", "out")

    def __init__(self, slabs: torch.Tensor, out: torch.Tensor):
        self.slabs, self.out = slabs, out

    @property
    def shape(self):
        return self.out.shape

    def materialize(self) -> torch.Tensor:
        torch.ops.bfly.splitk_reduce(self.slabs, self.out)
        return self.out


def materialize(x):
    return x.materialize() if isinstance(x, Partial) else x


class RowNormed:
    """RMSNorm output whose 1/rms row scale is left to the consuming GEMM (`rms_norm(...,
    rows=True)`, norm.hip rmsnorm_rows_kernel): `y` [M, dim] bf16 = x * w, `ssp` [M, chunks] f32
    partial sums of squares of x. `linear(RowNormed, ...)` scales row m of its result by
    rsqrt(sum(ssp[m]) / dim + eps) in the GEMM epilogue (before bias / SiLU / split-K slabs)."""

    __slots__ = ("y", "ssp", "eps")

    def __init__(self, y: torch.Tensor, ssp: torch.Tensor, eps: float):
        self.y, self.ssp, self.eps = y, ssp, eps

    @property
    def shape(self):
        return self.y.shape


_rowscale_ok: dict = {}


def rowscale_ok(M: int, N: int, K: int, epilogue: str = "none") -> bool:
    """True if the GEMM plan for this shape applies a RowScale (tile / decode-ring kernels)."""
    key = (M, N, K, epilogue)
    ok = _rowscale_ok.get(key)
    if ok is None:
        ok = load_library() and torch.ops.bfly.gemm_rowscale_check(M, N, K, EPILOGUES[epilogue]) == 0
        _rowscale_ok[key] = ok
    return ok


def rms_norm(x, w, eps: float, out=None, residual=None, rows: bool = False):
    """y = x * rsqrt(mean(x^2) + eps) * w; with `residual`: residual += x first (in place)
    and y is the norm of the updated residual (the fused add+norm of every block). `x` may be
    a deferred split-K GEMM output (`Partial`): its reduce is fused into this kernel.
    `rows=True` (GPU): return a `RowNormed` for a row-scaling consumer GEMM instead."""
    if rows and (isinstance(x, Partial) or _gpu(x)):
        src = x.slabs if isinstance(x, Partial) else x
        M, dim = src.shape[-2], src.shape[-1]
        if out is None:
            out = _empty(M, dim, dtype=w.dtype, device=w.device)
        ssp = _empty(M, torch.ops.bfly.rms_norm_rows_chunks(dim), dtype=torch.float32, device=w.device)
        torch.ops.bfly.rms_norm_rows(src, w, out, ssp, residual)
        return RowNormed(out, ssp, eps)
    if isinstance(x, Partial):
        if out is None:
            out = _empty_like(x.out)
        torch.ops.bfly.rms_norm_partial(x.slabs, w, eps, out, residual)
        return out
    if not _gpu(x):
        return ref.rms_norm(x, w, eps, out, residual)
    if out is None:
        out = _empty_like(x)
    torch.ops.bfly.rms_norm(x, w, eps, out, residual)
    return out


def rms_norm_route(x, w, eps: float, residual, router_w, top_k: int):
    """The fused add + RMSNorm of a MoE layer's FFN input that also routes the rows it
    normalises (norm.hip rmsnorm_partial_kernel<NV, E>): returns (y, (gates, topk_ids, topk_w))
    as `rms_norm` then `moe_route(y, router_w, top_k)` would, in one launch. Needs a deferred
    split-K input (`Partial`), a residual and 4 or 8 experts; otherwise returns (rms_norm(...),
    None) and the caller routes separately."""
    if (isinstance(x, Partial) and residual is not None
            and torch.ops.bfly.rms_norm_route_ok(router_w.shape[0], router_w.shape[1]) == 1):
        T = x.out.shape[0]
        E = router_w.shape[0]
        out = _empty_like(x.out)
        gates = _empty(T, E, dtype=torch.float32, device=out.device)
        ids = _empty(T, top_k, dtype=torch.int32, device=out.device)
        tw = _empty(T, top_k, dtype=torch.float32, device=out.device)
        torch.ops.bfly.rms_norm_partial_route(x.slabs, w, eps, out, residual, router_w, top_k, gates, ids, tw)
        return out, (gates, ids, tw)
    return rms_norm(x, w, eps, residual=residual), None


def layer_norm(x, w, b, eps: float, out=None, residual=None):
    if not _gpu(x):
        return ref.layer_norm(x, w, b, eps, out, residual)
    if out is None:
        out = _empty_like(x)
    torch.ops.bfly.layer_norm(x, w, b, eps, out, residual)
    return out


def rope_kv(qkv, positions, cos, sin, n_q: int, n_kv: int, slots=None, k_cache=None,
            v_cache=None):
    """In-place RoPE on the Q/K heads of a fused QKV row; optional paged KV append. Returns the
    (bf16) QKV rows; `qkv` may be a deferred split-K GEMM output whose reduce is fused here."""
    if isinstance(qkv, Partial):
        torch.ops.bfly.rope_kv(qkv.out, positions, cos, sin, n_q, n_kv, slots, k_cache, v_cache, qkv.slabs)
        return qkv.out
    if not _gpu(qkv):
        return ref.rope_kv(qkv, positions, cos, sin, n_q, n_kv, slots, k_cache, v_cache)
    torch.ops.bfly.rope_kv(qkv, positions, cos, sin, n_q, n_kv, slots, k_cache, v_cache)
    return qkv


def kv_append(k, v, slots, k_cache, v_cache):
    if not _gpu(k):
        return ref.kv_append(k, v, slots, k_cache, v_cache)
    torch.ops.bfly.kv_append(k, v, slots, k_cache, v_cache)


def silu_mul(gu, out=None, interleave: int = 0):
    if not _gpu(gu):
        return ref.silu_mul(gu, out, interleave)
    if out is None:
        out = _empty(*gu.shape[:-1], gu.shape[-1] // 2, dtype=gu.dtype, device=gu.device)
    torch.ops.bfly.silu_mul(gu, out, interleave)
    return out


def gelu(x, out=None):
    if not _gpu(x):
        return ref.gelu(x, out)
    if out is None:
        out = _empty_like(x)
    torch.ops.bfly.gelu(x, out)
    return out


def add(a, b, out=None):
    b = materialize(b)
    if not _gpu(a):
        return ref.add(a, b, out)
    if out is None:
        out = _empty_like(a)
    torch.ops.bfly.add(a, b, out)
    return out


def embed(ids, table, vstart: int = 0, out=None):
    if not _gpu(ids):
        return ref.embed(ids, table, vstart, out)
    if out is None:
        out = _empty(ids.numel(), table.shape[1], dtype=table.dtype, device=table.device)
    torch.ops.bfly.embed(ids, table, out, vstart)
    return out


def gather_rows(src, idx, out=None):
    """out[i] = src[idx[i]] (rows of a 2-D tensor; `idx` int32 / int64). Rows whose idx is < 0
    keep what `out` holds (pass a pre-filled `out`). Our row-gather kernel on the GPU, not
    torch's index_select (elementwise.hip gather_rows_kernel)."""
    if out is None:
        out = _empty(idx.numel(), *src.shape[1:], dtype=src.dtype, device=src.device)
    if not _gpu(src):
        return ref.gather_rows(src, idx, out)
    s2 = src if src.dim() == 2 else src.view(src.shape[0], -1)
    o2 = out if out.dim() == 2 else out.view(out.shape[0], -1)
    if _DEBUG_CHECKS and not torch.cuda.is_current_stream_capturing() and idx.numel():
        hi = int(idx.max())
        if hi >= src.shape[0]:
            raise IndexError(f"gather_rows: index {hi} out of range for {src.shape[0]} source rows")
    torch.ops.bfly.gather_rows(s2, idx, o2)
    return out


def sample_pack(scores, ids):
    """Per-shard sampling winners -> [rows, 2] f32 (score, id) pairs for the TP all-gather."""
    if not _gpu(scores):
        return ref.sample_pack(scores, ids)
    pair = _empty(scores.numel(), 2, dtype=torch.float32, device=scores.device)
    torch.ops.bfly.sample_pack(scores.contiguous(), ids.contiguous(), pair)
    return pair


def sample_merge(allp):
    """All-gathered pairs [tp, rows, 2] -> int32 ids of the best score per row (lowest rank on
    ties: torch.argmax's first maximum)."""
    if not _gpu(allp):
        return ref.sample_merge(allp)
    out = _empty(allp.shape[1], dtype=torch.int32, device=allp.device)
    torch.ops.bfly.sample_merge(allp.contiguous(), out)
    return out


def sample(logits, temps=None, seeds=None, vstart: int = 0, out_ids=None, out_scores=None, thresh=None,
           check_finite: bool = False):
    """Greedy / Gumbel-max sampling over a (vocab-shard of) logits -> (ids int32, scores f32).
    `thresh` [rows] f32: per-row lower bound on logit / temperature (top-k / top-p filter).
    `check_finite`: rows with an Inf / NaN logit get id -1 and score +inf (the NaN guard)."""
    if not _gpu(logits):
        return ref.sample(logits, temps, seeds, vstart, thresh, check_finite)
    rows = logits.shape[0]
    if out_ids is None:
        out_ids = _empty(rows, dtype=torch.int32, device=logits.device)
    if out_scores is None:
        out_scores = _empty(rows, dtype=torch.float32, device=logits.device)
    if logits.dtype == torch.float32:
        # f32 serving mode: greedy rows pick from the f32 values themselves; stochastic rows go
        # through the bf16 sampler on a rounded copy (16-byte rows)
        if temps is None and thresh is None:
            torch.ops.bfly.sample_greedy_f32(logits, vstart, out_ids, out_scores, check_finite)
            return out_ids, out_scores
        n = logits.shape[1]
        buf = torch.empty(rows, (n + 7) // 8 * 8, dtype=torch.bfloat16, device=logits.device)
        buf[:, :n].copy_(logits)
        logits = buf[:, :n]
    ws = _arena.get(logits.device, "sample", rows * 64, torch.int64)
    torch.ops.bfly.sample(logits, temps, seeds, vstart, out_ids, out_scores, ws, thresh, check_finite)
    return out_ids, out_scores


def topkp_threshold(logits, temps, top_k, top_p, reduce_sum=None, reduce_max=None,
                    use_k: bool = True, use_p: bool = True):
    """Exact per-row top-k / top-p threshold on logit / temperature by radix select (4 passes
    of 8 bits per filter, sample.hip tkp_*). `reduce_sum(t)` / `reduce_max(t)`: in-place
    all-reduces over the TP group applied to every histogram / the row maxima, so vocab shards
    select together (None: unsharded). `use_k` / `use_p`: skip a filter no row uses. Returns
    thresh [R] f32 (-inf = unfiltered row), the `thresh` argument of `sample`."""
    if not _gpu(logits):
        return ref.topkp_threshold(logits, temps, top_k, top_p, reduce_sum, reduce_max, use_k, use_p)
    R = logits.shape[0]
    L = torch.ops.bfly
    ws = _arena.get(logits.device, "tkp", R * 521, torch.float32)[: R * 521]
    zero_(ws)
    # the row-max slot starts at the smallest ordered key (INT_MIN = below signed_ordered(-inf)):
    # a zero would read as +0.0 and clamp the max of an all-negative row
    L.fill32_(ws[R * 8:R * 9], -2 ** 31)
    L.tkp_begin(logits, temps, top_k, top_p, ws)
    if reduce_max is not None:
        reduce_max(ws[R * 8:R * 9].view(torch.int32))
    hist = ws[R * 9:].view(R, 512)
    for phase, on in ((0, use_k), (1, use_p)):
        if not on:
            continue
        for p in range(4):
            L.tkp_pass(logits, temps, ws, p, phase)
            if reduce_sum is not None:
                reduce_sum(hist)
            L.tkp_select(top_p, ws, R, p, phase)
    thr = _empty(R, dtype=torch.float32, device=logits.device)
    L.tkp_final(ws, R, thr)
    return thr


def pack_w256(w: torch.Tensor) -> torch.Tensor:
    """A [N, K] weight in the K-tile-blocked layout [N/256][K/64][256][64] (returned viewed as
    [N, K]) that the packed decode GEMM reads (gemm.hip launch_gemm_packed)."""
    N, K = w.shape
    return w.view(N // 256, 256, K // 64, 64).permute(0, 2, 1, 3).contiguous().view(N, K)


def linear(x, w, bias=None, epilogue: str = "none", out=None, defer: bool = False, packed=None):
    """y = x @ w.T (+ bias) with optional fused SwiGLU epilogue ('silu': w rows gate/up
    interleaved in 16-row groups, output width w.shape[0] // 2) or fused clamped GLU with biases
    ('glu': the same row layout, `bias` = glu_bias_block(interleaved biases, limit, alpha,
    up_offset): g sigmoid(alpha g) (u + up_offset), g = min(gate, limit), u = clamp(up,
    +-limit)). `defer=True` (no bias /
    epilogue): when the plan splits K, return a `Partial` whose reduce the consumer fuses.
    `packed`: the weight's pack_w256 copy: used when the shape's plan has a packed form (decode
    tile plans), else `w`."""
    rn = None
    if isinstance(x, RowNormed):   # consumer of a row-split RMSNorm: the GEMM applies 1/rms
        rn, x = x, x.y
    if not _gpu(x):
        return ref.linear(x, w, bias, epilogue, out)
    if packed is not None and bias is None and epilogue in ("none", "silu") and not (defer and epilogue != "none"):
        M, N = x.shape[0], w.shape[0]
        if out is None:
            out = _empty(M, N // 2 if epilogue == "silu" else N, dtype=x.dtype, device=x.device)
        need = torch.ops.bfly.gemm_workspace_size(M, N, x.shape[1])
        ws = _arena.get(x.device, "gemm", need // 4 + 1, torch.float32, zero=True) if need else None
        sk = torch.ops.bfly.gemm_packed(x, packed, out, EPILOGUES[epilogue], rn.ssp if rn is not None else None,
                                        rn.eps if rn is not None else 0.0, None, 0, 1, ws, bool(defer))
        if sk == 1:
            return out
        if sk > 1:     # deferred split-K slabs for the consumer
            off = torch.ops.bfly.gemm_slab_offset()
            return Partial(ws[off:off + sk * M * N].view(sk, M, N), out)
    if defer and bias is None and epilogue == "none":
        M, N = x.shape[0], w.shape[0]
        if out is None:
            out = _empty(M, N, dtype=x.dtype, device=x.device)
        need = torch.ops.bfly.gemm_workspace_size(M, N, x.shape[1])
        ws = _arena.get(x.device, "gemm", need // 4 + 1, torch.float32, zero=True)
        if rn is not None:
            sk = torch.ops.bfly.gemm_deferred_rs(x, w, out, ws, rn.ssp, rn.eps)
        else:
            sk = torch.ops.bfly.gemm_deferred(x, w, out, ws)
        if sk == 1:
            return out
        off = torch.ops.bfly.gemm_slab_offset()
        return Partial(ws[off:off + sk * M * N].view(sk, M, N), out)
    epi = EPILOGUES["bias"] if (bias is not None and epilogue == "none") else EPILOGUES[epilogue]
    if epilogue == "silu" and bias is not None:
        raise ValueError("bias + silu epilogue not supported")
    M, N = x.shape[0], w.shape[0]
    nout = N // 2 if epilogue in ("silu", "glu") else N
    if out is None:
        out = _empty(M, nout, dtype=x.dtype, device=x.device)
    need = torch.ops.bfly.gemm_workspace_size(M, N, x.shape[1])
    # zero-initialised once: its head holds the split-K arrival counters, which every GEMM
    # leaves re-armed at zero
    ws = _arena.get(x.device, "gemm", need // 4 + 1, torch.float32, zero=True) if need else None
    if rn is not None:
        torch.ops.bfly.gemm_rs(x, w, out, bias, epi, ws, rn.ssp, rn.eps)
    else:
        torch.ops.bfly.gemm(x, w, out, bias, epi, ws)
    return out


def linear_silu_gate(x, w, gates, e0: int, num_local: int, packed=None):
    """The dense MoE decode gate/up GEMM over the concatenated local experts: SwiGLU, then every
    expert's column block scaled by its routing weight gates[:, e0 + e] — `linear(x, w, 'silu')`
    followed by `moe_gate_scale_`, bit for bit, in one launch (the tile kernel's epilogue).
    `packed`: the weight's pack_w256 copy (used when the plan has a packed form)."""
    if isinstance(x, RowNormed) or not _gpu(x):
        h = linear(x, w, epilogue="silu")
        return moe_gate_scale_(h, gates, e0, num_local)
    out = _empty(x.shape[0], w.shape[0] // 2, dtype=x.dtype, device=x.device)
    if packed is not None and torch.ops.bfly.gemm_packed(x, packed, out, 3, None, 0.0, gates, e0, num_local) > 0:
        return out
    torch.ops.bfly.gemm_silu_gate(x, w, out, gates, e0, num_local)
    return out


def gemm_plan(M: int, N: int, K: int) -> dict:
    load_library()
    k, mt, nt, bm, bn, sk, wk = torch.ops.bfly.gemm_plan(M, N, K)
    return {"kind": ("skinny", "tile", "big", "dec", "big8", "mid8", "big4", "mid4")[k], "mt": mt, "nt": nt, "wk": wk, "bm": bm, "bn": bn,
            "splitk": sk}


def attn_prefill(q, k, v, cu_seqlens, max_seqlen: int, scale: float, causal: bool = True,
                 out=None, cu_seqlens_k=None, return_lse: bool = False):
    """Varlen flash attention (K3). `cu_seqlens_k`: keys of each sequence come from other
    rows than its queries (non-causal; context-parallel ring steps). `return_lse`: also return
    the per-(row, head) natural-log sum-exp of the scaled scores [T, Hq] f32 (-inf: no keys),
    which `attn_lse_merge_` uses to combine attention over key chunks."""
    if not _gpu(q):
        return ref.attn_prefill(q, k, v, cu_seqlens, max_seqlen, scale, causal, out, cu_seqlens_k, return_lse)
    if out is None:
        out = _empty(q.shape, dtype=q.dtype, device=q.device)
    lse = _empty(q.shape[0], q.shape[1], dtype=torch.float32, device=q.device) if return_lse else None
    torch.ops.bfly.attn_prefill(q, k, v, cu_seqlens, max_seqlen, scale, causal, out, cu_seqlens_k, lse)
    return (out, lse) if return_lse else out


def attn_prefill_paged(q, k_cache, v_cache, tables, cu_q, positions, max_q: int, scale: float, out=None):
    """Chunked prefill attention over the paged cache (attention_paged.hip): query rows
    [cu_q[s], cu_q[s+1]) of sequence s at `positions` attend causally to the sequence's cached
    keys through tables[s] — the cached prefix and the chunk itself (already appended by
    rope_kv) in one pass, no gather, no log-sum-exp merge. Caches bf16 or FP8."""
    if not _gpu(q):
        return ref.attn_prefill_paged(q, k_cache, v_cache, tables, cu_q, positions, max_q, scale, out)
    if out is None:
        out = _empty(q.shape, dtype=q.dtype, device=q.device)
    torch.ops.bfly.attn_prefill_paged(q, k_cache, v_cache, tables, cu_q, positions, int(max_q), float(scale), out)
    return out


def attn_lse_merge_(acc_o, acc_lse, o, lse):
    """K16: fold a partial attention result (o bf16 [T, H, D], lse [T, H]) into running f32
    accumulators (acc_o [T, H, D], acc_lse [T, H]) in place."""
    if not _gpu(acc_o):
        return ref.attn_lse_merge_(acc_o, acc_lse, o, lse)
    torch.ops.bfly.attn_lse_merge(acc_o, acc_lse, o, lse)
    return acc_o, acc_lse


def attn_decode(q, k_cache, v_cache, block_tables, ctx_lens, scale: float, max_ctx: int,
                part_tokens: int = DECODE_PART_TOKENS, out=None):
    """One query token per sequence against the paged cache. `max_ctx` bounds ctx_lens (it
    fixes the split-KV grid, so it is a static parameter under graph capture)."""
    if not _gpu(q):
        return ref.attn_decode(q, k_cache, v_cache, block_tables, ctx_lens, scale, max_ctx,
                               part_tokens, out)
    B, Hq, D = q.shape
    Hkv = k_cache.shape[1]
    if out is None:
        out = _empty(B, Hq, D, dtype=q.dtype, device=q.device)
    if part_tokens <= 0:
        part_tokens = torch.ops.bfly.attn_decode_part_tokens(B, Hkv, max_ctx)
    ns = torch.ops.bfly.attn_decode_splits(max_ctx, part_tokens)
    po = pml = None
    if ns > 1:
        po = _arena.get(q.device, "attn_o", B * Hkv * ns * 16 * D, torch.float32)
        pml = _arena.get(q.device, "attn_ml", B * Hkv * ns * 16 * 2, torch.float32)
    torch.ops.bfly.attn_decode(q, k_cache, v_cache, block_tables, ctx_lens, scale, max_ctx,
                               part_tokens, out, po, pml)
    return out


def init_hash_(out, grow0: int, gcol0: int, gcols: int, seed: int, amp: float):
    """Fill a 2-D (view of a) weight shard with partition-independent hashed uniform values."""
    if not _gpu(out):
        return ref.init_hash(out, grow0, gcol0, gcols, seed, amp)
    torch.ops.bfly.init_hash(out, grow0, gcol0, gcols, seed & 0xFFFFFFFF, amp)
    return out


def moe_route(x, wr, top_k: int, gates=None, topk_ids=None, topk_w=None):
    if not _gpu(x):
        return ref.moe_route(x, wr, top_k)
    T, E = x.shape[0], wr.shape[0]
    if gates is None:
        gates = _empty(T, E, dtype=torch.float32, device=x.device)
    if topk_ids is None:
        topk_ids = _empty(T, top_k, dtype=torch.int32, device=x.device)
    if topk_w is None:
        topk_w = _empty(T, top_k, dtype=torch.float32, device=x.device)
    torch.ops.bfly.moe_route(x, wr, top_k, gates, topk_ids, topk_w)
    return gates, topk_ids, topk_w


def moe_sparse_ffn(x, topk_ids, topk_w, gu_w, down_w, e0: int, num_local: int, ffn: int,
                   expected_slots: Optional[int] = None, block_counts: Optional[tuple] = None):
    """Routed expert FFN: permute the (token, k) pairs of the local experts into per-expert
    row slots (moe_align), grouped gate/up GEMM with fused SiLU over gathered token rows,
    grouped down GEMM, weighted combine back to token order. Only routed rows are computed
    (the dense path computes every local expert for every token).
    `block_counts` = (counts [nblk] int32 on the device, cap): the rows are nblk blocks of `cap`
    rows of which only the first counts[b] are valid (the EP IPC prefill receive buffer, sized
    for the worst case): the other rows get no expert work and no output row."""
    if not _gpu(x):
        if block_counts is not None:
            cnt, cap = block_counts
            r = torch.arange(x.shape[0]) % cap
            ok = r < cnt.cpu().long()[torch.arange(x.shape[0]) // cap]
            topk_ids = topk_ids.masked_fill(~ok.unsqueeze(1), -1)
        return ref.moe_sparse_ffn(x, topk_ids, topk_w, gu_w, down_w, e0, num_local, ffn)
    T, H = x.shape
    k = topk_ids.shape[1]
    TK = T * k
    if TK == 0:
        return zero_(torch.empty(T, H, dtype=x.dtype, device=x.device))
    L = torch.ops.bfly
    dev = x.device
    bcnt, bcap = block_counts if block_counts is not None else (None, 0)
    # tile rows from the expected rows per expert (all slots are local in the EP dispatch):
    # one 128-row tile reads each expert's weights once where two 64-row tiles would twice
    # `expected_slots`: (token, k) pairs expected to be local (the EP dispatch pads with
    # non-local / empty slots; they cost nothing but must not size the launch)
    exp = TK if expected_slots is None else max(1, min(TK, expected_slots))
    # prefill-scale expert batches (>= 256 rows per local expert on average): the 8-phase
    # 256x256 tile over the tile list (gemm.hip gemm_big8_kernel<GROUPED>)
    bm = 256 if (exp >= 256 * num_local and H % 256 == 0 and (2 * ffn) % 256 == 0 and _BIG_MOE) else \
        (128 if exp >= 96 * num_local else 64)
    rows = _arena.get(dev, "moe_rows", TK, torch.int32)[:TK]
    slot_of = _arena.get(dev, "moe_slot", TK, torch.int32)[:TK]
    nt = L.moe_max_tiles(TK, num_local, bm)
    tiles = _arena.get(dev, "moe_tiles", nt * 4, torch.int32)[:nt * 4].view(nt, 4)
    count = _arena.get(dev, "moe_count", 1, torch.int32)[:1]
    L.moe_align(topk_ids, e0, num_local, rows, slot_of, tiles, count, bm, bcnt, bcap)
    hmid = _empty(TK, ffn, dtype=x.dtype, device=dev)
    L.moe_grouped_gemm(x, gu_w, hmid, rows, tiles, count, 2 * ffn * H, 2 * ffn, H, num_local, EPILOGUES["silu"], bm)
    out = _empty(T, H, dtype=x.dtype, device=dev)
    sk = moe_down_splits(exp, num_local, H, ffn, bm)
    if sk > 1:
        # decode-sized expert batches: split K of the down projection over sk workgroups so the
        # chip fills; the slab reduce is folded into the weighted combine
        part = _arena.get(dev, "moe_part", sk * TK * H, torch.float32)[: sk * TK * H].view(sk, TK, H)
        L.moe_grouped_gemm(hmid, down_w, hmid.new_empty(TK, H), None, tiles, count, ffn, H, ffn, num_local,
                           EPILOGUES["none"], bm, part)
        L.moe_combine_slabs(part, slot_of, topk_w, out, bcnt, bcap)
        return out
    y = _empty(TK, H, dtype=x.dtype, device=dev)
    L.moe_grouped_gemm(hmid, down_w, y, None, tiles, count, ffn, H, ffn, num_local, EPILOGUES["none"], bm)
    L.moe_combine(y, slot_of, topk_w, out, bcnt, bcap)
    return out


def ep_pack(x, ids, w, slots, experts_per_rank: int, ep: int, cap: int):
    """Pack a fixed-capacity EP dispatch (see ops.reference.ep_pack for the layout)."""
    if not _gpu(x):
        return ref.ep_pack(x, ids, w, slots, experts_per_rank, ep, cap)
    T, H = x.shape
    k = ids.shape[1]
    send = _empty(ep * cap, H, dtype=x.dtype, device=x.device)
    meta = _empty(ep * cap, 2 * k, dtype=torch.float32, device=x.device)
    slot = _empty(T, ep, dtype=torch.int32, device=x.device)
    torch.ops.bfly.ep_pack(x.contiguous(), ids.contiguous(), w.contiguous(), slots, experts_per_rank, ep, cap,
                           send, meta, slot)
    return send, meta, slot


def ep_combine(back, slot):
    """Sum each token's returned partial outputs (one per rank it was sent to)."""
    if not _gpu(back):
        return ref.ep_combine(back, slot)
    out = _empty(slot.shape[0], back.shape[1], dtype=back.dtype, device=back.device)
    torch.ops.bfly.ep_combine(back, slot, out)
    return out


def moe_down_splits(TK: int, num_local: int, H: int, ffn: int, bm: int, cus: int = 256) -> int:
    """Split-K factor of the grouped down projection: enough workgroups for ~2 per CU, with
    at least 16 K-tiles (1024 columns) per split (none for the 256-row big tile)."""
    if bm == 256:
        return 1
    tiles = -(-TK // bm) + (num_local if TK >= num_local else 0)
    wgs = max(1, tiles) * (H // 128)
    sk = 1
    while wgs * sk * 2 <= 2 * cus and (ffn // 64) // (sk * 2) >= 16 and sk < 8:
        sk *= 2
    return sk


def moe_gate_scale_(h, gates, e0: int, num_local: int):
    if not _gpu(h):
        return ref.moe_gate_scale(h, gates, e0, num_local)
    torch.ops.bfly.moe_gate_scale(h, gates, e0, num_local)
    return h


# ---------------------------------------------------------------------------------------
# Shape-generic ops (csrc/kernels/gemm_any.hip, hyper.hip, mixers.hip): bf16 or f32 tensors
# ---------------------------------------------------------------------------------------
ACTS = {"none": 0, "relu2": 1, "xielu": 2}


_tuned_ok: dict = {}


def _mfma_gemm_ok(x, w, out_dtype, bias=None) -> bool:
    """The tuned MFMA GEMM family takes bf16 operands with K % 64 == 0, N % 128 == 0 and 16-byte
    rows, when the plan it would choose for (M, N, K) accepts the shape (a dry run, cached: a
    shallow K can be too short for the plan's split or pipeline depth)."""
    if not (x.dtype == torch.bfloat16 and out_dtype in (None, torch.bfloat16) and w.shape[1] % 64 == 0
            and w.shape[0] % 128 == 0 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and x.shape[0] > 0
            and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0):
        return False
    key = (x.shape[0], w.shape[0], w.shape[1], bias is not None)
    ok = _tuned_ok.get(key)
    if ok is None:
        ok = _tuned_ok[key] = torch.ops.bfly.gemm_check(key[0], key[1], key[2],
                                                       EPILOGUES["bias" if bias is not None else "none"]) == 0
    return ok


def linear_act(x, w, bias=None, act: str = "none", out_dtype=None, act_params=None):
    """y = act(x w^T + bias) for any shape, bf16 or f32 (`out_dtype` f32: keep the f32
    accumulator). act: "none" | "relu2" | "xielu" (act_params = its two coefficients (a_pos,
    a_neg): z > 0: a_pos z^2 + z / 2, else a_neg (exp(z) - 1 - z) + z / 2). bf16 shapes the MFMA
    GEMMs tile go to them (the activation as a pass over the result); every other shape, and f32,
    runs the generic tile kernel."""
    if not _gpu(x):
        return ref.linear_act(x, w, bias, act, out_dtype, act_params)
    a0, a1 = (float(act_params[0]), float(act_params[1])) if act == "xielu" else (0.0, 0.0)
    if _mfma_gemm_ok(x, w, out_dtype, bias):
        y = linear(x, w, bias=bias)
        if act != "none":
            torch.ops.bfly.act_(y, ACTS[act], a0, a1)
        return y
    out = _empty(x.shape[0], w.shape[0], dtype=out_dtype or x.dtype, device=x.device)
    torch.ops.bfly.gemm_any(x, w, bias, ACTS[act], a0, a1, out)
    return out


def embed_norm_streams(ids, table, norm_w, eps: float, offset: float, streams: int):
    """Token embedding, RMS norm with weight (w + offset), copied into `streams` parallel
    residual streams: xs [T, streams, W] f32."""
    if not _gpu(table):
        return ref.embed_norm_streams(ids, table, norm_w, eps, offset, streams)
    xs = _empty(ids.numel(), streams, table.shape[1], dtype=torch.float32, device=table.device)
    torch.ops.bfly.embed_norm_streams(ids, table, norm_w, eps, offset, xs)
    return xs


def hc_pre(xs, w_in, norm_w, eps: float, offset: float, out_dtype):
    """A sublayer's input: the streams mixed by w_in [S], RMS-normed with weight (w + offset)."""
    if not _gpu(xs):
        return ref.hc_pre(xs, w_in, norm_w, eps, offset, out_dtype)
    out = _empty(xs.shape[0], xs.shape[2], dtype=out_dtype, device=xs.device)
    torch.ops.bfly.hc_pre(xs, w_in, norm_w, eps, offset, out)
    return out


def hc_post_(xs, y, mix, w_out):
    """xs[:, r] <- sum_s mix[s, r] xs[:, s] + w_out[r] y, in place (all streams from the old ones)."""
    if not _gpu(xs):
        return ref.hc_post_(xs, y, mix, w_out)
    torch.ops.bfly.hc_post(xs, y, mix, w_out)
    return xs


def hc_post_pre_(xs, y, mix, w_out, w_in2, norm_w2, eps: float, offset: float, out_dtype):
    """hc_post_ followed by the next sublayer's hc_pre on the updated streams, in one kernel (the
    residual update fused with the following norm, as the other families' add + norm)."""
    if not _gpu(xs):
        ref.hc_post_(xs, y, mix, w_out)
        return ref.hc_pre(xs, w_in2, norm_w2, eps, offset, out_dtype)
    out = _empty(xs.shape[0], xs.shape[2], dtype=out_dtype, device=xs.device)
    torch.ops.bfly.hc_post_pre(xs, y, mix, w_out, w_in2, norm_w2, eps, offset, out)
    return out


def hc_final(xs, norm_w, eps: float, offset: float, idx, out_dtype):
    """Sum of the streams of rows `idx` (None: all), RMS-normed with weight (w + offset)."""
    if not _gpu(xs):
        return ref.hc_final(xs, norm_w, eps, offset, idx, out_dtype)
    R = xs.shape[0] if idx is None else idx.numel()
    out = _empty(R, xs.shape[2], dtype=out_dtype, device=xs.device)
    torch.ops.bfly.hc_final(xs, norm_w, eps, offset, idx, out)
    return out


def rope_partial_kv(q, k, v, positions, inv_freq, slots=None, k_cache=None, v_cache=None):
    """Interleaved-pair rotary on the first 2 * len(inv_freq) dims of the q [T, H, D] and
    k [T, G, D] heads, in place, and the append of k, v [T, G, Dv] to the paged caches
    K [blocks, G, BS, D], V [blocks, G, Dv, BS] (V transposed, as the framework's other caches).
    k None: q only."""
    if not _gpu(q):
        return ref.rope_partial_kv(q, k, v, positions, inv_freq, slots, k_cache, v_cache)
    torch.ops.bfly.rope_partial_kv(q, k, v, positions, inv_freq, slots, k_cache, v_cache)
    return q


def row_seq(row_cu, T: int):
    """Row -> sequence map of a packed step (rows outside every sequence: -1); GPU only."""
    out = _empty(T, dtype=torch.int32, device=row_cu.device)
    torch.ops.bfly.row_seq(row_cu, out)
    return out


def attn_window_paged(q, k_cache, v_cache, tables, row_cu, positions, scale: float, window: int, keep_first: int,
                      sink, row_map=None, out=None, fold_heads: bool = False, out_scale=None, chunk: int = 0,
                      softcap: float = 0.0, dist_bias=None, q_temp=None, maps: int = 1, out_dtype=None):
    """Windowed attention of packed rows over the paged cache with kept first positions and a
    sink logit (mixers.hip attn_window_paged_kernel; sink None: an ordinary softmax). `row_map`:
    ops.row_seq(row_cu, T), when the caller already has it. `out_scale` [T, H] f32 multiplies
    every head's output (an output gate). `fold_heads` (one shared key / value head only): the
    heads of a token become rows of the attention tiles, so a token's heads read each cached
    page once instead of once per head.

    Score modifiers, applied in this order before the mask: `q_temp` (coef, every): the scale of a
    row at position p is multiplied by 1 + coef ln(floor((p + 1) / every) + 1); `softcap` > 0:
    s <- cap tanh(s / cap); `dist_bias` (a, b), f32 [H] each: s <- s - a[h] ln(1 + b[h] (p - j)); (a, None):
    the linear form s <- s - a[h] (p - j).
    `chunk` > 0 replaces the window: a row sees the keys of its own chunk of `chunk` positions
    (counted from position 0). `maps` > 1: the key cache holds `maps` key heads per value head
    (K [blocks, G * maps, BS, D]), the query heads are ordered (head, map), and query head (h, m)
    reads key head (g(h), m) and value head g(h): several attention maps over the same values.
    `out_dtype` torch.float32: the output keeps the f32 accumulator."""
    if not _gpu(q):
        return ref.attn_window_paged(q, k_cache, v_cache, tables, row_cu, positions, scale, window, keep_first, sink, out,
                                     out_scale, chunk, softcap, dist_bias, q_temp, maps, out_dtype)
    if out is None:
        out = _empty(q.shape[0], q.shape[1], v_cache.shape[2], dtype=out_dtype or q.dtype, device=q.device)
    if row_map is None:
        row_map = row_seq(row_cu, q.shape[0])
    # steps of few rows (decoding): scratch so that several workgroups can share a tile's pages
    part = None
    rows = q.shape[0] * q.shape[1]
    if q.dtype == torch.bfloat16 and rows <= 2048:
        part = _arena.get(q.device, "attn_window_part", 16 * rows * (v_cache.shape[2] + 2), torch.float32)
    da, db = dist_bias if dist_bias is not None else (None, None)
    qc, qe = q_temp if q_temp is not None else (0.0, 1)
    torch.ops.bfly.attn_window_paged(q, k_cache, v_cache, tables, row_map, row_cu, positions, float(scale), int(window),
                                     int(keep_first), sink, out_scale, bool(fold_heads), part, out, int(chunk),
                                     float(softcap), da, db, float(qc), int(qe), int(maps))
    return out


def gla_scan(q, k, v, z, state, state_slots, row_cu, positions, tau: float, q_scale: float):
    """Gated linear attention over packed rows with the state pooled in `state` [slots, H, D, Dv]
    f32 (updated in place). Returns o [T, H, Dv] f32."""
    if not _gpu(q):
        return ref.gla_scan(q, k, v, z, state, state_slots, row_cu, positions, tau, q_scale)
    o = _empty(q.shape[0], q.shape[1], v.shape[2], dtype=torch.float32, device=q.device)
    torch.ops.bfly.gla_scan(q, k, v, z, state, state_slots, row_cu, positions, float(tau), float(q_scale), o)
    return o


def gla_out(o, g, norm_w, eps: float, out_dtype):
    if not _gpu(o):
        return ref.gla_out(o, g, norm_w, eps, out_dtype)
    out = _empty(o.shape[0], o.shape[1] * o.shape[2], dtype=out_dtype, device=o.device)
    torch.ops.bfly.gla_out(o, g, norm_w, eps, out)
    return out


def moe_route_scores(x, wr, top_k: int, scoring: str = "softmax", renorm: bool = True, bias=None, select_bias=None):
    """Router with f32 logits -> (topk_ids [T, k] int32, topk_w [T, k] f32); scoring "softmax" |
    "sigmoid", `renorm`: divide the chosen scores by their sum ("softmax" + renorm = the softmax
    over the chosen logits alone); `bias` [E] f32 is added to the logits; `select_bias` [E] f32 is
    added to the scores for the choice only, the weights being the chosen experts' plain scores."""
    if not _gpu(x):
        return ref.moe_route_scores(x, wr, top_k, scoring, renorm, bias, select_bias)
    T = x.shape[0]
    # logits: a GEMM with f32 accumulation and f32 output (steps of a few rows: one wave per
    # (token, expert) instead of a one-workgroup GEMM), then one wave per token picks
    if T * wr.shape[0] <= 4096:
        logits = _empty(T, wr.shape[0], dtype=torch.float32, device=x.device)
        torch.ops.bfly.router_logits(x, wr, logits)
    else:
        logits = linear_act(x, wr, out_dtype=torch.float32)
    ids = _empty(T, top_k, dtype=torch.int32, device=x.device)
    w = _empty(T, top_k, dtype=torch.float32, device=x.device)
    torch.ops.bfly.moe_topk_scores(logits, bias, top_k, {"softmax": 0, "sigmoid": 1}[scoring], bool(renorm), ids, w,
                                   select_bias)
    return ids, w


def moe_glu_ffn(x, topk_ids, topk_w, gate_up_w, down_w, limit: float, alpha: float, up_offset: float = 1.0,
                scale_input: bool = True, plain_act=None):
    """Routed GLU experts y = g' sigmoid(alpha g') (u' + up_offset) with g', u' clamped at `limit`
    (inf, alpha 1, up_offset 0: the plain silu GLU). scale_input: each expert runs on (routing
    score * x) and the outputs are summed; otherwise it runs on x and the sum is weighted by the
    scores. See ops.reference.moe_glu_ffn. gate_up_w [E, 2F, H], down_w [E, H, F]. plain_act
    "relu2": experts without a gate, y = relu(W_up h)^2 with gate_up_w [E, F, H] (limit, alpha and
    up_offset unused)."""
    if not _gpu(x):
        return ref.moe_glu_ffn(x, topk_ids, topk_w, gate_up_w, down_w, limit, alpha, None, up_offset, scale_input,
                               plain_act)
    T, H = x.shape
    E, F = gate_up_w.shape[0], down_w.shape[2]
    TK = T * topk_ids.shape[1]
    mt = torch.ops.bfly.moe_sort_max_tiles(TK, E)
    dev = x.device
    work = _arena.get(dev, "moe_glu_work", TK + E + 1 + 2 * mt + 1, torch.int32)
    hmid = _arena.get(dev, "moe_glu_mid", TK * F, x.dtype)
    y = _arena.get(dev, "moe_glu_y", TK * H, torch.float32)
    out = _empty(T, H, dtype=x.dtype, device=dev)
    torch.ops.bfly.moe_glu_ffn(x, topk_ids, topk_w, gate_up_w, down_w, float(limit), float(alpha), float(up_offset),
                               bool(scale_input), work, hmid, y, out, ACTS[plain_act or "none"])
    return out


# ---------------------------------------------------------------------------------------
# Post-norm residual stacks with latent attention (csrc/kernels/postnorm.hip)
# ---------------------------------------------------------------------------------------
def new_empty(*shape, dtype, device) -> torch.Tensor:
    """A step's scratch tensor (poisoned under BFLY_POISON_OUTPUTS like every op output)."""
    return _empty(*shape, dtype=dtype, device=device)


def embed_scaled(ids, table, scale: float, out=None):
    """out[t] = table[ids[t]] * scale, f32 [T, W]."""
    if not _gpu(table):
        return ref.embed_scaled(ids, table, scale, out)
    if out is None:
        out = _empty(ids.numel(), table.shape[1], dtype=torch.float32, device=table.device)
    torch.ops.bfly.embed_scaled(ids, table, float(scale), out)
    return out


def conv_mix(x, w, state, state_slots, row_cu, positions, out_dtype):
    """h_t = x_t + sum_j w[:, j] x_(t - taps + 1 + j): a causal per-channel convolution over the
    rows of each sequence of a packed step, added to its input. x [T, W] f32; w [W, taps] f32 (None:
    h = x); inputs before a sequence's first row of the step come from state[slot] ([slots,
    taps - 1, W] f32, oldest first) and are zero before position 0. Returns h in out_dtype. The
    state is not changed (conv_state_update_ does that, after every reader of the old state)."""
    if not _gpu(x):
        if w is None:
            return x.to(out_dtype)
        return ref.conv_mix(x, w, state, state_slots, row_cu, positions, out_dtype)
    out = _empty(x.shape[0], x.shape[1], dtype=out_dtype, device=x.device)
    torch.ops.bfly.conv_mix(x, w, state, state_slots, row_cu, positions, out)
    return out


def conv_state_update_(x, state, state_slots, row_cu, positions):
    """state[slot] <- the last taps - 1 inputs of every sequence of the step (older ones shift)."""
    if not _gpu(x):
        return ref.conv_state_update_(x, state, state_slots, row_cu, positions)
    torch.ops.bfly.conv_state_update(x, state, state_slots, row_cu, positions)
    return state


def post_norm_add(x, y, norm_w, norm_b, eps: float, scale, out, cast_dtype=None):
    """out = x + scale * layer_norm(y) with weight and bias, all f32 (out may be x); returns out
    rounded to cast_dtype (the next sublayer's GEMM operand), or None."""
    if not _gpu(x):
        return ref.post_norm_add(x, y, norm_w, norm_b, eps, scale, out, cast_dtype)
    cast = None if cast_dtype is None else _empty(x.shape[0], x.shape[1], dtype=cast_dtype, device=x.device)
    torch.ops.bfly.post_norm_add(x, y, norm_w, norm_b, float(eps), scale, out, cast)
    return cast


def post_norm_add_avg(x, y, norm_w, norm_b, eps: float, scale, stack, index: int, avg_w):
    """X = x + scale * layer_norm(y) (y None: X = x); stack[index] = X; x <- sum_(j <= index)
    avg_w[j] stack[j]: the residual update fused with a learned average over the results of all
    layers so far. stack [n, T, W] f32, avg_w [index + 1] f32."""
    if not _gpu(x):
        return ref.post_norm_add_avg(x, y, norm_w, norm_b, eps, scale, stack, index, avg_w)
    torch.ops.bfly.post_norm_add_avg(x, y, norm_w, norm_b, float(eps), scale, stack, int(index), avg_w)
    return x


def latent_prep(z, q_rank: int, kv_rank: int, rot_dim: int, heads: int, qn_w, kvn_w, eps: float, positions, inv_freq,
                slots, k_cache, v_cache, out_dtype):
    """Rows of z = [query latent | key/value latent | shared rotated key part | gate logits] ->
    (RMS-normed query latent [T, q_rank], sigmoid gates [T, heads] f32; q_rank 0 / heads 0: z has no
    such part and None stands in its place); the normed key/value
    latent and the rotated key part are appended to the paged caches K [blocks, 1, BS, kv_rank +
    rot_dim], V [blocks, 1, kv_rank, BS]."""
    if not _gpu(z):
        return ref.latent_prep(z, q_rank, kv_rank, rot_dim, heads, qn_w, kvn_w, eps, positions, inv_freq, slots,
                               k_cache, v_cache, out_dtype)
    T = z.shape[0]
    cq = _empty(T, q_rank, dtype=out_dtype, device=z.device) if q_rank else None
    gate = _empty(T, heads, dtype=torch.float32, device=z.device) if heads else None
    torch.ops.bfly.latent_prep(z, int(q_rank), int(kv_rank), int(rot_dim), int(heads), qn_w, kvn_w, float(eps), positions,
                               inv_freq, slots, k_cache, v_cache, cq, gate)
    return cq, gate


def linear_heads(x, w, out):
    """out[t, h] = w[h] x[t, h]: one small GEMM per head in a single launch. x [T, H, K] and out
    [T, H, N] may be views into wider rows; w [H, N, K] contiguous."""
    if not _gpu(x):
        return ref.linear_heads(x, w, out)
    torch.ops.bfly.linear_heads(x, w, out)
    return out


ATTN_MFMA_SIZES = (32, 64, 96, 128, 192, 256)


def attn_window_pad(size: int, dtype) -> int:
    """Head size a cache of `dtype` should be laid out with so that attn_window_paged takes its
    matrix-core form (bf16: the next of ATTN_MFMA_SIZES; the padding holds zeros). Other types,
    and sizes past the largest, stay as they are (the generic kernel takes any size)."""
    if dtype != torch.bfloat16:
        return size
    return next((s for s in ATTN_MFMA_SIZES if s >= size), size)


def rope_heads_copy(src, dst, positions, inv_freq):
    """dst[t, h, :n] = src[t, h] with the interleaved pairs (2i, 2i + 1), i < len(inv_freq), rotated
    by positions[t] * inv_freq[i]; dst[t, h, n:] = 0. src [T, H, n], dst [T, H, >= n] views into
    wider rows."""
    if not _gpu(src):
        return ref.rope_heads_copy(src, dst, positions, inv_freq)
    torch.ops.bfly.rope_heads_copy(src, dst, positions, inv_freq)
    return dst


def layer_norm_rows(x, w, b, eps: float, idx, out_dtype):
    """Layer norm with weight and bias of rows idx (None: all) of the f32 residual x."""
    if not _gpu(x):
        return ref.layer_norm_rows(x, w, b, eps, idx, out_dtype)
    R = x.shape[0] if idx is None else idx.numel()
    out = _empty(R, x.shape[1], dtype=out_dtype, device=x.device)
    torch.ops.bfly.layer_norm_rows(x, w, b, float(eps), idx, out)
    return out


# ---------------------------------------------------------------------------------------
# Parallel layers with a token shift, differential attention, dense clamped GLU
# (csrc/kernels/parlayer.hip)
# ---------------------------------------------------------------------------------------
def par_norm_shift(x, ya, yb, norm_a, norm_b, eps: float, offset: float, shift, state, state_slots, row_cu, positions,
                   out_dtype, x_out=None, row_map=None):
    """The step between two parallel layers, in one kernel: x' = x + (ya + yb) (the outputs of the
    previous layer's mixer and feed-forward, either may be None; written to x_out, which must be
    another buffer than x), then both inputs of the next layer from one RMS statistic of x':
    ha = x' / rms (norm_a + offset) for the mixer and hb = x' / rms (norm_b + offset) for the
    feed-forward (norm_b None: no hb). With `shift` [W] f32 the mixer's input is mixed with the
    previous token's: ha + (prev - ha) shift, where prev is the unmixed ha of the row before in the
    same sequence, state[slot] ([slots, W] f32) for a sequence's first row of the step, zero at
    position 0; state[slot] then takes the unmixed ha of the sequence's last row. Returns
    (x', ha, hb); x' is x itself when ya and yb are None."""
    if not _gpu(x):
        return ref.par_norm_shift(x, ya, yb, norm_a, norm_b, eps, offset, shift, state, state_slots, row_cu, positions,
                                  out_dtype, x_out)
    T, W = x.shape
    if ya is None and yb is None:
        x_out = None
    elif x_out is None:
        x_out = _empty(T, W, dtype=torch.float32, device=x.device)
    ha = _empty(T, W, dtype=out_dtype, device=x.device)
    hb = None if norm_b is None else _empty(T, W, dtype=out_dtype, device=x.device)
    if row_map is None:
        row_map = row_seq(row_cu, T)
    torch.ops.bfly.par_norm_shift(x, ya, yb, x_out, norm_a, norm_b, float(eps), float(offset), shift,
                                  state if shift is not None else None, state_slots if shift is not None else None,
                                  row_map, row_cu, positions, ha, hb)
    return (x if x_out is None else x_out), ha, hb


def par_final(x, ya, yb, norm_w, eps: float, offset: float, idx, out_dtype):
    """RMS norm with weight (w + offset) of rows idx (None: all) of x + (ya + yb): the last
    parallel layer's residual sum fused with the output norm."""
    if not _gpu(x):
        return ref.par_final(x, ya, yb, norm_w, eps, offset, idx, out_dtype)
    R = x.shape[0] if idx is None else idx.numel()
    out = _empty(R, x.shape[1], dtype=out_dtype, device=x.device)
    torch.ops.bfly.par_final(x, ya, yb, norm_w, float(eps), float(offset), idx, out)
    return out


def rope_table(positions, inv_freq):
    """cs [T, 2, n] f32: cosines and sines of positions[t] * inv_freq[i] (the f32 frequencies; product
    and evaluation in f64). One table serves every layer of a step that rotates by these
    frequencies (qk_norm_rope_kv's `cs`). None when nothing rotates."""
    if inv_freq.numel() == 0:
        return None
    if not _gpu(positions):
        a = positions.double()[:, None] * inv_freq.double()[None]
        return torch.stack([torch.cos(a), torch.sin(a)], 1).float()
    cs = _empty(positions.numel(), 2, inv_freq.numel(), dtype=torch.float32, device=positions.device)
    torch.ops.bfly.rope_table(positions, inv_freq, cs)
    return cs


def qk_norm_rope_kv(q, k, v, qn_w, kn_w, eps: float, positions, inv_freq, slots, k_cache, v_cache, q_out=None, cs=None):
    """Queries and keys prepared per head and the paged append, in one kernel: RMS norm over the
    head with weight qn_w / kn_w [D] f32 (None: no norm), then rotation of the first 2 n dims
    (n = len(inv_freq), may be 0) with dimension i paired with i + n by positions[t] * inv_freq[i].
    q [T, Hq, D] -> q_out [T, Hq, Dp] (Dp = the key cache's row size, zero padded); k [T, Gk, D],
    v [T, Gv, Dv] -> K [blocks, Gk, BS, Dp], V [blocks, Gv, Dvp, BS] at slots[t] >= 0 (the caches'
    padding keeps the zeros it was allocated with). `cs`: rope_table(positions, inv_freq), when the
    caller already has it. Returns q_out, or q itself when the queries need nothing (no norm, no
    rotation, no padding: only the keys and values are appended)."""
    plain = qn_w is None and inv_freq.numel() == 0 and k_cache.shape[3] == q.shape[2] and q_out is None
    if q_out is None and not (plain and _gpu(q)):
        q_out = _empty(q.shape[0], q.shape[1], k_cache.shape[3], dtype=q.dtype, device=q.device)
    if not _gpu(q):
        return ref.qk_norm_rope_kv(q, k, v, qn_w, kn_w, eps, positions, inv_freq, slots, k_cache, v_cache, q_out)
    if cs is None:
        cs = rope_table(positions, inv_freq)
    torch.ops.bfly.qk_norm_rope_kv(q, k, v, qn_w, kn_w, float(eps), cs, slots, k_cache, v_cache, q_out)
    return q if q_out is None else q_out


def diff_combine(a, lam: float, eps: float, out_mul: float, gate, Dv: int, out_dtype):
    """Differential attention's combination: a [T, 2 H, >= Dv] f32 with heads ordered (head, map);
    o = a[:, 2h] - lam a[:, 2h + 1] over the first Dv values, divided by its root mean square (eps
    inside the root), times out_mul, times sigmoid(gate) (gate [T, H * Dv] logits; None: no
    gate). Returns [T, H * Dv] in out_dtype."""
    if not _gpu(a):
        return ref.diff_combine(a, lam, eps, out_mul, gate, Dv, out_dtype)
    out = _empty(a.shape[0], (a.shape[1] // 2) * Dv, dtype=out_dtype, device=a.device)
    torch.ops.bfly.diff_combine(a, float(lam), float(eps), float(out_mul), gate, int(Dv), out)
    return out


def glu_clamp(gu, limit: float, alpha: float, up_offset: float, group: int = 0):
    """gu [T, 2 F] = [gate | up] (rows may be a view; group > 0: alternating blocks of `group` gate
    and up columns, the layout of the GEMMs' fused gate / up epilogues): g sigmoid(alpha g) (u +
    up_offset) with g = min(gate, limit), u = clamp(up, -limit, limit) -> [T, F]."""
    if not _gpu(gu):
        return ref.glu_clamp(gu, limit, alpha, up_offset, None, group)
    out = _empty(gu.shape[0], gu.shape[1] // 2, dtype=gu.dtype, device=gu.device)
    torch.ops.bfly.glu_clamp(gu, float(limit), float(alpha), float(up_offset), int(group), out)
    return out


def linear_glu(x, w, bias_block, F: int, limit: float, alpha: float, up_offset: float, group: int = 0):
    """The clamped-GLU half of a feed-forward: [gate | up] projection with biases and the
    activation, F columns wide. group == 0: w [2 F (+ padding), K] = [gate rows | up rows] with `bias_block` the
    matching bias vector; the activation is a pass over the projection. group == SILU_INTERLEAVE:
    the rows (and biases) alternate in 16-row gate / up blocks and `bias_block` is
    glu_bias_block(...); bf16 shapes whose GEMM plan has the fused epilogue run as ONE kernel that
    writes [T, F] only, every other case as projection + pass. Returns [T, rows / 2]."""
    N = w.shape[0]
    if group == 0:
        return glu_clamp(linear_act(x, w, bias=bias_block)[:, :2 * F], limit, alpha, up_offset)
    if _gpu(x) and _mfma_gemm_ok(x, w, None) and _glu_fused_ok(x.shape[0], N, w.shape[1]):
        return linear(x, w, bias=bias_block, epilogue="glu")
    return glu_clamp(linear_act(x, w, bias=bias_block[:N]), limit, alpha, up_offset, group)


_glu_ok: dict = {}


def _glu_fused_ok(M: int, N: int, K: int) -> bool:
    ok = _glu_ok.get((M, N, K))
    if ok is None:
        ok = _glu_ok[(M, N, K)] = torch.ops.bfly.gemm_check(M, N, K, EPILOGUES["glu"]) == 0
    return ok


# ---------------------------------------------------------------------------------------
# Sandwich-norm residual stacks with a gated delta rule (csrc/kernels/delta.hip)
# ---------------------------------------------------------------------------------------
def post_norm_add_norm(x, y, norm_w, norm_b, eps: float, mult: float, extra, norm2_w, norm2_b, out_dtype):
    """One launch between two sublayers of a stack with norms on both sides of every sublayer:
    x <- x + mult * layer_norm(y; norm_w, norm_b) (+ extra [T, W] f32, e.g. the embedding output
    re-entering before a repeated span), in place in f32, and the next sublayer's input
    layer_norm(x; norm2_w, norm2_b) in out_dtype (norm2_w None: no next input, returns None)."""
    if not _gpu(x):
        return ref.post_norm_add_norm(x, y, norm_w, norm_b, eps, mult, extra, norm2_w, norm2_b, out_dtype)
    h = None if norm2_w is None else _empty(x.shape[0], x.shape[1], dtype=out_dtype, device=x.device)
    torch.ops.bfly.post_norm_add_norm(x, y, norm_w, norm_b, float(eps), float(mult), extra, norm2_w, norm2_b, h)
    return h


CONV_ACTS = {"none": 0, "silu": 1}


def short_conv_act(z, w, state, state_slots, row_cu, positions, act: str = "silu", out_dtype=torch.float32):
    """y_t = act(sum_j w[:, j] z_(t - taps + 1 + j)): a short causal convolution over the rows of each
    sequence of a packed step, per channel, with an activation. z [T, C] may be a view into wider
    projected rows (any element type the model runs in); w [C, taps] f32, the last column weighs the
    current row; rows before a sequence's first row of the step come from state[slot] ([slots,
    taps - 1, C] f32, oldest first) and are zero before position 0. The state is not changed
    (short_conv_state_update_ does that, after every reader of the old state)."""
    if not _gpu(z):
        return ref.short_conv_act(z, w, state, state_slots, row_cu, positions, act, out_dtype)
    out = _empty(z.shape[0], z.shape[1], dtype=out_dtype, device=z.device)
    torch.ops.bfly.short_conv_act(z, w, state, state_slots, row_cu, positions, CONV_ACTS[act], out)
    return out


def short_conv_state_update_(z, state, state_slots, row_cu, positions):
    """state[slot] <- the last taps - 1 rows of z of every sequence of the step (older ones shift)."""
    if not _gpu(z):
        return ref.short_conv_state_update_(z, state, state_slots, row_cu, positions)
    torch.ops.bfly.short_conv_state_update(z, state, state_slots, row_cu, positions)
    return state


def delta_scan(q, k, v, b, a, a_log, dt_bias, state, state_slots, row_cu, positions, q_scale: float,
               unit_eps: float = 1e-6):
    """Gated delta rule over packed rows with the state pooled in `state` [slots, H, Dv, D] f32 (a
    head's D x Dv matrix stored column by column; updated in place; a sequence whose step starts at position 0 starts from zero). q, k [T, G, D],
    v [T, H, Dv] (views allowed); b, a [T, H] the logits of the write strength and the decay's step;
    a_log, dt_bias [H] f32. See ops.reference.delta_scan. Returns o [T, H, Dv] f32."""
    if not _gpu(q):
        return ref.delta_scan(q, k, v, b, a, a_log, dt_bias, state, state_slots, row_cu, positions, q_scale, unit_eps)
    o = _empty(q.shape[0], v.shape[1], v.shape[2], dtype=torch.float32, device=q.device)
    torch.ops.bfly.delta_scan(q, k, v, b, a, a_log, dt_bias, state, state_slots, row_cu, positions, float(q_scale),
                              float(unit_eps), o)
    return o
