"""Plain-PyTorch reference implementations of every butterfly_amd op.

Two roles:
  * the numerics oracle for the HIP kernels (tests compare each kernel against the fp32
    computation here), and
  * the CPU execution path for the gloo plumbing configuration (SURVEY.md §7.3 item 8:
    the GPU path is HIP-only; the CPU path exists for tests and the CPU/gloo config).

Semantics match the kernels exactly, including in-place side effects and cache layouts:
  k_cache [num_blocks, Hkv, BS, D], v_cache [num_blocks, Hkv, D, BS] (V transposed).
"""
from __future__ import annotations

import math
import struct

import torch
import torch.nn.functional as F

SILU_INTERLEAVE = 16  # gate/up row-group size of the fused SwiGLU weight layout


def rms_norm(x, w, eps, out=None, residual=None):
    if residual is not None:
        residual.copy_((x.float() + residual.float()).to(residual.dtype))
        src = residual
    else:
        src = x
    xf = src.float()
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    y = y.to(x.dtype)
    if out is None:
        return y
    out.copy_(y)
    return out


def layer_norm(x, w, b, eps, out=None, residual=None):
    if residual is not None:
        residual.copy_((x.float() + residual.float()).to(residual.dtype))
        src = residual
    else:
        src = x
    y = F.layer_norm(src.float(), (src.shape[-1],), w.float(), b.float(), eps).to(x.dtype)
    if out is None:
        return y
    out.copy_(y)
    return out


def rope_tables(head_dim: int, max_pos: int, theta: float, scaling: dict | None = None,
                device="cpu"):
    """cos/sin tables [max_pos, head_dim/2] (f32) for the rotate-half convention.

    `scaling` supports the Llama-3.1 "llama3" frequency remap
    ({"type": "llama3", "factor", "low_freq_factor", "high_freq_factor",
      "original_max_position_embeddings"}).
    """
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim))
    if scaling and scaling.get("type") == "llama3":
        factor = scaling["factor"]
        lo, hi = scaling["low_freq_factor"], scaling["high_freq_factor"]
        orig = scaling["original_max_position_embeddings"]
        lo_wl, hi_wl = orig / lo, orig / hi
        wl = 2 * math.pi / inv
        smooth = (orig / wl - lo) / (hi - lo)
        scaled = torch.where(wl > lo_wl, inv / factor, inv)
        mid = (wl <= lo_wl) & (wl >= hi_wl)
        scaled = torch.where(mid, (1 - smooth) * inv / factor + smooth * inv, scaled)
        inv = scaled
    t = torch.arange(max_pos, dtype=torch.float64)
    f = torch.outer(t, inv)
    return f.cos().float().to(device), f.sin().float().to(device)


def _rotate(x, cos, sin):
    h = x.shape[-1] // 2
    x0, x1 = x[..., :h].float(), x[..., h:].float()
    return torch.cat([x0 * cos - x1 * sin, x1 * cos + x0 * sin], -1)


def sample_pack(scores, ids):
    return torch.stack([scores.float(), ids.to(torch.float32)], 1)


def sample_merge(allp):
    best = allp[:, :, 0].argmax(0)
    return allp.gather(0, best.view(1, -1, 1).expand(1, -1, 2))[0, :, 1].to(torch.int32)


def gather_rows(src, idx, out):
    """out[i] = src[idx[i]] where idx[i] >= 0; other rows of `out` are left as they are."""
    ok = idx >= 0
    if bool(ok.all()):
        out.copy_(src.index_select(0, idx.long()))
    else:
        rows = ok.nonzero().flatten()
        out[rows] = src.index_select(0, idx[rows].long())
    return out


def rope_kv(qkv, positions, cos, sin, n_q, n_kv, slots=None, k_cache=None, v_cache=None):
    T = qkv.shape[0]
    D = qkv.shape[1] // (n_q + 2 * n_kv)
    v3 = qkv.view(T, n_q + 2 * n_kv, D)
    c = cos[positions.long()].unsqueeze(1)
    s = sin[positions.long()].unsqueeze(1)
    rot = _rotate(v3[:, : n_q + n_kv], c, s).to(qkv.dtype)
    v3[:, : n_q + n_kv] = rot
    if slots is not None:
        kv_append(v3[:, n_q: n_q + n_kv], v3[:, n_q + n_kv:], slots, k_cache, v_cache)
    return qkv


def kv_append(k, v, slots, k_cache, v_cache):
    BS = k_cache.shape[2]
    sl = slots.long()
    keep = sl >= 0
    sl = sl[keep]
    blk, off = sl // BS, sl % BS
    k, v = k[keep], v[keep]
    if k_cache.dtype == torch.float8_e4m3fn:   # the kernels clamp to the e4m3 range
        k, v = k.float().clamp(-448, 448), v.float().clamp(-448, 448)
    k_cache[blk, :, off, :] = k.to(k_cache.dtype)
    v_cache[blk, :, :, off] = v.to(v_cache.dtype)


def silu_mul(gu, out=None, interleave=0):
    ffn = gu.shape[-1] // 2
    g, u = split_gate_up(gu, interleave)
    y = (F.silu(g.float()) * u.float()).to(gu.dtype)
    if out is None:
        return y
    out.copy_(y.view(out.shape))
    return out


def split_gate_up(gu, interleave=0):
    ffn = gu.shape[-1] // 2
    if interleave == 0:
        return gu[..., :ffn], gu[..., ffn:]
    lead = gu.shape[:-1]
    r = gu.reshape(*lead, ffn // interleave, 2, interleave)
    return r[..., 0, :].reshape(*lead, ffn), r[..., 1, :].reshape(*lead, ffn)


def interleave_gate_up(gate_w, up_w, group=SILU_INTERLEAVE):
    """[ffn, K] gate and up weights -> [2*ffn, K] rows in alternating `group`-row blocks."""
    ffn, K = gate_w.shape
    g = gate_w.reshape(ffn // group, group, K)
    u = up_w.reshape(ffn // group, group, K)
    return torch.stack([g, u], 1).reshape(2 * ffn, K)


def gelu(x, out=None):
    y = F.gelu(x.float(), approximate="tanh").to(x.dtype)
    if out is None:
        return y
    out.copy_(y)
    return out


def add(a, b, out=None):
    y = (a.float() + b.float()).to(a.dtype)
    if out is None:
        return y
    out.copy_(y)
    return out


def embed(ids, table, vstart=0, out=None):
    local = ids.long() - vstart
    ok = (local >= 0) & (local < table.shape[0])
    y = table[local.clamp(0, table.shape[0] - 1)] * ok.unsqueeze(-1).to(table.dtype)
    if out is None:
        return y
    out.copy_(y.view(out.shape))
    return out


def _mix64(z):
    # splitmix64 finaliser on int64 tensors with wrap-around (matches sample.hip)
    m = (1 << 64) - 1
    z = z & m
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & m
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & m
    return z ^ (z >> 31)


def gumbel_uniform(seed: int, idx: torch.Tensor) -> torch.Tensor:
    """Python-int exact replica of the kernel's counter-based uniform (slow; tests only)."""
    m = (1 << 64) - 1
    out = []
    for i in idx.tolist():
        h = _mix64((seed * 0x9E3779B97F4A7C15 + i + 1) & m)
        out.append(((h >> 40) + 0.5) * (1.0 / 16777216.0))
    return torch.tensor(out, dtype=torch.float32)


def sample(logits, temps=None, seeds=None, vstart=0, thresh=None, check_finite=False):
    """Greedy (temp <= 0) or Gumbel-max temperature sampling; returns (ids int32, scores f32).
    `thresh[r]`: tokens whose logit / temperature is below it are excluded (top-k / top-p).
    `check_finite`: a row with an Inf / NaN logit gives id -1, score +inf."""
    lf = logits.float()
    rows, V = lf.shape
    ids, scores = [], []
    for r in range(rows):
        if check_finite and not bool(torch.isfinite(lf[r]).all()):
            ids.append(-1)
            scores.append(float("inf"))
            continue
        t = float(temps[r]) if temps is not None else 0.0
        s = lf[r]
        if t > 0:
            u = gumbel_uniform(int(seeds[r]), torch.arange(vstart, vstart + V))
            s = s * (1.0 / t)
            keep = s >= float(thresh[r]) if thresh is not None else torch.ones_like(s, dtype=torch.bool)
            s = torch.where(keep, s - torch.log(-torch.log(u)), torch.full_like(s, float("-inf")))
        i = int(torch.argmax(s))
        ids.append(i + vstart)
        scores.append(float(s[i]))
    return (torch.tensor(ids, dtype=torch.int32, device=logits.device),
            torch.tensor(scores, dtype=torch.float32, device=logits.device))


def ordered_key(s: torch.Tensor) -> torch.Tensor:
    """Order-preserving map of f32 values to u32 keys (held in int64), as in sample.hip."""
    u = s.float().contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    return torch.where((u & 0x80000000) != 0, (~u) & 0xFFFFFFFF, u | 0x80000000)


def unordered_key(k: int) -> float:
    u = (k & 0x7FFFFFFF) if (k & 0x80000000) else (~k & 0xFFFFFFFF)
    return struct.unpack("<f", struct.pack("<I", u))[0]


def topkp_threshold(logits, temps, top_k, top_p, reduce_sum=None, reduce_max=None,
                    use_k: bool = True, use_p: bool = True):
    """Exact top-k / top-p thresholds on s = logit * (1 / temperature) by the same 4-pass,
    8-bit radix select as the tkp_* kernels (sample.hip), pass for pass: `reduce_sum` /
    `reduce_max` (in-place all-reduces over the TP group, or None) see the same histograms
    and row maxima, so a vocab-parallel CPU run exercises the GPU path's collective pattern.
    Returns thresh [R] f32 (-inf: row unfiltered)."""
    lf = logits.float()
    R, V = lf.shape
    inv_t = torch.where(temps > 0, 1.0 / temps.float().clamp(min=1e-30), torch.ones_like(temps.float()))
    s = lf * inv_t.view(R, 1)
    key = ordered_key(s)
    smax = (ordered_key(s.max(1).values if V else torch.full((R,), float("-inf"))) ^ 0x80000000)
    smax = torch.where(smax >= 2 ** 31, smax - 2 ** 32, smax).to(torch.int32)
    if reduce_max is not None:
        reduce_max(smax)
    mx = torch.tensor([unordered_key((int(v) & 0xFFFFFFFF) ^ 0x80000000) for v in smax.tolist()],
                      dtype=torch.float32)
    k_act = [bool(temps[r] > 0 and top_k[r] > 0) for r in range(R)]
    p_act = [bool(temps[r] > 0 and top_p[r] < 1.0) for r in range(R)]
    tk_pre, k_rem = [0] * R, [int(top_k[r]) for r in range(R)]
    tp_pre, m_above, z = [0] * R, [0.0] * R, [0.0] * R
    mass = torch.exp(s - mx.view(R, 1))
    for phase, on in ((0, use_k), (1, use_p)):
        if not on:
            continue
        for p in range(4):
            shift = 24 - 8 * p
            hist = torch.zeros(R, 512, dtype=torch.float32)
            for r in range(R):
                if not (k_act[r] if phase == 0 else p_act[r]):
                    continue
                kr = key[r]
                sel = torch.ones(V, dtype=torch.bool)
                if phase == 1 and k_act[r]:
                    sel &= kr >= tk_pre[r]
                if p > 0:
                    sel &= (kr >> (shift + 8)) == (tk_pre[r] if phase == 0 else tp_pre[r])
                d = (kr[sel] >> shift) & 255
                hist[r, :256] = torch.bincount(d, minlength=256).float()
                if phase == 1:
                    hist[r, 256:] = torch.zeros(256).index_add_(0, d, mass[r][sel])
            if reduce_sum is not None:
                reduce_sum(hist)
            for r in range(R):
                cnt, ms = hist[r, :256].tolist(), hist[r, 256:].tolist()
                if phase == 0:
                    if not k_act[r]:
                        continue
                    if p == 0 and sum(cnt) < k_rem[r]:
                        k_act[r] = False
                        continue
                    run = 0.0
                    for d in range(255, -1, -1):
                        if run < k_rem[r] <= run + cnt[d]:
                            tk_pre[r] = (tk_pre[r] << 8) | d
                            k_rem[r] -= int(run)
                            break
                        run += cnt[d]
                else:
                    if not p_act[r]:
                        continue
                    if p == 0:
                        z[r], m_above[r] = float(sum(ms)), 0.0
                    lim = float(top_p[r]) * z[r]
                    run, best, best_above = 0.0, 255, 0.0
                    for d in range(255, -1, -1):
                        if cnt[d] > 0 and m_above[r] + run <= lim:
                            best, best_above = d, run
                        run += ms[d]
                    tp_pre[r] = (tp_pre[r] << 8) | best
                    m_above[r] += best_above
    out = torch.full((R,), float("-inf"), dtype=torch.float32)
    for r in range(R):
        if k_act[r] or p_act[r]:
            kk = max(tk_pre[r] if k_act[r] else 0, tp_pre[r] if p_act[r] else 0)
            out[r] = unordered_key(kk)
    return out


def glu_bias_block(bias, limit, alpha, up_offset):
    """The fused clamped-GLU epilogue's block: N bias values (bf16, interleaved like the weight's
    rows) followed by {limit, alpha, up_offset} as three f32 values in six bf16 slots."""
    blk = torch.zeros(bias.numel() + 6, dtype=torch.bfloat16, device=bias.device)
    blk[:bias.numel()] = bias.to(torch.bfloat16)
    blk[bias.numel():].view(torch.float32).copy_(torch.tensor([limit, alpha, up_offset], dtype=torch.float32))
    return blk


def linear(x, w, bias=None, epilogue="none", out=None):
    y = x.float() @ w.float().t()
    if epilogue == "glu":       # bias = glu_bias_block(...): clamped GLU on interleaved gate / up rows
        N = w.shape[0]
        lim, alpha, off = bias[N:].view(torch.float32).tolist()
        y = glu_clamp(y + bias[:N].float(), lim, alpha, off, torch.float32, SILU_INTERLEAVE)
        bias = None
    if bias is not None:
        y = y + bias.float()
    if epilogue == "silu":
        g, u = split_gate_up(y, SILU_INTERLEAVE)
        y = F.silu(g) * u
    y = y.to(x.dtype)
    if out is None:
        return y
    out.copy_(y)
    return out


def attn_prefill(q, k, v, cu_seqlens, max_seqlen, scale, causal=True, out=None, cu_seqlens_k=None,
                 return_lse=False):
    """q [T, Hq, D], k/v [Tk, Hkv, D]; varlen sequences given by cu_seqlens (int32), keys by
    cu_seqlens_k (default: the same rows). With return_lse also returns ln sum exp(scaled
    scores) per (row, head) [T, Hq] f32, -inf where a row sees no key."""
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    res = torch.zeros(T, Hq, D, dtype=q.dtype, device=q.device)
    lse = torch.full((T, Hq), float("-inf"), dtype=torch.float32, device=q.device)
    cu = cu_seqlens.tolist()
    cuk = cu_seqlens_k.tolist() if cu_seqlens_k is not None else cu
    for i in range(len(cu) - 1):
        a, b = cu[i], cu[i + 1]
        ka, kb = cuk[i], cuk[i + 1]
        if b <= a or kb <= ka:
            continue
        qs = q[a:b].float().transpose(0, 1)                       # [Hq, L, D]
        ks = k[ka:kb].float().transpose(0, 1).repeat_interleave(G, 0)
        vs = v[ka:kb].float().transpose(0, 1).repeat_interleave(G, 0)
        s = (qs @ ks.transpose(1, 2)) * scale
        if causal:
            L = b - a
            mask = torch.ones(L, kb - ka, dtype=torch.bool, device=q.device).triu(1)
            s = s.masked_fill(mask, float("-inf"))
        lse[a:b] = torch.logsumexp(s, -1).transpose(0, 1)
        p = torch.softmax(s, -1)
        res[a:b] = (p @ vs).transpose(0, 1).to(q.dtype)
    if out is not None:
        out.copy_(res)
        res = out
    return (res, lse) if return_lse else res


def attn_lse_merge_(acc_o, acc_lse, o, lse):
    """acc_lse <- log(e^acc_lse + e^lse); acc_o <- weighted mix of acc_o and o (in place)."""
    new = torch.logaddexp(acc_lse, lse)
    ok = new > float("-inf")
    wa = torch.where(ok, torch.exp(acc_lse - new), torch.zeros_like(new))
    wb = torch.where(ok, torch.exp(lse - new), torch.zeros_like(new))
    mixed = acc_o * wa.unsqueeze(-1) + o.float() * wb.unsqueeze(-1)
    acc_o.copy_(torch.where(ok.unsqueeze(-1), mixed, acc_o))
    acc_lse.copy_(torch.where(ok, new, acc_lse))
    return acc_o, acc_lse


def attn_decode(q, k_cache, v_cache, block_tables, ctx_lens, scale, max_ctx=None,
                part_tokens=None, out=None, **_):
    """q [B, Hq, D] (one token per sequence) against the paged cache."""
    B, Hq, D = q.shape
    Hkv, BS = k_cache.shape[1], k_cache.shape[2]
    G = Hq // Hkv
    res = torch.empty(B, Hq, D, dtype=q.dtype, device=q.device)
    for b in range(B):
        n = int(ctx_lens[b])
        nblk = (n + BS - 1) // BS
        blocks = block_tables[b, :nblk].long()
        ks = k_cache[blocks].permute(1, 0, 2, 3).reshape(Hkv, nblk * BS, D)[:, :n].float()
        vs = v_cache[blocks].permute(1, 0, 3, 2).reshape(Hkv, nblk * BS, D)[:, :n].float()
        ks = ks.repeat_interleave(G, 0)
        vs = vs.repeat_interleave(G, 0)
        s = torch.einsum("hd,hnd->hn", q[b].float(), ks) * scale
        p = torch.softmax(s, -1)
        res[b] = torch.einsum("hn,hnd->hd", p, vs).to(q.dtype)
    if out is None:
        return res
    out.copy_(res.view(out.shape))
    return out


def attn_prefill_paged(q, k_cache, v_cache, tables, cu_q, positions, max_q, scale, out=None):
    """Chunked prefill over the paged cache: rows [cu_q[s], cu_q[s+1]) of sequence s (query
    positions `positions[row]`) attend causally to keys [0, positions[row]] of the sequence,
    read through tables[s] (the chunk's own K/V are already in the cache)."""
    T, Hq, D = q.shape
    Hkv, BS = k_cache.shape[1], k_cache.shape[2]
    G = Hq // Hkv
    res = torch.zeros(T, Hq, D, dtype=q.dtype, device=q.device)
    cu = [int(x) for x in cu_q.tolist()]
    pos = positions.long()
    for s in range(len(cu) - 1):
        a, b = cu[s], cu[s + 1]
        if b <= a:
            continue
        n = int(pos[b - 1]) + 1
        nblk = (n + BS - 1) // BS
        blocks = tables[s, :nblk].long()
        ks = k_cache[blocks].permute(1, 0, 2, 3).reshape(Hkv, nblk * BS, D)[:, :n].float().repeat_interleave(G, 0)
        vs = v_cache[blocks].permute(1, 0, 3, 2).reshape(Hkv, nblk * BS, D)[:, :n].float().repeat_interleave(G, 0)
        sc = torch.einsum("thd,hnd->htn", q[a:b].float(), ks) * scale
        mask = torch.arange(n, device=q.device)[None, :] > pos[a:b, None]
        sc = sc.masked_fill(mask[None], float("-inf"))
        res[a:b] = torch.einsum("htn,hnd->thd", torch.softmax(sc, -1), vs).to(q.dtype)
    if out is None:
        return res
    out.copy_(res)
    return out


# ---------------------------------------------------------------------------------------
# Deterministic init and MoE gating
# ---------------------------------------------------------------------------------------
_M32 = 0xFFFFFFFF


def _fmix32(h):
    h = h ^ (h >> 16)
    h = (h * 0x85EBCA6B) & _M32
    h = h ^ (h >> 13)
    h = (h * 0xC2B2AE35) & _M32
    return h ^ (h >> 16)


def init_hash(out, grow0, gcol0, gcols, seed, amp):
    """Value of global element (r, c) = amp * (2u - 1), u = hash(seed, r*gcols + c)."""
    rows, cols = out.shape
    r = torch.arange(rows, dtype=torch.int64).unsqueeze(1) + grow0
    c = torch.arange(cols, dtype=torch.int64).unsqueeze(0) + gcol0
    idx = (r * gcols + c) & _M32
    h = _fmix32((idx * 0x9E3779B1 + seed) & _M32)
    u = (h >> 8).to(torch.float32) * (1.0 / 16777216.0) + (0.5 / 16777216.0)
    out.copy_((amp * (2.0 * u - 1.0)).to(out.dtype))
    return out


def moe_route(x, wr, top_k):
    """-> (gates [T, E] f32 dense, topk_ids [T, k] int32, topk_w [T, k] f32); Mixtral
    semantics: softmax over all experts, top-k, renormalise over the selected."""
    logits = x.float() @ wr.float().t()
    p = torch.softmax(logits, -1)
    w, ids = torch.topk(p, top_k, -1)
    w = w / w.sum(-1, keepdim=True)
    gates = torch.zeros_like(p).scatter_(1, ids, w)
    return gates, ids.to(torch.int32), w


def moe_gate_scale(h, gates, e0, num_local):
    T = h.shape[0]
    F = h.shape[1] // num_local
    g = gates[:, e0:e0 + num_local].to(torch.float32)
    v = h.float().view(T, num_local, F) * g.unsqueeze(-1)
    h.copy_(v.view(T, num_local * F).to(h.dtype))
    return h


def moe_sparse_ffn(x, topk_ids, topk_w, gu_w, down_w, e0: int, num_local: int, ffn: int):
    """Token-routed expert FFN over the local experts (SwiGLU, gate/up interleaved rows):
    out[t] = sum_j w[t, j] * down_e(silu(g_e x_t) * u_e x_t) for j with local e = ids[t, j]."""
    T, H = x.shape
    out = torch.zeros(T, H, dtype=torch.float32, device=x.device)
    ids = topk_ids.long() - e0
    for el in range(num_local):
        hit = (ids == el)
        tok = hit.any(-1).nonzero().flatten()
        if tok.numel() == 0:
            continue
        w_e = (topk_w * hit).sum(-1)[tok]
        gu = gu_w[el * 2 * ffn:(el + 1) * 2 * ffn]
        h = linear(x[tok], gu, epilogue="silu")
        y = linear(h, down_w[:, el * ffn:(el + 1) * ffn].contiguous())
        out[tok] += w_e.unsqueeze(-1).float() * y.float()
    return out.to(x.dtype)


def ep_pack(x, ids, w, slots, experts_per_rank: int, ep: int, cap: int):
    """Fixed-capacity EP dispatch (reference of ep_pack_kernel): token t goes once to every
    rank d owning one of its experts, at row d * cap + (number of earlier tokens bound for d).
    Returns send [ep*cap, H], meta [ep*cap, 2k] f32 (expert ids local to the row's rank as
    int32 bits, -1 otherwise; gate weights), slot [T, ep] int32 (-1: not sent)."""
    T, H = x.shape
    k = ids.shape[1]
    idl = ids.long()
    if slots is not None:
        idl = idl.masked_fill((slots < 0).unsqueeze(1), -1)
    dest = torch.where(idl >= 0, torch.div(idl.clamp(min=0), experts_per_rank, rounding_mode="floor"), ep)
    hit = torch.zeros(T, ep + 1, dtype=torch.int64)
    if T:
        hit.scatter_(1, dest, 1)
    hit = hit[:, :ep]
    pos = torch.cumsum(hit, 0) - hit
    slot = torch.where(hit > 0, torch.arange(ep) * cap + pos, -1)
    send = torch.zeros(ep * cap, H, dtype=x.dtype)
    mid = torch.full((ep * cap, k), -1, dtype=torch.int32)
    mw = torch.zeros(ep * cap, k, dtype=torch.float32)
    for t in range(T):
        for d in range(ep):
            r = int(slot[t, d])
            if r < 0:
                continue
            send[r] = x[t]
            mine = dest[t] == d
            mid[r] = torch.where(mine, idl[t], -1).to(torch.int32)
            mw[r] = torch.where(mine, w[t].float(), 0.0)
    meta = torch.cat([mid.view(torch.float32), mw], 1)
    return send, meta, slot.to(torch.int32)


def ep_combine(back, slot):
    """out[t] = sum of back[slot[t, d]] over the ranks d token t was sent to (f32 sum)."""
    T, ep = slot.shape
    if T == 0:
        return back.new_zeros(0, back.shape[1])
    ext = torch.cat([back.float(), back.new_zeros(1, back.shape[1]).float()])
    idx = torch.where(slot >= 0, slot.long(), back.shape[0])
    return ext.index_select(0, idx.view(-1)).view(T, ep, -1).sum(1).to(back.dtype)


# ---------------------------------------------------------------------------------------
# Heterogeneous-stack mechanisms: offset-weight norms over parallel residual streams
# (hyper-connections), partial interleaved rotary, windowed attention with kept first tokens
# and a sink logit, gated linear attention with a per-sequence recurrent state, sigmoid-scored
# MoE with clamped GLU experts. Caches of these mixers: K [blocks, G, BS, D], V [blocks, G, Dv, BS]
# (V transposed), recurrent state [slots, H, D, Dv] f32.
# ---------------------------------------------------------------------------------------
def xielu(y, a_pos: float, a_neg: float):
    """z > 0: a_pos z^2 + z / 2;  z <= 0: a_neg (exp(z) - 1 - z) + z / 2."""
    return torch.where(y > 0, a_pos * y * y + 0.5 * y, a_neg * (torch.expm1(y) - y) + 0.5 * y)


def linear_act(x, w, bias=None, act="none", out_dtype=None, act_params=None):
    """y = act(x w^T + bias), f32 accumulation; act: none | relu2 (relu squared) | xielu (the two
    coefficients in act_params)."""
    y = x.float() @ w.float().t()
    if bias is not None:
        y = y + bias.float()
    if act == "relu2":
        y = torch.relu(y).square()
    elif act == "xielu":
        y = xielu(y, float(act_params[0]), float(act_params[1]))
    elif act != "none":
        raise ValueError(act)
    return y.to(out_dtype or x.dtype)


def _rms_offset(x, w, eps, offset):
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * (w.float() + offset)


def embed_norm_streams(ids, table, norm_w, eps, offset, streams):
    x = _rms_offset(table[ids.long()].float(), norm_w, eps, offset)
    return x.unsqueeze(1).repeat(1, streams, 1).contiguous()


def hc_pre(xs, w_in, norm_w, eps, offset, out_dtype):
    u = torch.einsum("s,tsw->tw", w_in.float(), xs)
    return _rms_offset(u, norm_w, eps, offset).to(out_dtype)


def hc_post_(xs, y, mix, w_out):
    new = torch.einsum("sr,tsw->trw", mix.float(), xs) + w_out.float()[None, :, None] * y.float()[:, None, :]
    xs.copy_(new)
    return xs


def hc_final(xs, norm_w, eps, offset, idx, out_dtype):
    x = xs.sum(1) if idx is None else xs[idx.long()].sum(1)
    return _rms_offset(x, norm_w, eps, offset).to(out_dtype)


def rope_partial_kv(q, k, v, positions, inv_freq, slots, k_cache, v_cache):
    """Rotate the first 2 * len(inv_freq) dims of every q / k head in place (pairs (2i, 2i+1),
    angle position * inv_freq[i], f32) and append k, v rows to their cache slots."""
    n = inv_freq.numel()
    a = positions.float()[:, None] * inv_freq.float()[None]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    for t in (q, k):
        if t is None or n == 0:
            continue
        tf = t.float()
        u, w = tf[..., 0:2 * n:2], tf[..., 1:2 * n:2]
        r = torch.stack([u * c - w * s, w * c + u * s], -1).flatten(-2)
        t[..., :2 * n] = r.to(t.dtype)
    if k is not None and slots is not None:
        bs = k_cache.shape[2]
        ok = slots >= 0
        sl = slots[ok].long()
        k_cache[sl // bs, :, sl % bs] = k[ok].to(k_cache.dtype)
        v_cache[sl // bs, :, :, sl % bs] = v[ok].to(v_cache.dtype)
    return q


def attn_window_paged(q, k_cache, v_cache, tables, row_cu, positions, scale, window, keep_first, sink, out=None,
                      out_scale=None, chunk=0, softcap=0.0, dist_bias=None, q_temp=None, maps=1, out_dtype=None):
    """Row r of sequence s (rows row_cu[s] .. row_cu[s+1]) at position p attends to the cached
    keys j <= p of tables[s] with p - j < window or j < keep_first; the softmax denominator
    also holds exp(sink[h]) (sink None: an ordinary softmax). out_scale [T, H] f32: every head's
    output is multiplied by its entry (an output gate). chunk > 0: instead of the window, the
    keys of the row's own chunk of `chunk` positions (j >= p - p % chunk). q_temp (coef, every):
    the score is multiplied by 1 + coef ln(floor((p + 1) / every) + 1); softcap > 0: s <- cap
    tanh(s / cap); dist_bias (a, b) [H] f32: s <- s - a[h] ln(1 + b[h] (p - j)), or with b None the
    linear form s <- s - a[h] (p - j), in that order.
    maps > 1: the key cache holds `maps` key heads per value head, and query head h reads key
    head ((h / maps) / R) * maps + h % maps (R query-head groups per value head) and its value
    head."""
    T, H, D = q.shape
    Gk, bs, Dv = k_cache.shape[1], k_cache.shape[2], v_cache.shape[2]
    G = v_cache.shape[1]
    R = (H // maps) // G
    o = torch.zeros(T, H, Dv, dtype=torch.float32, device=q.device)
    cu = row_cu.tolist()
    pos = positions.tolist()
    for s in range(len(cu) - 1):
        if cu[s + 1] == cu[s]:
            continue
        pmax = max(pos[cu[s]:cu[s + 1]])
        nb = pmax // bs + 1
        blk = tables[s, :nb].long()
        K = k_cache[blk].float().permute(1, 0, 2, 3).reshape(Gk, nb * bs, D)
        V = v_cache[blk].float().permute(1, 0, 3, 2).reshape(G, nb * bs, Dv)
        j = torch.arange(nb * bs, device=q.device)[None, :]
        p = positions[cu[s]:cu[s + 1]].long()[:, None]
        ok = (j <= p) & ((p - j < window) | (j < keep_first))
        if chunk > 0:
            ok = (j <= p) & ((j >= p - p % chunk) | (j < keep_first))
        qs = q[cu[s]:cu[s + 1]].float()
        rs = torch.full_like(p, scale, dtype=torch.float32)
        if q_temp is not None:
            rs = rs * (1.0 + q_temp[0] * torch.log(torch.floor((p + 1).float() / q_temp[1]) + 1.0))
        for h in range(H):
            gk = ((h // maps) // R) * maps + h % maps
            g = gk // maps
            sc = (qs[:, h] @ K[gk].t()) * rs
            if softcap > 0:
                sc = softcap * torch.tanh(sc / softcap)
            if dist_bias is not None and dist_bias[1] is None:
                sc = sc - dist_bias[0][h].float() * (p - j).clamp(min=0).float()
            elif dist_bias is not None:
                sc = sc - dist_bias[0][h].float() * torch.log1p(dist_bias[1][h].float() * (p - j).clamp(min=0).float())
            sc = sc.masked_fill(~ok, float("-inf"))
            if sink is None:
                w = torch.softmax(sc, -1)
            else:
                sk = sink[h].float().expand(sc.shape[0], 1)
                w = torch.softmax(torch.cat([sc, sk], 1), -1)[:, :-1]
            o[cu[s]:cu[s + 1], h] = w @ V[g]
    if out_scale is not None:
        o = o * out_scale.float()[:, :, None]
    o = o.to(out_dtype or q.dtype)
    if out is None:
        return o
    out.copy_(o)
    return out


def gla_scan(q, k, v, z, state, state_slots, row_cu, positions, tau, q_scale):
    """Gated linear attention over packed rows: per sequence and head S <- diag(a_t) S + k_t v_t^T,
    o_t = S^T (q_t * q_scale), a_t = sigmoid(z_t)^(1/tau), all f32. The state of sequence s is
    read from state[state_slots[s]] unless its first row is at position 0 (then zero), and
    written back after its last row. Returns o [T, H, Dv] f32."""
    T, H, D = q.shape
    Dv = v.shape[2]
    o = torch.zeros(T, H, Dv, dtype=torch.float32, device=q.device)
    la = F.logsigmoid(z.float().view(T, H, D)) / tau
    a = torch.exp(la)
    cu, pos, sl = row_cu.tolist(), positions.tolist(), state_slots.tolist()
    qf, kf, vf = q.float() * q_scale, k.float(), v.float()
    for s in range(len(cu) - 1):
        if cu[s + 1] == cu[s] or sl[s] < 0:
            continue
        S = torch.zeros(H, D, Dv, dtype=torch.float32, device=q.device) if pos[cu[s]] == 0 else state[sl[s]].clone()
        for t in range(cu[s], cu[s + 1]):
            S = a[t][:, :, None] * S + kf[t][:, :, None] * vf[t][:, None, :]
            o[t] = torch.einsum("hd,hdv->hv", qf[t], S)
        state[sl[s]] = S
    return o


def gla_out(o, g, norm_w, eps, out_dtype):
    """Per-head RMS norm of o [T, H, Dv] (weight [Dv] shared by the heads) times silu(g)."""
    T, H, Dv = o.shape
    y = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()
    return (y.reshape(T, H * Dv) * F.silu(g.float())).to(out_dtype)


def moe_route_scores(x, wr, top_k, scoring="softmax", renorm=True, bias=None, select_bias=None):
    """Router in f32. scoring "softmax" | "sigmoid"; the top_k largest scores are chosen (ties:
    lowest expert id); `renorm`: the chosen scores are divided by their sum (with "softmax" that
    is the softmax over the chosen logits alone). `bias` [E] f32 is added to the logits;
    `select_bias` [E] f32 is added to the scores for the choice only (the weights are the plain
    scores of the chosen experts)."""
    logits = x.float() @ wr.float().t()
    if bias is not None:
        logits = logits + bias.float()
    sc = torch.softmax(logits, -1) if scoring == "softmax" else torch.sigmoid(logits)
    if select_bias is not None:
        ids = torch.topk(sc + select_bias.float(), top_k, -1).indices
        w = torch.gather(sc, 1, ids)
    else:
        w, ids = torch.topk(sc, top_k, -1)
    if renorm:
        w = w / w.sum(-1, keepdim=True)
    return ids.to(torch.int32), w.contiguous()


def moe_glu_ffn(x, topk_ids, topk_w, gate_up_w, down_w, limit, alpha, out_dtype=None, up_offset=1.0,
                scale_input=True, plain_act=None):
    """Routed GLU experts: g = min(Wg h, limit), u = clamp(Wu h, -limit, limit),
    y = g sigmoid(alpha g) (u + up_offset), output Wd y (limit inf, alpha 1, up_offset 0: the plain
    silu GLU). scale_input: the expert runs on h = w * x and a token's expert outputs are summed;
    otherwise it runs on x and the sum is weighted by w (f32). gate_up_w [E, 2F, H] (gate rows,
    then up rows), down_w [E, H, F]. plain_act "relu2": experts without a gate, y = relu(Wu h)^2
    with gate_up_w [E, F, H]."""
    T, H = x.shape
    Fd = down_w.shape[2]
    out = torch.zeros(T, H, dtype=torch.float32, device=x.device)
    for j in range(topk_ids.shape[1]):
        for e in topk_ids[:, j].unique().tolist():
            if e < 0:
                continue
            tok = (topk_ids[:, j] == e).nonzero().flatten()
            wj = topk_w[tok, j:j + 1].float()
            h = (x[tok].float() * wj).to(x.dtype).float() if scale_input else x[tok].float()
            gu = h @ gate_up_w[e].float().t()
            if plain_act is not None:
                assert plain_act == "relu2"
                y = torch.relu(gu).pow(2).to(x.dtype).float()
            else:
                g = gu[:, :Fd].clamp(max=limit)
                u = gu[:, Fd:].clamp(-limit, limit)
                y = (g * torch.sigmoid(alpha * g) * (u + up_offset)).to(x.dtype).float()
            yd = y @ down_w[e].float().t()
            out[tok] += yd if scale_input else wj * yd
    return out.to(out_dtype or x.dtype)


# ---------------------------------------------------------------------------------------
# Post-norm residual stacks with latent attention: scaled embedding, causal per-channel
# convolution on a mixer's input (its last taps - 1 inputs pooled per sequence), layer norm on a
# sublayer's output with a per-channel scale before the residual sum, a learned average over the
# outputs of all earlier layers, latents / shared rotated key for an attention that caches only
# those, per-head batched projections.
# ---------------------------------------------------------------------------------------
def embed_scaled(ids, table, scale, out=None):
    """out[t] = table[ids[t]] * scale in f32."""
    x = table[ids.long()].float() * scale
    if out is None:
        return x
    out.copy_(x)
    return out


def conv_mix(x, w, state, state_slots, row_cu, positions, out_dtype):
    """h_t = x_t + sum_j w[:, j] x_(t - taps + 1 + j) per channel, over time inside a sequence.
    x [T, W] f32 packed rows; w [W, taps] f32; inputs before the step's first row of a sequence
    come from state[slot] ([taps - 1, W] f32, oldest first) and are zero before position 0."""
    T, W = x.shape
    taps = w.shape[1]
    h = x.clone()
    cu, pos = row_cu.tolist(), positions.tolist()
    sl = state_slots.tolist() if state_slots is not None else [0] * (len(cu) - 1)
    for s in range(len(cu) - 1):
        a, b = cu[s], cu[s + 1]
        if b <= a:
            continue
        p0 = pos[a]
        hist = state[sl[s]].clone() if (taps > 1 and sl[s] >= 0) else x.new_zeros(max(taps - 1, 0), W)
        for d in range(1, taps):           # hist[taps - 1 - d] is the input d steps before row a
            if p0 - d < 0:
                hist[taps - 1 - d] = 0
        ext = torch.cat([hist, x[a:b]], 0)
        for j in range(taps):
            h[a:b] += w[:, j].float() * ext[j:j + (b - a)]
    return h.to(out_dtype)


def conv_state_update_(x, state, state_slots, row_cu, positions):
    """After a step: state[slot] holds the sequence's last taps - 1 inputs (oldest first)."""
    n = state.shape[1]
    if n == 0:
        return state
    cu, pos, sl = row_cu.tolist(), positions.tolist(), state_slots.tolist()
    for s in range(len(cu) - 1):
        a, b = cu[s], cu[s + 1]
        if b <= a or sl[s] < 0:
            continue
        old = state[sl[s]].clone()
        for d in range(1, n + 1):
            if pos[a] - d < 0:
                old[n - d] = 0
        state[sl[s]] = torch.cat([old, x[a:b]], 0)[-n:]
    return state


def _layer_norm_f32(y, w, b, eps):
    y = y.float()
    m = y.mean(-1, keepdim=True)
    v = (y - m).pow(2).mean(-1, keepdim=True)
    return (y - m) * torch.rsqrt(v + eps) * w.float() + b.float()


def post_norm_add(x, y, norm_w, norm_b, eps, scale, out, cast_dtype=None):
    """out = x + scale * layer_norm(y) (f32; out may be x); returns out rounded to cast_dtype
    (None: nothing)."""
    out.copy_(x + scale.float() * _layer_norm_f32(y, norm_w, norm_b, eps))
    return None if cast_dtype is None else out.to(cast_dtype)


def post_norm_add_avg(x, y, norm_w, norm_b, eps, scale, stack, index, avg_w):
    """X = x + scale * layer_norm(y) (y None: X = x); stack[index] = X; x <- sum_j avg_w[j]
    stack[j], j <= index. stack [n, T, W] f32, avg_w [index + 1] f32."""
    X = x if y is None else x + scale.float() * _layer_norm_f32(y, norm_w, norm_b, eps)
    stack[index] = X
    x.copy_(torch.einsum("j,jtw->tw", avg_w.float(), stack[:index + 1]))
    return x


def latent_prep(z, q_rank, kv_rank, rot_dim, heads, qn_w, kvn_w, eps, positions, inv_freq, slots, k_cache, v_cache,
                out_dtype):
    """z [T, >= q_rank + kv_rank + rot_dim + heads] holds per row [query latent | key/value latent
    | shared rotated key part | gate logits] (q_rank 0: no query latent, heads 0: no gates; the
    result is None in its place). Returns (RMS-normed query latent [T, q_rank]
    out_dtype, sigmoid(gate logits) [T, heads] f32) and appends [normed latent | rotated key part]
    to K [blocks, 1, BS, kv_rank + rot_dim] and the normed latent to V [blocks, 1, kv_rank, BS]."""
    zf = z.float()
    o1, o2, o3 = q_rank, q_rank + kv_rank, q_rank + kv_rank + rot_dim
    rms = lambda u, w: u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * w.float()  # noqa: E731
    cq = rms(zf[:, :o1], qn_w).to(out_dtype) if q_rank else None
    c = rms(zf[:, o1:o2], kvn_w)
    kr = zf[:, o2:o3]
    n = inv_freq.numel()
    if n:
        a = positions.float()[:, None] * inv_freq.float()[None]
        cs, sn = torch.cos(a), torch.sin(a)
        u, w = kr[:, 0:2 * n:2], kr[:, 1:2 * n:2]
        kr = torch.cat([torch.stack([u * cs - w * sn, w * cs + u * sn], -1).flatten(-2), kr[:, 2 * n:]], 1)
    gate = torch.sigmoid(zf[:, o3:o3 + heads]).contiguous() if heads else None
    bs = k_cache.shape[2]
    ok = slots >= 0
    sl = slots[ok].long()
    k_cache[sl // bs, 0, sl % bs] = torch.cat([c, kr], 1)[ok].to(k_cache.dtype)
    v_cache[sl // bs, 0, :, sl % bs] = c[ok].to(v_cache.dtype)
    return cq, gate


def linear_heads(x, w, out):
    """out[t, h] = w[h] x[t, h] for every head: x [T, H, K] (a view), w [H, N, K], out [T, H, N]
    (a view), f32 accumulation."""
    out.copy_(torch.einsum("thk,hnk->thn", x.float(), w.float()).to(out.dtype))
    return out


def rope_heads_copy(src, dst, positions, inv_freq):
    """dst[t, h, :n] = src[t, h] with pairs (2i, 2i + 1), i < len(inv_freq), rotated by
    positions[t] * inv_freq[i] (f32); src [T, H, n], dst [T, H, >= n] views (the tail is zeroed)."""
    n = inv_freq.numel()
    a = positions.float()[:, None] * inv_freq.float()[None]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    sf = src.float()
    u, w = sf[..., 0:2 * n:2], sf[..., 1:2 * n:2]
    r = torch.cat([torch.stack([u * c - w * s, w * c + u * s], -1).flatten(-2), sf[..., 2 * n:]], -1)
    dst[..., :src.shape[-1]] = r.to(dst.dtype)
    dst[..., src.shape[-1]:] = 0
    return dst


def layer_norm_rows(x, w, b, eps, idx, out_dtype):
    """Layer norm (weight and bias, f32) of rows idx of x (None: all rows)."""
    xs = x if idx is None else x[idx.long()]
    return _layer_norm_f32(xs, w, b, eps).to(out_dtype)


# ---------------------------------------------------------------------------------------
# Parallel layers with a token shift; differential attention; dense clamped GLU
# ---------------------------------------------------------------------------------------
def par_norm_shift(x, ya, yb, norm_a, norm_b, eps, offset, shift, state, state_slots, row_cu, positions, out_dtype,
                   x_out=None):
    """x' = x + (ya + yb) (f32; either may be None), n = x' / rms(x'), ha = n (norm_a + offset) mixed
    with the previous token's unmixed ha (ha + (prev - ha) shift; zeros before position 0; for a
    sequence's first row of the step: state[slot]), hb = n (norm_b + offset). state[slot] <- the
    unmixed ha of the sequence's last row. Returns (x', ha, hb); hb None without norm_b."""
    xn = x.float()
    if ya is not None or yb is not None:
        y = (ya.float() if ya is not None else 0) + (yb.float() if yb is not None else 0)
        xn = xn + y
    if x_out is not None and xn is not x:
        x_out.copy_(xn)
        xn = x_out
    n = xn * torch.rsqrt(xn.pow(2).mean(-1, keepdim=True) + eps)
    ha = n * (norm_a.float() + offset)
    hb = None if norm_b is None else (n * (norm_b.float() + offset)).to(out_dtype)
    if shift is not None:
        prev = torch.zeros_like(ha)
        prev[1:] = ha[:-1]
        cu, pos = row_cu.tolist(), positions.tolist()
        sl = state_slots.tolist()
        for s in range(len(cu) - 1):
            a, b = cu[s], cu[s + 1]
            if b <= a:
                continue
            if pos[a] > 0 and sl[s] >= 0:
                prev[a] = state[sl[s]]
            else:
                prev[a] = 0
            if sl[s] >= 0:
                state[sl[s]] = ha[b - 1]
        ha = ha + (prev - ha) * shift.float()
    return xn, ha.to(out_dtype), hb


def par_final(x, ya, yb, norm_w, eps, offset, idx, out_dtype):
    """RMS norm with weight (w + offset) of rows idx (None: all) of x + (ya + yb)."""
    sel = (lambda t: t) if idx is None else (lambda t: t[idx.long()])
    xn = sel(x).float()
    if ya is not None or yb is not None:
        xn = xn + ((sel(ya).float() if ya is not None else 0) + (sel(yb).float() if yb is not None else 0))
    return _rms_offset(xn, norm_w, eps, offset).to(out_dtype)


def qk_norm_rope_kv(q, k, v, qn_w, kn_w, eps, positions, inv_freq, slots, k_cache, v_cache, q_out):
    """Per head: RMS norm over the head with weight qn_w / kn_w [D] (None: no norm), then rotation
    of the first 2 n dims (n = len(inv_freq)) with dimension i paired with i + n, angle position *
    inv_freq[i] (f32). q [T, Hq, D] -> q_out [T, Hq, >= D] (zero padded); k [T, Gk, D], v [T, Gv,
    Dv] -> cache rows K [blocks, Gk, BS, >= D], V [blocks, Gv, >= Dv, BS] at slots[t] >= 0."""
    n = inv_freq.numel()
    a = positions.double()[:, None] * inv_freq.double()[None]       # the f32 frequencies, f64 product and evaluation
    c, s = torch.cos(a).float()[:, None, :], torch.sin(a).float()[:, None, :]

    def prep(t, w):
        tf = t.float()
        if w is not None:
            tf = tf * torch.rsqrt(tf.pow(2).mean(-1, keepdim=True) + eps) * w.float()
        if n:
            u, z = tf[..., :n], tf[..., n:2 * n]
            tf = torch.cat([u * c - z * s, z * c + u * s, tf[..., 2 * n:]], -1)
        return tf

    D, Dv = q.shape[2], v.shape[2]
    q_out.zero_()
    q_out[..., :D] = prep(q, qn_w).to(q_out.dtype)
    kk = prep(k, kn_w)
    bs = k_cache.shape[2]
    ok = slots >= 0
    sl = slots[ok].long()
    k_cache[sl // bs, :, sl % bs, :D] = kk[ok].to(k_cache.dtype)
    v_cache[sl // bs, :, :Dv, sl % bs] = v[ok].to(v_cache.dtype)
    return q_out


def diff_combine(a, lam, eps, out_mul, gate, Dv, out_dtype):
    """a [T, 2 H, >= Dv] f32, heads ordered (head, map): o = a[:, 2h] - lam a[:, 2h + 1] over the
    first Dv values, divided by its root mean square (eps inside the root), times out_mul, times
    sigmoid(gate) (gate [T, H * Dv] logits, None: no gate). Returns [T, H * Dv]."""
    T, H2 = a.shape[0], a.shape[1]
    af = a.float()[..., :Dv]
    o = af[:, 0::2] - lam * af[:, 1::2]
    o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * out_mul
    o = o.reshape(T, (H2 // 2) * Dv)
    if gate is not None:
        o = o * torch.sigmoid(gate.float())
    return o.to(out_dtype)


def glu_clamp(gu, limit, alpha, up_offset, out_dtype=None, group=0):
    """gu [T, 2 F] = [gate | up] (group > 0: alternating blocks of `group` gate and up columns):
    min(g, limit) sigmoid(alpha min(g, limit)) (clamp(u, +-limit) + up_offset)."""
    g, u = split_gate_up(gu, group)
    g = g.float().clamp(max=limit)
    u = u.float().clamp(min=-limit, max=limit)
    return (g * torch.sigmoid(alpha * g) * (u + up_offset)).to(out_dtype or gu.dtype)


# ---------------------------------------------------------------------------------------
# Sandwich-norm residual stacks with a gated delta rule: layer norms before and after every
# sublayer, short causal convolutions with an activation on projected rows, the delta-rule
# recurrence with pooled per-sequence state.
# ---------------------------------------------------------------------------------------
def post_norm_add_norm(x, y, norm_w, norm_b, eps, mult, extra, norm2_w, norm2_b, out_dtype):
    """x <- x + mult * layer_norm(y; norm_w, norm_b) (+ extra), in place, f32; returns layer_norm(x;
    norm2_w, norm2_b) in out_dtype, the next sublayer's input (norm2_w None: nothing)."""
    v = x + mult * _layer_norm_f32(y, norm_w, norm_b, eps)
    if extra is not None:
        v = v + extra.float()
    x.copy_(v)
    return None if norm2_w is None else _layer_norm_f32(x, norm2_w, norm2_b, eps).to(out_dtype)


def short_conv_act(z, w, state, state_slots, row_cu, positions, act, out_dtype):
    """y_t = act(sum_j w[:, j] z_(t - taps + 1 + j)) per channel over the rows of each sequence of a
    packed step. z [T, C] (a view of projected rows, any element type); w [C, taps] f32, the last
    column the current row's; rows before the step's first come from state[slot] ([slots, taps - 1,
    C] f32, oldest first) and are zero before position 0. act "none" | "silu". The state is not changed."""
    T, C = z.shape
    taps = w.shape[1]
    zf = z.float()
    y = torch.zeros(T, C, dtype=torch.float32, device=z.device)
    cu, pos = row_cu.tolist(), positions.tolist()
    sl = state_slots.tolist() if state_slots is not None else [-1] * (len(cu) - 1)
    for s in range(len(cu) - 1):
        a, b = cu[s], cu[s + 1]
        if b <= a:
            continue
        p0 = pos[a]
        hist = state[sl[s]].clone() if (taps > 1 and sl[s] >= 0) else zf.new_zeros(max(taps - 1, 0), C)
        for d in range(1, taps):           # hist[taps - 1 - d] is the input d steps before row a
            if p0 - d < 0:
                hist[taps - 1 - d] = 0
        ext = torch.cat([hist, zf[a:b]], 0)
        for j in range(taps):
            y[a:b] += w[:, j].float() * ext[j:j + (b - a)]
    if act == "silu":
        y = F.silu(y)
    return y.to(out_dtype)


def short_conv_state_update_(z, state, state_slots, row_cu, positions):
    """After a step: state[slot] holds the last taps - 1 rows of z of every sequence (oldest first)."""
    return conv_state_update_(z.float(), state, state_slots, row_cu, positions)


def delta_scan(q, k, v, b, a, a_log, dt_bias, state, state_slots, row_cu, positions, q_scale, unit_eps):
    """Gated delta rule over packed rows, all f32. q, k [T, G, D] and v [T, H, Dv] (head h reads
    query / key group h // (H / G)); q and k are first made unit vectors, x / sqrt(sum x^2 +
    unit_eps), and q is multiplied by q_scale. Per row and head: beta = sigmoid(b), decay =
    exp(-exp(a_log[h]) softplus(a + dt_bias[h])); S <- decay S; u = beta (v - S^T k); S <- S + k u^T;
    o = S^T q. The state S [D, Dv] of sequence s is read from state[state_slots[s]] (stored column by
    column, [H, Dv, D]) unless its first row is at position 0 (then zero) and written back after its
    last row. Returns o [T, H, Dv] f32."""
    T, G, D = q.shape
    H, Dv = v.shape[1], v.shape[2]
    rep = H // G
    qf, kf, vf = q.float(), k.float(), v.float()
    qf = qf * torch.rsqrt(qf.pow(2).sum(-1, keepdim=True) + unit_eps) * q_scale
    kf = kf * torch.rsqrt(kf.pow(2).sum(-1, keepdim=True) + unit_eps)
    qf, kf = qf.repeat_interleave(rep, 1), kf.repeat_interleave(rep, 1)
    beta = torch.sigmoid(b.float())
    decay = torch.exp(-torch.exp(a_log.float()) * F.softplus(a.float() + dt_bias.float()))
    o = torch.zeros(T, H, Dv, dtype=torch.float32, device=q.device)
    cu, pos, sl = row_cu.tolist(), positions.tolist(), state_slots.tolist()
    for s in range(len(cu) - 1):
        if cu[s + 1] == cu[s] or sl[s] < 0:
            continue
        S = torch.zeros(H, D, Dv, dtype=torch.float32, device=q.device) if pos[cu[s]] == 0 \
            else state[sl[s]].transpose(1, 2).clone()
        for t in range(cu[s], cu[s + 1]):
            S = decay[t][:, None, None] * S
            u = beta[t][:, None] * (vf[t] - torch.einsum("hdv,hd->hv", S, kf[t]))
            S = S + kf[t][:, :, None] * u[:, None, :]
            o[t] = torch.einsum("hdv,hd->hv", S, qf[t])
        state[sl[s]] = S.transpose(1, 2)
    return o
