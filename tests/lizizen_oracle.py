"""A plain, slow float64 implementation of the Lizizen design, one function per mechanism, written
from the design's equations and sharing no code with the package: whole sequences at once, dense
score matrices, explicit masks, no cache. Tests build configurations and random weights here."""
import math

import torch

F64 = torch.float64


# ---- configuration builders ----------------------------------------------------------------
def dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def biased_layer(heads, kv_heads, dim, vdim, scale, coef, every, mlp):
    """Softmax attention with a distance bias, a position-dependent query temperature and a sink."""
    return {"type": "attention", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                      "q_temp": {"coef": coef, "every": every}}}


def diff_layer(heads, kv_heads, dim, vdim, scale, diff, chunk, base, rot_dims, softcap, mlp):
    """Differential attention over chunks with normed, rotated queries and keys."""
    return {"type": "attention_2", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff,
                      "mask": {"size": chunk}, "rot": {"base": base, "dims": rot_dims}, "softcap": softcap}}


def config(layers, width, vocab, eps, loop=None):
    c = {"architecture": "Lizizen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if loop is not None:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


def random_weights(cfg, seed):
    """name -> bf16 tensor, under the names a model folder uses."""
    g = torch.Generator().manual_seed(seed)
    W, out = cfg["width"], {}

    def mat(name, rows, cols, std=None):
        out[name] = (torch.randn(rows, cols, generator=g) * (std or 1.0 / math.sqrt(cols))).to(torch.bfloat16)

    def vec(name, n, mean, std):
        out[name] = (mean + std * torch.randn(n, generator=g)).to(torch.bfloat16)

    mat("embed", cfg["vocab"], W, 1.0)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        vec(p + "norm1", W, 0.0, 0.2)
        if L["mlp"]:
            vec(p + "norm2", W, 0.0, 0.2)
        out[p + "shift"] = torch.rand(W, generator=g).to(torch.bfloat16)
        if L["type"] == "attention":
            mat(p + "mix.q", H * D, W)
            mat(p + "mix.k", G * D, W)
            mat(p + "mix.v", G * Dv, W)
            out[p + "mix.r1"] = (0.2 + 0.8 * torch.rand(H, generator=g)).to(torch.bfloat16)
            out[p + "mix.r2"] = (0.05 + 0.5 * torch.rand(H, generator=g)).to(torch.bfloat16)
        else:
            mat(p + "mix.q", H * 2 * D, W)
            mat(p + "mix.k", G * 2 * D, W)
            mat(p + "mix.v", G * Dv, W)
            vec(p + "mix.q.norm", D, 1.0, 0.2)
            vec(p + "mix.k.norm", D, 1.0, 0.2)
            for n in ("lq1", "lk1", "lq2", "lk2"):
                vec(p + "mix." + n, D, 0.0, 0.1)
            mat(p + "mix.g", H * Dv, W)
        mat(p + "mix.o", W, H * Dv)
        f = L["mlp"]
        if f:
            for n, r, c in (("gate", f["ff"], W), ("up", f["ff"], W), ("down", W, f["ff"])):
                mat(p + "mlp." + n, r, c)
                vec(p + "mlp." + n + ".b", r, 0.0, 0.2)
    vec("final.norm", W, 0.0, 0.2)
    mat("head", cfg["vocab"], W)
    return out


# ---- mechanisms ----------------------------------------------------------------------------
def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """RMS norm whose weight is stored around zero."""
    return rms(x, eps) * (1.0 + w.to(F64))


def token_shift(h, s):
    """h_t <- h_t + (h_(t-1) - h_t) s, with the unshifted h_(t-1) (zeros before the first token)."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]])
    return h + (prev - h) * s.to(F64)


def query_temperature(n, coef, every):
    p = torch.arange(n, dtype=F64)
    return 1.0 + coef * torch.log(torch.floor((p + 1) / every) + 1.0)


def distance_bias(n, r1, r2):
    """[H, n, n]: r1_h ln(1 + r2_h (i - j)) for j <= i (0 elsewhere; those places are masked)."""
    i = torch.arange(n, dtype=F64)
    d = (i[:, None] - i[None, :]).clamp(min=0)
    return r1.to(F64)[:, None, None] * torch.log1p(r2.to(F64)[:, None, None] * d)


def causal_mask(n):
    i = torch.arange(n)
    return i[None, :] <= i[:, None]


def chunk_mask(n, size):
    i = torch.arange(n)
    return (i[None, :] <= i[:, None]) & ((i[None, :] // size) == (i[:, None] // size))


def softmax_with_sink(s, mask):
    """p_j = exp(s_j) / (1 + sum exp(s_j)) over the visible keys."""
    s = s.masked_fill(~mask, -math.inf)
    m = s.max(-1, keepdim=True).values.clamp(min=0.0)
    e = torch.exp(s - m)
    return e / (torch.exp(-m) + e.sum(-1, keepdim=True))


def softmax_plain(s, mask):
    return torch.softmax(s.masked_fill(~mask, -math.inf), -1)


def rotate_half(x, base, dims):
    """x [n, heads, D]: the first `dims` dimensions rotate, dimension i paired with i + dims / 2."""
    n = x.shape[0]
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    a = torch.arange(n, dtype=F64)[:, None] * f[None, :]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def biased_attend(q, k, v, r1, r2, scale, coef, every):
    """q [n, H, D], k [n, G, D], v [n, G, Dv] -> [n, H, Dv]: causal softmax attention whose scores
    lose the distance bias, with the query temperature and the sink."""
    n, H = q.shape[0], q.shape[1]
    G = k.shape[1]
    q = q * query_temperature(n, coef, every)[:, None, None]
    bias = distance_bias(n, r1, r2)
    mask = causal_mask(n)
    out = torch.zeros(n, H, v.shape[2], dtype=F64)
    for hq in range(H):
        g = hq // (H // G)
        s = (q[:, hq] @ k[:, g].T) * scale - bias[hq]
        out[:, hq] = softmax_with_sink(s, mask) @ v[:, g]
    return out


def biased_attention(h, w, p, m):
    n = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].to(F64).T).view(n, H, D)
    k = (h @ w[p + "k"].to(F64).T).view(n, G, D)
    v = (h @ w[p + "v"].to(F64).T).view(n, G, Dv)
    qt = m.get("q_temp") or {"coef": 0.0, "every": 1}
    out = biased_attend(q, k, v, w[p + "r1"], w[p + "r2"], m["scale"], qt["coef"], qt["every"])
    return out.reshape(n, H * Dv) @ w[p + "o"].to(F64).T


def diff_lambda(w, p, diff):
    f = lambda a, b: torch.exp((w[p + a].to(F64) * w[p + b].to(F64)).sum())       # noqa: E731
    return float(f("lq1", "lk1") - f("lq2", "lk2") + diff)


def normed_rotated(x, nw, eps, base, dims):
    """x [n, heads, maps, D]: RMS norm per head and map with the shared weight, then the rotation."""
    n, A, M, D = x.shape
    x = rms(x, eps) * nw.to(F64)
    return rotate_half(x.reshape(n, A * M, D), base, dims).view(n, A, M, D) if dims else x


def chunk_attend(q, k, v, scale, cap, size):
    """q [n, H, M, D], k [n, G, M, D], v [n, G, Dv] -> the maps' outputs [n, H, M, Dv]: capped scores,
    keys of the query's own chunk, ordinary softmax."""
    n, H, M = q.shape[0], q.shape[1], q.shape[2]
    G = k.shape[1]
    mask = chunk_mask(n, size)
    out = torch.zeros(n, H, M, v.shape[2], dtype=F64)
    for hq in range(H):
        g = hq // (H // G)
        for mp in range(M):
            s = (q[:, hq, mp] @ k[:, g, mp].T) * scale
            if cap:
                s = cap * torch.tanh(s / cap)
            out[:, hq, mp] = softmax_plain(s, mask) @ v[:, g]
    return out


def combine_maps(a, lam, diff, eps):
    """a [n, H, 2, Dv] -> [n, H, Dv]: a1 - lambda a2, unit RMS per head, times (1 - diff)."""
    return rms(a[:, :, 0] - lam * a[:, :, 1], eps) * (1.0 - diff)


def diff_attention(h, w, p, m, eps):
    n = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot = m.get("rot") or {"base": 1.0, "dims": 0}
    q = normed_rotated((h @ w[p + "q"].to(F64).T).view(n, H, 2, D), w[p + "q.norm"], eps, rot["base"], rot["dims"])
    k = normed_rotated((h @ w[p + "k"].to(F64).T).view(n, G, 2, D), w[p + "k.norm"], eps, rot["base"], rot["dims"])
    v = (h @ w[p + "v"].to(F64).T).view(n, G, Dv)
    a = chunk_attend(q, k, v, m["scale"], m.get("softcap") or 0.0, m["mask"]["size"])
    out = combine_maps(a, diff_lambda(w, p, m["diff"]), m["diff"], eps)
    gate = torch.sigmoid(h @ w[p + "g"].to(F64).T)
    return (out.reshape(n, H * Dv) * gate) @ w[p + "o"].to(F64).T


def glu_ffn(h, w, p, f):
    lim = f["limit"]
    g = (h @ w[p + "gate"].to(F64).T + w[p + "gate.b"].to(F64)).clamp(max=lim)
    u = (h @ w[p + "up"].to(F64).T + w[p + "up.b"].to(F64)).clamp(min=-lim, max=lim)
    y = g * torch.sigmoid(1.702 * g) * (u + 1.0)
    return y @ w[p + "down"].to(F64).T + w[p + "down.b"].to(F64)


def layer_runs(cfg):
    """Layer indices in the order they run (a looped span repeats with the same weights)."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp or lp["times"] <= 1:
        return list(range(n))
    span = list(range(lp["start"], lp["stop"]))
    return list(range(lp["start"])) + span * lp["times"] + list(range(lp["stop"], n))


def layer(x, cfg, w, i):
    L, p, eps = cfg["layers"][i], f"l{i}.", cfg["norm"]["eps"]
    h = token_shift(offset_norm(x, w[p + "norm1"], eps), w[p + "shift"])
    if L["type"] == "attention":
        y = biased_attention(h, w, p + "mix.", L["mixer"])
    else:
        y = diff_attention(h, w, p + "mix.", L["mixer"], eps)
    if L["mlp"]:
        y = y + glu_ffn(offset_norm(x, w[p + "norm2"], eps), w, p + "mlp.", L["mlp"])
    return x + y


def forward(cfg, w, tokens, layers_out=None):
    """Logits [n, vocab] (float64) of one whole sequence; `layers_out` collects the residual after
    every layer run."""
    x = w["embed"].to(F64)[torch.as_tensor(tokens, dtype=torch.long)]
    for i in layer_runs(cfg):
        x = layer(x, cfg, w, i)
        if layers_out is not None:
            layers_out.append(x.clone())
    return offset_norm(x, w["final.norm"], cfg["norm"]["eps"]) @ w["head"].to(F64).T


def greedy(cfg, w, prompt, n):
    """The n tokens greedy decoding appends to the prompt (ties to the lowest id)."""
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(cfg, w, toks)[-1].argmax()))
    return toks[len(prompt):]
