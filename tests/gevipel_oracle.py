"""A plain, slow float64 implementation of the Gevipel design, one function per mechanism, written
from the design's equations and sharing no code with the package: whole sequences at once, dense
score matrices, explicit masks, explicit token loops, no cache. Tests build configurations and
random weights here."""
import math

import torch

F64 = torch.float64


# ---- configuration builders ----------------------------------------------------------------
def moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def window_layer(heads, kv_heads, dim, scale, window, coef, every, mlp):
    """Sliding-window softmax attention whose values are the un-normed keys."""
    return {"type": "attention", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale,
                      "mask": {"size": window}, "q_temp": {"coef": coef, "every": every}}}


def delta_layer(heads, kv_heads, dim, vdim, taps, mlp):
    """Gated delta rule with short convolutions."""
    return {"type": "delta", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": taps}}


def latent_layer(heads, dim, rot_dim, vdim, kv_rank, scale, base, mlp):
    """Causal attention over a cached latent with a per-head sink."""
    return {"type": "latent_attention", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
                      "rot": {"base": base, "dims": rot_dim}}}


def config(layers, width, vocab, eps, embed_scale, residual_mult, loop=None):
    c = {"architecture": "Gevipel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers,
         "embedding": {"scale": embed_scale}, "residual_mult": residual_mult}
    if loop is not None:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


def random_weights(cfg, seed):
    """name -> bf16 tensor (router corrections too), under the names a model folder uses."""
    g = torch.Generator().manual_seed(seed)
    W, out = cfg["width"], {}

    def mat(name, rows, cols, std=None):
        out[name] = (torch.randn(rows, cols, generator=g) * (std or 1.0 / math.sqrt(cols))).to(torch.bfloat16)

    def vec(name, n, mean, std):
        out[name] = (mean + std * torch.randn(n, generator=g)).to(torch.bfloat16)

    mat("embed", cfg["vocab"], W, 1.0 / max(cfg["embedding"]["scale"], 1e-6))
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        for n in ("norm1", "norm1b") + (("norm2", "norm2b") if L["mlp"] else ()):
            vec(p + n, W, 1.0, 0.2)
            vec(p + n + ".b", W, 0.0, 0.2)
        H, D, Dv = m["heads"], m["dim"], m["vdim"]
        if L["type"] == "attention":
            G = m["kv_heads"]
            mat(p + "mix.q", H * D, W)
            mat(p + "mix.k", G * D, W)
            vec(p + "mix.q.norm", D, 1.0, 0.2)
            vec(p + "mix.k.norm", D, 1.0, 0.2)
            mat(p + "mix.o", W, H * D)
        elif L["type"] == "delta":
            G, taps = m["kv_heads"], m["conv"]
            for n, rows in (("q", G * D), ("k", G * D), ("v", H * Dv)):
                mat(p + "mix." + n, rows, W)
                mat(p + "mix." + n + ".conv", rows, taps, 0.5)
            mat(p + "mix.b", H, W)
            mat(p + "mix.a", H, W)
            vec(p + "mix.A_log", H, -1.0, 0.7)
            vec(p + "mix.dt_bias", H, 0.0, 1.0)
            vec(p + "mix.norm", Dv, 1.0, 0.2)
            mat(p + "mix.g", H * Dv, W)
            mat(p + "mix.o", W, H * Dv)
        else:
            R, rd = m["kv_rank"], m["rot_dim"]
            mat(p + "mix.q", H * (D + rd), W)
            mat(p + "mix.dkv", R + rd, W)
            vec(p + "mix.dkv.norm", R, 1.0, 0.2)
            mat(p + "mix.uk", H * D, R)
            mat(p + "mix.uv", H * Dv, R)
            vec(p + "mix.sink", H, 0.0, 1.0)
            mat(p + "mix.o", W, H * Dv)
        f = L["mlp"]
        if f:
            E, F = f["router"]["experts"], f["expert"]["ff"]
            mat(p + "mlp.router", E, W)
            vec(p + "mlp.correction", E, 0.0, 0.05)
            for e in range(E):
                mat(p + f"mlp.e{e}.up", F, W)
                mat(p + f"mlp.e{e}.down", W, F)
    vec("final.norm", W, 1.0, 0.2)
    vec("final.norm.b", W, 0.0, 0.2)
    mat("head", cfg["vocab"], W)
    return out


# ---- mechanisms ------------------------------------------------------------------------------
def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def silu(x):
    return x * torch.sigmoid(x)


def short_conv(x, taps_w):
    """x [T, C], taps_w [C, taps]: y_t = sum_j taps_w[:, j] x_(t - taps + 1 + j), zeros before the start."""
    T, C = x.shape
    n = taps_w.shape[1]
    y = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for j in range(n):
            s = t - (n - 1) + j
            if s >= 0:
                y[t] += taps_w[:, j] * x[s]
    return y


def delta_rule(q, k, v, beta, decay):
    """q, k [T, H, D], v [T, H, Dv], beta, decay [T, H] -> o [T, H, Dv]; one state matrix per head."""
    T, H, D = q.shape
    Dv = v.shape[2]
    o = torch.zeros(T, H, Dv, dtype=F64)
    for h in range(H):
        S = torch.zeros(D, Dv, dtype=F64)
        for t in range(T):
            S = decay[t, h] * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, h])
            S = S + torch.outer(k[t, h], u)
            o[t, h] = S.T @ q[t, h]
    return o


def delta_mixer(h, m, w, p, eps):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ w[p + "q"].T, w[p + "q.conv"])).view(T, G, D)
    k = silu(short_conv(h @ w[p + "k"].T, w[p + "k.conv"])).view(T, G, D)
    v = silu(short_conv(h @ w[p + "v"].T, w[p + "v.conv"])).view(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    rep = H // G
    q, k = q.repeat_interleave(rep, 1), k.repeat_interleave(rep, 1)      # head h reads group h // rep
    beta = torch.sigmoid(h @ w[p + "b"].T)
    decay = torch.exp(-torch.exp(w[p + "A_log"]) * torch.nn.functional.softplus(h @ w[p + "a"].T + w[p + "dt_bias"]))
    o = delta_rule(q, k, v, beta, decay)
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * w[p + "norm"]
    o = o * silu(h @ w[p + "g"].T).view(T, H, Dv)
    return o.reshape(T, H * Dv) @ w[p + "o"].T


def sloped_window_softmax(q, k, v, scale, window, q_temp):
    """q [T, H, D], k, v [T, G, D]: softmax attention of position i over the keys j with 0 <= i - j < window
    (None: all j <= i); the score of head h loses 2^(-8 (h + 1) / H) (i - j); q_temp (coef, every) or None
    multiplies the queries of position p by 1 + coef ln(floor((p + 1) / every) + 1)."""
    T, H, D = q.shape
    G = k.shape[1]
    pos = torch.arange(T)
    if q_temp:
        temp = 1.0 + q_temp[0] * torch.log(torch.floor((pos + 1).to(F64) / q_temp[1]) + 1.0)
        q = q * temp[:, None, None]
    dist = pos[:, None] - pos[None, :]
    seen = (dist >= 0) & ((dist < window) if window is not None else True)
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        slope = 2.0 ** (-8.0 * (hh + 1) / H)
        s = (q[:, hh] @ k[:, g].T) * scale - slope * dist.to(F64)
        s = s.masked_fill(~seen, -math.inf)
        out[:, hh] = torch.softmax(s, -1) @ v[:, g]
    return out


def window_attention(h, m, w, p, eps):
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ w[p + "q"].T).view(T, H, D)
    kraw = (h @ w[p + "k"].T).view(T, G, D)
    q = rms_norm(q, w[p + "q.norm"], eps)
    k = rms_norm(kraw, w[p + "k.norm"], eps)
    qt = m.get("q_temp")
    size = m["mask"]["size"] if m.get("mask") else None
    # the values are the keys as projected, before their norm
    out = sloped_window_softmax(q, k, kraw, m["scale"], size, (qt["coef"], qt["every"]) if qt else None)
    return out.reshape(T, H * D) @ w[p + "o"].T


def rotate_pairs(x, base, dims):
    """x [T, ..., n]: neighbouring pairs (2i, 2i + 1) of the first `dims` dimensions turn by t * base^(-2i / dims)."""
    T = x.shape[0]
    y = x.clone()
    pos = torch.arange(T, dtype=F64)
    for i in range(dims // 2):
        a = pos * base ** (-2.0 * i / dims)
        c, s = torch.cos(a), torch.sin(a)
        shape = (T,) + (1,) * (x.dim() - 2)
        c, s = c.view(shape), s.view(shape)
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        y[..., 2 * i] = u * c - v * s
        y[..., 2 * i + 1] = v * c + u * s
    return y


def causal_sink_softmax(s, sink):
    """Softmax weights of the scores s [T, T] over j <= i; the denominator also holds exp(sink), which
    has no key and no value, is not scaled and counts once."""
    T = s.shape[0]
    pos = torch.arange(T)
    s = s.masked_fill(pos[:, None] < pos[None, :], -math.inf)
    s = torch.cat([s, sink.expand(T, 1)], 1)
    return torch.softmax(s, -1)[:, :T]


def latent_attention(h, m, w, p, eps):
    T = h.shape[0]
    H, D, rd, Dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (h @ w[p + "q"].T).view(T, H, D + rd)
    q_plain, q_rot = q[..., :D], rotate_pairs(q[..., D:], m["rot"]["base"], m["rot"]["dims"])
    z = h @ w[p + "dkv"].T
    c = rms_norm(z[:, :R], w[p + "dkv.norm"], eps)
    k_rot = rotate_pairs(z[:, R:], m["rot"]["base"], m["rot"]["dims"])     # one rotated key part for all heads
    k_plain = (c @ w[p + "uk"].T).view(T, H, D)
    v = (c @ w[p + "uv"].T).view(T, H, Dv)
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hh in range(H):
        s = (q_plain[:, hh] @ k_plain[:, hh].T + q_rot[:, hh] @ k_rot.T) * m["scale"]
        out[:, hh] = causal_sink_softmax(s, w[p + "sink"][hh]) @ v[:, hh]
    return out.reshape(T, H * Dv) @ w[p + "o"].T


def routed_experts(h, f, w, p, choice=None):
    """Softmax scores over all experts; the top experts by (score + correction) weigh in with their
    plain scores. `choice` (a list) collects (score + correction) rows for tests that avoid close calls."""
    E, top = f["router"]["experts"], f["router"]["top"]
    s = torch.softmax(h @ w[p + "router"].T, -1)
    pick = s + w[p + "correction"]
    if choice is not None:
        choice.append(pick)
    idx = pick.topk(top, -1).indices
    y = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in idx[t].tolist():
            a = torch.relu(w[p + f"e{e}.up"] @ h[t]) ** 2
            y[t] += s[t, e] * (w[p + f"e{e}.down"] @ a)
    return y


MIXERS = {"attention": window_attention, "delta": delta_mixer, "latent_attention": latent_attention}


def layer_runs(cfg):
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, False) for i in range(n)]
    runs = [(i, False) for i in range(lp["start"])]
    for r in range(lp["times"]):
        runs += [(i, r > 0 and i == lp["start"]) for i in range(lp["start"], lp["stop"])]
    return runs + [(i, False) for i in range(lp["stop"], n)]


def forward(cfg, weights, tokens, layers_out=None, choice=None):
    """logits [T, vocab] of one sequence; layers_out (a list) collects the residual after every layer run."""
    w = {k: v.to(F64) for k, v in weights.items()}
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x0 = w["embed"][torch.as_tensor(tokens)] * cfg["embedding"]["scale"]
    x = x0
    for i, again in layer_runs(cfg):
        L, p = cfg["layers"][i], f"l{i}."
        if again:                      # a repeated pass starts from the residual plus the embedding output
            x = x + x0
        hin = layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps)
        y = MIXERS[L["type"]](hin, L["mixer"], w, p + "mix.", eps)
        x = x + mult * layer_norm(y, w[p + "norm1b"], w[p + "norm1b.b"], eps)
        if L["mlp"]:
            hin = layer_norm(x, w[p + "norm2"], w[p + "norm2.b"], eps)
            y = routed_experts(hin, L["mlp"], w, p + "mlp.", choice)
            x = x + mult * layer_norm(y, w[p + "norm2b"], w[p + "norm2b.b"], eps)
        if layers_out is not None:
            layers_out.append(x)
    return layer_norm(x, w["final.norm"], w["final.norm.b"], eps) @ w["head"].T


def greedy(cfg, weights, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(cfg, weights, toks)[-1].argmax()))
    return toks[len(prompt):]
