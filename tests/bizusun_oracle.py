"""Plain, slow implementation of the Bizusun design for the tests.

One function per mechanism, written token by token from the design's
equations; whole sequences only (no cache, no state object, no batching).
It shares no code with ``polyrl_amd``: the engine, its state manager and
its kernels are compared against these functions.

Conventions: ``W`` maps tensor names to torch tensors, linear weights are
[out, in] and applied as ``W @ x``; ``cfg`` is the parsed config dict.
Everything runs in ``DT`` (float64 by default) so the oracle's own rounding
is far below any tolerance used against it.
"""
import math

import torch

DT = torch.float64


def _f(t):
    return t.to(DT)


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0)


def gelu_tanh(z):
    c = math.sqrt(2.0 / math.pi)
    return 0.5 * z * (1.0 + torch.tanh(c * (z + 0.044715 * z ** 3)))


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def causal_taps(h, w, bias=None):
    """y_t = sum_j w[:, j] * h_(t - taps + 1 + j), zeros before t = 0.
    h [T, C], w [C, taps]; the last column weighs the current token."""
    T, C = h.shape
    taps = w.shape[1]
    y = torch.zeros(T, C, dtype=DT)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * h[s]
        if bias is not None:
            y[t] += bias
    return y


# ------------------------------------------------------------------ mixers
def general_delta(h, W, p, m, eps):
    """Generalised delta rule with per-channel decay and removal rate."""
    H, D = m["heads"], m["dim"]
    T = h.shape[0]
    out = torch.zeros(T, H * D, dtype=DT)
    S = torch.zeros(H, D, D, dtype=DT)          # [head, key, value]
    for t in range(T):
        x = h[t]
        r = (_f(W[p + "r"]) @ x).view(H, D)
        k = (_f(W[p + "k"]) @ x).view(H, D)
        v = (_f(W[p + "v"]) @ x).view(H, D)
        lo = _f(W[p + "w2"]) @ torch.tanh(_f(W[p + "w1"]) @ x) + _f(W[p + "w0"])
        w = torch.exp(-math.exp(-0.5) * sigmoid(lo)).view(H, D)
        a = sigmoid(_f(W[p + "a"]) @ x + _f(W[p + "a.b"])).view(H, D)
        for hd in range(H):
            u = k[hd] / torch.sqrt((k[hd] ** 2).sum() + 1e-6)
            old = S[hd]
            S[hd] = (w[hd][:, None] * old
                     - torch.outer(a[hd] * u, u @ old)
                     + torch.outer(k[hd], v[hd]))
            o = S[hd].t() @ r[hd]
            out[t, hd * D:(hd + 1) * D] = unit_rms(o, eps)
        out[t] = out[t] * _f(W[p + "norm"]) * sigmoid(_f(W[p + "g"]) @ x)
    return out @ _f(W[p + "o"]).t()


def mamba2(h, W, p, m, eps):
    """Selective state space layer, one scalar decay per head."""
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    T = h.shape[0]
    proj = h @ _f(W[p + "in"]).t()
    z = proj[:, :inner]
    xbc = proj[:, inner:2 * inner + 2 * G * N]
    dt = proj[:, 2 * inner + 2 * G * N:]
    assert dt.shape[1] == H
    xbc = silu(causal_taps(xbc, _f(W[p + "conv"]), _f(W[p + "conv.b"])))
    x = xbc[:, :inner].reshape(T, H, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + _f(W[p + "dt_bias"]))
    A = torch.exp(_f(W[p + "A_log"]))
    Dk = _f(W[p + "D"])
    S = torch.zeros(H, N, P, dtype=DT)
    y = torch.zeros(T, H, P, dtype=DT)
    per = H // G
    for t in range(T):
        for hd in range(H):
            g = hd // per
            S[hd] = torch.exp(-A[hd] * dt[t, hd]) * S[hd] \
                + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S[hd].t() @ C[t, g] + Dk[hd] * x[t, hd]
    y = y.reshape(T, inner) * silu(z)
    ng = m["norm_groups"]
    y = unit_rms(y.reshape(T, ng, inner // ng), eps).reshape(T, inner)
    return (y * _f(W[p + "norm"])) @ _f(W[p + "o"]).t()


def rotate(vec, pos, dims, base):
    """Rotate-half pairs (i, i + dims/2) of the first ``dims`` entries."""
    out = vec.clone()
    half = dims // 2
    for i in range(half):
        ang = pos * base ** (-2.0 * i / dims)
        c, s = math.cos(ang), math.sin(ang)
        a, b = vec[..., i], vec[..., i + half]
        out[..., i] = a * c - b * s
        out[..., i + half] = b * c + a * s
    return out


def latent_kv(h, W, p, m, eps):
    """The cached part of a latent-attention layer: normed latent and the
    rotated shared key part, per token."""
    R, rd = m["kv_rank"], m["rot_dim"]
    T = h.shape[0]
    d = h @ _f(W[p + "dkv"]).t()
    c = unit_rms(d[:, :R], eps) * _f(W[p + "dkv.norm"])
    kr = torch.stack([rotate(d[t, R:], t, m["rot"]["dims"], m["rot"]["base"])
                      for t in range(T)])
    assert kr.shape[1] == rd
    return c, kr


def latent_attention(h, W, p, m, eps, shared=None):
    """Windowed attention over a low-rank latent with a sink in the softmax
    denominator. ``shared`` = (c, kr) of the layer named by kv_from."""
    H, D, rd, V = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    T = h.shape[0]
    c, kr = shared if shared is not None else latent_kv(h, W, p, m, eps)
    q = (h @ _f(W[p + "q"]).t()).view(T, H, D + rd)
    kn = (c @ _f(W[p + "uk"]).t()).view(T, H, D)
    vv = (c @ _f(W[p + "uv"]).t()).view(T, H, V)
    sink = _f(W[p + "sink"])
    win = m["mask"]["size"]
    out = torch.zeros(T, H, V, dtype=DT)
    for t in range(T):
        lo = max(0, t - win + 1)
        for hd in range(H):
            qn = q[t, hd, :D]
            qr = rotate(q[t, hd, D:], t, m["rot"]["dims"], m["rot"]["base"])
            sc = torch.stack([(qn @ kn[j, hd] + qr @ kr[j]) * m["scale"]
                              for j in range(lo, t + 1)])
            mx = max(float(sc.max()), float(sink[hd]))
            e = torch.exp(sc - mx)
            den = e.sum() + math.exp(float(sink[hd]) - mx)
            for n, j in enumerate(range(lo, t + 1)):
                out[t, hd] += e[n] / den * vv[j, hd]
    out = out.reshape(T, H * V) * sigmoid(h @ _f(W[p + "g"]).t())
    return out @ _f(W[p + "o"]).t(), (c, kr)


# ------------------------------------------------------------ feed-forward
def gated_ff(h, gate, up, down):
    return (silu(h @ _f(gate).t()) * (h @ _f(up).t())) @ _f(down).t()


def table_moe(h, tokens, W, p, top):
    table = W[p + "table"]
    out = torch.zeros_like(h)
    for t, tok in enumerate(tokens):
        for e in table[tok].tolist():
            q = f"{p}e{e}."
            out[t] += gated_ff(h[t:t + 1], W[q + "gate"], W[q + "up"],
                               W[q + "down"])[0] / top
    return out


def token_side(x, tokens, W, li, cfg):
    d = cfg["token_side"]["dim"]
    p = f"l{li}.side."
    out = x.clone()
    for t, tok in enumerate(tokens):
        e = _f(W["side.embed"][tok, li * d:(li + 1) * d])
        g = gelu_tanh(_f(W[p + "gate"]) @ x[t]) * e
        y = _f(W[p + "proj"]) @ g
        out[t] = x[t] + unit_rms(y, cfg["norm"]["eps"]) * _f(W[p + "norm"])
    return out


# ------------------------------------------------------------------ model
def forward(cfg, W, tokens, return_layers=False):
    """Logits [T, vocab] of one whole sequence (positions 0..T-1)."""
    eps = cfg["norm"]["eps"]
    x = _f(W["embed"][torch.tensor(tokens)])
    caches, layers = {}, []
    for li, L in enumerate(cfg["layers"]):
        p = f"l{li}."
        h = unit_rms(x, eps) * _f(W[p + "norm1"])
        h = h + causal_taps(h, _f(W[p + "canon1"]))
        m = L["mixer"]
        if L["type"] == "general_delta":
            y = general_delta(h, W, p + "mix.", m, eps)
        elif L["type"] == "mamba2":
            y = mamba2(h, W, p + "mix.", m, eps)
        elif L["type"] == "latent_attention":
            src = m.get("kv_from")
            y, kv = latent_attention(h, W, p + "mix.", m, eps,
                                     None if src is None else caches[src])
            caches[li] = kv
        else:
            raise ValueError(L["type"])
        x = x + y
        if L.get("mlp") is not None:
            h = unit_rms(x, eps) * _f(W[p + "norm2"])
            if L["mlp"]["kind"] == "dense":
                y = gated_ff(h, W[p + "mlp.gate"], W[p + "mlp.up"],
                             W[p + "mlp.down"])
            else:
                y = table_moe(h, tokens, W, p + "mlp.",
                              L["mlp"]["router"]["top"])
            x = x + y
        x = token_side(x, tokens, W, li, cfg)
        layers.append(x.clone())
    h = unit_rms(x, eps) * _f(W["final.norm"])
    logits = (h @ _f(W["head"]).t()) * cfg["logit_scale"]
    return (logits, torch.stack(layers)) if return_layers else logits


# ----------------------------------------------------------- random models
def random_weights(cfg, seed=0, std=None):
    """Random bf16-representable weights for ``cfg`` (names as in a
    checkpoint of this design); returns name -> tensor."""
    g = torch.Generator().manual_seed(seed)
    Wd, V, S = cfg["width"], cfg["vocab"], cfg["token_side"]["dim"]
    nL = len(cfg["layers"])
    W = {}

    def mat(o, i, scale=1.0):
        t = torch.randn(o, i, generator=g) * (scale / math.sqrt(i))
        return t.bfloat16().float()

    def vec(n, mean=0.0, sd=1.0):
        return (mean + sd * torch.randn(n, generator=g)).bfloat16().float()

    W["embed"] = torch.randn(V, Wd, generator=g).bfloat16().float()
    W["side.embed"] = torch.randn(V, nL * S, generator=g).bfloat16().float()
    W["head"] = mat(V, Wd)
    W["final.norm"] = vec(1, 1.0, 0.1)[0]
    for li, L in enumerate(cfg["layers"]):
        p = f"l{li}."
        W[p + "norm1"] = vec(1, 1.0, 0.1)[0]
        W[p + "norm2"] = vec(1, 1.0, 0.1)[0]
        W[p + "canon1"] = vec(Wd * cfg["canon"]["taps"], 0, 0.3).view(Wd, -1)
        W[p + "side.gate"] = mat(S, Wd)
        W[p + "side.proj"] = mat(Wd, S)
        W[p + "side.norm"] = vec(Wd, 0.5, 0.1)
        m, q = L["mixer"], p + "mix."
        if L["type"] == "general_delta":
            n = m["heads"] * m["dim"]
            rank = m.get("_decay_rank", 8)
            for nm in "rkvga":
                W[q + nm] = mat(n, Wd, 1.5)
            W[q + "a.b"] = vec(n, 0, 0.5)
            W[q + "w1"] = mat(rank, Wd)
            W[q + "w2"] = mat(n, rank, 2.0)
            W[q + "w0"] = vec(n, 0, 1.0)
            W[q + "norm"] = vec(n, 1.0, 0.1)
            W[q + "o"] = mat(Wd, n)
        elif L["type"] == "mamba2":
            H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            inner, ch = H * P, H * P + 2 * G * N
            W[q + "in"] = mat(2 * inner + 2 * G * N + H, Wd, 1.5)
            W[q + "conv"] = vec(ch * m["conv"], 0, 0.4).view(ch, -1)
            W[q + "conv.b"] = vec(ch, 0, 0.2)
            W[q + "dt_bias"] = vec(H, 0, 0.5)
            W[q + "A_log"] = vec(H, -0.5, 0.5)
            W[q + "D"] = vec(H, 1.0, 0.2)
            W[q + "norm"] = vec(inner, 1.0, 0.1)
            W[q + "o"] = mat(Wd, inner)
        else:
            H, D, rd, Vd, R = (m["heads"], m["dim"], m["rot_dim"], m["vdim"],
                               m["kv_rank"])
            W[q + "q"] = mat(H * (D + rd), Wd, 2.0)
            if m.get("kv_from") is None:
                W[q + "dkv"] = mat(R + rd, Wd, 2.0)
                W[q + "dkv.norm"] = vec(R, 1.0, 0.1)
            W[q + "uk"] = mat(H * D, R, 2.0)
            W[q + "uv"] = mat(H * Vd, R)
            W[q + "sink"] = vec(H, 0, 1.0)
            W[q + "g"] = mat(H * Vd, Wd)
            W[q + "o"] = mat(Wd, H * Vd)
        mlp = L.get("mlp")
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            W[p + "mlp.gate"] = mat(mlp["ff"], Wd)
            W[p + "mlp.up"] = mat(mlp["ff"], Wd)
            W[p + "mlp.down"] = mat(Wd, mlp["ff"])
        else:
            E, top, ff = (mlp["router"]["experts"], mlp["router"]["top"],
                          mlp["expert"]["ff"])
            for e in range(E):
                W[f"{p}mlp.e{e}.gate"] = mat(ff, Wd)
                W[f"{p}mlp.e{e}.up"] = mat(ff, Wd)
                W[f"{p}mlp.e{e}.down"] = mat(Wd, ff)
            W[p + "mlp.table"] = torch.stack(
                [torch.randperm(E, generator=g)[:top] for _ in range(V)]
            ).to(torch.int32)
    return W
