"""Plain, slow implementation of the Kuforax design for the tests.

One function per mechanism, written from the design's equations; whole
sequences only (no cache, no batching, no paging).  It shares no code with
``polyrl_amd``: the engine, its cache manager and its kernels are compared
against these functions.

Conventions: ``W`` maps tensor names to torch tensors, linear weights are
[out, in] and applied as ``W @ x``; ``cfg`` is the parsed config dict.
Everything runs in ``DT`` (float64 by default).
"""
import math

import torch

DT = torch.float64


def _f(t):
    return t.to(DT)


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    """RMS norm whose stored weight is an offset from one."""
    return unit_rms(x, eps) * (1.0 + _f(w))


# ------------------------------------------------------------- rotation
def yarn_frequencies(rot):
    """Per-pair frequencies and the amplitude factor of the rotation.
    Without a 'scaling' entry: f_i = base^(-2i/dims), amplitude 1."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=DT), 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def turn_dim(turns):
        return dims * math.log(orig / (2 * math.pi * turns)) / \
            (2 * math.log(base))
    lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / factor * ramp + f[i] * (1.0 - ramp))
    return torch.tensor(out, dtype=DT), 0.1 * math.log(factor) + 1.0


def rotate(vec, pos, freqs, amp):
    """Rotate-half on the first 2*len(freqs) entries of the last axis of
    vec [..., D] at integer position pos; the rest passes through."""
    half = freqs.numel()
    ang = pos * freqs
    c, s = torch.cos(ang) * amp, torch.sin(ang) * amp
    u, v = vec[..., :half], vec[..., half:2 * half]
    return torch.cat([u * c - v * s, v * c + u * s, vec[..., 2 * half:]], -1)


# ------------------------------------------------------------ attention
def visible_window_keep(i, j, size, keep):
    return j <= i and (i - j < size or j < keep)


def visible_window(i, j, size):
    return 0 <= i - j < size


def softmax_attend(scores, allowed, v):
    """scores [T, T] (query, key), allowed bool [T, T], v [T, dv]."""
    s = scores.masked_fill(~allowed, float("-inf"))
    p = torch.softmax(s, -1)
    return p @ v


def attention_rot(h, W, p, m, eps):
    """Grouped-query attention whose values are the raw key projections,
    with whole-projection query/key norms, partial rotation, a sliding
    window that also keeps the first tokens, and a per-head output gate.
    h [T, width]."""
    T = h.shape[0]
    H, G, D = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
    q = h @ _f(W[p + "q"]).T
    k = h @ _f(W[p + "k"]).T
    v = k.clone().view(T, G, D)                  # values: keys as projected
    q = (unit_rms(q, eps) * _f(W[p + "q.norm"])).view(T, H, D)
    k = (unit_rms(k, eps) * _f(W[p + "k.norm"])).view(T, G, D)
    freqs, amp = yarn_frequencies(m["rot"])
    q = torch.stack([rotate(q[t], t, freqs, amp) for t in range(T)])
    k = torch.stack([rotate(k[t], t, freqs, amp) for t in range(T)])
    size = int(m["mask"]["size"])
    keep = int(m["mask"].get("keep_first", 0))
    allowed = torch.tensor([[visible_window_keep(i, j, size, keep)
                             for j in range(T)] for i in range(T)])
    gate = sigmoid(h @ _f(W[p + "g"]).T)         # [T, H]
    outs = []
    for hd in range(H):
        g = hd // (H // G)
        sc = (q[:, hd] @ k[:, g].T) * float(m["scale"])
        outs.append(softmax_attend(sc, allowed, v[:, g]) * gate[:, hd:hd + 1])
    return torch.cat(outs, -1) @ _f(W[p + "o"]).T


def distance_bucket(n, rows, far):
    """Row of the distance-bias table for distance n >= 0: exact below
    rows/2, logarithmic steps up to distance ``far`` above."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(
        math.log(n / half) / math.log(far / half) * (rows - half))))


def attention_bias(h, W, p, m, eps):
    """Grouped-query attention without rotation: a learned bias per
    distance bucket and head is added to the scaled scores; plain sliding
    window.  h [T, width]."""
    T = h.shape[0]
    H, G = int(m["heads"]), int(m["kv_heads"])
    D, Dv = int(m["dim"]), int(m["vdim"])
    q = (h @ _f(W[p + "q"]).T).view(T, H, D)
    k = (h @ _f(W[p + "k"]).T).view(T, G, D)
    v = (h @ _f(W[p + "v"]).T).view(T, G, Dv)
    rel = _f(W[p + "rel"])
    rows, far = rel.shape[0], float(m["bias_max"])
    size = int(m["mask"]["size"])
    allowed = torch.tensor([[visible_window(i, j, size) for j in range(T)]
                            for i in range(T)])
    bucket = torch.tensor([[distance_bucket(max(i - j, 0), rows, far)
                            for j in range(T)] for i in range(T)])
    outs = []
    for hd in range(H):
        g = hd // (H // G)
        sc = (q[:, hd] @ k[:, g].T) * float(m["scale"]) + rel[:, hd][bucket]
        outs.append(softmax_attend(sc, allowed, v[:, g]))
    return torch.cat(outs, -1) @ _f(W[p + "o"]).T


# --------------------------------------------------------- feed-forward
def plain_expert(h, up, down):
    return gelu_erf(h @ _f(up).T) @ _f(down).T


def route(h, W, p, r):
    """Chosen experts and their weights for every row of h.  Returns
    (index [T, top], weight [T, top]); indices >= experts name identity
    experts."""
    E, n_id, top = int(r["experts"]), int(r.get("identity", 0)), int(r["top"])
    groups = r.get("groups") or {"count": 1, "keep": 1}
    n_grp, keep = int(groups["count"]), int(groups["keep"])
    s = torch.softmax(h @ _f(W[p + "router"]).T, -1)       # [T, E + n_id]
    choice = s + _f(W[p + "correction"])
    per = (E + n_id) // n_grp
    grp_best = choice.view(-1, n_grp, per).max(-1).values
    kept = grp_best.topk(keep, -1).indices                 # [T, keep]
    open_ = torch.zeros_like(grp_best, dtype=torch.bool)
    open_.scatter_(1, kept, True)
    open_ = open_.repeat_interleave(per, 1)
    choice = choice.masked_fill(~open_, float("-inf"))
    idx = choice.topk(top, -1).indices
    w = s.gather(1, idx)
    return idx, w / (w.sum(-1, keepdim=True) + 1e-20)


def routed_moe(h, W, p, f):
    r = f["router"]
    E = int(r["experts"])
    idx, w = route(h, W, p, r)
    y = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(idx[t].tolist(), w[t]):
            if e >= E:
                y[t] += a * h[t]                            # identity expert
            else:
                y[t] += a * plain_expert(h[t], W[f"{p}e{e}.up"],
                                         W[f"{p}e{e}.down"])
    if f.get("shared"):
        y = y + plain_expert(h, W[p + "shared.up"], W[p + "shared.down"])
    return y


# ---------------------------------------------------------------- model
def layer_runs(cfg):
    """Layer indices in execution order (the looped span repeated)."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or int(loop["times"]) <= 1:
        return list(range(n))
    a, b, t = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(a)) + list(range(a, b)) * t + list(range(b, n))


_MIXERS = {"attention": attention_rot, "attention_2": attention_bias}


def forward(cfg, W, tokens, return_layers=False):
    """Logits [T, vocab] of one whole sequence (and the residual stream
    after every layer run)."""
    eps = float(cfg["norm"]["eps"])
    x = _f(W["embed"])[torch.as_tensor(tokens, dtype=torch.long)]
    seen = []
    for li in layer_runs(cfg):
        L = cfg["layers"][li]
        p = f"l{li}."
        y = _MIXERS[L["type"]](norm_one_plus(x, W[p + "norm1"], eps), W,
                               p + "mix.", L["mixer"], eps)
        x = x + norm_one_plus(y, W[p + "norm1b"], eps)
        if L.get("mlp") is not None:
            y = routed_moe(norm_one_plus(x, W[p + "norm2"], eps), W,
                           p + "mlp.", L["mlp"])
            x = x + norm_one_plus(y, W[p + "norm2b"], eps)
        seen.append(x.clone())
    logits = norm_one_plus(x, W["final.norm"], eps) @ _f(W["head"]).T
    if return_layers:
        return logits, torch.stack(seen)
    return logits


def random_weights(cfg, seed=0, bias_rows=8):
    """name -> tensor for a config; values are bf16-representable so every
    engine dtype loads them exactly."""
    g = torch.Generator().manual_seed(seed)
    Wd, V = int(cfg["width"]), int(cfg["vocab"])

    def rnd(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean) \
            .bfloat16().float()

    def lin(o, i, gain=1.0):
        return rnd(o, i, std=gain / math.sqrt(i))
    W = {"embed": rnd(V, Wd), "final.norm": rnd(Wd, std=0.1),
         "head": lin(V, Wd)}
    for li, L in enumerate(cfg["layers"]):
        p, m = f"l{li}.", L["mixer"]
        H, G = int(m["heads"]), int(m["kv_heads"])
        D, Dv = int(m["dim"]), int(m["vdim"])
        for n in ("norm1", "norm1b"):
            W[p + n] = rnd(Wd, std=0.1)
        W[p + "mix.q"], W[p + "mix.k"] = lin(H * D, Wd), lin(G * D, Wd)
        W[p + "mix.o"] = lin(Wd, H * Dv)
        if L["type"] == "attention":
            W[p + "mix.q.norm"] = rnd(H * D, std=0.1, mean=1.0)
            W[p + "mix.k.norm"] = rnd(G * D, std=0.1, mean=1.0)
            W[p + "mix.g"] = lin(H, Wd, gain=2.0)
        else:
            W[p + "mix.v"] = lin(G * Dv, Wd)
            W[p + "mix.rel"] = rnd(bias_rows, H)
        f = L.get("mlp")
        if f is None:
            continue
        for n in ("norm2", "norm2b"):
            W[p + n] = rnd(Wd, std=0.1)
        r = f["router"]
        E, n_id = int(r["experts"]), int(r.get("identity", 0))
        ff = int(f["expert"]["ff"])
        for e in range(E):
            W[f"{p}mlp.e{e}.up"] = lin(ff, Wd)
            W[f"{p}mlp.e{e}.down"] = lin(Wd, ff)
        W[p + "mlp.router"] = lin(E + n_id, Wd, gain=3.0)
        W[p + "mlp.correction"] = rnd(E + n_id, std=0.05)
        if f.get("shared"):
            sf = int(f["shared"]["ff"])
            W[p + "mlp.shared.up"] = lin(sf, Wd)
            W[p + "mlp.shared.down"] = lin(Wd, sf)
    return W
