"""The Kuforax family in the rollout engine against the plain oracle
(tests/kuforax_oracle.py): each mixer and the routed feed-forward alone,
whole prompts against token-by-token decoding, portions down to two tokens,
unequal batches, reuse of pages and slots, keys at window, kept-first and
page edges and far behind, looped layers, first tokens, long decoding, odd
sizes, the checkpoint-folder loader, the trace replay entry point and greedy
generation through the engine's scheduler.

Every case runs on the CPU tier (PyTorch forms of the ops, fp32) and, marked
``gpu``, on the HIP kernels in fp32 and bf16.  Configurations are small and
made here; weights are random with a fixed seed (bf16-representable), or
built so that one key is loud where random weights would hide a fault.
"""
import copy
import io
import json
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import kuforax_oracle as O  # noqa: E402

from polyrl_amd.models.hybrid import (kuforax_config_from_json,  # noqa: E402
                                      kuforax_config_to_json)
from polyrl_amd.rollout.engine import Engine, SamplingParams  # noqa: E402
from polyrl_amd.rollout.hybrid_model import HybridInferenceModel  # noqa: E402

CPU = ("cpu", torch.float32)
GPU32 = pytest.param(("cuda", torch.float32), marks=pytest.mark.gpu)
GPU16 = pytest.param(("cuda", torch.bfloat16), marks=pytest.mark.gpu)
TARGETS = [CPU, GPU32, GPU16]
VOCAB = 89


def rot_attn(window=7, keep=2, heads=4, kv=2, dim=24, rot=8, scaling=True,
             scale=0.3):
    r = {"base": 50.0, "dims": rot}
    if scaling:
        r["scaling"] = {"factor": 3.0, "original": 24, "fast": 4.0,
                        "slow": 0.5}
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim,
                      "scale": scale, "rot": r,
                      "mask": {"size": window, "keep_first": keep}}}


def bias_attn(window=11, far=9, heads=4, kv=2, dim=16, vdim=20, scale=0.25):
    return {"type": "attention_2",
            "mixer": {"heads": heads, "kv_heads": kv, "dim": dim,
                      "vdim": vdim, "scale": scale, "bias_max": far,
                      "mask": {"size": window}}}


def moe(experts=6, top=2, identity=3, groups=3, keep=2, ff=24, shared=40):
    f = {"kind": "moe", "expert": {"ff": ff},
         "router": {"experts": experts, "top": top, "identity": identity,
                    "groups": {"count": groups, "keep": keep}}}
    if shared:
        f["shared"] = {"ff": shared}
    return f


def config(layers, width=48, loop=None):
    c = {"architecture": "Kuforax", "vocab": VOCAB, "width": width,
         "layers": [dict(copy.deepcopy(m), mlp=copy.deepcopy(f))
                    for m, f in layers],
         "norm": {"eps": 1e-5}}
    if loop:
        c["loop"] = dict(zip(("start", "stop", "times"), loop))
    return c


FULL = config([(rot_attn(), moe()), (bias_attn(), moe(top=1, groups=1, keep=1)),
               (rot_attn(window=5, keep=0, rot=24, scaling=False), None),
               (bias_attn(window=6, far=30, kv=4), moe(identity=0, shared=0))],
              loop=(1, 3, 2))


def engine(cfg, W, target, tokens=512, slots=4, page=4, **kw):
    dev, dt = target
    c = kuforax_config_from_json(cfg)
    HybridInferenceModel.resolve_shapes(
        c, {k: tuple(v.shape) for k, v in W.items()})
    e = Engine(c, device=dev, dtype=dt, page_size=page,
               kv_token_capacity=tokens, max_running_requests=slots,
               max_num_batched_tokens=kw.pop("budget", 1 << 20), **kw)
    e.model.load_state_dict(W)
    return e


def close(got, want, target, what="", routed=True):
    """Logit rows agree: error (mean removed, RMS over the vocabulary) over
    the oracle's own spread.  In bf16 a router choice can flip on a near
    tie and the rows after it inherit some of that in these tiny models, so
    with routed experts only the bulk of the rows is held to the limit
    (fp32 is the sharp comparison); without them every row is."""
    got, want = got.double().cpu(), want.double()
    assert got.shape == want.shape, f"{what}: {got.shape} vs {want.shape}"
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    err = d.pow(2).mean(-1).sqrt() / want.std(-1).clamp_min(1e-6)
    if target[1] == torch.float32:
        assert float(err.max()) < 3e-4, f"{what}: {float(err.max()):.3g}"
        return
    n_far = int((err > 0.12).sum())
    assert n_far <= (max(3, err.numel() // 2) if routed else 0), \
        f"{what}: {n_far} of {err.numel()} rows off, worst {float(err.max()):.3g}"
    assert float(err.median()) < 0.04, f"{what}: median {float(err.median()):.3g}"


def toks(n, seed=0, avoid=()):
    g = torch.Generator().manual_seed(seed)
    t = torch.randint(0, VOCAB, (n,), generator=g).tolist()
    return [x if x not in avoid else (x + 7) % VOCAB for x in t]


def run(e, rid, t, want=None, end=True):
    want = list(range(len(t))) if want is None else want
    return e.step_forced([(rid, t, want)], [rid] if end else [])


def decode_after(e, rid, t, cut):
    rows = [e.step_forced([(rid, t[:cut], list(range(cut)))], [])]
    rows += [e.step_forced([(rid, [x], [0])], []) for x in t[cut:]]
    e.step_forced([], [rid])
    return torch.cat(rows)


def in_portions(e, rid, t, sizes):
    rows, at, i = [], 0, 0
    while at < len(t):
        n = min(sizes[i % len(sizes)], len(t) - at)
        rows.append(e.step_forced([(rid, t[at:at + n], list(range(n)))], []))
        at += n
        i += 1
    e.step_forced([], [rid])
    return torch.cat(rows)


# ------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("name,layers,loop", [
    ("rotary", [(rot_attn(), None)], None),
    ("rotary-all-dims-plain-freq", [(rot_attn(rot=24, scaling=False), None)],
     None),
    ("rotary-one-kv-head", [(rot_attn(kv=1, keep=0), None)], None),
    ("rotary-mha-32", [(rot_attn(heads=2, kv=2, dim=32, rot=16), None)], None),
    ("bias", [(bias_attn(), None)], None),
    ("bias-far-beyond-window", [(bias_attn(window=9, far=200, dim=32,
                                           vdim=32), None)], None),
    ("bias-one-head", [(bias_attn(heads=1, kv=1, window=3), None)], None),
    ("experts", [(bias_attn(), moe())], None),
    ("experts-top1-one-group", [(rot_attn(), moe(top=1, groups=1, keep=1))],
     None),
    ("experts-no-identity-no-shared",
     [(rot_attn(), moe(identity=0, shared=0))], None),
    ("experts-all-groups-kept", [(bias_attn(), moe(top=3, groups=3, keep=3))],
     None),
    ("loop-whole-stack", [(rot_attn(), moe()), (bias_attn(), None)],
     (0, 2, 3)),
    ("loop-once", [(rot_attn(), None), (bias_attn(), moe())], (1, 2, 1)),
])
def test_mechanism_alone(target, name, layers, loop):
    cfg = config(layers, loop=loop)
    W = O.random_weights(cfg, seed=3)
    t = toks(29, seed=1)
    got = run(engine(cfg, W, target), "a", t)
    close(got, O.forward(cfg, W, t), target, name,
          routed=any(f is not None for _, f in layers))


def test_router_choice_with_negative_scores():
    """All choice scores negative: experts of closed groups must count as
    minus infinity (never as zero), the correction must steer the choice
    only, and the weights must come from the uncorrected scores."""
    from polyrl_amd.ops import seq
    r = {"experts": 9, "identity": 3, "top": 3,
         "groups": {"count": 4, "keep": 2}}
    g = torch.Generator().manual_seed(5)
    W = {"x.router": torch.randn(12, 20, generator=g),
         "x.correction": -1.0 + 0.3 * torch.randn(12, generator=g)}
    h = torch.randn(64, 20, generator=g)
    idx, w = O.route(h.double(), W, "x.", r)
    z = h @ W["x.router"].t()
    got_i, got_s = seq.moe_route(z, W["x.correction"], 3, 4, 2)
    assert torch.equal(got_i.long().sort(-1).values, idx.sort(-1).values)
    got_w = got_s / got_s.sum(-1, keepdim=True)
    torch.testing.assert_close(got_w.double().sort(-1).values,
                               w.sort(-1).values, rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
def test_router_kernel_matches_oracle():
    from polyrl_amd.ops import seq
    for E, n_id, top, groups, keep in ((9, 3, 3, 4, 2), (5, 0, 1, 1, 1),
                                       (70, 10, 4, 8, 3), (6, 2, 2, 2, 1)):
        r = {"experts": E, "identity": n_id, "top": top,
             "groups": {"count": groups, "keep": keep}}
        g = torch.Generator().manual_seed(E)
        W = {"x.router": torch.randn(E + n_id, 24, generator=g),
             "x.correction": -0.5 + 0.3 * torch.randn(E + n_id, generator=g)}
        h = torch.randn(133, 24, generator=g)
        idx, w = O.route(h.double(), W, "x.", r)
        z = (h @ W["x.router"].t()).cuda()
        got_i, got_s = seq.moe_route(z, W["x.correction"].cuda(), top,
                                     groups, keep)
        same = (got_i.long().cpu().sort(-1).values ==
                idx.sort(-1).values).all(-1)
        assert int((~same).sum()) <= 1, (E, int((~same).sum()))   # fp32 ties
        got_w = (got_s / got_s.sum(-1, keepdim=True)).cpu()
        torch.testing.assert_close(
            got_w.double().sort(-1).values[same], w.sort(-1).values[same],
            rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("skewed", [False, True])
def test_prompt_sized_expert_batches(target, skewed):
    """300 rows take the sorted per-expert products, with routing spread
    over the experts and with every token sent to one of them."""
    cfg = config([(bias_attn(window=5), moe(experts=8, top=1, identity=0,
                                            groups=1, keep=1, shared=0))])
    W = O.random_weights(cfg, seed=9)
    if skewed:
        W["l0.mlp.correction"].zero_()
        W["l0.mlp.correction"][3] = 4.0
    t = toks(300, seed=8)
    e = engine(cfg, W, target, tokens=320)
    want = O.forward(cfg, W, t)
    close(run(e, "a", t), want, target, f"skewed={skewed}")


@pytest.mark.parametrize("target", TARGETS)
def test_residual_after_every_layer_run(target):
    W = O.random_weights(FULL, seed=7)
    t = toks(17, seed=2)
    e = engine(FULL, W, target)
    e.model.capture_layers = []
    run(e, "a", t)
    _, want = O.forward(FULL, W, t, return_layers=True)
    assert len(e.model.capture_layers) == want.shape[0] == 6
    for i, got in enumerate(e.model.capture_layers):
        d = (got.double().cpu() - want[i]).abs().max() / want[i].abs().max()
        lim = 2e-5 if target[1] == torch.float32 else 0.2
        assert float(d) < lim, f"layer run {i}: {float(d):.3g}"


# ---------------------------------------------- schedules give one answer
@pytest.mark.parametrize("target", TARGETS)
def test_prefill_decode_and_portions_agree_with_oracle(target):
    W = O.random_weights(FULL, seed=11)
    t = toks(41, seed=3)
    want = O.forward(FULL, W, t)
    e = engine(FULL, W, target, page=4)
    close(run(e, "whole", t), want, target, "whole")
    close(decode_after(e, "dec", t, 1), want, target, "token by token")
    close(decode_after(e, "dec9", t, 9), want, target, "prefill 9 + decode")
    for sizes in ((2,), (3, 2, 7), (16, 5), (4,), (13, 1, 1, 2)):
        close(in_portions(e, f"p{sizes}", t, sizes), want, target,
              f"portions {sizes}")
    assert e.kv.free_pages == e.kv.num_pages


@pytest.mark.parametrize("target", TARGETS)
def test_unequal_batch_matches_each_alone(target):
    W = O.random_weights(FULL, seed=13)
    seqs = {"a": toks(33, seed=4), "b": toks(2, seed=5), "c": toks(19, seed=6),
            "d": toks(1, seed=7)}
    want = {k: O.forward(FULL, W, v) for k, v in seqs.items()}
    e = engine(FULL, W, target, page=4)
    at = {k: 0 for k in seqs}
    got = {k: [] for k in seqs}
    plan = [{"a": 5, "b": 2, "c": 1, "d": 1}, {"a": 1, "c": 9},
            {"c": 1, "a": 20}, {"a": 1, "c": 8}, {"a": 6}]
    for step in plan:
        entries, end = [], []
        for k, n in step.items():
            entries.append((k, seqs[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == len(seqs[k]):
                end.append(k)
        out = e.step_forced(entries, end)
        o = 0
        for k, n in step.items():
            got[k].append(out[o:o + n])
            o += n
    for k in seqs:
        assert at[k] == len(seqs[k])
        close(torch.cat(got[k]), want[k], target, f"request {k}")


@pytest.mark.parametrize("target", TARGETS)
def test_pages_and_slots_are_reused_clean(target):
    """A pool of 6 pages and 2 slots serves a stream of requests: every page
    and slot is handed out again with another request's rows in it."""
    W = O.random_weights(FULL, seed=17)
    e = engine(FULL, W, target, tokens=24, slots=2, page=4)
    for i, n in enumerate((21, 7, 13, 24, 3, 10)):
        t = toks(n, seed=20 + i)
        got = decode_after(e, f"r{i}", t, max(1, n - 3)) if i % 2 else \
            run(e, f"r{i}", t)
        close(got, O.forward(FULL, W, t), target, f"request {i}")
        assert e.kv.free_pages == e.kv.num_pages
    a, b = toks(11, seed=40), toks(12, seed=41)
    e.step_forced([("a", a[:6], []), ("b", b[:2], [])], [])
    ga = e.step_forced([("a", a[6:], list(range(5)))], ["a"])
    c = toks(9, seed=42)                     # takes a's pages and slot
    gc = e.step_forced([("c", c, list(range(9))), ("b", b[2:], [])], ["c"])
    close(ga, O.forward(FULL, W, a)[6:], target, "a")
    close(gc[:9], O.forward(FULL, W, c), target, "c in a's pages")


# ------------------------------------------- edges made visible by a loud key
LOUD = 5


def _loud_key_model(layer, width=32):
    """One attention layer in which token LOUD's key is loud for every
    query: channel 0 of every embedding carries a constant, channel 1 is
    set for LOUD only; the last entry of every query head reads channel 0,
    the last entry of every key head reads channel 1.  Whoever still sees
    LOUD attends to it, so an edge that is one token off moves the logits."""
    cfg = config([(layer, None)], width=width)
    W = O.random_weights(cfg, seed=23)
    m = layer["mixer"]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    W["embed"][:, 0] = 3.0
    W["embed"][:, 1] = 0.0
    W["embed"][LOUD, 1] = 6.0
    W["l0.norm1"][:2] = 0.0
    for h in range(H):
        W["l0.mix.q"][h * D + D - 1] = 0.0
        W["l0.mix.q"][h * D + D - 1, 0] = 4.0
    for g in range(G):
        W["l0.mix.k"][g * D + D - 1] = 0.0
        W["l0.mix.k"][g * D + D - 1, 1] = 16.0
    m["scale"] = 1.0
    return cfg, W


def _edge_case(target, cfg, W, t, edges, tag):
    want = O.forward(cfg, W, t)
    e = engine(cfg, W, target, page=4, tokens=1024)
    close(run(e, "whole", t), want, target, f"{tag} prompt", routed=False)
    first = min(edges)
    close(decode_after(e, "dec", t, max(1, first - 2)), want, target,
          f"{tag} decoded", routed=False)
    for cut in sorted({c for x in edges for c in (x - 1, x, x + 1)}):
        if 0 < cut < len(t):
            rows = [e.step_forced([("p", t[:cut], list(range(cut)))], []),
                    e.step_forced([("p", t[cut:], list(range(len(t) - cut)))],
                                  ["p"])]
            close(torch.cat(rows), want, target, f"{tag} cut at {cut}",
                  routed=False)
    close(in_portions(e, "two", t, (2,)), want, target, f"{tag} in twos",
          routed=False)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("window", [1, 4, 9, 16])
@pytest.mark.parametrize("kind", ["rotary", "bias"])
def test_window_edge_in_prompt_and_decode(target, window, kind):
    layer = rot_attn(window=window, keep=0, dim=16, rot=8) if kind == "rotary" \
        else bias_attn(window=window, far=12)
    cfg, W = _loud_key_model(layer)
    t = toks(3 * window + 11, seed=9, avoid=(LOUD,))
    loud = window + 1                        # crosses a page edge for page=4
    t[loud] = LOUD
    t2 = list(t)
    t2[loud] = LOUD + 1
    d = (O.forward(cfg, W, t) - O.forward(cfg, W, t2)).abs().max(-1).values
    assert float(d[loud + window - 1]) > 0.05, "test model hides the edge"
    assert float(d[loud + window]) < 1e-9, "edge is not where it should be"
    _edge_case(target, cfg, W, t, [loud + window - 1, loud + window], kind)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("keep", [1, 3, 4, 6])
def test_kept_first_tokens_stay_visible_far_away(target, keep):
    """LOUD as the last kept token is seen from hundreds of tokens away;
    LOUD as the first token that is not kept leaves with the window."""
    window = 5
    cfg, W = _loud_key_model(rot_attn(window=window, keep=keep, dim=16,
                                      rot=8))
    n = 150
    for where, seen in ((keep - 1, True), (keep, False)):
        t = toks(n, seed=10 + keep, avoid=(LOUD,))
        t[where] = LOUD
        t2 = list(t)
        t2[where] = LOUD + 1
        d = (O.forward(cfg, W, t) - O.forward(cfg, W, t2)).abs().max(-1).values
        assert (float(d[-1]) > 0.05) == seen, "test model hides the kept key"
        _edge_case(target, cfg, W, t[:40], [where + window - 1,
                                             where + window], f"keep {keep}")
        e = engine(cfg, W, target, page=4, tokens=256)
        got = decode_after(e, "far", t, n - 6)
        close(got, O.forward(cfg, W, t), target, f"far key, kept={seen}",
              routed=False)


@pytest.mark.parametrize("target", TARGETS)
def test_distance_buckets_show_in_the_logits(target):
    """A bias table with one huge row per bucket in turn: a distance that
    lands in the wrong bucket changes which key wins."""
    layer = bias_attn(window=40, far=24, heads=2, kv=1)
    cfg = config([(layer, None)], width=32)
    W = O.random_weights(cfg, seed=27, bias_rows=10)
    t = toks(64, seed=12)
    for row in range(10):
        W["l0.mix.rel"].zero_()
        W["l0.mix.rel"][row] = 9.0
        e = engine(cfg, W, target, page=4)
        want = O.forward(cfg, W, t)
        close(run(e, "w", t), want, target, f"bucket row {row}",
              routed=False)
        close(decode_after(e, "d", t, 30), want, target,
              f"bucket row {row} decoded", routed=False)


@pytest.mark.parametrize("target", TARGETS)
def test_first_tokens_and_long_decoding(target):
    W = O.random_weights(FULL, seed=31)
    e = engine(FULL, W, target)
    for n in (1, 2, 3, 4):
        t = toks(n, seed=50 + n)
        close(run(e, f"s{n}", t), O.forward(FULL, W, t), target, f"len {n}")
    t = toks(120, seed=55)
    close(decode_after(e, "long", t, 2), O.forward(FULL, W, t), target,
          "118 decoded tokens")


# ------------------------------------- loader, replay entry, generation
def _save(tmp_path, cfg, W):
    from safetensors.torch import save_file
    d = tmp_path / "ckpt"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.bfloat16().contiguous() for k, v in W.items()},
              str(d / "model.safetensors"))
    return str(d)


def test_config_round_trip():
    c = kuforax_config_from_json(FULL)
    assert c.run_order() == [0, 1, 2, 1, 2, 3]
    assert kuforax_config_from_json(kuforax_config_to_json(c)) == c


@pytest.mark.parametrize("target", [CPU, GPU32])
def test_folder_loader_and_trace_replay(target, tmp_path, monkeypatch, capsys):
    from polyrl_amd.models import get_model_config
    from polyrl_amd.rollout import trace_replay
    W = O.random_weights(FULL, seed=37)
    path = _save(tmp_path, FULL, W)
    c = get_model_config(path)
    assert c.arch == "kuforax" and c.num_hidden_layers == 4
    a, b = toks(13, seed=60), toks(6, seed=61)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:8], "want": [7]},
                                {"id": "b", "tokens": b, "want": [0, 5]}],
         "end": ["b"]},
        {"step": 1, "entries": [{"id": "a", "tokens": a[8:9], "want": []}],
         "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": a[9:], "want": [3]}],
         "end": ["a"]},
    ]
    monkeypatch.setattr(sys, "stdin",
                        io.StringIO("\n".join(map(json.dumps, steps)) + "\n"))
    out = tmp_path / "out"
    rc = trace_replay.main(["--model", path, "--dtype", "float32", "--out",
                            str(out), "--max-tokens", "128", "--device",
                            target[0]])
    assert rc == 0
    assert capsys.readouterr().out.split() == ["done", "0", "done", "1",
                                               "done", "2"]
    import numpy as np
    wa, wb = O.forward(FULL, W, a), O.forward(FULL, W, b)
    g0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4")
                          .reshape(3, -1))
    close(g0, torch.stack([wa[7], wb[0], wb[5]]), target, "step 0")
    assert not (out / "1.f32").exists()
    g2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4")
                          .reshape(1, -1))
    close(g2, wa[12:13], target, "step 2")


@pytest.mark.parametrize("target", TARGETS)
def test_greedy_generation_through_the_scheduler(target):
    """Engine.generate: admission, chunked prompts (token budget of 8),
    mixed steps, sampling at temperature 0, pages and slots released."""
    if target[0] == "cuda":
        from polyrl_amd.ops import seq
        assert seq.seq_extension_loaded()
    W = O.random_weights(FULL, seed=41)
    e = engine(FULL, W, target, slots=3, budget=8)
    prompts = [toks(n, seed=70 + n) for n in (11, 2, 17, 5)]
    outs = e.generate(prompts, SamplingParams(temperature=0.0,
                                              max_new_tokens=5), "g")
    for p, o in zip(prompts, outs):
        ids = list(p)
        for got_tok in o.output_ids:
            logits = O.forward(FULL, W, ids)[-1]
            top2 = logits.topk(2).values
            tie = 1e-3 if target[1] == torch.float32 else \
                0.25 * float(logits.std())
            if float(top2[0] - top2[1]) > tie:      # skip near ties
                assert got_tok == int(logits.argmax())
            ids.append(got_tok)
        assert len(o.output_ids) == 5 and o.finish_reason == "length"
    assert e.kv.free_pages == e.kv.num_pages
    assert e.states.free_slots == e.states.num_slots


def test_registry_preset_runs_and_resumes_memory():
    from polyrl_amd.models import get_model_config
    c = get_model_config("kuforax-debug")
    e = Engine(c, device="cpu", dtype=torch.float32, page_size=4,
               kv_token_capacity=64, max_running_requests=2)
    e.model.init_random(seed=1)
    t = toks(9, seed=90)
    a = run(e, "a", t)
    assert a.shape == (9, c.vocab_size) and torch.isfinite(a).all()
    e.release_memory()
    assert not e.kv.rows
    e.resume_memory()
    torch.testing.assert_close(run(e, "b", t), a)
