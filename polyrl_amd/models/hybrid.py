"""Configuration of hybrid decoders: a stack whose layers each pick one
sequence mixer (recurrent, state-space or windowed latent attention) and one
feed-forward (dense, table-routed experts, or none).

The Bizusun design is the first family described this way.  Everything that
can differ between two models of a family is a field here and is read from
the checkpoint's ``config.json``; constants that the design fixes (the decay
constant of the delta rule, its key epsilon) are defaults of the mixer
parameters, so another design can set them differently.
"""
from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass, field
from typing import List, Optional


@dataclass
class DeltaRuleSpec:
    """Generalised delta rule: per-channel decay and removal rate."""
    heads: int
    dim: int
    decay_rank: Optional[int] = None      # rows of w1; None = from the tensor
    decay_scale: float = math.exp(-0.5)   # w = exp(-decay_scale * sigmoid(.))
    key_eps: float = 1e-6                 # unit key: k / sqrt(sum k^2 + eps)
    kind: str = "general_delta"


@dataclass
class SSMSpec:
    """Mamba-2 style selective state space layer."""
    heads: int
    vdim: int
    state: int
    groups: int = 1
    norm_groups: int = 1
    conv: int = 4
    kind: str = "mamba2"

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state


@dataclass
class LatentAttnSpec:
    """Windowed multi-head attention over a shared low-rank latent."""
    heads: int
    dim: int              # unrotated query/key size per head
    rot_dim: int          # rotated query/key size per head (key part shared)
    vdim: int
    kv_rank: int
    window: int           # a query sees itself and window-1 tokens before it
    scale: float
    rope_base: float = 10000.0
    rope_dims: Optional[int] = None       # rotated pairs cover the first dims
    kv_from: Optional[int] = None         # reuse that layer's latent cache
    kind: str = "latent_attention"

    def __post_init__(self):
        if self.rope_dims is None:
            self.rope_dims = self.rot_dim


@dataclass
class FFSpec:
    kind: str                 # dense | moe
    ff: int                   # hidden size (of one expert for moe)
    experts: int = 0
    top: int = 0


@dataclass
class HybridLayerSpec:
    mixer: object
    ff: Optional[FFSpec]


@dataclass
class HybridConfig:
    arch: str = "bizusun"
    vocab_size: int = 512
    hidden_size: int = 128
    layers: List[HybridLayerSpec] = field(default_factory=list)
    norm_eps: float = 1e-6
    canon_taps: int = 4
    token_side_dim: int = 0
    logit_scale: float = 1.0
    max_position_embeddings: int = 1 << 20   # no learned positions: a fence

    # the engine's generic accessors
    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @property
    def is_hybrid(self) -> bool:
        return True

    def cache_owner(self, li: int) -> Optional[int]:
        """Layer whose latent cache layer ``li`` reads (itself unless it
        shares), or None for a layer without a paged cache."""
        m = self.layers[li].mixer
        if m.kind != "latent_attention":
            return None
        return li if m.kv_from is None else m.kv_from

    def validate(self):
        for li, L in enumerate(self.layers):
            m = L.mixer
            if m.kind == "latent_attention" and m.kv_from is not None:
                src = self.layers[m.kv_from].mixer
                if not (0 <= m.kv_from < li) or \
                        src.kind != "latent_attention" or \
                        src.kv_from is not None:
                    raise ValueError(f"layer {li}: kv_from must name an "
                                     "earlier layer that owns its cache")
                if (src.kv_rank, src.rot_dim) != (m.kv_rank, m.rot_dim):
                    raise ValueError(f"layer {li}: a shared cache needs "
                                     "equal latent and rotated sizes")
            if m.kind == "mamba2":
                assert m.heads % m.groups == 0
                assert m.inner % m.norm_groups == 0
            if L.ff is not None and L.ff.kind == "moe":
                assert 0 < L.ff.top <= L.ff.experts
        return self


def _mixer_from_json(kind: str, m: dict):
    if kind == "general_delta":
        return DeltaRuleSpec(heads=int(m["heads"]), dim=int(m["dim"]))
    if kind == "mamba2":
        return SSMSpec(heads=int(m["heads"]), vdim=int(m["vdim"]),
                       state=int(m["state"]), groups=int(m.get("groups", 1)),
                       norm_groups=int(m.get("norm_groups", 1)),
                       conv=int(m["conv"]))
    if kind == "latent_attention":
        rot = m.get("rot", {})
        return LatentAttnSpec(
            heads=int(m["heads"]), dim=int(m["dim"]),
            rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
            kv_rank=int(m["kv_rank"]), window=int(m["mask"]["size"]),
            scale=float(m["scale"]),
            rope_base=float(rot.get("base", 10000.0)),
            rope_dims=int(rot.get("dims", m["rot_dim"])),
            kv_from=(None if m.get("kv_from") is None
                     else int(m["kv_from"])))
    raise ValueError(f"unknown mixer type {kind!r}")


def _ff_from_json(f: Optional[dict]) -> Optional[FFSpec]:
    if f is None:
        return None
    if f["kind"] == "dense":
        return FFSpec(kind="dense", ff=int(f["ff"]))
    if f["kind"] == "moe":
        return FFSpec(kind="moe", ff=int(f["expert"]["ff"]),
                      experts=int(f["router"]["experts"]),
                      top=int(f["router"]["top"]))
    raise ValueError(f"unknown feed-forward kind {f['kind']!r}")


def bizusun_config_from_json(d: dict) -> HybridConfig:
    """Read a Bizusun ``config.json`` (already parsed)."""
    layers = [HybridLayerSpec(_mixer_from_json(L["type"], L["mixer"]),
                              _ff_from_json(L.get("mlp")))
              for L in d["layers"]]
    return HybridConfig(
        arch="bizusun", vocab_size=int(d["vocab"]),
        hidden_size=int(d["width"]), layers=layers,
        norm_eps=float(d["norm"]["eps"]),
        canon_taps=int(d["canon"]["taps"]),
        token_side_dim=int(d["token_side"]["dim"]),
        logit_scale=float(d.get("logit_scale", 1.0))).validate()


def bizusun_config_to_json(cfg: HybridConfig) -> dict:
    """Inverse of :func:`bizusun_config_from_json` (checkpoint export)."""
    layers = []
    for L in cfg.layers:
        m = L.mixer
        if m.kind == "general_delta":
            mj = {"heads": m.heads, "dim": m.dim}
        elif m.kind == "mamba2":
            mj = {"heads": m.heads, "vdim": m.vdim, "state": m.state,
                  "groups": m.groups, "norm_groups": m.norm_groups,
                  "conv": m.conv}
        else:
            mj = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim,
                  "vdim": m.vdim, "kv_rank": m.kv_rank,
                  "mask": {"size": m.window}, "scale": m.scale,
                  "rot": {"base": m.rope_base, "dims": m.rope_dims}}
            if m.kv_from is not None:
                mj["kv_from"] = m.kv_from
        if L.ff is None:
            fj = None
        elif L.ff.kind == "dense":
            fj = {"kind": "dense", "ff": L.ff.ff}
        else:
            fj = {"kind": "moe", "expert": {"ff": L.ff.ff},
                  "router": {"experts": L.ff.experts, "top": L.ff.top}}
        layers.append({"type": m.kind, "mixer": mj, "mlp": fj})
    return {"architecture": "Bizusun", "vocab": cfg.vocab_size,
            "width": cfg.hidden_size, "layers": layers,
            "norm": {"eps": cfg.norm_eps},
            "canon": {"taps": cfg.canon_taps},
            "token_side": {"dim": cfg.token_side_dim},
            "logit_scale": cfg.logit_scale}


def bizusun_preset(width: int, layers: int, vocab: int = 32000,
                   heads: int = 16, ff_mult: float = 2.5, experts: int = 16,
                   top: int = 2, window: int = 1024,
                   pattern=("general_delta", "mamba2", "latent_attention",
                            "latent_attention")) -> HybridConfig:
    """A Bizusun stack of realistic layer sizes (random weights): the mixer
    kinds cycle through ``pattern``; the second latent-attention layer of
    each cycle shares the first one's cache; the first layer is dense, the
    rest use table-routed experts of equal total active width."""
    hd = width // heads
    out: List[HybridLayerSpec] = []
    last_owner = None
    for li in range(layers):
        kind = pattern[li % len(pattern)]
        if kind == "general_delta":
            mixer = DeltaRuleSpec(heads=heads, dim=hd)
            last_owner = None
        elif kind == "mamba2":
            mixer = SSMSpec(heads=2 * heads, vdim=hd, state=128,
                            groups=max(1, heads // 8), norm_groups=1, conv=4)
            last_owner = None
        else:
            mixer = LatentAttnSpec(
                heads=heads, dim=hd, rot_dim=hd // 2, vdim=hd,
                kv_rank=4 * hd, window=window,
                scale=1.0 / math.sqrt(hd + hd // 2), kv_from=last_owner)
            if last_owner is None:
                last_owner = li
        dense_ff = int(width * ff_mult) // 64 * 64
        ff = FFSpec("dense", dense_ff) if li == 0 else \
            FFSpec("moe", max(64, dense_ff // top // 64 * 64), experts, top)
        out.append(HybridLayerSpec(mixer, ff))
    return HybridConfig(arch="bizusun", vocab_size=vocab, hidden_size=width,
                        layers=out, norm_eps=1e-6, canon_taps=4,
                        token_side_dim=max(8, width // 16),
                        logit_scale=1.0).validate()


def read_config_dir(path: str):
    """Model config from a checkpoint folder's ``config.json``.  The
    ``architecture`` key names the family; HF-style folders
    (``model_type``) map onto the dense decoder config."""
    with open(os.path.join(path, "config.json")) as f:
        d = json.load(f)
    arch = d.get("architecture")
    if arch == "Bizusun":
        return bizusun_config_from_json(d)
    mt = d.get("model_type")
    if mt in ("llama", "qwen2"):
        from .registry import DecoderConfig
        return DecoderConfig(
            arch=mt, vocab_size=d["vocab_size"], hidden_size=d["hidden_size"],
            intermediate_size=d["intermediate_size"],
            num_hidden_layers=d["num_hidden_layers"],
            num_attention_heads=d["num_attention_heads"],
            num_key_value_heads=d.get("num_key_value_heads",
                                      d["num_attention_heads"]),
            head_dim=d.get("head_dim"),
            max_position_embeddings=d.get("max_position_embeddings", 8192),
            rms_norm_eps=d.get("rms_norm_eps", 1e-5),
            rope_theta=d.get("rope_theta", 10000.0),
            tie_word_embeddings=d.get("tie_word_embeddings", False),
            attention_bias=d.get("attention_bias", mt == "qwen2"))
    raise ValueError(f"{path}: unknown architecture "
                     f"{arch or mt!r} in config.json")
