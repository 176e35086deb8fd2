"""Fagunex: a decoder-only stack whose layers are listed one by one in config.json, with a span of them that
may run several times in a row on the same weights (`loop`), each pass with a cache and state of its own.

  norm          Dynamic Tanh, tanh(alpha x) w + b, before AND after each sublayer: x += n_b(f(n(x)))
  token shift   the mixer's input is blended with the previous token's: h + (h_prev - h) * shift
  mixers        'hgrn2'              gated linear recurrence, the forget gate (bounded below per channel) also
                                     scales what is written; unit-RMS per head on the output
                'latent_attention'   keys and values from one cached latent per token plus one rotated key part
                                     shared by the heads; queries through a normed latent, interleaved rotation,
                                     sliding window, a sink in the softmax, sigmoid output gate
                'latent_attention_2' the same cache; direct queries, rotation of halves, causal, plain softmax
  feed-forward  routed SwiGLU experts (top-k of the router logits, softmax over the chosen) plus a shared
                expert scaled by a sigmoid of one number per token; or none
  token side    after the feed-forward a slice of a second embedding table enters through a GELU-gated low-rank
                path and a unit-RMS norm
The residual stream is fp32.

This module holds the configuration (every size and constant is read from config.json), the tensor names and a
random-weight builder for tests and benchmarks.  The compute path is core/layer/ragged_runner.py.
"""
import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch

from .pagazen import PagazenModel

MIXERS = ("hgrn2", "latent_attention", "latent_attention_2")


@dataclass
class FagunexConfig:
    vocab_size: int
    width: int
    layers: List[dict]
    eps: float = 1e-6
    loop: Optional[dict] = None          # {"start", "stop", "times"}
    side_dim: int = 0                    # width of a layer's slice of the second embedding table (0: none)
    name: str = "fagunex"
    architecture: str = "Fagunex"
    family: str = "ragged"
    raw: dict = field(default_factory=dict, repr=False)

    @property
    def hidden_size(self):
        return self.width

    @property
    def num_hidden_layers(self):
        return len(self.runs)

    @property
    def max_position_embeddings(self):
        return 1 << 20

    @property
    def runs(self) -> List[int]:
        """The layer each layer RUN takes its tensors from, in running order."""
        n = len(self.layers)
        if not self.loop:
            return list(range(n))
        a, b, times = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        return list(range(a)) + list(range(a, b)) * times + list(range(b, n))

    def layer_runs(self):
        """[(index of the layer whose tensors the run uses, its description)] in running order."""
        return [(i, self.layers[i]) for i in self.runs]

    @classmethod
    def from_json(cls, d: dict, name: str = "fagunex") -> "FagunexConfig":
        layers = d["layers"]
        for i, layer in enumerate(layers):
            if layer["type"] not in MIXERS:
                raise ValueError(f"layer {i}: unknown mixer type {layer['type']!r}")
            mlp = layer.get("mlp")
            if mlp is not None and mlp.get("kind") != "moe":
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            m = layer["mixer"]
            if layer["type"] != "hgrn2":
                rot = m.get("rot") or {"dims": 0}
                if int(rot["dims"]) > int(m["rot_dim"]) or int(rot["dims"]) % 2:
                    raise ValueError(f"layer {i}: rotation over {rot['dims']} of {m['rot_dim']} dimensions")
        loop = d.get("loop")
        if loop:
            a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
            if not (0 <= a <= b <= len(layers)) or times < 1:
                raise ValueError(f"loop {loop!r} does not fit {len(layers)} layers")
        side = d.get("token_side")
        return cls(vocab_size=int(d["vocab"]), width=int(d["width"]), layers=layers, eps=float(d["norm"]["eps"]),
                   loop=loop, side_dim=int(side["dim"]) if side else 0, name=name, raw=d)

    def to_json(self) -> dict:
        d = {"architecture": self.architecture, "layers": self.layers, "norm": {"eps": self.eps},
             "vocab": self.vocab_size, "width": self.width}
        if self.loop:
            d["loop"] = self.loop
        if self.side_dim:
            d["token_side"] = {"dim": self.side_dim}
        return d


def tensor_shapes(cfg: FagunexConfig) -> Dict[str, tuple]:
    """Name -> shape of every tensor a checkpoint of this configuration holds."""
    W = cfg.width
    out = {"embed": (cfg.vocab_size, W), "head": (cfg.vocab_size, W)}

    def norm(prefix):
        out.update({prefix: (W,), prefix + ".b": (W,), prefix + ".alpha": ()})

    norm("final.norm")
    if cfg.side_dim:
        out["side.embed"] = (cfg.vocab_size, len(cfg.layers) * cfg.side_dim)
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.", layer["mixer"]
        norm(p + "norm1")
        norm(p + "norm1b")
        out[p + "shift"] = (W,)
        H = int(m["heads"])
        if layer["type"] == "hgrn2":
            n, pv = int(m["dim"]), int(m["vdim"])
            out.update({p + "mix.q": (H * n, W), p + "mix.f": (H * n, W), p + "mix.f.b": (H * n,),
                        p + "mix.lower": (H * n,), p + "mix.v": (H * pv, W), p + "mix.norm": (pv,),
                        p + "mix.o": (W, H * pv)})
        else:
            d, r, dv, R = int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
            if layer["type"] == "latent_attention":
                Q = int(m["q_rank"])
                out.update({p + "mix.dq": (Q, W), p + "mix.dq.norm": (Q,), p + "mix.uq": (H * (d + r), Q),
                            p + "mix.sink": (H,), p + "mix.g": (H * dv, W)})
            else:
                out[p + "mix.q"] = (H * (d + r), W)
            out.update({p + "mix.dkv": (R + r, W), p + "mix.dkv.norm": (R,), p + "mix.uk": (H * d, R),
                        p + "mix.uv": (H * dv, R), p + "mix.o": (W, H * dv)})
        mlp = layer.get("mlp")
        if mlp:
            norm(p + "norm2")
            norm(p + "norm2b")
            ff, E = int(mlp["expert"]["ff"]), int(mlp["router"]["experts"])
            out[p + "mlp.router"] = (E, W)
            for e in range(E):
                out.update({p + f"mlp.e{e}.gate": (ff, W), p + f"mlp.e{e}.up": (ff, W), p + f"mlp.e{e}.down": (W, ff)})
            if mlp.get("shared"):
                sf = int(mlp["shared"]["ff"])
                out.update({p + "mlp.shared.gate": (sf, W), p + "mlp.shared.up": (sf, W),
                            p + "mlp.shared.down": (W, sf), p + "mlp.shared.sg": (1, W)})
        if cfg.side_dim:
            out.update({p + "side.gate": (cfg.side_dim, W), p + "side.proj": (W, cfg.side_dim), p + "side.norm": (W,)})
    return out


class FagunexModel(PagazenModel):
    """Configuration plus a name -> tensor source (`get(name)`): a checkpoint's files or a dict."""


def random_weights(cfg: FagunexConfig, seed: int = 0, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random tensors of the right shapes and sensible ranges (projections ~ 1/sqrt(fan-in), norm weights near
    one, lower bounds of the forget gates spread over (0, 1), sinks and biases of order one)."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if name.endswith(".alpha"):
            t = torch.rand(shape, generator=g) * 0.5 + 0.5
        elif name.endswith("mix.lower"):
            t = torch.rand(shape, generator=g) * 0.9
        elif name.endswith(".shift"):
            t = torch.rand(shape, generator=g)
        elif name.endswith(".sink") or name.endswith("f.b"):
            t = torch.randn(shape, generator=g)
        elif len(shape) == 2 and name not in ("embed", "side.embed"):
            t = torch.randn(shape, generator=g) / math.sqrt(shape[1])
            if name.endswith("mlp.router"):
                t = t * 4.0          # logits spread enough that the choice of experts is no close call
        elif len(shape) == 2:
            t = torch.randn(shape, generator=g)
        elif name.endswith(".b"):
            t = torch.randn(shape, generator=g) * 0.1
        else:
            t = 1.0 + torch.randn(shape, generator=g) * 0.1
        out[name] = t.to(dtype)
    return out


def build_random_model(cfg: FagunexConfig, seed: int = 0) -> FagunexModel:
    return FagunexModel(cfg, random_weights(cfg, seed))


def bench_config(width: int, n_layers: int, vocab: int = 32000, ff_mult: int = 4, every: int = 4, experts: int = 8,
                 top: int = 2) -> FagunexConfig:
    """A configuration with the proportions of a served model: every `every`-th layer a latent attention
    (alternately the windowed and the causal kind), the others hgrn2; routed experts whose active
    feed-forward width (top experts + the shared one) is ff_mult * width."""
    layers = []
    ff = (ff_mult * width // (top + 1) + 63) // 64 * 64
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}, "shared": {"ff": ff}}
    k = 0
    for i in range(n_layers):
        if i % every == every - 1:
            mixer = {"heads": width // 128, "dim": 128, "rot_dim": 64, "vdim": 128, "kv_rank": 512,
                     "rot": {"base": 10000.0, "dims": 64}, "scale": 192 ** -0.5}
            if k % 2 == 0:
                mixer.update({"q_rank": max(256, width // 2), "mask": {"size": 1024}})
            layers.append({"type": "latent_attention" if k % 2 == 0 else "latent_attention_2", "mixer": mixer,
                           "mlp": mlp})
            k += 1
        else:
            layers.append({"type": "hgrn2", "mixer": {"heads": width // 128, "dim": 128, "vdim": 128}, "mlp": mlp})
    return FagunexConfig(vocab_size=vocab, width=width, layers=layers, eps=1e-6, loop=None, side_dim=64,
                         name=f"fagunex-w{width}-l{n_layers}")
