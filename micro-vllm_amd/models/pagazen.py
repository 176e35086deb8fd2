"""Pagazen: a decoder-only stack whose layers are listed one by one in config.json.  Each layer has a
token mixer - 'mamba2' (a state-space-duality head group behind a short convolution) or 'parallel'
(sliding-window softmax attention with a linear distance penalty beside fixed-decay retention with
rotary positions, summed with two scales) - and an optional dense feed-forward with a squared-ReLU.
The residual stream is fp32; the RMS norm sits on each sublayer's OUTPUT with its weight stored as an
offset from one; a layer may reuse an earlier layer's weights with a cache and state of its own.

This module holds the configuration (every size and constant is read from config.json), the tensor
names, and a random-weight builder for tests and benchmarks.  The compute path is
core/layer/ragged_runner.py.
"""
import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch

MIXERS = ("mamba2", "parallel")


@dataclass
class PagazenConfig:
    vocab_size: int
    width: int
    layers: List[dict]
    embed_scale: float = 1.0
    eps: float = 1e-6
    logit_softcap: Optional[float] = None
    name: str = "pagazen"
    architecture: str = "Pagazen"
    family: str = "ragged"
    raw: dict = field(default_factory=dict, repr=False)

    # the names the engine and the HTTP front end read
    @property
    def hidden_size(self):
        return self.width

    @property
    def num_hidden_layers(self):
        return len(self.layers)

    @property
    def max_position_embeddings(self):
        return 1 << 20

    def weights_layer(self, i: int) -> int:
        """The layer whose tensors layer run i uses."""
        j = self.layers[i].get("weights_of", i)
        return i if j is None else int(j)

    def layer_runs(self):
        """[(index of the layer whose tensors the run uses, its description)] in running order."""
        return [(self.weights_layer(i), layer) for i, layer in enumerate(self.layers)]

    @classmethod
    def from_json(cls, d: dict, name: str = "pagazen") -> "PagazenConfig":
        layers = d["layers"]
        for i, layer in enumerate(layers):
            if layer["type"] not in MIXERS:
                raise ValueError(f"layer {i}: unknown mixer type {layer['type']!r}")
            mlp = layer.get("mlp")
            if mlp is not None and mlp.get("kind") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            j = layer.get("weights_of")
            if j is not None and not (0 <= int(j) < len(layers) and layers[int(j)].get("weights_of") is None):
                raise ValueError(f"layer {i}: weights_of {j!r} does not name a layer with tensors of its own")
        return cls(vocab_size=int(d["vocab"]), width=int(d["width"]), layers=layers,
                   embed_scale=float(d.get("embedding", {}).get("scale", 1.0)), eps=float(d["norm"]["eps"]),
                   logit_softcap=(float(d["logit_softcap"]) if d.get("logit_softcap") else None), name=name, raw=d)

    def to_json(self) -> dict:
        d = {"architecture": self.architecture, "embedding": {"scale": self.embed_scale}, "layers": self.layers,
             "norm": {"eps": self.eps}, "vocab": self.vocab_size, "width": self.width}
        if self.logit_softcap:
            d["logit_softcap"] = self.logit_softcap
        return d


def mamba2_sizes(m: dict):
    heads, p, n, g = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"])
    inner = heads * p
    return dict(heads=heads, p=p, n=n, groups=g, inner=inner, conv_ch=inner + 2 * g * n,
                proj=2 * inner + 2 * g * n + heads, taps=int(m["conv"]), norm_groups=int(m["norm_groups"]))


def tensor_shapes(cfg: PagazenConfig) -> Dict[str, tuple]:
    """Name -> shape of every tensor a checkpoint of this configuration holds."""
    W = cfg.width
    out = {"embed": (cfg.vocab_size, W), "final.norm": (W,), "head": (cfg.vocab_size, W)}
    for i, layer in enumerate(cfg.layers):
        if layer.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (W,)
        if layer["type"] == "mamba2":
            s = mamba2_sizes(m)
            out.update({p + "mix.in": (s["proj"], W), p + "mix.conv": (s["conv_ch"], s["taps"]),
                        p + "mix.conv.b": (s["conv_ch"],), p + "mix.dt_bias": (s["heads"],),
                        p + "mix.A_log": (s["heads"],), p + "mix.D": (s["heads"],),
                        p + "mix.norm": (s["inner"],), p + "mix.o": (W, s["inner"])})
        else:
            L, R = m["left"], m["right"]
            out.update({p + "mix.left.q": (L["heads"] * L["dim"], W), p + "mix.left.k": (L["kv_heads"] * L["dim"], W),
                        p + "mix.left.v": (L["kv_heads"] * L["vdim"], W), p + "mix.left.o": (W, L["heads"] * L["vdim"]),
                        p + "mix.right.q": (R["heads"] * R["dim"], W), p + "mix.right.k": (R["heads"] * R["dim"], W),
                        p + "mix.right.v": (R["heads"] * R["vdim"], W), p + "mix.right.g": (R["heads"] * R["vdim"], W),
                        p + "mix.right.o": (W, R["heads"] * R["vdim"])})
        if layer.get("mlp"):
            ff = int(layer["mlp"]["ff"])
            out.update({p + "norm2": (W,), p + "mlp.up": (ff, W), p + "mlp.down": (W, ff)})
    return out


class PagazenModel:
    """Configuration plus a name -> tensor source (`get(name)`): a checkpoint's files or a dict."""
    family = "ragged"

    def __init__(self, config: PagazenConfig, source):
        self.config, self._source = config, source

    def get(self, name: str) -> torch.Tensor:
        if isinstance(self._source, dict):
            return self._source[name]
        return self._source.get(name, dtype=None)

    def names(self):
        return self._source.keys() if isinstance(self._source, dict) else self._source.names()

    def eval(self):
        return self


def random_weights(cfg: PagazenConfig, seed: int = 0, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random tensors of the right shapes and sensible ranges (projections ~ 1/sqrt(fan-in), norm
    offsets and biases small, A_log and dt_bias so that decays spread over (0, 1))."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if len(shape) == 2 and not name.endswith("mix.conv"):
            t = torch.randn(shape, generator=g) / math.sqrt(shape[1])
            if name == "embed":
                t = torch.randn(shape, generator=g) / max(cfg.embed_scale, 1.0)
        elif name.endswith("mix.conv"):
            t = torch.randn(shape, generator=g) * 0.5
        elif name.endswith("A_log"):
            t = torch.rand(shape, generator=g) * 2.0 - 1.5
        elif name.endswith("dt_bias"):
            t = torch.rand(shape, generator=g) * 3.0 - 3.0
        elif name.endswith(".D"):
            t = torch.randn(shape, generator=g) * 0.5
        else:
            t = torch.randn(shape, generator=g) * 0.1
        out[name] = t.to(dtype)
    return out


def build_random_model(cfg: PagazenConfig, seed: int = 0) -> PagazenModel:
    return PagazenModel(cfg, random_weights(cfg, seed))


def bench_config(width: int, n_layers: int, vocab: int = 32000, ff_mult: int = 4, every: int = 4) -> PagazenConfig:
    """A configuration with the proportions of a served model: head width 64/128, every `every`-th
    layer a parallel mixer, the others mamba2."""
    heads = width // 64
    layers = []
    for i in range(n_layers):
        if i % every == every - 1:
            mixer = {"left": {"dim": 128, "vdim": 128, "heads": width // 128, "kv_heads": max(1, width // 512),
                              "mask": {"size": 1024}, "scale": 128 ** -0.5},
                     "right": {"dim": 128, "vdim": 64, "heads": max(1, width // 256), "rot": {"base": 10000.0, "dims": 64},
                               "decay": [1.0 - 2.0 ** (-5 - j % 4) for j in range(max(1, width // 256))]},
                     "left_scale": 1.0, "right_scale": 1.0}
            layers.append({"type": "parallel", "mixer": mixer, "mlp": {"kind": "dense", "ff": ff_mult * width}})
        else:
            mixer = {"conv": 4, "groups": 1, "heads": 2 * heads, "norm_groups": 1, "state": 128, "vdim": 64}
            layers.append({"type": "mamba2", "mixer": mixer, "mlp": {"kind": "dense", "ff": ff_mult * width}})
    return PagazenConfig(vocab_size=vocab, width=width, layers=layers, embed_scale=1.0, eps=1e-5,
                         logit_softcap=30.0, name=f"pagazen-w{width}-l{n_layers}")
