"""Kabidra: a decoder stack that mixes gated recurrences (minGRU) and latent attention.

Per layer, with x the float32 residual stream:
    x <- x + N(mixer(C(N(x))))      x <- x + N(ff(C(N(x))))      (the second line only for layers with a feed-forward)
N is an RMS norm whose stored weight is the deviation from one, C adds a short causal convolution over time to its
input (per channel; the last taps - 1 inputs of every sequence are state), ff = W_down relu(W_up h)^2.  What a layer
hands on is a learned weighted sum of the embedding output and the results of all layers up to itself.  The embedding
is normed, so is the last stream before the LM head.  config.json gives the sizes, the order of the layers and the
constants (`norm.eps`, `canon.taps`, each mixer's sizes and scale); nothing is fixed here but the equations.

Between the matrix products (library GEMMs) every step is a HIP kernel of this package: ops.boundary_norm (post-norm +
residual + depth sum + next pre-norm, one launch per sublayer boundary), ops.canon_conv, ops.mingru_scan,
ops.latent_prep / ops.latent_attn, ops.relu2.  Norms, residual stream, recurrent state, gates of the recurrence,
attention scores and weights are float32 in every activation format.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Iterable

import torch
import torch.nn.functional as F
from torch import nn

from . import distributed as tpd
from . import ops
from .layers.latent_attention import LatentAttention
from .layers.recurrent import MinGRU

MIXERS = ("mingru", "latent_attention")


@dataclass
class KabidraConfig:
    vocab_size: int
    width: int
    eps: float
    taps: int
    layers: list = field(default_factory=list)     # per layer: {"type", "mixer": {...}, "mlp": {"kind", "ff"} | None}
    torch_dtype: str = "bfloat16"
    architecture: str = "Kabidra"

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: dict) -> "KabidraConfig":
        layers = []
        for i, layer in enumerate(d["layers"]):
            kind, m, mlp = layer["type"], dict(layer["mixer"]), layer.get("mlp")
            if kind == "mingru":
                m = {"width": int(m["width"])}
            elif kind == "latent_attention":
                m = {"heads": int(m["heads"]), "dim": int(m["dim"]), "vdim": int(m["vdim"]), "q_rank": int(m["q_rank"]),
                     "kv_rank": int(m["kv_rank"]), "scale": float(m["scale"])}
            else:
                raise ValueError(f"layer {i}: unknown mixer {kind!r} (known: {MIXERS})")
            if mlp is not None:
                if mlp.get("kind") != "dense":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
                mlp = {"kind": "dense", "ff": int(mlp["ff"])}
            layers.append({"type": kind, "mixer": m, "mlp": mlp})
        return cls(vocab_size=int(d["vocab"]), width=int(d["width"]), eps=float(d["norm"]["eps"]), taps=int(d["canon"]["taps"]),
                   layers=layers, torch_dtype=d.get("torch_dtype", d.get("dtype", "bfloat16")))

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.width, "norm": {"eps": self.eps},
                "canon": {"taps": self.taps}, "layers": self.layers}


def _f32(*shape):
    return nn.Parameter(torch.zeros(*shape, dtype=torch.float32))


class SquaredReLUMLP(nn.Module):
    def __init__(self, width: int, ff: int):
        super().__init__()
        self.up_proj = nn.Linear(width, ff, bias=False)
        self.down_proj = nn.Linear(ff, width, bias=False)

    def forward(self, h):
        return self.down_proj(ops.relu2(self.up_proj(h)))


class KabidraLayer(nn.Module):
    def __init__(self, cfg: KabidraConfig, i: int):
        super().__init__()
        spec = cfg.layers[i]
        w, m = cfg.width, spec["mixer"]
        self.kind = spec["type"]
        if self.kind == "mingru":
            self.mixer = MinGRU(w, m["width"], state_name=(i, "gru"))
        else:
            self.mixer = LatentAttention(w, m["heads"], m["dim"], m["vdim"], m["q_rank"], m["kv_rank"], m["scale"], cfg.eps, layer_id=i)
        self.mlp = SquaredReLUMLP(w, spec["mlp"]["ff"]) if spec["mlp"] is not None else None
        # norm weights are stored as deviations from one; norms, taps and depth weights stay float32 in every format
        # (the taps are kept as (taps, width): a tap's weights for neighbouring channels are neighbours in memory)
        self.norm1, self.norm1b, self.canon1 = _f32(w), _f32(w), _f32(cfg.taps, w)
        if self.mlp is not None:
            self.norm2, self.norm2b, self.canon2 = _f32(w), _f32(w), _f32(cfg.taps, w)
        self.dwa = _f32(i + 2)


class KabidraForCausalLM(nn.Module):
    family = "seq_state"       # what kind of cache and step metadata the runner builds for this model

    def __init__(self, cfg: KabidraConfig):
        super().__init__()
        if tpd.tp_size() * tpd.pp_size() != 1:
            raise NotImplementedError("Kabidra runs on one rank: its recurrent state and latent cache are not sharded")
        self.config = cfg
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, cfg.width))
        self.embed_norm = _f32(cfg.width)
        self.layers = nn.ModuleList(KabidraLayer(cfg, i) for i in range(len(cfg.layers)))
        self.final_norm = _f32(cfg.width)
        self.head = nn.Parameter(torch.empty(cfg.vocab_size, cfg.width))
        self.metadata = None
        self.start_layer, self.end_layer = 0, len(cfg.layers)

    # -- what the runner asks -------------------------------------------------------------------------
    def finalize(self):
        pass

    def pack_decode_weights(self):
        pass

    def set_attention_metadata(self, metadata):
        self.metadata = metadata

    def latent_ranks(self) -> dict:
        return {i: l.mixer.kv_rank for i, l in enumerate(self.layers) if l.kind == "latent_attention"}

    def state_shapes(self) -> dict:
        cfg, shapes = self.config, {}
        for i, l in enumerate(self.layers):
            if cfg.taps > 1:
                shapes[(i, "canon1")] = (cfg.taps - 1, cfg.width)
                if l.mlp is not None:
                    shapes[(i, "canon2")] = (cfg.taps - 1, cfg.width)
            if l.kind == "mingru":
                shapes.update(l.mixer.state_shapes())
        return shapes

    # -- forward ----------------------------------------------------------------------------------------
    def _canon(self, hn, taps, name, md, dtype):
        state = md.cache.state(name) if self.config.taps > 1 else None
        return ops.canon_conv(hn, taps, state, md.layout, dtype)

    def _boundary(self, y, post, x, md, dtype, pre, taps, name, **hist):
        """A sublayer boundary and the convolution in front of the next sublayer: (new stream, that sublayer's input).  A
        step with one token per sequence takes both in one launch; otherwise the convolution, which reads the pre-normed
        rows of a token's predecessors, is a launch of its own."""
        eps = self.config.eps
        if md.layout.qo_indptr is None and ops.boundary_canon_fits(self.config.width):
            state = md.cache.state(name) if self.config.taps > 1 else None
            return ops.boundary_norm(y, post, eps, res=x, w_pre=pre, canon=(taps, state, md.layout), **hist)
        x, hn = ops.boundary_norm(y, post, eps, res=x, w_pre=pre, **hist)
        return x, self._canon(hn, taps, name, md, dtype)

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """Final-normed hidden states (tokens, width) in the activations' format.  Positions enter nowhere: the order of a
        sequence's tokens is in its state and in the causal mask."""
        md, cfg = self.metadata, self.config
        assert md is not None
        eps, n_layers, dtype = cfg.eps, len(self.layers), self.embed.dtype
        t = input_ids.numel()
        hist = torch.empty((n_layers + 1, t, cfg.width), dtype=torch.float32, device=input_ids.device)
        emb = F.embedding(input_ids, self.embed)
        if n_layers == 0:
            return ops.boundary_norm(emb, self.embed_norm, eps, w_pre=self.final_norm, pre_f32=False)[1]
        x, h = self._boundary(emb, self.embed_norm, None, md, dtype, self.layers[0].norm1, self.layers[0].canon1, (0, "canon1"),
                              hist=hist, hist_slot=0)
        for i, layer in enumerate(self.layers):
            y = layer.mixer(h, md)
            post = layer.norm1b
            if layer.mlp is not None:
                x, h = self._boundary(y, layer.norm1b, x, md, dtype, layer.norm2, layer.canon2, (i, "canon2"))
                y = layer.mlp(h)
                post = layer.norm2b
            if i + 1 == n_layers:
                return ops.boundary_norm(y, post, eps, res=x, hist=hist, hist_slot=i + 1, mix=layer.dwa, w_pre=self.final_norm,
                                         pre_f32=False)[1]
            nxt = self.layers[i + 1]
            x, h = self._boundary(y, post, x, md, dtype, nxt.norm1, nxt.canon1, (i + 1, "canon1"), hist=hist, hist_slot=i + 1, mix=layer.dwa)

    def compute_logits(self, hidden_states: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden_states, self.head)

    # -- weights ----------------------------------------------------------------------------------------
    @torch.no_grad()
    def load_weights(self, weights: Iterable):
        """Checkpoint tensors under the design's names ('embed', 'l<i>.mix.z', ...) -> the fused parameters."""
        got = set()
        for name, w in weights:
            self._load_one(name, w)
            got.add(name)
        missing = [n for n in checkpoint_names(self.config) if n not in got]
        if missing:
            raise KeyError(f"checkpoint lacks {len(missing)} tensors, e.g. {missing[:4]}")

    def _load_one(self, name: str, w: torch.Tensor):
        def put(p, rows=None):
            dst = p if rows is None else p[rows[0]:rows[1]]
            if dst.shape != w.shape:
                raise ValueError(f"{name}: checkpoint shape {tuple(w.shape)}, model wants {tuple(dst.shape)}")
            dst.copy_(w)

        top = {"embed": self.embed, "embed.norm": self.embed_norm, "final.norm": self.final_norm, "head": self.head}
        if name in top:
            return put(top[name])
        head, _, rest = name.partition(".")
        if not (head[:1] == "l" and head[1:].isdigit() and int(head[1:]) < len(self.layers)):
            raise KeyError(f"unexpected tensor {name!r}")
        layer = self.layers[int(head[1:])]
        if rest in ("canon1", "canon2") and hasattr(layer, rest):
            w = w.t()                        # stored (width, taps), kept (taps, width)
            return put(getattr(layer, rest))
        if rest in ("norm1", "norm1b", "norm2", "norm2b", "dwa") and hasattr(layer, rest):
            return put(getattr(layer, rest))
        if rest == "mlp.up" and layer.mlp is not None:
            return put(layer.mlp.up_proj.weight)
        if rest == "mlp.down" and layer.mlp is not None:
            return put(layer.mlp.down_proj.weight)
        m = layer.mixer
        if layer.kind == "mingru":
            n = m.inner
            where = {"mix.z": (m.zxg_proj.weight, (0, n)), "mix.x": (m.zxg_proj.weight, (n, 2 * n)), "mix.g": (m.zxg_proj.weight, (2 * n, 3 * n)),
                     "mix.z.b": (m.zxg_proj.bias, (0, n)), "mix.x.b": (m.zxg_proj.bias, (n, 2 * n)), "mix.o": (m.o_proj.weight, None)}
            if rest in where:
                if rest == "mix.g":
                    m.zxg_proj.bias[2 * n:].zero_()
                return put(*where[rest])
        else:
            a, b = m.q_rank, m.q_rank + m.kv_rank
            where = {"mix.dq": (m.down_proj.weight, (0, a)), "mix.dkv": (m.down_proj.weight, (a, b)), "mix.g": (m.down_proj.weight, (b, b + m.heads)),
                     "mix.dq.norm": (m.q_norm, None), "mix.dkv.norm": (m.kv_norm, None), "mix.uq": (m.uq_proj.weight, None),
                     "mix.o": (m.o_proj.weight, None)}
            if rest in where:
                return put(*where[rest])
            if rest == "mix.uk":
                w = w.view(m.heads, m.dim, m.kv_rank)
                return put(m.uk)
            if rest == "mix.uv":
                w = w.view(m.heads, m.vdim, m.kv_rank)
                return put(m.uv)
        raise KeyError(f"unexpected tensor {name!r}")

    @torch.no_grad()
    def init_random(self, seed: int = 0):
        self.load_weights(random_checkpoint(self.config, seed))


def checkpoint_shapes(cfg: KabidraConfig) -> dict:
    """name -> shape of every tensor of a checkpoint of this configuration."""
    w, shapes = cfg.width, {"embed": (cfg.vocab_size, cfg.width), "embed.norm": (cfg.width,)}
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.", layer["mixer"]
        shapes[p + "norm1"] = shapes[p + "norm1b"] = (w,)
        shapes[p + "canon1"] = (w, cfg.taps)
        if layer["type"] == "mingru":
            n = m["width"]
            shapes.update({p + "mix.z": (n, w), p + "mix.z.b": (n,), p + "mix.x": (n, w), p + "mix.x.b": (n,), p + "mix.g": (n, w),
                           p + "mix.o": (w, n)})
        else:
            hd, hv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            shapes.update({p + "mix.dq": (m["q_rank"], w), p + "mix.dq.norm": (m["q_rank"],), p + "mix.uq": (hd, m["q_rank"]),
                           p + "mix.dkv": (m["kv_rank"], w), p + "mix.dkv.norm": (m["kv_rank"],), p + "mix.uk": (hd, m["kv_rank"]),
                           p + "mix.uv": (hv, m["kv_rank"]), p + "mix.g": (m["heads"], w), p + "mix.o": (w, hv)})
        if layer["mlp"] is not None:
            shapes[p + "norm2"] = shapes[p + "norm2b"] = (w,)
            shapes[p + "canon2"] = (w, cfg.taps)
            shapes[p + "mlp.up"] = (layer["mlp"]["ff"], w)
            shapes[p + "mlp.down"] = (w, layer["mlp"]["ff"])
        shapes[p + "dwa"] = (i + 2,)
    shapes["final.norm"] = (w,)
    shapes["head"] = (cfg.vocab_size, w)
    return shapes


def checkpoint_names(cfg: KabidraConfig) -> list:
    return list(checkpoint_shapes(cfg))


def random_checkpoint(cfg: KabidraConfig, seed: int = 0):
    """(name, tensor) pairs of a seeded random checkpoint, rounded to bfloat16 values (as a stored checkpoint is), one
    tensor at a time.  Matrices are scaled by 1/sqrt(fan-in); norm weights, taps and biases are small; the depth weights
    put most of their mass on the newest result."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    for name, shape in checkpoint_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        if leaf == "dwa":
            w = 0.1 * torch.randn(shape, generator=gen)
            w[-1] += 0.9
        elif leaf in ("norm", "norm1", "norm1b", "norm2", "norm2b") and not name.endswith(("dq.norm", "dkv.norm")):
            w = 0.1 * torch.randn(shape, generator=gen)
        elif name.endswith(("dq.norm", "dkv.norm")):
            w = 1.0 + 0.1 * torch.randn(shape, generator=gen)
        elif leaf in ("canon1", "canon2"):
            w = 0.2 * torch.randn(shape, generator=gen)
        elif leaf == "b":
            w = 0.5 * torch.randn(shape, generator=gen)
        elif name == "embed":
            w = torch.randn(shape, generator=gen)
        else:
            w = torch.randn(shape, generator=gen) * shape[-1] ** -0.5
        yield name, w.to(torch.bfloat16).float()
