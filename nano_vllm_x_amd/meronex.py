"""Meronex: a decoder stack whose layers mix tokens in one of three ways -- a matrix memory with exponential gating
(mlstm), a gated delta rule behind short convolutions (delta), or softmax attention and an RWKV-style recurrence side by
side (parallel) -- each followed by a mixture of small experts.

With x the float32 residual stream, N a grouped RMS norm (a row is cut into `norm.groups` slices, each divided by its own
root mean square) and c = residual_mult:
    h = N1(x);  x <- x + c * mixer(h) * sigmoid(W_rg1 h + b_rg1)
    h = N2(x);  x <- x + c * ff(h)    * sigmoid(W_rg2 h + b_rg2)          (only for layers with a feed-forward)
and the logits are head(N_final(x)).  The parallel mixer returns the mean of its two branches after each was divided by
its root mean square over the width and multiplied by a weight of its own.

config.json gives every size, the order of the layers and the constants; the mechanisms live in layers/ (recurrent.py,
cap_attention.py, moe.py) with their constants as arguments.  Between the matrix products (library GEMMs) every step is a
HIP kernel of this package; one launch per sublayer boundary takes the gate, the residual add and the next norm
(ops.gated_residual_norm).  Norms, the stream, recurrent state, the gates of the recurrences, routers, attention scores and
positions are float32 in every activation format.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Iterable

import torch
import torch.nn.functional as F
from torch import nn

from . import distributed as tpd
from . import ops
from .layers.cap_attention import SoftcapAttention
from .layers.moe import SigmoidInputMoE
from .layers.recurrent import MLSTM, GatedDelta, TimeMix

MIXERS = ("mlstm", "delta", "parallel")
EXPERT_SIGMOID_SLOPE = 1.702      # y = g * sigmoid(1.702 g) * (u + 1)


def _attention_spec(m: dict) -> dict:
    rot = m.get("rot")
    if rot is not None:
        sc = rot.get("scaling")
        rot = {"dims": int(rot["dims"]), "base": float(rot["base"]),
               "scaling": None if not sc else {k: float(sc[k]) for k in ("factor", "original", "fast", "slow")}}
    return {"heads": int(m["heads"]), "kv_heads": int(m.get("kv_heads", m["heads"])), "dim": int(m["dim"]), "vdim": int(m.get("vdim", m["dim"])),
            "rot": rot, "scale": float(m["scale"]), "softcap": float(m["softcap"]) if m.get("softcap") else None}


@dataclass
class MeronexConfig:
    vocab_size: int
    width: int
    eps: float
    groups: int
    residual_mult: float
    layers: list = field(default_factory=list)     # per layer: {"type", "mixer": {...}, "mlp": {...} | None}
    torch_dtype: str = "bfloat16"
    architecture: str = "Meronex"

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: dict) -> "MeronexConfig":
        layers = []
        for i, layer in enumerate(d["layers"]):
            kind, m, mlp = layer["type"], layer["mixer"], layer.get("mlp")
            if kind == "mlstm":
                m = {"heads": int(m["heads"]), "dim": int(m["dim"]), "vdim": int(m["vdim"]), "gate_cap": float(m["gate_cap"])}
            elif kind == "delta":
                m = {"heads": int(m["heads"]), "kv_heads": int(m.get("kv_heads", m["heads"])), "dim": int(m["dim"]), "vdim": int(m["vdim"]),
                     "conv": int(m["conv"])}
            elif kind == "parallel":
                # the inner size of the decay's two small projections is a tensor's shape in a checkpoint; "decay_rank" only
                # sizes a model that is built without one
                m = {"left": _attention_spec(m["left"]), "right": {"heads": int(m["right"]["heads"]), "dim": int(m["right"]["dim"]),
                                                                   "decay_rank": int(m["right"].get("decay_rank", 16))}}
            else:
                raise ValueError(f"layer {i}: unknown mixer {kind!r} (known: {MIXERS})")
            if mlp is not None:
                if mlp.get("kind") != "moe":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
                mlp = {"kind": "moe", "expert": {"ff": int(mlp["expert"]["ff"]), "limit": float(mlp["expert"]["limit"])},
                       "router": {"experts": int(mlp["router"]["experts"]), "top": int(mlp["router"]["top"])}}
            layers.append({"type": kind, "mixer": m, "mlp": mlp})
        return cls(vocab_size=int(d["vocab"]), width=int(d["width"]), eps=float(d["norm"]["eps"]), groups=int(d["norm"].get("groups", 1)),
                   residual_mult=float(d.get("residual_mult", 1.0)), layers=layers, torch_dtype=d.get("torch_dtype", d.get("dtype", "bfloat16")))

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.width, "norm": {"eps": self.eps, "groups": self.groups},
                "residual_mult": self.residual_mult, "layers": self.layers}


def _f32(*shape):
    return nn.Parameter(torch.zeros(*shape, dtype=torch.float32))


class ParallelMixer(nn.Module):
    """Attention (left) and time mixing (right) on the same input; the boundary kernel norms and averages the two results."""

    def __init__(self, width: int, m: dict, eps: float, i: int):
        super().__init__()
        a, r = m["left"], m["right"]
        self.left = SoftcapAttention(width, a["heads"], a["kv_heads"], a["dim"], a["vdim"], a["rot"], a["scale"], a["softcap"], eps,
                                     cache_names=((i, "k"), (i, "v")))
        self.right = TimeMix(width, r["heads"], r["dim"], r["decay_rank"], eps, state_name=(i, "mix"))
        self.left_out, self.right_out = _f32(width), _f32(width)


class MeronexLayer(nn.Module):
    def __init__(self, cfg: MeronexConfig, i: int):
        super().__init__()
        spec = cfg.layers[i]
        w, m = cfg.width, spec["mixer"]
        self.kind = spec["type"]
        if self.kind == "mlstm":
            self.mixer = MLSTM(w, m["heads"], m["dim"], m["vdim"], m["gate_cap"], cfg.eps, state_name=(i, "mix"))
        elif self.kind == "delta":
            self.mixer = GatedDelta(w, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"], cfg.eps, state_name=(i, "mix"))
        else:
            self.mixer = ParallelMixer(w, m, cfg.eps, i)
        self.norm1 = _f32(w)
        self.rg1, self.rg1_b = nn.Linear(w, w, bias=False), _f32(w)
        self.mlp = None
        if spec["mlp"] is not None:
            e, r = spec["mlp"]["expert"], spec["mlp"]["router"]
            self.mlp = SigmoidInputMoE(w, r["experts"], r["top"], e["ff"], e["limit"], EXPERT_SIGMOID_SLOPE)
            self.norm2 = _f32(w)
            self.rg2, self.rg2_b = nn.Linear(w, w, bias=False), _f32(w)


class MeronexForCausalLM(nn.Module):
    family = "seq_state"       # per-token cache rows + per-sequence state slots; ragged steps

    def __init__(self, cfg: MeronexConfig):
        super().__init__()
        if tpd.tp_size() * tpd.pp_size() != 1:
            raise NotImplementedError("Meronex runs on one rank: its recurrent state and token cache are not sharded")
        self.config = cfg
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, cfg.width))
        self.layers = nn.ModuleList(MeronexLayer(cfg, i) for i in range(len(cfg.layers)))
        self.final_norm = _f32(cfg.width)
        self.head = nn.Parameter(torch.empty(cfg.vocab_size, cfg.width))
        self.metadata = None
        self.layer_streams = None      # a list: forward() appends a copy of the residual stream after every layer (diagnostics)
        self.start_layer, self.end_layer = 0, len(cfg.layers)

    # -- what the runner asks -------------------------------------------------------------------------
    def finalize(self):
        pass

    def pack_decode_weights(self):
        pass

    def set_attention_metadata(self, metadata):
        self.metadata = metadata

    def latent_ranks(self) -> dict:
        """Rows of the per-token cache: name -> elements per token (the keys and values of every attention branch)."""
        rows = {}
        for l in self.layers:
            if l.kind == "parallel":
                rows.update(l.mixer.left.cache_rows())
        return rows

    def state_shapes(self) -> dict:
        shapes = {}
        for l in self.layers:
            shapes.update((l.mixer.right if l.kind == "parallel" else l.mixer).state_shapes())
        return shapes

    # -- forward ----------------------------------------------------------------------------------------
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """Final-normed hidden states (tokens, width) in the activations' format."""
        md, cfg = self.metadata, self.config
        assert md is not None
        eps, groups, mult, dtype = cfg.eps, cfg.groups, cfg.residual_mult, self.embed.dtype
        decode_step = md.layout.qo_indptr is None
        x = F.embedding(input_ids, self.embed).float()
        n_layers = len(self.layers)
        first = self.layers[0].norm1 if n_layers else self.final_norm
        h = ops.gated_residual_norm(x, w_norm=first, groups=groups, eps=eps, dtype=dtype)
        for i, layer in enumerate(self.layers):
            after = self.layers[i + 1].norm1 if i + 1 < n_layers else self.final_norm
            w_next = layer.norm2 if layer.mlp is not None else after
            gate = layer.rg1(h)
            if layer.kind == "parallel":
                mx = layer.mixer
                h = ops.gated_residual_norm(x, y=mx.left(h, positions, md), y2=mx.right(h, md), w_y=mx.left_out, w_y2=mx.right_out, gate=gate,
                                            gate_bias=layer.rg1_b, mult=mult, w_norm=w_next, groups=groups, eps=eps)
            else:
                h = ops.gated_residual_norm(x, y=layer.mixer(h, md), gate=gate, gate_bias=layer.rg1_b, mult=mult, w_norm=w_next, groups=groups,
                                            eps=eps)
            if layer.mlp is not None:
                h = ops.gated_residual_norm(x, y=layer.mlp(h, decode_step), gate=layer.rg2(h), gate_bias=layer.rg2_b, mult=mult, w_norm=after,
                                            groups=groups, eps=eps)
            if self.layer_streams is not None:
                self.layer_streams.append(x.clone())
        return h

    def compute_logits(self, hidden_states: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden_states, self.head)

    # -- weights ----------------------------------------------------------------------------------------
    @torch.no_grad()
    def load_weights(self, weights: Iterable):
        """Checkpoint tensors under the design's names ('embed', 'l<i>.mix.q', 'l<i>.mlp.e<j>.up', ...) -> the fused parameters."""
        got = set()
        for name, w in weights:
            self._load_one(name, w)
            got.add(name)
        missing = [n for n in checkpoint_names(self.config) if n not in got]
        if missing:
            raise KeyError(f"checkpoint lacks {len(missing)} tensors, e.g. {missing[:4]}")
        for i, l in enumerate(self.layers):
            if l.kind == "parallel" and l.mixer.right.w1.shape[0] != l.mixer.right.w2.shape[1]:
                raise ValueError(f"layer {i}: the decay's two projections disagree on their inner size")

    def _load_one(self, name: str, w: torch.Tensor):
        def put(p, rows=None):
            dst = p if rows is None else p[rows[0]:rows[1]]
            if dst.shape != w.shape:
                raise ValueError(f"{name}: checkpoint shape {tuple(w.shape)}, model wants {tuple(dst.shape)}")
            dst.copy_(w)

        top = {"embed": self.embed, "final.norm": self.final_norm, "head": self.head}
        if name in top:
            return put(top[name])
        head, _, rest = name.partition(".")
        if not (head[:1] == "l" and head[1:].isdigit() and int(head[1:]) < len(self.layers)):
            raise KeyError(f"unexpected tensor {name!r}")
        layer = self.layers[int(head[1:])]
        plain = {"norm1": "norm1", "rg1.b": "rg1_b", "norm2": "norm2", "rg2.b": "rg2_b"}
        if rest in plain and hasattr(layer, plain[rest]):
            return put(getattr(layer, plain[rest]))
        if rest in ("rg1", "rg2") and hasattr(layer, rest):
            return put(getattr(layer, rest).weight)
        if rest.startswith("mlp.") and layer.mlp is not None:
            moe, what = layer.mlp, rest[4:]
            if what == "router":
                return put(moe.router)
            e, _, part = what.partition(".")
            if e[:1] == "e" and e[1:].isdigit() and int(e[1:]) < moe.experts:
                j, ff = int(e[1:]), moe.ff
                where = {"gate": (moe.w_gu[j], (0, ff)), "up": (moe.w_gu[j], (ff, 2 * ff)), "down": (moe.w_d[j], None)}
                if part in where:
                    return put(*where[part])
        if rest in ("mix.right.w1", "mix.right.w2") and layer.kind == "parallel":
            # the decay's inner size comes with the checkpoint: the two parameters take the stored shapes
            r = layer.mixer.right
            ok = (w.dim() == 2 and w.shape[1] == r.w1.shape[1]) if rest.endswith("w1") else (w.dim() == 2 and w.shape[0] == r.w2.shape[0])
            if not ok:
                raise ValueError(f"{name}: checkpoint shape {tuple(w.shape)} does not fit the model")
            new = nn.Parameter(w.to(device=r.w0.device, dtype=torch.float32).contiguous(), requires_grad=False)
            if rest.endswith("w1"):
                r.w1 = new
            else:
                r.w2 = new
            return
        if rest.startswith("mix."):
            where = self._mixer_targets(layer).get(rest[4:])
            if where is not None:
                if where[2]:
                    w = w.t()
                return put(where[0], where[1])
        raise KeyError(f"unexpected tensor {name!r}")

    @staticmethod
    def _mixer_targets(layer) -> dict:
        """Checkpoint name below '<layer>.mix.' -> (parameter, row range or None, stored transposed)."""
        m = layer.mixer
        if layer.kind == "mlstm":
            hd, he, h = m.heads * m.dim, m.heads * m.vdim, m.heads
            p = m.qkvg_proj.weight
            return {"q": (p, (0, hd), False), "k": (p, (hd, 2 * hd), False), "v": (p, (2 * hd, 2 * hd + he), False),
                    "g": (p, (2 * hd + he, 2 * hd + 2 * he), False), "o": (m.o_proj.weight, None, False), "norm": (m.norm, None, False),
                    "i": (m.gate_w, (0, h), False), "f": (m.gate_w, (h, 2 * h), False), "i.b": (m.gate_b, (0, h), False),
                    "f.b": (m.gate_b, (h, 2 * h), False)}
        if layer.kind == "delta":
            gd, he, h, c = m.kv_heads * m.dim, m.heads * m.vdim, m.heads, m.conv_ch
            p = m.qkvg_proj.weight
            cw = m.conv_w
            return {"q": (p, (0, gd), False), "k": (p, (gd, 2 * gd), False), "v": (p, (2 * gd, c), False), "g": (p, (c, c + he), False),
                    "q.conv": (cw[:, 0:gd], None, True), "k.conv": (cw[:, gd:2 * gd], None, True), "v.conv": (cw[:, 2 * gd:c], None, True),
                    "a": (m.ab_w, (0, h), False), "b": (m.ab_w, (h, 2 * h), False), "A_log": (m.a_log, None, False),
                    "dt_bias": (m.dt_bias, None, False), "norm": (m.norm, None, False), "o": (m.o_proj.weight, None, False)}
        a, r = m.left, m.right
        qd, kd = a.heads * a.dim, a.kv_heads * a.dim
        p = a.qkv_proj.weight
        out = {"left.q": (p, (0, qd), False), "left.k": (p, (qd, qd + kd), False), "left.v": (p, (qd + kd, p.shape[0]), False),
               "left.o": (a.o_proj.weight, None, False), "left.out": (m.left_out, None, False), "right.out": (m.right_out, None, False),
               "right.w1": (r.w1, None, False), "right.w2": (r.w2, None, False), "right.w0": (r.w0, None, False),
               "right.u": (r.bonus, None, False), "right.norm": (r.norm, None, False), "right.o": (r.o_proj.weight, None, False)}
        for j, s in enumerate(TimeMix.MIXES):
            out["right.mu." + s] = (r.mu[j], None, False)
            if j < 4:
                out["right." + s] = (r.rkvg[j], None, False)
        return out

    @torch.no_grad()
    def init_random(self, seed: int = 0):
        self.load_weights(random_checkpoint(self.config, seed))


def checkpoint_shapes(cfg: MeronexConfig) -> dict:
    """name -> shape of every tensor of a checkpoint of this configuration."""
    w, shapes = cfg.width, {"embed": (cfg.vocab_size, cfg.width)}
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.", layer["mixer"]
        shapes[p + "norm1"] = (w,)
        shapes[p + "rg1"], shapes[p + "rg1.b"] = (w, w), (w,)
        if layer["type"] == "mlstm":
            h, hd, he = m["heads"], m["heads"] * m["dim"], m["heads"] * m["vdim"]
            shapes.update({p + "mix.q": (hd, w), p + "mix.k": (hd, w), p + "mix.v": (he, w), p + "mix.g": (he, w), p + "mix.o": (w, he),
                           p + "mix.norm": (he,), p + "mix.i": (h, w), p + "mix.i.b": (h,), p + "mix.f": (h, w), p + "mix.f.b": (h,)})
        elif layer["type"] == "delta":
            h, gd, he = m["heads"], m["kv_heads"] * m["dim"], m["heads"] * m["vdim"]
            shapes.update({p + "mix.q": (gd, w), p + "mix.q.conv": (gd, m["conv"]), p + "mix.k": (gd, w), p + "mix.k.conv": (gd, m["conv"]),
                           p + "mix.v": (he, w), p + "mix.v.conv": (he, m["conv"]), p + "mix.b": (h, w), p + "mix.A_log": (h,),
                           p + "mix.norm": (m["vdim"],), p + "mix.a": (h, w), p + "mix.dt_bias": (h,), p + "mix.g": (he, w), p + "mix.o": (w, he)})
        else:
            a, r = m["left"], m["right"]
            hd, rank = r["heads"] * r["dim"], r["decay_rank"]
            shapes.update({p + "mix.left.q": (a["heads"] * a["dim"], w), p + "mix.left.k": (a["kv_heads"] * a["dim"], w),
                           p + "mix.left.v": (a["kv_heads"] * a["vdim"], w), p + "mix.left.o": (w, a["heads"] * a["vdim"])})
            for s in TimeMix.MIXES:
                shapes[p + "mix.right.mu." + s] = (w,)
            for s in "rkvg":
                shapes[p + "mix.right." + s] = (hd, w)
            shapes.update({p + "mix.right.w1": (rank, w), p + "mix.right.w2": (hd, rank), p + "mix.right.w0": (hd,),
                           p + "mix.right.u": (r["heads"], r["dim"]), p + "mix.right.norm": (hd,), p + "mix.right.o": (w, hd),
                           p + "mix.left.out": (w,), p + "mix.right.out": (w,)})
        if layer["mlp"] is not None:
            ff, n = layer["mlp"]["expert"]["ff"], layer["mlp"]["router"]["experts"]
            shapes[p + "norm2"] = (w,)
            for j in range(n):
                shapes.update({f"{p}mlp.e{j}.gate": (ff, w), f"{p}mlp.e{j}.up": (ff, w), f"{p}mlp.e{j}.down": (w, ff)})
            shapes[p + "mlp.router"] = (n, w)
            shapes[p + "rg2"], shapes[p + "rg2.b"] = (w, w), (w,)
    shapes["final.norm"] = (w,)
    shapes["head"] = (cfg.vocab_size, w)
    return shapes


def checkpoint_names(cfg: MeronexConfig) -> list:
    return list(checkpoint_shapes(cfg))


def random_checkpoint(cfg: MeronexConfig, seed: int = 0):
    """(name, tensor) pairs of a seeded random checkpoint, rounded to bfloat16 values (as a stored checkpoint is), one
    tensor at a time.  Matrices are scaled by 1/sqrt(fan-in); norm weights are near one; biases, blends and decay
    parameters are small, so that memories neither vanish nor saturate over a few hundred tokens."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    for name, shape in checkpoint_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        rnd = torch.randn(shape, generator=gen)
        if leaf in ("norm", "norm1", "norm2", "out") or name == "final.norm":
            w = 1.0 + 0.1 * rnd
        elif name.endswith((".rg1.b", ".rg2.b", ".i.b", ".dt_bias", ".A_log", ".w0")):
            w = 0.5 * rnd
        elif name.endswith(".f.b"):
            w = 2.0 + 0.5 * rnd
        elif ".mu." in name:
            w = torch.rand(shape, generator=gen)
        elif leaf == "u":
            w = 0.5 * rnd
        elif leaf == "conv":
            w = rnd * shape[-1] ** -0.5
        elif name == "embed":
            w = rnd
        else:
            w = rnd * shape[-1] ** -0.5
        yield name, w.to(torch.bfloat16).float()
