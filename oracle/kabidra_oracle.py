"""Plain restatement of the Kabidra design: one function per mechanism, float32 (or float64) on the CPU, token by token
where a recurrence or a cache is involved.  For tests only: it shares no code with the package and is written for
clarity, not speed.

Notation: x is the residual stream (tokens, width); a layer computes
    x <- x + N_1b(mixer(C_1(N_1(x))))        x <- x + N_2b(ff(C_2(N_2(x))))
with N(v) = v / sqrt(mean(v^2) + eps) * (1 + w) and C(h)_t = h_t + sum_j k[:, j] * h_(t - taps + 1 + j) (zeros before the
sequence starts).  After layer i the stream handed on is the weighted sum of the embedding output and the results of
layers 0..i.
"""
from __future__ import annotations

import torch


def rms(v: torch.Tensor, eps: float) -> torch.Tensor:
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def norm_zero_centred(v, w, eps):
    """RMS norm whose stored weight is the deviation from one."""
    return rms(v, eps) * (1.0 + w)


def norm_plain(v, w, eps):
    return rms(v, eps) * w


def canon(h: torch.Tensor, k: torch.Tensor) -> torch.Tensor:
    """h (tokens, width) of ONE sequence from its first token; k (width, taps).  Returns h + causal convolution."""
    taps = k.shape[1]
    out = h.clone()
    for t in range(h.shape[0]):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += k[:, j] * h[s]
    return out


def gru_scan(z_pre: torch.Tensor, u: torch.Tensor, g_pre: torch.Tensor, s0=None):
    """The recurrence alone, from pre-activations (tokens, n): returns (outputs before the output projection, last state)."""
    z = torch.sigmoid(z_pre)
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    gate = g_pre * torch.sigmoid(g_pre)
    s = torch.zeros(z.shape[1], dtype=z.dtype) if s0 is None else s0.clone()
    ys = []
    for t in range(z.shape[0]):
        s = (1.0 - z[t]) * s + z[t] * cand[t]
        ys.append(s * gate[t])
    return torch.stack(ys), s


def mingru(h: torch.Tensor, p: dict) -> torch.Tensor:
    """minGRU layer (gates from the current token alone) with its projections; h (tokens, width) of one sequence from its start."""
    y, _ = gru_scan(h @ p["z"].T + p["z.b"], h @ p["x"].T + p["x.b"], h @ p["g"].T)
    return y @ p["o"].T


def latent_attention(h: torch.Tensor, p: dict, m: dict, eps: float) -> torch.Tensor:
    """Attention whose keys and values are both expanded from one cached latent per token; no positions."""
    heads, dim, vdim = m["heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    cq = norm_plain(h @ p["dq"].T, p["dq.norm"], eps)
    q = (cq @ p["uq"].T).view(n, heads, dim)
    c = norm_plain(h @ p["dkv"].T, p["dkv.norm"], eps)
    k = (c @ p["uk"].T).view(n, heads, dim)
    v = (c @ p["uv"].T).view(n, heads, vdim)
    gate = torch.sigmoid(h @ p["g"].T)                       # (tokens, heads)
    out = torch.zeros(n, heads, vdim, dtype=h.dtype)
    for i in range(n):
        for a in range(heads):
            s = (k[: i + 1, a] @ q[i, a]) * m["scale"]
            w = torch.softmax(s, 0)
            out[i, a] = (w[:, None] * v[: i + 1, a]).sum(0) * gate[i, a]
    return out.reshape(n, heads * vdim) @ p["o"].T


def feed_forward(h: torch.Tensor, p: dict) -> torch.Tensor:
    a = torch.relu(h @ p["up"].T)
    return (a * a) @ p["down"].T


def sub(w: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}


def forward(w: dict, cfg: dict, tokens, dtype=torch.float32, layers_out=None) -> torch.Tensor:
    """Logits (tokens, vocab) of one whole sequence.  `w`: name -> tensor; `layers_out`, if a list, receives every
    layer's result (before the weighted sum over the depth)."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    eps = cfg["norm"]["eps"]
    x = norm_zero_centred(w["embed"][torch.as_tensor(tokens)], w["embed.norm"], eps)
    hist = [x]
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        h = canon(norm_zero_centred(x, w[pre + "norm1"], eps), w[pre + "canon1"])
        if layer["type"] == "mingru":
            y = mingru(h, sub(w, pre + "mix."))
        elif layer["type"] == "latent_attention":
            y = latent_attention(h, sub(w, pre + "mix."), layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + norm_zero_centred(y, w[pre + "norm1b"], eps)
        if layer.get("mlp") is not None:
            if layer["mlp"]["kind"] != "dense":
                raise ValueError(layer["mlp"]["kind"])
            h = canon(norm_zero_centred(x, w[pre + "norm2"], eps), w[pre + "canon2"])
            x = x + norm_zero_centred(feed_forward(h, sub(w, pre + "mlp.")), w[pre + "norm2b"], eps)
        hist.append(x)
        if layers_out is not None:
            layers_out.append(x)
        x = sum(w[pre + "dwa"][j] * hist[j] for j in range(i + 2))
    return norm_zero_centred(x, w["final.norm"], eps) @ w["head"].T
