"""Plain restatement of the Meronex design: one slow function per mechanism, whole sequences, token by token where the
design has a recurrence.  CPU tensors, float64 by default.  Nothing here is shared with the product path
(nano_vllm_x_amd/meronex.py and the kernels it launches); the tests compare the two.

Notation: T tokens, W model width, H heads, G key/value heads, D key size, E value size.  A weight dictionary `p` maps
the checkpoint's tensor names to tensors.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def _lin(w, x):
    return x @ w.to(x.dtype).T


def rms(x, eps, dim=-1):
    return x / torch.sqrt((x * x).mean(dim=dim, keepdim=True) + eps)


def grouped_norm(x, w, groups: int, eps: float):
    """x (T, W): each of `groups` consecutive slices of a row is scaled to unit mean square, then the row times w."""
    t, width = x.shape
    parts = x.view(t, groups, width // groups)
    return rms(parts, eps).reshape(t, width) * w.to(x.dtype)


# ---- rotary positions ----------------------------------------------------------------------------------------------
def rotary_table(rot: dict, dtype=F64):
    """(frequencies (dims/2), factor on cos and sin) of a rotary specification {base, dims, scaling | None}."""
    dims, base = int(rot["dims"]), float(rot["base"])
    idx = torch.arange(dims // 2, dtype=dtype)
    freq = base ** (-2.0 * idx / dims)
    sc = rot.get("scaling")
    if not sc:
        return freq, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def turn_dim(turns):
        return dims * math.log(original / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
    ramp = ((idx - lo) / max(hi - lo, 0.001)).clamp(0, 1)
    freq = freq / factor * ramp + freq * (1 - ramp)
    return freq, 0.1 * math.log(factor) + 1.0


def rotate(x, pos, rot: dict):
    """x (T, heads, D); the first rot.dims of D are rotated in pairs (i, i + dims/2) by pos * freq_i."""
    if not rot:
        return x
    dims = int(rot["dims"])
    freq, mag = rotary_table(rot, x.dtype)
    ang = pos.to(x.dtype)[:, None] * freq[None, :]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    a, b = x[..., :dims // 2], x[..., dims // 2:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], dim=-1)


# ---- mixers ------------------------------------------------------------------------------------------------------------
def softcap_attention(h, p, pre, m: dict, eps: float):
    """Causal attention with rotary positions, unit-mean-square values, capped scores and grouped heads."""
    t = h.shape[0]
    hq, g, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(t)
    q = rotate(_lin(p[pre + "q"], h).view(t, hq, d), pos, m["rot"])
    k = rotate(_lin(p[pre + "k"], h).view(t, g, d), pos, m["rot"])
    v = rms(_lin(p[pre + "v"], h).view(t, g, e), eps)
    out = torch.zeros(t, hq, e, dtype=h.dtype)
    cap = m.get("softcap")
    for head in range(hq):
        kv = head // (hq // g)
        s = (q[:, head] @ k[:, kv].T) * float(m["scale"])
        if cap:
            s = float(cap) * torch.tanh(s / float(cap))
        s = s.masked_fill(torch.ones(t, t).triu(1).bool(), float("-inf"))
        out[:, head] = torch.softmax(s, dim=-1) @ v[:, kv]
    return _lin(p[pre + "o"], out.reshape(t, hq * e))


def mlstm(h, p, pre, m: dict, eps: float):
    """Matrix memory with exponential input gate, sigmoid forget gate (both capped) and a running maximum that starts at 0."""
    t = h.shape[0]
    hd, d, e, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    q = _lin(p[pre + "q"], h).view(t, hd, d) * d ** -0.5
    k = _lin(p[pre + "k"], h).view(t, hd, d)
    v = _lin(p[pre + "v"], h).view(t, hd, e)
    gi = cap * torch.tanh((_lin(p[pre + "i"], h) + p[pre + "i.b"].to(h.dtype)) / cap)
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh((_lin(p[pre + "f"], h) + p[pre + "f.b"].to(h.dtype)) / cap))
    out = torch.zeros(t, hd, e, dtype=h.dtype)
    for head in range(hd):
        s = torch.zeros(d, e, dtype=h.dtype)
        n = torch.zeros(d, dtype=h.dtype)
        mx = torch.zeros((), dtype=h.dtype)
        for i in range(t):
            new = torch.maximum(gf[i, head] + mx, gi[i, head])
            keep, put = torch.exp(gf[i, head] + mx - new), torch.exp(gi[i, head] - new)
            s = keep * s + put * torch.outer(k[i, head], v[i, head])
            n = keep * n + put * k[i, head]
            mx = new
            den = torch.maximum((n @ q[i, head]).abs(), torch.exp(-mx)) + 1e-6
            out[i, head] = (s.T @ q[i, head]) / den
    y = rms(out, eps).reshape(t, hd * e) * p[pre + "norm"].to(h.dtype) * torch.sigmoid(_lin(p[pre + "g"], h))
    return _lin(p[pre + "o"], y)


def short_conv_silu(x, w):
    """x (T, C), w (C, taps): y_t = silu(sum_j w[:, j] x_(t - taps + 1 + j)), zeros before the start."""
    t, c = x.shape
    taps = w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, c, dtype=x.dtype), x])
    y = sum(pad[j:j + t] * w[:, j].to(x.dtype) for j in range(taps))
    return y * torch.sigmoid(y)


def gated_delta(h, p, pre, m: dict, eps: float):
    """Delta rule with a per-head decay: the memory forgets, is corrected towards the new value along the key, then read."""
    t = h.shape[0]
    hd, g, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = short_conv_silu(_lin(p[pre + "q"], h), p[pre + "q.conv"]).view(t, g, d)
    k = short_conv_silu(_lin(p[pre + "k"], h), p[pre + "k.conv"]).view(t, g, d)
    v = short_conv_silu(_lin(p[pre + "v"], h), p[pre + "v.conv"]).view(t, hd, e)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(_lin(p[pre + "b"], h))
    decay = torch.exp(-torch.exp(p[pre + "A_log"].to(h.dtype)) * torch.nn.functional.softplus(_lin(p[pre + "a"], h) + p[pre + "dt_bias"].to(h.dtype)))
    out = torch.zeros(t, hd, e, dtype=h.dtype)
    for head in range(hd):
        kv = head // (hd // g)
        s = torch.zeros(d, e, dtype=h.dtype)
        for i in range(t):
            s = decay[i, head] * s
            u = beta[i, head] * (v[i, head] - s.T @ k[i, kv])
            s = s + torch.outer(k[i, kv], u)
            out[i, head] = s.T @ q[i, kv]
    gate = _lin(p[pre + "g"], h)
    y = (rms(out, eps) * p[pre + "norm"].to(h.dtype)).reshape(t, hd * e) * (gate * torch.sigmoid(gate))
    return _lin(p[pre + "o"], y)


def time_mix(h, p, pre, m: dict, eps: float):
    """Token-shift mixing and a per-channel decayed outer-product memory with a bonus for the current token."""
    t, width = h.shape
    hd, d = m["heads"], m["dim"]
    prev = torch.cat([torch.zeros(1, width, dtype=h.dtype), h[:-1]])
    mix = {s: h + (prev - h) * p[pre + "mu." + s].to(h.dtype) for s in "rkvgw"}
    r = _lin(p[pre + "r"], mix["r"]).view(t, hd, d)
    k = _lin(p[pre + "k"], mix["k"]).view(t, hd, d)
    v = _lin(p[pre + "v"], mix["v"]).view(t, hd, d)
    gate = _lin(p[pre + "g"], mix["g"])
    gate = gate * torch.sigmoid(gate)
    w = torch.exp(-torch.exp(_lin(p[pre + "w2"], torch.tanh(_lin(p[pre + "w1"], mix["w"]))) + p[pre + "w0"].to(h.dtype))).view(t, hd, d)
    bonus = p[pre + "u"].to(h.dtype)
    out = torch.zeros(t, hd, d, dtype=h.dtype)
    for head in range(hd):
        s = torch.zeros(d, d, dtype=h.dtype)
        for i in range(t):
            kv = torch.outer(k[i, head], v[i, head])
            out[i, head] = (s + bonus[head][:, None] * kv).T @ r[i, head]
            s = w[i, head][:, None] * s + kv
    y = rms(out, eps).reshape(t, hd * d) * p[pre + "norm"].to(h.dtype) * gate
    return _lin(p[pre + "o"], y)


def parallel_mixer(h, p, pre, m: dict, eps: float):
    left = softcap_attention(h, p, pre + "left.", m["left"], eps)
    right = time_mix(h, p, pre + "right.", m["right"], eps)
    return 0.5 * (rms(left, eps) * p[pre + "left.out"].to(h.dtype) + rms(right, eps) * p[pre + "right.out"].to(h.dtype))


MIXERS = {"mlstm": mlstm, "delta": gated_delta, "parallel": parallel_mixer}


# ---- feed-forward ----------------------------------------------------------------------------------------------------
def expert(x, p, pre, limit: float):
    g = _lin(p[pre + "gate"], x).clamp(max=limit)
    u = _lin(p[pre + "up"], x).clamp(-limit, limit)
    return _lin(p[pre + "down"], g * torch.sigmoid(1.702 * g) * (u + 1))


def moe(h, p, pre, spec: dict):
    """Sigmoid router; the `top` largest scores pick the experts and scale their INPUT; no renormalisation."""
    n, top, limit = spec["router"]["experts"], spec["router"]["top"], float(spec["expert"]["limit"])
    score = torch.sigmoid(_lin(p[pre + "router"], h))
    val, idx = score.topk(top, dim=-1)
    out = torch.zeros_like(h)
    for e in range(n):
        for j in range(top):
            rows = (idx[:, j] == e).nonzero().flatten()
            if rows.numel():
                out[rows] += expert(h[rows] * val[rows, j:j + 1], p, f"{pre}e{e}.", limit)
    return out


# ---- the stack -------------------------------------------------------------------------------------------------------
def forward(cfg: dict, p: dict, tokens, dtype=F64, keep_layers: bool = False):
    """Logits (T, vocab) of one sequence from position 0 [and the stream after every layer, (layers, T, W)]."""
    eps, groups, mult = float(cfg["norm"]["eps"]), int(cfg["norm"]["groups"]), float(cfg["residual_mult"])
    x = p["embed"].to(dtype)[torch.as_tensor(tokens, dtype=torch.long)]
    kept = []
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        h = grouped_norm(x, p[pre + "norm1"], groups, eps)
        y = MIXERS[layer["type"]](h, p, pre + "mix.", layer["mixer"], eps)
        x = x + mult * y * torch.sigmoid(_lin(p[pre + "rg1"], h) + p[pre + "rg1.b"].to(dtype))
        if layer.get("mlp") is not None:
            h = grouped_norm(x, p[pre + "norm2"], groups, eps)
            y = moe(h, p, pre + "mlp.", layer["mlp"])
            x = x + mult * y * torch.sigmoid(_lin(p[pre + "rg2"], h) + p[pre + "rg2.b"].to(dtype))
        kept.append(x)
    logits = _lin(p["head"], grouped_norm(x, p["final.norm"], groups, eps))
    return (logits, torch.stack(kept)) if keep_layers else logits
