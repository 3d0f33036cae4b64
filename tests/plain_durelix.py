"""The Durelix design, plainly: whole sequences, float64, no cache, one function per mechanism.

Slow on purpose (loops over tokens and heads where a loop says most clearly what is computed)
and independent of ``pyre_amd``: it reads ``config.json`` as a dictionary and the tensors by
their names. The tests compare the engine with it.

Notation: ``h`` the rows [T, width] that a sublayer reads, ``i`` a query's position, ``j`` a
key's, both counted from 0 within the sequence.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch

F = torch.float64


def read_folder(folder) -> tuple[dict, dict]:
    """(config as a dictionary, tensors as float64 / int64) of a model folder."""
    from safetensors.torch import load_file

    folder = Path(folder)
    cfg = json.loads((folder / "config.json").read_text())
    raw = load_file(str(folder / "model.safetensors"))
    return cfg, {k: (v.to(F) if v.is_floating_point() else v.long()) for k, v in raw.items()}


# ----------------------------------------------------------------------------- small pieces


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, gain, eps):
    return unit_rms(x, eps) * gain


def silu(z):
    return z * torch.sigmoid(z)


def short_conv(u, taps_w):
    """y[t, c] = sum_j taps_w[c, j] * u[t - (taps - 1) + j, c], rows before the sequence's start being zero:
    the last tap multiplies the token itself, the first the one ``taps - 1`` back."""
    T, taps = u.shape[0], taps_w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                y[t] += taps_w[:, j] * u[s]
    return y


def rotate_neighbours(x, base, dims):
    """x [T, heads, d]: elements (2e, 2e + 1), e < dims / 2, of every head turned by the angle
    position * base^(-2e / dims); the elements from ``dims`` on pass."""
    out = x.clone()
    T = x.shape[0]
    for t in range(T):
        for e in range(dims // 2):
            a = t * base ** (-2.0 * e / dims)
            u, v = x[t, :, 2 * e], x[t, :, 2 * e + 1]
            out[t, :, 2 * e] = u * math.cos(a) - v * math.sin(a)
            out[t, :, 2 * e + 1] = v * math.cos(a) + u * math.sin(a)
    return out


def rotate_halves(x, base, dims):
    """The same with element e paired with element e + dims / 2."""
    out = x.clone()
    T, half = x.shape[0], dims // 2
    for t in range(T):
        for e in range(half):
            a = t * base ** (-2.0 * e / dims)
            u, v = x[t, :, e], x[t, :, e + half]
            out[t, :, e] = u * math.cos(a) - v * math.sin(a)
            out[t, :, e + half] = v * math.cos(a) + u * math.sin(a)
    return out


def sees(i: int, j: int, window: int) -> bool:
    """Causal, and within the last ``window`` positions (0: every earlier position)."""
    return j <= i and (not window or i - j < window)


# ----------------------------------------------------------------------------- the softmax branch


def sink_attention(h, w, p, c, eps):
    """Grouped-query softmax attention over a window: projections followed by a short convolution over time,
    queries and keys normed per head and turned in neighbouring pairs, a learned number per head in the softmax's
    denominator (a key without a value), a sigmoid gate per output element."""
    T = h.shape[0]
    H, G, d, dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q, k, v = h @ w[f"{p}.q"].T, h @ w[f"{p}.k"].T, h @ w[f"{p}.v"].T
    if c.get("conv"):
        q, k, v = short_conv(q, w[f"{p}.q.conv"]), short_conv(k, w[f"{p}.k.conv"]), short_conv(v, w[f"{p}.v.conv"])
    q = rms_norm(q.view(T, H, d), w[f"{p}.q.norm"], eps)
    k = rms_norm(k.view(T, G, d), w[f"{p}.k.norm"], eps)
    v = v.view(T, G, dv)
    rot = c.get("rot")
    if rot:
        q, k = rotate_neighbours(q, rot["base"], rot["dims"]), rotate_neighbours(k, rot["base"], rot["dims"])
    window = (c.get("mask") or {}).get("size", 0)
    sink = w[f"{p}.sink"]
    out = torch.zeros(T, H, dv, dtype=F)
    seen = torch.tensor([[sees(i, j, window) for j in range(T)] for i in range(T)])
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T * c["scale"]).masked_fill(~seen, -math.inf)       # [i, j]
        m = torch.maximum(s.max(-1).values, sink[a])
        e = torch.exp(s - m[:, None])
        weights = e / (e.sum(-1) + torch.exp(sink[a] - m))[:, None]              # the sink: one more term below, no value
        out[:, a] = weights @ v[:, g]
    gate = torch.sigmoid(h @ w[f"{p}.g"].T)
    return (out.reshape(T, H * dv) * gate) @ w[f"{p}.o"].T


# ----------------------------------------------------------------------------- the recurrent branch


def retention(h, w, p, c, eps):
    """Linear attention with one fixed decay per head: S <- decay S + k v^T, o = S^T q, no softmax and no
    denominator; queries and keys turned in halves, keys scaled by dim^-1/2 after that; every head's o divided by
    its root mean square, times silu of a gate, then the output matrix."""
    T = h.shape[0]
    H, d, dv = c["heads"], c["dim"], c["vdim"]
    q = (h @ w[f"{p}.q"].T).view(T, H, d)
    k = (h @ w[f"{p}.k"].T).view(T, H, d)
    v = (h @ w[f"{p}.v"].T).view(T, H, dv)
    rot = c.get("rot")
    if rot:
        q, k = rotate_halves(q, rot["base"], rot["dims"]), rotate_halves(k, rot["base"], rot["dims"])
    k = k * d ** -0.5
    o = torch.zeros(T, H, dv, dtype=F)
    for a in range(H):
        S = torch.zeros(d, dv, dtype=F)
        for t in range(T):
            S = c["decay"][a] * S + torch.outer(k[t, a], v[t, a])
            o[t, a] = S.T @ q[t, a]
    o = unit_rms(o, eps).reshape(T, H * dv) * silu(h @ w[f"{p}.g"].T)
    return o @ w[f"{p}.o"].T


def parallel_mixer(h, w, p, c, eps):
    """Half the sum of the two branches, each normed over the width with a gain of its own."""
    left = rms_norm(sink_attention(h, w, f"{p}.left", c["left"], eps), w[f"{p}.left.out"], eps)
    right = rms_norm(retention(h, w, f"{p}.right", c["right"], eps), w[f"{p}.right.out"], eps)
    return 0.5 * (left + right)


# ----------------------------------------------------------------------------- feed-forwards


def dense_ff(h, w, p):
    """down(relu(up h)^2)."""
    return torch.relu(h @ w[f"{p}.up"].T) ** 2 @ w[f"{p}.down"].T


def choose(s, correction, top, count, keep):
    """The experts chosen for one token with scores ``s``: by s + correction, among the experts of the ``keep`` of
    ``count`` equal groups of neighbours whose largest such number is largest (the lower index among equals). Also
    returns how close the call was: the least gap between something taken and the best thing left out."""
    choice = s + correction
    size = len(s) // count
    tops = [float(choice[g * size:(g + 1) * size].max()) for g in range(count)]
    best = sorted(range(count), key=lambda g: (-tops[g], g))
    allowed = [e for g in best[:keep] for e in range(g * size, (g + 1) * size)]
    ranked = sorted(allowed, key=lambda e: (-float(choice[e]), e))
    gap = math.inf
    if keep < count:
        gap = min(gap, tops[best[keep - 1]] - tops[best[keep]])
    if top < len(ranked):
        gap = min(gap, float(choice[ranked[top - 1]] - choice[ranked[top]]))
    return ranked[:top], gap


def route(h, w, p, c, calls=None):
    """For every token the chosen experts and their weights, [(expert, weight), ...]: scores softmax(router h) over
    experts and identity experts alike; the weight of a chosen expert is its score itself. ``calls`` collects, per
    token, how close the choice was."""
    r = c["router"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    out = []
    for t in range(h.shape[0]):
        s = torch.softmax(w[f"{p}.router"] @ h[t], -1)
        chosen, gap = choose(s, w[f"{p}.correction"], r["top"], groups["count"], groups["keep"])
        if calls is not None:
            calls.append(gap)
        out.append([(e, s[e]) for e in chosen])
    return out


def moe_ff(h, w, p, c, calls=None):
    """The weighted sum of the chosen experts' results; an expert is down(silu(gate h) * (up h)), an identity
    expert (the last ``identity`` outputs of the router) hands the row back as it is."""
    real = c["router"]["experts"]
    out = torch.zeros_like(h)
    for t, picks in enumerate(route(h, w, p, c, calls)):
        for e, weight in picks:
            if e >= real:
                out[t] += weight * h[t]
            else:
                x = silu(w[f"{p}.e{e}.gate"] @ h[t]) * (w[f"{p}.e{e}.up"] @ h[t])
                out[t] += weight * (w[f"{p}.e{e}.down"] @ x)
    return out


def feed_forward(h, w, p, c, calls=None):
    return dense_ff(h, w, p) if c["kind"] == "dense" else moe_ff(h, w, p, c, calls)


#: layer type -> its mixer (h, w, prefix, the layer's 'mixer' entry, eps); tests of one branch alone add theirs
MIXERS = {"parallel": parallel_mixer}


# ----------------------------------------------------------------------------- the model


def embed(w, cfg, ids):
    """Row of the token plus a row of a second table chosen by the pair (previous token, token); a sequence's
    first token takes that table's last row."""
    x = w["embed"][torch.tensor(ids)].clone()
    b = (cfg.get("embedding") or {}).get("bigram")
    if b:
        for t, tok in enumerate(ids):
            row = b["buckets"] if t == 0 else (ids[t - 1] * b["mul_prev"] + tok * b["mul_cur"]) % b["buckets"]
            x[t] += w["bigram"][row]
    return x


def forward(w, cfg, ids, return_hidden=False, calls=None):
    """Logits [T, vocab] of one sequence (and the residual stream after every layer). ``calls``: a list that
    receives one list per routed layer, how close each token's choice of experts was."""
    eps = cfg["norm"]["eps"]
    x = embed(w, cfg, ids)
    hidden = []
    for n, layer in enumerate(cfg["layers"]):
        p = f"l{n}"
        # every sublayer reads the stream itself; its result is normed before it is added
        x = x + rms_norm(MIXERS[layer["type"]](x, w, f"{p}.mix", layer["mixer"], eps), w[f"{p}.norm1"], eps)
        if layer.get("mlp") is not None:
            mine = [] if calls is not None and layer["mlp"]["kind"] == "moe" else None
            x = x + rms_norm(feed_forward(x, w, f"{p}.mlp", layer["mlp"], mine), w[f"{p}.norm2"], eps)
            if mine is not None:
                calls.append(mine)
        hidden.append(x)
    logits = rms_norm(x, w["final.norm"], eps) @ w["embed"].T
    return (logits, hidden) if return_hidden else logits


def closest_call(w, cfg, ids):
    """Per position the least gap, over the routed layers, by which the choice of experts was made (inf without any)."""
    calls = []
    forward(w, cfg, ids, calls=calls)
    out = torch.full((len(ids),), math.inf, dtype=F)
    for layer in calls:
        out = torch.minimum(out, torch.tensor(layer, dtype=F))
    return out
