"""The Zorulix design, plainly: whole sequences, float64, no cache, one function per mechanism.

Slow on purpose (loops over tokens and heads where a loop says most clearly what is computed)
and independent of ``pyre_amd``: it reads ``config.json`` as a dictionary and the tensors by
their names. The tests compare the engine with it.

Notation: ``h`` the rows [T, width] that a sublayer reads, ``i`` a query's position, ``j`` a
key's, both counted from 0 within the sequence; ``W x`` for a matrix stored [out, in].
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


def one_plus_norm(x, w, eps):
    """The model's norm: the weight is stored around zero."""
    return unit_rms(x, eps) * (1.0 + w)


def silu(z):
    return z * torch.sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def linear(w, name, x, bias=False):
    y = x @ w[name].T
    return y + w[name + ".b"] if bias else y


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


def frequencies(rot) -> tuple[list[float], float]:
    """(angle per position of every pair, factor on cosines and sines) of a ``rot`` entry, with its scaling if any."""
    base, dims = float(rot["base"]), int(rot["dims"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def turns_to_dim(t):
        return dims * math.log(original / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo = max(math.floor(turns_to_dim(float(sc["fast"]))), 0)
    hi = min(math.ceil(turns_to_dim(float(sc["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate_halves(x, rot):
    """x [T, heads, d]: element e of every head paired with element e + dims / 2, e < dims / 2, turned by the angle
    position * f_e; the elements from ``dims`` on pass."""
    if not rot:
        return x
    f, mag = frequencies(rot)
    half = int(rot["dims"]) // 2
    out = x.clone()
    for t in range(x.shape[0]):
        for e in range(half):
            a = t * f[e]
            c, s = math.cos(a) * mag, math.sin(a) * mag
            u, v = x[t, :, e], x[t, :, e + half]
            out[t, :, e] = u * c - v * s
            out[t, :, e + half] = v * c + u * s
    return out


def window_attention(q, k, v, scale, window, sink):
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H * dv]. Query i sees keys j with 0 <= i - j < window (window 0:
    every j <= i). ``sink``: one more term of score 0 in the softmax's denominator, without a value."""
    T, H, _ = q.shape
    G, dv = k.shape[1], v.shape[2]
    out = torch.zeros(T, H, dv, dtype=F)
    for i in range(T):
        lo = max(0, i - window + 1) if window else 0
        for hd in range(H):
            g = hd // (H // G)
            s = (k[lo:i + 1, g] @ q[i, hd]) * scale
            m = max(float(s.max()), 0.0) if sink else float(s.max())
            e = torch.exp(s - m)
            den = e.sum() + (math.exp(-m) if sink else 0.0)
            out[i, hd] = (e / den) @ v[lo:i + 1, g]
    return out.reshape(T, H * dv)


# ----------------------------------------------------------------------------- mixers


def project_kv(w, p, m, h, eps):
    """Keys as a cache would hold them (normed over the whole projection where the mixer does that, then turned) and
    values of an attention mixer with projections of its own."""
    T = h.shape[0]
    G, d, dv = m["kv_heads"], m["dim"], m["vdim"]
    k = linear(w, f"{p}.k", h, True)
    if f"{p}.k.norm" in w:
        k = unit_rms(k, eps) * w[f"{p}.k.norm"]
    k = rotate_halves(k.reshape(T, G, d), m.get("rot"))
    return k, linear(w, f"{p}.v", h, True).reshape(T, G, dv)


def attention_mixer(w, p, m, h, eps, kv=None, sink=True, whole_norm=True, out_bias=False):
    """Grouped softmax attention over a window. ``kv``: another layer's keys and values instead of projections of its
    own. ``whole_norm``: queries (and keys) are RMS-normed over all their heads at once, with a weight over the whole
    projection, before they are turned."""
    T = h.shape[0]
    H, d = m["heads"], m["dim"]
    q = linear(w, f"{p}.q", h, True)
    if whole_norm:
        q = unit_rms(q, eps) * w[f"{p}.q.norm"]
    q = rotate_halves(q.reshape(T, H, d), m.get("rot"))
    k, v = kv if kv is not None else project_kv(w, p, m, h, eps)
    o = window_attention(q, k, v, float(m["scale"]), int((m.get("mask") or {}).get("size") or 0), sink)
    return linear(w, f"{p}.o", o, out_bias), (k, v)


def delta_rule_mixer(w, p, m, h, eps):
    """The gated delta rule: per head a state S [dim, vdim] that is decayed per key channel, corrected towards the
    token's value along its key and then read with the query."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(linear(w, f"{p}.q", h), w[f"{p}.q.conv"])).reshape(T, G, d)
    k = silu(short_conv(linear(w, f"{p}.k", h), w[f"{p}.k.conv"])).reshape(T, G, d)
    v = silu(short_conv(linear(w, f"{p}.v", h), w[f"{p}.v.conv"])).reshape(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(linear(w, f"{p}.b", h))                                     # [T, H]
    step = softplus(linear(w, f"{p}.a2", linear(w, f"{p}.a1", h)) + w[f"{p}.dt_bias"]).reshape(T, H, d)
    decay = torch.exp(-torch.exp(w[f"{p}.A_log"]).reshape(1, H, 1) * step)            # [T, H, d]
    gate = torch.sigmoid(linear(w, f"{p}.g2", linear(w, f"{p}.g1", h))).reshape(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=F)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(d, dv, dtype=F)
        for t in range(T):
            S = decay[t, hd].unsqueeze(1) * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, hd] = S.T @ q[t, g]
    out = unit_rms(out, eps) * w[f"{p}.norm"] * gate
    return linear(w, f"{p}.o", out.reshape(T, H * dv))


def parallel_mixer(w, p, m, h, eps):
    left, _ = attention_mixer(w, f"{p}.left", m["left"], h, eps, sink=False, whole_norm=False, out_bias=True)
    right = delta_rule_mixer(w, f"{p}.right", m["right"], h, eps)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


# ----------------------------------------------------------------------------- feed-forward, side input


def gated_unit(w, p, h):
    return (silu(linear(w, f"{p}.gate", h)) * linear(w, f"{p}.up", h)) @ w[f"{p}.down"].T


def router_logits(w, p, h):
    return linear(w, f"{p}.router", h, True)


def mixture(w, p, f, h, calls=None):
    """The ``top`` experts of largest router logit, weighted by the softmax over their logits alone; a shared expert,
    if the layer has one, for every token, times one sigmoid per token. ``calls`` (a list) receives, per token, the gap
    between the last logit that was chosen and the first that was not (inf if all were)."""
    E, top = f["router"]["experts"], f["router"]["top"]
    z = router_logits(w, p, h)
    out = torch.zeros_like(h)
    gaps = []
    for t in range(h.shape[0]):
        ranked = sorted(range(E), key=lambda e: (-float(z[t, e]), e))
        gaps.append(float(z[t, ranked[top - 1]] - z[t, ranked[top]]) if top < E else math.inf)
        order = ranked[:top]
        weights = torch.softmax(z[t, order], dim=0)
        for e, a in zip(order, weights):
            out[t] += a * gated_unit(w, f"{p}.e{e}", h[t:t + 1])[0]
    if f.get("shared"):
        out = out + torch.sigmoid(h @ w[f"{p}.shared.sg"].T) * gated_unit(w, f"{p}.shared", h)
    if calls is not None:
        calls.append(gaps)
    return out


def token_side(w, p, x, ids, i, dim, eps):
    """What a layer adds for the token itself: a slice of a second table, gated by the stream, carried to the width and
    RMS-normed with a plain weight."""
    e = w["side.embed"][ids][:, i * dim:(i + 1) * dim]
    y = (gelu_tanh(linear(w, f"{p}.side.gate", x)) * e) @ w[f"{p}.side.proj"].T
    return unit_rms(y, eps) * w[f"{p}.side.norm"]


# ----------------------------------------------------------------------------- the model


def forward(w, cfg, ids, return_hidden=False, calls=None):
    """Logits [T, vocab] of one sequence (float64); with ``return_hidden`` also the stream after every layer. ``calls``:
    see :func:`mixture` (one list per routed layer)."""
    eps = float(cfg["norm"]["eps"])
    ids = torch.as_tensor(list(ids), dtype=torch.long)
    x = w["embed"][ids] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    side = int((cfg.get("token_side") or {}).get("dim") or 0)
    kept, hidden = {}, []
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}", layer["mixer"]
        h = one_plus_norm(x, w[f"{p}.norm1"], eps)
        if layer["type"] == "attention":
            src = m.get("kv_from")
            mixed, kept[i] = attention_mixer(w, f"{p}.mix", m, h, eps, kv=kept[src] if src is not None else None)
        elif layer["type"] == "parallel":
            mixed = parallel_mixer(w, f"{p}.mix", m, h, eps)
        else:
            raise ValueError(f"layer {i}: unknown type {layer['type']!r}")
        x = x + mixed
        if layer.get("mlp"):
            x = x + mixture(w, f"{p}.mlp", layer["mlp"], one_plus_norm(x, w[f"{p}.norm2"], eps), calls)
        if side:
            x = x + token_side(w, p, x, ids, i, side, eps)
        hidden.append(x.clone())
    logits = one_plus_norm(x, w["final.norm"], eps) @ w["head"].T
    return (logits, hidden) if return_hidden else logits


def closest_call(w, cfg, ids):
    """Per position the least gap, over the routed layers, by which the choice of experts was made (inf without any)."""
    calls = []
    forward(w, cfg, ids, calls=calls)
    out = torch.full((len(ids),), math.inf, dtype=F)
    for layer in calls:
        out = torch.minimum(out, torch.tensor(layer, dtype=F))
    return out
