"""A plain, slow Mofulix: whole sequences, no cache, no carried state, float64, one function a mechanism.

It shares no code with `liyab_amd`: it takes a dict of numpy tensors by their file names and config.json
as a dict, and computes with numpy from the design's equations. In this file's notation (x: the residual
stream, rows = tokens; p: a row's position):

  x_0     = embed[token] * embedding.scale
  layer:    h = tanh(alpha * x) * w + b                     (the layer's one norm)
            x <- x + mixer(h) + feed_forward(h)             (both read the same h)
  logits  = head (tanh(alpha_f * x) * w_f + b_f)

  feed-forward:  g = min(Wg h, L), u = clip(Wu h, -L, L), Wd (g * s(1.702 g) * (u + 1))      s: logistic

  mixer "attention": q = Wq h, k = Wk h per head; values are k as projected; q, k <- unit_rms(.) * weight per head,
      then pairs (2i, 2i + 1) of the first rot.dims entries turned by p * f_i; score = cap * tanh(scale q.k / cap);
      causal softmax; heads side by side, times s(Wg h), then Wo.
  mixer "wkv":  per sub-input c in (r, k, v, g, w): m_c = h + (h_prev - h) * mu_c; r, k, v = W m; gate = silu(Wg m_g);
      decay d = exp(-exp(W2 tanh(W1 m_w) + w0)); per head, state S [key, value]:
      o = (S + (u * k) v^T)^T r;  S <- d * S (rows) + k v^T;  out = Wo (unit_rms(o) per head * weight * gate).
  mixer "parallel": 0.5 * (unit_rms(left(h)) * w_left + unit_rms(right(h)) * w_right)
      left:  q = Wq h * (1 + coef * ln(floor((p + 1) / every) + 1)), k = Wk h, v = Wv h;
             score = scale q.k + rel[bucket(i - j), head]; causal softmax; Wo.
      right: [z | x | B | C | dt] = Win h; (x, B, C) <- silu(conv(.) + bias) over time; dt <- softplus(dt + dt_bias);
             per head, state S [state, value]: S <- exp(-exp(A_log) dt) S + dt B x^T;  y = S^T C + D x;
             Wo (unit_rms(y * silu(z)) in norm_groups parts * weight).
"""

from __future__ import annotations

import math

import numpy as np


def round_to_bf16(a):
    """float -> the nearest bfloat16 (ties to even), as float64."""
    f = np.ascontiguousarray(a, dtype=np.float32)
    bits = f.view(np.uint32).astype(np.uint64)
    bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
    return bits.astype(np.uint32).view(np.float32).astype(np.float64).reshape(np.shape(a))


def logistic(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * logistic(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def unit_rms(v, eps):
    """v / sqrt(mean(v^2) + eps) over the last axis."""
    return v / np.sqrt((v * v).mean(axis=-1, keepdims=True) + eps)


def tanh_norm(x, t, name):
    """tanh(alpha x) * w + b with the scalar alpha and the vectors w, b stored as name, name.alpha, name.b."""
    return np.tanh(float(t[name + ".alpha"]) * x) * t[name] + t[name + ".b"]


def feed_forward(h, t, prefix, m):
    L = m["limit"]
    g = np.minimum(h @ t[prefix + "gate"].T, L)
    u = np.clip(h @ t[prefix + "up"].T, -L, L)
    return (g * logistic(1.702 * g) * (u + 1.0)) @ t[prefix + "down"].T


def causal_softmax(scores):
    """scores [n, n]: row i over columns j <= i."""
    n = scores.shape[0]
    seen = np.arange(n)[None, :] <= np.arange(n)[:, None]
    s = np.where(seen, scores, -np.inf)
    p = np.exp(s - s.max(axis=-1, keepdims=True))
    return p / p.sum(axis=-1, keepdims=True)


def rotary_frequencies(rot):
    """f_i = base^(-2i / dims), then stretched by wavelength as rot.scaling says (none: as they are)."""
    dims = rot["dims"]
    f = np.array([rot["base"] ** (-2.0 * i / dims) for i in range(dims // 2)])
    sc = rot.get("scaling")
    if sc:
        factor, low, high, orig = sc["factor"], sc["low"], sc["high"], sc["original"]
        out = []
        for fi in f:
            wl = 2.0 * math.pi / fi
            if wl < orig / high:
                out.append(fi)
            elif wl > orig / low:
                out.append(fi / factor)
            else:
                s = (orig / wl - low) / (high - low)
                out.append((1.0 - s) * fi / factor + s * fi)
        f = np.array(out)
    return f


def rotate_pairs(v, positions, rot):
    """v [n, heads, dim]: pairs (2i, 2i + 1) of the first rot.dims entries turned by position * f_i."""
    f = rotary_frequencies(rot)
    a = positions[:, None] * f[None, :]  # [n, dims / 2]
    c, s = np.cos(a)[:, None, :], np.sin(a)[:, None, :]
    dims = rot["dims"]
    out = v.copy()
    e, o = v[..., 0:dims:2], v[..., 1:dims:2]
    out[..., 0:dims:2] = e * c - o * s
    out[..., 1:dims:2] = o * c + e * s
    return out


def gated_attention(h, t, prefix, m, eps, positions):
    n = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ t[prefix + "q"].T).reshape(n, H, D)
    k = (h @ t[prefix + "k"].T).reshape(n, G, D)
    v = k.copy()
    q = unit_rms(q, eps) * t[prefix + "q.norm"]
    k = unit_rms(k, eps) * t[prefix + "k.norm"]
    if m.get("rot"):
        q, k = rotate_pairs(q, positions, m["rot"]), rotate_pairs(k, positions, m["rot"])
    cap = m.get("softcap")
    out = np.zeros((n, H, v.shape[-1]))
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"]
        if cap:
            s = cap * np.tanh(s / cap)
        out[:, hd] = causal_softmax(s) @ v[:, g]
    out = out.reshape(n, -1) * logistic(h @ t[prefix + "g"].T)
    return out @ t[prefix + "o"].T


def distance_bucket(n, B, D):
    """The row of a distance table of B rows for the distance n >= 0: itself below B / 2, then logarithmic up to D."""
    half = B // 2
    if n < half:
        return n
    return min(B - 1, half + int(math.floor(math.log(n / half) / math.log(D / half) * (B - half))))


def biased_attention(h, t, prefix, m, positions):
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ t[prefix + "q"].T).reshape(n, H, D)
    k = (h @ t[prefix + "k"].T).reshape(n, G, D)
    v = (h @ t[prefix + "v"].T).reshape(n, G, V)
    qt = m.get("q_temp")
    if qt:
        q = q * (1.0 + qt["coef"] * np.log(np.floor((positions + 1) / qt["every"]) + 1.0))[:, None, None]
    rel = t[prefix + "rel"]
    B = rel.shape[0]
    dist = positions[:, None] - positions[None, :]
    rows = np.array([[distance_bucket(int(d), B, m["bias_max"]) if d >= 0 else 0 for d in r] for r in dist])
    out = np.zeros((n, H, V))
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"] + rel[rows, hd]
        out[:, hd] = causal_softmax(s) @ v[:, g]
    return out.reshape(n, H * V) @ t[prefix + "o"].T


def short_convolution(x, w, bias):
    """x [n, channels], w [channels, taps] (last column: the current row), zeros before the first row."""
    n, taps = x.shape[0], w.shape[1]
    padded = np.concatenate([np.zeros((taps - 1, x.shape[1])), x])
    out = np.zeros_like(x) + bias
    for j in range(taps):
        out += w[:, j] * padded[j:j + n]
    return out


def state_space(h, t, prefix, m, eps):
    n = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    proj = h @ t[prefix + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(short_convolution(xbc, t[prefix + "conv"], t[prefix + "conv.b"]))
    x = xbc[:, :inner].reshape(n, H, P)
    Bm = xbc[:, inner:inner + G * N].reshape(n, G, N)
    Cm = xbc[:, inner + G * N:].reshape(n, G, N)
    dt = softplus(dt + t[prefix + "dt_bias"])
    A = -np.exp(t[prefix + "A_log"])
    y = np.zeros((n, H, P))
    for hd in range(H):
        g = hd // (H // G)
        S = np.zeros((N, P))
        for i in range(n):
            S = math.exp(A[hd] * dt[i, hd]) * S + dt[i, hd] * np.outer(Bm[i, g], x[i, hd])
            y[i, hd] = S.T @ Cm[i, g] + t[prefix + "D"][hd] * x[i, hd]
    y = y.reshape(n, inner) * silu(z)
    parts = m["norm_groups"]
    y = unit_rms(y.reshape(n, parts, inner // parts), eps).reshape(n, inner) * t[prefix + "norm"]
    return y @ t[prefix + "o"].T


def parallel_mixer(h, t, prefix, m, eps, positions):
    a = biased_attention(h, t, prefix + "left.", m["left"], positions)
    b = state_space(h, t, prefix + "right.", m["right"], eps)
    return 0.5 * (unit_rms(a, eps) * t[prefix + "left.out"] + unit_rms(b, eps) * t[prefix + "right.out"])


def wkv(h, t, prefix, m, eps):
    n = h.shape[0]
    H, D = m["heads"], m["dim"]
    prev = np.concatenate([np.zeros((1, h.shape[1])), h[:-1]])
    mix = {c: h + (prev - h) * t[prefix + "mu." + c] for c in "rkvgw"}
    r = (mix["r"] @ t[prefix + "r"].T).reshape(n, H, D)
    k = (mix["k"] @ t[prefix + "k"].T).reshape(n, H, D)
    v = (mix["v"] @ t[prefix + "v"].T).reshape(n, H, D)
    gate = silu(mix["g"] @ t[prefix + "g"].T)
    decay = np.exp(-np.exp(np.tanh(mix["w"] @ t[prefix + "w1"].T) @ t[prefix + "w2"].T + t[prefix + "w0"])).reshape(n, H, D)
    u = t[prefix + "u"]
    o = np.zeros((n, H, D))
    for hd in range(H):
        S = np.zeros((D, D))
        for i in range(n):
            kv = np.outer(k[i, hd], v[i, hd])
            o[i, hd] = (S + u[hd][:, None] * kv).T @ r[i, hd]
            S = decay[i, hd][:, None] * S + kv
    o = unit_rms(o, eps).reshape(n, H * D) * t[prefix + "norm"] * gate
    return o @ t[prefix + "o"].T


def run_mixer(kind, h, t, prefix, m, eps, positions):
    if kind == "attention":
        return gated_attention(h, t, prefix, m, eps, positions)
    if kind == "wkv":
        return wkv(h, t, prefix, m, eps)
    if kind == "parallel":
        return parallel_mixer(h, t, prefix, m, eps, positions)
    raise ValueError(kind)


def forward(config, t, tokens, streams=None):
    """float64 logits [n, vocab] of a whole sequence; `streams` (a list) gets the stream after every layer."""
    tokens = np.asarray(tokens)
    positions = np.arange(len(tokens), dtype=np.float64)
    eps = config["norm"]["eps"]
    x = t["embed"][tokens] * config["embedding"]["scale"]
    for i, layer in enumerate(config["layers"]):
        p = f"l{layer.get('weights_of', i) if layer.get('weights_of') is not None else i}."
        h = tanh_norm(x, t, p + "norm1")
        y = run_mixer(layer["type"], h, t, p + "mix.", layer["mixer"], eps, positions)
        if layer.get("mlp") is not None:
            y = y + feed_forward(h, t, p + "mlp.", layer["mlp"])
        x = x + y
        if streams is not None:
            streams.append(x.copy())
    return tanh_norm(x, t, "final.norm") @ t["head"].T
