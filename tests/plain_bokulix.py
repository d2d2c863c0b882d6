"""A plain, slow Bokulix: whole sequences, no cache, no state, float64, one function a mechanism.

It shares no code with `liyab_amd`: it reads the model folder with the `safetensors` package
(through the GPT-2 twin's reader) and computes with numpy from the design's equations:

  x_0 = embed[token] + pos[p]
  layer:  u = x + conv(x);  x <- x + rms(sigmoid(Rg1 x + b1) * mixer(u)) * n1
          x <- x + rms(sigmoid(Rg2 x + b2) * experts(x)) * n2          (if the layer has a feed-forward)
  logits = head (rms(x) * nf)

Keys and values are made here the long way round (k = Wuk c, v = Wuv c for every position), which the
engine never does.
"""

from __future__ import annotations

import numpy as np

from plain_gpt2 import read_model, round_to_bf16  # noqa: F401  (the reader and the rounding are the twin's)


def round_matrices(tensors):
    """What the bfloat16 path holds: matrices and tables rounded to bfloat16; vectors and the
    convolution's taps (kept in 32 bits by the engine) untouched."""
    return {k: (round_to_bf16(v) if v.ndim >= 2 and not k.endswith(".canon1") else v) for k, v in tensors.items()}


def rms(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * weight over the last axis."""
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps) * weight


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def input_convolution(h, taps_w):
    """h_t + sum_j w[:, j] h_(t - taps + 1 + j), zeros before the first row. taps_w [width, taps]."""
    n, taps = h.shape[0], taps_w.shape[1]
    padded = np.concatenate([np.zeros((taps - 1, h.shape[1])), h])
    out = h.copy()
    for j in range(taps):
        out += taps_w[:, j] * padded[j:j + n]
    return out


def window_mask(n, window):
    """[n, n]: query i sees key j with 0 <= i - j < window (every j <= i when window is 0)."""
    i, j = np.arange(n)[:, None], np.arange(n)[None, :]
    seen = j <= i
    if window > 0:
        seen &= i - j < window
    return seen


def latent_attention(u, t, prefix, m, eps):
    """The mixer on its input u [n, width]; m: the layer's `mixer` entry of config.json."""
    n = u.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = (u @ t[prefix + "q"].T).reshape(n, H, D)
    c = rms(u @ t[prefix + "dkv"].T, t[prefix + "dkv.norm"], eps)
    k = (c @ t[prefix + "uk"].T).reshape(n, H, D)
    v = (c @ t[prefix + "uv"].T).reshape(n, H, V)
    seen = window_mask(n, (m.get("mask") or {}).get("size", 0))
    out = np.zeros((n, H, V))
    for h in range(H):
        s = (q[:, h] @ k[:, h].T) * m["scale"]
        s = np.where(seen, s, -np.inf)
        p = np.exp(s - s.max(axis=-1, keepdims=True))
        p /= p.sum(axis=-1, keepdims=True)
        out[:, h] = p @ v[:, h]
    out = out.reshape(n, H * V) * sigmoid(u @ t[prefix + "g"].T)
    return out @ t[prefix + "o"].T


def route(h, t, prefix, top):
    """(experts [n, top], weights [n, top]): the largest logits (the lower number among equals),
    softmax over them alone."""
    z = h @ t[prefix + "router"].T + t[prefix + "router.b"]
    order = np.argsort(-z, axis=-1, kind="stable")[:, :top]
    chosen = np.take_along_axis(z, order, axis=-1)
    w = np.exp(chosen - chosen.max(axis=-1, keepdims=True))
    return order, w / w.sum(axis=-1, keepdims=True)


def expert(h, t, prefix):
    g = h @ t[prefix + "gate"].T
    return ((g * sigmoid(g)) * (h @ t[prefix + "up"].T)) @ t[prefix + "down"].T


def routed_experts(h, t, prefix, mlp):
    experts, weights = route(h, t, prefix, mlp["router"]["top"])
    out = np.zeros_like(h)
    for i in range(h.shape[0]):
        for e, w in zip(experts[i], weights[i]):
            out[i] += w * expert(h[i], t, f"{prefix}e{int(e)}.")
    return out


def layer(x, t, config, i):
    entry = config["layers"][i]
    p = f"l{entry.get('weights_of', i) if entry.get('weights_of') is not None else i}."
    eps = config["norm"]["eps"]
    u = input_convolution(x, t[p + "canon1"]) if config.get("canon") is not None else x
    y = latent_attention(u, t, p + "mix.", entry["mixer"], eps)
    x = x + rms(y * sigmoid(x @ t[p + "rg1"].T + t[p + "rg1.b"]), t[p + "norm1"], eps)
    if entry.get("mlp") is not None:
        y = routed_experts(x, t, p + "mlp.", entry["mlp"])
        x = x + rms(y * sigmoid(x @ t[p + "rg2"].T + t[p + "rg2.b"]), t[p + "norm2"], eps)
    return x


def forward(config, t, ids, streams=None):
    """Logits [len(ids), vocab] of a whole sequence from position 0; `streams` (a list) gets the
    residual stream after every layer."""
    ids = np.asarray(ids)
    x = t["embed"][ids] + t["pos"][np.arange(len(ids))]
    for i in range(len(config["layers"])):
        x = layer(x, t, config, i)
        if streams is not None:
            streams.append(x.copy())
    return rms(x, t["final.norm"], config["norm"]["eps"]) @ t["head"].T


def generate_greedy(config, t, prompt, n):
    ids, out = list(prompt), []
    for _ in range(n):
        tok = int(np.argmax(forward(config, t, ids)[-1]))
        out.append(tok)
        ids.append(tok)
    return out
