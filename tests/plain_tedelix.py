"""A plain, slow implementation of the Tedelix decoder: whole sequences, no cache, no
batches, 64-bit arithmetic, one function for each mechanism, and no code shared with
``rustinfer_amd``.

The design in this file's own notation.  A model is an embedding, a list of layers and an
output head that reuses the embedding table.  A layer is *parallel*: with ``n = rmsnorm(x)``
the mixer and the feed-forward both read ``n`` and ``x <- x + mixer(n) + ff(n)``.  A layer's
mixer is one of

* ``attention``: grouped softmax attention inside a sliding window, rotary angles on the
  first ``rot.dims`` features of queries and keys (feature i paired with i + dims/2), and
  *rotated values*: the value of position j is turned by j over all of its features before it
  is summed, and the sum at position i is turned back by i;
* ``lightning``: linear attention with one fixed decay per head,
  ``S <- decay S + k v^T, o = S^T q`` on silu-activated q, k, v, then a norm over all heads,
  a sigmoid gate and the output projection;
* ``general_delta``: a generalized delta rule,
  ``S <- diag(w) S - (a u)(u^T S) + k v^T, o = S^T r`` with a unit key ``u``, a decay ``w`` and
  a removal rate ``a`` per key channel, then a norm per head, a weight, a gate, the projection.

The feed-forward is ``W_down relu(W_up n)^2``.  The logits are
``cap * tanh(scale * (E n_final) / cap)``.
"""
from __future__ import annotations

import json
import math
import os
import struct
from typing import Dict, List, Optional

import numpy as np


# ---------------------------------------------------------------------------
# reading a model folder (a reader of its own)
# ---------------------------------------------------------------------------
def read_safetensors(path: str) -> Dict[str, np.ndarray]:
    with open(path, "rb") as f:
        (hlen,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(hlen))
        data = f.read()
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        b, e = info["data_offsets"]
        raw, dt = data[b:e], info["dtype"]
        if dt == "F32":
            arr = np.frombuffer(raw, dtype="<f4").astype(np.float64)
        elif dt == "BF16":
            arr = (np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        elif dt == "F16":
            arr = np.frombuffer(raw, dtype="<f2").astype(np.float64)
        elif dt == "I32":
            arr = np.frombuffer(raw, dtype="<i4").astype(np.int64)
        else:
            raise ValueError(f"{name}: dtype {dt}")
        out[name] = arr.reshape(info["shape"])
    return out


def read_model(model_dir: str):
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    return cfg, read_safetensors(os.path.join(model_dir, "model.safetensors"))


# ---------------------------------------------------------------------------
# small functions
# ---------------------------------------------------------------------------
def unit_rms(x: np.ndarray, eps: float) -> np.ndarray:
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def rmsnorm(x, w, eps):
    return unit_rms(x, eps) * w


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def relu_squared(z):
    return np.maximum(z, 0.0) ** 2


def turn_halves(x: np.ndarray, positions: np.ndarray, base: float, dims: int, sign: float = 1.0) -> np.ndarray:
    """Rotate the first ``dims`` features of ``x [T, heads, size]``: feature i with feature
    i + dims/2 by the angle ``sign * position * base^(-2i/dims)``; the others pass."""
    out = x.copy()
    half = dims // 2
    f = base ** (-2.0 * np.arange(half) / dims)
    ang = sign * positions[:, None].astype(np.float64) * f[None, :]           # [T, half]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    out[..., :half] = a * c - b * s
    out[..., half:dims] = b * c + a * s
    return out


# ---------------------------------------------------------------------------
# the mixers; every one maps the normed rows n [T, width] of ONE sequence to [T, width]
# ---------------------------------------------------------------------------
def windowed_attention(n, w, m, start: int = 0):
    """``m``: the layer's 'mixer' entry of config.json; ``w``: name -> array for 'q', 'k', 'v', 'o'."""
    T = n.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    pos = np.arange(start, start + T)
    q = turn_halves((n @ w["q"].T).reshape(T, H, dk), pos, base, dims)
    k = turn_halves((n @ w["k"].T).reshape(T, G, dk), pos, base, dims)
    v = turn_halves((n @ w["v"].T).reshape(T, G, dv), pos, base, dv)          # the value carries its position
    out = np.zeros((T, H, dv))
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            lo = max(0, i - m["mask"]["size"] + 1)
            s = (k[lo:i + 1, g] @ q[i, h]) * m["scale"]
            p = np.exp(s - s.max())
            p /= p.sum()
            out[i, h] = p @ v[lo:i + 1, g]
    out = turn_halves(out, pos, base, dv, sign=-1.0)                          # and the sum is turned back
    return out.reshape(T, H * dv) @ w["o"].T


def lightning_attention(n, w, m, eps):
    T = n.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(n @ w["q"].T).reshape(T, H, dk)
    k = silu(n @ w["k"].T).reshape(T, H, dk)
    v = silu(n @ w["v"].T).reshape(T, H, dv)
    o = np.zeros((T, H, dv))
    for h in range(H):
        S = np.zeros((dk, dv))
        for t in range(T):
            S = m["decay"][h] * S + np.outer(k[t, h], v[t, h])
            o[t, h] = S.T @ q[t, h]
    y = rmsnorm(o.reshape(T, H * dv), w["norm"], eps) * sigmoid(n @ w["g"].T)
    return y @ w["o"].T


def general_delta_rule(n, w, m, eps):
    T = n.shape[0]
    H, d = m["heads"], m["dim"]
    r = (n @ w["r"].T).reshape(T, H, d)
    k = (n @ w["k"].T).reshape(T, H, d)
    v = (n @ w["v"].T).reshape(T, H, d)
    decay = np.exp(-math.exp(-0.5) * sigmoid(np.tanh(n @ w["w1"].T) @ w["w2"].T + w["w0"])).reshape(T, H, d)
    rate = sigmoid(n @ w["a"].T + w["a.b"]).reshape(T, H, d)
    o = np.zeros((T, H, d))
    for h in range(H):
        S = np.zeros((d, d))
        for t in range(T):
            u = k[t, h] / math.sqrt(float(k[t, h] @ k[t, h]) + 1e-6)
            S = decay[t, h][:, None] * S - np.outer(rate[t, h] * u, u @ S) + np.outer(k[t, h], v[t, h])
            o[t, h] = S.T @ r[t, h]
    y = unit_rms(o, eps).reshape(T, H * d) * w["norm"] * sigmoid(n @ w["g"].T)
    return y @ w["o"].T


def dense_ff(n, w):
    return relu_squared(n @ w["up"].T) @ w["down"].T


# ---------------------------------------------------------------------------
# the model
# ---------------------------------------------------------------------------
def _sub(w: Dict[str, np.ndarray], prefix: str) -> Dict[str, np.ndarray]:
    return {k[len(prefix):]: a for k, a in w.items() if k.startswith(prefix)}


def forward(cfg: dict, w: Dict[str, np.ndarray], ids, layers_out: Optional[List[np.ndarray]] = None) -> np.ndarray:
    """Logits [T, vocab] of one sequence from its first token.  ``layers_out`` collects the
    residual stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][np.asarray(ids, dtype=np.int64)]
    for i, layer in enumerate(cfg["layers"]):
        n = rmsnorm(x, w[f"l{i}.norm1"], eps)
        mw, m = _sub(w, f"l{i}.mix."), layer["mixer"]
        if layer["type"] == "attention":
            y = windowed_attention(n, mw, m)
        elif layer["type"] == "lightning":
            y = lightning_attention(n, mw, m, eps)
        elif layer["type"] == "general_delta":
            y = general_delta_rule(n, mw, m, eps)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp") is not None:
            y = y + dense_ff(n, _sub(w, f"l{i}.mlp."))
        x = x + y
        if layers_out is not None:
            layers_out.append(x.copy())
    z = (rmsnorm(x, w["final.norm"], eps) @ w["embed"].T) * cfg["logit_scale"]
    cap = cfg["logit_softcap"]
    return cap * np.tanh(z / cap)


def greedy(logits: np.ndarray) -> int:
    return int(np.argmax(logits))
