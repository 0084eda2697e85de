"""A plain, slow implementation of the Belorax decoder: whole sequences, no cache, no batches,
64-bit arithmetic, one function for each mechanism, and no code shared with ``rustinfer_amd``.

The design in this file's own notation.  ``x`` is the residual stream, ``m`` the model's
``residual_mult``, ``unit(y) = y / sqrt(mean(y^2) + eps)``.

* embedding: ``x = E[token] * embedding.scale``;
* a layer: ``x <- x + m * unit(mixer(x)) * (1 + w1)``, then, if it has a feed-forward,
  ``x <- x + m * unit(ff(x)) * (1 + w2)``: the sub-layers read ``x`` as it is and the norm sits
  on what they return;
* mixer ``attention``: grouped softmax attention over all earlier positions; queries and keys
  are unit-normed per head and multiplied by a weight of the head's size; no rotation; the
  query at position p is multiplied by ``1 + coef * ln(floor((p + 1) / every) + 1)``; a layer
  with ``kv_from: j`` has no keys and values of its own and reads those of layer j;
* mixer ``latent_attention``: one latent vector ``c = unit(first kv_rank rows of W_dkv h) * w``
  and one rotated key part (the remaining ``rot_dim`` rows) serve all heads; head h's key is
  ``[W_uk,h c, rotated part]`` and its value ``W_uv,h c``; the rotation pairs feature 2i with
  2i + 1 and its frequencies are stretched as YaRN does;
* mixer ``retention``: ``S <- decay_h S + k v^T, o = S^T q`` with rotated q and k (feature i
  paired with i + dims/2), ``k`` divided by ``sqrt(dim)``; each head's ``o`` is unit-normed, the
  heads are gated by ``silu(W_g h)`` and projected;
* feed-forward ``dense``: ``W_down (silu(W_gate h) * W_up h)``; ``moe``: the same for each of
  ``experts`` experts, of which the ``top`` with the largest ``softmax(W_router h)`` are summed
  with those probabilities as weights (not renormalised);
* output: ``logits = W_head (unit(x) * (1 + w_final))``.
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
def unit(y: np.ndarray, eps: float) -> np.ndarray:
    return y / np.sqrt(np.mean(y * y, axis=-1, keepdims=True) + eps)


def silu(z):
    return z / (1.0 + np.exp(-z))


def softmax_rows(s: np.ndarray) -> np.ndarray:
    e = np.exp(s - np.max(s, axis=-1, keepdims=True))
    return e / np.sum(e, axis=-1, keepdims=True)


def causal_softmax_attention(q, k, v, scale):
    """q [T, dk], k [T, dk], v [T, dv] of one head: row i sees rows j <= i."""
    T = q.shape[0]
    s = (q @ k.T) * scale
    s = np.where(np.tril(np.ones((T, T), dtype=bool)), s, -np.inf)
    return softmax_rows(s) @ v


def plain_frequencies(dims: int, base: float) -> np.ndarray:
    return np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])


def yarn_frequencies(dims: int, base: float, sc: dict):
    """(frequencies, the factor on cos and sin)."""
    f = plain_frequencies(dims, base)
    where = lambda turns: dims * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(where(sc["fast"])), 0)
    hi = min(math.ceil(where(sc["slow"])), dims - 1)
    ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / sc["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def rotate(y: np.ndarray, freqs: np.ndarray, dims: int, interleaved: bool, mag: float = 1.0) -> np.ndarray:
    """y [T, n]: the first ``dims`` features turned by the row's position; pair i is (2i, 2i+1)
    if interleaved, else (i, i + dims/2)."""
    T = y.shape[0]
    ang = np.arange(T)[:, None] * freqs[None, :]
    c, s = np.cos(ang) * mag, np.sin(ang) * mag
    out = y.copy()
    h = dims // 2
    a, b = (slice(0, dims, 2), slice(1, dims, 2)) if interleaved else (slice(0, h), slice(h, dims))
    out[:, a] = y[:, a] * c - y[:, b] * s
    out[:, b] = y[:, b] * c + y[:, a] * s
    return out


# ---------------------------------------------------------------------------
# mixers
# ---------------------------------------------------------------------------
def attention_keys_values(h, w, m, eps):
    """What an attention layer leaves for itself and for layers that borrow from it:
    normed keys [T, G, dim] and values [T, G, vdim]."""
    T, G = h.shape[0], m["kv_heads"]
    k = unit((h @ w["k"].T).reshape(T, G, m["dim"]), eps) * w["k.norm"]
    v = (h @ w["v"].T).reshape(T, G, m["vdim"])
    return k, v


def qknorm_attention(h, w, m, eps, kv):
    T, H, G = h.shape[0], m["heads"], m["kv_heads"]
    k, v = kv
    q = unit((h @ w["q"].T).reshape(T, H, m["dim"]), eps) * w["q.norm"]
    if m.get("q_temp"):
        p = np.arange(T)
        temp = 1.0 + m["q_temp"]["coef"] * np.log(np.floor((p + 1) / m["q_temp"]["every"]) + 1.0)
        q = q * temp[:, None, None]
    heads = [causal_softmax_attention(q[:, i], k[:, i // (H // G)], v[:, i // (H // G)], m["scale"]) for i in range(H)]
    return np.concatenate(heads, axis=1) @ w["o"].T


def latent_attention(h, w, m, eps):
    T, H, d, r, dv, R = h.shape[0], m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = m["rot"]
    if rot.get("scaling"):
        freqs, mag = yarn_frequencies(rot["dims"], rot["base"], rot["scaling"])
    else:
        freqs, mag = plain_frequencies(rot["dims"], rot["base"]), 1.0
    q = (h @ w["q"].T).reshape(T, H, d + r)
    down = h @ w["dkv"].T
    c = unit(down[:, :R], eps) * w["dkv.norm"]
    k_rot = rotate(down[:, R:], freqs, rot["dims"], True, mag)
    k_up = (c @ w["uk"].T).reshape(T, H, d)
    v = (c @ w["uv"].T).reshape(T, H, dv)
    heads = []
    for i in range(H):
        qi = np.concatenate([q[:, i, :d], rotate(q[:, i, d:], freqs, rot["dims"], True, mag)], axis=1)
        ki = np.concatenate([k_up[:, i], k_rot], axis=1)
        heads.append(causal_softmax_attention(qi, ki, v[:, i], m["scale"]))
    return np.concatenate(heads, axis=1) @ w["o"].T


def retention(h, w, m, eps):
    T, H, d, dv = h.shape[0], m["heads"], m["dim"], m["vdim"]
    rot = m["rot"]
    freqs, mag = yarn_frequencies(rot["dims"], rot["base"], rot["scaling"]) if rot.get("scaling") else (plain_frequencies(rot["dims"], rot["base"]), 1.0)
    q = (h @ w["q"].T).reshape(T, H, d)
    k = (h @ w["k"].T).reshape(T, H, d)
    v = (h @ w["v"].T).reshape(T, H, dv)
    out = np.zeros((T, H, dv))
    for i in range(H):
        qi = rotate(q[:, i], freqs, rot["dims"], False, mag)
        ki = rotate(k[:, i], freqs, rot["dims"], False, mag) / math.sqrt(d)
        S = np.zeros((d, dv))
        for t in range(T):
            S = m["decay"][i] * S + np.outer(ki[t], v[t, i])
            out[t, i] = S.T @ qi[t]
    out = unit(out, eps).reshape(T, H * dv)
    return (out * silu(h @ w["g"].T)) @ w["o"].T


# ---------------------------------------------------------------------------
# feed-forwards
# ---------------------------------------------------------------------------
def gated_ff(h, w):
    return (silu(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def routed_ff(h, w, mlp, gaps=None):
    """``gaps`` (a list) receives, for every row, how far the last chosen expert's probability lies
    above the first one left out, relative to it (infinite where all experts are chosen)."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    s = softmax_rows(h @ w["router"].T)
    if gaps is not None:
        ranked = -np.sort(-s, axis=1)
        gaps.append((ranked[:, top - 1] - ranked[:, top]) / ranked[:, top - 1] if top < E else np.full(h.shape[0], np.inf))
    out = np.zeros((h.shape[0], w["e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e in np.argsort(-s[t], kind="stable")[:top]:
            out[t] += s[t, e] * gated_ff(h[t:t + 1], _sub(w, f"e{e}."))[0]
    return out


# ---------------------------------------------------------------------------
# the model
# ---------------------------------------------------------------------------
def _sub(w: Dict[str, np.ndarray], prefix: str) -> Dict[str, np.ndarray]:
    return {k[len(prefix):]: a for k, a in w.items() if k.startswith(prefix)}


def forward(cfg: dict, w: Dict[str, np.ndarray], ids, layers_out: Optional[List[np.ndarray]] = None,
            gaps: Optional[List[np.ndarray]] = None) -> np.ndarray:
    """Logits [T, vocab] of one sequence from its first token.  ``layers_out`` collects the
    residual stream after every layer, ``gaps`` every routed layer's margins (``routed_ff``)."""
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x = w["embed"][np.asarray(ids, dtype=np.int64)] * cfg["embedding"]["scale"]
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        mw, m = _sub(w, f"l{i}.mix."), layer["mixer"]
        if layer["type"] == "attention":
            if m.get("kv_from") is None:
                kept[i] = attention_keys_values(x, mw, m, eps)
            y = qknorm_attention(x, mw, m, eps, kept[i if m.get("kv_from") is None else m["kv_from"]])
        elif layer["type"] == "latent_attention":
            y = latent_attention(x, mw, m, eps)
        elif layer["type"] == "retention":
            y = retention(x, mw, m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + mult * unit(y, eps) * (1.0 + w[f"l{i}.norm1"])
        mlp = layer.get("mlp")
        if mlp is not None:
            fw = _sub(w, f"l{i}.mlp.")
            y = gated_ff(x, fw) if mlp["kind"] == "dense" else routed_ff(x, fw, mlp, gaps)
            x = x + mult * unit(y, eps) * (1.0 + w[f"l{i}.norm2"])
        if layers_out is not None:
            layers_out.append(x.copy())
    return (unit(x, eps) * (1.0 + w["final.norm"])) @ w["head"].T


def greedy(logits: np.ndarray) -> int:
    return int(np.argmax(logits))
