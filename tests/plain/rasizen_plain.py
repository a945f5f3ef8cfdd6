"""A plain, slow implementation of the Rasizen decoder.

Whole sequences, no cache, no state carried between calls, one function per mechanism, NumPy in
float64 throughout.  It shares no code with ``sonicboom_amd``: the configuration is the dict of
config.json and the weights a dict of arrays by the file's tensor names.

The design in this file's notation (``n`` tokens, position t = 0 .. n-1, stream x [n, width]):

* a layer: x += m * mixer(gnorm(x, norm1)); and, if it has a feed-forward, x += m * ff(gnorm(x, norm2));
  m = ``residual_mult``.
* gnorm: the vector in ``norm.groups`` consecutive parts, each part divided by sqrt(mean(part^2) + eps),
  the whole times the weight.
* mixer ``mingru``: z = sigmoid(Wz h + bz), u = Wx h + bx, cand = u + 1/2 (u >= 0) or sigmoid(u) (u < 0),
  S_t = (1 - z_t) S_{t-1} + z_t cand_t from S = 0, output Wo (S_t * silu(Wg h_t)).
* mixer ``latent_attention``: queries q = Wq h, per head [dim plain | rot_dim rotated]; W_dkv h gives
  kv_rank numbers that are RMS-normed (weight, the layer's eps) into the latent c, and rot_dim more that
  are rotated into a key part r shared by the heads; head a: key [W_uk,a c | r], value W_uv,a c; position t
  sees s with 0 <= t - s < window; softmax of scale * q.k; the heads' results times sigmoid(Wg h), then Wo.
  A mixer with ``kv_from`` takes c and r of that earlier layer.
* rotation: pairs (2i, 2i + 1) of the first ``rot.dims`` numbers turn by the angle t * base^(-2i / dims).
* feed-forward ``dense``: W_down act(W_up h), act(z) = softplus(p) z^2 + z/2 for z > 0 and
  (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2 else, (p, q) the two numbers of ``act``.
* logits: gnorm(x, final.norm) times the embedding table.
"""
from __future__ import annotations

import numpy as np

F64 = np.float64


def sigmoid(a):
    a = np.asarray(a, dtype=F64)
    return 1.0 / (1.0 + np.exp(-a))


def softplus(a):
    return np.logaddexp(0.0, np.asarray(a, dtype=F64))


def grouped_rms_norm(x, weight, eps: float, groups: int = 1):
    x = np.asarray(x, dtype=F64)
    n = x.shape[-1]
    parts = x.reshape(*x.shape[:-1], groups, n // groups)
    parts = parts / np.sqrt((parts * parts).mean(-1, keepdims=True) + eps)
    y = parts.reshape(x.shape)
    return y if weight is None else y * np.asarray(weight, dtype=F64)


def linear(x, weight, bias=None):
    y = np.asarray(x, dtype=F64) @ np.asarray(weight, dtype=F64).T
    return y if bias is None else y + np.asarray(bias, dtype=F64)


def rotate_pairs(x, positions, dims: int, base: float):
    """Turn the pairs (2i, 2i+1), i < dims/2, of the last axis of ``x`` [n, ..., d]; the rest passes."""
    x = np.array(x, dtype=F64)
    pos = np.asarray(positions, dtype=F64).reshape((-1,) + (1,) * (x.ndim - 2))
    for i in range(dims // 2):
        a = pos * F64(base) ** (-2.0 * i / dims)
        u, v = x[..., 2 * i].copy(), x[..., 2 * i + 1].copy()
        x[..., 2 * i] = u * np.cos(a) - v * np.sin(a)
        x[..., 2 * i + 1] = v * np.cos(a) + u * np.sin(a)
    return x


def mingru_gates(h, w, p):
    """(z, candidate) [n, width] of the gated recurrence."""
    z = sigmoid(linear(h, w[p + "z"], w[p + "z.b"]))
    u = linear(h, w[p + "x"], w[p + "x.b"])
    cand = np.where(u >= 0, u + 0.5, sigmoid(u))
    return z, cand


def mingru_scan(z, cand, start=None):
    """S_t = (1 - z_t) S_{t-1} + z_t cand_t, token after token; returns all S_t [n, width]."""
    s = np.zeros(z.shape[1], dtype=F64) if start is None else np.asarray(start, dtype=F64)
    out = np.empty_like(z)
    for t in range(z.shape[0]):
        s = (1.0 - z[t]) * s + z[t] * cand[t]
        out[t] = s
    return out


def mingru_mixer(h, w, p):
    z, cand = mingru_gates(h, w, p)
    s = mingru_scan(z, cand)
    g = linear(h, w[p + "g"])
    return linear(s * (g * sigmoid(g)), w[p + "o"])


def latent_kv(h, positions, w, p, mx, eps):
    """What a latent-attention layer keeps per token: (c [n, kv_rank], r [n, rot_dim])."""
    rank = mx["kv_rank"]
    d = linear(h, w[p + "dkv"])
    c = grouped_rms_norm(d[:, :rank], w[p + "dkv.norm"], eps, 1)
    r = rotate_pairs(d[:, rank:], positions, mx["rot"]["dims"], mx["rot"]["base"])
    return c, r


def windowed_softmax_attention(q, k, v, scale: float, window: int):
    """q, k [n, heads, dk], v [n, heads, dv]; token t sees s with 0 <= t - s < window (0: all before it)."""
    n, heads = q.shape[:2]
    out = np.zeros((n, heads, v.shape[-1]), dtype=F64)
    for t in range(n):
        lo = 0 if window <= 0 else max(0, t - window + 1)
        for a in range(heads):
            s = (k[lo:t + 1, a] @ q[t, a]) * scale
            e = np.exp(s - s.max())
            out[t, a] = (e / e.sum()) @ v[lo:t + 1, a]
    return out


def latent_attention_mixer(h, positions, w, p, mx, eps, kv):
    """``kv``: (c, r) of this layer or of the layer it reads."""
    H, dim, rot, vdim = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"]
    n = h.shape[0]
    c, r = kv
    q = linear(h, w[p + "q"]).reshape(n, H, dim + rot)
    q = np.concatenate([q[..., :dim], rotate_pairs(q[..., dim:], positions, mx["rot"]["dims"], mx["rot"]["base"])], -1)
    k = np.concatenate([linear(c, w[p + "uk"]).reshape(n, H, dim), np.repeat(r[:, None, :], H, 1)], -1)
    v = linear(c, w[p + "uv"]).reshape(n, H, vdim)
    window = int((mx.get("mask") or {}).get("size", 0) or 0)
    a = windowed_softmax_attention(q, k, v, mx["scale"], window).reshape(n, H * vdim)
    return linear(a * sigmoid(linear(h, w[p + "g"])), w[p + "o"])


def xielu(z, p, q):
    z = np.asarray(z, dtype=F64)
    neg = np.minimum(z, 0.0)
    return np.where(z > 0, softplus(p) * z * z + z / 2, (0.5 + softplus(q)) * np.expm1(neg) - (0.5 + softplus(q)) * neg + z / 2)


def dense_ff(h, w, p):
    act = np.asarray(w[p + "act"], dtype=F64)
    return linear(xielu(linear(h, w[p + "up"]), act[0], act[1]), w[p + "down"])


def forward(cfg: dict, w: dict, tokens, return_layers: bool = False):
    """Logits [n, vocab] of one whole sequence (and the stream after every layer)."""
    tokens = np.asarray(tokens, dtype=np.int64)
    pos = np.arange(len(tokens))
    eps, groups, m = cfg["norm"]["eps"], cfg["norm"]["groups"], cfg["residual_mult"]
    x = np.asarray(w["embed"], dtype=F64)[tokens]
    kept, layers = {}, []
    for i, layer in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", layer["mixer"]
        h = grouped_rms_norm(x, w[p + "norm1"], eps, groups)
        if layer["type"] == "mingru":
            y = mingru_mixer(h, w, p + "mix.")
        elif layer["type"] == "latent_attention":
            src = mx.get("kv_from")
            kept[i] = kept[src] if src is not None else latent_kv(h, pos, w, p + "mix.", mx, eps)
            y = latent_attention_mixer(h, pos, w, p + "mix.", mx, eps, kept[i])
        else:
            raise ValueError(f"unknown layer type {layer['type']!r}")
        x = x + m * y
        if layer.get("mlp") is not None:
            x = x + m * dense_ff(grouped_rms_norm(x, w[p + "norm2"], eps, groups), w, p + "mlp.")
        layers.append(x.copy())
    logits = linear(grouped_rms_norm(x, w["final.norm"], eps, groups), w["embed"])
    return (logits, layers) if return_layers else logits


def greedy(cfg: dict, w: dict, prompt, n_new: int):
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(np.argmax(forward(cfg, w, tokens)[-1])))
    return tokens[len(prompt):]
