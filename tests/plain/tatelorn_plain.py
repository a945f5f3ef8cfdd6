"""A plain, slow implementation of the Tatelorn decoder.

Whole sequences, no cache, one function per mechanism, NumPy in float64 throughout.  It shares no
code with ``sonicboom_amd``: the configuration is the dict of config.json and the weights a dict of
arrays by the file's tensor names.

The design in this file's notation (``n`` tokens, position t = 0 .. n-1, stream x [n, width]):

* unit norm: un(v, w) = v / sqrt(mean(v^2) + eps) * (1 + w); the file keeps the multiplier minus one.
* start: x = un(table[token] * embedding.scale + pos[t], embed.norm).
* a layer reads the stream as it is and norms what comes out of a sublayer:
  x += un(mixer(x), norm1); and, if it has a feed-forward, x += un(ff(x), norm2).
* mixer ``attention``: q = Wq x, k = Wk x, v = Wv x; every head of q and of k is divided by its root
  mean square (eps inside the root) and multiplied by a weight of the head's size that all heads share
  (no one-plus here); nothing rotates.  s(t, j) = cap * tanh(scale * q_t.k_j / cap) for j <= t (no cap: as it is);
  the weights are exp(s_j) / (1 + sum_j exp(s_j)): a key of score 0 without a value takes part.
  Query head a reads key/value head a // (heads / kv_heads).  Layers that mix values: all of them but
  the first replace v by (1 - lam) v + lam v0, v0 the first such layer's v of the same token, lam the
  layer's number.  Then Wo.
* feed-forward ``dense``: Wdown (relu(Wgate x) * (Wup x)).
* feed-forward ``moe``: z = Wrouter x; the ``top`` largest z are chosen, their weights are the softmax
  over the chosen z alone; an expert is Wdown y, y = g * sigmoid(1.702 g) * (u + 1) with
  g = min(Wgate x, limit), u = clip(Wup x, -limit, limit); the result is the weighted sum of the chosen
  experts plus, if there is one, sigmoid(Wsg x) times a shared expert of the same form.
* logits: un(x, final.norm) times the table (unscaled), times logit_scale.
"""
from __future__ import annotations

import numpy as np

F64 = np.float64


def sigmoid(a):
    a = np.asarray(a, dtype=F64)
    return 1.0 / (1.0 + np.exp(-a))


def linear(x, weight):
    return np.asarray(x, dtype=F64) @ np.asarray(weight, dtype=F64).T


def rms_divide(v, eps: float):
    v = np.asarray(v, dtype=F64)
    return v / np.sqrt((v * v).mean(-1, keepdims=True) + eps)


def unit_norm(v, weight, eps: float):
    """The file keeps the multiplier minus one."""
    return rms_divide(v, eps) * (1.0 + np.asarray(weight, dtype=F64))


def head_norm(v, weight, eps: float):
    """Per head, plain weight shared by the heads: v [n, heads, dim]."""
    return rms_divide(v, eps) * np.asarray(weight, dtype=F64)


def start(cfg, w, tokens, first_position: int = 0):
    t = np.arange(first_position, first_position + len(tokens))
    x = np.asarray(w["embed"], dtype=F64)[np.asarray(tokens)] * F64(cfg["embedding"]["scale"])
    x = x + np.asarray(w["pos"], dtype=F64)[t]
    return unit_norm(x, w["embed.norm"], cfg["norm"]["eps"])


def capped_scores(q, k, scale: float, cap: float):
    """q [n, dim], k [m, dim] -> [n, m]; a cap of 0 (or none) leaves the scores as they are."""
    s = (q @ k.T) * F64(scale)
    return F64(cap) * np.tanh(s / F64(cap)) if cap else s


def sink_softmax(s, visible):
    """exp(s_j) / (1 + sum over visible j of exp(s_j)), row by row; hidden keys weigh nothing."""
    s = np.where(visible, s, -np.inf)
    m = np.maximum(s.max(-1, keepdims=True), 0.0)          # the sink's score is 0
    e = np.exp(s - m)
    return e / (np.exp(-m) + e.sum(-1, keepdims=True))


def attention_values(cfg_mixer, w, p, x, v_first):
    """The values this layer keeps, and what later mixing layers take as v0."""
    v = linear(x, w[p + "v"])
    if not cfg_mixer.get("v_mix"):
        return v, v_first
    if v_first is None:
        return v, v                                  # the first mixing layer: its own number is unused
    lam = F64(np.asarray(w[p + "vmix"], dtype=F64).reshape(()))
    return (1.0 - lam) * v + lam * v_first, v_first


def attention(cfg_mixer, eps, w, p, x, v_first=None, positions=None):
    """Returns (mixer output [n, width], v_first for the layers after)."""
    n = x.shape[0]
    H, G, D, E = cfg_mixer["heads"], cfg_mixer["kv_heads"], cfg_mixer["dim"], cfg_mixer["vdim"]
    q = head_norm(linear(x, w[p + "q"]).reshape(n, H, D), w[p + "q.norm"], eps)
    k = head_norm(linear(x, w[p + "k"]).reshape(n, G, D), w[p + "k.norm"], eps)
    v, v_first = attention_values(cfg_mixer, w, p, x, v_first)
    v = v.reshape(n, G, E)
    t = np.arange(n)
    visible = t[None, :] <= t[:, None]
    out = np.empty((n, H, E), dtype=F64)
    for a in range(H):
        g = a // (H // G)
        s = capped_scores(q[:, a], k[:, g], cfg_mixer["scale"], cfg_mixer["softcap"])
        out[:, a] = sink_softmax(s, visible) @ v[:, g]
    return linear(out.reshape(n, H * E), w[p + "o"]), v_first


def dense_ff(w, p, x):
    return linear(np.maximum(linear(x, w[p + "gate"]), 0.0) * linear(x, w[p + "up"]), w[p + "down"])


def expert(w, p, x, limit: float):
    g = np.minimum(linear(x, w[p + "gate"]), limit)
    u = np.clip(linear(x, w[p + "up"]), -limit, limit)
    return linear(g * sigmoid(1.702 * g) * (u + 1.0), w[p + "down"])


def route(z, top: int):
    """z [n, experts] -> (chosen [n, top] in falling order of z, weights [n, top])."""
    order = np.argsort(-z, axis=-1, kind="stable")[:, :top]
    zc = np.take_along_axis(z, order, axis=-1)
    e = np.exp(zc - zc.max(-1, keepdims=True))
    return order, e / e.sum(-1, keepdims=True)


def moe_ff(cfg_mlp, w, p, x):
    n = x.shape[0]
    z = linear(x, w[p + "router"])
    chosen, weight = route(z, cfg_mlp["router"]["top"])
    out = np.zeros((n, np.asarray(w[p + "e0.down"]).shape[0]), dtype=F64)
    for e in range(cfg_mlp["router"]["experts"]):
        rows, slot = np.nonzero(chosen == e)
        if len(rows):
            out[rows] += weight[rows, slot][:, None] * expert(w, f"{p}e{e}.", x[rows], cfg_mlp["expert"]["limit"])
    if cfg_mlp.get("shared"):
        gate = sigmoid(linear(x, w[p + "shared.sg"]))            # [n, 1]
        out += gate * expert(w, p + "shared.", x, cfg_mlp["shared"]["limit"])
    return out


def feed_forward(cfg_mlp, w, p, x):
    if cfg_mlp["kind"] == "dense":
        return dense_ff(w, p, x)
    if cfg_mlp["kind"] == "moe":
        return moe_ff(cfg_mlp, w, p, x)
    raise ValueError(f"no feed-forward of kind {cfg_mlp['kind']!r}")


def forward(cfg, w, tokens, layers_out=None):
    """Logits [n, vocab] of one whole sequence from position 0.  ``layers_out``: a list that
    receives the stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = start(cfg, w, tokens)
    v_first = None
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        if layer["type"] != "attention":
            raise ValueError(f"layer {i}: no mixer of type {layer['type']!r}")
        y, v_first = attention(layer["mixer"], eps, w, p + "mix.", x, v_first)
        x = x + unit_norm(y, w[p + "norm1"], eps)
        if layer.get("mlp"):
            x = x + unit_norm(feed_forward(layer["mlp"], w, p + "mlp.", x), w[p + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    h = unit_norm(x, w["final.norm"], eps)
    return linear(h, w["embed"]) * F64(cfg["logit_scale"])


def greedy(cfg, w, prompt, n: int):
    """``n`` tokens after ``prompt``, each the first largest logit of the whole sequence so far."""
    tokens, out = list(prompt), []
    for _ in range(n):
        t = int(np.argmax(forward(cfg, w, tokens)[-1]))
        out.append(t)
        tokens.append(t)
    return out
