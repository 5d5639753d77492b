"""A plain, slow float64 implementation of the Zebutar decoder, one function per mechanism, written
from the model's equations and sharing no code with distributed_llms_amd: whole sequences only,
Python loops, no cache, no batching.  The tests compare the engine against it.

The model: token embedding followed by an RMS norm; a list of layers in which the sublayers read the
stream itself and only their OUTPUT is normed, x += norm1(mixer(x)), x += norm2(ff(x)); a mixer made
of two mixers side by side on the same input -- softmax attention inside fixed chunks of positions
(grouped K/V heads, an RMS norm over the whole query and the whole key projection, a half-split
rotation of part of every head) and a gated delta rule (short causal convolutions with silu, unit
queries and keys, a per-head decay and write strength, a gated per-head output norm) -- summed with
two fixed scales; feed-forwards that are absent, a squared-ReLU pair of matrices, or a mixture of
SwiGLU experts (biased router, softmax over the chosen logits, a shared expert); a final norm and
the output head.

Checkpoint names: embed, embed.norm, final.norm, head, l<i>.norm1, l<i>.norm2, l<i>.mix.left.*,
l<i>.mix.right.*, l<i>.mlp.*.  Linear weights are [out, in].
"""
import math

import numpy as np


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def norm_one_plus(x, w, eps):
    """The layer norm of this design: the weight is stored around zero."""
    return rms(x, eps) * (1.0 + w)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.log1p(np.exp(-np.abs(z))) + np.maximum(z, 0.0)


def rotate_half(x, base, dims, first_pos=0):
    """x [T, heads, D]: dimension i < dims / 2 of every head is paired with dimension i + dims / 2; the
    pair turns by the angle p * base^(-2i / dims), p the token's position.  Dimensions from ``dims`` on
    pass unchanged."""
    out = x.copy()
    half = dims // 2
    for t in range(x.shape[0]):
        p = first_pos + t
        for i in range(half):
            a = p * base ** (-2.0 * i / dims)
            u, v = x[t, :, i], x[t, :, i + half]
            out[t, :, i] = u * math.cos(a) - v * math.sin(a)
            out[t, :, i + half] = v * math.cos(a) + u * math.sin(a)
    return out


def first_visible(i, size):
    """Query position i sees the key positions j <= i of its own chunk of ``size`` positions, chunks
    counted from position 0: j >= floor(i / size) * size (size None or 0: plain causal, j >= 0)."""
    return (i // size) * size if size else 0


def chunked_attention(h, w, m, eps):
    """h [T, W]; w: q, k, v, q.norm, k.norm, o; m: heads, kv_heads, dim, vdim, rot {base, dims}, scale,
    mask {size}."""
    t = h.shape[0]
    hh, g, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms(h @ w["q"].T, eps) * w["q.norm"]            # over the whole projection, plain weight
    k = rms(h @ w["k"].T, eps) * w["k.norm"]
    v = (h @ w["v"].T).reshape(t, g, dv)
    q = rotate_half(q.reshape(t, hh, d), m["rot"]["base"], m["rot"]["dims"])
    k = rotate_half(k.reshape(t, g, d), m["rot"]["base"], m["rot"]["dims"])
    size = (m.get("mask") or {}).get("size")
    out = np.zeros((t, hh, dv))
    for a in range(hh):
        kv = a // (hh // g)
        for i in range(t):
            lo = first_visible(i, size)
            s = (k[lo:i + 1, kv] @ q[i, a]) * m["scale"]
            e = np.exp(s - s.max())
            out[i, a] = (e / e.sum()) @ v[lo:i + 1, kv]
    return out.reshape(t, hh * dv) @ w["o"].T


def short_conv(x, wc):
    """x [T, C], wc [C, taps]: y_t = sum_j wc[:, j] x_(t - taps + 1 + j), zeros before the start."""
    t, c = x.shape
    taps = wc.shape[1]
    y = np.zeros((t, c))
    for i in range(t):
        for j in range(taps):
            s = i - (taps - 1) + j
            if s >= 0:
                y[i] += wc[:, j] * x[s]
    return y


def delta_rule(q, k, v, beta, g):
    """One head.  q, k [T, dim], v [T, vdim], beta, g [T].  S <- g S;  u = beta (v - S^T k);
    S <- S + k u^T;  o = S^T q (the read-out sees the token's own write).  Returns o [T, vdim]."""
    t, d = q.shape
    s = np.zeros((d, v.shape[1]))
    o = np.zeros_like(v)
    for i in range(t):
        s = g[i] * s
        u = beta[i] * (v[i] - s.T @ k[i])
        s = s + np.outer(k[i], u)
        o[i] = s.T @ q[i]
    return o


def gated_delta_mixer(h, w, m, eps):
    """h [T, W]; w: q, k, v (+ .conv), b, a, A_log, dt_bias, g, norm, o; m: heads, kv_heads, dim, vdim, conv."""
    t = h.shape[0]
    hh, g, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ w["q"].T, w["q.conv"])).reshape(t, g, d)
    k = silu(short_conv(h @ w["k"].T, w["k.conv"])).reshape(t, g, d)
    v = silu(short_conv(h @ w["v"].T, w["v.conv"])).reshape(t, hh, dv)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * d ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    beta = sigmoid(h @ w["b"].T)                                                # [T, heads]
    decay = np.exp(-np.exp(w["A_log"]) * softplus(h @ w["a"].T + w["dt_bias"]))  # [T, heads]
    gate = silu(h @ w["g"].T).reshape(t, hh, dv)
    out = np.zeros((t, hh, dv))
    for a in range(hh):
        kv = a // (hh // g)
        o = delta_rule(q[:, kv], k[:, kv], v[:, a], beta[:, a], decay[:, a])
        out[:, a] = rms(o, eps) * w["norm"] * gate[:, a]
    return out.reshape(t, hh * dv) @ w["o"].T


def sub(w, prefix):
    """The tensors under ``prefix`` with the prefix taken off."""
    return {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}


def parallel_mixer(h, w, m, eps):
    left = chunked_attention(h, sub(w, "left."), m["left"], eps)
    right = gated_delta_mixer(h, sub(w, "right."), m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


def dense_ff(h, w):
    return np.square(np.maximum(h @ w["up"].T, 0.0)) @ w["down"].T


def glu_expert(h, w):
    return (silu(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def route_top(z, top):
    """z [E] router logits -> (indices of the ``top`` largest, softmax over those logits only)."""
    idx = np.argsort(-z, kind="stable")[:top]
    e = np.exp(z[idx] - z[idx].max())
    return idx, e / e.sum()


def moe_ff(h, w, mlp, margins=None):
    """``margins``: a list that receives, per token, the gap between the last chosen logit and the best
    one left out (how far the choice is from turning over)."""
    out = np.zeros_like(h)
    z = h @ w["router"].T + w["router.b"]
    top = mlp["router"]["top"]
    if margins is not None:
        zs = -np.sort(-z, axis=-1)
        margins.append(zs[:, top - 1] - zs[:, top] if top < z.shape[1] else np.full(h.shape[0], np.inf))
    for i in range(h.shape[0]):
        idx, p = route_top(z[i], top)
        for j, pj in zip(idx, p):
            out[i] += pj * glu_expert(h[i:i + 1], sub(w, f"e{j}."))[0]
    if mlp.get("shared"):
        out += glu_expert(h, sub(w, "shared."))
    return out


def shapes(cfg):
    """Checkpoint name -> shape."""
    w = cfg["width"]
    s = {"embed": (cfg["vocab"], w), "embed.norm": (w,), "final.norm": (w,), "head": (cfg["vocab"], w)}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        l, r = layer["mixer"]["left"], layer["mixer"]["right"]
        s[p + "norm1"] = (w,)
        s.update({p + "mix.left.q": (l["heads"] * l["dim"], w), p + "mix.left.k": (l["kv_heads"] * l["dim"], w),
                  p + "mix.left.v": (l["kv_heads"] * l["vdim"], w), p + "mix.left.q.norm": (l["heads"] * l["dim"],),
                  p + "mix.left.k.norm": (l["kv_heads"] * l["dim"],), p + "mix.left.o": (w, l["heads"] * l["vdim"])})
        qk, vv = r["kv_heads"] * r["dim"], r["heads"] * r["vdim"]
        s.update({p + "mix.right.q": (qk, w), p + "mix.right.q.conv": (qk, r["conv"]), p + "mix.right.k": (qk, w),
                  p + "mix.right.k.conv": (qk, r["conv"]), p + "mix.right.v": (vv, w),
                  p + "mix.right.v.conv": (vv, r["conv"]), p + "mix.right.b": (r["heads"], w),
                  p + "mix.right.a": (r["heads"], w), p + "mix.right.A_log": (r["heads"],),
                  p + "mix.right.dt_bias": (r["heads"],), p + "mix.right.g": (vv, w), p + "mix.right.norm": (r["vdim"],),
                  p + "mix.right.o": (w, vv)})
        mlp = layer.get("mlp")
        if not mlp:
            continue
        s[p + "norm2"] = (w,)
        if mlp["kind"] == "dense":
            s.update({p + "mlp.up": (mlp["ff"], w), p + "mlp.down": (w, mlp["ff"])})
        else:
            f = mlp["expert"]["ff"]
            s.update({p + "mlp.router": (mlp["router"]["experts"], w), p + "mlp.router.b": (mlp["router"]["experts"],)})
            for j in range(mlp["router"]["experts"]):
                s.update({p + f"mlp.e{j}.gate": (f, w), p + f"mlp.e{j}.up": (f, w), p + f"mlp.e{j}.down": (w, f)})
            if mlp.get("shared"):
                fs = mlp["shared"]["ff"]
                s.update({p + "mlp.shared.gate": (fs, w), p + "mlp.shared.up": (fs, w), p + "mlp.shared.down": (w, fs)})
    return s


def make_weights(cfg, seed=0):
    """Random float64 weights under the checkpoint names: projections ~ N(0, 1 / fan_in), stream norms
    stored around zero, plain norms around one, decays from slow to fast per head, a router wide enough
    that few choices are close calls."""
    rng = np.random.default_rng(seed)
    sd = {}
    for name, shape in shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        if leaf in ("norm1", "norm2") or name in ("embed.norm", "final.norm"):
            t = 0.15 * rng.standard_normal(shape)
        elif leaf == "norm":
            t = 1.0 + 0.2 * rng.standard_normal(shape)
        elif leaf == "A_log":
            t = rng.uniform(-4.0, 0.5, shape)
        elif leaf == "dt_bias":
            t = rng.standard_normal(shape)
        elif leaf == "conv":
            t = rng.standard_normal(shape) / shape[1] ** 0.5
        elif name.endswith("router.b"):
            t = 0.5 * rng.standard_normal(shape)
        elif leaf == "router":
            t = 4.0 * rng.standard_normal(shape) / shape[-1] ** 0.5
        elif name == "embed":
            t = rng.standard_normal(shape)
        else:
            t = rng.standard_normal(shape) / shape[-1] ** 0.5
        sd[name] = t
    return sd


def forward(cfg, sd, tokens, taps=None, margins=None):
    """Logits [T, vocab] of one whole sequence.  ``sd``: checkpoint name -> float64 array.  ``taps``: a
    list that receives the stream after every layer; ``margins``: one that receives every router's."""
    eps = cfg["norm"]["eps"]
    x = norm_one_plus(sd["embed"][np.asarray(tokens)], sd["embed.norm"], eps)
    for i, layer in enumerate(cfg["layers"]):
        w = sub(sd, f"l{i}.")
        if layer["type"] != "parallel":
            raise ValueError(layer["type"])
        x = x + norm_one_plus(parallel_mixer(x, sub(w, "mix."), layer["mixer"], eps), w["norm1"], eps)
        mlp = layer.get("mlp")
        if mlp:
            f = dense_ff(x, sub(w, "mlp.")) if mlp["kind"] == "dense" else moe_ff(x, sub(w, "mlp."), mlp, margins)
            x = x + norm_one_plus(f, w["norm2"], eps)
        if taps is not None:
            taps.append(x.copy())
    return norm_one_plus(x, sd["final.norm"], eps) @ sd["head"].T
