"""A plain, slow float64 implementation of the Fekizen decoder, one function per mechanism, written
from the model's equations and sharing no code with distributed_llms_amd: whole sequences only,
Python loops, no cache, no batching.  The tests compare the engine against it.

The model: token embedding times a scale plus a learned position vector, then an RMS norm; a list of
pre-norm layers, x += mixer(shift(norm1(x))), x += ff(norm2(x)), where ``shift`` blends every channel of
the mixer's input with the previous token's; a span of the list may run several times with the same
weights (the embedding output and a per-pass vector are added on entry).  Mixers: "lightning" (linear
attention with one fixed decay per head) and "parallel" -- softmax attention over a sliding window plus
one averaged key per block of older tokens, with a score cap and a per-head sink, values = unrotated
keys, beside gated linear attention with a decay per key channel; the two outputs are normed apart and
averaged.  Feed-forward: a mixture of SwiGLU experts (softmax over the chosen logits) and a shared one.

Checkpoint names: embed, pos, embed.norm, loop.step, final.norm, head, l<i>.norm1, l<i>.norm2, l<i>.shift,
l<i>.mix.*, l<i>.mlp.*.  Linear weights are [out, in].
"""
import math

import numpy as np


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def sub(w, prefix):
    """The tensors under ``prefix`` with the prefix taken off."""
    return {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}


def embed_tokens(tokens, sd, scale, eps, first_pos=0):
    t = len(tokens)
    x = sd["embed"][np.asarray(tokens)] * scale + sd["pos"][first_pos:first_pos + t]
    return rms(x, eps) * sd["embed.norm"]


def token_shift(h, w):
    """h [T, W]: every token's row is blended with the row before it (zeros before the first):
    h_t + (h_(t-1) - h_t) * w, the rows on the right being the unblended ones."""
    prev = np.concatenate([np.zeros_like(h[:1]), h[:-1]], 0)
    return h + (prev - h) * w


def blended_frequencies(rot):
    """(f [dims / 2], magnitude) of a rotation: f_i = base^(-2i / dims); with ``scaling`` (factor, original,
    fast, slow) the slow frequencies are divided by factor, blended over a ramp between the dimensions
    that make ``fast`` and ``slow`` turns inside ``original`` positions; cos and sin are then multiplied by
    0.1 ln(factor) + 1."""
    dims, base = rot["dims"], rot["base"]
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0

    def dim_of(turns):
        return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))
    lo = max(math.floor(dim_of(sc["fast"])), 0)
    hi = min(math.ceil(dim_of(sc["slow"])), dims - 1)
    out = f.copy()
    for i in range(dims // 2):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out[i] = f[i] / sc["factor"] * ramp + f[i] * (1 - ramp)
    return out, 0.1 * math.log(sc["factor"]) + 1.0


def rotate_half(x, rot, first_pos=0):
    """x [T, heads, D]: dimension i < dims / 2 of every head is paired with dimension i + dims / 2 and the
    pair turns by the angle p * f_i; dimensions from ``dims`` on pass unchanged."""
    f, mag = blended_frequencies(rot)
    half = rot["dims"] // 2
    out = x.copy()
    for t in range(x.shape[0]):
        p = first_pos + t
        for i in range(half):
            c, s = math.cos(p * f[i]) * mag, math.sin(p * f[i]) * mag
            u, v = x[t, :, i], x[t, :, i + half]
            out[t, :, i] = u * c - v * s
            out[t, :, i + half] = v * c + u * s
    return out


def visible_blocks(i, size, pool):
    """How many averaged blocks of ``pool`` positions query position i sees: block b (positions b pool ..
    b pool + pool - 1) counts once its last position has left the window, b pool + pool - 1 <= i - size."""
    n = 0
    while n * pool + pool - 1 <= i - size:
        n += 1
    return n


def pooled_window_attention(h, w, m):
    """h [T, W]; w: q, k, sink, o; m: heads, kv_heads, dim, vdim, rot, scale, softcap, mask {size, pool}.
    Values are the keys before their rotation."""
    t = h.shape[0]
    hh, g, d = m["heads"], m["kv_heads"], m["dim"]
    size, pool, cap = m["mask"]["size"], m["mask"]["pool"], m["softcap"]
    k_raw = (h @ w["k"].T).reshape(t, g, d)
    q = rotate_half((h @ w["q"].T).reshape(t, hh, d), m["rot"])
    k = rotate_half(k_raw, m["rot"])
    v = k_raw
    nb = t // pool
    kp = np.stack([k[b * pool:(b + 1) * pool].mean(0) for b in range(nb)]) if nb else np.zeros((0, g, d))
    vp = np.stack([v[b * pool:(b + 1) * pool].mean(0) for b in range(nb)]) if nb else np.zeros((0, g, d))
    out = np.zeros((t, hh, d))
    for a in range(hh):
        kv = a // (hh // g)
        for i in range(t):
            lo = max(0, i - size + 1)
            n = visible_blocks(i, size, pool)
            keys = np.concatenate([kp[:n, kv], k[lo:i + 1, kv]], 0)
            vals = np.concatenate([vp[:n, kv], v[lo:i + 1, kv]], 0)
            s = (keys @ q[i, a]) * m["scale"]
            s = cap * np.tanh(s / cap)
            top = max(s.max(), w["sink"][a])
            e = np.exp(s - top)
            out[i, a] = (e @ vals) / (e.sum() + math.exp(w["sink"][a] - top))
    return out.reshape(t, hh * d) @ w["o"].T


def decayed_outer_scan(q, k, v, a):
    """One head.  q, k [T, dim], v [T, vdim], a [T, dim] (a decay per key channel and token):
    S <- diag(a_t) S + k_t v_t^T;  o_t = S^T q_t.  Returns o [T, vdim]."""
    s = np.zeros((q.shape[1], v.shape[1]))
    o = np.zeros_like(v)
    for i in range(q.shape[0]):
        s = a[i][:, None] * s + np.outer(k[i], v[i])
        o[i] = s.T @ q[i]
    return o


def gated_linear_attention(h, w, m, eps):
    """h [T, W]; w: q, k, v, g, o, norm, a1, a2, a2.b; m: heads, dim, vdim, tau."""
    t = h.shape[0]
    hh, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).reshape(t, hh, d) * d ** -0.5
    k = (h @ w["k"].T).reshape(t, hh, d)
    v = (h @ w["v"].T).reshape(t, hh, dv)
    z = (h @ w["a1"].T) @ w["a2"].T + w["a2.b"]
    alpha = (sigmoid(z) ** (1.0 / m["tau"])).reshape(t, hh, d)
    gate = silu(h @ w["g"].T).reshape(t, hh, dv)
    out = np.zeros((t, hh, dv))
    for a in range(hh):
        o = decayed_outer_scan(q[:, a], k[:, a], v[:, a], alpha[:, a])
        out[:, a] = rms(o, eps) * w["norm"] * gate[:, a]
    return out.reshape(t, hh * dv) @ w["o"].T


def parallel_mixer(h, w, m, eps):
    left = pooled_window_attention(h, sub(w, "left."), m["left"])
    right = gated_linear_attention(h, sub(w, "right."), m["right"], eps)
    return 0.5 * (rms(left, eps) * w["left.out"] + rms(right, eps) * w["right.out"])


def lightning_mixer(h, w, m, eps):
    """h [T, W]; w: q, k, v, g, o, norm; m: heads, dim, vdim, decay [heads]."""
    t = h.shape[0]
    hh, d, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w["q"].T).reshape(t, hh, d)
    k = silu(h @ w["k"].T).reshape(t, hh, d)
    v = silu(h @ w["v"].T).reshape(t, hh, dv)
    out = np.zeros((t, hh, dv))
    for a in range(hh):
        out[:, a] = decayed_outer_scan(q[:, a], k[:, a], v[:, a], np.full((t, d), m["decay"][a]))
    y = rms(out.reshape(t, hh * dv), eps) * w["norm"] * sigmoid(h @ w["g"].T)
    return y @ w["o"].T


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
    z = h @ w["router"].T
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


def layer_runs(cfg):
    """[(layer index, pass number or None)]: the order in which layers run; a pass number marks the first
    layer of a pass through the looped span."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    runs = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        runs += [(i, t if i == loop["start"] else None) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, None) for i in range(loop["stop"], n)]


def shapes(cfg):
    """Checkpoint name -> shape."""
    w = cfg["width"]
    s = {"embed": (cfg["vocab"], w), "pos": (cfg["max_positions"], w), "embed.norm": (w,), "final.norm": (w,),
         "head": (cfg["vocab"], w)}
    if cfg.get("loop"):
        s["loop.step"] = (cfg["loop"]["times"], w)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        s.update({p + "norm1": (w,), p + "shift": (w,)})
        if layer["type"] == "lightning":
            qk, vv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            s.update({p + "mix.q": (qk, w), p + "mix.k": (qk, w), p + "mix.v": (vv, w), p + "mix.g": (vv, w),
                      p + "mix.o": (w, vv), p + "mix.norm": (vv,)})
        else:
            l, r = m["left"], m["right"]
            s.update({p + "mix.left.q": (l["heads"] * l["dim"], w), p + "mix.left.k": (l["kv_heads"] * l["dim"], w),
                      p + "mix.left.sink": (l["heads"],), p + "mix.left.o": (w, l["heads"] * l["vdim"]),
                      p + "mix.left.out": (w,), p + "mix.right.out": (w,)})
            qk, vv = r["heads"] * r["dim"], r["heads"] * r["vdim"]
            rank = r.get("rank", 8)
            s.update({p + "mix.right.q": (qk, w), p + "mix.right.k": (qk, w), p + "mix.right.v": (vv, w),
                      p + "mix.right.g": (vv, w), p + "mix.right.o": (w, vv), p + "mix.right.norm": (r["vdim"],),
                      p + "mix.right.a1": (rank, w), p + "mix.right.a2": (qk, rank), p + "mix.right.a2.b": (qk,)})
        mlp = layer.get("mlp")
        if not mlp:
            continue
        s[p + "norm2"] = (w,)
        f = mlp["expert"]["ff"]
        s[p + "mlp.router"] = (mlp["router"]["experts"], w)
        for j in range(mlp["router"]["experts"]):
            s.update({p + f"mlp.e{j}.gate": (f, w), p + f"mlp.e{j}.up": (f, w), p + f"mlp.e{j}.down": (w, f)})
        if mlp.get("shared"):
            fs = mlp["shared"]["ff"]
            s.update({p + "mlp.shared.gate": (fs, w), p + "mlp.shared.up": (fs, w), p + "mlp.shared.down": (w, fs)})
    return s


def make_weights(cfg, seed=0):
    """Random float64 weights under the checkpoint names: projections ~ N(0, 1 / fan_in), norm weights
    around one, shift weights in (0, 1), sinks and decay biases of moderate size, a router wide enough
    that few choices are close calls."""
    rng = np.random.default_rng(seed)
    sd = {}
    for name, shape in shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        if leaf in ("norm1", "norm2", "norm", "out") or name in ("embed.norm", "final.norm"):
            t = 1.0 + 0.2 * rng.standard_normal(shape)
        elif leaf == "shift":
            t = rng.uniform(0.0, 1.0, shape)
        elif leaf == "sink":
            t = rng.standard_normal(shape)
        elif name.endswith("a2.b"):
            t = 2.0 + rng.standard_normal(shape)
        elif leaf == "router":
            t = 4.0 * rng.standard_normal(shape) / shape[-1] ** 0.5
        elif name == "embed":
            t = rng.standard_normal(shape) / cfg["embedding"]["scale"]
        elif name in ("pos", "loop.step"):
            t = 0.3 * rng.standard_normal(shape)
        else:
            t = rng.standard_normal(shape) / shape[-1] ** 0.5
        sd[name] = t
    return sd


def forward(cfg, sd, tokens, taps=None, margins=None):
    """Logits [T, vocab] of one whole sequence.  ``sd``: checkpoint name -> float64 array.  ``taps``: a
    list that receives the stream after every layer run; ``margins``: one that receives every router's."""
    eps = cfg["norm"]["eps"]
    x0 = embed_tokens(tokens, sd, cfg["embedding"]["scale"], eps)
    x = x0.copy()
    for i, enters in layer_runs(cfg):
        layer, w = cfg["layers"][i], sub(sd, f"l{i}.")
        if enters is not None:
            if enters > 0:
                x = x + x0
            x = x + sd["loop.step"][enters]
        h = token_shift(rms(x, eps) * w["norm1"], w["shift"])
        if layer["type"] == "lightning":
            x = x + lightning_mixer(h, sub(w, "mix."), layer["mixer"], eps)
        elif layer["type"] == "parallel":
            x = x + parallel_mixer(h, sub(w, "mix."), layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        mlp = layer.get("mlp")
        if mlp:
            x = x + moe_ff(rms(x, eps) * w["norm2"], sub(w, "mlp."), mlp, margins)
        if taps is not None:
            taps.append(x.copy())
    return (rms(x, eps) * sd["final.norm"]) @ sd["head"].T
