"""Ops of layer-list models whose layers carry per-sequence state: a float32 residual stream with
pre- and post-sublayer RMS norms (also for sublayers that read the stream unnormed, and for two mixer
outputs summed with scales), short causal convolutions with a state tail, the real-gated linear
recurrent unit (RG-LRU), sliding-window and chunked attention over a paged K/V cache whose key and value
widths differ (optionally with capped scores, per-head sinks and one averaged key / value per block of
positions older than the window), two attention input stages (convolution + per-head norm + interleaved
rotation; whole-projection norm + half-split rotation, also without norms and with the values taken from
the keys), the close of pre-norm sublayers whose outputs are normed apart, a token shift, the entry of a
looped span of layers, a clipped GLU and the logit soft cap.

Same dispatch as :mod:`distributed_llms_amd.ops`: a CUDA tensor goes to the in-tree HIP kernels
(csrc/kernels/seqmix.hip, attention_window.hip) and raises if they are not built; CPU tensors run
the plain PyTorch forms below (the ``_ref_*`` functions).  Activations (``act``) are bfloat16 or
float32; what feeds a norm, a softmax, a rotation angle, a gate of the recurrence or the recurrent
state itself is float32 in both.

Varlen batches: a step's tokens are the concatenation of B sequence chunks, ``cu`` [B + 1] their
offsets, ``positions`` [T] each token's position in its sequence, ``tok_seq`` [T] its chunk,
``state_slots`` [B] the row of every state pool the sequence owns.  A chunk that starts at position
0 starts from zero state (its slot's previous content is never read).
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from .. import _ext

ACT_DTYPES = (torch.bfloat16, torch.float32)
SCAN_SEGMENT = 128        # tokens per segment of the segmented RG-LRU scan (kSeg in seqmix.hip)
SCAN_MIN_WAVES = 2048     # below this many (sequence, 64-channel) waves a long chunk is scanned in segments


@dataclass
class SeqBatch:
    """Device-side varlen metadata of one step (a view of the stage's BatchMeta)."""
    cu: torch.Tensor            # [B + 1] int32
    positions: torch.Tensor     # [T] int32
    tok_seq: torch.Tensor       # [T] int32
    state_slots: Optional[torch.Tensor]   # [B] int32 (None: the model keeps no state besides K/V)
    num_seqs: int
    num_tokens: int
    max_q_len: int


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _k():
    return _ext.kernels()


def _f32flag(t: torch.Tensor) -> int:
    if t.dtype not in ACT_DTYPES:
        raise TypeError(f"activation dtype {t.dtype} (bfloat16 or float32)")
    return 1 if t.dtype == torch.float32 else 0


def _ck(t: torch.Tensor, name: str, dtype=None):
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name}: expected {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name}: must be contiguous")


def _ptr(t: Optional[torch.Tensor]) -> int:
    return 0 if t is None else t.data_ptr()


# ------------------------------------------------------------------ embedding / norms
def embedding_f32(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """Rows of ``table`` as a float32 residual stream [T, W]."""
    if not table.is_cuda:
        return table.index_select(0, ids.long()).float()
    _ck(ids, "ids", torch.int32)
    _ck(table, "table")
    t, (v, w) = ids.numel(), table.shape
    out = torch.empty(t, w, dtype=torch.float32, device=table.device)
    _k().sm_embed_f32(out.data_ptr(), ids.data_ptr(), table.data_ptr(), t, w, v, _f32flag(table), _stream())
    return out


def embedding_norm_f32(ids: torch.Tensor, table: torch.Tensor, w: torch.Tensor, eps: float, one_plus: bool = True,
                       rounded: bool = False, scale: float = 1.0, pos_table: Optional[torch.Tensor] = None,
                       positions: Optional[torch.Tensor] = None):
    """The RMS norm of the looked-up rows, rms(e) * ((1 if one_plus else 0) + w) with e = table[ids] * scale
    (+ pos_table[positions]: a learned vector per position, unscaled), as a float32 residual stream [T, W];
    with ``rounded`` also in the table's dtype (the stream tensor itself when that is float32): the input of
    a first sublayer that reads the stream unnormed."""
    if pos_table is not None and (positions is None or pos_table.shape[1] != table.shape[1] or pos_table.dtype != table.dtype):
        raise ValueError("embedding_norm_f32: positions / position table mismatch")
    if not table.is_cuda:
        e = table.index_select(0, ids.long()).float() * scale
        if pos_table is not None:
            if int(positions.max()) >= pos_table.shape[0]:
                raise ValueError("embedding_norm_f32: position beyond the position table")
            e = e + pos_table.index_select(0, positions.long()).float()
        x = _ref_rms(e, w, eps, 1.0 if one_plus else 0.0)
        return x, ((x if table.dtype == torch.float32 else x.to(table.dtype)) if rounded else None)
    _ck(ids, "ids", torch.int32)
    _ck(table, "table")
    _ck(w, "w", table.dtype)
    if pos_table is not None:
        _ck(pos_table, "pos_table", table.dtype)
        _ck(positions, "positions", torch.int32)
    t, (v, width) = ids.numel(), table.shape
    x = torch.empty(t, width, dtype=torch.float32, device=table.device)
    h = torch.empty(t, width, dtype=table.dtype, device=table.device) if rounded and table.dtype != torch.float32 else None
    _k().sm_embed_norm(x.data_ptr(), _ptr(h), ids.data_ptr(), table.data_ptr(), w.data_ptr(), t, width, v, float(eps),
                       1.0 if one_plus else 0.0, float(scale), _ptr(pos_table),
                       _ptr(positions) if pos_table is not None else 0, 0 if pos_table is None else pos_table.shape[0],
                       _f32flag(table), _stream())
    return x, ((x if h is None else h) if rounded else None)


def _ref_rms(x: torch.Tensor, w: torch.Tensor, eps: float, offset: float) -> torch.Tensor:
    x = x.float()
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * (offset + w.float())


def rms_norm_f32(x: torch.Tensor, w: torch.Tensor, eps: float, act_dtype, one_plus: bool = True) -> torch.Tensor:
    """x [T, W] float32 -> x / sqrt(mean(x^2) + eps) * ((1 if one_plus else 0) + w) in ``act_dtype``."""
    if not x.is_cuda:
        return _ref_rms(x, w, eps, 1.0 if one_plus else 0.0).to(act_dtype)
    _ck(x, "x", torch.float32)
    _ck(w, "w", act_dtype)
    t, width = x.shape
    y = torch.empty(t, width, dtype=act_dtype, device=x.device)
    _k().sm_rms_norm(y.data_ptr(), x.data_ptr(), w.data_ptr(), t, width, float(eps), 1.0 if one_plus else 0.0,
                     _f32flag(y), _stream())
    return y


def post_norm_add(x: torch.Tensor, o: torch.Tensor, w_post: torch.Tensor, eps: float, mult: float,
                  bias: Optional[torch.Tensor] = None, w_next: Optional[torch.Tensor] = None, one_plus: bool = True,
                  o2: Optional[torch.Tensor] = None, scales=(1.0, 1.0), plain_next: bool = False):
    """The close of a sublayer, fused: ``x += mult * rms_norm(o + bias) * (1 + w_post)`` in place on the
    float32 residual stream; with ``w_next`` also returns the next sublayer's input
    ``rms_norm(x) * (1 + w_next)`` in ``o``'s dtype (None otherwise).  ``one_plus`` False: both norm
    weights are plain (``* w``).  ``o2``: the sublayer's output is ``scales[0] * o + scales[1] * o2`` (two
    mixers side by side).  ``plain_next`` (without ``w_next``): the next sublayer reads the stream itself;
    returns it in ``o``'s dtype (the stream tensor when that is float32)."""
    off = 1.0 if one_plus else 0.0
    if not x.is_cuda:
        ob = o.float() if o2 is None else scales[0] * o.float() + scales[1] * o2.float()
        if bias is not None:
            ob = ob + bias.float()
        x.add_(mult * _ref_rms(ob, w_post, eps, off))
        if w_next is None:
            return x, ((x if o.dtype == torch.float32 else x.to(o.dtype)) if plain_next else None)
        return x, _ref_rms(x, w_next, eps, off).to(o.dtype)
    _ck(x, "x", torch.float32)
    _ck(o, "o")
    t, width = x.shape
    if o.shape != x.shape or (o2 is not None and (o2.shape != x.shape or o2.dtype != o.dtype or not o2.is_contiguous())):
        raise ValueError("post_norm_add: o / x shape mismatch")
    h = None
    if w_next is not None or (plain_next and o.dtype != torch.float32):
        h = torch.empty_like(o)
    _k().sm_post_norm_add(x.data_ptr(), o.data_ptr(), _ptr(bias), w_post.data_ptr(), _ptr(w_next), _ptr(h), t, width,
                          float(eps), float(mult), off, _ptr(o2), float(scales[0]), float(scales[1]), _f32flag(o),
                          _stream())
    return x, (x if (plain_next and w_next is None and h is None) else h)


def stream_enter(x: torch.Tensor, x0: Optional[torch.Tensor], vec: Optional[torch.Tensor]) -> torch.Tensor:
    """The entry of a pass through a looped span of layers, in place on the float32 stream: x += x0 (a
    second stream, e.g. the embedding output; None: nothing) + vec (one learned row [W] for every token;
    None: nothing)."""
    if x0 is not None and x0.shape != x.shape:
        raise ValueError("stream_enter: stream shapes differ")
    if vec is not None and vec.numel() != x.shape[1]:
        raise ValueError("stream_enter: vector width")
    if not x.is_cuda:
        if x0 is not None:
            x.add_(x0)
        if vec is not None:
            x.add_(vec.float())
        return x
    _ck(x, "x", torch.float32)
    if x0 is not None:
        _ck(x0, "x0", torch.float32)
    if vec is not None:
        _ck(vec, "vec")
    _k().sm_stream_enter(x.data_ptr(), _ptr(x0), _ptr(vec), x.shape[0], x.shape[1],
                         0 if vec is None else _f32flag(vec), _stream())
    return x


def mix_add(x: torch.Tensor, o: torch.Tensor, eps: float, w_o: Optional[torch.Tensor] = None,
            o2: Optional[torch.Tensor] = None, w_o2: Optional[torch.Tensor] = None, coef: float = 1.0,
            w_next: Optional[torch.Tensor] = None):
    """The close of a pre-norm sublayer, fused, in place on the float32 stream:
    ``x += coef * (f(o, w_o) + f(o2, w_o2))`` with f(o, w) = rms_norm(o) * w (plain weight) when ``w`` is given
    and o itself otherwise (``o2`` None: one term) -- two mixers side by side are normed apart before they
    are summed; with ``w_next`` also returns the next sublayer's input rms_norm(x) * w_next in ``o``'s dtype."""
    if o.shape != x.shape or (o2 is not None and (o2.shape != x.shape or o2.dtype != o.dtype)):
        raise ValueError("mix_add: o / x shape mismatch")
    if not x.is_cuda:
        f = lambda a, w: a.float() if w is None else _ref_rms(a, w, eps, 0.0)
        y = f(o, w_o)
        if o2 is not None:
            y = y + f(o2, w_o2)
        x.add_(coef * y)
        return x, (None if w_next is None else _ref_rms(x, w_next, eps, 0.0).to(o.dtype))
    _ck(x, "x", torch.float32)
    _ck(o, "o")
    if o2 is not None:
        _ck(o2, "o2")
    for n, w in (("w_o", w_o), ("w_o2", w_o2), ("w_next", w_next)):
        if w is not None:
            _ck(w, n, o.dtype)
    h = torch.empty_like(o) if w_next is not None else None
    _k().sm_mix_add(x.data_ptr(), o.data_ptr(), _ptr(w_o), _ptr(o2), _ptr(w_o2), _ptr(w_next), _ptr(h), x.shape[0],
                    x.shape[1], float(eps), float(coef), _f32flag(o), _stream())
    return x, h


def token_shift(h: torch.Tensor, w: torch.Tensor, state: torch.Tensor, sb: SeqBatch) -> torch.Tensor:
    """Every channel of a token's row blended with the same channel of the token before it:
    y_t = h_t + (h_(t-1) - h_t) * w, with h_(t-1) the UNBLENDED previous row of the same sequence -- the
    chunk's own earlier row, the row ``state`` [slots, W] keeps across chunk borders, zeros before position
    0.  ``state`` is brought up to date (the chunk's last row).  float32 arithmetic, ``h``'s dtype out."""
    t, width = h.shape
    if w.numel() != width or state.shape[1] != width or state.dtype != h.dtype:
        raise ValueError("token_shift: shape / dtype mismatch")
    if not h.is_cuda:
        out = torch.empty_like(h)
        cu, pos, slots = sb.cu.tolist(), sb.positions.tolist(), sb.state_slots.tolist()
        for b in range(sb.num_seqs):
            lo, hi = cu[b], cu[b + 1]
            if hi == lo:
                continue
            first = state[slots[b]].float() if pos[lo] > 0 else torch.zeros(width)
            cur = h[lo:hi].float()
            prev = torch.cat([first[None], cur[:-1]], 0)
            out[lo:hi] = (cur + (prev - cur) * w.float()).to(h.dtype)
            state[slots[b]] = h[hi - 1]
        return out
    _ck(h, "h")
    _ck(w, "w", h.dtype)
    _ck(state, "state", h.dtype)
    out = torch.empty_like(h)
    _k().sm_token_shift(out.data_ptr(), h.data_ptr(), w.data_ptr(), state.data_ptr(), sb.cu.data_ptr(),
                        sb.positions.data_ptr(), sb.tok_seq.data_ptr(), sb.state_slots.data_ptr(), t, width, _f32flag(h),
                        _stream())
    return out


# ------------------------------------------------------------------ causal convolution with state
def _ref_conv_gather(u: torch.Tensor, state: torch.Tensor, sb: SeqBatch, taps: int,
                     in_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """[taps, T, C] float32: tap j of token t is the input at position p_t - (taps - 1) + j (the
    chunk's own rows, the state tail before the chunk's start, zeros before the sequence's)."""
    t, c = u.shape
    out = torch.zeros(taps, t, c, dtype=torch.float32, device=u.device)
    cu = sb.cu.tolist()
    pos = sb.positions.tolist()
    slots = sb.state_slots.tolist()
    for b in range(sb.num_seqs):
        a, e = cu[b], cu[b + 1]
        if e == a:
            continue
        start = pos[a]
        prev = state[slots[b]].float() if start > 0 else torch.zeros(taps - 1, c, device=u.device)
        if 0 < start < taps - 1:
            prev = torch.cat([torch.zeros(taps - 1 - start, c, device=u.device), prev[taps - 1 - start:]], 0)
        full = torch.cat([prev, u[a:e].float()], 0)
        state[slots[b]] = full[full.shape[0] - (taps - 1):].to(state.dtype)
        if in_bias is not None:        # added to every input that exists (not to the zeros before position 0)
            full = full.clone()
            full[max(0, taps - 1 - start):] += in_bias.float()
        for j in range(taps):
            out[j, a:e] = full[j:j + (e - a)]
    return out


def causal_conv(u: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor,
                sb: SeqBatch, out_dtype=torch.float32, in_bias: Optional[torch.Tensor] = None,
                act: Optional[str] = None) -> torch.Tensor:
    """Per-channel causal convolution over time, y_t = bias + sum_j w[:, j] (u + in_bias)_(t - taps + 1 + j)
    (zeros before the sequence's start), across chunk borders: ``state`` [slots, taps - 1, C] holds each
    sequence's last taps - 1 rows of ``u`` and is brought up to date.  ``u`` [T, C] may be a column slice
    of a wider projection (row stride); ``in_bias`` is the bias of the projection that made it.  ``w`` is
    tap-major [taps, C], the last row the current token's.  ``act`` "silu": y <- y sigmoid(y) (float32)."""
    if act not in (None, "silu"):
        raise ValueError(f"causal_conv: activation {act!r} (None, 'silu')")
    taps, c = w.shape
    if u.shape[1] != c or state.shape[1:] != (taps - 1, c):
        raise ValueError("causal_conv: shape mismatch")
    if not u.is_cuda:
        g = _ref_conv_gather(u, state, sb, taps, in_bias)
        y = (g * w.float()[:, None, :]).sum(0)
        if bias is not None:
            y = y + bias.float()
        if act == "silu":
            y = y * torch.sigmoid(y)
        return y.to(out_dtype)
    if u.stride(1) != 1:
        raise ValueError("causal_conv: channels must be contiguous")
    _ck(w, "w", u.dtype)
    _ck(state, "state", u.dtype)
    y = torch.empty(u.shape[0], c, dtype=out_dtype, device=u.device)
    _k().sm_causal_conv(y.data_ptr(), u.data_ptr(), u.stride(0), w.data_ptr(), _ptr(bias), _ptr(in_bias), state.data_ptr(),
                        sb.cu.data_ptr(), sb.positions.data_ptr(), sb.tok_seq.data_ptr(), sb.state_slots.data_ptr(),
                        sb.num_tokens, sb.num_seqs, c, taps, _f32flag(u), 1 if out_dtype == torch.float32 else 0,
                        1 if act == "silu" else 0, _stream())
    return y


# ------------------------------------------------------------------ RG-LRU
def gelu_tanh_f32(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z * z * z)))


def rglru(u: torch.Tensor, y_raw: torch.Tensor, y_bias: torch.Tensor, ra_t: torch.Tensor, ra_b: torch.Tensor,
          ri_t: torch.Tensor, ri_b: torch.Tensor, lam: torch.Tensor, state: torch.Tensor, sb: SeqBatch,
          act_dtype, decay_scale: float = 8.0) -> torch.Tensor:
    """Real-gated linear recurrent unit over a varlen batch.

    ``u`` [T, C] float32 (the convolved branch), split into ``nb`` blocks of ``bw`` channels;
    r = sigmoid(Ra_b u_b + ra_b), i = sigmoid(Ri_b u_b + ri_b) with ``ra_t`` / ``ri_t`` [nb, bw_in, bw_out]
    (the gate matrices TRANSPOSED, so consecutive outputs are consecutive in memory);
    a = exp(-decay_scale * r * softplus(lam)); S_t = a S_(t-1) + sqrt(1 - a^2) * i * u, all float32,
    ``state`` [slots, C] float32 carried between chunks.  Returns S_t * gelu_tanh(y_raw + y_bias) in
    ``act_dtype`` (``y_raw`` [T, C], row-strided allowed)."""
    t, c = u.shape
    nb, bw, _ = ra_t.shape
    if nb * bw != c:
        raise ValueError("rglru: blocks x block width != channels")
    if not u.is_cuda:
        ub = u.float().view(t, nb, bw)
        r = torch.sigmoid(torch.einsum("tbi,bio->tbo", ub, ra_t.float()).reshape(t, c) + ra_b.float().reshape(c))
        ig = torch.sigmoid(torch.einsum("tbi,bio->tbo", ub, ri_t.float()).reshape(t, c) + ri_b.float().reshape(c))
        a = torch.exp(-decay_scale * r * torch.nn.functional.softplus(lam.float()))
        g = torch.sqrt(1.0 - a * a) * ig * u.float()
        s_all = torch.empty(t, c, dtype=torch.float32)
        cu, pos, slots = sb.cu.tolist(), sb.positions.tolist(), sb.state_slots.tolist()
        for b in range(sb.num_seqs):
            lo, hi = cu[b], cu[b + 1]
            if hi == lo:
                continue
            s = state[slots[b]].clone() if pos[lo] > 0 else torch.zeros(c)
            for k in range(lo, hi):
                s = a[k] * s + g[k]
                s_all[k] = s
            state[slots[b]] = s
        return (s_all * gelu_tanh_f32(y_raw.float() + y_bias.float())).to(act_dtype)
    _ck(u, "u", torch.float32)
    _ck(state, "state", torch.float32)
    if y_raw.stride(1) != 1:
        raise ValueError("rglru: y_raw channels must be contiguous")
    for n, x in (("ra_t", ra_t), ("ri_t", ri_t), ("ra_b", ra_b), ("ri_b", ri_b), ("lam", lam), ("y_bias", y_bias)):
        _ck(x, n, act_dtype)
    a = torch.empty(t, c, dtype=torch.float32, device=u.device)
    g = torch.empty(t, c, dtype=torch.float32, device=u.device)
    f = _f32flag(y_raw)
    _k().sm_rglru_gates(a.data_ptr(), g.data_ptr(), u.data_ptr(), ra_t.data_ptr(), ra_b.data_ptr(), ri_t.data_ptr(),
                        ri_b.data_ptr(), lam.data_ptr(), t, nb, bw, float(decay_scale), f, _stream())
    out = torch.empty(t, c, dtype=act_dtype, device=u.device)
    # few sequences with long chunks: the segmented two-launch scan (its waves = sequences x segments x
    # C / 64); many sequences fill the chip with one wave per (sequence, 64 channels) already
    ab = None
    nseg = -(-sb.max_q_len // SCAN_SEGMENT)
    if nseg > 1 and sb.num_seqs * (-(-c // 64)) < SCAN_MIN_WAVES:
        ab = torch.empty(sb.num_seqs * (nseg * 2 + 1) * c, dtype=torch.float32, device=u.device)
    _k().sm_rglru_scan(out.data_ptr(), a.data_ptr(), g.data_ptr(), y_raw.data_ptr(), y_raw.stride(0),
                       y_bias.data_ptr(), state.data_ptr(), sb.cu.data_ptr(), sb.positions.data_ptr(),
                       sb.state_slots.data_ptr(), sb.num_seqs, c, sb.max_q_len, _ptr(ab), f, _stream())
    return out


# ------------------------------------------------------------------ clipped GLU / soft cap
def clipped_glu(gu: torch.Tensor, bias_gu: Optional[torch.Tensor], limit: float, alpha: float = 1.702) -> torch.Tensor:
    """[T, 2F] = gate | up (+ bias): g = min(gate, limit), u = clamp(up, -limit, limit);
    g * sigmoid(alpha g) * (u + 1)  -> [T, F]."""
    t, two_f = gu.shape
    f = two_f // 2
    if not gu.is_cuda:
        x = gu.float() if bias_gu is None else gu.float() + bias_gu.float()
        g = torch.clamp(x[:, :f], max=limit)
        u = torch.clamp(x[:, f:], -limit, limit)
        return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gu.dtype)
    _ck(gu, "gu")
    out = torch.empty(t, f, dtype=gu.dtype, device=gu.device)
    _k().sm_clipped_glu(out.data_ptr(), gu.data_ptr(), _ptr(bias_gu), t, f, float(limit), float(alpha), _f32flag(gu),
                        _stream())
    return out


def softcap_f32(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """float32 cap * tanh(logits / cap) (cap <= 0: a plain float32 copy)."""
    if not logits.is_cuda:
        x = logits.float()
        return cap * torch.tanh(x / cap) if cap > 0 else x
    _ck(logits, "logits")
    out = torch.empty(logits.shape, dtype=torch.float32, device=logits.device)
    _k().sm_softcap(out.data_ptr(), logits.data_ptr(), logits.numel(), float(cap), _f32flag(logits), _stream())
    return out


# ------------------------------------------------------------------ rotary tables
def yarn_frequencies(dims: int, base: float, scaling: Optional[dict]) -> Tuple[torch.Tensor, float]:
    """(f [dims / 2] float32, magnitude): rotary frequencies f_i = base^(-2i/dims), blended by YaRN
    (``scaling``: factor, original, fast, slow): with d(t) = dims ln(original / (2 pi t)) / (2 ln base),
    lo = max(floor(d(fast)), 0), hi = min(ceil(d(slow)), dims - 1), ramp_i = clamp((i - lo) / max(hi - lo,
    0.001), 0, 1), f_i <- f_i / factor * ramp_i + f_i (1 - ramp_i); cos and sin are scaled by
    0.1 ln(factor) + 1."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims)
    mag = 1.0
    if scaling:
        factor = float(scaling["factor"])

        def d(turns):
            return dims * math.log(scaling["original"] / (2 * math.pi * turns)) / (2 * math.log(base))
        lo = max(math.floor(d(scaling["fast"])), 0)
        hi = min(math.ceil(d(scaling["slow"])), dims - 1)
        ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0, 1)
        f = f / factor * ramp + f * (1 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    return f.float(), float(mag)


def _ref_rope_interleaved(x: torch.Tensor, pos: torch.Tensor, freqs: torch.Tensor, mag: float) -> torch.Tensor:
    """x [T, H, D] float32; pairs (2i, 2i + 1) for i < len(freqs) rotate by pos * f_i."""
    n = freqs.numel()
    ang = pos.float()[:, None] * freqs.float()[None]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    out = x.clone()
    a, b = x[..., 0:2 * n:2], x[..., 1:2 * n:2]
    out[..., 0:2 * n:2] = a * c - b * s
    out[..., 1:2 * n:2] = b * c + a * s
    return out


# ------------------------------------------------------------------ attention input: conv + norm + rotation + append
def attn_prep(qkv: torch.Tensor, conv_w: torch.Tensor, state: torch.Tensor, q_norm: torch.Tensor,
              k_norm: Optional[torch.Tensor], freqs: torch.Tensor, mag: float, eps: float,
              k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], slot_mapping: torch.Tensor,
              sb: SeqBatch, heads: int, kv_heads: int, dim: int, vdim: int) -> torch.Tensor:
    """From the fused projection [T, heads * dim (+ kv_heads * dim + kv_heads * vdim)]: the short causal
    convolution on every channel (``conv_w`` [taps, C], tap-major; tail in ``state`` [slots, taps - 1, C]), the
    per-head RMS norm of q and k (plain weight), the interleaved-pair rotation of their first
    2 len(freqs) dims, and the append of k [.., dim] and v [.., vdim] (convolved only) at
    ``slot_mapping`` into caches k [NB, kv_heads, BS, dim] / v [NB, kv_heads, vdim, BS] (V transposed inside
    a block: the keys of one value channel are contiguous, which is what the matrix cores read).  With
    ``k_cache`` None the projection holds q only (the layer reads another layer's K/V).
    Returns q [T, heads, dim]."""
    t, c = qkv.shape
    own_kv = k_cache is not None
    qc, kc, vc = heads * dim, kv_heads * dim, kv_heads * vdim
    if c != qc + (kc + vc if own_kv else 0) or conv_w.shape[1] != c:
        raise ValueError("attn_prep: projection width mismatch")
    taps = conv_w.shape[0]
    if not qkv.is_cuda:
        g = _ref_conv_gather(qkv, state, sb, taps)
        y = (g * conv_w.float()[:, None, :]).sum(0)
        pos = sb.positions
        q = _ref_rms(y[:, :qc].view(t, heads, dim), q_norm, eps, 0.0)
        q = _ref_rope_interleaved(q, pos, freqs, mag).to(qkv.dtype)
        if own_kv:
            k = _ref_rms(y[:, qc:qc + kc].view(t, kv_heads, dim), k_norm, eps, 0.0)
            k = _ref_rope_interleaved(k, pos, freqs, mag)
            v = y[:, qc + kc:].view(t, kv_heads, vdim)
            bs = k_cache.shape[2]
            sm = slot_mapping.long()
            k_cache[sm // bs, :, sm % bs] = k.to(k_cache.dtype)
            v_cache[sm // bs, :, :, sm % bs] = v.to(v_cache.dtype)
        return q
    _ck(qkv, "qkv")
    _ck(conv_w, "conv_w", qkv.dtype)
    _ck(state, "state", qkv.dtype)
    _ck(freqs, "freqs", torch.float32)
    if state.shape[1:] != (taps - 1, c):
        raise ValueError("attn_prep: state shape")
    if own_kv:
        _ck(k_cache, "k_cache", qkv.dtype)
        _ck(v_cache, "v_cache", qkv.dtype)
        if k_cache.shape[1:] != (kv_heads, k_cache.shape[2], dim) or v_cache.shape[1:] != (kv_heads, vdim, k_cache.shape[2]):
            raise ValueError("attn_prep: cache shape")
    if 2 * freqs.numel() > dim:
        raise ValueError("attn_prep: rotary dims exceed the head size")
    q = torch.empty(t, heads, dim, dtype=qkv.dtype, device=qkv.device)
    _k().sm_attn_prep(q.data_ptr(), qkv.data_ptr(), conv_w.data_ptr(), state.data_ptr(), q_norm.data_ptr(),
                      _ptr(k_norm), freqs.data_ptr(), freqs.numel(), float(mag), float(eps), _ptr(k_cache),
                      _ptr(v_cache), slot_mapping.data_ptr(), sb.cu.data_ptr(), sb.positions.data_ptr(),
                      sb.tok_seq.data_ptr(), sb.state_slots.data_ptr(), sb.num_tokens, sb.num_seqs, heads,
                      kv_heads if own_kv else 0, dim, vdim, taps, k_cache.shape[2] if own_kv else 1,
                      _f32flag(qkv), _stream())
    return q


# ------------------------------------------------------------------ attention input: row norm + half-split rotation + append
def rotary_frequencies(dims: int, base: float) -> torch.Tensor:
    """f_i = base^(-2i / dims), i < dims / 2, computed in float64 and rounded once to float32."""
    return yarn_frequencies(dims, base, None)[0]


def _ref_rope_half(x: torch.Tensor, pos: torch.Tensor, freqs: torch.Tensor, mag: float = 1.0) -> torch.Tensor:
    """x [T, H, D] float32; dimension i < len(freqs) is paired with dimension i + len(freqs); the pair
    (u, v) turns to (u cos a - v sin a, v cos a + u sin a), a = pos * f_i (cos and sin times ``mag``)."""
    n = freqs.numel()
    ang = pos.float()[:, None] * freqs.float()[None]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    out = x.clone()
    a, b = x[..., :n], x[..., n:2 * n]
    out[..., :n] = a * c - b * s
    out[..., n:2 * n] = b * c + a * s
    return out


def rownorm_rope(qkv: torch.Tensor, col0: int, q_norm: Optional[torch.Tensor], k_norm: Optional[torch.Tensor],
                 freqs: torch.Tensor, eps: float, k_cache: torch.Tensor, v_cache: torch.Tensor, slot_mapping: torch.Tensor,
                 positions: torch.Tensor, heads: int, kv_heads: int, dim: int, vdim: int, mag: float = 1.0,
                 v_from_k: bool = False) -> torch.Tensor:
    """From columns ``col0 ..`` of a fused projection [T, .. | q (heads dim) | k (kv_heads dim) | v (kv_heads
    vdim) | ..]: an RMS norm over the WHOLE q projection and over the whole k projection (all heads at
    once; plain weights ``q_norm`` [heads dim], ``k_norm`` [kv_heads dim]; both None: no norm), then the
    half-split rotation of the first 2 len(freqs) dimensions of every q and k head (dimension i paired
    with i + len(freqs), angle position * freqs[i], cos and sin times ``mag``), and the append of k and v
    (v unchanged) at ``slot_mapping`` into caches k [NB, kv_heads, BS, dim] / v [NB, kv_heads, vdim, BS].
    ``v_from_k``: the projection has no v columns; the values are the keys as projected, BEFORE norm and
    rotation (vdim = dim).  Returns q [T, heads, dim]."""
    t = qkv.shape[0]
    nq, nk, nv = heads * dim, kv_heads * dim, kv_heads * vdim
    normed = q_norm is not None
    if (k_norm is not None) != normed or (v_from_k and vdim != dim) or 2 * freqs.numel() > dim:
        raise ValueError("rownorm_rope: norm weights for both or neither; values from keys need vdim = dim")
    if qkv.shape[1] < col0 + nq + nk + (0 if v_from_k else nv) or (normed and (q_norm.numel() != nq or k_norm.numel() != nk)):
        raise ValueError("rownorm_rope: shape mismatch")
    bs = k_cache.shape[2]
    if k_cache.shape[1:] != (kv_heads, bs, dim) or v_cache.shape[1:] != (kv_heads, vdim, bs):
        raise ValueError("rownorm_rope: cache shape")
    if not qkv.is_cuda:
        x = qkv[:, col0:col0 + nq + nk].float()
        xq, xk = x[:, :nq], x[:, nq:]
        if normed:
            xq, xk = _ref_rms(xq, q_norm, eps, 0.0), _ref_rms(xk, k_norm, eps, 0.0)
        q = _ref_rope_half(xq.reshape(t, heads, dim), positions, freqs, mag)
        k = _ref_rope_half(xk.reshape(t, kv_heads, dim), positions, freqs, mag)
        slot = slot_mapping.long()
        k_cache[slot // bs, :, slot % bs] = k.to(k_cache.dtype)
        v0 = col0 + nq if v_from_k else col0 + nq + nk
        v_cache[slot // bs, :, :, slot % bs] = qkv[:, v0:v0 + nv].reshape(t, kv_heads, vdim).to(v_cache.dtype)
        return q.to(qkv.dtype)
    _ck(qkv, "qkv")
    if normed:
        _ck(q_norm, "q_norm", qkv.dtype)
        _ck(k_norm, "k_norm", qkv.dtype)
    _ck(freqs, "freqs", torch.float32)
    _ck(k_cache, "k_cache", qkv.dtype)
    _ck(v_cache, "v_cache", qkv.dtype)
    q = torch.empty(t, heads, dim, dtype=qkv.dtype, device=qkv.device)
    _k().sm_rownorm_rope(q.data_ptr(), qkv.data_ptr(), qkv.shape[1], int(col0), _ptr(q_norm), _ptr(k_norm),
                         freqs.data_ptr(), freqs.numel(), float(eps), k_cache.data_ptr(), v_cache.data_ptr(),
                         slot_mapping.data_ptr(), positions.data_ptr(), t, heads, kv_heads, dim, vdim, bs, float(mag),
                         1 if v_from_k else 0, _f32flag(qkv), _stream())
    return q


# ------------------------------------------------------------------ averaged blocks of old keys
def pooled_block_size(block_size: int, pool: int) -> int:
    """Entries per cache block of the averaged-key cache: a power of two >= 8 that holds at least
    ceil(block_size / pool) entries, so that entry b (written when position b pool + pool - 1 arrives) lies in
    a block the sequence already owns: block floor(b / entries) <= floor((b pool + pool - 1) / block_size)."""
    need, n = -(-block_size // pool), 8
    while n < need:
        n *= 2
    return n


def pool_blocks(k_cache: torch.Tensor, v_cache: torch.Tensor, kp_cache: torch.Tensor, vp_cache: torch.Tensor,
                block_tables: torch.Tensor, sb: SeqBatch, pool: int) -> None:
    """Averaged keys and values of whole blocks of ``pool`` positions: for every token of the step whose
    position p ends a block (p + 1 a multiple of pool), the float32 mean of the block's ``pool`` keys and of
    its values AS THE CACHES HOLD THEM goes to entry b = (p + 1) / pool - 1 of the sequence's averaged
    caches kp [NB, G, PB, dim] / vp [NB, G, vdim, PB] (the K/V layouts with PB entries per block, behind the
    same block table: entry b at block b // PB, place b % PB).  Run after the step's keys are appended: a
    block's keys may come from earlier steps and from this one."""
    g, bs, d = k_cache.shape[1], k_cache.shape[2], k_cache.shape[3]
    dv, pb = v_cache.shape[2], kp_cache.shape[2]
    if pool < 1 or kp_cache.shape[1:] != (g, pb, d) or vp_cache.shape[1:] != (g, dv, pb) or pb * pool < bs:
        raise ValueError("pool_blocks: cache shapes")
    if not k_cache.is_cuda:
        pos, seq = sb.positions.tolist(), sb.tok_seq.tolist()
        for i in range(sb.num_tokens):
            if (pos[i] + 1) % pool:
                continue
            b = (pos[i] + 1) // pool - 1
            bt = block_tables[seq[i]].long()
            idx = torch.arange(b * pool, (b + 1) * pool)
            kk = k_cache[bt[idx // bs], :, idx % bs].float().mean(0)          # [G, d]
            vv = v_cache[bt[idx // bs], :, :, idx % bs].float().mean(0)       # [G, dv]
            kp_cache[bt[b // pb], :, b % pb] = kk.to(kp_cache.dtype)
            vp_cache[bt[b // pb], :, :, b % pb] = vv.to(vp_cache.dtype)
        return
    for n, c in (("k_cache", k_cache), ("v_cache", v_cache), ("kp_cache", kp_cache), ("vp_cache", vp_cache)):
        _ck(c, n, k_cache.dtype)
    _ck(block_tables, "block_tables", torch.int32)
    _k().sm_pool_blocks(k_cache.data_ptr(), v_cache.data_ptr(), kp_cache.data_ptr(), vp_cache.data_ptr(),
                        block_tables.data_ptr(), block_tables.shape[1], sb.cu.data_ptr(), sb.positions.data_ptr(),
                        sb.num_seqs, sb.max_q_len, g, d, dv, bs, pb, int(pool), _f32flag(k_cache), _stream())


# ------------------------------------------------------------------ sliding-window attention
DECODE_SPLIT_KEYS = 256     # fewest keys worth a workgroup of their own
DECODE_TARGET_WGS = 512     # workgroups wanted on the chip (256 CUs, two each)


def decode_splits(rows: int, heads: int, kv_heads: int, ctx: int) -> int:
    """Runs to cut each decode row's keys into: enough workgroups (rows x K/V heads x 16-head groups x
    runs) to fill the chip, none shorter than DECODE_SPLIT_KEYS keys; 1 when the bound ``ctx`` is unknown."""
    wgs = max(1, rows * kv_heads * -(-(heads // kv_heads) // 16))
    return max(1, min(DECODE_TARGET_WGS // wgs, ctx // DECODE_SPLIT_KEYS, 64))


def window_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                     sb: SeqBatch, window: int, scale: float, num_decode: Optional[int] = None,
                     sinks: Optional[torch.Tensor] = None, max_ctx: Optional[int] = None, chunk: int = 0,
                     softcap: float = 0.0, pooled: Optional[tuple] = None) -> torch.Tensor:
    """Softmax attention of every query token over the keys j of its own sequence with
    0 <= p - j < window (p the query's position) and, with ``chunk`` > 0, floor(j / chunk) =
    floor(p / chunk) (attention inside fixed chunks of positions counted from position 0, wherever a
    prompt was cut for processing), keys / values read through ``block_tables`` from
    caches k [NB, G, BS, dim] / v [NB, G, vdim, BS]; query head h reads K/V head h // (H / G).
    Scores and weights are float32.  ``num_decode``: the first that many sequences are one-token
    rows (they take the decode kernel; None: every sequence is one); the rest are prompt chunks.
    ``sinks`` [H] float32: exp(sinks[h]) is added to head h's softmax denominator -- a learned per-head
    logit that takes part in the normalisation only (nothing is attended to through it; it enters as it
    is, without the score scale).  ``max_ctx``: a bound on the decode
    rows' context; with few rows of long context their keys are cut into runs on separate workgroups
    (results equal up to rounding).  ``softcap`` > 0: every scaled score s becomes softcap * tanh(s / softcap).
    ``pooled`` = (kp_cache, vp_cache, pool): beside the tokens of its window a query at position p sees one
    averaged key and value for every block of ``pool`` positions that lies wholly before the window -- entries
    b < floor((p - window + 1) / pool) of the averaged caches (:func:`pool_blocks`), scored, capped and
    normalised in the same softmax; tokens that left the window inside a block not yet complete are not
    seen at all.  Returns [T, H, vdim]."""
    t, h, d = q.shape
    g, bs, dv = k_cache.shape[1], k_cache.shape[2], v_cache.shape[2]
    kp = vp = None
    pool, pb = 0, 1
    if pooled is not None:
        kp, vp, pool = pooled
        pb = kp.shape[2]
        if pool < 1 or chunk or kp.shape[1:] != (g, pb, d) or vp.shape[1:] != (g, dv, pb) or pb * pool < bs:
            raise ValueError("window_attention: averaged caches do not fit (and exclude a chunk mask)")
    if not q.is_cuda:
        out = torch.empty(t, h, dv, dtype=torch.float32)
        pos, seq = sb.positions.tolist(), sb.tok_seq.tolist()
        rep = h // g
        for i in range(t):
            p = pos[i]
            lo = max(0, p - window + 1, p - p % chunk if chunk > 0 else 0)
            idx = torch.arange(lo, p + 1)
            blk = block_tables[seq[i]].long()[idx // bs]
            kk = k_cache[blk, :, idx % bs].float().repeat_interleave(rep, 1)     # [n, H, d]
            vv = v_cache[blk, :, :, idx % bs].float().repeat_interleave(rep, 1)
            if pool and p - window + 1 >= pool:
                pidx = torch.arange((p - window + 1) // pool)
                pblk = block_tables[seq[i]].long()[pidx // pb]
                kk = torch.cat([kp[pblk, :, pidx % pb].float().repeat_interleave(rep, 1), kk], 0)
                vv = torch.cat([vp[pblk, :, :, pidx % pb].float().repeat_interleave(rep, 1), vv], 0)
            s = torch.einsum("hd,nhd->hn", q[i].float(), kk) * scale
            if softcap > 0:
                s = softcap * torch.tanh(s / softcap)
            if sinks is not None:      # one more column in the softmax whose weight is dropped
                pr = torch.softmax(torch.cat([s, sinks.float()[:, None]], -1), -1)[:, :-1]
            else:
                pr = torch.softmax(s, -1)
            out[i] = torch.einsum("hn,nhd->hd", pr, vv)
        return out.to(q.dtype)
    _ck(q, "q")
    _ck(k_cache, "k_cache", q.dtype)
    _ck(v_cache, "v_cache", q.dtype)
    _ck(block_tables, "block_tables", torch.int32)
    if h % g or k_cache.shape[3] != d or v_cache.shape[3] != bs or window < 1 or chunk < 0:
        raise ValueError("window_attention: head / size mismatch")
    if sinks is not None:
        _ck(sinks, "sinks", torch.float32)
        if sinks.numel() != h:
            raise ValueError("window_attention: one sink per query head")
    if pool:
        _ck(kp, "kp_cache", q.dtype)
        _ck(vp, "vp_cache", q.dtype)
    out = torch.empty(t, h, dv, dtype=q.dtype, device=q.device)
    nd = sb.num_seqs if num_decode is None else int(num_decode)
    f = _f32flag(q)
    if nd:       # one-token rows are the first nd tokens
        span = min(int(window), int(chunk)) if chunk > 0 else int(window)
        ctx = int(max_ctx or 0)
        keys = min(span, ctx) + (max(0, ctx - span) // pool if pool else 0)      # window tokens + averaged entries
        splits, ws = decode_splits(nd, h, g, keys), None
        if splits > 1 and not f:
            ws = torch.empty(nd * h * splits * (dv + 2), dtype=torch.float32, device=q.device)
        _k().sm_window_attn_decode(out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                   block_tables.data_ptr(), block_tables.shape[1], sb.positions.data_ptr(),
                                   sb.tok_seq.data_ptr(), nd, h, g, d, dv, bs, int(window), int(chunk), float(scale), _ptr(sinks),
                                   splits if ws is not None else 1, _ptr(ws), float(softcap), _ptr(kp), _ptr(vp), int(pool),
                                   int(pb), f, _stream())
    if t > nd:
        _k().sm_window_attn_prefill(out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                    block_tables.data_ptr(), block_tables.shape[1], sb.cu.data_ptr(),
                                    sb.positions.data_ptr(), sb.tok_seq.data_ptr(), nd, sb.num_seqs, t, sb.max_q_len,
                                    h, g, d, dv, bs,
                                    int(window), int(chunk), float(scale), _ptr(sinks), float(softcap), _ptr(kp), _ptr(vp),
                                    int(pool), int(pb), f, _stream())
    return out
