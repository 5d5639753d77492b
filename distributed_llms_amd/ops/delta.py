"""Gated delta rule: a linear-attention token mixer with a float32 matrix state per head.

Per head, with unit-length q and k [dim], values v [vdim], a write strength beta in (0, 1) and a decay
g in (0, 1):

    S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q

so the read-out sees the current token's write.  ``S`` [dim, vdim] starts at zero and is carried from token
to token in a state slot (float32, whatever the activation type); query / key head ``h // (heads /
kv_heads)`` serves value head h.  The pieces, each an op of its own:

  :func:`unit_qk_gates`    q and k to unit length (q also times dim^-1/2), beta = sigmoid(b),
                           g = exp(-exp(A_log) softplus(a + dt_bias))
  :func:`delta_scan`       the recurrence over a varlen batch, state slots read and written
  :func:`conv_unit_gates`  the same behind the short convolutions + silu, from the fused projection (what the
                           mixer runs: one launch)
  :func:`gated_head_norm`  o / rms(o) * w * silu(gate) per head

Same dispatch as the other ops: CUDA tensors go to the in-tree HIP kernels (csrc/kernels/delta.hip) and
raise if those are not built; CPU tensors run the plain PyTorch forms.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn.functional as F

from .seqmix import SeqBatch, _ck, _f32flag, _k, _stream

UNIT_EPS = 1e-6          # inside the root of the unit norms: x / sqrt(sum(x^2) + UNIT_EPS)
MAX_KEY_DIM = 256        # the scan kernel keeps a state column in registers
PREP_LDS_BYTES = 48 * 1024   # the fused input stage holds a token's q | k (float32) in LDS


@dataclass
class DeltaSpec:
    """Sizes of one gated-delta-rule mixer."""
    heads: int           # value heads (one state each)
    kv_heads: int        # query / key heads
    dim: int             # query / key size per head
    vdim: int            # value size per head
    taps: int            # taps of the short convolutions on q, k, v

    @property
    def conv_width(self) -> int:          # q | k | v channels
        return 2 * self.kv_heads * self.dim + self.heads * self.vdim

    @property
    def in_width(self) -> int:            # q | k | v | gate | b | a
        return self.conv_width + self.heads * self.vdim + 2 * self.heads


def unit_qk_gates(u: torch.Tensor, ab: torch.Tensor, bcol: int, a_log: torch.Tensor, dt_bias: torch.Tensor,
                  spec: DeltaSpec, unit_eps: float = UNIT_EPS) -> torch.Tensor:
    """``u`` [T, conv_width] float32 (q | k | v after convolution and activation): every q and k head is
    scaled IN PLACE to x / sqrt(sum(x^2) + unit_eps), q also times dim^-1/2.  ``ab`` [T, *] holds the write
    logits b [heads] from column ``bcol`` and the decay logits a [heads] after them.  Returns
    [T, 2 heads] float32: beta = sigmoid(b) | g = exp(-exp(a_log) softplus(a + dt_bias))."""
    t = u.shape[0]
    hh, g, d = spec.heads, spec.kv_heads, spec.dim
    if u.dtype != torch.float32 or u.shape[1] != spec.conv_width or ab.shape[1] < bcol + 2 * hh:
        raise ValueError("unit_qk_gates: shape / dtype mismatch")
    if not u.is_cuda:
        qk = u[:, :2 * g * d].view(t, 2 * g, d)
        m = torch.rsqrt(qk.pow(2).sum(-1, keepdim=True) + unit_eps)
        m[:, :g] *= d ** -0.5
        qk.mul_(m)
        b, a = ab[:, bcol:bcol + hh].float(), ab[:, bcol + hh:bcol + 2 * hh].float()
        return torch.cat([torch.sigmoid(b), torch.exp(-torch.exp(a_log.float()) * F.softplus(a + dt_bias.float()))], 1)
    _ck(u, "u", torch.float32)
    _ck(ab, "ab")
    _ck(a_log, "a_log", torch.float32)
    _ck(dt_bias, "dt_bias", torch.float32)
    bd = torch.empty(t, 2 * hh, dtype=torch.float32, device=u.device)
    _k().dr_prep(u.data_ptr(), u.shape[1], ab.data_ptr(), ab.shape[1], int(bcol), a_log.data_ptr(), dt_bias.data_ptr(),
                 bd.data_ptr(), t, hh, g, d, d ** -0.5, float(unit_eps), _f32flag(ab), _stream())
    return bd


def delta_scan(u: torch.Tensor, bd: torch.Tensor, state: torch.Tensor, sb: SeqBatch, spec: DeltaSpec) -> torch.Tensor:
    """The recurrence.  ``u`` [T, conv_width] float32 (unit q | unit k | v), ``bd`` [T, 2 heads] (beta | g),
    ``state`` [slots, heads, dim, vdim] float32: a chunk that starts at position 0 starts from zero, any
    other from its slot; the slot holds the state after the chunk's last token.  Returns o
    [T, heads, vdim] float32."""
    t = u.shape[0]
    hh, g, d, dv = spec.heads, spec.kv_heads, spec.dim, spec.vdim
    if state.shape[1:] != (hh, d, dv) or state.dtype != torch.float32 or u.shape[1] != spec.conv_width:
        raise ValueError("delta_scan: shape / dtype mismatch")
    if not u.is_cuda:
        q = u[:, :g * d].view(t, g, d).repeat_interleave(hh // g, 1)
        k = u[:, g * d:2 * g * d].view(t, g, d).repeat_interleave(hh // g, 1)
        v = u[:, 2 * g * d:].view(t, hh, dv)
        o = torch.empty(t, hh, dv, dtype=torch.float32)
        cu, pos, slots = sb.cu.tolist(), sb.positions.tolist(), sb.state_slots.tolist()
        for b in range(sb.num_seqs):
            lo, hi = cu[b], cu[b + 1]
            if hi == lo:
                continue
            s = state[slots[b]].clone() if pos[lo] > 0 else torch.zeros(hh, d, dv)
            for i in range(lo, hi):
                s = s * bd[i, hh:, None, None]
                w = bd[i, :hh, None] * (v[i] - torch.einsum("hdv,hd->hv", s, k[i]))
                s = s + k[i][:, :, None] * w[:, None, :]
                o[i] = torch.einsum("hdv,hd->hv", s, q[i])
            state[slots[b]] = s
        return o
    if d > MAX_KEY_DIM:
        raise ValueError(f"delta_scan: key size {d} > {MAX_KEY_DIM}")
    _ck(u, "u", torch.float32)
    _ck(bd, "bd", torch.float32)
    _ck(state, "state", torch.float32)
    o = torch.empty(t, hh, dv, dtype=torch.float32, device=u.device)
    _k().dr_scan(o.data_ptr(), u.data_ptr(), u.shape[1], bd.data_ptr(), state.data_ptr(), sb.cu.data_ptr(),
                 sb.positions.data_ptr(), sb.state_slots.data_ptr(), sb.num_seqs, sb.max_q_len, hh, g, d, dv, _stream())
    return o


def conv_unit_gates(proj: torch.Tensor, col0: int, conv_w: torch.Tensor, conv_state: torch.Tensor, a_log: torch.Tensor,
                    dt_bias: torch.Tensor, sb: SeqBatch, spec: DeltaSpec, unit_eps: float = UNIT_EPS):
    """The mixer's input stage from its fused projection ``proj`` [T, *] = .. | q | k | v | gate | b | a from
    column ``col0``: the short causal convolutions of q | k | v (``conv_w`` [taps, conv_width] tap-major, tail in
    ``conv_state`` [slots, taps - 1, conv_width], brought up to date) with silu, then :func:`unit_qk_gates`.
    One launch (+ the tail update) on the GPU.  Returns (u [T, conv_width] float32, bd [T, 2 heads] float32)."""
    from . import seqmix as sm
    t = proj.shape[0]
    c = spec.conv_width
    bcol = col0 + c + spec.heads * spec.vdim
    taps = conv_w.shape[0]
    if proj.shape[1] < bcol + 2 * spec.heads or conv_w.shape != (spec.taps, c) or conv_state.shape[1:] != (taps - 1, c):
        raise ValueError("conv_unit_gates: shape mismatch")
    if not proj.is_cuda or 8 * spec.kv_heads * spec.dim > PREP_LDS_BYTES:
        # (on the GPU: q | k of a token wider than the fused kernel's LDS buffer -- the two mechanisms apart)
        u = sm.causal_conv(proj[:, col0:col0 + c], conv_w, None, conv_state, sb, out_dtype=torch.float32, act="silu")
        return u, unit_qk_gates(u, proj, bcol, a_log, dt_bias, spec, unit_eps)
    _ck(proj, "proj")
    _ck(conv_w, "conv_w", proj.dtype)
    _ck(conv_state, "conv_state", proj.dtype)
    _ck(a_log, "a_log", torch.float32)
    _ck(dt_bias, "dt_bias", torch.float32)
    u = torch.empty(t, c, dtype=torch.float32, device=proj.device)
    bd = torch.empty(t, 2 * spec.heads, dtype=torch.float32, device=proj.device)
    f = _f32flag(proj)
    _k().dr_conv_prep(u.data_ptr(), bd.data_ptr(), proj.data_ptr(), proj.shape[1], int(col0), int(bcol), conv_w.data_ptr(),
                      conv_state.data_ptr(), a_log.data_ptr(), dt_bias.data_ptr(), sb.cu.data_ptr(), sb.positions.data_ptr(),
                      sb.tok_seq.data_ptr(), sb.state_slots.data_ptr(), t, spec.heads, spec.kv_heads, spec.dim, spec.vdim,
                      taps, spec.dim ** -0.5, float(unit_eps), f, _stream())
    _k().sm_conv_tail(conv_state.data_ptr(), proj.data_ptr() + col0 * proj.element_size(), proj.shape[1], sb.cu.data_ptr(),
                      sb.positions.data_ptr(), sb.state_slots.data_ptr(), sb.num_seqs, c, taps, f, _stream())
    return u, bd


def gated_head_norm(o: torch.Tensor, gate: torch.Tensor, gcol: int, w: torch.Tensor, eps: float,
                    out_scale: float = 1.0, gate_act: str = "silu") -> torch.Tensor:
    """o [T, heads, vdim] float32 -> o / sqrt(mean(o^2) + eps) * w * act(gate[:, gcol + h vdim + :]) *
    out_scale as [T, heads vdim] in ``gate``'s dtype; ``w`` [vdim] is shared by the heads.  ``gate_act``:
    "silu" (g sigmoid(g)) or "sigmoid"."""
    t, hh, dv = o.shape
    if gate.shape[1] < gcol + hh * dv or w.numel() != dv or gate_act not in ("silu", "sigmoid"):
        raise ValueError("gated_head_norm: shape mismatch")
    if not o.is_cuda:
        z = gate[:, gcol:gcol + hh * dv].float().view(t, hh, dv)
        ga = z * torch.sigmoid(z) if gate_act == "silu" else torch.sigmoid(z)
        y = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * w.float() * ga * out_scale
        return y.reshape(t, hh * dv).to(gate.dtype)
    _ck(o, "o", torch.float32)
    _ck(gate, "gate")
    _ck(w, "w", gate.dtype)
    y = torch.empty(t, hh * dv, dtype=gate.dtype, device=o.device)
    _k().dr_out_norm(y.data_ptr(), hh * dv, o.data_ptr(), gate.data_ptr(), gate.shape[1], int(gcol), w.data_ptr(), t, hh,
                     dv, float(eps), float(out_scale), 1 if gate_act == "sigmoid" else 0, _f32flag(gate), _stream())
    return y


def gated_delta_mixer(proj: torch.Tensor, col0: int, w: dict, spec: DeltaSpec, conv_state: torch.Tensor,
                      state: torch.Tensor, sb: SeqBatch, eps: float, out_scale: float = 1.0) -> torch.Tensor:
    """The mixer between its input and output projections.  ``proj`` [T, *] holds from column ``col0`` the
    fused projection q | k | v | gate | b | a.  ``w``: ``conv_w`` [taps, conv_width] (tap-major), ``a_log`` and
    ``dt_bias`` [heads] float32, ``norm`` [vdim].  ``conv_state`` [slots, taps - 1, conv_width] holds the
    last inputs of the convolutions, ``state`` the matrices.  Returns [T, heads vdim]."""
    c = spec.conv_width
    u, bd = conv_unit_gates(proj, col0, w["conv_w"], conv_state, w["a_log"], w["dt_bias"], sb, spec)
    o = delta_scan(u, bd, state, sb, spec)
    return gated_head_norm(o, proj, col0 + c, w["norm"], eps, out_scale)
