"""Linear attention with a decayed float32 matrix state per head.

Per head, with queries and keys q, k [dim], values v [vdim] and a decay a in (0, 1] per key channel:

    S <- diag(a) S + k v^T;   o = S^T q

so the read-out sees the current token's write.  ``S`` starts at zero and is carried from token to token in
a state slot (float32, whatever the activation type).  Two forms of the decay share the scan:

  * one fixed number per head (``decay`` [heads] float32) -- every key channel of the head, every token;
  * one number per key channel and token from a logit z: a = sigmoid(z + bias)^(1 / tau), evaluated in
    float32 as exp(log_sigmoid(z + bias) / tau).

q, k and v are columns of a fused projection; ``act`` "silu" applies x sigmoid(x) to each as it is read, and
``q_scale`` multiplies q.  The state pool is [slots, heads, vdim, dim]: a value column's key channels are
contiguous, which is how the scan kernel holds them in registers.

  :func:`decay_scan`        the recurrence over a varlen batch, state slots read and written
  :func:`gated_norm`        o / rms(o) * w * act(gate) per group of channels (``ops.delta.gated_head_norm``
                            with the gate's activation as a parameter)

Same dispatch as the other ops: CUDA tensors go to the in-tree HIP kernels (csrc/kernels/linattn.hip) and
raise if those are not built; CPU tensors run the plain PyTorch forms.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn.functional as F

from .seqmix import SeqBatch, _ck, _f32flag, _k, _ptr, _stream

MAX_KEY_DIM = 256        # the scan kernel keeps a state column in registers


@dataclass
class LinAttnSpec:
    """Sizes of one linear-attention mixer."""
    heads: int
    dim: int             # query / key size per head
    vdim: int            # value size per head


def decay_scan(proj: torch.Tensor, qcol: int, kcol: int, vcol: int, spec: LinAttnSpec, state: torch.Tensor,
               sb: SeqBatch, act: Optional[str] = None, q_scale: float = 1.0, decay: Optional[torch.Tensor] = None,
               z: Optional[torch.Tensor] = None, z_bias: Optional[torch.Tensor] = None, tau: float = 1.0) -> torch.Tensor:
    """The recurrence.  ``proj`` [T, *] holds q [heads, dim] from column ``qcol``, k from ``kcol``, v
    [heads, vdim] from ``vcol``.  Decay: ``decay`` [heads] float32, or ``z`` [T, heads dim] (activation
    type) with ``z_bias`` [heads dim] float32 and ``tau``.  ``state`` [slots, heads, vdim, dim] float32: a chunk
    that starts at position 0 starts from zero, any other from its slot; the slot holds the state after the
    chunk's last token.  Returns o [T, heads, vdim] float32."""
    t = proj.shape[0]
    hh, d, dv = spec.heads, spec.dim, spec.vdim
    if act not in (None, "silu"):
        raise ValueError(f"decay_scan: activation {act!r} (None, 'silu')")
    if (decay is None) == (z is None):
        raise ValueError("decay_scan: a decay per head or a logit per key channel, one of them")
    if state.shape[1:] != (hh, dv, d) or state.dtype != torch.float32 or proj.shape[1] < max(
            qcol + hh * d, kcol + hh * d, vcol + hh * dv):
        raise ValueError("decay_scan: shape / dtype mismatch")
    if decay is not None and (decay.numel() != hh or decay.dtype != torch.float32):
        raise ValueError("decay_scan: decay [heads] float32")
    if z is not None and (z.shape != (t, hh * d) or z_bias is None or z_bias.numel() != hh * d
                          or z_bias.dtype != torch.float32 or z.dtype != proj.dtype):
        raise ValueError("decay_scan: z [T, heads dim] with a float32 bias [heads dim]")
    if not proj.is_cuda:
        f = (lambda x: x * torch.sigmoid(x)) if act == "silu" else (lambda x: x)
        q = f(proj[:, qcol:qcol + hh * d].float()).view(t, hh, d) * q_scale
        k = f(proj[:, kcol:kcol + hh * d].float()).view(t, hh, d)
        v = f(proj[:, vcol:vcol + hh * dv].float()).view(t, hh, dv)
        if decay is not None:
            a = decay.float().view(1, hh, 1).expand(t, hh, d)
        else:
            a = torch.exp(F.logsigmoid(z.float() + z_bias.float()) / tau).view(t, hh, d)
        o = torch.empty(t, hh, dv, dtype=torch.float32)
        cu, pos, slots = sb.cu.tolist(), sb.positions.tolist(), sb.state_slots.tolist()
        for b in range(sb.num_seqs):
            lo, hi = cu[b], cu[b + 1]
            if hi == lo:
                continue
            s = state[slots[b]].clone() if pos[lo] > 0 else torch.zeros(hh, dv, d)
            for i in range(lo, hi):
                s = s * a[i][:, None, :] + v[i][:, :, None] * k[i][:, None, :]
                o[i] = torch.einsum("hvd,hd->hv", s, q[i])
            state[slots[b]] = s
        return o
    if d > MAX_KEY_DIM:
        raise ValueError(f"decay_scan: key size {d} > {MAX_KEY_DIM}")
    _ck(proj, "proj")
    _ck(state, "state", torch.float32)
    if decay is not None:
        _ck(decay, "decay", torch.float32)
    else:
        _ck(z, "z", proj.dtype)
        _ck(z_bias, "z_bias", torch.float32)
    o = torch.empty(t, hh, dv, dtype=torch.float32, device=proj.device)
    _k().la_scan(o.data_ptr(), proj.data_ptr(), proj.shape[1], int(qcol), int(kcol), int(vcol), _ptr(decay), _ptr(z),
                 _ptr(z_bias), 1.0 / float(tau), float(q_scale), 1 if act == "silu" else 0, state.data_ptr(),
                 sb.cu.data_ptr(), sb.positions.data_ptr(), sb.state_slots.data_ptr(), sb.num_seqs, sb.max_q_len, hh, d,
                 dv, _f32flag(proj), _stream())
    return o


def gated_norm(o: torch.Tensor, gate: torch.Tensor, gcol: int, w: torch.Tensor, eps: float, groups: int,
               gate_act: str = "silu") -> torch.Tensor:
    """o [T, C] float32 in ``groups`` equal groups of channels -> o / sqrt(mean_group(o^2) + eps) * w *
    act(gate[:, gcol + c]) as [T, C] in ``gate``'s dtype.  ``w`` has one group's channels (shared by the groups).
    ``gate_act``: "silu" (g sigmoid(g)) or "sigmoid"."""
    from .delta import gated_head_norm
    t, c = o.shape[0], o[0].numel()
    if c % groups or w.numel() != c // groups:
        raise ValueError("gated_norm: groups do not fit")
    return gated_head_norm(o.view(t, groups, c // groups), gate, gcol, w, eps, gate_act=gate_act)
