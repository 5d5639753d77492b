"""Mixtral MoE: router (K11) and expert MLPs (K12).

GPU path (bf16):
  router logits  = linear(x, W_router)                                   [T, E]
  moe_route      : softmax -> top-k -> renormalise, expert-sorted slots    (HIP, one launch)
  decode-sized T : grouped weight-streaming GEMMs on the sorted slots (gate|up + SwiGLU, then down)
                   entirely on device -- no host sync, so the decode step stays graph-capturable
  prefill-sized T: grouped 256 x 256-tile GEMMs over the expert-sorted slots (gemm_pp.hip
                   gemm_pp_moe: one launch per projection, every expert's row tiles in one grid,
                   counts / offsets read on the device -- no host sync, no per-expert loop; gate|up
                   with the SwiGLU in its epilogue, the token gather in its A staging)
  W8A8 experts   : the grouped fp8 kernel (moe_wide_gemm_fp8) at every T, also without a host sync
  moe_combine    : weighted sum of each token's top-k expert outputs        (HIP)
CPU path: the PyTorch reference (ops/reference.py).
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F

from .. import _ext, knobs
from . import reference as ref

GROUPED_MAX_TOKENS = 256      # beyond this the per-expert row count makes library GEMMs cheaper
ROUTER_FUSED_MAX_TOKENS = 64  # up to this many tokens the grouped-choice router product runs inside the selection kernel
# knobs.moe_variant: 0 = pick by expected rows per expert; 1..6 force a kernel variant
# (bench/moe_bench.py sweeps them).  knobs.moe_wide_min_pairs: token-expert pairs (T x top_k) from
# which the MFMA-tiled grouped kernel (gemm_wide.hip moe_wide_gemm) replaces the weight-streaming
# one (moe.hip); 0 disables it.  Mixtral-8x7B end to end (in-engine A/B,
# profiles/moe_wide.md): B=1 0.95x, B=4 1.10x, B=16 1.10x, B=64 1.25x, B=128 1.52x, B=256 2.23x.
# knobs.moe_fused_router: decode router as fused GEMV + top-k + scatter kernels instead of library
# GEMM + route kernel.


def route(router_logits: torch.Tensor, top_k: int):
    return ref.moe_route(router_logits, top_k)


def mlp(x, w_gate_up, w_down, topk_w, topk_ids):
    return ref.moe_mlp(x, w_gate_up, w_down, topk_w, topk_ids)


def forward(x: torch.Tensor, w_router: torch.Tensor, w_gate_up: torch.Tensor, w_down: torch.Tensor,
            top_k: int, expert_offset: int = 0) -> torch.Tensor:
    """``w_gate_up`` / ``w_down`` may hold a contiguous range of the experts (expert parallelism):
    experts ``[expert_offset, expert_offset + w_gate_up.shape[0])`` of the router's E.  Routing is
    always over all E; tokens routed elsewhere contribute zero here, so the expert-parallel
    group's sum (an all-reduce) is the full MoE output."""
    e_all = w_router.shape[0]
    if not (0 <= expert_offset and expert_offset + w_gate_up.shape[0] <= e_all):
        raise ValueError(f"experts [{expert_offset}, {expert_offset + w_gate_up.shape[0]}) outside the router's {e_all}")
    from . import quant
    fp8 = isinstance(w_gate_up, quant.Fp8Experts)
    if fp8 != isinstance(w_down, quant.Fp8Experts):
        raise TypeError("moe: gate|up and down experts must both be fp8 or both not")
    if not x.is_cuda:
        tw, tid = ref.moe_route(ref.linear(x, w_router), top_k)
        if fp8:
            return quant.moe_mlp_ref(x, w_gate_up, w_down, tw, tid - expert_offset)
        return ref.moe_mlp(x, w_gate_up, w_down, tw, tid - expert_offset)
    from . import linear, linear_swiglu
    k = _ext.kernels()
    st = torch.cuda.current_stream().cuda_stream
    t, h = x.shape
    e_loc, two_i, _ = w_gate_up.shape
    e = e_all
    ep = e_loc != e_all
    inter = two_i // 2
    if not (x.is_contiguous() and w_gate_up.is_contiguous() and w_down.is_contiguous()):
        raise ValueError("moe: operands must be contiguous")
    dev = x.device
    topk_w = torch.empty(t, top_k, dtype=torch.float32, device=dev)
    topk_ids = torch.empty(t, top_k, dtype=torch.int32, device=dev)
    counts = torch.empty(e, dtype=torch.int32, device=dev)
    offsets = torch.empty(e + 1, dtype=torch.int32, device=dev)
    sorted_tok = torch.empty(t * top_k, dtype=torch.int32, device=dev)
    inv = torch.empty(t * top_k, dtype=torch.int32, device=dev)
    if knobs.K.moe_fused_router and e in (8, 16) and h % 32 == 0 and x.dtype == w_router.dtype == torch.bfloat16 \
            and w_router.is_contiguous():
        # router GEMV + softmax/top-k + scatter in two launches (no [T, E] logits round trip), at
        # decode and prefill T alike
        k.moe_router_route(x.data_ptr(), w_router.data_ptr(), t, h, e, top_k, topk_w.data_ptr(), topk_ids.data_ptr(),
                           counts.data_ptr(), offsets.data_ptr(), sorted_tok.data_ptr(), inv.data_ptr(), st)
    else:
        logits = linear(x, w_router)
        k.moe_route(logits.data_ptr(), t, e, top_k, topk_w.data_ptr(), topk_ids.data_ptr(), counts.data_ptr(),
                    offsets.data_ptr(), sorted_tok.data_ptr(), inv.data_ptr(), st)
    # expert parallel: only this rank's experts fill their slot rows; the others stay zero
    ys = (torch.zeros if ep else torch.empty)(t * top_k, h, dtype=x.dtype, device=dev)
    # the local experts' counts / offsets are a contiguous slice of the routing arrays
    cnt_p, off_p = counts.data_ptr() + 4 * expert_offset, offsets.data_ptr() + 4 * expert_offset
    if fp8:
        # W8A8 experts (ops/quant.py): per-token e4m3 x gathered by the grouped kernel (its scales in
        # slot order), SwiGLU output re-quantized per slot row for the down projection
        if x.dtype != torch.bfloat16 or two_i % 128 or h % 128 or inter % 128:
            raise ValueError("moe fp8: bf16 activations, expert dims multiples of 128")
        # one grouped launch per projection at every T (decode and prefill): each workgroup walks its
        # expert's row chunks for one column tile, counts / offsets read on the device -- no host
        # sync, no per-expert loop (round-4 review: the prefill used to loop over experts on the host)
        xq, xsc = quant.quantize_rows(x)
        sa = xsc.index_select(0, sorted_tok.long())
        act = torch.empty(t * top_k, inter, dtype=x.dtype, device=dev)
        k.moe_wide_gemm_fp8(act.data_ptr(), xq.data_ptr(), sorted_tok.data_ptr(), w_gate_up.q.data_ptr(), cnt_p,
                            off_p, e_loc, two_i, h, 1, sa.data_ptr(), w_gate_up.scale.data_ptr(), st)
        aq, asc = quant.quantize_rows(act)
        k.moe_wide_gemm_fp8(ys.data_ptr(), aq.data_ptr(), 0, w_down.q.data_ptr(), cnt_p, off_p, e_loc, h, inter,
                            0, asc.data_ptr(), w_down.scale.data_ptr(), st)
    elif t <= GROUPED_MAX_TOKENS:
        act = torch.empty(t * top_k, inter, dtype=x.dtype, device=dev)
        rows = -(-t * top_k // e)        # expected rows per expert picks the kernel's row tile
        if 0 < knobs.K.moe_wide_min_pairs <= t * top_k and x.dtype == torch.bfloat16 and two_i % 128 == 0 and h % 128 == 0 \
                and h % 64 == 0 and inter % 64 == 0:
            ring = 0 if knobs.K.moe_deep_ring else 4          # mode bit 2: the 3-slot LDS ring
            k.moe_wide_gemm(act.data_ptr(), x.data_ptr(), sorted_tok.data_ptr(), w_gate_up.data_ptr(),
                            cnt_p, off_p, e_loc, two_i, h, 1 | ring, st)
            k.moe_wide_gemm(ys.data_ptr(), act.data_ptr(), 0, w_down.data_ptr(), cnt_p, off_p, e_loc, h, inter,
                            ring, st)
        else:
            k.moe_grouped_gemm(act.data_ptr(), x.data_ptr(), sorted_tok.data_ptr(), w_gate_up.data_ptr(),
                               cnt_p, off_p, e_loc, two_i, h, 1, rows, knobs.K.moe_variant, st)
            k.moe_grouped_gemm(ys.data_ptr(), act.data_ptr(), 0, w_down.data_ptr(), cnt_p, off_p, e_loc, h, inter, 0,
                               rows, knobs.K.moe_variant, st)
    elif x.dtype == torch.bfloat16 and two_i % 256 == 0 and h % 256 == 0 and inter % 64 == 0 and h % 64 == 0 \
            and t * h * 2 < (1 << 32) and t * top_k * inter * 2 < (1 << 32):
        # prefill: one grouped launch per projection over every local expert's row tiles (the kernel
        # addresses each A operand with 32-bit buffer offsets: larger batches take the per-expert path)
        slots = t * top_k
        act = torch.empty(slots, inter, dtype=x.dtype, device=dev)
        k.gemm_pp_moe(act.data_ptr(), x.data_ptr(), sorted_tok.data_ptr(), w_gate_up.data_ptr(), cnt_p, off_p,
                      e_loc, two_i, h, t, slots, 1, st)
        k.gemm_pp_moe(ys.data_ptr(), act.data_ptr(), 0, w_down.data_ptr(), cnt_p, off_p, e_loc, h, inter, slots,
                      slots, 0, st)
    else:
        # odd expert dims (test-size models): per-expert GEMMs, counts read on the host
        xs = x.index_select(0, sorted_tok.long())
        off = offsets.cpu().tolist()
        for j in range(e_loc):
            a, b = off[expert_offset + j], off[expert_offset + j + 1]
            if b > a:
                ys[a:b] = F.linear(linear_swiglu(xs[a:b], w_gate_up[j]), w_down[j])
    out = torch.empty_like(x)
    k.moe_combine(out.data_ptr(), ys.data_ptr(), topk_w.data_ptr(), inv.data_ptr(), t, h, top_k, st)
    return out


# ------------------------------------------------------------------ grouped-choice router, squared-ReLU experts
def route_grouped_choice(logits: torch.Tensor, correction: Optional[torch.Tensor], num_experts: int, top: int,
                         groups: int = 1, keep: int = 1, scale: float = 1.0):
    """Reference (PyTorch, any device) of the grouped-choice router: scores s = sigmoid(logits[:, :E]);
    selection ranks s + correction; the experts are split into ``groups`` contiguous blocks of equal size,
    blocks are ranked by the sum of their top two selection values, and experts outside the ``keep``
    highest-ranked blocks are masked with -inf; the mixing weights are the selected experts' plain s,
    normalised to sum one (+ 1e-20 in the divisor) and multiplied by ``scale``.  Returns (weights
    [T, top] float32, ids [T, top] int64)."""
    t = logits.shape[0]
    e = num_experts
    s = torch.sigmoid(logits[:, :e].float())
    ch = s if correction is None else s + correction.float()
    if keep < groups:
        gsz = e // groups
        gs = ch.view(t, groups, gsz).topk(min(2, gsz), dim=-1).values.sum(-1)
        kept = torch.zeros(t, groups, dtype=torch.bool, device=logits.device)
        kept.scatter_(1, gs.topk(keep, dim=-1).indices, True)
        ch = ch.masked_fill(~kept.repeat_interleave(gsz, 1), float("-inf"))
    ids = ch.topk(top, dim=-1).indices
    w = s.gather(1, ids)
    return w / (w.sum(-1, keepdim=True) + 1e-20) * scale, ids


def grouped_choice_ffn(x: torch.Tensor, w_router: torch.Tensor, correction: Optional[torch.Tensor],
                       w_up: torch.Tensor, w_down: torch.Tensor, top: int, groups: int = 1, keep: int = 1,
                       scale: float = 1.0, shared_up: Optional[torch.Tensor] = None,
                       shared_down: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Mixture of experts of the form down_e(relu(up_e x)^2) with the grouped-choice router
    (:func:`route_grouped_choice`).  ``w_router`` [E (+ 1), W] float32: the router rows, then -- with a
    shared expert -- the row of its gate; the logits are a float32 product.  ``w_up`` [E, F, W],
    ``w_down`` [E, W, F].  ``shared_up`` [Fs, W] / ``shared_down`` [W, Fs]: an expert of the same form that
    every token uses, times sigmoid(gate logit), one gate per token."""
    e, f, width = w_up.shape
    t = x.shape[0]
    has_shared = shared_up is not None
    if w_router.shape[0] != e + (1 if has_shared else 0) or w_router.dtype != torch.float32:
        raise ValueError("grouped_choice_ffn: router rows = experts (+ 1 with a shared expert), float32")
    if not x.is_cuda:
        logits = F.linear(x.float(), w_router)                   # float32 also for bf16 activations
        tw, ids = route_grouped_choice(logits, correction, e, top, groups, keep, scale)
        out = torch.zeros(t, width, dtype=torch.float32)
        xf = x.float()
        for j in range(e):
            rows, col = (ids == j).nonzero(as_tuple=True)
            if rows.numel():
                y = F.linear(torch.relu(F.linear(xf[rows], w_up[j].float())).square(), w_down[j].float())
                out.index_add_(0, rows, y * tw[rows, col, None])
        if has_shared:
            y = F.linear(torch.relu(F.linear(xf, shared_up.float())).square(), shared_down.float())
            out += y * torch.sigmoid(logits[:, e:e + 1])
        return out.to(x.dtype)
    from . import linear
    k = _ext.kernels()
    st = torch.cuda.current_stream().cuda_stream
    dev = x.device
    f32 = 1 if x.dtype == torch.float32 else 0
    if not (x.is_contiguous() and w_up.is_contiguous() and w_down.is_contiguous() and w_router.is_contiguous()):
        raise ValueError("grouped_choice_ffn: operands must be contiguous")
    if correction is not None and (correction.dtype != torch.float32 or correction.numel() != e):
        raise ValueError("grouped_choice_ffn: correction is float32 [E]")
    topk_w = torch.empty(t, top, dtype=torch.float32, device=dev)
    topk_ids = torch.empty(t, top, dtype=torch.int32, device=dev)
    counts = torch.empty(e, dtype=torch.int32, device=dev)
    offsets = torch.empty(e + 1, dtype=torch.int32, device=dev)
    sorted_tok = torch.empty(t * top, dtype=torch.int32, device=dev)
    inv = torch.empty(t * top, dtype=torch.int32, device=dev)
    cp = 0 if correction is None else correction.data_ptr()
    if t <= ROUTER_FUSED_MAX_TOKENS:
        # few tokens: the float32 router product and the selection in one launch (+ the scatter)
        logits = torch.empty(t, w_router.shape[0], dtype=torch.float32, device=dev)
        k.moe_router_groups(x.data_ptr(), w_router.data_ptr(), width, w_router.shape[0], logits.data_ptr(), cp, t, e, top,
                            groups, keep, float(scale), 0, topk_w.data_ptr(), topk_ids.data_ptr(), counts.data_ptr(),
                            offsets.data_ptr(), sorted_tok.data_ptr(), inv.data_ptr(), f32, st)
    else:
        logits = F.linear(x.float(), w_router)                   # float32 also for bf16 activations
        k.moe_route_groups(logits.data_ptr(), logits.shape[1], cp, t, e, top, groups, keep, float(scale), 0,
                           topk_w.data_ptr(), topk_ids.data_ptr(), counts.data_ptr(), offsets.data_ptr(),
                           sorted_tok.data_ptr(), inv.data_ptr(), st)
    slots = t * top
    ys = torch.empty(slots, width, dtype=x.dtype, device=dev)
    bf = x.dtype == torch.bfloat16
    if bf and t <= GROUPED_MAX_TOKENS and width % 128 == 0 and f % 128 == 0 and 0 < knobs.K.moe_wide_min_pairs <= slots:
        # decode-sized with several rows per expert: the MFMA-tiled grouped kernel (it has no squared-ReLU
        # epilogue: the activation is a launch of its own on the small [slots, F] tensor), no host sync
        act = torch.empty(slots, f, dtype=x.dtype, device=dev)
        ring = 0 if knobs.K.moe_deep_ring else 4
        k.moe_wide_gemm(act.data_ptr(), x.data_ptr(), sorted_tok.data_ptr(), w_up.data_ptr(), counts.data_ptr(),
                        offsets.data_ptr(), e, f, width, ring, st)
        k.relu_sq(act.data_ptr(), act.numel(), 0, st)
        k.moe_wide_gemm(ys.data_ptr(), act.data_ptr(), 0, w_down.data_ptr(), counts.data_ptr(), offsets.data_ptr(), e,
                        width, f, ring, st)
    elif bf and t <= GROUPED_MAX_TOKENS and width % 128 == 0 and f % 128 == 0:
        # a few rows: grouped weight-streaming GEMMs on the expert-sorted slots, no host sync
        act = torch.empty(slots, f, dtype=x.dtype, device=dev)
        rows = -(-slots // e)
        k.moe_grouped_gemm(act.data_ptr(), x.data_ptr(), sorted_tok.data_ptr(), w_up.data_ptr(), counts.data_ptr(),
                           offsets.data_ptr(), e, f, width, 2, rows, knobs.K.moe_variant, st)     # mode 2: relu^2
        k.moe_grouped_gemm(ys.data_ptr(), act.data_ptr(), 0, w_down.data_ptr(), counts.data_ptr(), offsets.data_ptr(),
                           e, width, f, 0, rows, knobs.K.moe_variant, st)
    elif bf and f % 256 == 0 and width % 256 == 0 and t * width * 2 < (1 << 32) and slots * f * 2 < (1 << 32):
        # prompt-sized: one grouped 256 x 256-tile launch per projection over every expert's row tiles
        act = torch.empty(slots, f, dtype=x.dtype, device=dev)
        k.gemm_pp_moe(act.data_ptr(), x.data_ptr(), sorted_tok.data_ptr(), w_up.data_ptr(), counts.data_ptr(),
                      offsets.data_ptr(), e, f, width, t, slots, 2, st)                                  # mode 2: relu^2
        k.gemm_pp_moe(ys.data_ptr(), act.data_ptr(), 0, w_down.data_ptr(), counts.data_ptr(), offsets.data_ptr(), e,
                      width, f, slots, slots, 0, st)
    else:
        # float32 and odd expert sizes: per-expert library GEMMs, counts read on the host
        xs = x.index_select(0, sorted_tok.long())
        off = offsets.cpu().tolist()
        for j in range(e):
            a, b = off[j], off[j + 1]
            if b > a:
                u = F.linear(xs[a:b], w_up[j])
                k.relu_sq(u.data_ptr(), u.numel(), f32, st)
                ys[a:b] = F.linear(u, w_down[j])
    sh = None
    if has_shared:
        u = linear(x, shared_up)
        k.relu_sq(u.data_ptr(), u.numel(), f32, st)
        sh = linear(u, shared_down)
    out = torch.empty_like(x)
    k.moe_combine_gated(out.data_ptr(), ys.data_ptr(), topk_w.data_ptr(), inv.data_ptr(), 0 if sh is None else sh.data_ptr(),
                        logits.data_ptr() + 4 * e if has_shared else 0, logits.shape[1], t, width, top, f32, st)
    return out


def relu_sq_(y: torch.Tensor) -> torch.Tensor:
    """y <- max(y, 0)^2 in place (the activation of feed-forwards of the form down(relu(up x)^2))."""
    if not y.is_cuda:
        return y.copy_(torch.relu(y.float()).square().to(y.dtype))
    if not y.is_contiguous() or y.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError("relu_sq_: contiguous bfloat16 or float32")
    _ext.kernels().relu_sq(y.data_ptr(), y.numel(), 1 if y.dtype == torch.float32 else 0,
                           torch.cuda.current_stream().cuda_stream)
    return y


# ------------------------------------------------------------------ biased router, softmax over the chosen logits, GLU experts
def route_softmax_top(logits: torch.Tensor, top: int, scale: float = 1.0):
    """Reference (PyTorch, any device): the ``top`` largest logits per row (ties: the lower index) and the
    softmax over those logits only.  Returns (weights [T, top] float32, ids [T, top] int64)."""
    v, ids = torch.sort(logits.float(), dim=-1, descending=True, stable=True)
    return torch.softmax(v[:, :top], -1) * scale, ids[:, :top]


def softmax_top_ffn(x: torch.Tensor, w_router: torch.Tensor, b_router: Optional[torch.Tensor],
                    w_gate_up: torch.Tensor, w_down: torch.Tensor, top: int,
                    shared_gate_up: Optional[torch.Tensor] = None, shared_down: Optional[torch.Tensor] = None,
                    scale: float = 1.0) -> torch.Tensor:
    """Mixture of GLU experts down_e(silu(gate_e x) * (up_e x)): router logits ``w_router x + b_router``
    are a float32 product (``w_router`` [E, W] and ``b_router`` [E] float32), every token uses the ``top``
    experts with the largest logits, weighted by the softmax over those logits only.  ``w_gate_up``
    [E, 2 F, W] (gate rows, then up rows), ``w_down`` [E, W, F].  ``shared_gate_up`` [2 Fs, W] /
    ``shared_down`` [W, Fs]: an expert of the same form that every token uses, added unweighted."""
    e, two_f, width = w_gate_up.shape
    f = two_f // 2
    t = x.shape[0]
    if w_router.shape != (e, width) or w_router.dtype != torch.float32 or (
            b_router is not None and (b_router.dtype != torch.float32 or b_router.numel() != e)):
        raise ValueError("softmax_top_ffn: router [E, W] and bias [E] in float32")
    if not 1 <= top <= min(e, 16):
        raise ValueError("softmax_top_ffn: 1 <= top <= min(experts, 16)")
    if not x.is_cuda:
        xf = x.float()
        tw, ids = route_softmax_top(F.linear(xf, w_router, b_router), top, scale)
        out = torch.zeros(t, width, dtype=torch.float32)

        def glu(h, wgu, wd):
            gu = F.linear(h, wgu.float())
            return F.linear(F.silu(gu[:, :wgu.shape[0] // 2]) * gu[:, wgu.shape[0] // 2:], wd.float())
        for j in range(e):
            rows, col = (ids == j).nonzero(as_tuple=True)
            if rows.numel():
                out.index_add_(0, rows, glu(xf[rows], w_gate_up[j], w_down[j]) * tw[rows, col, None])
        if shared_gate_up is not None:
            out += glu(xf, shared_gate_up, shared_down)
        return out.to(x.dtype)
    from . import linear
    from .latent import linear_swiglu
    k = _ext.kernels()
    st = torch.cuda.current_stream().cuda_stream
    dev = x.device
    f32 = 1 if x.dtype == torch.float32 else 0
    if not (x.is_contiguous() and w_gate_up.is_contiguous() and w_down.is_contiguous() and w_router.is_contiguous()):
        raise ValueError("softmax_top_ffn: operands must be contiguous")
    topk_w = torch.empty(t, top, dtype=torch.float32, device=dev)
    topk_ids = torch.empty(t, top, dtype=torch.int32, device=dev)
    counts = torch.empty(e, dtype=torch.int32, device=dev)
    offsets = torch.empty(e + 1, dtype=torch.int32, device=dev)
    sorted_tok = torch.empty(t * top, dtype=torch.int32, device=dev)
    inv = torch.empty(t * top, dtype=torch.int32, device=dev)
    bp = 0 if b_router is None else b_router.data_ptr()
    if t <= ROUTER_FUSED_MAX_TOKENS:
        # few tokens: the float32 router product and the selection in one launch (+ the scatter)
        logits = torch.empty(t, e, dtype=torch.float32, device=dev)
        k.moe_router_groups(x.data_ptr(), w_router.data_ptr(), width, e, logits.data_ptr(), bp, t, e, top, 1, 1,
                            float(scale), 1, topk_w.data_ptr(), topk_ids.data_ptr(), counts.data_ptr(),
                            offsets.data_ptr(), sorted_tok.data_ptr(), inv.data_ptr(), f32, st)
    else:
        logits = F.linear(x.float(), w_router)                   # float32 also for bf16 activations
        k.moe_route_groups(logits.data_ptr(), e, bp, t, e, top, 1, 1, float(scale), 1, topk_w.data_ptr(),
                           topk_ids.data_ptr(), counts.data_ptr(), offsets.data_ptr(), sorted_tok.data_ptr(),
                           inv.data_ptr(), st)
    slots = t * top
    ys = torch.empty(slots, width, dtype=x.dtype, device=dev)
    bf = x.dtype == torch.bfloat16
    cp, op = counts.data_ptr(), offsets.data_ptr()
    if bf and t <= GROUPED_MAX_TOKENS and width % 128 == 0 and f % 128 == 0:
        # decode-sized: grouped GEMMs on the expert-sorted slots with the SwiGLU in the first one's
        # epilogue, no host sync (the MFMA-tiled kernel from several rows per expert on)
        act = torch.empty(slots, f, dtype=x.dtype, device=dev)
        if 0 < knobs.K.moe_wide_min_pairs <= slots:
            ring = 0 if knobs.K.moe_deep_ring else 4
            k.moe_wide_gemm(act.data_ptr(), x.data_ptr(), sorted_tok.data_ptr(), w_gate_up.data_ptr(), cp, op, e, two_f,
                            width, 1 | ring, st)
            k.moe_wide_gemm(ys.data_ptr(), act.data_ptr(), 0, w_down.data_ptr(), cp, op, e, width, f, ring, st)
        else:
            rows = -(-slots // e)
            k.moe_grouped_gemm(act.data_ptr(), x.data_ptr(), sorted_tok.data_ptr(), w_gate_up.data_ptr(), cp, op, e,
                               two_f, width, 1, rows, knobs.K.moe_variant, st)
            k.moe_grouped_gemm(ys.data_ptr(), act.data_ptr(), 0, w_down.data_ptr(), cp, op, e, width, f, 0, rows,
                               knobs.K.moe_variant, st)
    elif bf and two_f % 256 == 0 and width % 256 == 0 and f % 64 == 0 and t * width * 2 < (1 << 32) \
            and slots * f * 2 < (1 << 32):
        # prompt-sized: one grouped 256 x 256-tile launch per projection over every expert's row tiles
        act = torch.empty(slots, f, dtype=x.dtype, device=dev)
        k.gemm_pp_moe(act.data_ptr(), x.data_ptr(), sorted_tok.data_ptr(), w_gate_up.data_ptr(), cp, op, e, two_f,
                      width, t, slots, 1, st)
        k.gemm_pp_moe(ys.data_ptr(), act.data_ptr(), 0, w_down.data_ptr(), cp, op, e, width, f, slots, slots, 0, st)
    else:
        # float32 and odd expert sizes: per-expert library GEMMs, counts read on the host
        xs = x.index_select(0, sorted_tok.long())
        off = offsets.cpu().tolist()
        for j in range(e):
            a, b = off[j], off[j + 1]
            if b > a:
                ys[a:b] = F.linear(linear_swiglu(xs[a:b], w_gate_up[j]), w_down[j])
    sh = None
    if shared_gate_up is not None:
        sh = linear(linear_swiglu(x, shared_gate_up), shared_down)
    out = torch.empty_like(x)
    k.moe_combine_gated(out.data_ptr(), ys.data_ptr(), topk_w.data_ptr(), inv.data_ptr(), 0 if sh is None else sh.data_ptr(),
                        0, 0, t, width, top, f32, st)
    return out
