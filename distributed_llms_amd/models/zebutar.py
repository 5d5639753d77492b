"""Zebutar: a layer-list decoder whose sublayers read the residual stream itself and whose OUTPUTS are
normed, with a mixer made of two mixers side by side -- softmax attention inside fixed chunks of
positions and a gated delta rule -- and dense or mixture-of-experts feed-forwards.

``config.json`` keys (read by ``config._from_zebutar``): ``width``, ``vocab``, ``norm.eps`` and ``layers``:
per layer ``type`` ("parallel"), ``mixer`` and ``mlp``.

  mixer: ``left`` -- attention: ``heads``, ``kv_heads``, ``dim`` (q / k head size), ``vdim``, ``scale``, ``rot``
      (``base``, ``dims``: the first ``dims`` dimensions of every head turn, dimension i paired with
      i + dims / 2), ``mask.size`` (a query sees the keys of its own chunk of that many positions,
      chunks counted from position 0; absent: plain causal); q and k pass an RMS norm over the WHOLE
      projection (all heads at once, plain weights) before the rotation.
      ``right`` -- gated delta rule: ``heads`` (value heads), ``kv_heads`` (q / k heads), ``dim``, ``vdim``,
      ``conv`` (taps of the short causal convolutions on q, k and v, each followed by silu).
      ``left_scale``, ``right_scale``: the mixer's output is their weighted sum.
  mlp: None, {"kind": "dense", "ff"} (down(relu(up x)^2)) or {"kind": "moe", "expert": {"ff"}, "router":
      {"experts", "top"}, "shared": {"ff"} | None} (SwiGLU experts, biased float32 router, softmax over
      the chosen logits, an ungated shared expert).

One layer: x += rms(mixer(x)) (1 + w1);  x += rms(ff(x)) (1 + w2).  The embedding passes an RMS norm of the
same form before the first layer, the stream another before the head.

Checkpoint names: ``embed``, ``embed.norm``, ``final.norm``, ``head``; per layer ``l<i>.``: ``norm1``, ``norm2``;
``mix.left.q|k|v|o``, ``mix.left.q.norm``, ``mix.left.k.norm``; ``mix.right.q|k|v`` (+ ``.conv`` [channels, taps]),
``mix.right.b``, ``mix.right.a``, ``mix.right.A_log``, ``mix.right.dt_bias``, ``mix.right.g``, ``mix.right.norm``,
``mix.right.o``; ``mlp.up|down`` or ``mlp.router`` (+ ``.b``), ``mlp.e<j>.gate|up|down``, ``mlp.shared.gate|up|down``.
Linear weights are [out, in].

What a sequence keeps between steps: paged K/V of every layer's attention (one block table for all,
from the engine's BlockManager) and one STATE SLOT: per layer the last ``conv - 1`` projected rows of the
delta rule's q | k | v and its float32 state matrices [heads, dim, vdim].  The residual stream, norms,
rotation angles, attention scores and weights, router logits, and everything inside the recurrence
are float32 also when activations are bfloat16.
"""
from __future__ import annotations

from typing import Any, Dict, Optional

import torch

from .. import ops
from ..config import ModelConfig
from ..ops import delta as dl
from ..ops import moe
from ..ops import seqmix as sm
from .hybrid import LayerListStage
from .stage import BatchMeta
from .weights import tensor_seed


def delta_spec(layer: Dict[str, Any]) -> dl.DeltaSpec:
    r = layer["mixer"]["right"]
    return dl.DeltaSpec(heads=int(r["heads"]), kv_heads=int(r["kv_heads"]), dim=int(r["dim"]), vdim=int(r["vdim"]),
                        taps=int(r["conv"]))


def left_width(layer: Dict[str, Any]) -> int:
    """Columns of the attention's fused input projection: q | k | v."""
    m = layer["mixer"]["left"]
    return m["heads"] * m["dim"] + m["kv_heads"] * (m["dim"] + m["vdim"])


def layer_shapes(width: int, layer: Dict[str, Any]) -> Dict[str, tuple]:
    """Checkpoint tensor name (without the ``l<i>.`` prefix) -> shape."""
    l, sp = layer["mixer"]["left"], delta_spec(layer)
    h, g, d, dv = l["heads"], l["kv_heads"], l["dim"], l["vdim"]
    s: Dict[str, tuple] = {
        "norm1": (width,),
        "mix.left.q": (h * d, width), "mix.left.k": (g * d, width), "mix.left.v": (g * dv, width),
        "mix.left.q.norm": (h * d,), "mix.left.k.norm": (g * d,), "mix.left.o": (width, h * dv),
        "mix.right.q": (sp.kv_heads * sp.dim, width), "mix.right.q.conv": (sp.kv_heads * sp.dim, sp.taps),
        "mix.right.k": (sp.kv_heads * sp.dim, width), "mix.right.k.conv": (sp.kv_heads * sp.dim, sp.taps),
        "mix.right.v": (sp.heads * sp.vdim, width), "mix.right.v.conv": (sp.heads * sp.vdim, sp.taps),
        "mix.right.b": (sp.heads, width), "mix.right.a": (sp.heads, width), "mix.right.A_log": (sp.heads,),
        "mix.right.dt_bias": (sp.heads,), "mix.right.g": (sp.heads * sp.vdim, width), "mix.right.norm": (sp.vdim,),
        "mix.right.o": (width, sp.heads * sp.vdim)}
    mlp = layer.get("mlp")
    if mlp:
        s["norm2"] = (width,)
    if mlp and mlp["kind"] == "dense":
        s.update({"mlp.up": (mlp["ff"], width), "mlp.down": (width, mlp["ff"])})
    elif mlp:
        e, f = mlp["router"]["experts"], mlp["expert"]["ff"]
        s.update({"mlp.router": (e, width), "mlp.router.b": (e,)})
        for j in range(e):
            s.update({f"mlp.e{j}.gate": (f, width), f"mlp.e{j}.up": (f, width), f"mlp.e{j}.down": (width, f)})
        if mlp.get("shared"):
            fs = mlp["shared"]["ff"]
            s.update({"mlp.shared.gate": (fs, width), "mlp.shared.up": (fs, width), "mlp.shared.down": (width, fs)})
    return s


def model_shapes(cfg: ModelConfig) -> Dict[str, tuple]:
    w = cfg.hidden_size
    s = {"embed": (cfg.vocab_size, w), "embed.norm": (w,), "final.norm": (w,), "head": (cfg.vocab_size, w)}
    for i, layer in enumerate(cfg.layers):
        s.update({f"l{i}.{n}": shp for n, shp in layer_shapes(w, layer).items()})
    return s


def synth_state_dict(cfg: ModelConfig, seed: int = 0, dtype=torch.float32) -> Dict[str, torch.Tensor]:
    """Seeded random weights under the checkpoint names (CPU): projections ~ N(0, 1 / fan_in), one-plus norm
    weights small around zero, plain norm weights around one, decays spread per head, the router wide
    enough that choices are not close calls."""
    sd = {}
    for name, shape in model_shapes(cfg).items():
        g = torch.Generator().manual_seed(tensor_seed(seed, 0, name))
        leaf = name.rsplit(".", 1)[-1]
        if leaf in ("norm1", "norm2") or name in ("embed.norm", "final.norm"):
            t = 0.1 * torch.randn(shape, generator=g)
        elif leaf == "norm":
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif leaf == "A_log":
            t = torch.rand(shape, generator=g) * 3.0 - 3.0
        elif leaf == "dt_bias":
            t = torch.randn(shape, generator=g)
        elif leaf == "conv":
            t = torch.randn(shape, generator=g) / shape[1] ** 0.5
        elif name.endswith("router.b"):
            t = 0.5 * torch.randn(shape, generator=g)
        elif leaf == "router":
            t = 3.0 * torch.randn(shape, generator=g) / shape[-1] ** 0.5
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) / shape[-1] ** 0.5
        sd[name] = t.to(dtype)
    return sd


class ZebutarStage(LayerListStage):
    """All layers of a Zebutar model on one device (see the module docstring)."""

    @staticmethod
    def layer_param_count(width: int, layer: Dict[str, Any]) -> int:
        return sum(int(torch.Size(s).numel()) for s in layer_shapes(width, layer).values())

    @staticmethod
    def kv_elements_per_token(cfg: ModelConfig) -> int:
        return sum(l["mixer"]["left"]["kv_heads"] * (l["mixer"]["left"]["dim"] + l["mixer"]["left"]["vdim"])
                   for l in cfg.layers)

    def __init__(self, cfg: ModelConfig, layer_start: int = 0, layer_end: Optional[int] = None, device="cpu",
                 dtype=torch.bfloat16, units: Optional[tuple] = None, tp=None, unit_group: int = 2):
        super().__init__(cfg, layer_start, layer_end, device, dtype, units, tp, unit_group)
        self.dspec = [delta_spec(l) for l in self.specs]
        self.freqs = []
        for i, l in enumerate(self.specs):
            if l["type"] != "parallel":
                raise ValueError(f"layer {i}: unsupported type {l['type']!r}")
            m, sp = l["mixer"]["left"], self.dspec[i]
            r = m["rot"]
            if m["heads"] % m["kv_heads"] or r["dims"] % 2 or r["dims"] > m["dim"]:
                raise ValueError(f"layer {i}: attention heads / kv_heads / rot.dims do not fit")
            if sp.heads % sp.kv_heads or sp.taps < 1 or sp.dim > dl.MAX_KEY_DIM:
                raise ValueError(f"layer {i}: delta rule heads / kv_heads / conv / dim do not fit")
            self.freqs.append(sm.rotary_frequencies(int(r["dims"]), float(r["base"])).to(self.device))
            mlp = l.get("mlp")
            if mlp and mlp["kind"] == "moe" and not 1 <= mlp["router"]["top"] <= min(16, mlp["router"]["experts"]):
                raise ValueError(f"layer {i}: router top does not fit")

    # ------------------------------------------------------------------ weights
    def load_hf_state(self, sd: Dict[str, torch.Tensor]) -> "ZebutarStage":
        """From checkpoint-named tensors: one input projection per layer (attention q | k | v, then the
        delta rule's q | k | v | g | b | a), convolution weights tap-major ([taps, C]), gate | up stacked per
        expert; what feeds float32 math directly (router rows and bias, A_log, dt_bias) is float32."""
        want = model_shapes(self.cfg)
        for n, shp in want.items():
            if n not in sd:
                raise KeyError(f"checkpoint lacks {n}")
            if tuple(sd[n].shape) != tuple(shp):
                raise ValueError(f"{n}: shape {tuple(sd[n].shape)}, config says {tuple(shp)}")
        cv = lambda t: t.to(device=self.device, dtype=self.dtype).contiguous()
        f32 = lambda t: t.to(device=self.device, dtype=torch.float32).contiguous()
        self.embed = {"embed": cv(sd["embed"]), "norm": cv(sd["embed.norm"])}
        self.head = {"final_norm": cv(sd["final.norm"]), "lm_head": cv(sd["head"])}
        self.layers = []
        for i, layer in enumerate(self.specs):
            p = f"l{i}."
            pl, pr = p + "mix.left.", p + "mix.right."
            w: Dict[str, Any] = {"norm1": cv(sd[p + "norm1"])}
            w["w_in"] = cv(torch.cat([sd[pl + "q"], sd[pl + "k"], sd[pl + "v"], sd[pr + "q"], sd[pr + "k"], sd[pr + "v"],
                                      sd[pr + "g"], sd[pr + "b"], sd[pr + "a"]], 0))
            w["q_norm"], w["k_norm"] = cv(sd[pl + "q.norm"]), cv(sd[pl + "k.norm"])
            w["wo_left"], w["wo_right"] = cv(sd[pl + "o"]), cv(sd[pr + "o"])
            w["right"] = {"conv_w": cv(torch.cat([sd[pr + "q.conv"], sd[pr + "k.conv"], sd[pr + "v.conv"]], 0).t()),
                          "a_log": f32(sd[pr + "A_log"]), "dt_bias": f32(sd[pr + "dt_bias"]), "norm": cv(sd[pr + "norm"])}
            mlp = layer.get("mlp")
            if mlp:
                w["norm2"] = cv(sd[p + "norm2"])
            if mlp and mlp["kind"] == "dense":
                w["w_up"], w["w_down"] = cv(sd[p + "mlp.up"]), cv(sd[p + "mlp.down"])
            elif mlp:
                e = mlp["router"]["experts"]
                w["router"], w["router_b"] = f32(sd[p + "mlp.router"]), f32(sd[p + "mlp.router.b"])
                w["e_gu"] = cv(torch.stack([torch.cat([sd[p + f"mlp.e{j}.gate"], sd[p + f"mlp.e{j}.up"]], 0)
                                            for j in range(e)], 0))
                w["e_down"] = cv(torch.stack([sd[p + f"mlp.e{j}.down"] for j in range(e)], 0))
                if mlp.get("shared"):
                    w["s_gu"] = cv(torch.cat([sd[p + "mlp.shared.gate"], sd[p + "mlp.shared.up"]], 0))
                    w["s_down"] = cv(sd[p + "mlp.shared.down"])
            self.layers.append(w)
        return self

    def init_synthetic(self, seed: int = 0) -> "ZebutarStage":
        return self.load_hf_state(synth_state_dict(self.cfg, seed))

    # ------------------------------------------------------------------ cache and state
    def cache_shapes(self, block_size: int) -> Dict[Any, tuple]:
        """Per layer the attention's paged pair: k [NB, G, BS, dim], v [NB, G, vdim, BS] (transposed inside a block)."""
        out = {}
        for i, l in enumerate(self.specs):
            m = l["mixer"]["left"]
            out[i] = ((m["kv_heads"], block_size, m["dim"]), (m["kv_heads"], m["vdim"], block_size))
        return out

    def allocate_state(self, num_slots: int):
        """State pools, one row per BlockManager state slot: per layer the convolution tail
        [slots, taps - 1, q | k | v channels] (activation dtype) and the delta rule's matrices
        [slots, heads, dim, vdim] float32."""
        self.num_state_slots = num_slots
        self.state = [{"conv": torch.zeros(num_slots, sp.taps - 1, sp.conv_width, dtype=self.dtype, device=self.device),
                       "s": torch.zeros(num_slots, sp.heads, sp.dim, sp.vdim, dtype=torch.float32, device=self.device)}
                      for sp in self.dspec]
        return self.state

    def state_bytes_per_slot(self) -> int:
        e = torch.empty((), dtype=self.dtype).element_size()
        return sum(e * (sp.taps - 1) * sp.conv_width + 4 * sp.heads * sp.dim * sp.vdim for sp in self.dspec)

    @property
    def graph_capturable(self) -> bool:
        """Whether a decode step runs without a host round trip.  Experts whose sizes the grouped
        kernels do not take (and float32) read the per-expert row counts on the host, which a HIP-graph
        capture cannot record: such a model decodes with eager launches."""
        for l in self.specs:
            mlp = l.get("mlp")
            if mlp and mlp["kind"] == "moe" and (self.dtype != torch.bfloat16 or self.cfg.hidden_size % 128
                                                 or mlp["expert"]["ff"] % 128):
                return False
        return True

    # ------------------------------------------------------------------ forward
    def _mixer(self, i: int, h: torch.Tensor, w, meta: BatchMeta, sb: sm.SeqBatch):
        """Both mixers on the same input: (attention output, delta rule output), each [T, W]."""
        m, sp = self.specs[i]["mixer"]["left"], self.dspec[i]
        kc, vc = self.kv.caches[i]
        proj = ops.linear(h, w["w_in"])
        q = sm.rownorm_rope(proj, 0, w["q_norm"], w["k_norm"], self.freqs[i], self.cfg.norm_eps, kc, vc,
                            meta.slot_mapping, sb.positions, m["heads"], m["kv_heads"], m["dim"], m["vdim"])
        nd = meta.num_decode if meta.is_prefill else meta.num_seqs
        chunk = int((m.get("mask") or {}).get("size") or 0)                   # no mask entry: plain causal attention
        a = sm.window_attention(q, kc, vc, meta.block_tables, sb, 1 << 30, float(m["scale"]), num_decode=nd, chunk=chunk,
                                max_ctx=meta.max_ctx_d if (meta.is_prefill and nd) else meta.max_ctx)
        st = self.state[i]
        r = dl.gated_delta_mixer(proj, left_width(self.specs[i]), w["right"], sp, st["conv"], st["s"], sb,
                                 self.cfg.norm_eps)
        return ops.linear(a.view(a.shape[0], -1), w["wo_left"]), ops.linear(r, w["wo_right"])

    def _ff(self, h: torch.Tensor, w, mlp) -> torch.Tensor:
        if mlp["kind"] == "dense":
            return ops.linear(moe.relu_sq_(ops.linear(h, w["w_up"])), w["w_down"])
        return moe.softmax_top_ffn(h, w["router"], w["router_b"], w["e_gu"], w["e_down"], int(mlp["router"]["top"]),
                                   w.get("s_gu"), w.get("s_down"))

    @torch.inference_mode()
    def forward(self, inp: torch.Tensor, meta: BatchMeta) -> torch.Tensor:
        if self.kv is None or self.state is None:
            raise RuntimeError("allocate_kv() and allocate_state() before forward()")
        eps = self.cfg.norm_eps
        sb = self._seq_batch(meta)
        x, h = sm.embedding_norm_f32(inp, self.embed["embed"], self.embed["norm"], eps, rounded=True)
        for i, (spec, w) in enumerate(zip(self.specs, self.layers)):
            mix = spec["mixer"]
            left, right = self._mixer(i, h, w, meta, sb)
            x, h = sm.post_norm_add(x, left, w["norm1"], eps, 1.0, o2=right,
                                    scales=(float(mix["left_scale"]), float(mix["right_scale"])), plain_next=True)
            if spec.get("mlp"):
                x, h = sm.post_norm_add(x, self._ff(h, w, spec["mlp"]), w["norm2"], eps, 1.0, plain_next=True)
            if self.taps is not None:
                self.taps.append(x.clone())
        if meta.logits_idx is not None:
            x = x.index_select(0, meta.logits_idx)
        hf = sm.rms_norm_f32(x, self.head["final_norm"], eps, self.dtype)
        return sm.softcap_f32(ops.linear(hf, self.head["lm_head"]), 0.0)
