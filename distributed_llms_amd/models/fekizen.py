"""Fekizen: a pre-norm layer-list decoder with learned positions on a scaled token embedding, a token
shift in front of every mixer, two linear-attention mixers with float32 matrix states, softmax attention
over a sliding window plus averaged blocks of older tokens, mixtures of SwiGLU experts, and a span of
layers that may run several times with the same weights.

``config.json`` keys (read by ``config._from_fekizen``): ``width``, ``vocab``, ``norm.eps``, ``embedding.scale``,
``max_positions``, optionally ``loop`` (``start``, ``stop``, ``times``), and ``layers``: per layer ``type``, ``mixer``, ``mlp``.

  type "lightning": ``heads``, ``dim``, ``vdim``, ``decay`` [heads].  q, k, v = silu(W h); per head
      S <- decay_h S + k v^T, o = S^T q; the concatenated heads pass ONE RMS norm (weight [heads vdim]), times
      sigmoid(W_g h), then the output projection.
  type "parallel": two mixers on the same input, each output RMS-normed over the model width with a weight
      of its own, then averaged.
      ``left`` -- attention: ``heads``, ``kv_heads``, ``dim`` (= ``vdim``: the values are the keys as projected,
      before their rotation), ``rot`` (``base``, ``dims``, optional YaRN ``scaling``; the first ``dims`` dimensions
      of every head turn, dimension i paired with i + dims / 2), ``scale``, ``softcap`` (scores become
      cap tanh(score / cap)), ``mask`` (``size``: sliding window; ``pool``: beside its window a query sees the mean
      key and mean value of every block of ``pool`` positions that lies wholly before the window), a
      learned sink per head in the softmax denominator.
      ``right`` -- gated linear attention: ``heads``, ``dim``, ``vdim``, ``tau``.  q = W_q h dim^-1/2, k, v; a decay
      per key channel a = sigmoid(W_a2 W_a1 h + b)^(1 / tau); S <- diag(a) S + k v^T, o = S^T q; every head's o
      passes an RMS norm (weight [vdim] shared by the heads), times silu(W_g h), then the output projection.
  mlp: None or {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top"}, "shared": {"ff"} | None}: SwiGLU
      experts, float32 router logits, the ``top`` largest, softmax over those only, an ungated shared expert.

One layer: x += mixer(shift(norm1(x))); x += ff(norm2(x)), norms with plain weights.  ``shift`` blends every
channel with the previous token's: h_t + (h_(t-1) - h_t) * w.  The stream starts as
norm(embed[token] * scale + pos[p]).  Layers [start, stop) run ``times`` times in a row; before pass t the
embedding output (t > 0) and the row t of ``loop.step`` are added to the stream; every pass has caches and
state of its own.

Checkpoint names: ``embed``, ``pos``, ``embed.norm``, ``loop.step``, ``final.norm``, ``head``; per layer ``l<i>.``:
``norm1``, ``norm2``, ``shift``; ``mix.q|k|v|g|o|norm`` (lightning); ``mix.left.q|k|o|sink|out``,
``mix.right.q|k|v|g|o|norm|a1|a2|a2.b|out`` (parallel); ``mlp.router``, ``mlp.e<j>.gate|up|down``,
``mlp.shared.gate|up|down``.  Linear weights are [out, in]; the rank of ``a1`` / ``a2`` is read from the tensors.

What a sequence keeps between steps, per layer RUN: the shift's previous row, the float32 matrix states
[heads, vdim, dim] (state slots), and for attention paged K / V and averaged K / V (one block table for
all, from the engine's BlockManager).  Stream, norms, angles, scores and softmax weights, router logits,
decays and states are float32 also when activations are bfloat16.
"""
from __future__ import annotations

from typing import Any, Dict, List, Optional, Tuple

import torch

from .. import ops
from ..config import ModelConfig
from ..ops import linattn as la
from ..ops import moe
from ..ops import seqmix as sm
from .hybrid import LayerListStage
from .stage import BatchMeta
from .weights import tensor_seed

DEFAULT_DECAY_RANK = 8       # synthetic weights only: a checkpoint's tensors give the rank


def layer_runs(cfg: ModelConfig) -> List[Tuple[int, Optional[int]]]:
    """[(layer index, number of the loop pass this run opens, or None)] in execution order."""
    n, lp = len(cfg.layers), cfg.loop
    if not lp:
        return [(i, None) for i in range(n)]
    runs: List[Tuple[int, Optional[int]]] = [(i, None) for i in range(lp["start"])]
    for t in range(lp["times"]):
        runs += [(i, t if i == lp["start"] else None) for i in range(lp["start"], lp["stop"])]
    return runs + [(i, None) for i in range(lp["stop"], n)]


def lin_spec(layer: Dict[str, Any]) -> la.LinAttnSpec:
    m = layer["mixer"] if layer["type"] == "lightning" else layer["mixer"]["right"]
    return la.LinAttnSpec(heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]))


def layer_shapes(width: int, layer: Dict[str, Any], rank: Optional[int] = None) -> Dict[str, tuple]:
    """Checkpoint tensor name (without the ``l<i>.`` prefix) -> shape (``rank``: of the decay's low-rank pair)."""
    sp = lin_spec(layer)
    qk, vv = sp.heads * sp.dim, sp.heads * sp.vdim
    s: Dict[str, tuple] = {"norm1": (width,), "shift": (width,)}
    if layer["type"] == "lightning":
        s.update({"mix.q": (qk, width), "mix.k": (qk, width), "mix.v": (vv, width), "mix.g": (vv, width),
                  "mix.o": (width, vv), "mix.norm": (vv,)})
    else:
        l = layer["mixer"]["left"]
        rank = rank or int(layer["mixer"]["right"].get("rank", DEFAULT_DECAY_RANK))
        s.update({"mix.left.q": (l["heads"] * l["dim"], width), "mix.left.k": (l["kv_heads"] * l["dim"], width),
                  "mix.left.sink": (l["heads"],), "mix.left.o": (width, l["heads"] * l["vdim"]),
                  "mix.left.out": (width,), "mix.right.out": (width,),
                  "mix.right.q": (qk, width), "mix.right.k": (qk, width), "mix.right.v": (vv, width),
                  "mix.right.g": (vv, width), "mix.right.o": (width, vv), "mix.right.norm": (sp.vdim,),
                  "mix.right.a1": (rank, width), "mix.right.a2": (qk, rank), "mix.right.a2.b": (qk,)})
    mlp = layer.get("mlp")
    if mlp:
        e, f = mlp["router"]["experts"], mlp["expert"]["ff"]
        s.update({"norm2": (width,), "mlp.router": (e, width)})
        for j in range(e):
            s.update({f"mlp.e{j}.gate": (f, width), f"mlp.e{j}.up": (f, width), f"mlp.e{j}.down": (width, f)})
        if mlp.get("shared"):
            fs = mlp["shared"]["ff"]
            s.update({"mlp.shared.gate": (fs, width), "mlp.shared.up": (fs, width), "mlp.shared.down": (width, fs)})
    return s


def model_shapes(cfg: ModelConfig, sd: Optional[Dict[str, torch.Tensor]] = None) -> Dict[str, tuple]:
    """Every checkpoint tensor's shape; with ``sd`` the decay ranks are read from its ``a1`` tensors."""
    w = cfg.hidden_size
    s = {"embed": (cfg.vocab_size, w), "pos": (cfg.max_position, w), "embed.norm": (w,), "final.norm": (w,),
         "head": (cfg.vocab_size, w)}
    if cfg.loop:
        s["loop.step"] = (cfg.loop["times"], w)
    for i, layer in enumerate(cfg.layers):
        a1 = None if sd is None else sd.get(f"l{i}.mix.right.a1")
        rank = int(a1.shape[0]) if a1 is not None and a1.dim() == 2 else None
        s.update({f"l{i}.{n}": shp for n, shp in layer_shapes(w, layer, rank).items()})
    return s


def synth_state_dict(cfg: ModelConfig, seed: int = 0, dtype=torch.float32) -> Dict[str, torch.Tensor]:
    """Seeded random weights under the checkpoint names (CPU): projections ~ N(0, 1 / fan_in), norm weights
    around one, shift weights in (0, 1), decay biases that keep the decays near one, the router wide
    enough that choices are not close calls, an embedding whose scaled rows have unit size."""
    sd = {}
    for name, shape in model_shapes(cfg).items():
        g = torch.Generator().manual_seed(tensor_seed(seed, 0, name))
        leaf = name.rsplit(".", 1)[-1]
        if leaf in ("norm1", "norm2", "norm", "out") or name in ("embed.norm", "final.norm"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif leaf == "shift":
            t = torch.rand(shape, generator=g)
        elif leaf == "sink":
            t = torch.randn(shape, generator=g)
        elif name.endswith("a2.b"):
            t = 2.0 + torch.randn(shape, generator=g)
        elif leaf == "router":
            t = 3.0 * torch.randn(shape, generator=g) / shape[-1] ** 0.5
        elif name == "embed":
            t = torch.randn(shape, generator=g) / cfg.embed_scale
        elif name in ("pos", "loop.step"):
            t = 0.3 * torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) / shape[-1] ** 0.5
        sd[name] = t.to(dtype)
    return sd


class FekizenStage(LayerListStage):
    """All layers of a Fekizen model on one device (see the module docstring)."""

    @staticmethod
    def layer_param_count(width: int, layer: Dict[str, Any]) -> int:
        return sum(int(torch.Size(s).numel()) for s in layer_shapes(width, layer).values())

    @staticmethod
    def kv_elements_per_token(cfg: ModelConfig) -> int:
        """K + V elements a token adds over all layer runs (the averaged caches' share of a block included)."""
        n = 0
        for i, _ in layer_runs(cfg):
            l = cfg.layers[i]
            if l["type"] == "parallel":
                m = l["mixer"]["left"]
                n += 2 * m["kv_heads"] * (m["dim"] + m["vdim"])
        return n

    def __init__(self, cfg: ModelConfig, layer_start: int = 0, layer_end: Optional[int] = None, device="cpu",
                 dtype=torch.bfloat16, units: Optional[tuple] = None, tp=None, unit_group: int = 2):
        super().__init__(cfg, layer_start, layer_end, device, dtype, units, tp, unit_group)
        self.runs = layer_runs(cfg)
        self.lspec = [lin_spec(l) for l in self.specs]
        self.rot: Dict[int, tuple] = {}          # parallel layer -> (freqs [dims / 2] f32, magnitude)
        self.decay: Dict[int, torch.Tensor] = {}  # lightning layer -> [heads] f32
        for i, (l, sp) in enumerate(zip(self.specs, self.lspec)):
            if sp.dim > la.MAX_KEY_DIM:
                raise ValueError(f"layer {i}: key size {sp.dim} > {la.MAX_KEY_DIM}")
            if l["type"] == "lightning":
                d = [float(v) for v in l["mixer"]["decay"]]
                if len(d) != sp.heads:
                    raise ValueError(f"layer {i}: one decay per head")
                self.decay[i] = torch.tensor(d, dtype=torch.float32, device=self.device)
            elif l["type"] == "parallel":
                m = l["mixer"]["left"]
                r = m["rot"]
                if m["heads"] % m["kv_heads"] or r["dims"] % 2 or r["dims"] > m["dim"] or m["vdim"] != m["dim"]:
                    raise ValueError(f"layer {i}: attention heads / kv_heads / rot.dims / vdim do not fit")
                f, mag = sm.yarn_frequencies(int(r["dims"]), float(r["base"]), r.get("scaling"))
                self.rot[i] = (f.to(self.device), mag)
            else:
                raise ValueError(f"layer {i}: unsupported type {l['type']!r}")
            mlp = l.get("mlp")
            if mlp and not 1 <= mlp["router"]["top"] <= min(16, mlp["router"]["experts"]):
                raise ValueError(f"layer {i}: router top does not fit")

    # ------------------------------------------------------------------ weights
    def load_hf_state(self, sd: Dict[str, torch.Tensor]) -> "FekizenStage":
        """From checkpoint-named tensors: ONE input projection per layer (lightning: q | k | v | g; parallel:
        attention q | k, then the gated linear attention's q | k | v | g | a1), gate | up stacked per expert;
        what feeds float32 math directly (router rows, sinks, decay biases) is float32."""
        want = model_shapes(self.cfg, sd)
        for n, shp in want.items():
            if n not in sd:
                raise KeyError(f"checkpoint lacks {n}")
            if tuple(sd[n].shape) != tuple(shp):
                raise ValueError(f"{n}: shape {tuple(sd[n].shape)}, config says {tuple(shp)}")
        cv = lambda t: t.to(device=self.device, dtype=self.dtype).contiguous()
        f32 = lambda t: t.to(device=self.device, dtype=torch.float32).contiguous()
        self.embed = {"embed": cv(sd["embed"]), "pos": cv(sd["pos"]), "norm": cv(sd["embed.norm"])}
        if self.cfg.loop:
            self.embed["loop_step"] = cv(sd["loop.step"])
        self.head = {"final_norm": cv(sd["final.norm"]), "lm_head": cv(sd["head"])}
        self.layers = []
        for i, layer in enumerate(self.specs):
            p = f"l{i}."
            w: Dict[str, Any] = {"norm1": cv(sd[p + "norm1"]), "shift": cv(sd[p + "shift"])}
            if layer["type"] == "lightning":
                w["w_in"] = cv(torch.cat([sd[p + "mix.q"], sd[p + "mix.k"], sd[p + "mix.v"], sd[p + "mix.g"]], 0))
                w["mix_norm"], w["wo"] = cv(sd[p + "mix.norm"]), cv(sd[p + "mix.o"])
            else:
                pl, pr = p + "mix.left.", p + "mix.right."
                w["w_in"] = cv(torch.cat([sd[pl + "q"], sd[pl + "k"], sd[pr + "q"], sd[pr + "k"], sd[pr + "v"], sd[pr + "g"],
                                          sd[pr + "a1"]], 0))
                w["rank"] = int(sd[pr + "a1"].shape[0])
                w["w_a2"], w["a2_b"] = cv(sd[pr + "a2"]), f32(sd[pr + "a2.b"])
                w["sinks"] = f32(sd[pl + "sink"])
                w["wo_left"], w["wo_right"] = cv(sd[pl + "o"]), cv(sd[pr + "o"])
                w["mix_norm"] = cv(sd[pr + "norm"])
                w["out_left"], w["out_right"] = cv(sd[pl + "out"]), cv(sd[pr + "out"])
            mlp = layer.get("mlp")
            if mlp:
                e = mlp["router"]["experts"]
                w["norm2"] = cv(sd[p + "norm2"])
                w["router"] = f32(sd[p + "mlp.router"])
                w["e_gu"] = cv(torch.stack([torch.cat([sd[p + f"mlp.e{j}.gate"], sd[p + f"mlp.e{j}.up"]], 0)
                                            for j in range(e)], 0))
                w["e_down"] = cv(torch.stack([sd[p + f"mlp.e{j}.down"] for j in range(e)], 0))
                if mlp.get("shared"):
                    w["s_gu"] = cv(torch.cat([sd[p + "mlp.shared.gate"], sd[p + "mlp.shared.up"]], 0))
                    w["s_down"] = cv(sd[p + "mlp.shared.down"])
            self.layers.append(w)
        return self

    def init_synthetic(self, seed: int = 0) -> "FekizenStage":
        return self.load_hf_state(synth_state_dict(self.cfg, seed))

    # ------------------------------------------------------------------ cache and state
    def _pool(self, i: int) -> int:
        return int((self.specs[i]["mixer"]["left"].get("mask") or {}).get("pool") or 0)

    def cache_shapes(self, block_size: int) -> Dict[Any, tuple]:
        """Per RUN of a parallel layer the attention's paged pair k [NB, G, BS, dim], v [NB, G, vdim, BS]
        (transposed inside a block) and, with pooling, the averaged pair in the same layouts with
        ``pooled_block_size`` entries per block."""
        out = {}
        for r, (i, _) in enumerate(self.runs):
            if self.specs[i]["type"] != "parallel":
                continue
            m = self.specs[i]["mixer"]["left"]
            out[(r, "kv")] = ((m["kv_heads"], block_size, m["dim"]), (m["kv_heads"], m["vdim"], block_size))
            if self._pool(i):
                pb = sm.pooled_block_size(block_size, self._pool(i))
                out[(r, "pool")] = ((m["kv_heads"], pb, m["dim"]), (m["kv_heads"], m["vdim"], pb))
        return out

    def allocate_state(self, num_slots: int):
        """State pools, one row per BlockManager state slot, per layer RUN: the shift's previous row
        [slots, W] (activation dtype) and the linear attention's matrices [slots, heads, vdim, dim] float32."""
        self.num_state_slots = num_slots
        w = self.cfg.hidden_size
        self.state = [{"shift": torch.zeros(num_slots, w, dtype=self.dtype, device=self.device),
                       "s": torch.zeros(num_slots, self.lspec[i].heads, self.lspec[i].vdim, self.lspec[i].dim,
                                        dtype=torch.float32, device=self.device)} for i, _ in self.runs]
        return self.state

    def state_bytes_per_slot(self) -> int:
        e = torch.empty((), dtype=self.dtype).element_size()
        return sum(e * self.cfg.hidden_size + 4 * self.lspec[i].heads * self.lspec[i].vdim * self.lspec[i].dim
                   for i, _ in self.runs)

    @property
    def graph_capturable(self) -> bool:
        """Whether a decode step runs without a host round trip.  Experts whose sizes the grouped
        kernels do not take (and float32) read the per-expert row counts on the host, which a HIP-graph
        capture cannot record: such a model decodes with eager launches."""
        for l in self.specs:
            mlp = l.get("mlp")
            if mlp and (self.dtype != torch.bfloat16 or self.cfg.hidden_size % 128 or mlp["expert"]["ff"] % 128):
                return False
        return True

    # ------------------------------------------------------------------ forward
    def _lightning(self, r: int, i: int, h: torch.Tensor, w, sb: sm.SeqBatch) -> torch.Tensor:
        sp = self.lspec[i]
        qk, vv = sp.heads * sp.dim, sp.heads * sp.vdim
        proj = ops.linear(h, w["w_in"])
        o = la.decay_scan(proj, 0, qk, 2 * qk, sp, self.state[r]["s"], sb, act="silu", decay=self.decay[i])
        y = la.gated_norm(o, proj, 2 * qk + vv, w["mix_norm"], self.cfg.norm_eps, groups=1, gate_act="sigmoid")
        return ops.linear(y, w["wo"])

    def _parallel(self, r: int, i: int, h: torch.Tensor, w, meta: BatchMeta, sb: sm.SeqBatch):
        """Both mixers on the same input: (attention output, gated linear attention output), each [T, W]."""
        m, mr, sp = self.specs[i]["mixer"]["left"], self.specs[i]["mixer"]["right"], self.lspec[i]
        hh, g, d = m["heads"], m["kv_heads"], m["dim"]
        qk, vv = sp.heads * sp.dim, sp.heads * sp.vdim
        c_right = (hh + g) * d                         # first column of the right mixer's q | k | v | g | a1
        kc, vc = self.kv.caches[(r, "kv")]
        freqs, mag = self.rot[i]
        proj = ops.linear(h, w["w_in"])
        q = sm.rownorm_rope(proj, 0, None, None, freqs, self.cfg.norm_eps, kc, vc, meta.slot_mapping, sb.positions, hh, g,
                            d, d, mag=mag, v_from_k=True)
        mask = m.get("mask") or {}
        pool, pooled = self._pool(i), None
        if pool:
            kp, vp = self.kv.caches[(r, "pool")]
            sm.pool_blocks(kc, vc, kp, vp, meta.block_tables, sb, pool)
            pooled = (kp, vp, pool)
        nd = meta.num_decode if meta.is_prefill else meta.num_seqs
        a = sm.window_attention(q, kc, vc, meta.block_tables, sb, int(mask.get("size") or (1 << 30)), float(m["scale"]),
                                num_decode=nd, sinks=w["sinks"], softcap=float(m.get("softcap") or 0.0), pooled=pooled,
                                max_ctx=meta.max_ctx_d if (meta.is_prefill and nd) else meta.max_ctx)
        a1 = c_right + 2 * qk + 2 * vv
        z = ops.linear(proj[:, a1:a1 + w["rank"]].contiguous(), w["w_a2"])
        o = la.decay_scan(proj, c_right, c_right + qk, c_right + 2 * qk, sp, self.state[r]["s"], sb,
                          q_scale=sp.dim ** -0.5, z=z, z_bias=w["a2_b"], tau=float(mr["tau"]))
        y = la.gated_norm(o, proj, c_right + 2 * qk + vv, w["mix_norm"], self.cfg.norm_eps, groups=sp.heads)
        return ops.linear(a.view(a.shape[0], -1), w["wo_left"]), ops.linear(y, w["wo_right"])

    def _ff(self, h: torch.Tensor, w, mlp) -> torch.Tensor:
        return moe.softmax_top_ffn(h, w["router"], None, w["e_gu"], w["e_down"], int(mlp["router"]["top"]),
                                   w.get("s_gu"), w.get("s_down"))

    @torch.inference_mode()
    def forward(self, inp: torch.Tensor, meta: BatchMeta) -> torch.Tensor:
        if self.kv is None or self.state is None:
            raise RuntimeError("allocate_kv() and allocate_state() before forward()")
        cfg = self.cfg
        eps = cfg.norm_eps
        sb = self._seq_batch(meta)
        x0, _ = sm.embedding_norm_f32(inp, self.embed["embed"], self.embed["norm"], eps, one_plus=False,
                                      scale=cfg.embed_scale, pos_table=self.embed["pos"], positions=sb.positions)
        x = x0.clone() if cfg.loop else x0
        h = None                        # norm1 of the coming layer, when the previous sublayer's close made it
        last = len(self.runs) - 1
        for r, (i, enters) in enumerate(self.runs):
            spec, w = self.specs[i], self.layers[i]
            if enters is not None:
                sm.stream_enter(x, x0 if enters > 0 else None, self.embed["loop_step"][enters])
                h = None
            if h is None:
                h = sm.rms_norm_f32(x, w["norm1"], eps, self.dtype, one_plus=False)
            h = sm.token_shift(h, w["shift"], self.state[r]["shift"], sb)
            mlp = spec.get("mlp")
            nxt = None                  # the next run's norm1, unless a loop entry changes the stream first
            if r < last and self.runs[r + 1][1] is None:
                nxt = self.layers[self.runs[r + 1][0]]["norm1"]
            after = w["norm2"] if mlp else nxt
            if spec["type"] == "lightning":
                x, h = sm.mix_add(x, self._lightning(r, i, h, w, sb), eps, w_next=after)
            else:
                left, right = self._parallel(r, i, h, w, meta, sb)
                x, h = sm.mix_add(x, left, eps, w_o=w["out_left"], o2=right, w_o2=w["out_right"], coef=0.5, w_next=after)
            if mlp:
                x, h = sm.mix_add(x, self._ff(h, w, mlp), eps, w_next=nxt)
            if self.taps is not None:
                self.taps.append(x.clone())
        if meta.logits_idx is not None:
            x = x.index_select(0, meta.logits_idx)
        hf = sm.rms_norm_f32(x, self.head["final_norm"], eps, self.dtype, one_plus=False)
        return sm.softcap_f32(ops.linear(hf, self.head["lm_head"]), 0.0)
