"""The Zebutar decoder (attention inside fixed chunks of positions beside a gated delta rule, sublayers
that read the stream unnormed and are normed on the way out, squared-ReLU and mixture-of-experts
feed-forwards) against the plain float64 oracle of tests/oracle_zebutar.py: every mechanism alone,
then the engine -- whole prompts, token-by-token decoding, prompt portions down to two tokens,
batches of unequal requests, blocks and state slots that are freed and used again, keys just inside
and just outside a chunk, far writes into the recurrent state, the first tokens, long decoding, and
greedy generation through the scheduler.  Each case runs on the CPU path in float32 and, marked gpu,
on the HIP kernels in float32 and bfloat16.
"""
import json

import numpy as np
import pytest
import torch

import oracle_zebutar as O
from distributed_llms_amd.config import EngineConfig, ModelConfig
from distributed_llms_amd.engine.llm_engine import LLMEngine
from distributed_llms_amd.engine.replay import TraceReplayer
from distributed_llms_amd.engine.sequence import SamplingParams
from distributed_llms_amd.models import make_stage
from distributed_llms_amd.ops import delta as dl
from distributed_llms_amd.ops import moe
from distributed_llms_amd.ops import seqmix as sm

gpu = pytest.mark.gpu
TARGETS = [pytest.param(("cpu", torch.float32), id="cpu-f32"),
           pytest.param(("cuda", torch.float32), id="gpu-f32", marks=gpu),
           pytest.param(("cuda", torch.bfloat16), id="gpu-bf16", marks=gpu)]


def _left(heads, kv_heads, dim, vdim, chunk, scale, rot_dims, base=10000.0):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
         "rot": {"base": base, "dims": rot_dims}}
    if chunk:
        m["mask"] = {"size": chunk}
    return m


def _right(heads, kv_heads, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def _layer(left, right, ls, rs, mlp):
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": ls, "right_scale": rs}, "mlp": mlp}


def _moe(experts, top, ff, shared):
    return {"kind": "moe", "expert": {"ff": ff}, "shared": {"ff": shared} if shared else None,
            "router": {"experts": experts, "top": top}}


def cfg_a():
    """Layers that differ from one another: chunks that are no power of two and no multiple of a cache
    block, rotated parts shorter than the head, key and value sizes that differ, grouped heads on both
    sides, convolutions of two to four taps, every feed-forward kind and a layer without one."""
    return {"architecture": "Zebutar", "vocab": 200, "width": 96, "norm": {"eps": 1e-6},
            "layers": [
                _layer(_left(4, 2, 24, 40, 24, 0.2, 16), _right(4, 2, 16, 24, 4), 0.9, 0.7, {"kind": "dense", "ff": 160}),
                _layer(_left(6, 3, 16, 8, 10, 0.3, 16, base=500.0), _right(2, 2, 40, 72, 2), 1.1, 0.6, _moe(6, 2, 48, 64)),
                _layer(_left(4, 4, 24, 40, 33, 0.2, 8), _right(4, 1, 16, 24, 3), 1.0, 1.3, None),
                _layer(_left(3, 1, 32, 16, 50, 0.15, 32), _right(3, 3, 24, 16, 3), 0.5, 1.5, _moe(5, 3, 40, 0)),
            ]}


def cfg_b():
    """Degenerate sizes: one head everywhere, one expert per token and every expert per token, a one-tap
    convolution (no tail), a chunk of one position (a token sees itself only), no mask at all (plain
    causal), no rotation, odd widths."""
    return {"architecture": "Zebutar", "vocab": 131, "width": 72, "norm": {"eps": 1e-5},
            "layers": [
                _layer(_left(1, 1, 12, 20, 1, 0.3, 12), _right(1, 1, 8, 8, 1), 1.0, 1.0, _moe(3, 1, 24, 0)),
                _layer(_left(2, 1, 10, 14, 0, 0.25, 4), _right(5, 1, 12, 10, 2), 0.7, 0.7, _moe(4, 4, 16, 8)),
                _layer(_left(5, 5, 8, 8, 7, 0.35, 0, base=100.0), _right(2, 2, 70, 6, 5), 1.2, 0.4,
                       {"kind": "dense", "ff": 40}),
            ]}


def cfg_c():
    """Sizes that the matrix-core attention kernels and the grouped expert kernels take."""
    return {"architecture": "Zebutar", "vocab": 160, "width": 128, "norm": {"eps": 1e-6},
            "layers": [
                _layer(_left(4, 2, 64, 64, 32, 0.12, 32), _right(6, 2, 32, 128, 4), 1.0, 1.0, _moe(8, 2, 128, 128)),
                _layer(_left(4, 1, 32, 128, 48, 0.2, 32), _right(2, 1, 128, 128, 3), 0.8, 1.2, {"kind": "dense", "ff": 256}),
            ]}


CONFIGS = {"a": cfg_a, "b": cfg_b, "c": cfg_c}


def _round(sd, dtype):
    """Weights as the engine will hold them (rounded to bf16 for a bf16 run), for engine and oracle."""
    return {k: torch.from_numpy(v).to(dtype).float() for k, v in sd.items()}


def _np(sd):
    return {k: v.double().numpy() for k, v in sd.items()}


def make_engine(cfg, sd, target, tmp_path, max_tokens=512, max_requests=4, block_size=32, graphs=False):
    device, dtype = target
    if device == "cuda" and not torch.cuda.is_available():
        pytest.skip("no GPU")
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    mcfg = ModelConfig.from_hf_config(cfg)
    stage = make_stage(mcfg, device=device, dtype=dtype).load_hf_state(sd)
    ecfg = EngineConfig(model=str(tmp_path), shard_dir=str(tmp_path), device=device,
                        dtype="float32" if dtype == torch.float32 else "bfloat16", max_batch=max_requests,
                        max_seq_len=max_tokens + 1, kv_block_size=block_size,
                        num_kv_blocks=-(-max_tokens // block_size) + max_requests + 1,
                        max_prefill_tokens=max_tokens, use_graphs=graphs, graph_batch_sizes=(1, 2, 4))
    return LLMEngine(ecfg, stage)


def row_errs(got, want):
    """Per position: rms of the difference (mean over the vocabulary taken off) over the rms of the oracle's logits."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / np.sqrt((want ** 2).mean())


def oracle(cfg, sd, tokens, taps=None):
    """(logits, decided): ``decided`` [T] marks the positions up to which no token's expert choice was a
    close call in any layer (a token's choice also reaches later positions, through both mixers)."""
    margins = []
    want = O.forward(cfg, _np(sd), np.array(tokens), taps, margins)
    ok = np.ones(len(tokens), dtype=bool)
    for m in margins:
        ok &= m > 0.1
    return want, np.logical_and.accumulate(ok)


def assert_close(got, want, target, what=""):
    """float32: every position within 2e-4, 2e-5 at the median (a wrong key, weight or state shows at
    1e-2 and more).  bfloat16, at the positions before a router's first close call (rounded activations
    may turn it the other way, which is no fault): 2.5e-2 at the median, 5e-2 at all but one position in
    fifteen (two at least), 0.3 at every one -- a norm on a sublayer's OUTPUT amplifies rounding where that output happens
    to be small, so single positions stand out in the plain bfloat16 forms as well."""
    want, decided = want
    e = row_errs(got, want)
    if target[1] == torch.float32:
        assert np.median(e) < 2e-5 and e.max() < 2e-4, (what, float(np.median(e)), float(e.max()), int(e.argmax()))
    elif decided.any():
        d = e[decided]
        over = int((d > 5e-2).sum())
        assert np.median(d) < 2.5e-2 and over <= max(2, len(d) // 15) and d.max() < 0.3, (
            what, int(decided.sum()), float(np.median(d)), over, float(d.max()))


def replay(engine, schedule, prompts):
    """schedule: steps, each a list of (request name, token count); returns name -> logits [len, V]."""
    rp = TraceReplayer(engine)
    at = {n: 0 for n in prompts}
    out = {n: [] for n in prompts}
    for step in schedule:
        entries, end = [], []
        for n, c in step:
            toks = prompts[n][at[n]:at[n] + c]
            entries.append((n, toks, list(range(len(toks)))))
            at[n] += c
            if at[n] == len(prompts[n]):
                end.append(n)
        logits = rp.step(entries, end).cpu().numpy()
        row = 0
        for n, toks, _ in entries:
            out[n].append(logits[row:row + len(toks)])
            row += len(toks)
    return {n: np.concatenate(v) for n, v in out.items() if v}


def prompts_for(cfg, lens, seed=1):
    rng = np.random.default_rng(seed)
    return {f"r{i}": rng.integers(0, cfg["vocab"], n).tolist() for i, n in enumerate(lens)}


def _sb(chunks, device, slots=None):
    """SeqBatch for chunks [(start position, length)]."""
    cu = np.concatenate([[0], np.cumsum([n for _, n in chunks])]).astype(np.int32)
    pos = np.concatenate([np.arange(s, s + n) for s, n in chunks]).astype(np.int32)
    seq = np.concatenate([np.full(n, i) for i, (_, n) in enumerate(chunks)]).astype(np.int32)
    t = lambda a: torch.from_numpy(a).to(device)
    st = None if slots is None else torch.tensor(slots, dtype=torch.int32, device=device)
    return sm.SeqBatch(t(cu), t(pos), t(seq), st, len(chunks), int(cu[-1]), max(n for _, n in chunks))


def _dev(target):
    if target[0] == "cuda" and not torch.cuda.is_available():
        pytest.skip("no GPU")
    return target


def _atol(dtype, f32=2e-5, bf16=3e-2):
    return f32 if dtype == torch.float32 else bf16


# ------------------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("shape", [(4, 2, 56, 48, 16, 24), (6, 3, 32, 32, 32, 64), (3, 1, 20, 20, 16, 10), (2, 2, 64, 128, 32, 33),
                                   (2, 1, 12, 12, 32, 1), (2, 1, 160, 192, 32, 40), (20, 1, 40, 40, 32, 70)])
def test_keys_at_the_edges_of_a_chunk(target, shape):
    """Attention inside chunks of C positions.  One key gets a score far above the rest: (a) the first key
    of the query's chunk, the query anywhere in the chunk up to its last position -- it owns the output;
    (b) the last key of the chunk before -- it must not show, although it is the query's neighbour.  As a
    prompt portion cut inside the chunk and for a decoded token, cache blocks scattered in the pool, the
    chunk's edges on both sides of block borders."""
    device, dtype = _dev(target)
    h, g, d, dv, bs, c = shape
    rng = np.random.default_rng(h * d + c)
    n = 150
    q = rng.standard_normal((n, h, d)).astype(np.float32) * 0.5
    k = rng.standard_normal((n, g, d)).astype(np.float32) * 0.5
    v = rng.standard_normal((n, g, dv)).astype(np.float32)
    table = list(rng.permutation(np.arange(1, 30))[:-(-n // bs)])
    T = lambda a: torch.from_numpy(a).to(dtype)
    bt = torch.tensor([table], dtype=torch.int32, device=device)
    tol = _atol(dtype)

    def paged(kk, vv):
        kc = torch.zeros(30, g, bs, d, dtype=dtype)
        vc = torch.zeros(30, g, dv, bs, dtype=dtype)
        for j in range(n):
            kc[table[j // bs], :, j % bs] = kk[j]
            vc[table[j // bs], :, :, j % bs] = vv[j]
        return kc.to(device), vc.to(device)

    def want_row(qq, kk, vv, p):
        lo = O.first_visible(p, c)
        out = np.zeros((h, dv))
        for a in range(h):
            s = kk[lo:p + 1, a // (h // g)].double().numpy() @ qq[p, a].double().numpy() * 0.3
            e = np.exp(s - s.max())
            out[a] = (e / e.sum()) @ vv[lo:p + 1, a // (h // g)].double().numpy()
        return out

    def both(qq, kc, vc, kk, vv, p, span):
        lo = max(0, p - span + 1)
        want = np.stack([want_row(qq, kk, vv, i) for i in range(lo, p + 1)])
        o = sm.window_attention(qq[lo:p + 1].contiguous().to(device), kc, vc, bt, _sb([(lo, p + 1 - lo)], device),
                                1 << 30, 0.3, num_decode=0, chunk=c)
        np.testing.assert_allclose(o.float().cpu().numpy(), want, rtol=tol, atol=tol)
        o = sm.window_attention(qq[p:p + 1].contiguous().to(device), kc, vc, bt, _sb([(p, 1)], device), 1 << 30, 0.3,
                                chunk=c)
        np.testing.assert_allclose(o.float().cpu().numpy(), want[-1:], rtol=tol, atol=tol)
        return want[-1]

    qq, kk, vv = T(q), T(k), T(v)
    kc, vc = paged(kk, vv)
    # the whole sequence in one portion
    o = sm.window_attention(qq.to(device), kc, vc, bt, _sb([(0, n)], device), 1 << 30, 0.3, num_decode=0, chunk=c)
    np.testing.assert_allclose(o.float().cpu().numpy(), np.stack([want_row(qq, kk, vv, i) for i in range(n)]), rtol=tol,
                               atol=tol)
    for start in sorted({c * (n // c - 1), c * (n // c // 2), c}):       # chunk starts late, in the middle, early
        if start <= 0 or start >= n:
            continue
        for p in sorted({start, min(start + 1, n - 1), min(start + c - 1, n - 1)}):
            for j, owns in ((start, True), (start - 1, False)):
                k2, q2 = k.copy(), q.copy()
                k2[j] = 0.0
                k2[j, :, 0] = 8.0
                q2[p, :, 0] = 16.0              # score 16 * 8 * 0.3 far above the rest
                q2b, k2b = T(q2), T(k2)
                kc2, vc2 = paged(k2b, vv)
                got = both(q2b, kc2, vc2, k2b, vv, p, span=min(5, c + 2))
                seen = np.abs(got[0] - vv[j, 0].double().numpy()).max() < 1e-3
                assert seen == owns or (c == 1 and p == j) or p - j >= c, (start, p, j)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("shape", [(4, 2, 24, 40, 16), (3, 1, 16, 8, 16), (2, 2, 64, 128, 32), (5, 5, 10, 6, 4), (2, 1, 12, 12, 0)])
def test_row_norm_and_half_split_rotation(target, shape):
    """The attention input stage: q and k are normed over ALL their heads at once (heads of very different
    size in the input, so a per-head norm would show), the first ``rot`` dimensions of a head turn in pairs
    (i, i + rot / 2) and the rest pass; positions far out; k and v land in scattered cache blocks."""
    device, dtype = _dev(target)
    h, g, d, dv, rot = shape
    rng = np.random.default_rng(d)
    pos = [0, 1, 2, 63, 64, 1000, 50000, 50001]
    t = len(pos)
    pad = 8                                     # columns before q in the fused projection
    x = rng.standard_normal((t, pad + h * d + g * d + g * dv)).astype(np.float32)
    x[:, pad:pad + d] *= 6.0                    # one loud q head
    x[:, pad + h * d:pad + h * d + d] *= 0.05   # one quiet k head
    qw, kw = 1 + 0.3 * rng.standard_normal(h * d), 1 + 0.3 * rng.standard_normal(g * d)
    T = lambda a: torch.from_numpy(np.asarray(a, dtype=np.float32)).to(dtype)
    xx, qwt, kwt = T(x), T(qw), T(kw)
    bs = 16
    slots = [5 * bs + 3, 2 * bs, 2 * bs + 1, 7 * bs + 15, 1 * bs, 3 * bs + 8, 4 * bs + 15, 6 * bs]
    kc = torch.zeros(9, g, bs, d, dtype=dtype, device=device)
    vc = torch.zeros(9, g, dv, bs, dtype=dtype, device=device)
    freqs = sm.rotary_frequencies(rot, 10000.0).to(device) if rot else torch.zeros(0, device=device)
    q = sm.rownorm_rope(xx.to(device), pad, qwt.to(device), kwt.to(device), freqs, 1e-6, kc, vc,
                        torch.tensor(slots, dtype=torch.int32, device=device),
                        torch.tensor(pos, dtype=torch.int32, device=device), h, g, d, dv)
    xd = xx.double().numpy()
    wq = np.zeros((t, h, d))
    wk = np.zeros((t, g, d))
    for i, p in enumerate(pos):
        qn = O.rms(xd[i, pad:pad + h * d], 1e-6) * qwt.double().numpy()
        kn = O.rms(xd[i, pad + h * d:pad + h * d + g * d], 1e-6) * kwt.double().numpy()
        wq[i] = O.rotate_half(qn.reshape(1, h, d), 10000.0, rot, first_pos=p)[0] if rot else qn.reshape(h, d)
        wk[i] = O.rotate_half(kn.reshape(1, g, d), 10000.0, rot, first_pos=p)[0] if rot else kn.reshape(g, d)
    # float32 angles at position 5e4 carry an error of 5e4 * 2^-24
    tol = _atol(dtype, 4e-3 * np.abs(wq).max(), 4e-2 * np.abs(wq).max())
    np.testing.assert_allclose(q.float().cpu().numpy(), wq, atol=tol)
    np.testing.assert_allclose(q.float().cpu().numpy()[:5], wq[:5], atol=_atol(dtype, 2e-5, 4e-2) * np.abs(wq).max())
    for i, s in enumerate(slots):
        np.testing.assert_allclose(kc[s // bs, :, s % bs].float().cpu().numpy(), wk[i], atol=tol)
        np.testing.assert_array_equal(vc[s // bs, :, :, s % bs].float().cpu().numpy(),
                                      xx[i, pad + h * d + g * d:].float().numpy().reshape(g, dv))
    # a norm per head would give the loud head the same size as the others
    assert np.abs(wq[:, 0]).mean() > 3 * np.abs(wq[:, 1:]).mean() if h > 1 else True


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("taps,c", [(4, 40), (2, 17), (3, 64), (1, 8), (5, 24)])
def test_short_convolution_with_silu_across_portions(target, taps, c):
    """Causal convolution + silu on a column slice of a wider projection: portions of one to many tokens
    (shorter than the tail, too) give the whole sequence's result; a sequence in a slot another one used
    before starts from zeros."""
    device, dtype = _dev(target)
    rng = np.random.default_rng(taps)
    n, off = 37, 8
    x = torch.from_numpy(rng.standard_normal((n, off + c + 8)).astype(np.float32)).to(dtype)
    w = torch.from_numpy((rng.standard_normal((c, taps)) / taps ** 0.5).astype(np.float32)).to(dtype)
    want = O.silu(O.short_conv(x[:, off:off + c].double().numpy(), w.double().numpy()))
    state = torch.full((3, taps - 1, c), 7.0, dtype=dtype, device=device)         # junk of an earlier owner
    wt = w.t().contiguous().to(device)
    xd = x.to(device)
    got, at = [], 0
    for size in [1, 2, 1, 5, 3, 1, 1, 9, 2, 12]:
        y = sm.causal_conv(xd[at:at + size, off:off + c], wt, None, state, _sb([(at, size)], device, slots=[2]),
                           out_dtype=torch.float32, act="silu")
        got.append(y.cpu().numpy())
        at += size
    assert at == n
    np.testing.assert_allclose(np.concatenate(got), want, atol=_atol(dtype, 2e-5, 1e-5), rtol=_atol(dtype, 2e-5, 1e-5))
    # two sequences in one step: a new one in a used slot beside the continuation of the first
    more = torch.from_numpy(rng.standard_normal((4, off + c + 8)).astype(np.float32)).to(dtype)
    want_more = O.silu(O.short_conv(torch.cat([x, more], 0)[:, off:off + c].double().numpy(), w.double().numpy()))[n:]
    y = sm.causal_conv(torch.cat([xd[:6], more.to(device)], 0)[:, off:off + c], wt, None, state,
                       _sb([(0, 6), (n, 4)], device, slots=[1, 2]), out_dtype=torch.float32, act="silu")
    np.testing.assert_allclose(y.cpu().numpy(), np.concatenate([want[:6], want_more]), atol=_atol(dtype, 2e-5, 1e-5),
                               rtol=_atol(dtype, 2e-5, 1e-5))


def _delta_inputs(sp, n, rng, dtype):
    """Random projection rows q | k | v | gate | b | a behind 8 columns of something else."""
    x = rng.standard_normal((n, 8 + sp.in_width)).astype(np.float32)
    return torch.from_numpy(x).to(dtype)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("sizes", [(4, 2, 16, 24, 4), (2, 2, 40, 72, 2), (3, 1, 128, 128, 3), (1, 1, 8, 8, 1), (2, 1, 200, 20, 2),
                                   (5, 5, 33, 65, 3)])
def test_gated_delta_rule_through_state_slots(target, sizes):
    """The delta rule mixer between its projections: whole sequences, portions of one to many tokens and
    token-by-token decoding give the oracle's outputs (state and convolution tail carried in the slot);
    two sequences side by side do not mix; a new sequence in a used slot starts from zero."""
    device, dtype = _dev(target)
    hh, g, d, dv, taps = sizes
    sp = dl.DeltaSpec(hh, g, d, dv, taps)
    rng = np.random.default_rng(d + dv)
    n = 70
    eps = 1e-6
    x = _delta_inputs(sp, n, rng, dtype)
    c = sp.conv_width
    wq, wk, wv = (torch.from_numpy((rng.standard_normal((m, taps)) / taps ** 0.5).astype(np.float32)).to(dtype)
                  for m in (g * d, g * d, hh * dv))
    a_log = torch.from_numpy(rng.uniform(-4, 0.5, hh).astype(np.float32))
    dt_bias = torch.from_numpy(rng.standard_normal(hh).astype(np.float32))
    norm = torch.from_numpy((1 + 0.2 * rng.standard_normal(dv)).astype(np.float32)).to(dtype)

    def want_for(xx):
        xd = xx[:, 8:].double().numpy()
        t = xd.shape[0]
        q = O.silu(O.short_conv(xd[:, :g * d], wq.double().numpy())).reshape(t, g, d)
        k = O.silu(O.short_conv(xd[:, g * d:2 * g * d], wk.double().numpy())).reshape(t, g, d)
        v = O.silu(O.short_conv(xd[:, 2 * g * d:c], wv.double().numpy())).reshape(t, hh, dv)
        q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * d ** -0.5
        k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
        gate = O.silu(xd[:, c:c + hh * dv]).reshape(t, hh, dv)
        beta = O.sigmoid(xd[:, c + hh * dv:c + hh * dv + hh])
        dec = np.exp(-np.exp(a_log.double().numpy()) * O.softplus(xd[:, c + hh * dv + hh:] + dt_bias.double().numpy()))
        out = np.zeros((t, hh, dv))
        for a in range(hh):
            o = O.delta_rule(q[:, a // (hh // g)], k[:, a // (hh // g)], v[:, a], beta[:, a], dec[:, a])
            out[:, a] = O.rms(o, eps) * norm.double().numpy() * gate[:, a]
        return out.reshape(t, hh * dv)

    w = {"conv_w": torch.cat([wq, wk, wv], 0).t().contiguous().to(device), "a_log": a_log.to(device),
         "dt_bias": dt_bias.to(device), "norm": norm.to(device)}
    conv_state = torch.full((4, taps - 1, c), 3.0, dtype=dtype, device=device)     # junk of earlier owners
    state = torch.full((4, hh, d, dv), 5.0, dtype=torch.float32, device=device)
    want = want_for(x)
    xd = x.to(device)
    tol = _atol(dtype, 3e-5, 3e-2) * max(1.0, np.abs(want).max())
    run = lambda rows, chunks, slots: dl.gated_delta_mixer(rows, 8, w, sp, conv_state, state, _sb(chunks, device, slots),
                                                           eps).float().cpu().numpy()
    np.testing.assert_allclose(run(xd, [(0, n)], [1]), want, atol=tol)
    got, at = [], 0
    for size in [2, 1, 1, 9, 3, 17, 1, 2, 30, 1, 1, 2]:
        got.append(run(xd[at:at + size], [(at, size)], [2]))
        at += size
    assert at == n
    np.testing.assert_allclose(np.concatenate(got), want, atol=tol)
    # another sequence beside the continuation of the first, in a slot that was used: rows do not mix
    x2 = _delta_inputs(sp, 12, rng, dtype)
    state[3] = state[2]                       # the first sequence's state after n tokens, moved to slot 3
    conv_state[3] = conv_state[2]
    x3 = _delta_inputs(sp, 5, rng, dtype)
    both = run(torch.cat([x2, x3], 0).to(device), [(0, 12), (n, 5)], [2, 3])
    np.testing.assert_allclose(both[:12], want_for(x2), atol=tol)
    np.testing.assert_allclose(both[12:], want_for(torch.cat([x, x3], 0))[n:], atol=tol)


@pytest.mark.parametrize("target", TARGETS)
def test_a_write_far_back_is_read_from_the_state(target):
    """With decays next to one, what the first token wrote is read hundreds of tokens later by a query that
    matches its key (and nothing else): a state that is dropped, zeroed or decayed wrongly between portions
    or steps shows.  Inputs are built so that the unit keys are orthogonal one-hot directions."""
    device, dtype = _dev(target)
    d, dv, n = 16, 32, 400
    sp = dl.DeltaSpec(1, 1, d, dv, 1)
    rng = np.random.default_rng(0)
    u = np.zeros((n, sp.conv_width), dtype=np.float32)
    u[:, d + 1 + np.arange(n) % (d - 1)] = 0.0
    for i in range(n):
        u[i, d + 1 + i % (d - 1)] = 1.0           # keys: directions 1 .. d - 1 in turn
        u[i, 1 + i % (d - 1)] = 1.0               # queries read the same direction
    u[0, d:2 * d] = 0.0
    u[0, d] = 1.0                                  # the first token alone writes direction 0
    u[0, :d] = 0.0
    u[0, 0] = 1.0
    u[n - 1, :d] = 0.0
    u[n - 1, 0] = 1.0                              # the last token reads it
    v = rng.standard_normal((n, dv)).astype(np.float32)
    u[:, 2 * d:] = v
    ab = np.zeros((n, 2), dtype=np.float32)
    ab[:, 0] = 20.0                                # beta = 1
    ab[:, 1] = -20.0                               # softplus ~ 2e-9: decay ~ 1
    a_log, dt_bias = torch.zeros(1, device=device), torch.zeros(1, device=device)
    state = torch.full((2, 1, d, dv), 9.0, dtype=torch.float32, device=device)
    outs, at = [], 0
    for size in [50, 1, 1, 100, 2, 200, 45, 1]:
        uu = torch.from_numpy(u[at:at + size]).to(device)
        sb = _sb([(at, size)], device, slots=[1])
        bd = dl.unit_qk_gates(uu, torch.from_numpy(ab[at:at + size]).to(device), 0, a_log, dt_bias, sp)
        outs.append(dl.delta_scan(uu, bd, state, sb, sp).cpu().numpy())
        at += size
    assert at == n
    o = np.concatenate(outs)[:, 0]
    np.testing.assert_allclose(o[n - 1], v[0] * d ** -0.5, atol=1e-4)
    np.testing.assert_allclose(o[0], v[0] * d ** -0.5, atol=1e-4)
    q64 = u[:, :d].astype(np.float64)
    k64 = u[:, d:2 * d].astype(np.float64)
    q64 = q64 / np.sqrt((q64 ** 2).sum(-1, keepdims=True) + 1e-6) * d ** -0.5
    k64 = k64 / np.sqrt((k64 ** 2).sum(-1, keepdims=True) + 1e-6)
    dec = np.exp(-O.softplus(ab[:, 1].astype(np.float64)))
    want = O.delta_rule(q64, k64, v.astype(np.float64), O.sigmoid(ab[:, 0].astype(np.float64)), dec)
    np.testing.assert_allclose(o, want, atol=1e-4)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("width", [96, 72, 256, 33])
def test_output_normed_sublayers_on_the_stream(target, width):
    """Embedding + norm opens the stream and gives the first sublayer its unnormed input; the close of a
    sublayer adds the normed weighted sum of two mixer outputs and hands the next sublayer the stream."""
    device, dtype = _dev(target)
    rng = np.random.default_rng(width)
    t, vocab, eps = 9, 50, 1e-6
    T = lambda a: torch.from_numpy(np.asarray(a, dtype=np.float32)).to(dtype).to(device)
    table, w0, w1 = T(rng.standard_normal((vocab, width))), T(0.2 * rng.standard_normal(width)), T(
        0.2 * rng.standard_normal(width))
    ids = torch.tensor(rng.integers(0, vocab, t), dtype=torch.int32, device=device)
    x, h = sm.embedding_norm_f32(ids, table, w0, eps, rounded=True)
    want = O.norm_one_plus(table.double().cpu().numpy()[ids.cpu().numpy()], w0.double().cpu().numpy(), eps)
    np.testing.assert_allclose(x.cpu().numpy(), want, atol=2e-5)
    assert x.dtype == torch.float32 and h.dtype == dtype
    np.testing.assert_allclose(h.float().cpu().numpy(), want, atol=_atol(dtype, 2e-5, 3e-2))
    a, b = T(rng.standard_normal((t, width))), T(3 * rng.standard_normal((t, width)))
    x0 = x.clone()
    x2, h2 = sm.post_norm_add(x, a, w1, eps, 1.0, o2=b, scales=(1.3, 0.45), plain_next=True)
    want2 = x0.double().cpu().numpy() + O.norm_one_plus(
        1.3 * a.double().cpu().numpy() + 0.45 * b.double().cpu().numpy(), w1.double().cpu().numpy(), eps)
    np.testing.assert_allclose(x2.cpu().numpy(), want2, atol=3e-5)
    np.testing.assert_allclose(h2.float().cpu().numpy(), want2, atol=_atol(dtype, 3e-5, 4e-2))
    x3, h3 = sm.post_norm_add(x2, a, w1, eps, 1.0, plain_next=True)
    want3 = want2 + O.norm_one_plus(a.double().cpu().numpy(), w1.double().cpu().numpy(), eps)
    np.testing.assert_allclose(x3.cpu().numpy(), want3, atol=4e-5)
    np.testing.assert_allclose(h3.float().cpu().numpy(), want3, atol=_atol(dtype, 4e-5, 4e-2))


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("case", [(8, 3, 48, 40, 96, 70), (6, 2, 32, 0, 72, 33), (3, 1, 24, 0, 40, 5), (4, 4, 16, 8, 72, 130),
                                  (8, 2, 128, 128, 128, 300), (8, 2, 256, 128, 256, 300), (5, 3, 40, 0, 96, 1)])
def test_router_and_expert_feed_forward(target, case):
    """Biased float32 router, the ``top`` largest logits, softmax over those only (a bias that decides the
    choice; all experts chosen; one), SwiGLU experts, an ungated shared expert; few tokens and many (the
    fused and the library router product, every expert kernel path); and the squared-ReLU feed-forward."""
    device, dtype = _dev(target)
    e, top, f, fs, width, t = case
    rng = np.random.default_rng(e * t)
    mlp = _moe(e, top, f, fs)
    cfg = {"vocab": 4, "width": width, "norm": {"eps": 1e-6}, "layers": [
        _layer(_left(1, 1, 8, 8, 4, 0.3, 8), _right(1, 1, 8, 8, 2), 1.0, 1.0, mlp)]}
    sd = {k[len("l0.mlp."):]: torch.from_numpy(v).to(dtype).float() for k, v in O.make_weights(cfg, seed=e).items()
          if k.startswith("l0.mlp.")}
    sd["router.b"][0] += 8.0                        # a bias large enough to pull its expert into most choices
    x = torch.from_numpy(rng.standard_normal((t, width)).astype(np.float32)).to(dtype)
    margins = []
    want = O.moe_ff(x.double().numpy(), _np(sd), mlp, margins)
    cv = lambda a: a.to(device=device, dtype=dtype).contiguous()
    gu = cv(torch.stack([torch.cat([sd[f"e{j}.gate"], sd[f"e{j}.up"]], 0) for j in range(e)]))
    down = cv(torch.stack([sd[f"e{j}.down"] for j in range(e)]))
    sgu = cv(torch.cat([sd["shared.gate"], sd["shared.up"]], 0)) if fs else None
    sdown = cv(sd["shared.down"]) if fs else None
    got = moe.softmax_top_ffn(x.to(device), sd["router"].to(device), sd["router.b"].to(device), gu, down, top, sgu, sdown)
    ok = margins[0] > (1e-4 if dtype == torch.float32 else 0.05)
    assert ok.sum() >= 0.7 * t
    np.testing.assert_allclose(got.float().cpu().numpy()[ok], want[ok], atol=_atol(dtype, 5e-5, 5e-2) * max(1, np.abs(want).max()))
    # choices and weights themselves
    z = x.double().numpy() @ sd["router"].double().numpy().T + sd["router.b"].double().numpy()
    tw, ids = moe.route_softmax_top(torch.from_numpy(z), top)
    for i in np.nonzero(ok)[0][:20]:
        idx, p = O.route_top(z[i], top)
        assert list(ids[i].numpy()) == list(idx)
        np.testing.assert_allclose(tw[i].numpy(), p, atol=1e-6)
    assert (ids == 0).any(-1).float().mean() > 0.7 or top == e
    # squared ReLU
    up, dn = cv(torch.from_numpy(rng.standard_normal((f, width)).astype(np.float32) / width ** 0.5)), cv(
        torch.from_numpy(rng.standard_normal((width, f)).astype(np.float32) / f ** 0.5))
    from distributed_llms_amd import ops
    y = ops.linear(moe.relu_sq_(ops.linear(x.to(device), up)), dn)
    wantd = O.dense_ff(x.double().numpy(), {"up": up.double().cpu().numpy(), "down": dn.double().cpu().numpy()})
    np.testing.assert_allclose(y.float().cpu().numpy(), wantd, atol=_atol(dtype, 5e-5, 5e-2) * max(1, np.abs(wantd).max()))


# ------------------------------------------------------------------------------ the engine
@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_whole_prompts_and_layers(target, name, tmp_path):
    cfg = CONFIGS[name]()
    sd = _round(O.make_weights(cfg, seed=3), target[1])
    eng = make_engine(cfg, sd, target, tmp_path)
    prompts = prompts_for(cfg, [1, 2, 45, 130])
    eng.stage.taps = []
    got = replay(eng, [[(n, len(p))] for n, p in prompts.items()], prompts)
    taps = eng.stage.taps
    eng.stage.taps = None
    runs = len(cfg["layers"])
    for i, (n, p) in enumerate(prompts.items()):
        layers = []
        want = oracle(cfg, sd, p, layers)
        assert_close(got[n], want, target, n)
        if target[1] == torch.float32:            # the residual stream after every layer
            mine = torch.stack(taps[i * runs:(i + 1) * runs]).cpu().numpy()
            np.testing.assert_allclose(mine, np.stack(layers), rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_decode_and_portions_match_the_whole(target, name, tmp_path):
    """Token-by-token decoding after a prompt (90 steps, over several block and chunk borders), portions of
    changing sizes down to two tokens and one, cut inside blocks and chunks, and decoding from the very
    first token."""
    cfg = CONFIGS[name]()
    sd = _round(O.make_weights(cfg, seed=4), target[1])
    eng = make_engine(cfg, sd, target, tmp_path)
    p = prompts_for(cfg, [150], seed=7)
    want = oracle(cfg, sd, p["r0"])
    got = replay(eng, [[("r0", 60)]] + [[("r0", 1)]] * 90, p)
    assert_close(got["r0"], want, target, "decode")
    sizes = [2, 3, 1, 31, 2, 33, 5, 64, 2, 7]
    assert sum(sizes) == 150
    got = replay(eng, [[("r0", s)] for s in sizes], p)
    assert_close(got["r0"], want, target, "portions")
    got = replay(eng, [[("r0", 1)]] * 40, {"r0": p["r0"][:40]})
    assert_close(got["r0"], (want[0][:40], want[1][:40]), target, "from the first token")


@pytest.mark.parametrize("target", TARGETS)
def test_mixed_batches_and_reused_blocks_and_slots(target, tmp_path):
    """Up to four unequal requests per step, portions beside single tokens; finished requests give their
    blocks and their state slot to new ones (a pool sized for the live tokens only, four slots for seven
    requests).  Every request matches its own whole-sequence oracle: the batch, the pool and the slots do
    not show."""
    cfg = cfg_a()
    sd = _round(O.make_weights(cfg, seed=5), target[1])
    eng = make_engine(cfg, sd, target, tmp_path, max_tokens=288, max_requests=4)
    lens = [70, 9, 33, 64, 20, 50, 3]
    prompts = prompts_for(cfg, lens, seed=9)
    names = list(prompts)
    at = {n: 0 for n in names}
    waiting, live, schedule = list(names), [], []
    rng = np.random.default_rng(0)
    while waiting or live:
        while waiting and len(live) < 4:
            live.append(waiting.pop(0))
        step = []
        for n in list(live):
            left = len(prompts[n]) - at[n]
            c = min(left, int(rng.choice([1, 1, 2, 3, 17, 32])))
            if rng.random() < 0.15 and len(live) > 1:
                continue                                # left out of this step, goes on later
            step.append((n, c))
            at[n] += c
            if at[n] == len(prompts[n]):
                live.remove(n)
        if step:
            schedule.append(step)
    got = replay(eng, schedule, prompts)
    assert eng.bm.num_free() == eng.bm.num_blocks - 1            # all given back (block 0 is the scratch block)
    for n in names:
        assert_close(got[n], oracle(cfg, sd, prompts[n]), target, n)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("name,graphs", [("a", False), ("c", True)])
def test_greedy_generation_through_the_scheduler(target, name, graphs, tmp_path):
    """LLMEngine.generate (scheduler, continuous batching, sampler; for the model whose experts the
    grouped kernels take, decode steps replayed from HIP graphs) on three prompts at once: every
    generated token is the argmax of the oracle's logits for the sequence so far (where the oracle's
    top two are not within rounding of each other)."""
    cfg = CONFIGS[name]()
    sd = _round(O.make_weights(cfg, seed=6), target[1])
    eng = make_engine(cfg, sd, target, tmp_path, graphs=graphs)
    prompts = list(prompts_for(cfg, [5, 40, 17], seed=11).values())
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=24, ignore_eos=True))
    margin = 1e-3 if target[1] == torch.float32 else 0.3
    checked = 0
    for p, o in zip(prompts, outs):
        assert len(o) == 24
        logits = O.forward(cfg, _np(sd), np.array(p + o))
        for i, tok in enumerate(o):
            row = logits[len(p) + i - 1]
            top = np.sort(row)[-2:]
            if top[1] - top[0] > margin:
                checked += 1
                assert tok == int(row.argmax()), (i, tok, int(row.argmax()))
    assert checked > (36 if target[1] == torch.float32 else 12)


def random_config(seed):
    """A model whose every size is drawn: widths, head counts and groupings, key / value sizes, rotated parts,
    chunk lengths, taps, feed-forward kinds and their sizes, scales, layer count and order."""
    rng = np.random.default_rng(1000 + seed)
    pick = lambda xs: xs[int(rng.integers(len(xs)))]
    width = pick([64, 72, 96, 128, 160, 192, 256])
    layers = []
    for _ in range(int(rng.integers(2, 5))):
        g = pick([1, 2, 3, 4])
        h = g * pick([1, 2, 3, 4])
        d = pick([8, 16, 24, 32, 40, 64, 80, 128])
        left = _left(h, g, d, pick([8, 16, 24, 48, 64, 72, 128]), pick([0, 1, 2, 5, 16, 31, 32, 64, 100]),
                     float(rng.uniform(0.05, 0.4)), pick([r for r in (0, 2, 4, 8, 16, 32, 64, 128) if r <= d]),
                     base=float(pick([100.0, 10000.0, 50000.0, 1e6])))
        gr = pick([1, 2, 3])
        right = _right(gr * pick([1, 2, 4]), gr, pick([8, 16, 24, 32, 48, 64, 96, 128]), pick([8, 16, 40, 64, 128, 136]),
                       pick([1, 2, 3, 4, 5]))
        kind = pick(["dense", "moe", "moe", None])
        if kind == "dense":
            mlp = {"kind": "dense", "ff": pick([40, 64, 128, 200, 256])}
        elif kind == "moe":
            e = pick([2, 3, 4, 8, 12, 20])
            mlp = _moe(e, pick([t for t in (1, 2, 3, 4, 6) if t <= e]), pick([16, 40, 64, 128]), pick([0, 24, 64, 128]))
        else:
            mlp = None
        layers.append(_layer(left, right, float(rng.uniform(0.3, 1.6)), float(rng.uniform(0.3, 1.6)), mlp))
    return {"architecture": "Zebutar", "vocab": pick([97, 128, 200, 333]), "width": width,
            "norm": {"eps": pick([1e-6, 1e-5, 1e-4])}, "layers": layers}


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("seed", range(8))
def test_drawn_models_on_a_mixed_schedule(target, seed, tmp_path):
    """Models of drawn sizes: three unequal requests, portions of changing size beside single tokens, a
    fourth request that takes over freed blocks and a freed slot; each equals its whole-sequence oracle."""
    cfg = random_config(seed)
    sd = _round(O.make_weights(cfg, seed=seed), target[1])
    eng = make_engine(cfg, sd, target, tmp_path, max_tokens=320, max_requests=3)
    prompts = prompts_for(cfg, [75, 18, 110, 40], seed=seed)
    schedule = [[("r0", 33), ("r1", 2)], [("r0", 1), ("r1", 16), ("r2", 64)], [("r0", 1), ("r2", 3)], [("r0", 30), ("r2", 1)],
                [("r2", 2), ("r0", 1)], [("r0", 9), ("r2", 39), ("r3", 7)], [("r3", 1), ("r2", 1)], [("r3", 32)]]
    got = replay(eng, schedule, prompts)
    assert eng.bm.num_free() == eng.bm.num_blocks - 1
    for n, p in prompts.items():
        assert_close(got[n], oracle(cfg, sd, p), target, (seed, n))


def test_config_round_trip_and_registry(tmp_path):
    from distributed_llms_amd.config import get_model_config
    from distributed_llms_amd.models.zebutar import ZebutarStage, model_shapes
    cfg = cfg_a()
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    m = get_model_config(str(tmp_path))
    assert m.arch == "zebutar" and m.num_layers == 4 and m.hidden_size == 96
    assert m.needs_seq_index and m.needs_state_slots
    back = ModelConfig.from_hf_config(m.to_hf_config())
    assert back.layers == m.layers and back.norm_eps == m.norm_eps
    st = make_stage(m)
    assert isinstance(st, ZebutarStage) and st.num_layers == 4
    assert {k: tuple(v.shape) for k, v in O.make_weights(cfg).items()} == model_shapes(m)
    assert st.kv_bytes_per_block(32) == 2 * 32 * sum(
        l["mixer"]["left"]["kv_heads"] * (l["mixer"]["left"]["dim"] + l["mixer"]["left"]["vdim"]) for l in cfg["layers"])
    for bad in ({"type": "attention"}, {"mlp": {"kind": "glu", "ff": 8}}):
        c = cfg_a()
        c["layers"][0].update(bad)
        with pytest.raises(ValueError):
            ModelConfig.from_hf_config(c)
    c = cfg_a()
    c["layers"][0]["mixer"]["left"]["rot"]["dims"] = 64
    with pytest.raises(ValueError):
        make_stage(ModelConfig.from_hf_config(c))
    assert get_model_config("tiny-zebutar").arch == "zebutar"
    make_stage(get_model_config("tiny-zebutar")).init_synthetic(0)


@pytest.mark.parametrize("target", [t for t in TARGETS if "gpu" in t.id])
def test_decode_graphs_replay_like_eager_steps(target, tmp_path):
    """Decode steps replayed from captured HIP graphs (several replays, eager prompt steps and
    synchronisations between them) give the logits of eager decode steps, recurrent state included."""
    if target[1] != torch.bfloat16:
        pytest.skip("the float32 expert path reads row counts on the host: it decodes eagerly")
    cfg = cfg_c()
    sd = _round(O.make_weights(cfg, seed=8), target[1])
    p = prompts_for(cfg, [40, 23], seed=3)
    sched = [[("r0", 30), ("r1", 13)]] + [[("r0", 1), ("r1", 1)]] * 10
    eager = replay(make_engine(cfg, sd, target, tmp_path, graphs=False), sched, p)
    eng = make_engine(cfg, sd, target, tmp_path, graphs=True)
    assert eng.runner.graphs is not None
    graphed = replay(eng, sched, p)
    for n in p:
        np.testing.assert_allclose(graphed[n], eager[n], rtol=1e-3, atol=1e-3)


def test_trace_run_program_loads_a_model_folder(tmp_path):
    """bin/trace_run on a folder with config.json + model.safetensors (bfloat16): the registry picks the
    stage by the config, the checkpoint loader reads the tensors, steps with portions beside single tokens
    answer with the wanted logits (CPU path, float32)."""
    import os
    import subprocess
    import sys
    from safetensors.torch import save_file
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = cfg_a()
    sd = {k: torch.from_numpy(v).to(torch.bfloat16) for k, v in O.make_weights(cfg, seed=21).items()}
    model = tmp_path / "model"
    model.mkdir()
    (model / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in sd.items()}, str(model / "model.safetensors"))
    rng = np.random.default_rng(3)
    toks = {"a": rng.integers(0, cfg["vocab"], 50).tolist(), "b": rng.integers(0, cfg["vocab"], 21).tolist()}
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": toks["a"][:30], "want": [0, 29]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": toks["a"][30:31], "want": [0]},
                                {"id": "b", "tokens": toks["b"][:20], "want": [19]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": toks["b"][20:], "want": []}], "end": ["b"]},
        {"step": 3, "entries": [{"id": "a", "tokens": toks["a"][31:], "want": [18]}], "end": ["a"]},
    ]
    out = tmp_path / "out"
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(model), "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "128", "--device", "cpu"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    assert not (out / "2.f32").exists()                       # nothing wanted in step 2
    f64 = {k: v.double().numpy() for k, v in sd.items()}
    ref = {n: O.forward(cfg, f64, t) for n, t in toks.items()}
    got = {i: np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, cfg["vocab"]) for i in (0, 1, 3)}
    assert row_errs(got[0], ref["a"][[0, 29]]).max() < 1e-4
    assert row_errs(got[1], np.stack([ref["a"][30], ref["b"][19]])).max() < 1e-4
    assert row_errs(got[3], ref["a"][[49]]).max() < 1e-4
