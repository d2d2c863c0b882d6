"""Mofulix through the engine against its plain twin (`plain_mofulix.py`): each mechanism alone, then whole models of
several geometries under every way of cutting and batching the work, in 32-bit and in bfloat16 (needs the GPU). The
geometries differ from each other in every size; one has sizes no kernel tiles evenly, one has no attention at all
(no cache group), one has nothing but attention (no state), layers run with other layers' tensors."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_mofulix as plain
import trace_tools as tt
from conftest import ROOT, TOL
from plain_gpt2 import read_model

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]
# float32: the largest difference of a row relative to its largest |logit|, as for the other models.
# bfloat16, against the twin in float64 with the same rounded matrices: the root mean square of a row's difference over
# that of the row's logits, both with their means taken off (what a softmax sees of them). The families below show 0.004
# to 0.018 (the largest among the drawn geometries); a fault in a mechanism makes it about 1. Fixed at 0.05.
TOL_B = {"float32": TOL["float32"], "bfloat16": 5e-2}
KEPT_32BIT = (".conv", ".u", ".rel")  # 2-D tensors that the engine keeps in 32 bits


def check_logits(got, reqs, ref, dtype, what, family=None):
    if dtype == "float32":
        return tt.check_against_plain(got, reqs, ref, TOL_B[dtype], what, family=family)
    key = ((family or what.split(" ")[0]) + " (rms)", TOL_B[dtype])
    for rid, toks in reqs.items():
        assert rid in got, f"{what}: no logits for request {rid}"
        for p in sorted(got[rid]):
            row, want = np.asarray(got[rid][p], dtype=np.float64), ref[rid][p]
            assert np.isfinite(row).all(), f"{what}: request {rid} position {p}: non-finite logits"
            diff = row - want
            e = float(np.sqrt(np.mean((diff - diff.mean()) ** 2)) / np.sqrt(np.mean((want - want.mean()) ** 2)))
            tt.WORST[key] = max(tt.WORST.get(key, 0.0), e)
            assert e <= TOL_B[dtype], f"{what}: request {rid} (length {len(toks)}) first differs at position {p}: {e:.3e} > {TOL_B[dtype]:.1e}"


# ---------------------------------------------------------------------------
# configurations
# ---------------------------------------------------------------------------
def attention(heads, kv_heads, dim, scale=None, softcap=None, rot=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale if scale is not None else dim ** -0.5}
    if softcap:
        m["softcap"] = softcap
    if rot:
        m["rot"] = rot
    return m


def rot(dims, base=10000.0, scaling=None):
    r = {"dims": dims, "base": base}
    if scaling:
        r["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return r


def wkv(heads, dim, rank):
    return {"heads": heads, "dim": dim, "decay_rank": rank}


def biased(heads, kv_heads, dim, vdim, rows, far, q_temp=None, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5,
         "bias_max": far, "bias_rows": rows}
    if q_temp:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return m


def space(heads, vdim, state, groups, conv, norm_groups):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def layer(kind, m, ff=None, limit=1.5, weights_of=None):
    entry = {"type": kind, "mixer": m, "mlp": {"kind": "dense", "ff": ff, "limit": limit} if ff else None}
    if weights_of is not None:
        entry["weights_of"] = weights_of
    return entry


def config(vocab, width, eps, scale, layers):
    return {"architecture": "Mofulix", "vocab": vocab, "width": width, "embedding": {"scale": scale}, "norm": {"eps": eps}, "layers": layers}


_PAR = {"left": biased(4, 2, 16, 24, 12, 40, q_temp=(0.3, 7)), "right": space(4, 16, 24, 2, 4, 2)}
CONFIGS = {
    # every kind of layer, two layers that run with another's tensors, a layer without a feed-forward
    "mix": (config(300, 96, 1e-5, 6.0, [
        layer("attention", attention(4, 2, 24, softcap=8.0, rot=rot(16, 5000.0, (8.0, 1.0, 4.0, 64))), ff=160),
        layer("wkv", wkv(3, 32, 8), ff=128, limit=0.8),
        layer("parallel", _PAR, ff=64),
        layer("wkv", wkv(3, 32, 8), ff=128, limit=0.8, weights_of=1),
        layer("parallel", _PAR, ff=64, weights_of=2),
        layer("attention", attention(2, 1, 48, rot=rot(48)), None),
    ]), 21),
    # sizes that no kernel tiles evenly; no soft cap, no query factor, an odd number of bias rows, one tap
    "odd": (config(211, 100, 1e-6, 1.0, [
        layer("parallel", {"left": biased(3, 3, 6, 10, 9, 50), "right": space(3, 14, 10, 3, 1, 3)}, ff=50, limit=0.7),
        layer("attention", attention(3, 3, 10, rot=rot(6)), ff=50),
        layer("wkv", wkv(5, 12, 7), ff=30),
    ]), 22),
    # no attention anywhere: no cache group, state only
    "recurrent": (config(128, 64, 1e-5, 3.0, [layer("wkv", wkv(1, 64, 16), ff=96), layer("wkv", wkv(1, 64, 16), ff=96, weights_of=0)]), 23),
    # attention only: no state; one head in all, heads that all share one key head
    "keys": (config(150, 64, 1e-5, 2.0, [layer("attention", attention(1, 1, 32, softcap=30.0, rot=rot(32, 100.0, (2.0, 1.0, 2.0, 16))), ff=48),
                                         layer("attention", attention(8, 1, 8, scale=0.5), None)]), 24),
    # five taps, heads in one group, one norm part, a far bias edge near the table's half
    "taps": (config(128, 72, 1e-5, 1.5, [
        layer("parallel", {"left": biased(2, 1, 8, 8, 6, 7, q_temp=(1.0, 3)), "right": space(2, 20, 8, 1, 5, 1)}, ff=40, limit=5.0),
        layer("parallel", {"left": biased(1, 1, 32, 16, 32, 100), "right": space(6, 8, 16, 3, 2, 2)}, None),
    ]), 25),
}
LENGTHS = {"mix": [1, 2, 23, 70, 131, 260], "odd": [3, 40, 97, 200], "recurrent": [1, 50, 140], "keys": [2, 65, 150], "taps": [4, 5, 66, 150]}


def twin_tensors(tensors, dtype):
    if dtype == "float32":
        return tensors
    return {k: (plain.round_to_bf16(v) if v.ndim == 2 and not k.endswith(KEPT_32BIT) else v) for k, v in tensors.items()}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    from liyab_amd.weights import write_random_model

    out = {}
    for name, (cfg, seed) in CONFIGS.items():
        d = str(tmp_path_factory.mktemp(f"mofulix_{name}"))
        write_random_model(d, json.loads(json.dumps(cfg)), seed)
        raw, tensors = read_model(d)
        for dtype in DTYPES:
            out[(name, dtype)] = (d, raw, twin_tensors(tensors, dtype))
    return out


def make_requests(name):
    cfg, seed = CONFIGS[name]
    return {f"{name}{i}": tt.random_tokens(seed * 50 + i, n, cfg["vocab"]) for i, n in enumerate(LENGTHS[name])}


@pytest.fixture(scope="module")
def reference(models):
    return {(name, dtype): {rid: plain.forward(raw, t, toks) for rid, toks in make_requests(name).items()}
            for (name, dtype), (_, raw, t) in models.items()}


def make_core(model_dir, dtype, max_tokens, page_size=16, max_requests=4, **kw):
    from liyab_amd.engine import EngineCore

    core = EngineCore(model_dir, dtype=dtype, page_size=page_size, max_tokens=max_tokens, max_requests=max_requests, **kw)
    # free pages and unused state hold NaN: a kernel that reads past a request's length, or a slot's old state, shows it
    for c in core.storage.layers.values():
        for t in c.rows.values():
            t.fill_(float("nan"))
    for t in core.storage.states.values():
        t.fill_(float("nan"))
    torch.cuda.synchronize()
    return core


def rand(rng, *shape, scale=1.0, mean=0.0):
    return torch.from_numpy((rng.standard_normal(shape) * scale + mean).astype(np.float32))


def f64(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


# ---------------------------------------------------------------------------
# each mechanism alone
# ---------------------------------------------------------------------------
class _Layer:
    """A model of one layer, for driving its parts by hand through steps of one request."""

    def __init__(self, dtype, entry, width=64, tensors=None, page_size=8, eps=1e-5):
        from liyab_amd.config import config_from_dict
        from liyab_amd.engine import EngineCore
        from liyab_amd.weights.random_init import random_tensors

        self.raw = config(50, width, eps, 1.0, [entry])
        cfg = config_from_dict(self.raw)
        t = random_tensors(cfg, 5)
        for k, v in (tensors or {}).items():
            assert k in t and tuple(t[k].shape) == tuple(v.shape), (k, tuple(v.shape))
            t[k] = v
        if dtype == "bfloat16":
            t = {k: (v.to(torch.bfloat16).float() if v.dim() == 2 and not k.endswith(KEPT_32BIT) else v) for k, v in t.items()}
        self.t = {k: f64(v) for k, v in t.items()}
        self.core = EngineCore.from_plan(cfg.plan(), t, dtype=dtype, page_size=page_size, num_pages=300, max_requests=3, use_graphs=False)
        for s in self.core.storage.states.values():
            s.fill_(float("nan"))
        for c in self.core.storage.layers.values():
            for rows in c.rows.values():
                rows.fill_(float("nan"))
        self.block = self.core.model.blocks[0]
        self.width, self.dtype, self.eps = width, dtype, eps

    def run(self, rid, rows, portions, fn):
        from liyab_amd.engine import StepItem

        out, done = [], 0
        for take in portions:
            item = StepItem(rid, [1] * take, [])
            ctx, lengths = self.core.step_fn.prepare([item])
            out.append(fn(ctx, rows[done:done + take].to(DEV)))
            self.core.step_fn.commit([item], lengths)
            done += take
        assert done == rows.shape[0]
        return np.concatenate(out)


def _mixer_alone(p, x, portions, rid="m"):
    """The layer's mixer over the rows x (its input) of one request, in portions; both ways of handing the result over."""
    core, mix = p.core, p.block.mixer
    core.open(rid)

    def step(ctx, xs):
        h = xs.to(core.dtype)
        y = torch.empty(xs.shape[0], p.width, dtype=torch.float32, device=DEV)
        mix.forward(h, ctx, core.storage.layer(0), core.storage.state(0), None, out=y)
        return f64(y)

    got = p.run(rid, x, portions, step)
    core.close(rid)
    core.manager.check()
    return got


def _inputs(p, rng, n, scale=1.0):
    x = rand(rng, n, p.width, scale=scale)
    return x, f64(x.to(torch.bfloat16).float() if p.dtype == "bfloat16" else x)


MIXER_TOL = {"float32": 2e-5, "bfloat16": 3e-2}
PORTIONS = ((75,), (25, 1, 9, 1, 1, 2, 36), (2,) * 10 + (1,) * 5 + (50,), (1,) * 75)
# portions long enough to run in segments side by side: a whole number of segments, one token more, one less, and a long
# portion that starts from a state earlier portions left
LONG_PORTIONS = ((257,), (192, 1, 64), (3, 255), (320,))


@pytest.mark.parametrize("d,n", [(96, 5), (100, 33), (2500, 3)])
def test_tanh_norm_alone(d, n):
    from liyab_amd.kernels import ops

    rng = np.random.default_rng(1)
    x, w, b = rand(rng, n, d, scale=3.0).to(DEV), rand(rng, d, mean=1.0).to(DEV), rand(rng, d).to(DEV)
    alpha = torch.tensor([0.37], device=DEV)
    t = {"n": f64(w), "n.b": f64(b), "n.alpha": np.float64(0.37)}
    for dtype in (torch.float32, torch.bfloat16):
        out = torch.empty(n, d, dtype=dtype, device=DEV)
        ops.dyt(out, x, w, b, alpha)
        assert tt.rel_err(f64(out), plain.tanh_norm(f64(x), t, "n")) < (1e-6 if dtype == torch.float32 else 5e-3)
    rows = torch.tensor([n - 1, 0], dtype=torch.int32, device=DEV)
    out = torch.empty(2, d, dtype=torch.float32, device=DEV)
    ops.dyt(out, x, w, b, alpha, rows=rows)
    assert tt.rel_err(f64(out), plain.tanh_norm(f64(x)[[n - 1, 0]], t, "n")) < 1e-6


@pytest.mark.parametrize("M,K,N", [(1, 96, 240), (1, 768, 2304), (8, 768, 2304), (3, 320, 512), (24, 1024, 64), (1, 64, 48), (2, 1600, 4800)])
def test_the_norm_folded_into_a_product(M, K, N):
    """The product that applies the norm to its own operand against the norm's kernel followed by the product."""
    from liyab_amd.kernels import ops

    rng = np.random.default_rng(11)
    x, w, b = rand(rng, M, K, scale=2.0).to(DEV), rand(rng, K, scale=0.1, mean=1.0).to(DEV), rand(rng, K, scale=0.1).to(DEV)
    alpha = torch.tensor([0.5], device=DEV)
    W = rand(rng, N, K, scale=K ** -0.5).to(torch.bfloat16).to(DEV)
    h = torch.empty(M, K, dtype=torch.bfloat16, device=DEV)
    ops.dyt(h, x, w, b, alpha)
    want = f64(h) @ f64(W).T
    out = torch.full((M, N), float("nan"), dtype=torch.float32, device=DEV)
    ops.gemm_skinny_dyt(x, w, b, alpha, W, None, out=out)
    assert tt.rel_err(f64(out), want) < 1e-3  # (the two tanh differ by a rounding of the bfloat16 rows here and there)
    exact = (np.tanh(0.5 * f64(x)) * f64(w) + f64(b)) @ f64(W).T
    assert tt.rel_err(f64(out), exact) < 1e-2


def test_the_recurrence_kernels_sizes():
    """The sizes the host says the recurrence kernel takes are the ones its launcher takes."""
    from liyab_amd.kernels import lib, ops

    native = lib.load().liyab_scan_takes
    for rows in (1, 3, 4, 8, 10, 16, 32, 64, 100, 128, 256, 300, 512, 600):
        for cols in (1, 4, 8, 14, 16, 24, 48, 64, 100, 128, 256, 512, 600):
            assert bool(native(rows, cols)) == ops.scan_takes(rows, cols), (rows, cols)
    assert ops.scan_takes(64, 64) and ops.scan_takes(128, 128) and ops.scan_takes(128, 64) and not ops.scan_takes(64, 1000)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,ff,limit", [(64, 96, 1.5), (100, 50, 0.3), (72, 200, 50.0)])
def test_clamped_feed_forward_alone(dtype, width, ff, limit):
    """Limits that clamp most entries, some, and none."""
    p = _Layer(dtype, layer("wkv", wkv(2, 16, 4), ff=ff, limit=limit), width=width)
    x, xs = _inputs(p, np.random.default_rng(2), 37, scale=2.0)
    y = torch.zeros(37, width, dtype=torch.float32, device=DEV)
    from liyab_amd.engine import StepItem

    p.core.open("f")
    ctx, _ = p.core.step_fn.prepare([StepItem("f", [1] * 37, [])])
    p.block.ffn.forward(x.to(DEV).to(p.core.dtype), ctx, y)
    want = plain.feed_forward(xs, p.t, "l0.mlp.", p.raw["layers"][0]["mlp"])
    assert tt.rel_err(f64(y), want) < MIXER_TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m", [wkv(3, 32, 8), wkv(5, 12, 7), wkv(1, 64, 16), wkv(2, 128, 4), wkv(4, 8, 1)])
def test_wkv_alone_in_portions(dtype, m):
    """The state and the previous input row travel from portion to portion, down to single tokens; a second request in a
    slot that was used before starts from zeros whatever the slot holds."""
    p = _Layer(dtype, layer("wkv", m), width=72)
    rng = np.random.default_rng(3)
    # (a decay of rank 1 is one bfloat16 number a token: over hundreds of tokens its rounding alone passes the tolerance)
    for k, portions in enumerate(PORTIONS + (LONG_PORTIONS if dtype == "float32" or m["decay_rank"] > 1 else ())):
        x, xs = _inputs(p, rng, sum(portions))
        want = plain.wkv(xs, p.t, "l0.mix.", m, p.eps)
        got = _mixer_alone(p, x, portions, rid=f"w{k}")
        assert tt.rel_err(got, want) < MIXER_TOL[dtype], (m, portions[:4])


def test_wkv_remembers_far_back():
    """Channels that hardly decay carry one early token's value to the end of a long sequence: the output there changes by
    much when that token's input changes, and the engine follows the twin whole, in portions and token by token."""
    m = wkv(2, 16, 4)
    H, D, width = 2, 16, 64
    t = {"l0.mix.w0": torch.full((H * D,), -9.0), "l0.mix.w2": torch.zeros(H * D, 4)}  # decay exp(-exp(-9)): 0.9999 a token
    p = _Layer("float32", layer("wkv", m), width=width, tensors=t)
    rng = np.random.default_rng(4)
    n = 400
    x, xs = _inputs(p, rng, n)
    want = plain.wkv(xs, p.t, "l0.mix.", m, p.eps)
    blind = xs.copy()
    blind[3] = 0.0
    assert np.abs(plain.wkv(blind, p.t, "l0.mix.", m, p.eps)[-1] - want[-1]).max() > 1e-3
    for k, portions in enumerate(((n,), (n - 40,) + (1,) * 40, (100, 2, 150, 37, 2, 107, 2))):
        assert tt.rel_err(_mixer_alone(p, x, portions, rid=f"f{k}"), want) < 2e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m", [space(4, 16, 24, 2, 4, 2), space(3, 14, 10, 3, 1, 3), space(2, 20, 8, 1, 5, 1), space(6, 8, 16, 3, 2, 2),
                               space(1, 64, 128, 1, 3, 4)])
def test_state_space_alone_in_portions(dtype, m):
    """The convolution's last inputs and the heads' matrices travel from portion to portion; one tap (no ring), heads in
    groups, norm parts that span several heads and parts of one head."""
    entry = layer("parallel", {"left": biased(1, 1, 8, 8, 4, 9), "right": m})
    p = _Layer(dtype, entry, width=72)
    rng = np.random.default_rng(5)
    core, mix = p.core, p.block.mixer.right
    for k, portions in enumerate(PORTIONS + LONG_PORTIONS):
        x, xs = _inputs(p, rng, sum(portions))
        want = plain.state_space(xs, p.t, "l0.mix.right.", m, p.eps)
        rid = f"s{k}"
        core.open(rid)

        def step(ctx, rows):
            y = torch.empty(rows.shape[0], p.width, dtype=torch.float32, device=DEV)
            mix.forward(rows.to(core.dtype), ctx, None, core.storage.state(0), None, out=y)
            return f64(y)

        got = p.run(rid, x, portions, step)
        core.close(rid)
        assert tt.rel_err(got, want) < MIXER_TOL[dtype], (m, portions[:4])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m", [attention(4, 2, 24, softcap=8.0, rot=rot(16, 5000.0, (8.0, 1.0, 4.0, 64))), attention(3, 3, 10, rot=rot(6)),
                               attention(8, 1, 8, scale=0.5), attention(1, 1, 32, softcap=2.0, rot=rot(32, 100.0, (2.0, 1.0, 2.0, 16))),
                               attention(2, 1, 40, rot=rot(40, 200000.0, (3.0, 1.0, 8.0, 1024)))])
def test_gated_attention_alone_in_portions(dtype, m):
    """Normed and turned queries and keys, values that are the keys as projected, a soft cap that bites (2.0) and one that
    hardly does, frequencies on both sides of the stretch and in between, a head whose entries are only partly turned."""
    p = _Layer(dtype, layer("attention", m), width=72)
    rng = np.random.default_rng(6)
    for k, portions in enumerate(PORTIONS):
        n = sum(portions)
        x, xs = _inputs(p, rng, n)
        want = plain.gated_attention(xs, p.t, "l0.mix.", m, p.eps, np.arange(n, dtype=np.float64))
        got = _mixer_alone(p, x, portions, rid=f"a{k}")
        assert tt.rel_err(got, want) < MIXER_TOL[dtype], (m, portions[:4])


def test_rotary_frequencies_follow_the_stretch():
    from liyab_amd.config.plan import RotarySpec
    from liyab_amd.parts.scored_attention import rotary_frequencies

    for dims, base, sc in ((16, 5000.0, (8.0, 1.0, 4.0, 64)), (40, 200000.0, (3.0, 1.0, 8.0, 1024)), (32, 100.0, None), (6, 10000.0, (2.0, 1.0, 2.0, 16))):
        got = rotary_frequencies(RotarySpec(dims=dims, base=base, scaling=sc))
        want = plain.rotary_frequencies(rot(dims, base, sc))
        assert np.allclose(got, want, rtol=1e-14)
        if sc:  # all three branches occur in the first two
            wl = 2 * np.pi / np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
            kinds = {("short" if w < sc[3] / sc[2] else "long" if w > sc[3] / sc[1] else "between") for w in wl}
            assert dims == 6 or kinds == {"short", "long", "between"}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m", [biased(4, 2, 16, 24, 12, 40, q_temp=(0.3, 7)), biased(3, 3, 6, 10, 9, 50), biased(2, 1, 8, 8, 6, 7, q_temp=(1.0, 3)),
                               biased(1, 1, 32, 16, 32, 100), biased(2, 2, 64, 32, 4, 3, q_temp=(0.5, 64)),
                               biased(4, 1, 16, 16, 10, 30, q_temp=(0.5, 5)), biased(2, 2, 64, 64, 32, 112), biased(3, 1, 8, 8, 7, 11)])
def test_biased_attention_alone_in_portions(dtype, m):
    """Keys and values of different widths and of one width (which the matrix-core kernels take), the query's factor across
    several of its steps, the bias by distance over all its rows and past its last."""
    entry = layer("parallel", {"left": m, "right": space(1, 8, 4, 1, 2, 1)})
    p = _Layer(dtype, entry, width=72)
    rng = np.random.default_rng(7)
    core, mix = p.core, p.block.mixer.left
    for k, portions in enumerate(PORTIONS + ((140,),)):
        n = sum(portions)
        x, xs = _inputs(p, rng, n)
        want = plain.biased_attention(xs, p.t, "l0.mix.left.", m, np.arange(n, dtype=np.float64))
        rid = f"b{k}"
        core.open(rid)

        def step(ctx, rows):
            y = torch.empty(rows.shape[0], p.width, dtype=torch.float32, device=DEV)
            mix.forward(rows.to(core.dtype), ctx, core.storage.layer(0), None, None, out=y)
            return f64(y)

        got = p.run(rid, x, portions, step)
        core.close(rid)
        assert tt.rel_err(got, want) < MIXER_TOL[dtype], (m, portions[:4])


def test_distance_rows_follow_the_twin():
    from liyab_amd.parts.scored_attention import distance_rows

    for rows, far in ((32, 112), (12, 40), (9, 50), (6, 7), (4, 3), (32, 256), (16, 64), (7, 1000)):
        got = distance_rows(rows, far)
        assert got.tolist() == [plain.distance_bucket(n, rows, far) for n in range(far + 1)]
        assert got[-1] == rows - 1 and plain.distance_bucket(far + 1000, rows, far) == rows - 1


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("row", [3, 5, 7, 8, 11])
@pytest.mark.parametrize("page_size,dk,dv", [(8, 8, 12), (16, 8, 12), (16, 16, 16)])
def test_a_bias_row_that_stands_out_at_its_edges(dtype, row, page_size, dk, dv):
    """One row of the distance table is far above the others and the scores themselves are small, so that a query's result is
    nearly the mean of the values at that row's distances: a distance counted one off, or a row's edge one off, shows in
    full. Rows below the table's half (one distance each), logarithmic rows, and the last row (every distance from the
    far edge on, hundreds back), in prompts' portions and decoded alone."""
    rows, far, H = 12, 40, 2
    m = biased(H, 1, dk, dv, rows, far, scale=0.01)
    rel = torch.zeros(rows, H)
    rel[row, 0] = 14.0
    rel[(row + 3) % rows, 1] = 14.0
    entry = layer("parallel", {"left": m, "right": space(1, 8, 4, 1, 2, 1)})
    p = _Layer(dtype, entry, width=64, tensors={"l0.mix.left.rel": rel}, page_size=page_size)
    core, mix = p.core, p.block.mixer.left
    n = 300
    x, xs = _inputs(p, np.random.default_rng(8), n, scale=2.0)
    pos = np.arange(n, dtype=np.float64)
    want = plain.biased_attention(xs, p.t, "l0.mix.left.", m, pos)
    # the marked row matters: the table one row off gives another result
    shifted = dict(p.t)
    shifted["l0.mix.left.rel"] = np.roll(p.t["l0.mix.left.rel"], 1, axis=0)
    assert np.abs(plain.biased_attention(xs, shifted, "l0.mix.left.", m, pos) - want)[far + 5:].max() > 0.05
    for k, portions in enumerate(((n,), (n - 60,) + (1,) * 60, (100, 2, 150, 9, 2, 35, 2))):
        rid = f"e{k}"
        core.open(rid)

        def step(ctx, rws):
            y = torch.empty(rws.shape[0], p.width, dtype=torch.float32, device=DEV)
            mix.forward(rws.to(core.dtype), ctx, core.storage.layer(0), None, None, out=y)
            return f64(y)

        got = p.run(rid, x, portions, step)
        core.close(rid)
        assert tt.rel_err(got, want) < (2e-5 if dtype == "float32" else 3e-2), (row, portions[:3])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page_size", [8, 16])
def test_a_marked_key_far_away(dtype, page_size):
    """One earlier position's key lies along the query's own (weights made so that a head's query and key are the input's
    first channels), and the scale is such that it and the query's own position share nearly all the weight: whether the
    query finds it among hundreds, at page borders, as the last row of a portion and decoded alone, is most of its
    result. Few entries are turned, so that the match survives the distance."""
    H, D, width = 2, 48, 64
    m = attention(H, 1, D, scale=0.7, rot=rot(4, 10000.0))
    eye = torch.eye(width)
    t = {"l0.mix.q": torch.cat([eye[4:4 + D]] * H).clone(), "l0.mix.k": eye[4:4 + D].clone(),
         "l0.mix.q.norm": torch.ones(D), "l0.mix.k.norm": torch.ones(D), "l0.mix.g": torch.zeros(H * D, width)}
    p = _Layer(dtype, layer("attention", m), width=width, tensors=t, page_size=page_size)
    rng = np.random.default_rng(9)
    n = 330
    query_at = [n - 1, n - 2, 290, 2 * page_size * 8 + 1]
    for case, distance in enumerate([n - 4, 200, 257, n - 1 - page_size]):
        x = rand(rng, n, width)
        x[query_at, 4:8] = 0.0  # the turned entries of the marked queries: their match does not depend on the distance
        marks = {}
        for i in query_at:
            j = i - distance
            if j < 0 or j in marks or j in query_at or any(abs(j - o) < 2 for o in marks):
                continue
            marks[j] = i
            x[j, 4:4 + D] = 3.0 * x[i, 4:4 + D]  # the same direction (keys are normed), a value of its own (values are not)
        xs = f64(x.to(torch.bfloat16).float() if dtype == "bfloat16" else x)
        pos = np.arange(n, dtype=np.float64)
        want = plain.gated_attention(xs, p.t, "l0.mix.", m, p.eps, pos)
        blind = xs.copy()
        for j in marks:
            blind[j] = 0.01
        moved = np.abs(plain.gated_attention(blind, p.t, "l0.mix.", m, p.eps, pos) - want)[list(marks.values())].max(-1)
        assert len(marks) > 0 and (moved > 0.05).all(), (distance, moved)
        for portions in ((n,), (n - 40,) + (1,) * 40, (100, 2, 150, 37, 2, 37, 2)):
            got = _mixer_alone(p, x, portions, rid=f"k{case}")
            assert tt.rel_err(got, want) < (2e-5 if dtype == "float32" else 6e-2), (distance, portions[:3])


@pytest.mark.parametrize("dtype", DTYPES)
def test_two_mixers_side_by_side(dtype):
    entry = layer("parallel", _PAR)
    p = _Layer(dtype, entry, width=80)
    rng = np.random.default_rng(10)
    for k, portions in enumerate(PORTIONS[:3]):
        n = sum(portions)
        x, xs = _inputs(p, rng, n)
        want = plain.parallel_mixer(xs, p.t, "l0.mix.", _PAR, p.eps, np.arange(n, dtype=np.float64))
        got = _mixer_alone(p, x, portions, rid=f"p{k}")
        assert tt.rel_err(got, want) < MIXER_TOL[dtype], portions[:4]


# ---------------------------------------------------------------------------
# whole models
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_each_request_alone_and_whole_and_every_layer(name, dtype, models, reference):
    reqs = make_requests(name)
    steps = tt.schedule_whole(reqs)
    core = make_core(models[(name, dtype)][0], dtype, tt.max_live_tokens(steps))
    got = tt.run_schedule(core, steps)
    check_logits(got, reqs, reference[(name, dtype)], dtype, f"mofulix-whole {name} {dtype}")
    core.manager.check()
    assert not core.manager.groups or core.manager.pages_in_use() == 0
    if dtype == "float32":
        from liyab_amd.engine import StepItem

        rid, toks = list(reqs.items())[2]
        streams, caught = [], []
        plain.forward(models[(name, dtype)][1], models[(name, dtype)][2], toks, streams)
        plain_core = make_core(models[(name, dtype)][0], dtype, 512, use_graphs=False)
        plain_core.model.replay_layers = False
        for block in plain_core.model.blocks:
            def wrapped(x, ctx, cache, state, writes_cache=True, _f=block.forward):
                out = _f(x, ctx, cache, state, writes_cache=writes_cache)
                caught.append(f64(x)[:len(toks)])
                return out
            block.forward = wrapped
        plain_core.open(rid)
        plain_core.step([StepItem(rid, toks, [])])
        assert len(caught) == len(streams)
        for got_x, want_x in zip(caught, streams):
            assert tt.rel_err(got_x, want_x) < 1e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_a_prompt_then_its_last_tokens_one_by_one(name, dtype, models, reference):
    reqs = make_requests(name)
    steps = tt.schedule_bulk_tail(reqs, tail=45)
    core = make_core(models[(name, dtype)][0], dtype, tt.max_live_tokens(steps))
    got = tt.run_schedule(core, steps)
    check_logits(got, reqs, reference[(name, dtype)], dtype, f"mofulix-decode {name} {dtype}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(5, 2, 17, 3, 48, 2, 31, 7), (2, 2, 2, 3), (1, 64, 1, 16, 2)])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_portions_of_changing_size(name, dtype, sizes, models, reference):
    reqs = make_requests(name)
    if sizes[0] == 2:
        reqs = dict(list(reqs.items())[:3])
    steps = tt.schedule_portions(reqs, sizes)
    core = make_core(models[(name, dtype)][0], dtype, tt.max_live_tokens(steps), page_size=8 if sizes[0] == 1 else 16)
    got = tt.run_schedule(core, steps)
    check_logits(got, reqs, reference[(name, dtype)], dtype, f"mofulix-portions {name} {dtype}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seed,max_live,page_size", [(0, 4, 16), (1, 3, 8), (2, 2, 24)])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_mixed_batches_with_pages_and_slots_used_again(name, dtype, seed, max_live, page_size, models, reference):
    """Up to `max_live` requests at a time, portions of some beside single tokens of others, in a pool and with state slots
    just large enough: what a finished request gives back is used by the next."""
    base = make_requests(name)
    reqs = {f"{rid}#{k}": toks for k in range(2) for rid, toks in base.items()}
    ref = {f"{rid}#{k}": reference[(name, dtype)][rid] for k in range(2) for rid in base}
    steps = tt.schedule_mixed(reqs, seed=seed, max_live=max_live)
    core = make_core(models[(name, dtype)][0], dtype, None, page_size=page_size, max_requests=max_live, num_pages=tt.max_live_pages(steps, page_size))
    got = tt.run_schedule(core, steps)
    check_logits(got, reqs, ref, dtype, f"mofulix-mixed {name} {dtype}")
    core.manager.check()
    assert not core.manager.groups or core.manager.pages_in_use() == 0
    assert core.step_fn.graph_replays > 0  # the decode-only steps of the tail were replayed from graphs


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mix", "recurrent"])
def test_long_decoding_from_the_first_token(name, dtype, models, reference):
    rid, toks = list(make_requests(name).items())[-1]
    reqs = {rid: toks}
    steps = tt.schedule_bulk_tail(reqs, tail=len(toks))
    core = make_core(models[(name, dtype)][0], dtype, tt.max_live_tokens(steps))
    got = tt.run_schedule(core, steps)
    check_logits(got, reqs, reference[(name, dtype)], dtype, f"mofulix-long {name} {dtype}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_trace_program(dtype, models, reference, tmp_path):
    name = "odd"
    reqs = make_requests(name)
    steps = tt.schedule_mixed(reqs, seed=5, max_live=4)
    got = tt.run_trace_program(models[(name, dtype)][0], dtype, steps, str(tmp_path), tt.max_live_tokens(steps), CONFIGS[name][0]["vocab"])
    check_logits(got, reqs, reference[(name, dtype)], dtype, f"mofulix-trace {dtype}")


def draw_config(seed):
    """A geometry drawn from the seed: every size, constant and count, the layers' kinds and order, and which layers run with
    another's tensors."""
    rng = np.random.default_rng(1000 + seed)
    pick = lambda *options: options[int(rng.integers(len(options)))]  # noqa: E731
    width = pick(40, 48, 64, 96, 104, 160)

    def one():
        kind = pick("attention", "wkv", "parallel")
        if kind == "attention":
            kv = pick(1, 2, 3)
            dim = pick(4, 8, 10, 16, 24, 32)
            sc = pick(None, (pick(2.0, 8.0), 1.0, pick(2.0, 4.0), pick(16, 64, 256)))
            m = attention(kv * pick(1, 2, 4), kv, dim, softcap=pick(None, 5.0, 50.0), rot=pick(None, rot(pick(2, dim // 2 * 2, dim // 4 * 2 or 2), pick(100.0, 10000.0), sc)))
        elif kind == "wkv":
            m = wkv(pick(1, 2, 3, 5), pick(4, 8, 12, 16, 32, 64), pick(1, 3, 8, 16))
        else:
            kv = pick(1, 2, 3)
            rows = pick(4, 6, 9, 12, 32)
            groups = pick(1, 2, 3)
            heads = groups * pick(1, 2)
            vdim = pick(4, 8, 14, 16, 24)
            norm_groups = pick(1, heads, 2 if heads * vdim % 2 == 0 else 1)
            m = {"left": biased(kv * pick(1, 2), kv, pick(4, 6, 16, 32), pick(4, 10, 16, 24), rows, rows // 2 + pick(1, 5, 30, 200),
                                q_temp=pick(None, (pick(0.2, 1.0), pick(3, 16, 100)))),
                 "right": space(heads, vdim, pick(4, 10, 16, 32), groups, pick(1, 2, 3, 4, 6), norm_groups)}
        return layer(kind, m, ff=pick(None, 8, 20, 24, 40, 56), limit=pick(0.5, 2.0, 7.0))

    layers = [one() for _ in range(int(rng.integers(1, 5)))]
    owners = {}
    for _ in range(int(rng.integers(0, 3))):
        owner = layers[int(rng.integers(len(layers)))]
        owner = owners.get(id(owner), owner)
        entry = json.loads(json.dumps(owner))
        owners[id(entry)] = owner
        layers.insert(int(rng.integers(0, len(layers) + 1)), entry)  # before or behind the layer whose tensors it uses
    for entry in layers:
        if id(entry) in owners:
            entry["weights_of"] = next(i for i, other in enumerate(layers) if other is owners[id(entry)])
    return config(pick(97, 256, 500), width, pick(1e-5, 1e-6, 1e-3), pick(1.0, 4.0, 9.0), layers), pick(8, 16, 24)


@pytest.mark.parametrize("seed", range(12))
def test_drawn_geometries_whole_and_mixed(seed, tmp_path):
    from liyab_amd.weights import write_random_model

    cfg, page_size = draw_config(seed)
    d = str(tmp_path / "m")
    write_random_model(d, json.loads(json.dumps(cfg)), 100 + seed)
    raw, tensors = read_model(d)
    for i, entry in enumerate(raw["layers"]):
        if entry.get("weights_of") is not None:
            assert raw["layers"][entry["weights_of"]].get("weights_of") is None and entry["weights_of"] != i
    reqs = {f"g{i}": tt.random_tokens(seed * 10 + i, n, raw["vocab"]) for i, n in enumerate([1, 19, 77, 150, 260])}
    for dtype in DTYPES:
        t = twin_tensors(tensors, dtype)
        ref = {rid: plain.forward(raw, t, toks) for rid, toks in reqs.items()}
        steps = tt.schedule_whole(reqs)
        core = make_core(d, dtype, tt.max_live_tokens(steps), page_size=page_size)
        check_logits(tt.run_schedule(core, steps), reqs, ref, dtype, f"mofulix-drawn seed {seed} whole {dtype}", family="mofulix-drawn")
        steps = tt.schedule_mixed(reqs, seed=seed, max_live=3)
        core = make_core(d, dtype, None, page_size=page_size, max_requests=3, num_pages=tt.max_live_pages(steps, page_size))
        check_logits(tt.run_schedule(core, steps), reqs, ref, dtype, f"mofulix-drawn seed {seed} mixed {dtype}", family="mofulix-drawn")
        core.manager.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_real_widths_in_long_steps(dtype, tmp_path):
    """Heads of 64 and 128, a width of 512, prompts of hundreds of tokens in one step and in mixed batches: the tiles of the
    large products, the matrix-core attention with capped and with biased scores (keys and values of one width and of two),
    the recurrences with states of 64 x 64 and 128 x 64 a head."""
    from liyab_amd.weights import write_random_model

    par = {"left": biased(8, 4, 64, 64, 32, 100, q_temp=(0.2, 128)), "right": space(8, 64, 128, 2, 4, 1)}
    cfg = config(1000, 512, 1e-5, 2.0, [
        layer("attention", attention(8, 8, 64, softcap=25.0, rot=rot(64, 10000.0, (8.0, 1.0, 4.0, 256))), ff=1024, limit=6.0),
        layer("wkv", wkv(8, 64, 32), ff=1024, limit=6.0),
        layer("parallel", par, ff=1024, limit=6.0),
        layer("attention", attention(4, 1, 128, rot=rot(32)), None),
        layer("parallel", {"left": biased(4, 4, 128, 64, 16, 300), "right": space(4, 128, 16, 1, 2, 4)}, ff=768, limit=3.0),
        layer("wkv", wkv(8, 64, 32), ff=1024, limit=6.0, weights_of=1),
    ])
    d = str(tmp_path / "m")
    write_random_model(d, json.loads(json.dumps(cfg)), 31)
    raw, tensors = read_model(d)
    t = twin_tensors(tensors, dtype)
    reqs = {f"r{i}": tt.random_tokens(900 + i, n, raw["vocab"]) for i, n in enumerate([330, 700, 45])}
    ref = {rid: plain.forward(raw, t, toks) for rid, toks in reqs.items()}
    steps = tt.schedule_whole(reqs)
    core = make_core(d, dtype, tt.max_live_tokens(steps))
    check_logits(tt.run_schedule(core, steps), reqs, ref, dtype, f"mofulix-wide whole {dtype}", family="mofulix-wide")
    steps = tt.schedule_mixed(reqs, seed=3, max_live=3, portions=(2, 130, 64, 300, 17))
    core = make_core(d, dtype, None, max_requests=3, num_pages=tt.max_live_pages(steps, 16))
    check_logits(tt.run_schedule(core, steps), reqs, ref, dtype, f"mofulix-wide mixed {dtype}", family="mofulix-wide")
    core.manager.check()


def generate_greedy(raw, t, prompt, n_new):
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(np.argmax(plain.forward(raw, t, toks)[-1])))
    return toks[len(prompt):]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mix", "odd"])
def test_greedy_generation_through_the_entry_point(name, dtype, models):
    """Engine.generate: the scheduler batches the prompts in portions beside decoding requests, in a pool that does not hold
    them all at once (requests are preempted and computed again, their slots' state starting over); each token is the twin's
    greedy choice given the tokens so far."""
    from liyab_amd import Engine, SamplingParams

    d, raw, t = models[(name, dtype)]
    prompts = [tt.random_tokens(70 + i, n, raw["vocab"]) for i, n in enumerate([1, 13, 64, 100, 7])]
    n_new = 12
    engine = Engine(d, dtype=dtype, page_size=16, num_pages=14, max_num_seqs=3, max_batched_tokens=48, prefill_chunk=24)
    engine.stop_at_eos = False
    results = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=n_new))
    for prompt, res in zip(prompts, results):
        assert len(res.tokens) == n_new
        ref = plain.forward(raw, t, prompt + res.tokens[:-1])
        for i, tok in enumerate(res.tokens):
            row = ref[len(prompt) - 1 + i]
            slack = (1e-5 if dtype == "float32" else 5e-2) * np.abs(row).max()
            assert row[tok] >= row.max() - slack, f"token {i} of prompt length {len(prompt)}: {tok} vs {int(np.argmax(row))}"
        if dtype == "float32":
            assert res.tokens == generate_greedy(raw, t, prompt, n_new)
    engine.core.manager.check()


def test_command_line(models):
    d, raw, tensors = models[("taps", "float32")]
    prompt = tt.random_tokens(90, 11, raw["vocab"])
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "liyab-cli"), "-m", d, "-p", ",".join(map(str, prompt)), "-n", "6",
                        "--temp", "0", "--dtype", "float32", "--json", "--phases"], capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    turn = [json.loads(l) for l in p.stdout.splitlines() if l.startswith("{")][1]
    assert turn["tokens"] == generate_greedy(raw, tensors, prompt, 6)
    assert set(turn["phases_ms"]) == {"embed", "side_by_side", "clamped_glu", "lm_head"}
