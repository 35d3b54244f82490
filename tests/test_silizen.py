"""The Silizen design against the plain implementation in ``tests/plain/silizen_plain.py``: every mechanism alone,
then whole models of several small shapes replayed whole, token by token, in portions and in mixed batches (32-bit
and bfloat16 through graphs), and greedy generation through the engine's own entry point."""
import copy
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from tests import traces
from tests.plain import silizen_plain as P
from tests.test_gidurax import BF16_NOISE, F32_ATOL, _Ctx, _in_portions, _paged, _replay, requests_for, write_model

gpu = pytest.mark.gpu


# ================================================================================================ configurations
def dense(ff):
    return {"kind": "dense", "ff": ff}


def rotated(heads, kv_heads, dim, vdim, scale, softcap, base, dims, scaling=None):
    rot = {"base": base, "dims": dims}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "softcap": softcap, "rot": rot}


def parallel(left, heads, dim, vdim, tau, left_scale, right_scale, mlp):
    return {"type": "parallel", "mlp": mlp,
            "mixer": {"left": left, "right": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau},
                      "left_scale": left_scale, "right_scale": right_scale}}


def parallel_2(heads, kv_heads, dim, vdim, scale, size, r_heads, r_kv, r_dim, r_vdim, conv, mlp):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if size is not None:
        left["mask"] = {"size": size}
    return {"type": "parallel_2", "mlp": mlp,
            "mixer": {"left": left, "right": {"heads": r_heads, "kv_heads": r_kv, "dim": r_dim, "vdim": r_vdim, "conv": conv}}}


def wkv(heads, dim, mlp):
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim}, "mlp": mlp}


def config(vocab, width, eps, logit_scale, layers, loop=None):
    c = {"architecture": "Silizen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "logit_scale": logit_scale,
         "layers": layers}
    if loop is not None:
        c["loop"] = dict(zip(("start", "stop", "times"), loop))
    return c


# ranks of the low-rank maps, by layer: they are tensor shapes, not config.json keys
RANKS = {"P": {0: (5,), 1: (7, 3), 2: (4,), 3: (6, 9)}, "Q": {0: (8, 8), 1: (3,), 2: (12,)}, "R": {0: (6,), 1: (5,), 2: (2, 4)},
         "S": {0: (16,), 1: (8, 8), 2: (8,)}, "T": {0: (3,), 1: (3, 5)}}

# Shapes that differ in every size and in the order of their layers: a looped stretch at the start, in the middle, over
# the whole model and none; a stretch walked once; windows shorter and longer than a page; groups of one, two and three
# query heads; key and value sizes that differ either way; all, some or none of a head's entries rotated; frequency
# scaling with and without; recurrences whose q/k heads are shared by two value heads; two to five taps; a layer
# without a feed-forward; scales of the two halves on either side of one.
SHAPES = {
    "P": config(211, 96, 1e-5, 0.5, [
        parallel(rotated(6, 2, 16, 24, 0.3, 5.0, 10000.0, 8, (8.0, 1.0, 4.0, 64)), 3, 12, 20, 8.0, 0.7, 1.3, dense(128)),
        parallel_2(4, 2, 24, 16, 0.2, 20, 4, 2, 16, 12, 3, dense(72)),
        wkv(3, 20, None),
        parallel_2(3, 3, 32, 32, 0.15, 7, 2, 2, 24, 40, 5, dense(64))], loop=(0, 2, 2)),
    "Q": config(330, 128, 3e-6, 2.0, [
        parallel_2(4, 1, 24, 40, 0.25, 33, 6, 3, 8, 16, 2, dense(200)),
        wkv(4, 32, dense(96)),
        parallel(rotated(2, 2, 64, 16, 0.125, 30.0, 500.0, 64), 2, 40, 24, 4.0, 1.0, 0.5, None)], loop=(1, 3, 3)),
    "R": config(150, 64, 1e-6, 1.0, [
        wkv(2, 36, dense(72)),
        parallel(rotated(6, 3, 8, 40, 0.4, 2.0, 100000.0, 0), 1, 70, 10, 32.0, 1.5, 0.4, dense(40)),
        parallel_2(2, 1, 40, 8, 0.3, 1, 1, 1, 20, 20, 4, dense(96))]),
}
# heads of 64 and of 32 with values of the same size and pages of 16: shapes the matrix cores take in bfloat16
SHAPES["S"] = config(257, 160, 1e-5, 0.25, [
    parallel(rotated(6, 2, 64, 64, 0.11, 15.0, 10000.0, 32, (4.0, 1.0, 4.0, 128)), 4, 32, 32, 16.0, 0.6, 1.1, dense(192)),
    parallel_2(4, 4, 32, 32, 0.18, 40, 4, 2, 64, 64, 4, dense(128)),
    wkv(5, 64, dense(64))], loop=(1, 2, 1))
# sizes that are multiples of nothing much (a width of 100, heads of 10 and 14), the whole model one looped stretch
SHAPES["T"] = config(77, 100, 1e-5, 0.8, [
    parallel(rotated(5, 5, 10, 14, 0.3, 8.0, 10000.0, 6), 2, 18, 26, 2.0, 0.9, 1.0, dense(36)),
    parallel_2(2, 2, 14, 10, 0.3, None, 3, 1, 10, 14, 3, None)], loop=(0, 2, 2))
# heads of 128 (one key/value head for four query heads), a window of several pages, every entry of a head rotated, wide
# recurrences, the first layer alone walked three times
SHAPES["U"] = config(301, 256, 1e-5, 0.3, [
    parallel_2(4, 1, 128, 128, 0.09, 50, 2, 1, 128, 96, 4, dense(256)),
    parallel(rotated(4, 2, 128, 128, 0.09, 12.0, 1000000.0, 128, (2.0, 1.0, 8.0, 256)), 2, 128, 64, 16.0, 0.6, 1.1, dense(192)),
    wkv(2, 128, dense(128))], loop=(0, 1, 3))
RANKS["U"] = {0: (16, 24), 1: (16,), 2: (32,)}
PAGES = {"P": 16, "Q": 8, "R": 4, "S": 16, "T": 16, "U": 16}
SEEDS = {"P": 84, "Q": 92, "R": 81, "S": 98, "T": 82, "U": 77}


def tensor_shapes(cfg, ranks):
    """Names and shapes, stated here from the design (not asked of the product)."""
    W, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, W), "final.norm": (W,), "final.norm.b": (W,)}
    if cfg.get("loop"):
        out["loop.in"] = (W, 2 * W)
    for i, layer in enumerate(cfg["layers"]):
        p, m, rk = f"l{i}.", layer["mixer"], ranks[i]
        out[p + "norm1"] = out[p + "norm1.b"] = (W,)
        if layer["type"] == "wkv":
            H, D = m["heads"], m["dim"]
            for s in "rkvgw":
                out[p + "mix.mu." + s] = (W,)
            for s in "rkvg":
                out[p + "mix." + s] = (H * D, W)
            out.update({p + "mix.w1": (rk[0], W), p + "mix.w2": (H * D, rk[0]), p + "mix.w0": (H * D,), p + "mix.u": (H, D),
                        p + "mix.norm": (H * D,), p + "mix.o": (W, H * D)})
        else:
            l, r = m["left"], m["right"]
            H, G, D, E = l["heads"], l["kv_heads"], l["dim"], l["vdim"]
            a = p + "mix.left."
            out.update({a + "q": (H * D, W), a + "k": (G * D, W), a + "v": (G * E, W), a + "g": (H, W), a + "o": (W, H * E)})
            b = p + "mix.right."
            if layer["type"] == "parallel":
                out.update({a + "q.norm": (D,), a + "k.norm": (D,)})
                h, d, e = r["heads"], r["dim"], r["vdim"]
                out.update({b + "q": (h * d, W), b + "k": (h * d, W), b + "v": (h * e, W), b + "g": (h * e, W), b + "o": (W, h * e),
                            b + "norm": (e,), b + "a1": (rk[0], W), b + "a2": (h * d, rk[0]), b + "a2.b": (h * d,)})
            else:
                out.update({a + "q.b": (H * D,), a + "k.b": (G * D,), a + "v.b": (G * E,)})
                h, g, d, e, taps = r["heads"], r["kv_heads"], r["dim"], r["vdim"], r["conv"]
                out.update({b + "q": (g * d, W), b + "q.conv": (g * d, taps), b + "k": (g * d, W), b + "k.conv": (g * d, taps),
                            b + "v": (h * e, W), b + "v.conv": (h * e, taps), b + "b": (h, W), b + "A_log": (h,),
                            b + "norm": (e,), b + "a1": (rk[0], W), b + "a2": (h * d, rk[0]), b + "dt_bias": (h * d,),
                            b + "g1": (rk[1], W), b + "g2": (h * e, rk[1]), b + "o": (W, h * e),
                            p + "mix.left.out": (W,), p + "mix.right.out": (W,)})
        mlp = layer["mlp"]
        if mlp is not None:
            out.update({p + "mlp.gate": (mlp["ff"], W), p + "mlp.up": (mlp["ff"], W), p + "mlp.down": (W, mlp["ff"])})
    return out


def random_weights(cfg, ranks, seed, dtype=torch.bfloat16):
    """Weights large enough that every mechanism moves the logits: scores of order one that reach the cap, decays between
    slow and fast, gates half open, biases that count."""
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg, ranks).items():
        leaf = name.split(".")[-1]
        r = torch.randn(shape, generator=g)
        if name.endswith(("norm1", "final.norm", "q.norm", "k.norm", "right.norm", "mix.norm", "left.out", "right.out")):
            t = 1.0 + 0.2 * r
        elif name.endswith(("norm1.b", "final.norm.b")):
            t = 0.2 * r
        elif name.endswith(("q.b", "k.b", "v.b")):
            t = 0.5 * r
        elif name == "embed":
            t = r
        elif name == "loop.in":
            t = r / math.sqrt(shape[-1] / 2)
        elif leaf == "conv":
            t = 0.6 * r
        elif leaf == "A_log":
            t = -0.5 + 0.5 * r
        elif leaf == "dt_bias":
            t = r
        elif name.endswith("a2.b"):
            t = 2.0 + r
        elif leaf == "w0":
            t = -2.0 + 0.7 * r
        elif leaf == "u":
            t = 0.5 * r
        elif ".mu." in name:
            t = 0.5 + 0.3 * r
        elif leaf in ("a2", "g2", "w2"):
            t = r / math.sqrt(shape[-1])
        else:
            t = r * (2.0 / math.sqrt(shape[-1]))
        w[name] = t
    # A recurrence's first read-out is (q . k) v, and the norm that follows keeps only its sign: where q . k is next to
    # zero, rounding decides the sign and no bound on rounding errors holds.  Keys that lean towards their queries
    # (and a bonus that is mostly positive) keep the first tokens away from that.
    for name in list(w):
        for key, query in ((".right.k", ".right.q"), (".right.k.conv", ".right.q.conv"), (".mix.k", ".mix.r")):
            if name.endswith(key):
                w[name] = w[name[:-len(key)] + query] + 0.4 * w[name]
        if name.endswith(".mix.u"):
            w[name] = 0.6 + 0.2 * w[name]
    return {name: t.to(dtype).contiguous() for name, t in w.items()}


# ================================================================================================ the oracle's own pins
def test_plain_pieces_against_library_routines():
    torch.manual_seed(0)
    x = torch.randn(9, 6, dtype=torch.float64)
    w, b = torch.randn(6, dtype=torch.float64), torch.randn(6, dtype=torch.float64)
    assert torch.allclose(P.layer_norm(x, w, b, 1e-5), F.layer_norm(x, (6,), w, b, 1e-5), atol=1e-12)
    assert torch.allclose(P.unit_rms(x, 1e-5), F.rms_norm(x, (6,), None, 1e-5), atol=1e-12)
    assert torch.allclose(P.gelu_tanh(x), F.gelu(x, approximate="tanh"), atol=1e-12)
    assert torch.allclose(P.silu(x), F.silu(x), atol=1e-12)
    assert torch.allclose(P.softplus(5 * x), F.softplus(5 * x), atol=1e-12)
    taps = torch.randn(6, 4, dtype=torch.float64)
    ref = F.conv1d(F.pad(x.T[None], (3, 0)), taps[:, None, :], groups=6)[0].T
    assert torch.allclose(P.causal_conv(x, taps), ref, atol=1e-12)
    # the rotation is a complex product of (entry i, entry i + half) with exp(i p f_i); entries past 2 half stay
    f = P.rotary_frequencies(4, 100.0)
    assert torch.allclose(f, torch.tensor([1.0, 0.1], dtype=torch.float64))
    v = torch.randn(5, 2, 7, dtype=torch.float64)
    pos = torch.tensor([0, 1, 2, 50, 1000])
    got = P.rotate_half(v, pos, f)
    z = torch.complex(v[..., :2], v[..., 2:4]) * torch.polar(torch.ones(5, 2, dtype=torch.float64), pos[:, None] * f[None, :])[:, None, :]
    assert torch.allclose(got[..., :2], z.real, atol=1e-12) and torch.allclose(got[..., 2:4], z.imag, atol=1e-12)
    assert torch.equal(got[..., 4:], v[..., 4:]) and torch.equal(got[0], v[0])
    # frequency scaling: short waves stay, long waves are divided, one in between is blended
    fs = P.rotary_frequencies(8, 10000.0, {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64})
    f0 = P.rotary_frequencies(8, 10000.0)
    wave = 2 * math.pi / f0
    assert wave[0] < 16 and float(fs[0]) == float(f0[0])
    assert wave[3] > 64 and abs(float(fs[3]) - float(f0[3]) / 8.0) < 1e-15
    s = (64 / float(wave[1]) - 1.0) / 3.0
    assert 16 < wave[1] < 64 and abs(float(fs[1]) - ((1 - s) * float(f0[1]) / 8 + s * float(f0[1]))) < 1e-15
    # with one more key of score zero and value zero the attention is the library's causal attention
    q, k, vv = (torch.randn(7, 2, 5, dtype=torch.float64) for _ in range(3))
    got = P.sink_attention(q, k, vv, 0.3)
    for i in range(7):
        ke = torch.cat([k[:i + 1], torch.zeros(1, 2, 5, dtype=torch.float64)]).transpose(0, 1)
        ve = torch.cat([vv[:i + 1], torch.zeros(1, 2, 5, dtype=torch.float64)]).transpose(0, 1)
        ref = F.scaled_dot_product_attention(q[i][:, None, :], ke, ve, scale=0.3)[:, 0]
        assert torch.allclose(got[i], ref, atol=1e-12)
    # a first token whose score is zero gives half of its value
    got = P.sink_attention(torch.zeros(1, 1, 5, dtype=torch.float64), k[:1, :1], vv[:1, :1], 1.0)
    assert torch.allclose(got[0, 0], 0.5 * vv[0, 0])
    assert torch.allclose(P.distance_slopes(4), torch.tensor([0.25, 0.0625, 0.015625, 0.00390625], dtype=torch.float64))


def test_plain_attention_at_the_edges_of_cap_window_and_distance():
    torch.manual_seed(1)
    T = 12
    q = torch.zeros(T, 1, 4, dtype=torch.float64)
    k = torch.zeros(T, 1, 4, dtype=torch.float64)
    v = torch.randn(T, 1, 3, dtype=torch.float64)
    # equal scores: a window of 5 gives the mean of the last five values times 5 / 6 (the sink takes a sixth)
    got = P.sink_attention(q, k, v, 1.0, window=5)
    assert torch.allclose(got[9, 0], v[5:10, 0].sum(0) / 6, atol=1e-12)
    assert torch.allclose(got[2, 0], v[0:3, 0].sum(0) / 4, atol=1e-12)
    # a window of one sees the token alone
    assert torch.allclose(P.sink_attention(q, k, v, 1.0, window=1)[7, 0], v[7, 0] / 2, atol=1e-12)
    # the distance penalty: weights fall by exp(-slope) per token of distance
    got = P.sink_attention(q, k, v, 1.0, slopes=torch.tensor([0.5], dtype=torch.float64), window=3)
    e = torch.exp(torch.tensor([-1.0, -0.5, 0.0], dtype=torch.float64))
    assert torch.allclose(got[6, 0], (e[:, None] * v[4:7, 0]).sum(0) / (1 + e.sum()), atol=1e-12)
    # the cap: a huge score counts as the cap itself
    q[:, 0, 0], k[3, 0, 0] = 1.0, 1000.0
    got = P.sink_attention(q, k, v, 1.0, softcap=2.0)
    e = torch.ones(6, dtype=torch.float64)
    e[3] = math.exp(2.0)
    assert torch.allclose(got[5, 0], (e[:, None] * v[:6, 0]).sum(0) / (1 + e.sum()), atol=1e-9)


def test_plain_recurrences_have_their_closed_forms():
    torch.manual_seed(2)
    T, H, d, e = 6, 2, 3, 4
    q, k = torch.randn(T, H, d, dtype=torch.float64), torch.randn(T, H, d, dtype=torch.float64)
    v = torch.randn(T, H, e, dtype=torch.float64)
    # a constant decay a: o_t = sum_j a^(t - j) (q_t . k_j) v_j, the current token undecayed
    a = 0.7
    got = P.gated_linear_attention(q, k, v, torch.full((T, H, d), a, dtype=torch.float64))
    want = torch.stack([sum(a ** (t - j) * (q[t] * k[j]).sum(-1, keepdim=True) * v[j] for j in range(t + 1)) for t in range(T)])
    assert torch.allclose(got, want, atol=1e-12)
    # a decay per channel acts on the key's channel
    al = torch.rand(T, H, d, dtype=torch.float64)
    got = P.gated_linear_attention(q, k, v, al)
    assert torch.allclose(got[1], ((q[1] * al[1] * k[0]).sum(-1, keepdim=True) * v[0]) + (q[1] * k[1]).sum(-1, keepdim=True) * v[1], atol=1e-12)
    # the bonus recurrence: the current token is weighted by u, earlier ones decay from the token after them on
    u, w = torch.randn(H, d, dtype=torch.float64), torch.rand(T, H, d, dtype=torch.float64)
    got = P.bonus_recurrence(q, k, v, w, u)
    assert torch.allclose(got[0], (q[0] * u * k[0]).sum(-1, keepdim=True) * v[0], atol=1e-12)
    want2 = (q[2] * w[1] * k[0]).sum(-1, keepdim=True) * v[0] + (q[2] * k[1]).sum(-1, keepdim=True) * v[1] + \
        (q[2] * u * k[2]).sum(-1, keepdim=True) * v[2]
    assert torch.allclose(got[2], want2, atol=1e-12)
    # the delta rule with beta = 1, no decay and a unit key: the key's value is replaced, and read back at once
    kk = F.normalize(k, dim=-1)
    got = P.gated_delta_rule(kk, kk, v, torch.ones(T, H, d, dtype=torch.float64), torch.ones(T, H, dtype=torch.float64))
    assert torch.allclose(got, v, atol=1e-12)


def test_plain_order_of_a_looped_stretch():
    cfg = SHAPES["Q"]
    assert P.run_order(cfg) == [(0, False), (1, True), (2, False), (1, True), (2, False), (1, True), (2, False)]
    assert P.run_order(SHAPES["R"]) == [(0, False), (1, False), (2, False)]
    assert P.run_order(SHAPES["S"]) == [(0, False), (1, True), (2, False)]


def test_config_reads_every_size_and_refuses_what_it_does_not_know():
    from llm_infrence_engine_amd.config import ConfigError, config_from_dict
    from llm_infrence_engine_amd.parts.model import Model

    for name, cfg in SHAPES.items():
        shapes = tensor_shapes(cfg, RANKS[name])
        c = config_from_dict(copy.deepcopy(cfg))
        assert type(c).__name__ == "SilizenConfig" and c.to_dict() == cfg
        with pytest.raises(ConfigError):
            c.to_spec()                                   # the ranks are not in config.json
        c = c.with_tensor_shapes(lambda n: shapes.get(n))
        model = Model(c.to_spec())
        assert {s.name: tuple(s.shape) for s in model.tensor_specs()} == shapes
        order = P.run_order(cfg)
        assert [r.layer for r in model.spec.order] == [i for i, _ in order]
        assert [r.opens_pass is not None for r in model.spec.order] == [o for _, o in order]
        for (i, _), (kv, state, _) in zip(order, model.run_needs()):
            layer, m = cfg["layers"][i], cfg["layers"][i]["mixer"]
            states = list(state) if isinstance(state, tuple) else [state]
            if layer["type"] == "wkv":
                assert kv is None and [s.shape for s in states] == [(1, cfg["width"]), (m["heads"], m["dim"], m["dim"])]
                assert states[1].dtype == torch.float32
            else:
                l, r = m["left"], m["right"]
                assert [(t.name, t.heads, t.width) for t in kv.tensors] == [("k", l["kv_heads"], l["dim"]), ("v", l["kv_heads"], l["vdim"])]
                assert kv.window == (l["mask"]["size"] if l.get("mask") else None)
                assert states[-1].shape == (r["heads"], r["dim"], r["vdim"]) and states[-1].dtype == torch.float32
                if layer["type"] == "parallel_2":
                    assert states[0].shape == (r["conv"] - 1, 2 * r["kv_heads"] * r["dim"] + r["heads"] * r["vdim"])
        assert model.graph_safe() is True
    for change in (lambda c: c["layers"][0].__setitem__("type", "something_else"),
                   lambda c: c["layers"][0]["mixer"]["left"].pop("vdim"),
                   lambda c: c["layers"][0]["mixer"].pop("left_scale"),
                   lambda c: c["layers"][0]["mixer"]["left"]["rot"].__setitem__("dims", 7),
                   lambda c: c["layers"][0]["mixer"]["right"].__setitem__("tau", 0.0),
                   lambda c: c["layers"][1]["mixer"]["right"].pop("conv"),
                   lambda c: c["layers"][1]["mixer"]["left"].__setitem__("kv_heads", 3),
                   lambda c: c["layers"][2]["mixer"].pop("dim"),
                   lambda c: c["layers"][0]["mlp"].pop("ff"),
                   lambda c: c.__setitem__("loop", {"start": 2, "stop": 2, "times": 2})):
        bad = copy.deepcopy(SHAPES["P"])
        change(bad)
        with pytest.raises(ConfigError):
            config_from_dict(bad)


def test_plain_model_prefix_property():
    """The plain model is causal: the logits of a prefix do not change when tokens follow."""
    cfg = SHAPES["R"]
    w = {k: v.double() for k, v in random_weights(cfg, RANKS["R"], 5).items()}
    toks = requests_for(cfg["vocab"], [23], 1)["r0"]
    full = P.forward(cfg, w, toks)
    assert torch.allclose(P.forward(cfg, w, toks[:9]), full[:9], atol=1e-9)


# ================================================================================================ kernels alone
@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H", [96, 130, 1024])
def test_layer_norm_with_a_bias(dtype, H):
    from llm_infrence_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(H)
    x = (3.0 * torch.randn(11, H, generator=g) + 2.0)
    w, b = 1.0 + 0.3 * torch.randn(H, generator=g), torch.randn(H, generator=g)
    want = P.layer_norm(x.double(), w.double(), b.double(), 1e-5)
    out = ops.layer_norm(x.cuda(), w.cuda(), 1e-5, torch.empty(11, H, dtype=dtype, device="cuda"), bias=b.cuda())
    assert (out.cpu().double() - want).abs().max() < (1e-5 if dtype == torch.float32 else 4e-2)
    rows = torch.tensor([7, 0, 7], dtype=torch.int32, device="cuda")
    out = ops.layer_norm(x.cuda(), w.cuda(), 1e-5, torch.empty(3, H, dtype=dtype, device="cuda"), rows=rows, bias=b.cuda())
    assert (out.cpu().double() - want[[7, 0, 7]]).abs().max() < (1e-5 if dtype == torch.float32 else 4e-2)


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,E,dims,weighted", [(6, 2, 16, 24, 8, True), (4, 1, 64, 64, 64, True), (3, 3, 32, 8, 0, False),
                                                  (2, 1, 6, 10, 6, True), (5, 5, 10, 14, 0, True), (2, 2, 130, 16, 100, True)])
def test_head_norms_rotation_and_store(dtype, H, G, D, E, dims, weighted):
    """Norm (with or without weights), rotation of the first ``dims`` entries in half-split pairs with scaled frequencies,
    and the store of k and v at slots in no order; positions up to some thousands."""
    from llm_infrence_engine_amd.kernels import ops
    from llm_infrence_engine_amd.parts.positions import scaled_frequencies

    g = torch.Generator().manual_seed(D + dims)
    N, page = 9, 4
    pos = torch.tensor([0, 1, 2, 3, 63, 64, 1000, 4095, 7], dtype=torch.int32)
    qkv = torch.randn(N, (H + G) * D + G * E, generator=g).to(dtype)
    qw, kw = (1.0 + 0.3 * torch.randn(D, generator=g) for _ in range(2))
    scaling = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}
    f = P.rotary_frequencies(dims, 10000.0, scaling) if dims else torch.zeros(0, dtype=torch.float64)
    if dims:
        assert torch.allclose(scaled_frequencies(dims, 10000.0, scaling), f, rtol=1e-12)
    q = qkv[:, :H * D].double().view(N, H, D)
    k = qkv[:, H * D:(H + G) * D].double().view(N, G, D)
    v = qkv[:, (H + G) * D:].double().view(N, G, E)
    q, k = P.unit_rms(q, 1e-5), P.unit_rms(k, 1e-5)
    if weighted:
        q, k = q * qw.double(), k * kw.double()
    if dims:
        # angles as a 32-bit engine forms them: the product of the position and the rounded frequency, rounded once
        ang = (pos.float()[:, None] * f.float()[None, :]).double()[:, None, :]
        half = dims // 2

        def turn(x):
            a, b = x[..., :half], x[..., half:dims]
            return torch.cat([a * torch.cos(ang) - b * torch.sin(ang), b * torch.cos(ang) + a * torch.sin(ang), x[..., dims:]], -1)

        assert torch.allclose(turn(q)[:6], P.rotate_half(q, pos, f)[:6], atol=1e-4)     # the plain rotation, up to the angles' rounding
        q, k = turn(q), turn(k)
    slots = torch.tensor([13, 2, 7, 0, 31, 5, -1, 22, 9], dtype=torch.int32)
    k_pages = torch.full((8, G, page, D), 9.0, dtype=dtype, device="cuda")
    v_pages = torch.full((8, G, page, E), 9.0, dtype=dtype, device="cuda")
    dev = qkv.cuda()
    ops.qk_norm_store(dev, H, G, D, E, qw.cuda() if weighted else None, kw.cuda() if weighted else None, 1e-5, pos.cuda(),
                      slot_mapping=slots.cuda(), k_pages=k_pages, v_pages=v_pages, unit_norm=True,
                      inv_freq=f.float().cuda() if dims else None, rot_dim=dims)
    tol = 3e-5 if dtype == torch.float32 else 4e-2
    got = dev.cpu().double()
    assert (got[:, :H * D].view(N, H, D) - q).abs().max() < tol
    assert (got[:, H * D:(H + G) * D].view(N, G, D) - k).abs().max() < tol
    for n, s in enumerate(slots.tolist()):
        if s >= 0:
            assert (k_pages[s // page, :, s % page].cpu().double() - k[n]).abs().max() < tol
            assert (v_pages[s // page, :, s % page].cpu().double() - v[n]).abs().max() < 1e-6
    assert float(k_pages[6, 0, 3, 0]) == 9.0     # slot 27 belongs to nobody


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,E,page,window,softcap,slopes", [
    (6, 2, 16, 24, 4, None, 5.0, False), (4, 1, 64, 64, 16, 96, None, True), (3, 3, 32, 8, 8, 7, None, True),
    (2, 1, 6, 10, 4, 1, 3.0, True), (8, 2, 64, 64, 16, None, 20.0, False), (4, 4, 32, 32, 16, 33, 2.0, True),
    (3, 1, 128, 128, 16, 300, None, True), (5, 5, 10, 14, 16, None, None, False)])
def test_attention_with_cap_distance_window_gate_and_loud_keys(dtype, H, G, D, E, page, window, softcap, slopes):
    """One sequence of 300 tokens in pages in no order; a prompt's portion of 40 queries and then single tokens.  One key
    far back at a page's last slot, one just inside and one just outside the window are made loud for a query each, so
    that leaving one out, letting one in or being one token off shows; the sink of score zero, the cap, the distance
    penalty per head and the gate per token and head all count."""
    from llm_infrence_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(D + E)
    T, Tq = 300, 40
    q = torch.randn(T, H, D, generator=g).to(dtype)
    k = torch.randn(T, G, D, generator=g).to(dtype)
    v = torch.randn(T, G, E, generator=g).to(dtype)
    gate = torch.randn(T, H, generator=g).to(dtype)

    def loud(key, query, head=0):
        k[key, head // (H // G)] = (6.0 * q[query, head].float() / q[query, head].float().norm()).to(dtype)

    loud(3 * page - 1, T - 5)
    if window is not None and window < T - 20:
        loud(T - 10 - window + 1, T - 10)         # the oldest key the query at T - 10 sees
        loud(T - 20 - window, T - 20)             # the newest one the query at T - 20 no longer sees
        loud(T - 1 - window + 1, T - 1, H - 1)
        loud(T - 2 - window, T - 2, H - 1)
    scale = 1.3 / math.sqrt(D)
    sl = P.distance_slopes(H) if slopes else None
    want = P.sink_attention(q.double(), k.double(), v.double(), scale, softcap=softcap, slopes=sl, window=window)
    want = 0.7 * want * torch.sigmoid(gate.double())[:, :, None]
    order = list(np.random.default_rng(1).permutation(np.arange(1, 1 + -(-T // page))))
    sink = torch.zeros(H, device="cuda")
    slopes_dev = sl.float().cuda() if slopes else None
    tol = 3e-5 if dtype == torch.float32 else 3e-2
    # a padded projection: q in the first columns, the gate's numbers in the last
    pad = 8 + (-H) % 8          # rows of a multiple of 16 bytes, as the matrix-core kernel reads them
    packed = torch.cat([q.reshape(T, H * D), torch.zeros(T, pad, dtype=dtype), gate], dim=1).cuda()
    steps = [(T - Tq, Tq - 6)] + [(T - 6 + i, 1) for i in range(6)]
    # both value layouts: in bfloat16, transposed values of the keys' size in pages of 16 go to the matrix cores
    for transposed in (False, True):
        k_pages, v_pages, table = _paged(k, v, page, order, dtype, transposed)

        class KV:
            pass

        kv = KV()
        kv.k_pages, kv.v_pages, kv.v_transposed, kv.block_table = k_pages, v_pages, transposed, table
        kv.table_rows = torch.tensor([1], dtype=torch.int32, device="cuda")
        for start, n in steps:
            ctx = _Ctx([n], [0], [start])
            out = torch.empty(n, H * E, dtype=dtype, device="cuda")
            rows = packed[start:start + n]
            ops.paged_attention(rows[:, :H * D], kv, ctx, out, H, scale, window, sink, softcap or 0.0, slopes_dev,
                                rows[:, H * D + pad:], 0.7)
            err = (out.cpu().double().reshape(n, H, E) - want[start:start + n]).abs().max()
            assert err < tol, (transposed, start, n, float(err))


@gpu
@pytest.mark.parametrize("H,G,D,window,softcap,slopes", [(8, 2, 64, None, 20.0, False), (4, 4, 32, 700, None, True),
                                                         (14, 2, 128, None, 5.0, True), (6, 3, 64, 96, None, True)])
def test_changed_scores_when_single_tokens_are_decoded(H, G, D, window, softcap, slopes):
    """A step of single tokens in bfloat16 over contexts short and long (beyond the length from which a small batch's
    keys are split over blocks and combined): the matrix-core kernels with the cap, the distance penalty, the sink of
    score zero and the gate, against the plain attention."""
    from llm_infrence_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(H + D)
    page, lens = 16, [1300, 40, 700]
    scale = 1.1 / math.sqrt(D)
    sl = P.distance_slopes(H) if slopes else None
    qs, gates, want, tables, kps, vps, base = [], [], [], [], [], [], 1
    for T in lens:
        q = torch.randn(1, H, D, generator=g).bfloat16()
        k = torch.randn(T, G, D, generator=g).bfloat16()
        v = torch.randn(T, G, D, generator=g).bfloat16()
        gate = torch.randn(1, H, generator=g).bfloat16()
        k[5, 0] = (5.0 * q[0, 0].float() / q[0, 0].float().norm()).bfloat16()          # a loud key near the start
        if window is not None and T > window:
            k[T - window, 0] = (6.0 * q[0, 0].float() / q[0, 0].float().norm()).bfloat16()       # the oldest key in sight
            k[T - window - 1, G - 1] = (6.0 * q[0, H - 1].float() / q[0, H - 1].float().norm()).bfloat16()   # just out of it
        # the last query alone: the plain attention row by row is slow over 1,300 keys, so only that row is asked for
        rep = H // G
        row = torch.zeros(H, D, dtype=torch.float64)
        for h in range(H):
            lo = 0 if window is None else max(0, T - window)
            s_ = (k[lo:, h // rep].double() @ q[0, h].double()) * scale
            if softcap:
                s_ = softcap * torch.tanh(s_ / softcap)
            if sl is not None:
                s_ = s_ - sl[h] * (T - 1 - torch.arange(lo, T, dtype=torch.float64))
            e = torch.exp(s_)
            row[h] = 0.7 * torch.sigmoid(gate[0, h].double()) * (e[:, None] * v[lo:, h // rep].double()).sum(0) / (1 + e.sum())
        want.append(row)
        n = -(-T // page)
        order = [base + int(i) for i in np.random.default_rng(T).permutation(n)]
        kp, vp, table = _paged(k, v, page, order, torch.bfloat16, True)
        kps.append(kp), vps.append(vp), tables.append(table[1]), qs.append(q.reshape(1, H * D)), gates.append(gate)
        base += n
    P_ = base + 1
    k_pages = torch.zeros(P_, G, page, D, dtype=torch.bfloat16, device="cuda")
    v_pages = torch.zeros(P_, G, D, page, dtype=torch.bfloat16, device="cuda")
    width = max(t.numel() for t in tables)
    table = torch.zeros(len(lens) + 1, width, dtype=torch.int32, device="cuda")
    for r, (kp, vp, tb) in enumerate(zip(kps, vps, tables)):
        used = tb[tb > 0].long()
        k_pages[used], v_pages[used] = kp[used], vp[used]
        table[r + 1, :tb.numel()] = tb
    ctx = _Ctx([1] * len(lens), [0] * len(lens), [T - 1 for T in lens])

    class KV:
        pass

    kv = KV()
    kv.k_pages, kv.v_pages, kv.v_transposed, kv.block_table = k_pages, v_pages, True, table
    kv.table_rows = torch.tensor([1, 2, 3], dtype=torch.int32, device="cuda")
    out = torch.empty(len(lens), H * D, dtype=torch.bfloat16, device="cuda")
    packed = torch.cat([torch.cat(qs), torch.cat(gates), torch.zeros(len(lens), (-H) % 8, dtype=torch.bfloat16)], dim=1).cuda()
    ops.paged_attention_mfma(packed[:, :H * D], k_pages, v_pages, table, ctx.q_start, ctx.context_lens, out, H, scale, 1,
                             max(lens), window, kv.table_rows, torch.zeros(H, device="cuda"), softcap or 0.0,
                             sl.float().cuda() if slopes else None, packed[:, H * D:H * D + H], 0.7)
    for r in range(len(lens)):
        assert (out[r].cpu().double().reshape(H, D) - want[r]).abs().max() < 3e-2, r


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,D,E", [(3, 12, 20), (2, 48, 64), (1, 70, 10), (4, 32, 32), (2, 130, 24), (5, 16, 100)])
@pytest.mark.parametrize("bonus", [False, True])
@pytest.mark.parametrize("long", [False, True])
def test_decaying_recurrence_in_portions_and_batches(dtype, H, D, E, bonus, long):
    """Three sequences from slots in no order, in portions of unequal sizes (one token, two, more than a chunk), batched
    together, against the whole recurrence; q, k, v are slices of wider rows.  ``long``: portions of hundreds of tokens,
    which are spread over blocks in stretches (a stretch's edge inside a portion, a portion that ends a stretch exactly, a
    short portion beside long ones)."""
    from llm_infrence_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(D + E)
    lens = [700, 300, 9] if long else [150, 41, 9]
    cuts = [[300, 1, 399], [256, 43, 1], [1, 1, 7]] if long else [[70, 1, 1, 2, 76], [3, 30, 8], [1, 1, 7]]
    slots = [2, 0, 3]
    rows = [torch.randn(n, 2 * H * D + H * E + 5, generator=g).to(dtype) for n in lens]
    z = [torch.randn(n, H * D, generator=g) for n in lens]
    zb = torch.randn(H * D, generator=g) + (2.0 if not bonus else -2.0)
    u = torch.randn(H * D, generator=g)
    tau, q_scale = 4.0, D ** -0.5
    want = []
    for r_, z_ in zip(rows, z):
        a = r_.double()
        n = a.shape[0]
        q = a[:, :H * D].view(n, H, D) * q_scale
        k = a[:, H * D:2 * H * D].view(n, H, D)
        v = a[:, 2 * H * D + 5:].view(n, H, E)
        zz = (z_.double() + zb.double()).view(n, H, D)
        if bonus:
            want.append(P.bonus_recurrence(q, k, v, torch.exp(-torch.exp(zz)), u.double().view(H, D)).reshape(n, H * E))
        else:
            want.append(P.gated_linear_attention(q, k, v, torch.sigmoid(zz) ** (1 / tau)).reshape(n, H * E))
    state = torch.full((5, H, D, E), 7.0, device="cuda")
    state[torch.tensor(slots)] = 0.0

    def run(live, at, q_lens, ctx):
        r_ = torch.cat([rows[r][at[r]:at[r] + n] for r, n in zip(live, q_lens)]).cuda()
        z_ = torch.cat([z[r][at[r]:at[r] + n] for r, n in zip(live, q_lens)]).cuda()
        out = torch.empty(r_.shape[0], H * E, device="cuda")
        return ops.decay_recurrence(r_[:, :H * D], r_[:, H * D:2 * H * D], r_[:, 2 * H * D + 5:], z_, zb.cuda(), state, ctx, out,
                                    H, D, E, ops.DECAY_DOUBLE_EXP if bonus else ops.DECAY_SIGMOID_ROOT, tau=tau,
                                    bonus=u.cuda() if bonus else None, q_scale=q_scale)

    got = _in_portions(lens, cuts, slots, run)
    for a, b in zip(got, want):
        assert (a.double() - b).abs().max() < (5e-5 if long else 2e-5) * max(1.0, float(b.abs().max()))
    assert torch.equal(state[1].cpu(), torch.full((H, D, E), 7.0)) and torch.equal(state[4].cpu(), torch.full((H, D, E), 7.0))


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W", [64, 100, 300])
def test_token_shift_in_portions_and_batches(dtype, W):
    from llm_infrence_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(W)
    lens = [23, 9, 14]
    cuts = [[10, 1, 1, 11], [2, 7], [1, 13]]
    slots = [4, 1, 3]
    hs = [torch.randn(n, W, generator=g).to(dtype) for n in lens]
    mu = torch.rand(5, W, generator=g)
    want = []
    for h in hs:
        a = h.double()
        prev = torch.cat([torch.zeros(1, W, dtype=torch.float64), a[:-1]])
        want.append(torch.stack([a + (prev - a) * mu[m].double() for m in range(5)]))
    state = torch.full((6, 1, W), 7.0, dtype=dtype, device="cuda")
    state[slots] = 0

    def run(live, at, q_lens, ctx):
        x = torch.cat([hs[r][at[r]:at[r] + n] for r, n in zip(live, q_lens)]).cuda()
        out = ops.token_shift(x, mu.cuda(), state, ctx, torch.empty(5, x.shape[0], W, dtype=dtype, device="cuda"))
        return out.transpose(0, 1)

    got = _in_portions(lens, cuts, slots, run)
    for a, b in zip(got, want):
        assert (a.double().transpose(0, 1) - b).abs().max() < (1e-6 if dtype == torch.float32 else 3e-2)
    assert float(state[0, 0, 0]) == 7.0 and float(state[5, 0, 0]) == 7.0
    assert torch.equal(state[4, 0].cpu(), hs[0][-1])


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_small_kernels_between_the_products(dtype):
    from llm_infrence_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(4)
    N, W, F_ = 13, 100, 37
    tol = 2e-5 if dtype == torch.float32 else 4e-2
    a, b = (2.0 * torch.randn(N, W, generator=g)).to(dtype), torch.randn(N, W, generator=g).to(dtype)
    x = torch.randn(N, W, generator=g)
    wa, wb = 1.0 + 0.2 * torch.randn(W, generator=g), 1.0 + 0.2 * torch.randn(W, generator=g)
    got = ops.pair_sum(x.clone().cuda(), a.cuda(), b.cuda(), 0.6, 1.1)
    assert (got.cpu().double() - (x.double() + 0.6 * a.double() + 1.1 * b.double())).abs().max() < 1e-5
    got = ops.pair_sum(x.clone().cuda(), a.cuda(), b.cuda(), 0.5, 0.5, wa.cuda(), wb.cuda(), 1e-5)
    want = x.double() + 0.5 * (P.unit_rms(a.double(), 1e-5) * wa.double() + P.unit_rms(b.double(), 1e-5) * wb.double())
    assert (got.cpu().double() - want).abs().max() < 1e-5
    gu = (2.0 * torch.randn(N, 2 * F_, generator=g)).to(dtype)
    got = ops.gelu_tanh_glu(gu.cuda(), torch.empty(N, F_, dtype=dtype, device="cuda"))
    assert (got.cpu().double() - P.gelu_tanh(gu.double()[:, 0::2]) * gu.double()[:, 1::2]).abs().max() < tol
    got = ops.concat_rows(x.cuda(), (2 * x).cuda(), torch.empty(N, 2 * W, dtype=dtype, device="cuda"))
    assert (got.cpu().double() - torch.cat([x, 2 * x], 1).double()).abs().max() < tol
    t = torch.randn(N, 7, generator=g).to(dtype)
    assert (ops.tanh_(t.clone().cuda()).cpu().double() - torch.tanh(t.double())).abs().max() < tol
    # the read-out's norm with a weight per head and channel, and a scale
    o = torch.randn(N, 3 * 20, generator=g)
    wn, gt = 1.0 + 0.2 * torch.randn(60, generator=g), torch.randn(N, 60, generator=g).to(dtype)
    got = ops.gated_head_norm(o.cuda(), wn.cuda(), gt.cuda(), torch.empty(N, 60, dtype=dtype, device="cuda"), 3, 20, 1e-5, "silu",
                              scale=1.3)
    want = 1.3 * P.unit_rms(o.double().view(N, 3, 20), 1e-5).reshape(N, 60) * wn.double() * P.silu(gt.double())
    assert (got.cpu().double() - want).abs().max() < tol


@gpu
@pytest.mark.parametrize("M,K,F_", [(200, 128, 96), (70, 64, 40), (513, 256, 320)])
def test_gated_product_with_the_tanh_gelu_as_its_epilogue(M, K, F_):
    from llm_infrence_engine_amd.kernels import linear, ops

    g = torch.Generator().manual_seed(M)
    a = torch.randn(M, K, generator=g).bfloat16()
    gate, up = (torch.randn(F_, K, generator=g) / math.sqrt(K) * 2).bfloat16(), (torch.randn(F_, K, generator=g) / math.sqrt(K)).bfloat16()
    w = linear.interleave_rows(gate.cuda(), up.cuda())
    got = ops.gemm_tiled(a.cuda(), w, ops.EPI_GEGLU)
    want = P.gelu_tanh(a.double() @ gate.double().T) * (a.double() @ up.double().T)
    assert got.shape == (M, F_) and ((got.cpu().double() - want).abs() / want.abs().clamp(min=1.0)).max() < 2e-2


# ================================================================================================ whole models
def rounded_forward(cfg, w, toks):
    exact = P.forward(cfg, w, toks)
    return exact, float((P.forward(cfg, w, toks, act_dtype=torch.bfloat16) - exact).abs().max())


@pytest.fixture(scope="module", params=list(SHAPES))
def shape(request, tmp_path_factory):
    name = request.param
    cfg = SHAPES[name]
    weights = random_weights(cfg, RANKS[name], seed=SEEDS[name])
    folder = write_model(tmp_path_factory.mktemp("silizen" + name), cfg, weights)
    lengths = {"P": [5, 61, 2, 130, 33, 48], "Q": [1, 9, 90, 47, 110, 64], "R": [3, 26, 70, 17, 2, 41, 60, 33],
               "S": [70, 3, 140, 50, 97, 33], "T": [40, 2, 90, 17, 66], "U": [120, 5, 64, 33]}[name]
    reqs = requests_for(cfg["vocab"], lengths, seed=ord(name))
    w64 = {k: v.double() for k, v in weights.items()}
    want, noise = {}, {}
    for rid, toks in reqs.items():
        want[rid], noise[rid] = rounded_forward(cfg, w64, toks)
        want[rid] = want[rid].numpy()
    return name, cfg, folder, reqs, want, noise


def _compare(got, want, noise, dtype):
    assert got
    for (rid, pos), row in got.items():
        err = np.abs(row.astype(np.float64) - want[rid][pos]).max()
        bound = F32_ATOL if dtype == "float32" else BF16_NOISE * max(noise[rid], 0.02)
        assert err < bound, f"request {rid} position {pos}: max |dlogit| {err:.3e} >= {bound:.3e}"


@gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["whole", "bulk_then_single", "changing_portions", "mixed"])
def test_replay_against_plain(shape, tmp_path, dtype, mode):
    name, cfg, folder, reqs, want, noise = shape
    page = PAGES[name]
    up = lambda n: -(-n // 64) * 64
    if mode == "mixed":
        # room for the two longest requests only: pages and state slots are handed out again and again
        max_tokens = sum(sorted(up(len(t)) for t in reqs.values())[-2:])
        steps = traces.mixed(reqs, max_tokens, seed=3, max_live=4, tail=20)
    else:
        max_tokens = max(up(len(t)) for t in reqs.values())
        steps = {"whole": traces.whole, "bulk_then_single": lambda r: traces.bulk_then_single(r, tail=45),
                 "changing_portions": traces.changing_portions}[mode](reqs)
    runner = _replay(folder, dtype, steps, tmp_path / "out", max_tokens, page)
    _compare(traces.collect(steps, tmp_path / "out", cfg["vocab"]), want, noise, dtype)
    if mode == "mixed":
        assert runner.manager.groups[0].allocator.pages_granted_again() > 0


@gpu
def test_portions_and_batches_change_nothing_in_32_bit(shape, tmp_path):
    """The logits at a position do not depend on how the prompt was cut or on what else was in the batch, beyond
    rounding: whole against portions against mixed, directly (not through the oracle)."""
    name, cfg, folder, reqs, want, noise = shape
    page = PAGES[name]
    up = lambda n: -(-n // 64) * 64
    outs = {}
    total = sum(up(len(t)) for t in reqs.values())
    for mode, steps in (("whole", traces.whole(reqs)), ("portions", traces.changing_portions(reqs, sizes=(2, 3, 2, 31, 5, 2))),
                        ("mixed", traces.mixed(reqs, total, seed=9, tail=10))):
        _replay(folder, "float32", steps, tmp_path / mode, total, page)
        outs[mode] = traces.collect(steps, tmp_path / mode, cfg["vocab"])
    for mode in ("portions", "mixed"):
        for key, row in outs[mode].items():
            assert np.abs(row - outs["whole"][key]).max() < 2e-4, (mode, key)


@gpu
def test_one_row_and_few_pages_serve_every_request_in_turn(shape):
    """An engine with a single request row and pages for one request: every request gets the state slots and the pages
    its predecessor left, in portions, and must start from zero states, a zero previous token and none of the old keys."""
    from llm_infrence_engine_amd.engine.batch import StepEntry
    from llm_infrence_engine_amd.engine.runner import load_runner

    name, cfg, folder, reqs, want, noise = shape
    page = PAGES[name]
    longest = max(len(t) for t in reqs.values())
    runner = load_runner(folder, dtype="float32", page_size=page, num_pages=-(-longest // page) + 1, max_requests=1,
                         max_len=-(-longest // page) * page)
    for rid, toks in reqs.items():
        cut = max(1, len(toks) // 2)
        got = [runner.step([StepEntry(rid, toks[:cut], list(range(cut)))]).cpu().numpy()]
        assert runner.manager.row(rid) == 0
        if cut < len(toks):
            got.append(runner.step([StepEntry(rid, toks[cut:], list(range(len(toks) - cut)))]).cpu().numpy())
        runner.free_request(rid)
        assert np.abs(np.concatenate(got) - want[rid]).max() < F32_ATOL, rid
    runner.manager.check_invariants()
    assert runner.manager.groups[0].allocator.pages_granted_again() > 0


@gpu
@pytest.mark.parametrize("kind", ["parallel", "parallel_2", "wkv"])
def test_far_token_reaches_the_end(tmp_path, kind):
    """A token 400 places back still moves the last logits: through the attention's cache (a loud key: the far token's key
    is what the last queries look for) or through a recurrence's state (decays made slow), in the plain model and equally
    in the engine, whole and decoded token by token over hundreds of steps."""
    layer = {"parallel": parallel(rotated(2, 1, 16, 24, 0.25, 10.0, 10000.0, 8), 2, 12, 16, 64.0, 1.0, 1.0, dense(64)),
             "parallel_2": parallel_2(2, 1, 16, 24, 0.25, 8, 2, 1, 12, 16, 3, dense(64)),
             "wkv": wkv(2, 24, dense(64))}[kind]
    cfg = config(97, 64, 1e-5, 1.0, [layer])
    ranks = {0: (4, 4)}
    weights = random_weights(cfg, ranks, seed=1)
    for k_ in weights:
        if k_.endswith(("a2.b",)):
            weights[k_] = torch.full_like(weights[k_], 4.0)           # sigmoid(4)^(1/64): a memory of thousands of tokens
        if k_.endswith("dt_bias"):
            weights[k_] = torch.full_like(weights[k_], -8.0)          # softplus(-8): a decay of 1 - 3e-4 a token
        if k_.endswith("w0"):
            weights[k_] = torch.full_like(weights[k_], -6.0)          # exp(-exp(-6)): 1 - 2.5e-3 a token
        if k_.endswith(("right.a2", "mix.w2")):
            weights[k_] = 0.05 * weights[k_]
    folder = write_model(tmp_path / "m", cfg, weights)
    w64 = {k_: v.double() for k_, v in weights.items()}
    rng = np.random.default_rng(5)
    a = [int(t) for t in rng.integers(0, 97, 420)]
    b = list(a)
    b[7] = (b[7] + 50) % 97
    la, lb = P.forward(cfg, w64, a)[-1].numpy(), P.forward(cfg, w64, b)[-1].numpy()
    assert np.abs(la - lb).max() > 0.003, "the test's weights forget too fast to show anything"
    reqs = {"a": a, "b": b}
    for mode, steps in (("whole", traces.whole(reqs)), ("single", traces.bulk_then_single(reqs, tail=380))):
        _replay(folder, "float32", steps, tmp_path / mode, 2 * 448, 16)
        got = traces.collect(steps, tmp_path / mode, 97)
        assert np.abs(got[("a", 419)] - la).max() < 5e-4 and np.abs(got[("b", 419)] - lb).max() < 5e-4
    steps = traces.bulk_then_single(reqs, tail=40)
    _replay(folder, "bfloat16", steps, tmp_path / "bf16", 2 * 448, 16)
    got = traces.collect(steps, tmp_path / "bf16", 97)
    assert np.abs(got[("a", 419)] - la).max() < 0.15 and np.abs(got[("b", 419)] - lb).max() < 0.15


@gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine(shape, dtype):
    """``LLM.generate``: scheduler, prompt portions, continuous batching, graphs in bfloat16.  Every emitted token is
    the plain model's choice at its place, or within rounding of it."""
    import llm_infrence_engine_amd as eng

    name, cfg, folder, reqs, want, noise = shape
    weights = {k: v.double() for k, v in random_weights(cfg, RANKS[name], seed=SEEDS[name]).items()}
    prompts = [toks[:max(1, len(toks) // 3)] for toks in list(reqs.values())[:4]]
    llm = eng.LLM(str(folder), dtype=dtype, block_size=PAGES[name], max_len=128, max_seqs=3, max_prefill_chunk=7)
    outs = llm.generate(prompts, eng.SamplingParams(max_new_tokens=40))
    slack = 2 * F32_ATOL if dtype == "float32" else None
    for p, o in zip(prompts, outs):
        assert len(o.token_ids) == 40 and o.finish_reason == "length"
        logits = P.forward(cfg, weights, p + o.token_ids)[len(p) - 1:-1]
        for t, row in zip(o.token_ids, logits):
            gap = float(row.max() - row[t])
            assert gap <= (slack if slack is not None else BF16_NOISE * max(max(noise.values()), 0.02)), (name, dtype, gap)
    m = llm.engine.runner.manager
    m.check_invariants()
    assert all(g.allocator.num_in_use() == 0 for g in m.groups) and m.num_requests() == 0
    if dtype == "bfloat16":
        # four decode steps to a graph launch, each fed the token the one before chose on the device: the same tokens
        del llm
        several = eng.LLM(str(folder), dtype=dtype, block_size=PAGES[name], max_len=128, max_seqs=3, max_prefill_chunk=7,
                          decode_steps_per_launch=4)
        again = several.generate(prompts, eng.SamplingParams(max_new_tokens=40))
        assert [o.token_ids for o in again] == [o.token_ids for o in outs]


@gpu
def test_command_line_generates(shape):
    import subprocess
    import sys

    from tests.conftest import ROOT

    name, cfg, folder, reqs, want, noise = shape
    r = subprocess.run([sys.executable, "-m", "llm_infrence_engine_amd", "--model", str(folder), "--dtype", "float32",
                        "--prompt-ids", "5,17,3", "--max-new-tokens", "4"], cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
