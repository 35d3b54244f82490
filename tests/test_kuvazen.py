"""The Kuvazen design against the plain implementation in ``tests/plain/kuvazen_plain.py``: every mechanism alone,
then whole models of several small shapes replayed whole, token by token, in portions and in mixed batches (32-bit
and bfloat16 through graphs), and greedy generation through the engine's own entry point."""
import copy
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from tests import traces
from tests.plain import kuvazen_plain as P
from tests.test_gidurax import _Ctx, _in_portions, _paged, _replay, requests_for, write_model

gpu = pytest.mark.gpu


# ================================================================================================ configurations
def dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def gru_layer(width, mlp):
    return {"type": "mingru", "mixer": {"width": width}, "mlp": mlp}


def attention_layer(heads, kv_heads, dim, vdim, scale, size, pool, base, dims, mlp):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                                           "mask": {"size": size, "pool": pool}, "rot": {"base": base, "dims": dims}}, "mlp": mlp}


def config(vocab, width, eps, side, layers, loop=None):
    c = {"architecture": "Kuvazen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if side is not None:
        c["token_side"] = {"dim": side}
    if loop is not None:
        c["loop"] = dict(zip(("start", "stop", "times"), loop))
    return c


# Shapes that differ in every size and in the order of their layers: a looped stretch at the start, in the middle and
# none; attention inside and outside the loop; windows shorter and longer than a page and than a block; blocks of one
# token, of more tokens than the window, of sizes that do not divide a page; groups of one, two and three query heads;
# key and value sizes that differ either way; all, some or none of a key's entries turned; a top of one and of three;
# a layer without a feed-forward; a model without side inputs.
SHAPES = {
    "P": config(211, 96, 1e-5, 8, [
        gru_layer(72, dense(128, 0.8)),
        attention_layer(6, 2, 16, 24, 0.3, 20, 5, 10000.0, 8, moe(40, 5, 2)),
        gru_layer(40, None),
        attention_layer(3, 3, 32, 32, 0.2, 7, 16, 500.0, 32, dense(72, 2.5))], loop=(0, 2, 2)),
    "Q": config(330, 128, 3e-6, 5, [
        attention_layer(4, 1, 24, 40, 0.25, 33, 1, 1000.0, 24, moe(64, 7, 1)),
        gru_layer(150, moe(48, 4, 3)),
        attention_layer(2, 2, 64, 16, 0.125, 16, 8, 100000.0, 0, dense(200, 1.0)),
        gru_layer(96, dense(96, 7.0))], loop=(1, 3, 3)),
    "R": config(150, 64, 1e-6, None, [
        attention_layer(2, 1, 8, 40, 0.4, 1, 3, 50.0, 4, moe(24, 3, 2)),
        gru_layer(33, dense(72, 0.5)),
        attention_layer(6, 3, 16, 16, 0.3, 50, 7, 10000.0, 16, None)]),
}
# heads of 64 and of 32 with values of the same size and pages of 16: in bfloat16 these attentions run on the matrix cores
SHAPES["S"] = config(257, 160, 1e-5, 16, [
    attention_layer(6, 2, 64, 64, 0.11, 40, 12, 10000.0, 32, moe(64, 6, 2)),
    gru_layer(192, dense(192, 1.5)),
    attention_layer(4, 4, 32, 32, 0.18, 16, 16, 10000.0, 32, dense(128, 3.0))], loop=(0, 1, 2))
# sizes that are multiples of nothing much (a width of 100, heads of 10 and 14, five of them), the whole model one looped stretch
SHAPES["T"] = config(77, 100, 1e-5, 3, [
    gru_layer(50, moe(20, 3, 1)),
    attention_layer(5, 5, 10, 14, 0.3, 9, 4, 10000.0, 6, dense(36, 1.2))], loop=(0, 2, 2))
PAGES = {"P": 16, "Q": 8, "R": 4, "S": 16, "T": 16}
# seeds of the shapes' weights: a router's choice is a comparison of floats, and with some weights a token's last chosen
# and first unchosen expert lie closer together than bfloat16 activations can tell apart
SEEDS = {"P": 84, "Q": 92, "R": 81, "S": 98, "T": 82}


def tensor_shapes(cfg):
    """Names and shapes, stated here from the design (not asked of the product)."""
    W, V, n = cfg["width"], cfg["vocab"], len(cfg["layers"])
    out = {"embed": (V, W), "embed.norm": (W,), "final.norm": (W,), "head": (V, W)}
    side = (cfg.get("token_side") or {}).get("dim")
    if side:
        out["side.embed"] = (V, n * side)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = out[p + "ls1"] = (W,)
        if layer["type"] == "mingru":
            C = m["width"]
            out.update({p + "mix.z": (C, W), p + "mix.z.b": (C,), p + "mix.x": (C, W), p + "mix.x.b": (C,), p + "mix.g": (C, W),
                        p + "mix.o": (W, C)})
        else:
            H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({p + "mix.q": (H * D, W), p + "mix.k": (G * D, W), p + "mix.v": (G * E, W), p + "mix.o": (W, H * E)})
        mlp = layer["mlp"]
        if mlp is not None:
            out[p + "norm2"] = out[p + "ls2"] = (W,)
            if mlp["kind"] == "dense":
                out.update({p + "mlp.gate": (mlp["ff"], W), p + "mlp.up": (mlp["ff"], W), p + "mlp.down": (W, mlp["ff"])})
            else:
                F_ = mlp["expert"]["ff"]
                for e in range(mlp["router"]["experts"]):
                    out.update({f"{p}mlp.e{e}.gate": (F_, W), f"{p}mlp.e{e}.up": (F_, W), f"{p}mlp.e{e}.down": (W, F_)})
                out[p + "mlp.router"] = (mlp["router"]["experts"], W)
        if side:
            out.update({p + "side.gate": (side, W), p + "side.proj": (W, side), p + "side.norm": (W,)})
    return out


def random_weights(cfg, seed, dtype=torch.bfloat16):
    """Weights large enough that every mechanism moves the logits: scores of order one, gates of the recurrence between
    slow and fast, products that reach the clamps, routers that spread their choices, layer scales away from one."""
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        r = torch.randn(shape, generator=g)
        if leaf in ("norm1", "norm2") or name in ("final.norm", "embed.norm") or name.endswith("side.norm"):
            t = 1.0 + 0.2 * r
        elif leaf in ("ls1", "ls2"):
            t = 0.6 + 0.3 * r
        elif name.endswith("z.b"):
            t = -1.0 + r
        elif name.endswith("x.b"):
            t = 0.5 * r
        elif name in ("embed", "side.embed"):
            t = r
        elif leaf == "router":
            t = r * (3.0 / math.sqrt(shape[-1]))
        elif name.endswith("side.gate"):
            # the side input is normalised after its gate: where every gate of a token is shut, what is left of it is
            # rounding blown up to full size.  Gates of order one keep some of them open
            t = r * (0.03 / math.sqrt(shape[-1]))
        elif ".mlp.e" in name:
            # a token whose two best experts tie may run another expert in bfloat16 than in 64-bit; small experts keep
            # what such a token does to the logits within the bound that rounding sets (32-bit sees them exactly)
            t = r * ((0.3 if leaf == "down" else 1.0) / math.sqrt(shape[-1]))
        else:
            t = r * (2.0 / math.sqrt(shape[-1]))
        w[name] = t.to(dtype).contiguous()
    return w


# ================================================================================================ the oracle's own pins
def test_plain_pieces_against_library_routines():
    torch.manual_seed(0)
    x = torch.randn(9, 6, dtype=torch.float64)
    b = torch.randn(6, dtype=torch.float64)
    assert torch.allclose(P.layer_norm(x, b, 1e-5), F.layer_norm(x, (6,), b, None, 1e-5), atol=1e-12)
    assert torch.allclose(P.rms(x, 1e-5) * b, F.rms_norm(x, (6,), b, 1e-5), atol=1e-12)
    assert torch.allclose(P.gelu_tanh(x), F.gelu(x, approximate="tanh"), atol=1e-12)
    assert torch.allclose(P.silu(x), F.silu(x), atol=1e-12)
    # turning neighbours is a complex multiplication
    v = torch.randn(5, 2, 8, dtype=torch.float64)
    pos = torch.tensor([0, 3, 4, 9, 100])
    got = P.turn_pairs(v, pos, 100.0, 6)
    z = torch.view_as_complex(v[..., :6].reshape(5, 2, 3, 2).contiguous())
    ang = pos.double()[:, None] * 100.0 ** (-2.0 * torch.arange(3, dtype=torch.float64) / 6)
    want = torch.view_as_real(z * torch.polar(torch.ones_like(ang), ang)[:, None, :]).reshape(5, 2, 6)
    assert torch.allclose(got[..., :6], want, atol=1e-12) and torch.equal(got[..., 6:], v[..., 6:])
    assert torch.allclose(P.turn_pairs(got, pos, 100.0, 6, sign=-1.0), v, atol=1e-12)
    # a window as long as the sequence sees no block and is the library's causal attention
    q, k, val = (torch.randn(7, 2, 5, dtype=torch.float64) for _ in range(3))
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), val.transpose(0, 1), is_causal=True, scale=0.3)
    assert torch.allclose(P.windowed_pooled_attention(q, k, val, 0.3, 7, 2), ref.transpose(0, 1), atol=1e-12)


def test_plain_window_and_blocks_at_their_edges():
    # size 4, blocks of 3: position 6 sees tokens 3..6 and block 0 (tokens 0..2, last one 4 back); position 5 sees
    # tokens 2..5 and no block (token 2 is still in the window), so tokens 0 and 1 are not seen at all
    assert P.visible(6, 4, 3) == (3, 1) and P.visible(5, 4, 3) == (2, 0) and P.visible(0, 4, 3) == (0, 0)
    assert P.visible(9, 4, 3) == (6, 2) and P.visible(8, 4, 3) == (5, 1)
    assert P.visible(5, 1, 1) == (5, 5)            # a window of the token itself, every older token its own block
    T, D = 10, 4
    q = torch.zeros(T, 1, D, dtype=torch.float64)
    k = torch.zeros(T, 1, D, dtype=torch.float64)
    v = torch.arange(T, dtype=torch.float64)[:, None, None].repeat(1, 1, 2)
    out = P.windowed_pooled_attention(q, k, v, 1.0, 4, 3)
    # equal scores: the mean over what is seen, a block counting once with the mean of its values
    assert torch.allclose(out[6, 0], torch.full((2,), (1.0 + 3 + 4 + 5 + 6) / 5, dtype=torch.float64))
    assert torch.allclose(out[5, 0], torch.full((2,), (2.0 + 3 + 4 + 5) / 4, dtype=torch.float64))
    assert torch.allclose(out[9, 0], torch.full((2,), (1.0 + 4 + 6 + 7 + 8 + 9) / 6, dtype=torch.float64))


def test_plain_recurrence_router_and_order():
    # constant gates: a geometric series towards the candidate
    T, C = 7, 3
    z = torch.full((T, C), 0.25, dtype=torch.float64)
    c = torch.tensor([1.0, -2.0, 0.5], dtype=torch.float64).repeat(T, 1)
    S, last = P.mingru_recurrence(z, c)
    assert torch.allclose(last, c[0] * (1.0 - 0.75 ** T), atol=1e-12) and torch.allclose(S[0], 0.25 * c[0])
    u = torch.tensor([-1.0, 0.0, 2.0], dtype=torch.float64)
    assert torch.allclose(P.mingru_candidate(u), torch.tensor([1 / (1 + math.e), 0.5, 2.5], dtype=torch.float64))
    # sigmoid scores, not renormalised; the weight scales what the expert reads
    h = torch.eye(3, dtype=torch.float64)[:1] * 2.0
    wr = torch.tensor([[1.0, 0, 0], [0.5, 0, 0], [-1.0, 0, 0]], dtype=torch.float64)
    chosen, weights = P.route(h, wr, 2)
    assert chosen[0].tolist() == [0, 1]
    assert torch.allclose(weights[0], torch.sigmoid(torch.tensor([2.0, 1.0], dtype=torch.float64)))
    g = torch.randn(4, 3, dtype=torch.float64)
    up = torch.randn(4, 3, dtype=torch.float64)
    down = torch.randn(3, 4, dtype=torch.float64)
    w = {"m.router": wr[:1], "m.e0.gate": g, "m.e0.up": up, "m.e0.down": down}
    s = torch.sigmoid(torch.tensor(2.0, dtype=torch.float64))
    assert torch.allclose(P.moe_ff(h, w, "m.", {"router": {"experts": 1, "top": 1}}), P.expert_ff(s * h, g, up, down))
    # the clamps: a gate above the limit is cut, an up below -limit too
    one = torch.ones(1, 1, dtype=torch.float64)
    y = P.clamped_gated_ff(one, 5.0 * one, -9.0 * one, one, 2.0)
    assert torch.allclose(y, 2.0 * torch.sigmoid(torch.tensor(3.404, dtype=torch.float64)) * (-2.0 + 1.0) * one)
    assert P.layer_order({"layers": [0] * 5, "loop": {"start": 1, "stop": 3, "times": 3}}) == [0, 1, 2, 1, 2, 1, 2, 3, 4]
    assert P.layer_order({"layers": [0, 0]}) == [0, 1]


def test_config_reads_every_size_and_refuses_what_it_does_not_know():
    from llm_infrence_engine_amd.config import ConfigError, config_from_dict
    from llm_infrence_engine_amd.parts.model import Model

    for name, cfg in SHAPES.items():
        c = config_from_dict(copy.deepcopy(cfg))
        assert type(c).__name__ == "KuvazenConfig" and c.to_dict() == cfg
        model = Model(c.to_spec())
        assert {s.name: tuple(s.shape) for s in model.tensor_specs()} == tensor_shapes(cfg)
        order = P.layer_order(cfg)
        assert [r.layer for r in model.spec.order] == order
        for i, (kv, state, _) in zip(order, model.run_needs()):
            m = cfg["layers"][i]["mixer"]
            if cfg["layers"][i]["type"] == "attention":
                tokens, blocks = kv
                assert state is None and tokens.stride == 1 and tokens.window >= max(m["mask"]["size"], m["mask"]["pool"])
                assert blocks.stride == m["mask"]["pool"] and blocks.window is None
                for need in kv:
                    assert [(t.name, t.heads, t.width) for t in need.tensors] == [("k", m["kv_heads"], m["dim"]), ("v", m["kv_heads"], m["vdim"])]
            else:
                assert kv is None and state.shape == (m["width"],) and state.dtype == torch.float32
        assert model.graph_safe() is True
    for change in (lambda c: c["layers"][0].__setitem__("type", "something_else"),
                   lambda c: c["layers"][1]["mixer"].pop("vdim"),
                   lambda c: c["layers"][1]["mixer"]["mask"].pop("pool"),
                   lambda c: c["layers"][1]["mixer"]["rot"].__setitem__("dims", 7),
                   lambda c: c["layers"][0]["mlp"].pop("limit"),
                   lambda c: c.__setitem__("loop", {"start": 2, "stop": 2, "times": 2}),
                   lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 99)):
        bad = copy.deepcopy(SHAPES["P"])
        change(bad)
        with pytest.raises(ConfigError):
            config_from_dict(bad)


def test_plain_model_prefix_property():
    """The plain model is causal: the logits of a prefix do not change when tokens follow."""
    cfg = SHAPES["R"]
    w = {k: v.double() for k, v in random_weights(cfg, 5).items()}
    toks = requests_for(cfg["vocab"], [23], 1)["r0"]
    full = P.forward(cfg, w, toks)
    assert torch.allclose(P.forward(cfg, w, toks[:9]), full[:9], atol=1e-9)


def test_pages_of_one_entry_per_block():
    """The cache manager with a group that keeps an entry per whole block of tokens beside a windowed group: pages
    asked for, what fits, rows and pages given back."""
    from llm_infrence_engine_amd.cache.manager import CacheLayout, CacheManager
    from llm_infrence_engine_amd.parts.base import CacheNeed, PageTensor

    t = (PageTensor("k", 2, 8), PageTensor("v", 2, 8))
    needs = (CacheNeed(t, window=10), CacheNeed(t, stride=5))
    lay = CacheLayout([(needs, None, None), (None, None, None), (needs, None, None)])
    assert lay.run_group == [0, None, 0] and lay.run_more == [[(1, 0)], [], [(1, 1)]]
    assert [k.stride for k in lay.group_keys] == [1, 5]
    m = CacheManager(lay, page_size=4, num_pages=[12, 3], max_requests=2, max_len=48)
    m.add("a")
    assert m.pages_to_grow("a", 19) == [5, 1] and m.pages_to_grow("a", 20) == [5, 1] and m.pages_to_grow("a", 25) == [7, 2]
    assert m.tokens_that_fit("a") == 48                       # 12 pages of tokens; 3 pages of blocks reach 64 tokens
    m.grow("a", 23)
    m.advance("a", 23)
    assert [len(p) for p in m.pages_held("a")] == [3, 1]      # the window gave back the first three of six token pages
    assert m.pages_to_grow("a", 40) == [4, 1]
    m.add("b")
    m.grow("b", 32)                                           # eight token pages and two pages of blocks
    assert m.num_free_pages() == [1, 0]
    m.check_invariants()
    with pytest.raises(Exception):
        m.grow("a", 40)
    m.free("b")
    m.grow("a", 40)
    m.advance("a", 40)
    assert [len(p) for p in m.pages_held("a")] == [3, 2]
    m.free("a")
    m.check_invariants()
    assert all(g.allocator.num_in_use() == 0 for g in m.groups)


# ================================================================================================ kernels alone (GPU)
@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H", [96, 130, 1024])
def test_layer_norm_sums_and_rows(dtype, H):
    from llm_infrence_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(H)
    N = 13
    x = (3.0 * torch.randn(N, H, generator=g) + 2.0)
    y = torch.randn(N, H, generator=g).to(dtype)
    s = 0.5 + torch.rand(H, generator=g)
    w = 1.0 + 0.2 * torch.randn(H, generator=g)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    xd = x.cuda()
    out = ops.layer_norm(xd, w.cuda(), 1e-5, torch.empty(N, H, dtype=dtype, device="cuda"), delta=y.cuda(), delta_scale=s.cuda())
    total = x.double() + s.double() * y.double()
    assert (xd.cpu().double() - total).abs().max() < 1e-5
    assert (out.cpu().double() - P.layer_norm(total, w.double(), 1e-5)).abs().max() < tol
    rows = torch.tensor([4, 0, 12, 4], dtype=torch.int32, device="cuda")
    xd2 = x.cuda()
    got = ops.layer_norm(xd2, w.cuda(), 1e-5, torch.empty(4, H, dtype=dtype, device="cuda"), delta=y.cuda(), rows=rows, write_back=False)
    assert torch.equal(xd2.cpu(), x)
    assert (got.cpu().double() - P.layer_norm((x.double() + y.double())[rows.cpu().long()], w.double(), 1e-5)).abs().max() < tol
    ops.layer_norm(xd2, w.cuda(), 1e-5, xd2)             # in place
    assert (xd2.cpu().double() - P.layer_norm(x.double(), w.double(), 1e-5)).abs().max() < 1e-5
    xd3 = x.cuda()
    ops.layer_norm(xd3, None, 0.0, None, delta=y.cuda(), delta_scale=s.cuda())       # the scaled sum alone
    assert (xd3.cpu().double() - total).abs().max() < 1e-5


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,d,parts,N", [(96, 8, 4, 11), (130, 5, 3, 11), (512, 1, 2, 3), (64, 33, 1, 11), (256, 64, 2, 200)])
def test_token_side_input(dtype, H, d, parts, N):
    """Every layer's slice of the narrow table, with the scaled sum that is still due riding along."""
    from llm_infrence_engine_amd.parts.base import Runtime
    from llm_infrence_engine_amd.parts.side import TokenSide

    g = torch.Generator().manual_seed(H + d)
    V = 50
    x = 2.0 * torch.randn(N, H, generator=g)
    y = torch.randn(N, H, generator=g).to(dtype)
    s = 0.5 + torch.rand(H, generator=g)
    w = {"side.embed": torch.randn(V, parts * d, generator=g).to(dtype), "p.gate": (0.3 * torch.randn(d, H, generator=g) / math.sqrt(H)).to(dtype),
         "p.proj": torch.randn(H, d, generator=g).to(dtype), "p.norm": 1.0 + 0.2 * torch.randn(H, generator=g)}
    ids = torch.randint(0, V, (N,), generator=g)
    ctx = _Ctx([N], [0])
    ctx.token_ids = ids.int().cuda()
    for part in range(parts):
        total = x.double() + s.double() * y.double()
        want = total + P.side_input(total, ids, part, {k_: v_.double() for k_, v_ in w.items()}, "p.", d, 1e-6)
        side = TokenSide("p.", H, V, d, part, parts, 1e-6)
        side.load(lambda spec: (w[spec.name].float() if spec.role == "norm" else w[spec.name].to(dtype)).cuda(), Runtime(torch.device("cuda"), dtype))
        xd = x.cuda()
        side.forward(xd, ctx, delta=y.cuda(), delta_scale=s.cuda())
        assert (xd.cpu().double() - want).abs().max() < (2e-5 if dtype == torch.float32 else 3e-2) * max(1.0, float(want.abs().max()))
        xd = x.cuda()
        side.forward(xd, ctx)                  # nothing due
        want = x.double() + P.side_input(x.double(), ids, part, {k_: v_.double() for k_, v_ in w.items()}, "p.", d, 1e-6)
        assert (xd.cpu().double() - want).abs().max() < (2e-5 if dtype == torch.float32 else 3e-2) * max(1.0, float(want.abs().max()))


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("C", [72, 64, 33, 300])
def test_mingru_in_portions_and_batches(dtype, C):
    """Three sequences from slots in no order, in portions of unequal sizes (one token, two, more than the kernel
    holds in registers, more than a block walks at once), batched together, against the whole recurrence."""
    from llm_infrence_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(C)
    lens = [150, 41, 9]
    cuts = [[70, 1, 1, 2, 76], [3, 30, 8], [1, 1, 7]]
    slots = [2, 0, 3]
    zxg = [(1.5 * torch.randn(n, 3 * C, generator=g)).to(dtype) for n in lens]
    bz, bx = torch.randn(C, generator=g) - 1.0, torch.randn(C, generator=g)
    want = []
    for t in zxg:
        a = t.double()
        S, _ = P.mingru_recurrence(P.sigmoid(a[:, :C] + bz.double()), P.mingru_candidate(a[:, C:2 * C] + bx.double()))
        want.append(S * P.silu(a[:, 2 * C:]))
    state = torch.full((5, C), 7.0, device="cuda")
    state[torch.tensor(slots)] = 0.0

    def run(live, at, q_lens, ctx):
        rows = torch.cat([zxg[r][at[r]:at[r] + n] for r, n in zip(live, q_lens)]).cuda()
        return ops.mingru_scan(rows, bz.cuda(), bx.cuda(), state, ctx, torch.empty(rows.shape[0], C, dtype=dtype, device="cuda"))

    got = _in_portions(lens, cuts, slots, run)
    for a, b in zip(got, want):
        assert (a.double() - b).abs().max() < (2e-5 if dtype == torch.float32 else 3e-2) * max(1.0, float(b.abs().max()))
    assert torch.equal(state[1].cpu(), torch.full((C,), 7.0)) and torch.equal(state[4].cpu(), torch.full((C,), 7.0))


class _KV:
    def __init__(self, k, v, table, rows, slots, stride=1, store=True, flipped=False):
        self.pages, self.transposed = {"k": k, "v": v}, {"k": False, "v": flipped}
        self.block_table, self.table_rows, self.slot_mapping, self.store, self.stride = table, rows, slots, store, stride


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,E,page,size,pool,dims", [
    (6, 2, 16, 24, 4, 20, 5, 8), (4, 1, 64, 64, 16, 96, 12, 64), (3, 3, 32, 8, 8, 7, 16, 0), (2, 1, 6, 10, 4, 1, 1, 6),
    (2, 2, 40, 56, 16, 33, 3, 32), (8, 2, 128, 128, 16, 16, 16, 64), (4, 2, 32, 32, 16, 1, 1, 32), (2, 1, 64, 64, 16, 5, 3, 0),
    (3, 1, 48, 48, 16, 70, 9, 48)])
def test_window_and_pooled_blocks_through_the_pages(dtype, H, G, D, E, page, size, pool, dims):
    """One sequence of 230 tokens stored in three steps (the cuts fall inside a page, a block and the window) into pages
    in no order, then the last 60 queries.  For one query the key just inside the window and, for another, every key of
    the block that has just come into sight are made loud, so that a window one token off, a block seen one token early
    or late, or a block's mean over the wrong tokens shows; stale pages hold large values."""
    from llm_infrence_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(D + E + size)
    T, Tq, base = 230, 60, 1000.0
    q = torch.randn(T, H, D, generator=g).to(dtype)
    k = torch.randn(T, G, D, generator=g).to(dtype)
    v = torch.randn(T, G, E, generator=g).to(dtype)
    scale = 0.7 / math.sqrt(D)
    pos = torch.arange(T)
    i1, i2 = T - 9, T - 23
    rep = H // G
    # loud, as the cache will hold them: the rotation keeps q . k for equal positions, so set them before turning
    qt = P.turn_pairs(q.double(), pos, base, dims)
    kt = P.turn_pairs(k.double(), pos, base, dims)
    j_in = i1 - size + 1
    if j_in >= 0:
        kt[j_in, 0] = 5.0 * qt[i1, 0] / qt[i1, 0].norm()
    nb2 = (i2 - size + 1) // pool
    if nb2 > 0:
        kt[(nb2 - 1) * pool: nb2 * pool, 0] = 5.0 * qt[i2, 0] / qt[i2, 0].norm()
    kt = kt.to(dtype).double()
    vt = P.turn_pairs(v.double(), pos, base, E).to(dtype).double()
    nb = T // pool
    k_mean = kt[: nb * pool].reshape(nb, pool, G, D).mean(1).to(dtype).double()
    v_mean = vt[: nb * pool].reshape(nb, pool, G, E).mean(1).to(dtype).double()
    want = P.windowed_pooled_attention(qt.to(dtype).double(), kt.repeat_interleave(rep, 1), vt.repeat_interleave(rep, 1), scale, size, pool,
                                       k_mean.repeat_interleave(rep, 1), v_mean.repeat_interleave(rep, 1))
    want = P.turn_pairs(want, pos, base, E, sign=-1.0)[T - Tq:]
    # keys made loud after the turn cannot come from a projection: write the turned keys back through the inverse turn
    k_src = P.turn_pairs(kt, pos, base, dims, sign=-1.0)
    # pages in no order for tokens and for blocks; the kernels store
    n_pages, n_bpages = -(-T // page), -(-max(nb, 1) // page)
    order = [int(x) for x in np.random.default_rng(1).permutation(np.arange(1, 1 + n_pages))]
    border = [int(x) for x in np.random.default_rng(2).permutation(np.arange(1, 1 + n_bpages))]
    for flipped in (False, True):
        _through_the_pages(dtype, H, G, D, E, page, size, pool, dims, T, Tq, base, q, k_src, v, scale, want, order, border, nb, flipped,
                           blind_check=(j_in, i1, qt, kt, vt, rep, pos))


def _through_the_pages(dtype, H, G, D, E, page, size, pool, dims, T, Tq, base, q, k_src, v, scale, want, order, border, nb, flipped,
                       blind_check):
    from llm_infrence_engine_amd.kernels import ops

    j_in, i1, qt, kt, vt, rep, pos = blind_check
    k_pages, v_pages, table = _paged(torch.zeros(T, G, D), torch.zeros(T, G, E), page, order, dtype, flipped)
    pk_pages, pv_pages, ptable = _paged(torch.zeros(max(nb, 1), G, D), torch.zeros(max(nb, 1), G, E), page, border, dtype, flipped)
    k_pages.fill_(50.0), v_pages.fill_(50.0), pk_pages.fill_(50.0), pv_pages.fill_(50.0)
    if ptable.shape[1] < table.shape[1]:
        ptable = torch.cat([ptable, torch.zeros(2, table.shape[1] - ptable.shape[1], dtype=torch.int32, device="cuda")], 1)
    else:
        table = torch.cat([table, torch.zeros(2, ptable.shape[1] - table.shape[1], dtype=torch.int32, device="cuda")], 1)
    rows = torch.tensor([1], dtype=torch.int32, device="cuda")
    f = lambda n, th: (th ** (-torch.arange(0, n, 2, dtype=torch.float64) / max(1, n))).float().cuda()
    inv_freq, inv_freq_v = f(dims, base), f(E, base)
    outs = []
    on_cores = (flipped and dtype == torch.bfloat16 and D == E and ops.attention_mfma_supported(D, page))
    for a, b in ((0, 101), (101, T - Tq), (T - Tq, T)):
        n = b - a
        ctx = _Ctx([n], [0], [a])
        p_ = torch.arange(a, b)
        slots = torch.tensor([order[int(t) // page] * page + int(t) % page for t in p_], dtype=torch.int32, device="cuda")
        bslots = torch.tensor([border[((int(t) + 1) // pool - 1) // page] * page + ((int(t) + 1) // pool - 1) % page
                               if (int(t) + 1) % pool == 0 else -1 for t in p_], dtype=torch.int32, device="cuda")
        qkv = torch.cat([q[a:b].reshape(n, H * D).double(), k_src[a:b].reshape(n, G * D), v[a:b].reshape(n, G * E).double()], 1).to(dtype).cuda()
        kv = _KV(k_pages, v_pages, table, rows, slots, flipped=flipped)
        pooled = _KV(pk_pages, pv_pages, ptable, rows, bslots, pool, flipped=flipped)
        ops.pairs_rotate_store(qkv, H, G, D, E, dims, ctx.positions, inv_freq, inv_freq_v, kv)
        ops.pool_store(kv, pooled, ctx, pool)
        out = torch.empty(n, H * E, dtype=dtype, device="cuda")
        ops.pooled_attention(qkv, kv, pooled, ctx, out, H, scale, size, pool, inv_freq_v, matrix_cores=True if on_cores else None)
        outs.append(out.cpu())
        if on_cores:      # the same step on the vector ALUs
            again = torch.empty(n, H * E, dtype=dtype, device="cuda")
            ops.pooled_attention(qkv, kv, pooled, ctx, again, H, scale, size, pool, inv_freq_v, matrix_cores=False)
            assert (again.float() - out.float()).abs().max() < 6e-2
    err = (outs[-1].double().reshape(Tq, H, E) - want).abs().max()
    assert err < (1e-4 if dtype == torch.float32 else 6e-2), (flipped, float(err))
    if on_cores:
        # single tokens after it, two requests' worth of columns in one step: the narrow tiles of a decode step
        for t in (T - 3, T - 1):
            ctx = _Ctx([1], [0], [t])
            qkv = torch.cat([q[t:t + 1].reshape(1, H * D).double(), k_src[t:t + 1].reshape(1, G * D), v[t:t + 1].reshape(1, G * E).double()], 1).to(dtype).cuda()
            kv = _KV(k_pages, v_pages, table, rows, None, flipped=flipped, store=False)
            pooled = _KV(pk_pages, pv_pages, ptable, rows, None, pool, flipped=flipped, store=False)
            ops.pairs_rotate_store(qkv, H, G, D, E, dims, ctx.positions, inv_freq, inv_freq_v, kv)
            out = torch.empty(1, H * E, dtype=dtype, device="cuda")
            ops.pooled_attention(qkv, kv, pooled, ctx, out, H, scale, size, pool, inv_freq_v, matrix_cores=True)
            err = (out.cpu().double().reshape(H, E) - want[t - (T - Tq)]).abs().max()
            assert err < 6e-2, (t, float(err))
    if dtype == torch.float32 and not flipped:          # what the loud keys are there for
        blind = P.windowed_pooled_attention(qt, kt.repeat_interleave(rep, 1), vt.repeat_interleave(rep, 1), scale, max(1, size - 1), pool)
        if j_in >= 0 and size > 1:
            assert (P.turn_pairs(blind, pos, base, E, sign=-1.0)[i1] - want[i1 - (T - Tq)]).abs().max() > 0.05


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E,top,F_,W,N", [(5, 2, 40, 72, 37), (7, 1, 64, 96, 37), (4, 3, 48, 64, 5), (12, 1, 64, 128, 300), (3, 3, 24, 40, 1)])
def test_gated_experts_with_the_weight_on_their_input(dtype, E, top, F_, W, N):
    from llm_infrence_engine_amd.kernels import ops
    from llm_infrence_engine_amd.parts.base import Runtime
    from llm_infrence_engine_amd.parts.experts import RoutedExperts

    g = torch.Generator().manual_seed(E * 100 + top)
    w = {"m.router": (torch.randn(E, W, generator=g) * 3.0 / math.sqrt(W)).to(dtype)}
    for e in range(E):
        w[f"m.e{e}.gate"] = (torch.randn(F_, W, generator=g) * 2.0 / math.sqrt(W)).to(dtype)
        w[f"m.e{e}.up"] = (torch.randn(F_, W, generator=g) * 2.0 / math.sqrt(W)).to(dtype)
        w[f"m.e{e}.down"] = (torch.randn(W, F_, generator=g) * 2.0 / math.sqrt(F_)).to(dtype)
    h = torch.randn(N, W, generator=g).to(dtype)
    w64 = {k_: v_.double() for k_, v_ in w.items()}
    mlp = {"router": {"experts": E, "top": top}}
    want = P.moe_ff(h.double(), w64, "m.", mlp)
    part = RoutedExperts("m.", W, F_, E, top, activation="swiglu", scores="sigmoid", correction=False, weight_on="input")
    assert sorted(s.name for s in part.tensor_specs()) == sorted(w)
    part.load(lambda s: w[s.name].to(dtype).cuda(), Runtime(torch.device("cuda"), dtype))
    got = part.forward(h.cuda(), None)
    assert got.dtype == torch.float32
    assert (got.cpu().double() - want).abs().max() < (2e-5 if dtype == torch.float32 else 6e-2) * max(1.0, float(want.abs().max()) / 4)
    chosen, weights = P.route(h.double(), w64["m.router"], top)
    ids, wts = ops.moe_route((h.double() @ w64["m.router"].T).float().cuda(), None, top, scores="sigmoid")
    assert torch.equal(ids.cpu().long().sort(1).values, chosen.sort(1).values)
    assert torch.allclose(wts.cpu().double().sort(1).values, weights.sort(1).values, atol=1e-6)


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_clamped_gated_feed_forward(dtype):
    from llm_infrence_engine_amd.parts.base import Runtime
    from llm_infrence_engine_amd.parts.feed_forward import ClampedGLU

    g = torch.Generator().manual_seed(3)
    W, I, N = 72, 100, 70
    w = {"m.gate": (torch.randn(I, W, generator=g) * 2.0 / math.sqrt(W)).to(dtype), "m.up": (torch.randn(I, W, generator=g) * 2.0 / math.sqrt(W)).to(dtype),
         "m.down": (torch.randn(W, I, generator=g) / math.sqrt(I)).to(dtype)}
    h = torch.randn(N, W, generator=g).to(dtype)
    for limit in (0.5, 1.0, 7.0):
        want = P.clamped_gated_ff(h.double(), w["m.gate"].double(), w["m.up"].double(), w["m.down"].double(), limit)
        part = ClampedGLU("m.", W, I, limit)
        part.load(lambda s: w[s.name].cuda(), Runtime(torch.device("cuda"), dtype))
        for rows in (N, 3):
            got = part.forward(h[:rows].cuda(), None)
            # bfloat16 results of size 8 are 0.03 apart
            assert (got.cpu().double() - want[:rows]).abs().max() < (2e-5 if dtype == torch.float32 else 2e-2) * max(1.0, float(want.abs().max()))
    a, b = P.clamped_gated_ff(h.double(), w["m.gate"].double(), w["m.up"].double(), w["m.down"].double(), 0.5), \
        P.clamped_gated_ff(h.double(), w["m.gate"].double(), w["m.up"].double(), w["m.down"].double(), 7.0)
    assert (a - b).abs().max() > 0.1             # the clamps bite in this test


# ================================================================================================ whole models (GPU)
F32_ATOL = 2e-3
BF16_NOISE = 3.0


def rounded_forward(cfg, w, toks):
    exact = P.forward(cfg, w, toks)
    return exact, float((P.forward(cfg, w, toks, act_dtype=torch.bfloat16) - exact).abs().max())


@pytest.fixture(scope="module", params=list(SHAPES))
def shape(request, tmp_path_factory):
    name = request.param
    cfg = SHAPES[name]
    weights = random_weights(cfg, seed=SEEDS[name])
    folder = write_model(tmp_path_factory.mktemp("kuvazen" + name), cfg, weights)
    lengths = {"P": [5, 61, 2, 130, 33, 48], "Q": [1, 9, 90, 47, 110, 64], "R": [3, 26, 70, 17, 2, 41, 60, 33],
               "S": [70, 3, 140, 50, 97, 33], "T": [40, 2, 90, 17, 66]}[name]
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
    """An engine with a single request row and pages for one request: every request gets the state slot and the pages
    (of tokens and of blocks) its predecessor left, in portions, and must start from zero state and see none of the
    old keys or blocks."""
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
@pytest.mark.parametrize("kind", ["mingru", "attention"])
def test_far_token_reaches_the_end(tmp_path, kind):
    """A token 400 places back still moves the last logits, through the recurrence's state (gates made slow) or through
    the pooled block it fell into, in the plain model and equally in the engine, whole and decoded token by token (the
    decoded stretch fills many blocks and pushes many tokens out of the window)."""
    mixer = {"mingru": gru_layer(48, dense(64, 2.0)),
             "attention": attention_layer(2, 1, 16, 24, 0.25, 4, 8, 10000.0, 16, dense(64, 2.0))}[kind]
    cfg = config(97, 64, 1e-5, 4, [mixer])
    weights = random_weights(cfg, seed=1)
    for k_ in weights:
        if k_.endswith("z.b"):
            weights[k_] = torch.full_like(weights[k_], -6.0)         # a memory of some hundred tokens
        if k_.endswith("mix.z"):
            weights[k_] = 0.1 * weights[k_]
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
    # a model of one kind of layer alone (no state, or no pages at all) through the graphs of the bfloat16 path
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
    weights = {k: v.double() for k, v in random_weights(cfg, seed=SEEDS[name]).items()}
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
        # four decode steps to a graph launch, each fed the token the one before chose on the device (the slots of the
        # blocks' pages are worked out on the device too): the same tokens
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
