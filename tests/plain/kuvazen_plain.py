"""Plain, slow, whole-sequence Kuvazen decoder used only as the test oracle.

One function per mechanism, written from the design's equations in this file's own notation; no cache, no batching,
token-by-token loops where the design is a recurrence, position-by-position loops in attention, and no import from
the product package.  Everything runs in one floating type chosen by the caller (float64 by default).

Notation: a sequence is T tokens at positions 0..T-1; W is the model's width; every linear map is stored [out, in]
and applied as y = x @ M.T;  LN(x, w) = (x - mean x) / sqrt(var x + eps) * w (no bias);  RMS(x) = x / sqrt(mean x^2 + eps).

The design
* x = LN(embed[token], embed.norm)
* a stretch of layers [start, stop) is walked ``times`` times with the same weights, every walk with its own memory
* a layer i:  x <- x + ls1 * mixer(LN(x, norm1));  x <- x + ls2 * ff(LN(x, norm2))  (the second line only with a
  feed-forward);  then the token's own side input:  c = side.embed[token, i*d:(i+1)*d],
  y = side.proj (gelu_tanh(side.gate x) * c),  x <- x + RMS(y) * side.norm
* mixers: ``mingru`` (a gated recurrence per channel whose gates read the current token only) and ``attention``
  (grouped heads, neighbouring entries rotated by the position, values rotated too and the result turned back, a
  sliding window with means over blocks of older tokens beside it)
* feed-forward: a clamped gated one, or routed experts whose weights scale the expert's input
* logits = head LN(x, final.norm)
"""
from __future__ import annotations

import json
import math
from pathlib import Path

import torch
from safetensors import safe_open


# --------------------------------------------------------------------------- files
def read_config(model_dir) -> dict:
    return json.loads((Path(model_dir) / "config.json").read_text())


def read_weights(model_dir, dtype=torch.float64) -> dict:
    out = {}
    for f in sorted(Path(model_dir).glob("*.safetensors")):
        with safe_open(str(f), framework="pt") as fh:
            for name in fh.keys():
                out[name] = fh.get_tensor(name).to(dtype)
    return out


# --------------------------------------------------------------------------- small pieces
def same(x):
    return x


def rounder(act_dtype):
    """x as an engine that stores activations in ``act_dtype`` would hold it (None: exact); applied to what products
    and activations leave, never to the residual stream, norms, scores, gates of the recurrence or states."""
    return same if act_dtype is None else (lambda x: x.to(act_dtype).to(x.dtype))


def layer_norm(x, w, eps):
    mu = x.mean(dim=-1, keepdim=True)
    dev = x - mu
    return dev / torch.sqrt((dev * dev).mean(dim=-1, keepdim=True) + eps) * w


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# --------------------------------------------------------------------------- mixer: minGRU
def mingru_candidate(u):
    """u + 1/2 where u >= 0, sigmoid(u) below: continuous, positive, linear on the right."""
    return torch.where(u >= 0, u + 0.5, sigmoid(u))


def mingru_recurrence(z, c, S0=None):
    """z, c [T, C]:  S_t = (1 - z_t) S_(t-1) + z_t c_t, channel by channel, S_(-1) = 0.  Returns all S_t and the last."""
    T, C = z.shape
    S = torch.zeros(C, dtype=z.dtype) if S0 is None else S0.clone()
    out = torch.zeros(T, C, dtype=z.dtype)
    for t in range(T):
        S = (1.0 - z[t]) * S + z[t] * c[t]
        out[t] = S
    return out, S


def mingru_mixer(h, w, p, rd=same):
    z = sigmoid(rd(h @ w[p + "z"].T + w[p + "z.b"]))
    u = rd(h @ w[p + "x"].T + w[p + "x.b"])
    S, _ = mingru_recurrence(z, mingru_candidate(u))
    gate = silu(rd(h @ w[p + "g"].T))
    return rd(rd(S * gate) @ w[p + "o"].T)


# --------------------------------------------------------------------------- mixer: attention
def turn_pairs(x, pos, base: float, dims: int, sign: float = 1.0):
    """x [T, heads, D]: of every head's first ``dims`` entries the neighbours (2i, 2i + 1) are turned by the angle
    sign * pos * base^(-2i/dims); the rest stay."""
    if dims == 0:
        return x
    i = torch.arange(dims // 2, dtype=torch.float64)
    ang = sign * pos.to(torch.float64)[:, None] * base ** (-2.0 * i / dims)          # [T, dims/2]
    cos, sin = torch.cos(ang).to(x.dtype)[:, None, :], torch.sin(ang).to(x.dtype)[:, None, :]
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = a * cos - b * sin
    out[..., 1:dims:2] = b * cos + a * sin
    return out


def visible(i: int, size: int, pool: int):
    """What position i sees: (first token of its window, number of whole blocks of ``pool`` tokens before the window
    that are seen).  Tokens i - size + 1 .. i are in the window; block b = [b pool, (b + 1) pool) is seen once its last
    token is at least ``size`` back: (b + 1) pool - 1 <= i - size."""
    lo = max(0, i - size + 1)
    n_blocks = max(0, (i - size + 1) // pool)
    return lo, n_blocks


def windowed_pooled_attention(q, k, v, scale: float, size: int, pool: int, k_mean=None, v_mean=None):
    """q [T, H, D], k [T, H, D], v [T, H, E]: position i attends to the tokens of its window and to one key and value
    per seen block, the plain means of the block's keys and of its values; one softmax over both kinds."""
    T, H, _ = q.shape
    nb = T // pool
    if k_mean is None:
        k_mean = k[: nb * pool].reshape(nb, pool, H, -1).mean(dim=1)
        v_mean = v[: nb * pool].reshape(nb, pool, H, -1).mean(dim=1)
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for i in range(T):
        lo, n = visible(i, size, pool)
        for h in range(H):
            keys = torch.cat([k_mean[:n, h], k[lo: i + 1, h]])
            vals = torch.cat([v_mean[:n, h], v[lo: i + 1, h]])
            s = (keys @ q[i, h]) * scale
            e = torch.exp(s - s.max())
            out[i, h] = (e / e.sum()) @ vals
    return out


def attention_mixer(h, w, p, m, rd=same, pos0: int = 0):
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    base, dims = float(m["rot"]["base"]), int(m["rot"]["dims"])
    pos = torch.arange(pos0, pos0 + T)
    q = rd(turn_pairs(rd(h @ w[p + "q"].T).reshape(T, H, D), pos, base, dims))
    k = rd(turn_pairs(rd(h @ w[p + "k"].T).reshape(T, G, D), pos, base, dims))
    v = rd(turn_pairs(rd(h @ w[p + "v"].T).reshape(T, G, E), pos, base, E))       # values turn over their whole size
    nb = T // m["mask"]["pool"]
    P = m["mask"]["pool"]
    k_mean = rd(k[: nb * P].reshape(nb, P, G, D).mean(dim=1))
    v_mean = rd(v[: nb * P].reshape(nb, P, G, E).mean(dim=1))
    rep = H // G
    o = windowed_pooled_attention(q, k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1), float(m["scale"]),
                                  m["mask"]["size"], P, k_mean.repeat_interleave(rep, dim=1),
                                  v_mean.repeat_interleave(rep, dim=1))
    o = rd(turn_pairs(o, pos, base, E, sign=-1.0))                                 # and the result turns back
    return rd(o.reshape(T, H * E) @ w[p + "o"].T)


# --------------------------------------------------------------------------- feed-forward
def clamped_gated_ff(h, gate, up, down, limit: float, rd=same):
    g = torch.clamp(rd(h @ gate.T), max=limit)
    u = torch.clamp(rd(h @ up.T), min=-limit, max=limit)
    return rd(rd(g * sigmoid(1.702 * g) * (u + 1.0)) @ down.T)


def expert_ff(h, gate, up, down, rd=same):
    return rd(rd(silu(rd(h @ gate.T)) * rd(h @ up.T)) @ down.T)


def route(h, w_router, top: int):
    """Scores s = sigmoid(h W_router^T); the ``top`` largest are chosen and weigh in as they are."""
    s = sigmoid(h @ w_router.T)
    chosen = torch.topk(s, top, dim=-1).indices
    return chosen, torch.gather(s, 1, chosen)


def moe_ff(h, w, p, mlp, rd=same):
    chosen, weights = route(h, w[p + "router"], mlp["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(chosen.shape[1]):
            e = int(chosen[t, j])
            scaled = rd(weights[t, j] * h[t:t + 1])          # the weight scales what the expert reads
            out[t] += expert_ff(scaled, w[f"{p}e{e}.gate"], w[f"{p}e{e}.up"], w[f"{p}e{e}.down"], rd)[0]
    return out


def feed_forward(h, w, p, mlp, rd=same):
    if mlp["kind"] == "dense":
        return clamped_gated_ff(h, w[p + "gate"], w[p + "up"], w[p + "down"], float(mlp["limit"]), rd)
    if mlp["kind"] == "moe":
        return moe_ff(h, w, p, mlp, rd)
    raise ValueError(mlp["kind"])


# --------------------------------------------------------------------------- the token's side input
def side_input(x, ids, i: int, w, p, d: int, eps: float, rd=same):
    c = w["side.embed"][ids][:, i * d:(i + 1) * d]
    g = rd(gelu_tanh(rd(rd(x) @ w[p + "gate"].T)) * c)
    y = g @ w[p + "proj"].T
    return rms(y, eps) * w[p + "norm"]


# --------------------------------------------------------------------------- the model
def layer_order(cfg: dict):
    """Layer indices in running order."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    return list(range(start)) + list(range(start, stop)) * times + list(range(stop, n))


def run_layer(x, ids, i, entry, w, cfg, rd=same):
    eps = cfg["norm"]["eps"]
    p = f"l{i}."
    h = rd(layer_norm(x, w[p + "norm1"], eps))
    if entry["type"] == "mingru":
        y = mingru_mixer(h, w, p + "mix.", rd)
    elif entry["type"] == "attention":
        y = attention_mixer(h, w, p + "mix.", entry["mixer"], rd)
    else:
        raise ValueError(entry["type"])
    x = x + w[p + "ls1"] * y
    if entry.get("mlp") is not None:
        y = feed_forward(rd(layer_norm(x, w[p + "norm2"], eps)), w, p + "mlp.", entry["mlp"], rd)
        x = x + w[p + "ls2"] * y
    side = cfg.get("token_side")
    if side:
        x = x + side_input(x, ids, i, w, p + "side.", side["dim"], eps, rd)
    return x


def forward(cfg: dict, w: dict, tokens, dtype=torch.float64, layers_out=None, act_dtype=None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence.  ``layers_out``: a list that receives x after every layer run."""
    rd = rounder(act_dtype)
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    ids = torch.as_tensor(tokens, dtype=torch.long)
    eps = cfg["norm"]["eps"]
    x = layer_norm(w["embed"][ids], w["embed.norm"], eps)
    for i in layer_order(cfg):
        x = run_layer(x, ids, i, cfg["layers"][i], w, cfg, rd)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rd(layer_norm(x, w["final.norm"], eps)) @ w["head"].T


def greedy(cfg, w, prompt, n_new, dtype=torch.float64):
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(forward(cfg, w, tokens, dtype)[-1].argmax()))
    return tokens[len(prompt):]
