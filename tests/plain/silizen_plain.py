"""Plain, slow, whole-sequence Silizen decoder used only as the test oracle.

One function per mechanism, written from the design's equations in this file's own notation; no cache, no batching,
token-by-token loops where the design is a recurrence, position-by-position loops in attention, and no import from
the product package.  Everything runs in one floating type chosen by the caller (float64 by default).

Notation: a sequence is T tokens at positions 0..T-1; W is the model's width; every linear map is stored [out, in]
and applied as y = x @ M.T;  LN(x, w, b) = (x - mean x) / sqrt(var x + eps) * w + b;  RMS(x) = x / sqrt(mean x^2 + eps).

The design
* x = embed[token]; e = x as the embedding leaves it
* a stretch of layers [start, stop) is walked ``times`` times with the same weights, every walk with its own memory;
  right before every walk x <- loop.in [x ; e]
* a layer:  h = LN(x, norm1, norm1.b);  x <- x + (mixer(h) + ff(h)): one norm, both sublayers read it
* mixers: ``parallel`` (softmax attention with head norms, a partial rotation, capped scores, a sink of score zero and an
  output gate per head, beside gated linear attention with a decay per key channel; a weighted sum of the two),
  ``parallel_2`` (attention with biases, unit-RMS heads, a distance penalty per head and a sliding window, beside the
  gated delta rule with short convolutions; half the sum of the two after a norm each), ``wkv`` (a token-shifted
  recurrence with a decay per key channel and a bonus for the current token)
* feed-forward: down(gelu_tanh(gate h) * (up h))
* logits = embed LN(x, final.norm, final.norm.b) * logit_scale
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
    and activations leave, never to the residual stream, norms, scores, gates of a recurrence or states."""
    return same if act_dtype is None else (lambda x: x.to(act_dtype).to(x.dtype))


def layer_norm(x, w, b, eps):
    mu = x.mean(dim=-1, keepdim=True)
    dev = x - mu
    return dev / torch.sqrt((dev * dev).mean(dim=-1, keepdim=True) + eps) * w + b


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


# --------------------------------------------------------------------------- positions
def rotary_frequencies(dims: int, base: float, scaling=None, dtype=torch.float64):
    """f_i = base^(-2i/dims), i = 0 .. dims/2 - 1; with ``scaling`` {factor, low, high, original} every frequency whose
    wavelength 2 pi / f is longer than original/low is divided by factor, every one shorter than original/high kept, and
    those between are blended by s = (original/wavelength - low) / (high - low)."""
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if scaling is not None:
        factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
        out = []
        for fi in f:
            wl = 2.0 * math.pi / fi
            if wl < orig / high:
                out.append(fi)
            elif wl > orig / low:
                out.append(fi / factor)
            else:
                s = (orig / wl - low) / (high - low)
                out.append((1.0 - s) * fi / factor + s * fi)
        f = out
    return torch.tensor(f, dtype=dtype)


def rotate_half(x, positions, freqs):
    """x [T, heads, dim]: of every head's first 2 len(freqs) entries, entry i and entry i + len(freqs) turn together by
    the angle position * f_i; the rest stay."""
    half = freqs.numel()
    if half == 0:
        return x
    ang = positions.to(x.dtype)[:, None] * freqs.to(x.dtype)[None, :]          # [T, half]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., :half], x[..., half:2 * half]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * half:]], dim=-1)


# --------------------------------------------------------------------------- softmax attention with a sink of score 0
def sink_attention(q, k, v, scale, softcap=None, slopes=None, window=None):
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv].  Position i sees j <= i (with ``window``: the last ``window``
    of them, itself included).  score = scale q.k, then softcap * tanh(score / softcap), then minus slope_h (i - j);
    weights exp(s_j) / (1 + sum exp(s_j)): one more term of score 0 that carries no value."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            lo = 0 if window is None else max(0, i - window + 1)
            s = (k[lo:i + 1, g] @ q[i, h]) * scale
            if softcap is not None:
                s = softcap * torch.tanh(s / softcap)
            if slopes is not None:
                s = s - slopes[h] * (i - torch.arange(lo, i + 1, dtype=q.dtype))
            m = torch.clamp(s.max(), min=0.0)
            e = torch.exp(s - m)
            out[i, h] = (e[:, None] * v[lo:i + 1, g]).sum(0) / (torch.exp(-m) + e.sum())
    return out


def distance_slopes(H: int, dtype=torch.float64):
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=dtype)


# --------------------------------------------------------------------------- recurrences
def gated_linear_attention(q, k, v, alpha):
    """q, k, alpha [T, H, d], v [T, H, dv]: S <- diag(alpha_t) S + k_t v_t^T;  o_t = S^T q_t (after the write)."""
    T, H, d = q.shape
    S = torch.zeros(H, d, v.shape[-1], dtype=q.dtype)
    out = []
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out.append(torch.einsum("hde,hd->he", S, q[t]))
    return torch.stack(out)


def gated_delta_rule(q, k, v, g, beta):
    """q, k, g [T, H, d], v [T, H, dv], beta [T, H]: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T, H, d = q.shape
    S = torch.zeros(H, d, v.shape[-1], dtype=q.dtype)
    out = []
    for t in range(T):
        S = g[t][:, :, None] * S
        u = beta[t][:, None] * (v[t] - torch.einsum("hde,hd->he", S, k[t]))
        S = S + k[t][:, :, None] * u[:, None, :]
        out.append(torch.einsum("hde,hd->he", S, q[t]))
    return torch.stack(out)


def bonus_recurrence(r, k, v, w, u):
    """r, k, w [T, H, d], v [T, H, dv], u [H, d]: o_t = (S + diag(u) k_t v_t^T)^T r_t, then S <- diag(w_t) S + k_t v_t^T."""
    T, H, d = r.shape
    S = torch.zeros(H, d, v.shape[-1], dtype=r.dtype)
    out = []
    for t in range(T):
        kv = k[t][:, :, None] * v[t][:, None, :]
        out.append(torch.einsum("hde,hd->he", S + u[:, :, None] * kv, r[t]))
        S = w[t][:, :, None] * S + kv
    return torch.stack(out)


def causal_conv(x, taps_w):
    """x [T, C], taps_w [C, taps]: y_t = sum_j taps_w[:, j] x_(t - taps + 1 + j), zeros before the start."""
    T, C = x.shape
    taps = taps_w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x], dim=0)
    return sum(pad[j:j + T] * taps_w[:, j] for j in range(taps))


# --------------------------------------------------------------------------- the two attention halves
def attention_rotated(h, w, p, m, eps, positions, rnd):
    """The ``parallel`` mixer's left half."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rnd(h @ w[p + "q"].T).view(T, H, d)
    k = rnd(h @ w[p + "k"].T).view(T, G, d)
    v = rnd(h @ w[p + "v"].T).view(T, G, dv)
    q = unit_rms(q, eps) * w[p + "q.norm"]
    k = unit_rms(k, eps) * w[p + "k.norm"]
    rot = m.get("rot")
    if rot is not None and rot.get("dims", 0):
        f = rotary_frequencies(int(rot["dims"]), float(rot["base"]), rot.get("scaling"), h.dtype)
        q, k = rotate_half(q, positions, f), rotate_half(k, positions, f)
    q, k = rnd(q), rnd(k)
    o = sink_attention(q, k, v, float(m["scale"]), softcap=m.get("softcap"))
    gate = torch.sigmoid(rnd(h @ w[p + "g"].T))                      # [T, H]
    o = rnd(o * gate[:, :, None]).reshape(T, H * dv)
    return rnd(o @ w[p + "o"].T)


def attention_windowed(h, w, p, m, eps, rnd):
    """The ``parallel_2`` mixer's left half."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rnd(h @ w[p + "q"].T + w[p + "q.b"]).view(T, H, d)
    k = rnd(h @ w[p + "k"].T + w[p + "k.b"]).view(T, G, d)
    v = rnd(h @ w[p + "v"].T + w[p + "v.b"]).view(T, G, dv)
    q, k = rnd(unit_rms(q, eps)), rnd(unit_rms(k, eps))
    window = m["mask"]["size"] if m.get("mask") else None
    o = sink_attention(q, k, v, float(m["scale"]), slopes=distance_slopes(H, h.dtype), window=window)
    gate = torch.sigmoid(rnd(h @ w[p + "g"].T))
    o = rnd(o * gate[:, :, None]).reshape(T, H * dv)
    return rnd(o @ w[p + "o"].T)


# --------------------------------------------------------------------------- the recurrent halves
def linear_attention_half(h, w, p, m, eps, rnd):
    """The ``parallel`` mixer's right half."""
    T = h.shape[0]
    H, d, dv, tau = m["heads"], m["dim"], m["vdim"], float(m["tau"])
    q = rnd(h @ w[p + "q"].T).view(T, H, d) * d ** -0.5
    k = rnd(h @ w[p + "k"].T).view(T, H, d)
    v = rnd(h @ w[p + "v"].T).view(T, H, dv)
    z = rnd(h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]
    alpha = torch.sigmoid(z).view(T, H, d) ** (1.0 / tau)
    o = gated_linear_attention(q, k, v, alpha)
    o = unit_rms(o, eps) * w[p + "norm"]
    y = rnd(o.reshape(T, H * dv) * silu(rnd(h @ w[p + "g"].T)))
    return rnd(y @ w[p + "o"].T)


def delta_half(h, w, p, m, eps, rnd):
    """The ``parallel_2`` mixer's right half."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rnd(silu(causal_conv(rnd(h @ w[p + "q"].T), w[p + "q.conv"]))).view(T, G, d)
    k = rnd(silu(causal_conv(rnd(h @ w[p + "k"].T), w[p + "k.conv"]))).view(T, G, d)
    v = rnd(silu(causal_conv(rnd(h @ w[p + "v"].T), w[p + "v.conv"]))).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    q, k = q.repeat_interleave(H // G, dim=1), k.repeat_interleave(H // G, dim=1)
    beta = torch.sigmoid(rnd(h @ w[p + "b"].T))
    a = rnd(h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]
    g = torch.exp(-torch.exp(w[p + "A_log"])[None, :, None] * softplus(a).view(T, H, d))
    o = gated_delta_rule(q, k, v, g, beta)
    o = unit_rms(o, eps) * w[p + "norm"]
    gate = torch.sigmoid(rnd(rnd(h @ w[p + "g1"].T) @ w[p + "g2"].T)).view(T, H, dv)
    y = rnd((o * gate).reshape(T, H * dv))
    return rnd(y @ w[p + "o"].T)


# --------------------------------------------------------------------------- mixers
def mixer_parallel(h, w, p, m, eps, positions, rnd):
    left = attention_rotated(h, w, p + "left.", m["left"], eps, positions, rnd)
    right = linear_attention_half(h, w, p + "right.", m["right"], eps, rnd)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


def mixer_parallel_2(h, w, p, m, eps, rnd):
    left = attention_windowed(h, w, p + "left.", m["left"], eps, rnd)
    right = delta_half(h, w, p + "right.", m["right"], eps, rnd)
    return 0.5 * (unit_rms(left, eps) * w[p + "left.out"] + unit_rms(right, eps) * w[p + "right.out"])


def mixer_wkv(h, w, p, m, eps, rnd):
    T = h.shape[0]
    H, d = m["heads"], m["dim"]
    prev = torch.cat([torch.zeros(1, h.shape[1], dtype=h.dtype), h[:-1]], dim=0)

    def mix(s):
        return rnd(h + (prev - h) * w[p + "mu." + s])

    r = rnd(mix("r") @ w[p + "r"].T).view(T, H, d)
    k = rnd(mix("k") @ w[p + "k"].T).view(T, H, d)
    v = rnd(mix("v") @ w[p + "v"].T).view(T, H, d)
    gate = silu(rnd(mix("g") @ w[p + "g"].T))
    lw = rnd(torch.tanh(rnd(mix("w") @ w[p + "w1"].T))) @ w[p + "w2"].T + w[p + "w0"]
    decay = torch.exp(-torch.exp(lw)).view(T, H, d)
    o = bonus_recurrence(r, k, v, decay, w[p + "u"])
    o = unit_rms(o, eps).reshape(T, H * d) * w[p + "norm"]
    return rnd(rnd(o * gate) @ w[p + "o"].T)


def feed_forward(h, w, p, rnd):
    return rnd(rnd(gelu_tanh(rnd(h @ w[p + "gate"].T)) * rnd(h @ w[p + "up"].T)) @ w[p + "down"].T)


# --------------------------------------------------------------------------- the model
def run_order(cfg):
    """(layer index, opens a walk) for every layer run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return ([(i, False) for i in range(a)] + [(i, i == a) for _ in range(times) for i in range(a, b)] +
            [(i, False) for i in range(b, n)])


def forward(cfg, w, tokens, act_dtype=None, dtype=torch.float64, streams=None):
    """Logits [T, vocab] of one whole sequence.  ``streams``: a list that receives the residual stream after every
    layer run."""
    rnd = rounder(act_dtype)
    w = {k: v.to(dtype) for k, v in w.items()}
    eps = float(cfg["norm"]["eps"])
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(tokens.numel())
    x = w["embed"][tokens]
    e = x.clone()
    for i, opens in run_order(cfg):
        entry = cfg["layers"][i]
        p = f"l{i}."
        if opens:
            x = torch.cat([rnd(x), rnd(e)], dim=-1) @ w["loop.in"].T
        h = rnd(layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps))
        kind, m = entry["type"], entry["mixer"]
        if kind == "parallel":
            y = mixer_parallel(h, w, p + "mix.", m, eps, positions, rnd)
        elif kind == "parallel_2":
            y = mixer_parallel_2(h, w, p + "mix.", m, eps, rnd)
        elif kind == "wkv":
            y = mixer_wkv(h, w, p + "mix.", m, eps, rnd)
        else:
            raise ValueError(f"no mixer {kind!r}")
        if entry.get("mlp") is not None:
            y = y + feed_forward(h, w, p + "mlp.", rnd)
        x = x + y
        if streams is not None:
            streams.append(x.clone())
    hN = rnd(layer_norm(x, w["final.norm"], w["final.norm.b"], eps))
    return (hN @ w["embed"].T) * float(cfg["logit_scale"])
