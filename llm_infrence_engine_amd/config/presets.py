"""Named config.json contents for the random-weights mode: the shapes the published Qwen2.5 checkpoints
have, the two tiny ones the tests use and two Gemadra, two Gidurax and two Kuvazen shapes of the same widths, so that ``--random-config 0.5b``
needs no file.  These are data
of the kind a config.json holds; no part or kernel reads them.
"""
from __future__ import annotations

_QWEN2 = {"architectures": ["Qwen2ForCausalLM"], "rope_theta": 1000000.0, "rms_norm_eps": 1e-6}

PRESETS = {
    "tinyA": {**_QWEN2, "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
              "intermediate_size": 128, "vocab_size": 256, "rope_theta": 10000.0, "tie_word_embeddings": True},
    "tinyB": {**_QWEN2, "num_hidden_layers": 3, "hidden_size": 192, "num_attention_heads": 6, "num_key_value_heads": 2,
              "intermediate_size": 320, "vocab_size": 384, "rms_norm_eps": 1e-5, "tie_word_embeddings": False},
    "0.5b": {**_QWEN2, "num_hidden_layers": 24, "hidden_size": 896, "num_attention_heads": 14,
             "num_key_value_heads": 2, "intermediate_size": 4864, "vocab_size": 151936, "tie_word_embeddings": True},
    "7b": {**_QWEN2, "num_hidden_layers": 28, "hidden_size": 3584, "num_attention_heads": 28,
           "num_key_value_heads": 4, "intermediate_size": 18944, "vocab_size": 152064, "tie_word_embeddings": False},
    "32b": {**_QWEN2, "num_hidden_layers": 64, "hidden_size": 5120, "num_attention_heads": 40,
            "num_key_value_heads": 8, "intermediate_size": 27648, "vocab_size": 152064, "tie_word_embeddings": False},
}




def _gemadra(width, ff, layers, delta, latent, vocab=151936):
    """``layers`` layers, the two mixers in turn (the delta rule first); ranks of the delta mixer's low-rank maps stated."""
    d = {"type": "channel_delta", "mixer": dict(delta), "mlp": {"kind": "dense", "ff": ff}}
    a = {"type": "latent_attention", "mixer": dict(latent), "mlp": {"kind": "dense", "ff": ff}}
    return {"architecture": "Gemadra", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "canon": {"taps": 4},
            "layers": [dict(d) if i % 2 == 0 else dict(a) for i in range(layers)]}


# Gemadra at the widths of the two smaller Qwen2.5 shapes, with a feed-forward of as many weights (two matrices of
# 1.5 x the gated one's inner size) and mixers of a comparable number: for measurements beside those shapes
PRESETS["gemadra-0.5b"] = _gemadra(
    896, 7296, 24,
    {"heads": 14, "kv_heads": 7, "dim": 64, "vdim": 64, "conv": 4, "decay_rank": 64, "gate_rank": 64},
    {"heads": 14, "dim": 64, "rot_dim": 32, "vdim": 64, "kv_rank": 256, "q_rank": 384, "mask": {"size": 1024},
     "rot": {"base": 10000.0, "dims": 32}, "scale": 96 ** -0.5})
PRESETS["gemadra-7b"] = _gemadra(
    3584, 28416, 28,
    {"heads": 28, "kv_heads": 14, "dim": 128, "vdim": 128, "conv": 4, "decay_rank": 128, "gate_rank": 128},
    {"heads": 28, "dim": 128, "rot_dim": 64, "vdim": 128, "kv_rank": 512, "q_rank": 1536, "mask": {"size": 1024},
     "rot": {"base": 10000.0, "dims": 64}, "scale": 192 ** -0.5}, vocab=152064)


def _gidurax(width, ff, layers, scan, delta, attention, experts, vocab=151936):
    """``layers`` layers in the order scan, delta rule, attention, attention; every second one with routed experts
    (``experts``: (expert ff, experts, identities, top, shared ff)), the others with a dense feed-forward."""
    ef, n, ident, top, shared = experts
    routed = {"kind": "moe", "expert": {"ff": ef}, "router": {"experts": n, "identity": ident, "top": top}, "shared": {"ff": shared}}
    kinds = [("mamba1", scan), ("delta", delta), ("attention", attention), ("attention", attention)]
    return {"architecture": "Gidurax", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "residual_mult": 0.5,
            "embedding": {"scale": float(width) ** 0.5},
            "layers": [{"type": kinds[i % 4][0], "mixer": dict(kinds[i % 4][1]),
                        "mlp": dict(routed) if i % 2 else {"kind": "dense", "ff": ff}} for i in range(layers)]}


# Gidurax at the same widths: dense feed-forwards of Gemadra's size, routed ones whose chosen experts and shared expert
# together have about as many weights (three of sixteen experts and two identities, plus the shared one)
PRESETS["gidurax-0.5b"] = _gidurax(
    896, 7296, 24, {"inner": 1792, "state": 16, "dt_rank": 56, "conv": 4},
    {"heads": 14, "kv_heads": 7, "dim": 64, "vdim": 64, "conv": 4},
    {"heads": 14, "kv_heads": 2, "dim": 64, "vdim": 64, "scale": 64 ** -0.5, "q_temp": {"coef": 0.25, "every": 256}},
    (1824, 16, 2, 3, 1824))
PRESETS["gidurax-7b"] = _gidurax(
    3584, 28416, 28, {"inner": 7168, "state": 16, "dt_rank": 224, "conv": 4},
    {"heads": 28, "kv_heads": 14, "dim": 128, "vdim": 128, "conv": 4},
    {"heads": 28, "kv_heads": 4, "dim": 128, "vdim": 128, "scale": 128 ** -0.5, "q_temp": {"coef": 0.25, "every": 256}},
    (7104, 16, 2, 3, 7104), vocab=152064)


def _kuvazen(width, ff, layers, gru_width, attention, experts, side, vocab=151936):
    """``layers`` layers in the order minGRU, attention, minGRU, attention; the second and third with routed experts
    (``experts``: (expert ff, experts, top)), the others with the dense clamped feed-forward."""
    ef, n, top = experts
    routed = {"kind": "moe", "expert": {"ff": ef}, "router": {"experts": n, "top": top}}
    kinds = [("mingru", {"width": gru_width}), ("attention", attention)]
    return {"architecture": "Kuvazen", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "token_side": {"dim": side},
            "layers": [{"type": kinds[i % 2][0], "mixer": dict(kinds[i % 2][1]),
                        "mlp": dict(routed) if i % 4 in (1, 2) else {"kind": "dense", "ff": ff, "limit": 7.0}} for i in range(layers)]}


# Kuvazen at the same widths: gated dense feed-forwards of the Qwen2 shapes' size, routed ones whose three chosen experts
# of sixteen have as many weights together; a window of 256 tokens and blocks of 16, so that a 2,048-token prompt sees
# both tokens and blocks
PRESETS["kuvazen-0.5b"] = _kuvazen(
    896, 4864, 24, 1792,
    {"heads": 14, "kv_heads": 2, "dim": 64, "vdim": 64, "scale": 64 ** -0.5, "mask": {"size": 256, "pool": 16},
     "rot": {"base": 10000.0, "dims": 64}}, (1600, 16, 3), 64)
PRESETS["kuvazen-7b"] = _kuvazen(
    3584, 18944, 28, 7168,
    {"heads": 28, "kv_heads": 4, "dim": 128, "vdim": 128, "scale": 128 ** -0.5, "mask": {"size": 256, "pool": 16},
     "rot": {"base": 10000.0, "dims": 128}}, (6336, 16, 3), 256, vocab=152064)


def _silizen(width, ff, layers, attention, linear, delta, wkv_, window, rank, vocab=151936):
    """``layers`` layers in the order parallel, parallel_2, wkv, parallel, ...; every layer with the dense gated
    feed-forward; no looped stretch."""
    rotated = dict(attention, softcap=30.0, rot={"base": 1000000.0, "dims": attention["dim"] // 2,
                                                 "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}})
    kinds = [("parallel", {"left": rotated, "right": dict(linear, tau=16.0, decay_rank=rank), "left_scale": 0.5, "right_scale": 0.5}),
             ("parallel_2", {"left": dict(attention, mask={"size": window}), "right": dict(delta, conv=4, decay_rank=rank, gate_rank=rank)}),
             ("wkv", dict(wkv_, decay_rank=rank))]
    order = [0, 1, 2, 0]
    import copy

    return {"architecture": "Silizen", "vocab": vocab, "width": width, "norm": {"eps": 1e-5}, "logit_scale": 1.0,
            "layers": [{"type": kinds[order[i % 4]][0], "mixer": copy.deepcopy(kinds[order[i % 4]][1]),
                        "mlp": {"kind": "dense", "ff": ff}} for i in range(layers)]}


# Silizen at the same widths: attention of the Qwen2 shapes' heads beside a recurrence of the model's width, gated dense
# feed-forwards of the Qwen2 shapes' size, a window of 1,024 tokens in the windowed attention
PRESETS["silizen-0.5b"] = _silizen(
    896, 4864, 24, {"heads": 14, "kv_heads": 2, "dim": 64, "vdim": 64, "scale": 64 ** -0.5},
    {"heads": 7, "dim": 64, "vdim": 128}, {"heads": 14, "kv_heads": 7, "dim": 64, "vdim": 64}, {"heads": 14, "dim": 64}, 1024, 64)
PRESETS["silizen-7b"] = _silizen(
    3584, 18944, 28, {"heads": 28, "kv_heads": 4, "dim": 128, "vdim": 128, "scale": 128 ** -0.5},
    {"heads": 28, "dim": 64, "vdim": 128}, {"heads": 28, "kv_heads": 14, "dim": 128, "vdim": 128}, {"heads": 28, "dim": 128}, 1024,
    128, vocab=152064)


def preset(name: str) -> dict:
    if name not in PRESETS:
        raise KeyError(f"no preset {name!r}; there are {', '.join(sorted(PRESETS))}")
    import copy

    return copy.deepcopy(PRESETS[name])
