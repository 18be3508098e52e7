"""Qwen3 dense, whole sequences, no cache, float64 numpy. One function per part; each cites the
reference lines its formula is read from (paths under the reference tree).

Precision: everything is float64 except what the reference itself fixes in 32-bit and which
changes values at that level: the rotary frequencies and angles (float32 products of a float32
position and a float32 frequency, miniserve/model/qwen3.py:97-100,105-108).

The window (``layer_windows``) has no counterpart in the reference, which ignores the
sliding-window keys; its meaning here: a query at position p sees keys p-W+1 .. p. Parity unpinned.
"""

from __future__ import annotations

import numpy as np


# ---------------------------------------------------------------- configuration


def read_config(cfg: dict) -> dict:
    """The numbers the model needs, by the reference's rules (miniserve/model/qwen3.py:38-55):
    ``head_dim`` falls back to hidden // heads; rope_scaling / non-silu are refused."""
    if cfg.get("rope_scaling"):
        raise NotImplementedError("rope_scaling")
    if cfg.get("hidden_act", "silu") != "silu":
        raise NotImplementedError("hidden_act")
    layers = cfg["num_hidden_layers"]
    kinds = cfg.get("layer_types")
    if kinds is not None:
        windows = [cfg["sliding_window"] if k == "sliding_attention" else 0 for k in kinds]
    elif cfg.get("use_sliding_window"):
        first = cfg.get("max_window_layers", layers)
        windows = [cfg["sliding_window"] if i >= first else 0 for i in range(layers)]
    else:
        windows = [0] * layers
    return dict(
        H=cfg["hidden_size"],
        I=cfg["intermediate_size"],
        V=cfg["vocab_size"],
        L=layers,
        Hq=cfg["num_attention_heads"],
        Hkv=cfg["num_key_value_heads"],
        D=cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"],
        eps=cfg["rms_norm_eps"],
        theta=float(cfg["rope_theta"]),
        tied=cfg.get("tie_word_embeddings", False),
        windows=windows,
    )


# ---------------------------------------------------------------- parts


def rms_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """``w * x * rsqrt(mean(x^2, -1) + eps)``; plain weight, not ``1 + w``
    (miniserve/model/qwen3.py:78-82)."""
    ms = np.mean(x * x, axis=-1, keepdims=True)
    return w * (x / np.sqrt(ms + eps))


def rotary_angles(positions: np.ndarray, head_dim: int, theta: float) -> np.ndarray:
    """``ang[t, j] = float32(pos[t]) * inv_freq[j]`` with ``inv_freq[j] = 1 / theta**(2j/D)``, both
    in float32 (miniserve/model/qwen3.py:97-100,105-106). Returns ``[T, D/2]`` float32."""
    expo = np.arange(0, head_dim, 2, dtype=np.int64).astype(np.float32) / np.float32(head_dim)
    inv_freq = (np.float32(1.0) / np.power(np.float32(theta), expo, dtype=np.float32)).astype(np.float32)
    return positions.astype(np.float32)[:, None] * inv_freq[None, :]


def rotate_half(x: np.ndarray) -> np.ndarray:
    """``cat(-x[D/2:], x[:D/2])`` (miniserve/model/qwen3.py:85-87)."""
    half = x.shape[-1] // 2
    return np.concatenate((-x[..., half:], x[..., :half]), axis=-1)


def apply_rotary(x: np.ndarray, ang: np.ndarray) -> np.ndarray:
    """``x * cos + rotate_half(x) * sin`` with ``cos, sin`` of ``cat(ang, ang)``, broadcast over heads:
    pair (j, j + D/2) is turned by angle ``ang[j]`` (miniserve/model/qwen3.py:107-108,121-123).
    ``x``: ``[T, heads, D]``."""
    emb = np.concatenate((ang, ang), axis=-1).astype(np.float64)  # [T, D]
    cos, sin = np.cos(emb)[:, None, :], np.sin(emb)[:, None, :]
    return x * cos + rotate_half(x) * sin


def attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float, window: int = 0) -> np.ndarray:
    """Causal softmax attention of one whole sequence with grouped heads: query head h reads KV head
    ``h // (Hq / Hkv)``; ``softmax(q k^T * scale + mask) v`` (miniserve/model/attention.py:55-69, the
    SDPA call with ``is_causal``, ``scale`` and ``enable_gqa``). ``q``: ``[T, Hq, D]``, ``k, v``:
    ``[T, Hkv, D]``; returns ``[T, Hq, D]``."""
    T, Hq, D = q.shape
    group = Hq // k.shape[1]
    i = np.arange(T)[:, None]
    j = np.arange(T)[None, :]
    seen = j <= i
    if window:
        seen &= (i - j) < window
    out = np.empty_like(q)
    for h in range(Hq):
        kh, vh = k[:, h // group, :], v[:, h // group, :]
        s = (q[:, h, :] @ kh.T) * scale
        s = np.where(seen, s, -np.inf)
        s = s - s.max(axis=-1, keepdims=True)
        p = np.exp(s)
        p = p / p.sum(axis=-1, keepdims=True)
        out[:, h, :] = p @ vh
    return out


def silu(x: np.ndarray) -> np.ndarray:
    return x / (1.0 + np.exp(-x))


def swiglu(x: np.ndarray, w_gate: np.ndarray, w_up: np.ndarray, w_down: np.ndarray) -> np.ndarray:
    """``down(silu(gate(x)) * up(x))``, no biases (miniserve/model/qwen3.py:128-131)."""
    return (silu(x @ w_gate.T) * (x @ w_up.T)) @ w_down.T


def attention_layer(x, w, prefix, c, ang, window):
    """Projections, per-head QK-RMSNorm (same eps as every norm, weight ``[D]`` shared by all heads,
    before the rotation, v untouched), rotation, attention, output projection
    (miniserve/model/qwen3.py:110-126)."""
    T = x.shape[0]
    q = (x @ w[prefix + "q_proj.weight"].T).reshape(T, c["Hq"], c["D"])
    k = (x @ w[prefix + "k_proj.weight"].T).reshape(T, c["Hkv"], c["D"])
    v = (x @ w[prefix + "v_proj.weight"].T).reshape(T, c["Hkv"], c["D"])
    q = rms_norm(q, w[prefix + "q_norm.weight"], c["eps"])
    k = rms_norm(k, w[prefix + "k_norm.weight"], c["eps"])
    q, k = apply_rotary(q, ang), apply_rotary(k, ang)
    o = attention(q, k, v, c["D"] ** -0.5, window)  # scale fixed at D^-0.5 (model/qwen3.py:133-135)
    return o.reshape(T, c["Hq"] * c["D"]) @ w[prefix + "o_proj.weight"].T


def hidden_states(cfg: dict, w: dict, token_ids, positions=None) -> np.ndarray:
    """Embedding, then per layer ``h += attn(norm(h)); h += mlp(norm(h))`` (pre-norm)
    (miniserve/model/qwen3.py:197-218). ``positions`` default to 0..T-1."""
    c = read_config(cfg)
    ids = np.asarray(token_ids, dtype=np.int64)
    pos = np.arange(len(ids)) if positions is None else np.asarray(positions)
    ang = rotary_angles(pos, c["D"], c["theta"])
    h = w["model.embed_tokens.weight"][ids]  # no scaling (model/qwen3.py:211)
    for i in range(c["L"]):
        p = f"model.layers.{i}."
        x = rms_norm(h, w[p + "input_layernorm.weight"], c["eps"])
        h = h + attention_layer(x, w, p + "self_attn.", c, ang, c["windows"][i])
        y = rms_norm(h, w[p + "post_attention_layernorm.weight"], c["eps"])
        h = h + swiglu(y, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return h


def logits(cfg: dict, w: dict, token_ids, positions=None) -> np.ndarray:
    """Final norm and output projection at every position: ``[T, V]`` float64
    (miniserve/model/qwen3.py:151-152 with ``all_logits``)."""
    c = read_config(cfg)
    h = hidden_states(cfg, w, token_ids, positions)
    return rms_norm(h, w["model.norm.weight"], c["eps"]) @ w["lm_head.weight"].T


def greedy(cfg: dict, w: dict, prompt, max_new: int, stop_ids=()) -> list[int]:
    """One token per pass, first maximal index, the stop token kept
    (miniserve/model/generate.py:12-43)."""
    ids = list(prompt)
    out = []
    for _ in range(max_new):
        nxt = int(np.argmax(logits(cfg, w, ids)[-1]))
        out.append(nxt)
        ids.append(nxt)
        if nxt in stop_ids:
            break
    return out


# ---------------------------------------------------------------- sampling


_M32 = 0xFFFFFFFF


def mix32(x: int) -> int:
    """The 32-bit xor-shift-multiply hash (miniserve/engine/sampler.py:29-38)."""
    x = (((x >> 16) ^ x) * 0x45D9F3B) & _M32
    x = (((x >> 16) ^ x) * 0x45D9F3B) & _M32
    return (x >> 16) ^ x


def uniform_noise(seed: int, counter: int, vocab: int) -> np.ndarray:
    """``u[v] in (0,1)`` keyed by (seed, counter, v) (miniserve/engine/sampler.py:41-46)."""
    key = mix32(seed ^ mix32(counter))
    out = np.empty(vocab, dtype=np.float64)
    for v in range(vocab):
        h = mix32((key + v * 0x9E3779B9) & _M32)
        out[v] = ((h >> 8) + 0.5) / float(1 << 24)
    return out


def sample(logit_row: np.ndarray, temperature: float, seed: int, counter: int, top_p: float = 1.0) -> int:
    """Greedy at temperature 0, else ``argmax(logits / T + g)`` with Gumbel noise ``g = -log(-log u)``;
    with ``top_p < 1`` the tokens outside the nucleus are masked first: a token stays while the
    probability mass sorted before it is below ``top_p`` (miniserve/engine/sampler.py:86-112)."""
    if temperature == 0:
        return int(np.argmax(logit_row))
    z = np.asarray(logit_row, dtype=np.float64) / temperature
    if top_p < 1:
        p = np.exp(z - z.max())
        p /= p.sum()
        order = np.argsort(-p, kind="stable")
        before = np.cumsum(p[order]) - p[order]
        keep = np.zeros(len(z), dtype=bool)
        keep[order] = before < top_p
        z = np.where(keep, z, -np.inf)
    # The reference evaluates u in float32, where the one input 2^24 - 1 rounds up to u = 1 and the
    # noise becomes infinite; u is kept below 1 here (a deliberate departure, 2^-24 of the draws).
    u = np.minimum(uniform_noise(seed, counter, len(z)).astype(np.float32), np.float32(0.99999994))
    g = -np.log(-np.log(u.astype(np.float64)))
    return int(np.argmax(z + g))
