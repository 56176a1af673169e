"""Plain, slow Llama: the oracle every engine test is compared with.

Whole sequences, no cache, no paging, no batching; one function per part;
numpy only. It shares no code with the product package: it has its own
safetensors reader, its own config reading and its own random numbers.
Every function cites the line of the reference it was written from
(paths relative to the reference checkout).

All arithmetic runs in ``dtype`` (float64 by default: the truth both the
32-bit and the bfloat16 engine paths are measured against).
"""

from __future__ import annotations

import json
import math
import struct
from pathlib import Path
from typing import Any

import numpy as np

# --------------------------------------------------------------------- files


def read_safetensors(path: str | Path) -> dict[str, np.ndarray]:
    """name -> array. 8-byte little-endian header length, JSON header, raw data.
    bfloat16 is widened to float32 exactly (its 16 bits are the top half)."""
    raw = Path(path).read_bytes()
    (hlen,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8 : 8 + hlen])
    base = 8 + hlen
    out: dict[str, np.ndarray] = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        lo, hi = info["data_offsets"]
        buf = raw[base + lo : base + hi]
        shape = tuple(info["shape"])
        kind = info["dtype"]
        if kind == "BF16":
            u16 = np.frombuffer(buf, dtype="<u2").astype(np.uint32)
            arr = (u16 << 16).view(np.float32)
        elif kind == "F32":
            arr = np.frombuffer(buf, dtype="<f4")
        elif kind == "F16":
            arr = np.frombuffer(buf, dtype="<f2").astype(np.float32)
        elif kind == "F64":
            arr = np.frombuffer(buf, dtype="<f8")
        elif kind == "I32":
            arr = np.frombuffer(buf, dtype="<i4")
        elif kind == "I64":
            arr = np.frombuffer(buf, dtype="<i8")
        else:
            raise ValueError(f"{name}: dtype {kind} not handled by the plain reader")
        out[name] = arr.reshape(shape).copy()
    return out


class PlainConfig:
    """The numbers the formulas need, straight from config.json keys
    (prefixserve/model/config.py:62-104)."""

    def __init__(self, raw: dict[str, Any]) -> None:
        self.vocab = int(raw["vocab_size"])
        self.hidden = int(raw["hidden_size"])
        self.inter = int(raw["intermediate_size"])
        self.layers = int(raw["num_hidden_layers"])
        self.heads = int(raw["num_attention_heads"])
        self.kv_heads = int(raw.get("num_key_value_heads", self.heads))
        self.head_dim = int(raw.get("head_dim") or self.hidden // self.heads)
        self.eps = float(raw["rms_norm_eps"])
        rope = raw.get("rope_parameters") or raw.get("rope_scaling")
        theta = (raw.get("rope_parameters") or {}).get("rope_theta", raw.get("rope_theta"))
        self.theta = float(theta) if theta is not None else 10000.0
        kind = None if rope is None else rope.get("rope_type", rope.get("type"))
        self.scaling = None if kind in (None, "default") else rope
        self.tied = bool(raw.get("tie_word_embeddings", False))


# ------------------------------------------------------------------- formulas


def rope_inv_freq(head_dim: int, theta: float, scaling: dict[str, Any] | None) -> np.ndarray:
    """inv_freq[i] = 1/theta^(2i/D) with the llama3 three-band scaling
    (prefixserve/model/llama.py:24-46). Computed in float64 and rounded once to
    float32: the reference's float32 ``pow`` agrees with this to one ulp, and
    a correctly rounded value is the same in every library."""
    i = np.arange(0, head_dim, 2, dtype=np.float64)
    inv = 1.0 / (theta ** (i / head_dim))
    if scaling is not None:
        factor = float(scaling["factor"])
        low = float(scaling["low_freq_factor"])
        high = float(scaling["high_freq_factor"])
        old = float(scaling["original_max_position_embeddings"])
        low_wl = old / low
        high_wl = old / high
        wl = 2.0 * math.pi / inv
        scaled = np.where(wl > low_wl, inv / factor, inv)
        smooth = (old / wl - low) / (high - low)
        smoothed = (1.0 - smooth) * scaled / factor + smooth * scaled
        medium = ~(wl < high_wl) & ~(wl > low_wl)
        inv = np.where(medium, smoothed, scaled)
    return inv.astype(np.float32)


def rope_cos_sin(positions: np.ndarray, inv_freq: np.ndarray, dtype: Any = np.float64) -> tuple[np.ndarray, np.ndarray]:
    """cos/sin [n, D] of angle = float32(pos) * float32(inv_freq), the angle itself
    held in float32 as the reference's table does (prefixserve/model/llama.py:56-60);
    emb = cat(freqs, freqs)."""
    ang = positions.astype(np.float32)[:, None] * inv_freq.astype(np.float32)[None, :]
    assert ang.dtype == np.float32
    ang = np.concatenate([ang, ang], axis=-1).astype(np.float64)
    return np.cos(ang).astype(dtype), np.sin(ang).astype(dtype)


def apply_rope(x: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """Rotate-half layout: x*cos + cat(-x2, x1)*sin, x [n, heads, D], cos/sin [n, D]
    (prefixserve/model/llama.py:72-77)."""
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    rot = np.concatenate([-x2, x1], axis=-1)
    return x * cos[:, None, :] + rot * sin[:, None, :]


def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """weight * x * rsqrt(mean(x^2) + eps), eps inside the root
    (prefixserve/model/llama.py:63-69)."""
    ms = np.mean(x * x, axis=-1, keepdims=True)
    return weight * (x / np.sqrt(ms + eps))


def causal_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, window: int | None = None) -> np.ndarray:
    """q [n, Hq, D], k/v [n, Hkv, D], whole sequence. q head h uses kv head
    h // (Hq/Hkv); scores = q.k * 1/sqrt(D); keys after the query are masked;
    softmax; probs @ v (prefixserve/model/attention.py:109-120). ``window`` (not in the
    reference; used only by tests of the engine's windowed cache group) keeps keys with
    q_pos - k_pos < window."""
    n, hq, d = q.shape
    hkv = k.shape[1]
    group = hq // hkv
    scale = 1.0 / math.sqrt(d)
    out = np.empty_like(q)
    pos = np.arange(n)
    masked = pos[None, :] > pos[:, None]
    if window is not None:
        masked = masked | (pos[:, None] - pos[None, :] >= window)
    for h in range(hq):
        kh = k[:, h // group, :]
        vh = v[:, h // group, :]
        scores = (q[:, h, :] @ kh.T) * scale
        scores = np.where(masked, -np.inf, scores)
        scores = scores - scores.max(axis=-1, keepdims=True)
        p = np.exp(scores)
        p = p / p.sum(axis=-1, keepdims=True)
        out[:, h, :] = p @ vh
    return out


def silu(z: np.ndarray) -> np.ndarray:
    return z / (1.0 + np.exp(-z))


def swiglu_mlp(x: np.ndarray, w_gate: np.ndarray, w_up: np.ndarray, w_down: np.ndarray) -> np.ndarray:
    """(silu(x Wg^T) * (x Wu^T)) Wd^T (prefixserve/model/llama.py:120-121)."""
    return (silu(x @ w_gate.T) * (x @ w_up.T)) @ w_down.T


def round_bf16(x: np.ndarray) -> np.ndarray:
    """Rounds to the nearest bfloat16 (ties to even) and returns the values widened again."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = ((u >> 16) & 1) + np.uint32(0x7FFF)
    return ((u + r) & np.uint32(0xFFFF0000)).view(np.float32)


# ---------------------------------------------------------------------- model


class PlainLlama:
    """Whole-sequence forward from a model folder (config.json + model.safetensors)."""

    def __init__(self, model_dir: str | Path, dtype: Any = np.float64, bf16: bool = False,
                 weights: dict[str, np.ndarray] | None = None) -> None:
        """``bf16``: round the result of every operation to bfloat16, as a library that runs
        the reference's model code in bfloat16 does (prefixserve/model/llama.py:105-126 with
        dtype=bfloat16; softmax and the norm's statistics stay float32, llama.py:63-69 and
        prefixserve/model/attention.py:119). It is the yardstick for the engine's bfloat16 error."""
        model_dir = Path(model_dir)
        self.cfg = PlainConfig(json.loads((model_dir / "config.json").read_text()))
        self.bf16 = bf16
        if bf16:
            dtype = np.float32
        self.dtype = dtype
        # ``weights``: arrays another instance read from the same file (a large file is read once).
        source = weights if weights is not None else read_safetensors(model_dir / "model.safetensors")
        self.w = {k: v.astype(dtype, copy=False) for k, v in source.items()}
        self.inv_freq = rope_inv_freq(self.cfg.head_dim, self.cfg.theta, self.cfg.scaling)

    def _r(self, x: np.ndarray) -> np.ndarray:
        return round_bf16(x) if self.bf16 else x

    def _layer_bf16(self, i: int, h: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
        """The same layer with every operation's result rounded to bfloat16."""
        c, w, r = self.cfg, self.w, round_bf16
        p = f"model.layers.{i}."
        n = h.shape[0]

        def norm(x: np.ndarray, weight: np.ndarray) -> np.ndarray:
            xf = x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + np.float32(c.eps))
            return r(weight * r(xf))

        def rope(x: np.ndarray) -> np.ndarray:
            half = x.shape[-1] // 2
            rot = np.concatenate([-x[..., half:], x[..., :half]], axis=-1)
            return r(r(x * cos[:, None, :]) + r(rot * sin[:, None, :]))

        x = norm(h, w[p + "input_layernorm.weight"])
        q = rope(r(x @ w[p + "self_attn.q_proj.weight"].T).reshape(n, c.heads, c.head_dim))
        k = rope(r(x @ w[p + "self_attn.k_proj.weight"].T).reshape(n, c.kv_heads, c.head_dim))
        v = r(x @ w[p + "self_attn.v_proj.weight"].T).reshape(n, c.kv_heads, c.head_dim)
        group = c.heads // c.kv_heads
        scale = np.float32(1.0 / math.sqrt(c.head_dim))
        pos = np.arange(n)
        masked = pos[None, :] > pos[:, None]
        o = np.empty_like(q)
        for hd in range(c.heads):
            s = r(r(q[:, hd, :] @ k[:, hd // group, :].T) * scale)
            s = np.where(masked, -np.inf, s)
            e = np.exp(s - s.max(axis=-1, keepdims=True))
            pr = r(e / e.sum(axis=-1, keepdims=True))
            o[:, hd, :] = r(pr @ v[:, hd // group, :])
        h = r(h + r(o.reshape(n, -1) @ w[p + "self_attn.o_proj.weight"].T))
        x = norm(h, w[p + "post_attention_layernorm.weight"])
        g = r(x @ w[p + "mlp.gate_proj.weight"].T)
        u = r(x @ w[p + "mlp.up_proj.weight"].T)
        act = r(r(g / (1.0 + np.exp(-g))) * u)
        return r(h + r(act @ w[p + "mlp.down_proj.weight"].T))

    def layer(self, i: int, h: np.ndarray, cos: np.ndarray, sin: np.ndarray, window: int | None = None) -> np.ndarray:
        """One decoder layer in the reference's order (prefixserve/model/llama.py:111-121)."""
        if self.bf16:
            return self._layer_bf16(i, h, self._r(cos), self._r(sin))
        c, w = self.cfg, self.w
        p = f"model.layers.{i}."
        n = h.shape[0]
        x = rms_norm(h, w[p + "input_layernorm.weight"], c.eps)
        q = (x @ w[p + "self_attn.q_proj.weight"].T).reshape(n, c.heads, c.head_dim)
        k = (x @ w[p + "self_attn.k_proj.weight"].T).reshape(n, c.kv_heads, c.head_dim)
        v = (x @ w[p + "self_attn.v_proj.weight"].T).reshape(n, c.kv_heads, c.head_dim)
        q = apply_rope(q, cos, sin)
        k = apply_rope(k, cos, sin)
        o = causal_attention(q, k, v, window).reshape(n, c.heads * c.head_dim)
        h = h + o @ w[p + "self_attn.o_proj.weight"].T
        x = rms_norm(h, w[p + "post_attention_layernorm.weight"], c.eps)
        return h + swiglu_mlp(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])

    def hidden(self, tokens: Any, first_position: int = 0) -> np.ndarray:
        ids = np.asarray(tokens, dtype=np.int64)
        pos = np.arange(first_position, first_position + len(ids))
        cos, sin = rope_cos_sin(pos, self.inv_freq, self.dtype)
        h = self.w["model.embed_tokens.weight"][ids]
        for i in range(self.cfg.layers):
            h = self.layer(i, h, cos, sin)
        return h

    def logits(self, tokens: Any, first_position: int = 0) -> np.ndarray:
        """Logits at every position, [n, vocab] (prefixserve/model/llama.py:123-126);
        the head is the embedding table when tied (prefixserve/model/weights.py:133-136)."""
        h = self.hidden(tokens, first_position)
        head = self.w["model.embed_tokens.weight"] if self.cfg.tied else self.w["lm_head.weight"]
        if self.bf16:
            xf = h / np.sqrt(np.mean(h * h, axis=-1, keepdims=True) + np.float32(self.cfg.eps))
            return round_bf16(round_bf16(self.w["model.norm.weight"] * round_bf16(xf)) @ head.T)
        return rms_norm(h, self.w["model.norm.weight"], self.cfg.eps) @ head.T

    def logits_at(self, tokens: Any, rows: Any) -> np.ndarray:
        """The rows ``rows`` of ``logits(tokens)`` without the others: the output matrix of a
        large vocabulary is most of the work of a long sequence."""
        assert not self.bf16
        h = self.hidden(tokens)[np.asarray(rows, dtype=np.int64)]
        head = self.w["model.embed_tokens.weight"] if self.cfg.tied else self.w["lm_head.weight"]
        return rms_norm(h, self.w["model.norm.weight"], self.cfg.eps) @ head.T

    def greedy(self, prompt: Any, steps: int) -> tuple[list[int], list[np.ndarray]]:
        """Greedy generation by recomputing the whole sequence each step, as the
        reference's baseline does (tests/test_llama_exact.py:110-119)."""
        ids = [int(t) for t in prompt]
        toks: list[int] = []
        rows: list[np.ndarray] = []
        for _ in range(steps):
            last = self.logits(ids)[-1]
            rows.append(last)
            toks.append(int(np.argmax(last)))
            ids.append(toks[-1])
        return toks, rows


# ------------------------------------------------------------------- sampling

_M64 = (1 << 64) - 1


def _mix64(z: int) -> int:
    z = (z + 0x9E3779B97F4A7C15) & _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def uniform_for(seed: int, request_key: int, output_index: int) -> float:
    """u in [0,1) as a function of (seed, request, output index) only: 24 top bits of
    a splitmix64 chain. Not in the reference (it samples greedily only,
    prefixserve/llama_engine.py:146)."""
    z = _mix64(seed & _M64)
    z = _mix64(z ^ (request_key & _M64))
    z = _mix64(z ^ (output_index & _M64))
    return (z >> 40) / float(1 << 24)


def sample_plain(logits: np.ndarray, temperature: float, u: float) -> int:
    """Greedy (lowest index among equals) at temperature 0; else inverse CDF of
    softmax(logits/T) in vocabulary order."""
    if temperature <= 0.0:
        return int(np.argmax(logits))
    z = logits.astype(np.float64) / temperature
    p = np.exp(z - z.max())
    c = np.cumsum(p)
    return int(min(np.searchsorted(c, u * c[-1], side="right"), len(p) - 1))
