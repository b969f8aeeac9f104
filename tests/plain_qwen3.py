"""A plain, slow Qwen3 for tests: whole sequences, no cache, one function per part.

Written from the formulas of the reference (file:line cited at each function,
paths relative to the reference's root); it shares no code with the engine.
Everything runs on the CPU in float64, except where the reference fixes a
float32 rounding that belongs to the definition: the rotary frequencies and
angles (``src/backend/rope.h:9-13``, ``src/backend/cpu/cpu_backend.cpp:180-182``).
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

F64 = torch.float64


def embed(table: torch.Tensor, ids: Sequence[int]) -> torch.Tensor:
    """x[t] = table[ids[t]], no scaling. src/backend/cpu/cpu_backend.cpp:51-76; src/model/qwen3.cpp:213."""
    return table[torch.as_tensor(list(ids), dtype=torch.long)].to(F64)


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """out = x @ w^T with w stored [out, in], no bias. src/backend/cpu/cpu_backend.cpp:93-139."""
    return x.to(F64) @ w.to(F64).T


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """out_i = (x_i * inv) * w_i, inv = 1 / sqrt(sum(x^2) / n + eps), over the last dim.

    The weight multiplies after normalisation and is plain w. src/backend/cpu/cpu_backend.cpp:141-159.
    """
    x = x.to(F64)
    n = x.shape[-1]
    inv = 1.0 / torch.sqrt((x * x).sum(dim=-1, keepdim=True) / n + eps)
    return (x * inv) * w.to(F64)


def rope_inv_freq(theta: float, head_dim: int) -> np.ndarray:
    """inv_freq[i] = 1 / theta^(2i / head_dim) in float32. src/backend/rope.h:9-13."""
    out = np.empty(head_dim // 2, dtype=np.float32)
    for i in range(head_dim // 2):
        exponent = np.float32(2 * i) / np.float32(head_dim)
        out[i] = np.float32(1.0) / np.power(np.float32(theta), exponent, dtype=np.float32)
    return out


def rope_neox(x: torch.Tensor, positions: Sequence[int], theta: float) -> torch.Tensor:
    """Rotate-half rotary on x [T, heads, head_dim].

    Pairs are (i, i + head_dim/2); angle = float32(pos) * inv_freq[i] in float32;
    out[i] = x1 cos - x2 sin, out[i + half] = x2 cos + x1 sin.
    src/backend/cpu/cpu_backend.cpp:161-193.
    """
    x = x.to(F64)
    T, heads, dim = x.shape
    half = dim // 2
    inv_freq = rope_inv_freq(theta, dim)
    pos = np.asarray(list(positions), dtype=np.float32)
    angle = (pos[:, None] * inv_freq[None, :]).astype(np.float32)       # float32 product, as the reference
    c = torch.from_numpy(np.cos(angle.astype(np.float64)))[:, None, :]
    s = torch.from_numpy(np.sin(angle.astype(np.float64)))[:, None, :]
    x1, x2 = x[..., :half], x[..., half:]
    return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                     window: Optional[int] = None) -> torch.Tensor:
    """Causal grouped-query attention of one whole sequence.

    q [T, H, Dh], k and v [T, KVH, Dh]. Query head h reads KV head h // (H // KVH);
    score_j = scale * (q . k_j) for j <= pos (and j > pos - window if a window is given);
    softmax over those j; out = sum p_j v_j. The reference computes the same sum with a
    running maximum (online softmax): src/backend/cpu/cpu_backend.cpp:261-319.
    """
    q, k, v = q.to(F64), k.to(F64), v.to(F64)
    T, H, Dh = q.shape
    KVH = k.shape[1]
    group = H // KVH
    out = torch.zeros_like(q)
    for h in range(H):
        kvh = h // group
        scores = scale * (q[:, h, :] @ k[:, kvh, :].T)                  # [T, T]
        i = torch.arange(T)[:, None]
        j = torch.arange(T)[None, :]
        allowed = j <= i
        if window is not None:
            allowed = allowed & (j > i - window)
        scores = scores.masked_fill(~allowed, -math.inf)
        p = torch.softmax(scores, dim=-1)
        out[:, h, :] = p @ v[:, kvh, :]
    return out


def causal_attention_tail(q_tail: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                          window: Optional[int] = None) -> torch.Tensor:
    """The last ``n`` rows of ``causal_attention`` when only their queries are at hand.

    q_tail [n, H, Dh] are the queries at positions T-n .. T-1 of a sequence whose keys and values
    k, v [T, KVH, Dh] are all given: the same formula (src/backend/cpu/cpu_backend.cpp:261-319), without
    the T x T score matrix, so that a context of tens of thousands of keys stays affordable.
    """
    q_tail, k, v = q_tail.to(F64), k.to(F64), v.to(F64)
    n, H, Dh = q_tail.shape
    T, KVH = k.shape[0], k.shape[1]
    group = H // KVH
    out = torch.zeros_like(q_tail)
    for r in range(n):
        pos = T - n + r
        first = 0 if window is None else max(0, pos - window + 1)
        for h in range(H):
            kvh = h // group
            scores = scale * (k[first:pos + 1, kvh, :] @ q_tail[r, h, :])
            out[r, h, :] = torch.softmax(scores, dim=0) @ v[first:pos + 1, kvh, :]
    return out


def swiglu(h: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    """down(gate / (1 + exp(-gate)) * up). src/model/qwen3.cpp:235-238; src/backend/cpu/cpu_backend.cpp:195-207."""
    g = linear(h, w_gate)
    u = linear(h, w_up)
    a = g / (1.0 + torch.exp(-g)) * u
    return linear(a, w_down)


def attention_block(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, cfg: dict,
                    positions: Sequence[int]) -> torch.Tensor:
    """q/k/v projections, per-head q/k RMSNorm BEFORE rotary, rotary, causal attention, output projection.

    src/model/qwen3.cpp:219-230 (comment at 217: QK-norm runs per head and before RoPE).
    """
    T = h.shape[0]
    H, KVH, Dh = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps = cfg["rms_norm_eps"]
    q = linear(h, w[prefix + "self_attn.q_proj.weight"]).view(T, H, Dh)
    k = linear(h, w[prefix + "self_attn.k_proj.weight"]).view(T, KVH, Dh)
    v = linear(h, w[prefix + "self_attn.v_proj.weight"]).view(T, KVH, Dh)
    q = rms_norm(q, w[prefix + "self_attn.q_norm.weight"], eps)
    k = rms_norm(k, w[prefix + "self_attn.k_norm.weight"], eps)
    q = rope_neox(q, positions, cfg["rope_theta"])
    k = rope_neox(k, positions, cfg["rope_theta"])
    scale = float(np.float32(1.0) / np.sqrt(np.float32(Dh)))           # src/model/qwen3.cpp:195
    attn = causal_attention(q, k, v, scale).reshape(T, H * Dh)
    return linear(attn, w[prefix + "self_attn.o_proj.weight"])


def forward(weights: Dict[str, torch.Tensor], cfg: dict, tokens: Sequence[int],
            hidden_states: Optional[List[torch.Tensor]] = None, rows: Optional[Sequence[int]] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence. src/model/qwen3.cpp:213-259.

    x = embed; per layer: x += attention(norm(x)); x += mlp(norm(x)); logits = norm(x) @ lm_head^T,
    lm_head being the embedding matrix when tie_word_embeddings is set (qwen3.cpp:94-100).
    ``rows``: the positions whose logits are returned (all by default), as the reference's step
    returns logits at the requested rows only (qwen3.cpp:249-259). Weights may come in any float
    type: every product widens its operands to float64 itself.
    """
    cfg = normalized_config(cfg)
    eps = cfg["rms_norm_eps"]
    positions = list(range(len(tokens)))
    x = embed(weights["model.embed_tokens.weight"], tokens)
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        h = rms_norm(x, weights[p + "input_layernorm.weight"], eps)
        x = x + attention_block(h, weights, p, cfg, positions)
        h = rms_norm(x, weights[p + "post_attention_layernorm.weight"], eps)
        x = x + swiglu(h, weights[p + "mlp.gate_proj.weight"], weights[p + "mlp.up_proj.weight"],
                       weights[p + "mlp.down_proj.weight"])
        if hidden_states is not None:
            hidden_states.append(x.clone())
    if rows is not None:
        x = x[torch.as_tensor(list(rows), dtype=torch.long)]
    x = rms_norm(x, weights["model.norm.weight"], eps)
    head = weights["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else weights["lm_head.weight"]
    return linear(x, head)


def normalized_config(cfg: dict) -> dict:
    """Fills the defaults the reference applies. src/model/config.cpp:56-61."""
    cfg = dict(cfg)
    cfg.setdefault("num_key_value_heads", cfg["num_attention_heads"])
    cfg.setdefault("head_dim", cfg["hidden_size"] // cfg["num_attention_heads"])
    cfg.setdefault("rope_theta", 10000.0)
    cfg.setdefault("tie_word_embeddings", False)
    return cfg


def greedy(weights: Dict[str, torch.Tensor], cfg: dict, prompt: Sequence[int], max_tokens: int,
           stop: Sequence[int] = ()) -> List[int]:
    """Greedy generation by recomputing the whole sequence for every token; ties go to the lowest id."""
    tokens = list(prompt)
    out: List[int] = []
    for _ in range(max_tokens):
        logits = forward(weights, cfg, tokens)[-1]
        token = int(torch.argmax(logits))                               # first maximum = lowest id
        tokens.append(token)
        out.append(token)
        if token in stop:
            break
    return out


# ------------------------------------------------------------------ sampling
class MT19937_64:
    """The 64-bit Mersenne Twister (std::mt19937_64, which the reference seeds per request:
    src/engine/engine.cpp:58). Written from the published recurrence."""

    NN, MM = 312, 156
    MATRIX_A, UM, LM = 0xB5026F5AA96619E9, 0xFFFFFFFF80000000, 0x7FFFFFFF
    MASK = (1 << 64) - 1

    def __init__(self, seed: int):
        self.mt = [0] * self.NN
        self.mt[0] = seed & self.MASK
        for i in range(1, self.NN):
            self.mt[i] = (6364136223846793005 * (self.mt[i - 1] ^ (self.mt[i - 1] >> 62)) + i) & self.MASK
        self.index = self.NN

    def __call__(self) -> int:
        if self.index >= self.NN:
            mt = self.mt
            for i in range(self.NN):
                x = (mt[i] & self.UM) | (mt[(i + 1) % self.NN] & self.LM)
                mt[i] = mt[(i + self.MM) % self.NN] ^ (x >> 1) ^ (self.MATRIX_A if x & 1 else 0)
            self.index = 0
        x = self.mt[self.index]
        self.index += 1
        x ^= (x >> 29) & 0x5555555555555555
        x ^= (x << 17) & 0x71D67FFFEDA60000
        x ^= (x << 37) & 0xFFF7EEE000000000
        x ^= x >> 43
        return x & self.MASK

    def uniform(self, low: float, high: float) -> float:
        """std::uniform_real_distribution<double>(low, high): one 64-bit draw scaled by 2^-64."""
        u = self() / 18446744073709551616.0
        if u >= 1.0:
            u = math.nextafter(1.0, 0.0)
        return u * (high - low) + low


def sample(logits: Sequence[float], temperature: float, top_k: int, top_p: float, rng: MT19937_64) -> int:
    """One token from the logits. src/sampling/sampler.cpp:18-81.

    Greedy at temperature 0 or when 1/temperature is not finite; a +inf logit wins outright;
    otherwise (logit - max) / temperature, keep the top_k most likely (value descending, id
    ascending), softmax weights (unnormalised, float32 exp, double sum), keep the smallest
    prefix whose weight reaches top_p * total, draw r in [0, total) and walk the candidates.
    """
    logits = [float(np.float32(v)) for v in logits]
    if not logits:
        raise ValueError("cannot sample from empty logits")
    if any(math.isnan(v) for v in logits):
        raise ValueError("a logit is NaN")
    max_raw = max(logits)
    arg = logits.index(max_raw)
    if max_raw == -math.inf:
        raise ValueError("all logits are -inf")
    with np.errstate(divide="ignore", over="ignore"):
        inv_t = math.inf if temperature == 0.0 else float(np.float32(1.0) / np.float32(temperature))
    if not math.isfinite(inv_t) or max_raw == math.inf:
        return arg
    with np.errstate(over="ignore", invalid="ignore"):
        cand = [(float((np.float32(v) - np.float32(max_raw)) * np.float32(inv_t)), i) for i, v in enumerate(logits)]
    keep = len(cand)
    key = lambda c: (-c[0], c[1])
    if top_k > 0 and top_k < keep:
        keep = top_k
        cand.sort(key=key)
    elif top_p < 1.0:
        cand.sort(key=key)
    max_logit = max(c[0] for c in cand[:keep])
    weights = [float(np.exp(np.float32(c[0] - max_logit))) for c in cand[:keep]]
    total = sum(weights)
    if top_p < 1.0:
        cumulative = 0.0
        limit = float(np.float32(top_p)) * total
        for i in range(keep):
            cumulative += weights[i]
            if cumulative >= limit:
                keep = i + 1
                break
        total = cumulative
    r = rng.uniform(0.0, total)
    for i in range(keep):
        r -= weights[i]
        if r < 0.0:
            return cand[i][1]
    return cand[keep - 1][1]
