"""A plain, slow implementation of the Qwen3 dense decoder, whole sequences, no cache.

It is the oracle the engine is compared with.  It shares no code with the
product path: it takes a plain ``dict`` of tensors (as a library safetensors
loader returns them) and a plain ``dict`` of config.json keys, and it is built
of one function per part.  Every function cites the place in the reference
(paths under ``crates/pagedllm/src``) whose formula it follows.  Everything is
computed in float64 unless a dtype is given.
"""

from __future__ import annotations

import math

import torch


def rms_norm(x: torch.Tensor, gain: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x / sqrt(mean(x^2, last) + eps) * gain  (model/layers.rs:58-64).

    The statistic is the mean of squares over the last axis, eps is added
    inside the root, and the division is by the root (not a multiplication by
    an approximate reciprocal).
    """
    variance = (x * x).mean(dim=-1, keepdim=True)
    return x / torch.sqrt(variance + eps) * gain


def rope_inverse_frequencies(head_dim: int, theta: float) -> torch.Tensor:
    """inv_f[i] = 1 / theta^(2i/d), i in [0, d/2)  (model/rope.rs:38-41)."""
    half = head_dim // 2
    return torch.tensor(
        [1.0 / (theta ** (2.0 * i / head_dim)) for i in range(half)], dtype=torch.float64
    )


def rope_tables(head_dim: int, positions: torch.Tensor, theta: float):
    """cos/sin of position * inv_f, the half table laid twice over the head
    (model/rope.rs:45-56)."""
    inv = rope_inverse_frequencies(head_dim, theta)
    angle = positions.to(torch.float64)[:, None] * inv[None, :]
    angle = torch.cat([angle, angle], dim=-1)
    return angle.cos(), angle.sin()


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """[x1, x2] -> [-x2, x1], halves of the head (model/rope.rs:101-106)."""
    half = x.shape[-1] // 2
    return torch.cat([-x[..., half:], x[..., :half]], dim=-1)


def apply_rope(x: torch.Tensor, positions: torch.Tensor, theta: float) -> torch.Tensor:
    """out = x*cos + rotate_half(x)*sin at each token's own position
    (model/rope.rs:95-99).  ``x`` is [seq, heads, head_dim]."""
    cos, sin = rope_tables(x.shape[-1], positions, theta)
    cos = cos[:, None, :].to(x)
    sin = sin[:, None, :].to(x)
    return x * cos + rotate_half(x) * sin


def repeat_kv(x: torch.Tensor, group: int) -> torch.Tensor:
    """Query head h reads key head h // group (model/attention.rs:240-248).
    ``x`` is [seq, kv_heads, head_dim] -> [seq, kv_heads*group, head_dim]."""
    seq, kv_heads, head_dim = x.shape
    return x[:, :, None, :].expand(seq, kv_heads, group, head_dim).reshape(
        seq, kv_heads * group, head_dim
    )


def causal_mask(queries: int, keys: int, window: int | None = None) -> torch.Tensor:
    """Additive 0/-inf mask: the query at row i sits at position keys-queries+i
    and sees key j iff j <= its position (model/attention.rs:255-275).  With a
    window w it also needs j > position - w (not in the reference, which
    refuses a window: config.rs:104-106)."""
    offset = keys - queries
    q = torch.arange(queries)[:, None] + offset
    k = torch.arange(keys)[None, :]
    visible = k <= q
    if window is not None:
        visible &= k > q - window
    mask = torch.zeros(queries, keys, dtype=torch.float64)
    mask[~visible] = float("-inf")
    return mask


def softmax_last(x: torch.Tensor) -> torch.Tensor:
    """exp(x - max) / sum exp(x - max) over the last axis
    (model/attention.rs:282-289)."""
    peak = x.max(dim=-1, keepdim=True).values
    e = (x - peak).exp()
    return e / e.sum(dim=-1, keepdim=True)


def attention_core(q, k, v, scale: float, window: int | None = None) -> torch.Tensor:
    """softmax(q k^T * scale + mask) v per head (model/attention.rs:99-104).
    q [sq, heads, d]; k, v [sk, heads, d]; the queries are the last sq positions."""
    scores = torch.einsum("qhd,khd->hqk", q, k) * scale
    scores = scores + causal_mask(q.shape[0], k.shape[0], window).to(scores)[None]
    weights = softmax_last(scores)
    return torch.einsum("hqk,khd->qhd", weights, v)


def attention(x, w, prefix: str, cfg: dict, positions, trace=None, window=None):
    """Grouped-query attention with per-head RMSNorm on q and k before the
    rotation (model/attention.rs:62-114): project, split into heads, norm over
    one head's width, rotate, expand the key heads over their group, attend,
    concatenate heads (head slow), project out."""
    nq = cfg["num_attention_heads"]
    nkv = cfg["num_key_value_heads"]
    d = cfg["head_dim"]
    eps = cfg["rms_norm_eps"]
    theta = config_rope_theta(cfg)
    seq = x.shape[0]

    q = x @ w[f"{prefix}.q_proj.weight"].T
    k = x @ w[f"{prefix}.k_proj.weight"].T
    v = x @ w[f"{prefix}.v_proj.weight"].T
    _record(trace, f"{prefix}.q_proj.out", q)
    _record(trace, f"{prefix}.k_proj.out", k)
    _record(trace, f"{prefix}.v_proj.out", v)

    q = q.reshape(seq, nq, d)
    k = k.reshape(seq, nkv, d)
    v = v.reshape(seq, nkv, d)

    q = rms_norm(q, w[f"{prefix}.q_norm.weight"], eps)
    k = rms_norm(k, w[f"{prefix}.k_norm.weight"], eps)
    _record(trace, f"{prefix}.q_norm.out", q)
    _record(trace, f"{prefix}.k_norm.out", k)

    q = apply_rope(q, positions, theta)
    k = apply_rope(k, positions, theta)

    group = nq // nkv
    k = repeat_kv(k, group)
    v = repeat_kv(v, group)

    scale = 1.0 / math.sqrt(d)  # model/attention.rs:51
    out = attention_core(q, k, v, scale, window).reshape(seq, nq * d)
    _record(trace, f"{prefix}.o_proj.in", out)
    out = out @ w[f"{prefix}.o_proj.weight"].T
    _record(trace, f"{prefix}.o_proj.out", out)
    _record(trace, f"{prefix}.out", out)
    return out


def silu(x: torch.Tensor) -> torch.Tensor:
    """z * sigmoid(z)."""
    return x / (1.0 + torch.exp(-x))


def swiglu_mlp(x, w, prefix: str, trace=None) -> torch.Tensor:
    """down(silu(gate(x)) * up(x)); the activation is on the gate branch
    (model/layers.rs:93-106)."""
    gate = x @ w[f"{prefix}.gate_proj.weight"].T
    up = x @ w[f"{prefix}.up_proj.weight"].T
    _record(trace, f"{prefix}.gate_proj.out", gate)
    _record(trace, f"{prefix}.up_proj.out", up)
    gated = silu(gate) * up
    _record(trace, f"{prefix}.down_proj.in", gated)
    out = gated @ w[f"{prefix}.down_proj.weight"].T
    _record(trace, f"{prefix}.down_proj.out", out)
    _record(trace, f"{prefix}.out", out)
    return out


def decoder_block(x, w, prefix: str, cfg: dict, positions, trace=None, window=None):
    """Pre-norm block with two residuals (model/mod.rs:92-114)."""
    eps = cfg["rms_norm_eps"]
    normed = rms_norm(x, w[f"{prefix}.input_layernorm.weight"], eps)
    _record(trace, f"{prefix}.input_layernorm.out", normed)
    x = x + attention(normed, w, f"{prefix}.self_attn", cfg, positions, trace, window)
    normed = rms_norm(x, w[f"{prefix}.post_attention_layernorm.weight"], eps)
    _record(trace, f"{prefix}.post_attention_layernorm.out", normed)
    x = x + swiglu_mlp(normed, w, f"{prefix}.mlp", trace)
    _record(trace, f"{prefix}.out", x)
    return x


def config_rope_theta(cfg: dict) -> float:
    """Flat ``rope_theta`` or nested ``rope_parameters.rope_theta``
    (config.rs:139-145)."""
    if cfg.get("rope_theta") is not None:
        return float(cfg["rope_theta"])
    return float(cfg["rope_parameters"]["rope_theta"])


def lm_head_weight(w: dict, cfg: dict) -> torch.Tensor:
    """Stored lm_head.weight if present, else the embedding when tied
    (model/mod.rs:222-235)."""
    if "lm_head.weight" in w:
        return w["lm_head.weight"]
    if cfg["tie_word_embeddings"]:
        return w["model.embed_tokens.weight"]
    raise KeyError("no lm_head.weight, and the config does not tie the embeddings")


def forward(weights: dict, cfg: dict, tokens, *, offset: int = 0, trace: dict | None = None,
            dtype=torch.float64, window: int | None = None, device="cpu") -> torch.Tensor:
    """Logits [seq, vocab] for one whole sequence, no cache
    (model/mod.rs:271-303): embedding gather without scaling, every block,
    final norm on all positions, output projection.  ``device``: where torch does the
    arithmetic (a sequence of thousands of tokens takes a minute on the CPU); the result
    comes back to the CPU."""
    w = {k: v.to(device=device, dtype=dtype) for k, v in weights.items()}
    ids = torch.as_tensor(list(tokens), dtype=torch.long, device=device)
    if ids.numel() == 0:
        raise ValueError("cannot run a forward pass on no tokens")
    positions = torch.arange(ids.numel()) + offset
    x = w["model.embed_tokens.weight"][ids]
    _record(trace, "model.embed_tokens.out", x)
    for layer in range(cfg["num_hidden_layers"]):
        x = decoder_block(x, w, f"model.layers.{layer}", cfg, positions, trace, window)
    x = rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"])
    _record(trace, "model.norm.out", x)
    logits = x @ lm_head_weight(w, cfg).T
    _record(trace, "lm_head.out", logits)
    _record(trace, "logits", logits)
    return logits.cpu()


def greedy_generate(weights: dict, cfg: dict, prompt, steps: int) -> list[int]:
    """Argmax decoding by re-running the whole sequence each step; the first
    maximum wins (sampler.rs:186-194)."""
    tokens = list(prompt)
    out = []
    for _ in range(steps):
        logits = forward(weights, cfg, tokens)[-1]
        nxt = int(torch.argmax(logits))  # torch returns the first maximum
        out.append(nxt)
        tokens.append(nxt)
    return out


def _record(trace, name, tensor):
    if trace is not None:
        trace[name] = tensor


# ---------------------------------------------------------------------------
# Sampling and hashing, as plain as the model above.
# ---------------------------------------------------------------------------

MASK64 = (1 << 64) - 1


class SplitMix64:
    """sampler.rs:17-44."""

    def __init__(self, seed: int):
        self.state = seed & MASK64

    def next_u64(self) -> int:
        self.state = (self.state + 0x9E3779B97F4A7C15) & MASK64
        z = self.state
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK64
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK64
        return z ^ (z >> 31)

    def next_f32(self) -> float:
        return (self.next_u64() >> 40) / float(1 << 24)


def block_hash(parent: int | None, tokens) -> int:
    """FNV-1a over the little-endian bytes of (parent or 0, len, tokens as
    u64), finished with the splitmix64 mixer (blocks.rs:53-72)."""
    h = 0xCBF29CE484222325

    def mix(h, value):
        for byte in int(value).to_bytes(8, "little"):
            h ^= byte
            h = (h * 0x00000100000001B3) & MASK64
        return h

    h = mix(h, parent or 0)
    h = mix(h, len(tokens))
    for t in tokens:
        h = mix(h, t)
    z = (h + 0x9E3779B97F4A7C15) & MASK64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK64
    return z ^ (z >> 31)


def sample(logits, temperature: float, top_k, top_p, rng: SplitMix64) -> int:
    """Temperature, then top-k, then top-p, then one draw walked through the
    descending weights (sampler.rs:113-183).  Ties are ordered by
    (value descending, id ascending); the reference leaves them unspecified."""
    import numpy as np

    logits = np.asarray(logits, dtype=np.float32)
    if temperature <= 0.0:
        return int(np.argmax(logits))
    scaled = (logits * np.float32(1.0 / np.float32(temperature))).astype(np.float32)
    order = sorted(range(len(scaled)), key=lambda i: (-float(scaled[i]), i))
    if top_k is not None and top_k < len(order):
        order = order[:top_k]
    largest = scaled[order[0]]
    w = np.exp((scaled[order] - largest).astype(np.float32)).astype(np.float32)
    total = np.float32(0.0)
    for x in w:
        total = np.float32(total + x)
    if top_p is not None and top_p < 1.0:
        target = np.float32(np.float32(top_p) * total)
        running = np.float32(0.0)
        keep = 1
        for i, x in enumerate(w):
            running = np.float32(running + x)
            keep = i + 1
            if running >= target:
                break
        order, w = order[:keep], w[:keep]
        total = np.float32(0.0)
        for x in w:
            total = np.float32(total + x)
    point = np.float32(np.float32(rng.next_f32()) * total)
    for i, x in zip(order, w):
        point = np.float32(point - x)
        if point <= 0.0:
            return int(i)
    return int(order[-1])
