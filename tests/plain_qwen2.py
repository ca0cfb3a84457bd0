"""Plain, slow implementation of the Qwen2 dense decoder, written from the reference's formulas.

Whole sequences only, no cache, one function for each part.  It shares no code with the
engine: it reads config.json with ``json`` and the weights with the ``safetensors`` package,
and computes on the CPU with torch.  Precisions follow the reference: matrix products,
bias, SiLU*up and residual sums in float32; the RMSNorm reduction, all RoPE trigonometry and
all of attention (dot, softmax, weighted sum) in float64, stored back as float32.

Every function cites the reference lines (paths under the upstream repository) it restates.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


# --------------------------------------------------------------------------------------
# configuration  (src/model/model_config.cpp:9-33)
# --------------------------------------------------------------------------------------
def read_config(model_dir) -> dict:
    """Typed view of config.json with the reference's defaults.

    src/model/model_config.cpp:13-31: num_key_value_heads defaults to num_attention_heads,
    head_dim to hidden_size / num_attention_heads, rope_theta to 10000, rms_norm_eps to 1e-6,
    tie_word_embeddings to false; model_type "qwen2" forces the q/k/v bias on.
    """
    raw = json.loads((Path(model_dir) / "config.json").read_text())
    heads = int(raw["num_attention_heads"])
    cfg = {
        "hidden_size": int(raw["hidden_size"]),
        "num_hidden_layers": int(raw["num_hidden_layers"]),
        "num_attention_heads": heads,
        "num_key_value_heads": int(raw.get("num_key_value_heads", heads)),
        "head_dim": int(raw["head_dim"]) if "head_dim" in raw else int(raw["hidden_size"]) // heads,
        "intermediate_size": int(raw["intermediate_size"]),
        "vocab_size": int(raw["vocab_size"]),
        "rope_theta": float(raw.get("rope_theta", 10000.0)),
        "rms_norm_eps": float(raw.get("rms_norm_eps", 1e-6)),
        "qkv_bias": True if raw.get("model_type", "") == "qwen2" else bool(raw.get("attention_bias", False)),
    }
    return cfg


def read_weights(model_dir) -> dict:
    """All tensors of model.safetensors as float32 (src/model/safetensors.cpp:81-91: every
    stored dtype is converted to fp32 on load)."""
    from safetensors import safe_open

    out = {}
    with safe_open(str(Path(model_dir) / "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            out[name] = f.get_tensor(name).to(torch.float32)
    return out


# --------------------------------------------------------------------------------------
# one function for each part
# --------------------------------------------------------------------------------------
def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """y = x . W^T + b with W stored [out, in]  (src/model/nn.cpp:15-43)."""
    assert x.dtype == torch.float32 and weight.dtype == torch.float32
    y = x @ weight.t()
    if bias is not None:
        y = y + bias
    return y


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """Sum of squares and scale in float64; eps inside the sqrt; the weight multiplies after
    the cast back to float32; plain w, not 1+w  (src/model/nn.cpp:59-70)."""
    xd = x.to(torch.float64)
    sum_sq = (xd * xd).sum(dim=-1, keepdim=True)
    scale = 1.0 / torch.sqrt(sum_sq / x.shape[-1] + eps)
    return (xd * scale).to(torch.float32) * weight


def silu_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """(g / (1 + exp(-g))) * u in float32  (src/model/nn.cpp:83-86)."""
    return (gate / (1.0 + torch.exp(-gate))) * up


def embedding(weight: torch.Tensor, ids) -> torch.Tensor:
    """Row lookup, no scaling; ids outside [0, vocab) are an error  (src/model/nn.cpp:90-108)."""
    ids = torch.as_tensor(ids, dtype=torch.int64)
    if ids.numel() and (int(ids.min()) < 0 or int(ids.max()) >= weight.shape[0]):
        raise IndexError("embedding: token id out of range")
    return weight[ids]


def rope(x: torch.Tensor, n_heads: int, head_dim: int, theta: float, positions) -> torch.Tensor:
    """Rotate-half RoPE  (src/model/nn.cpp:110-149).

    inv_freq_i = theta^(-2i/head_dim), angle = pos * inv_freq_i, and the pair is
    (i, i + head_dim/2): x_i' = x_i cos - x_{i+half} sin, x_{i+half}' = x_{i+half} cos + x_i sin,
    all in float64, stored as float32.  The whole head is rotated.
    """
    s = x.shape[0]
    half = head_dim // 2
    i = torch.arange(half, dtype=torch.float64)
    inv_freq = torch.pow(torch.tensor(theta, dtype=torch.float64), -2.0 * i / head_dim)
    pos = torch.as_tensor(positions, dtype=torch.float64).reshape(s, 1)
    ang = pos * inv_freq.reshape(1, half)  # [S, half]
    c = torch.cos(ang).reshape(s, 1, half)
    sn = torch.sin(ang).reshape(s, 1, half)
    xh = x.to(torch.float64).reshape(s, n_heads, head_dim)
    x1 = xh[..., :half]
    x2 = xh[..., half:]
    out = torch.cat([x1 * c - x2 * sn, x2 * c + x1 * sn], dim=-1)
    return out.to(torch.float32).reshape(s, n_heads * head_dim)


def attention(q, k, v, n_heads: int, n_kv_heads: int, head_dim: int, query_offset: int = 0,
              window: int | None = None) -> torch.Tensor:
    """Causal grouped-query attention  (src/model/nn.cpp:151-226).

    kv head of query head h is h // (n_heads / n_kv_heads); scores (q.k) * 1/sqrt(head_dim);
    query row i (absolute position query_offset + i) sees keys 0..query_offset+i; softmax with
    max subtraction; all in float64, output float32.  ``window`` is not in the reference: when
    given, key j is seen only if j > position - window (used by the tests of the engine's
    windowed attention part).
    """
    q_len, total = q.shape[0], k.shape[0]
    assert n_heads % n_kv_heads == 0 and query_offset + q_len <= total
    group = n_heads // n_kv_heads
    scale = 1.0 / math.sqrt(head_dim)
    qd = q.to(torch.float64).reshape(q_len, n_heads, head_dim)
    kd = k.to(torch.float64).reshape(total, n_kv_heads, head_dim)
    vd = v.to(torch.float64).reshape(total, n_kv_heads, head_dim)
    out = torch.empty(q_len, n_heads, head_dim, dtype=torch.float64)
    qpos = torch.arange(q_len).reshape(q_len, 1) + query_offset
    kpos = torch.arange(total).reshape(1, total)
    visible = kpos <= qpos
    if window is not None:
        visible = visible & (kpos > qpos - window)
    for h in range(n_heads):
        kvh = h // group
        scores = (qd[:, h, :] @ kd[:, kvh, :].t()) * scale  # [q_len, total]
        scores = scores.masked_fill(~visible, float("-inf"))
        scores = scores - scores.max(dim=-1, keepdim=True).values
        e = torch.exp(scores)
        p = e / e.sum(dim=-1, keepdim=True)
        out[:, h, :] = p @ vd[:, kvh, :]
    return out.to(torch.float32).reshape(q_len, n_heads * head_dim)


def attention_block(x, w: dict, prefix: str, cfg: dict, positions) -> torch.Tensor:
    """q/k/v projections with bias, RoPE on q and k, attention, o projection without bias
    (src/model/model.cpp:110-129)."""
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]

    def proj(name):
        b = w.get(f"{prefix}self_attn.{name}_proj.bias") if cfg["qkv_bias"] else None
        return linear(x, w[f"{prefix}self_attn.{name}_proj.weight"], b)

    q, k, v = proj("q"), proj("k"), proj("v")
    q = rope(q, nh, hd, cfg["rope_theta"], positions)
    k = rope(k, nkv, hd, cfg["rope_theta"], positions)
    a = attention(q, k, v, nh, nkv, hd, 0)
    return linear(a, w[f"{prefix}self_attn.o_proj.weight"])


def mlp_block(x, w: dict, prefix: str) -> torch.Tensor:
    """down(silu(gate(x)) * up(x)), no biases  (src/model/model.cpp:134-138)."""
    gate = linear(x, w[f"{prefix}mlp.gate_proj.weight"])
    up = linear(x, w[f"{prefix}mlp.up_proj.weight"])
    return linear(silu_mul(gate, up), w[f"{prefix}mlp.down_proj.weight"])


def forward(cfg: dict, w: dict, ids, rows=None) -> torch.Tensor:
    """Logits [S, vocab] of one whole sequence  (src/model/model.cpp:90-149).

    Per layer: x += attn(norm1(x)); x += mlp(norm2(x)).  Then the final norm and the LM head,
    which is lm_head.weight if that tensor exists and the embedding table otherwise
    (src/model/model.cpp:144-148).  ``rows``: the positions whose logits are wanted (all by
    default; a long sequence at a large vocabulary is asked for a few).
    """
    ids = list(ids)
    positions = list(range(len(ids)))
    x = embedding(w["model.embed_tokens.weight"], ids)
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        normed = rms_norm(x, w[p + "input_layernorm.weight"], cfg["rms_norm_eps"])
        x = x + attention_block(normed, w, p, cfg, positions)
        normed2 = rms_norm(x, w[p + "post_attention_layernorm.weight"], cfg["rms_norm_eps"])
        x = x + mlp_block(normed2, w, p)
    if rows is not None:
        x = x[torch.as_tensor(list(rows), dtype=torch.int64)]
    normed = rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"])
    head = w["lm_head.weight"] if "lm_head.weight" in w else w["model.embed_tokens.weight"]
    return linear(normed, head)


def forward_dir(model_dir, ids) -> torch.Tensor:
    return forward(read_config(model_dir), read_weights(model_dir), ids)


# --------------------------------------------------------------------------------------
# sampling  (src/sampler/sampler.cpp)
# --------------------------------------------------------------------------------------
def argmax(logits: torch.Tensor) -> int:
    """First maximum wins: scan with strict '>'  (src/sampler/sampler.cpp:13-21)."""
    best = 0
    vals = logits.tolist()
    for i in range(1, len(vals)):
        if vals[i] > vals[best]:
            best = i
    return best


def sample(logits: torch.Tensor, temperature: float, top_k: int, top_p: float, u: float) -> int:
    """Temperature -> top-k -> top-p -> inverse CDF  (src/sampler/sampler.cpp:25-88).

    The reference orders candidates by logit (descending), keeps top_k, takes
    p_i = exp(l_i/T - max/T) normalised, keeps the smallest prefix whose cumulative mass
    reaches top_p, and draws against u * nucleus_sum.  Here the uniform number ``u`` is an
    argument, the kept set is the same, and the draw walks the kept tokens in vocabulary order
    (the engine's documented order); tokens tied with the last kept one are kept too.
    """
    if temperature <= 0.0:
        return argmax(logits)
    vals = logits.to(torch.float64)
    vocab = vals.numel()
    order = sorted(range(vocab), key=lambda i: (-float(vals[i]), i))
    keep = vocab if not (0 < top_k < vocab) else top_k
    while keep < vocab and float(vals[order[keep]]) == float(vals[order[keep - 1]]):
        keep += 1  # the engine keeps every token tied with the k-th
    order = order[:keep]
    mx = float(vals[order[0]]) / temperature
    probs = [math.exp(float(vals[i]) / temperature - mx) for i in order]
    total = sum(probs)
    probs = [p / total for p in probs]
    nucleus = keep
    if top_p < 1.0:
        cum = 0.0
        for n, p in enumerate(probs):
            cum += p
            if cum >= top_p:
                nucleus = n + 1
                break
        # the engine keeps every token tied with the last kept one
        last = float(vals[order[nucleus - 1]])
        while nucleus < keep and float(vals[order[nucleus]]) == last:
            nucleus += 1
    kept = sorted(order[:nucleus])
    mass = {i: p for i, p in zip(order[:nucleus], probs[:nucleus])}
    threshold = u * sum(mass.values())
    cum = 0.0
    for i in kept:
        cum += mass[i]
        if threshold < cum:
            return i
    return kept[-1]
