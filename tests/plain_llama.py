"""A plain, slow implementation of the dense Llama decoder, written from the reference's
formulas: whole sequences, no cache, one function per part, torch on the CPU.  It imports
nothing from the package under test; the GPU engine is compared with it.

Every function cites the reference lines (under /root/reference/) it is written from.  The
reference was read, not run.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import torch


# ------------------------------------------------------------------------- config
def read_config(folder: str) -> dict:
    """The keys the forward pass needs (crates/model/src/config.rs:5-26)."""
    with open(os.path.join(folder, "config.json")) as f:
        c = json.load(f)
    if c.get("head_dim") is None:                     # config.rs:44-47
        c["head_dim"] = c["hidden_size"] // c["num_attention_heads"]
    c.setdefault("tie_word_embeddings", False)        # config.rs:19-20
    c.setdefault("rope_scaling", None)                # config.rs:16-17
    return c


def read_weights(folder: str, dtype=torch.float32) -> Dict[str, torch.Tensor]:
    """All tensors of the folder's safetensors files by name, cast on the CPU
    (crates/model/src/llama.rs:59-63, 125-138).  Uses the safetensors package's own reader."""
    from safetensors import safe_open
    out = {}
    for fn in sorted(os.listdir(folder)):
        if fn.endswith(".safetensors"):
            with safe_open(os.path.join(folder, fn), framework="pt", device="cpu") as f:
                for name in f.keys():
                    out[name] = f.get_tensor(name).to(dtype)
    return out


# -------------------------------------------------------------------------- parts
def embedding(table: torch.Tensor, ids: Sequence[int]) -> torch.Tensor:
    """x[t] = E[ids[t]]; no scaling (crates/model/src/layers.rs:199-204; llama.rs:256-262)."""
    return table[torch.tensor(list(ids), dtype=torch.long)]


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x / sqrt(mean(x^2) + eps) * w over the last axis; the weight multiplies directly
    (crates/model/src/layers.rs:112-118, 141-146: candle's rms_norm(x, weight, eps))."""
    ms = (x * x).mean(dim=-1, keepdim=True)
    return x / torch.sqrt(ms + eps) * w


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """Bias-free x W^T with W (out, in) (crates/model/src/layers.rs:17-19, 72-99)."""
    return x @ w.t()


def inv_freqs(head_dim: int, theta: float, scaling: Optional[dict]) -> torch.Tensor:
    """Inverse frequencies in float32 with llama3 scaling (crates/model/src/rope.rs:19-49)."""
    f32 = torch.float32
    out = []
    th = torch.tensor(theta, dtype=f32)
    for i in range(0, head_dim, 2):                                       # rope.rs:22-25
        e = torch.tensor(float(i), dtype=f32) / torch.tensor(float(head_dim), dtype=f32)
        out.append(1.0 / torch.pow(th, e))
    base = torch.stack(out)
    if not scaling or scaling.get("rope_type", scaling.get("type")) != "llama3":
        return base                                                       # rope.rs:47
    factor = torch.tensor(float(scaling["factor"]), dtype=f32)            # rope.rs:28-32
    low = torch.tensor(float(scaling["low_freq_factor"]), dtype=f32)
    high = torch.tensor(float(scaling["high_freq_factor"]), dtype=f32)
    old = torch.tensor(float(scaling["original_max_position_embeddings"]), dtype=f32)
    low_wl, high_wl = old / low, old / high
    res = []
    for f in base:                                                        # rope.rs:33-45
        wl = torch.tensor(2.0, dtype=f32) * torch.tensor(math.pi, dtype=f32) / f
        if wl < high_wl:
            res.append(f)
        elif wl > low_wl:
            res.append(f / factor)
        else:
            smooth = (old / wl - low) / (high - low)
            res.append((1.0 - smooth) * f / factor + smooth * f)
    return torch.stack(res)


def rope_tables(inv: torch.Tensor, positions: Sequence[int]):
    """cos/sin rows for the given absolute positions: angle = float32(p) * inv_freq, in
    float32 (crates/model/src/rope.rs:61-78, 92-98)."""
    pos = torch.tensor(list(positions), dtype=torch.float32).reshape(-1, 1)
    ang = pos * inv.to(torch.float32).reshape(1, -1)
    return torch.cos(ang), torch.sin(ang)


def rope_apply(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Rotate-half on ``x (heads, T, d)``: o_j = x_j cos_j - x_{j+d/2} sin_j,
    o_{j+d/2} = x_{j+d/2} cos_j + x_j sin_j (crates/model/src/rope.rs:5-8, 111-117: candle's
    non-interleaved ``rope``)."""
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    c, s = cos.to(x.dtype), sin.to(x.dtype)
    return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1)


def causal_mask(seq: int, start_pos: int, window: Optional[int] = None) -> torch.Tensor:
    """Additive mask (seq, start_pos + seq): 0 where col <= row + start_pos, -inf beyond
    (crates/model/src/attention.rs:225-233).  ``window`` (not in the reference) also blocks
    col <= row + start_pos - window."""
    total = start_pos + seq
    rows = torch.arange(start_pos, total).reshape(seq, 1)
    cols = torch.arange(total).reshape(1, total)
    blocked = cols > rows
    if window:
        blocked = blocked | (cols <= rows - window)
    m = torch.zeros(seq, total)
    m[blocked] = float("-inf")
    return m


def gqa_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                  mask: Optional[torch.Tensor], scale: Optional[float] = None) -> torch.Tensor:
    """Grouped-query attention, q (nh, n, d), k and v (nkv, total, d) -> (nh, n, d).
    Query head h uses KV head h // n_rep: q is reshaped to (nkv, n_rep * n, d); scores =
    q k^T * (1/sqrt(d)), mask added, softmax over keys, times v
    (crates/model/src/attention.rs:166-171, 204-223)."""
    nh, n, d = q.shape
    nkv, total, _ = k.shape
    n_rep = nh // nkv
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    qg = q.reshape(nkv, n_rep * n, d)                                  # attention.rs:209
    scores = (qg @ k.transpose(1, 2)) * scale                          # attention.rs:210
    if mask is not None:                                               # attention.rs:212-217
        scores = (scores.reshape(nkv, n_rep, n, total) + mask.to(scores.dtype)).reshape(
            nkv, n_rep * n, total)
    probs = torch.softmax(scores, dim=-1)                              # attention.rs:219
    return (probs @ v).reshape(nh, n, v.shape[-1])                     # attention.rs:220-222


def attention_layer(x: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, cfg: dict,
                    inv: torch.Tensor, start_pos: int = 0,
                    window: Optional[int] = None) -> torch.Tensor:
    """q/k/v projections, head split, rotation of q and k, attention over the whole sequence,
    head merge, output projection (crates/model/src/attention.rs:61-103)."""
    T = x.shape[0]
    nh, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    q = linear(x, w[f"{prefix}.q_proj.weight"]).reshape(T, nh, d).transpose(0, 1)
    k = linear(x, w[f"{prefix}.k_proj.weight"]).reshape(T, nkv, d).transpose(0, 1)
    v = linear(x, w[f"{prefix}.v_proj.weight"]).reshape(T, nkv, d).transpose(0, 1)
    cos, sin = rope_tables(inv, range(start_pos, start_pos + T))
    q, k = rope_apply(q, cos, sin), rope_apply(k, cos, sin)           # attention.rs:88-93
    mask = causal_mask(T, 0, window) if T > 1 else None               # llama.rs:241-245
    o = gqa_attention(q, k, v, mask)
    o = o.transpose(0, 1).reshape(T, nh * d)                          # attention.rs:98-101
    return linear(o, w[f"{prefix}.o_proj.weight"])


def swiglu_mlp(x: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str) -> torch.Tensor:
    """down(silu(gate(x)) * up(x)), silu(z) = z * sigmoid(z)
    (crates/model/src/layers.rs:179-186)."""
    g = linear(x, w[f"{prefix}.gate_proj.weight"])
    u = linear(x, w[f"{prefix}.up_proj.weight"])
    return linear(g * torch.sigmoid(g) * u, w[f"{prefix}.down_proj.weight"])


def forward(w: Dict[str, torch.Tensor], cfg: dict, ids: Sequence[int],
            dtype=torch.float32) -> torch.Tensor:
    """Logits (T, vocab) of one whole sequence (crates/model/src/llama.rs:218-273, 306-311):
    embed; per layer x += attn(norm(x)); x += mlp(norm(x)); final norm; lm_head (the embedding
    table when tied, llama.rs:152-156)."""
    w = {k: v.to(dtype) for k, v in w.items()}
    inv = inv_freqs(cfg["head_dim"], cfg["rope_theta"], cfg.get("rope_scaling"))
    eps = cfg["rms_norm_eps"]
    x = embedding(w["model.embed_tokens.weight"], ids)
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}"
        h = rms_norm(x, w[f"{p}.input_layernorm.weight"], eps)               # llama.rs:265
        x = x + attention_layer(h, w, f"{p}.self_attn", cfg, inv)            # llama.rs:266-267
        h = rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], eps)      # llama.rs:268
        x = x + swiglu_mlp(h, w, f"{p}.mlp")                                 # llama.rs:269-270
    x = rms_norm(x, w["model.norm.weight"], eps)                             # llama.rs:272
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings") else w["lm_head.weight"]
    return linear(x, head).to(torch.float32)                                 # llama.rs:285


def greedy_generate(w: Dict[str, torch.Tensor], cfg: dict, prompt: Sequence[int],
                    max_tokens: int) -> List[int]:
    """Greedy continuation by recomputing the whole sequence each step."""
    ids = list(prompt)
    out = []
    for _ in range(max_tokens):
        nxt = argmax(forward(w, cfg, ids)[-1])
        out.append(nxt)
        ids.append(nxt)
    return out


# ----------------------------------------------------------------------- sampling
def perplexity(w: Dict[str, torch.Tensor], cfg: dict, tokens: Sequence[int], bos: int, ctx: int,
               max_windows: int = 0) -> dict:
    """crates/engine/src/perplexity.rs:26-80: windows of ``ctx`` tokens, the first token of
    each replaced by BOS, rows ctx/2 .. ctx-2 scored against the tokens that follow them;
    ppl = exp(mean NLL), one standard error = ppl * sqrt(var / n)."""
    windows = len(tokens) // ctx
    if max_windows > 0:
        windows = min(windows, max_windows)
    first = ctx // 2
    nll: List[float] = []
    for wi in range(windows):
        chunk = [int(t) for t in tokens[wi * ctx:(wi + 1) * ctx]]
        chunk[0] = bos
        logits = forward(w, cfg, chunk).double()
        for row in range(first, ctx - 1):
            r = logits[row]
            nll.append(float(torch.logsumexp(r, 0) - r[chunk[row + 1]]))
    n = len(nll)
    mean = sum(nll) / n
    var = max(sum(x * x for x in nll) / n - mean * mean, 0.0)
    return {"ppl": math.exp(mean), "ppl_stderr": math.exp(mean) * math.sqrt(var / n),
            "mean_nll": mean, "tokens_scored": n, "windows": windows}


def lowbias32(x: int) -> int:
    """crates/model/src/sampling.rs:11-18."""
    x &= 0xFFFFFFFF
    x ^= x >> 16
    x = (x * 0x7FEB352D) & 0xFFFFFFFF
    x ^= x >> 15
    x = (x * 0x846CA68B) & 0xFFFFFFFF
    x ^= x >> 16
    return x


def row_key(seed: int, position: int) -> int:
    """crates/model/src/sampling.rs:21-23."""
    lo, hi = seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF
    return lowbias32(lowbias32(lowbias32(lo) ^ hi) ^ (position & 0xFFFFFFFF))


def uniform(h: int) -> float:
    """Top 23 bits plus a half, in float32 (crates/model/src/sampling.rs:58-63)."""
    import numpy as np
    return float(np.float32(np.float32((h >> 9)) + np.float32(0.5)) * np.float32(1.0 / 8388608.0))


def gumbel(key: int, v: int) -> float:
    """-ln(-ln(u)) in float32 (crates/model/src/sampling.rs:53-56)."""
    import numpy as np
    u = np.float32(uniform(lowbias32(key ^ ((v * 0x9E3779B9) & 0xFFFFFFFF))))
    return float(-np.log(-np.log(u, dtype=np.float32), dtype=np.float32))


def argmax(row: torch.Tensor) -> int:
    """Largest value, ties to the lowest index (crates/engine/src/sampler.rs:237-246)."""
    best = 0
    vals = row.tolist()
    for i, x in enumerate(vals):
        if x > vals[best]:
            best = i
    return best


def sample_scores(row: torch.Tensor, key: int, inv_t: float):
    """The scores the device sampler compares (crates/model/src/sampling.rs:84-100):
    s = x * inv_t + gumbel(key, v) when inv_t > 0 else x, float32."""
    import numpy as np
    x = row.to(torch.float32).numpy()
    if not inv_t > 0:
        return x
    v = np.arange(x.shape[0], dtype=np.uint64)
    h = (np.uint64(key) ^ ((v * np.uint64(0x9E3779B9)) & np.uint64(0xFFFFFFFF))).astype(np.uint64)
    h = _lowbias32_np(h)
    u = (np.float32(1.0 / 8388608.0) * ((h >> np.uint64(9)).astype(np.float32) + np.float32(0.5))).astype(np.float32)
    g = -np.log(-np.log(u, dtype=np.float32), dtype=np.float32)
    return (x * np.float32(inv_t)).astype(np.float32) + g


def sample_row(row: torch.Tensor, key: int, inv_t: float) -> int:
    """One row of the device sampler's host reference: largest score, ties to the lowest id."""
    import numpy as np
    s = sample_scores(row, key, inv_t)
    best, best_v = float("-inf"), 2 ** 32 - 1
    top = np.flatnonzero(s == s.max()) if not np.isnan(s).all() else []
    for v in top:
        if s[v] > best or (s[v] == best and v < best_v):
            best, best_v = float(s[v]), int(v)
    if best_v == 2 ** 32 - 1:
        best_v = 0
    return best_v


def _lowbias32_np(x):
    import numpy as np
    m = np.uint64(0xFFFFFFFF)
    x = x & m
    x ^= x >> np.uint64(16)
    x = (x * np.uint64(0x7FEB352D)) & m
    x ^= x >> np.uint64(15)
    x = (x * np.uint64(0x846CA68B)) & m
    x ^= x >> np.uint64(16)
    return x


def apply_repetition_penalty(logits: List[float], history: Sequence[int], penalty: float) -> List[float]:
    """Each distinct seen token: l > 0 ? l / p : l * p (crates/engine/src/sampler.rs:223-235)."""
    out = list(logits)
    for t in set(int(t) for t in history):
        if t < len(out):
            out[t] = out[t] / penalty if out[t] > 0 else out[t] * penalty
    return out
