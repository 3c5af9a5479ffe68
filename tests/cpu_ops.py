"""A test double for the kernel layer: the same functions as ``rust_llm_inference_server_amd.ops``
in slow torch code on the CPU, so that the host logic around the kernels (batch layout, page
tables, cache manager, scheduler, engine loop) can be tested on a machine without a GPU.

It is installed by the ``cpu_ops`` fixture only; the package itself never falls back to it.
It follows the kernels' contracts (page layouts, in-place rotation, transposed values), not
their code.
"""
from __future__ import annotations


import torch


def embed(ids, table):
    return table[ids.long()].to(torch.float32)


def add_residual(resid, delta, round_parts=False):
    resid += delta.to(torch.float32)


def add_rmsnorm(resid, delta, weight, eps, out_dtype, rows=None, write_resid=True,
                round_parts=False):
    x = resid if delta is None else resid + delta.to(torch.float32)
    if rows is not None:
        x = x[rows.long()]
    elif delta is not None and write_resid:
        resid.copy_(x)
    ms = (x * x).mean(dim=-1, keepdim=True)
    return (x / torch.sqrt(ms + eps) * weight.to(torch.float32)).to(out_dtype)


def swiglu(gu):
    i = gu.shape[1] // 2
    g, u = gu[:, :i].float(), gu[:, i:].float()
    return (g / (1.0 + torch.exp(-g)) * u).to(gu.dtype)


def linear(x, w, out_dtype=None, partials=False):
    return (x.float() @ w.float().t()).to(out_dtype or x.dtype)


def pending_linear(x, w, out_dtype=None):
    return linear(x, w, out_dtype, partials=True)


def linear_swiglu(x, w_gate_up):
    return swiglu(linear(x, w_gate_up, x.dtype))


def can_fuse_norm_linear(resid, w, rows=None):
    return False


def rope_kv_write(qkv, num_heads, num_kv_heads, head_dim, cos, sin, positions, slots, k_pages,
                  v_pages, page_size, write_kv=True, interleaved=False):
    assert not interleaved, "the test double rotates halves only"
    T = qkv.shape[0]
    nh, nkv, d = num_heads, num_kv_heads, head_dim
    x = qkv.float()
    q = x[:, :nh * d].reshape(T, nh, d).clone()
    k = x[:, nh * d:(nh + nkv) * d].reshape(T, nkv, d).clone()
    v = x[:, (nh + nkv) * d:].reshape(T, nkv, d)
    if cos is not None:
        half = cos.shape[1]
        c = cos[positions.long()].unsqueeze(1)
        s = sin[positions.long()].unsqueeze(1)
        for t in (q, k):
            x1, x2 = t[..., :half].clone(), t[..., half:2 * half].clone()
            t[..., :half] = x1 * c - x2 * s
            t[..., half:2 * half] = x2 * c + x1 * s
    qkv[:, :nh * d] = q.reshape(T, nh * d).to(qkv.dtype)
    if write_kv:
        for t in range(T):
            page, off = int(slots[t]) // page_size, int(slots[t]) % page_size
            k_pages[page, :, off, :] = k[t].to(k_pages.dtype)
            v_pages[page, :, :, off] = v[t].to(v_pages.dtype)


def copy_pages(pages, src, dst):
    for s, d in zip(src.tolist(), dst.tolist()):
        pages[:, d] = pages[:, s]


def attention_planner(num_heads, num_kv_heads, head_dim, dtype, biased=False):
    from rust_llm_inference_server_amd.ops.attention_plan import AttentionPlanner
    return AttentionPlanner(num_heads, num_kv_heads, head_dim, matrix=dtype == torch.bfloat16)


def paged_attention(qkv, num_heads, num_kv_heads, head_dim, k_pages, v_pages, page_size,
                    block_tables, step, scale, window=None, force=None, plan=None,
                    bias_slopes=None, counters=None):
    assert bias_slopes is None, "the test double adds no bias"
    T = qkv.shape[0]
    nh, nkv, d = num_heads, num_kv_heads, head_dim
    g = nh // nkv
    q = qkv[:, :nh * d].float().reshape(T, nh, d)
    out = torch.zeros(T, nh * d)
    seq_of = step.seq_of_token.tolist()
    pos = step.positions.tolist()
    for t in range(T):
        table = block_tables[seq_of[t]].tolist()
        lo = max(0, pos[t] - window + 1) if window else 0
        keys = list(range(lo, pos[t] + 1))
        k = torch.stack([k_pages[table[p // page_size], :, p % page_size, :] for p in keys]).float()
        v = torch.stack([v_pages[table[p // page_size], :, :, p % page_size] for p in keys]).float()
        for h in range(nh):
            s = (k[:, h // g, :] @ q[t, h]) * scale
            p = torch.softmax(s, dim=0)
            out[t, h * d:(h + 1) * d] = p @ v[:, h // g, :]
    return out.to(qkv.dtype)


def rope_attention(qkv, num_heads, num_kv_heads, head_dim, cos, sin, positions, slots, k_pages,
                   v_pages, page_size, block_tables, step, scale, window=None, write_kv=True,
                   plan=None, interleaved=False, bias_slopes=None, counters=None):
    rope_kv_write(qkv, num_heads, num_kv_heads, head_dim, cos, sin, positions, slots, k_pages,
                  v_pages, page_size, write_kv=write_kv)
    return paged_attention(qkv, num_heads, num_kv_heads, head_dim, k_pages, v_pages, page_size,
                           block_tables, step, scale, window)


def _lowbias32(x):
    x ^= x >> 16
    x = (x * 0x7FEB352D) & 0xFFFFFFFF
    x ^= x >> 15
    x = (x * 0x846CA68B) & 0xFFFFFFFF
    x ^= x >> 16
    return x


def sample_rows(logits, keys, inv_temps):
    import numpy as np
    out = []
    for r in range(logits.shape[0]):
        x = logits[r].numpy().astype(np.float32)
        inv_t = float(inv_temps[r])
        if inv_t > 0:
            key = int(keys[r]) & 0xFFFFFFFF
            s = np.empty_like(x)
            for v in range(x.shape[0]):
                h = _lowbias32(key ^ ((v * 0x9E3779B9) & 0xFFFFFFFF))
                u = np.float32((np.float32(h >> 9) + np.float32(0.5)) * np.float32(1.0 / 8388608.0))
                s[v] = np.float32(x[v] * np.float32(inv_t)) + np.float32(-np.log(-np.log(u)))
            x = s
        out.append(int(np.argmax(x)))
    return torch.tensor(out, dtype=torch.int32)


def install(monkeypatch) -> None:
    """Replace the package's kernel functions with the ones above."""
    import rust_llm_inference_server_amd.ops as ops
    import rust_llm_inference_server_amd.engine.runner as runner
    for name in ("embed", "add_residual", "add_rmsnorm", "swiglu", "linear", "linear_swiglu",
                 "pending_linear", "can_fuse_norm_linear", "rope_kv_write", "rope_attention",
                 "copy_pages", "attention_planner", "paged_attention", "sample_rows"):
        monkeypatch.setattr(ops, name, globals()[name])
    monkeypatch.setattr(runner, "default_device", lambda: torch.device("cpu"))
