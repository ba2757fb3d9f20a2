"""Plain PyTorch twins of the HIP operations, with the same signatures.

They serve two purposes: each GPU kernel test compares a kernel with its twin
here, at float32; and the tests that have no GPU substitute these functions for
the package's operations (see conftest.py, fixture `cpu_ops`) so that the cache,
the step function and the scheduler can be exercised on the CPU. They are not
part of the product, which has no host implementation.
"""

import math

import torch


def embed_rows(ids, table, out=None):
    res = table[ids.long()].float()
    if out is not None:
        out.copy_(res)
        return out
    return res


def swiglu(gate_up, out=None):
    g = gate_up[:, 0::2].float()          # gate and up interleaved
    u = gate_up[:, 1::2].float()
    res = (g / (1.0 + torch.exp(-g)) * u).to(gate_up.dtype)
    if out is not None:
        out.copy_(res)
        return out
    return res


def rmsnorm(x, weight, eps, out_dtype, delta=None, rows=None, write_back=True, out=None):
    src = x if rows is None else x[rows.long()]
    if delta is not None:
        d = delta if rows is None else delta[rows.long()]
        src = src + d.float()
        if write_back and rows is None:
            x.copy_(src)
    ms = (src * src).mean(dim=-1, keepdim=True)
    res = (src * torch.rsqrt(ms + eps) * weight.float()).to(out_dtype)
    if out is not None:
        out.copy_(res)
        return out
    return res


def rope_table(inv_freq, max_positions):
    p = torch.arange(max_positions, dtype=torch.float32, device=inv_freq.device)
    ang = p[:, None] * inv_freq[None, :]
    return torch.cat((ang.cos(), ang.sin()), dim=-1)


def qk_norm_rope_store(qkv, num_q_heads, num_kv_heads, head_dim, positions, seq_index,
                       q_weight=None, k_weight=None, eps=0.0, table=None,
                       block_table=None, k_cache=None, v_cache=None,
                       cu_seqlens_q=None, kv_lens=None, max_q_len=0, max_kv_len=0):
    Hq, Hkv, D = num_q_heads, num_kv_heads, head_dim
    T = qkv.shape[0]
    if table is not None and max_kv_len > table.shape[0]:
        raise ValueError("the step reaches position %d, the rotation table ends at %d"
                         % (max_kv_len - 1, table.shape[0] - 1))
    x = qkv.view(T, Hq + 2 * Hkv, D).float()
    q, k, v = x[:, :Hq], x[:, Hq:Hq + Hkv], x[:, Hq + Hkv:]

    def norm(t, w):
        if w is None:
            return t
        ms = (t * t).mean(dim=-1, keepdim=True)
        return t * torch.rsqrt(ms + eps) * w.float()

    def rotate(t):
        if table is None:
            return t
        R = table.shape[1]
        half = R // 2
        cs = table[positions.long()]
        cos, sin = cs[:, None, :half], cs[:, None, half:]
        a, b = t[..., :half], t[..., half:R]
        return torch.cat((a * cos - b * sin, b * cos + a * sin, t[..., R:]), dim=-1)

    q = rotate(norm(q, q_weight))
    k = rotate(norm(k, k_weight))
    qkv.view(T, Hq + 2 * Hkv, D)[:, :Hq] = q.to(qkv.dtype)
    if k_cache is not None:
        page = k_cache.shape[2]
        pos = positions.long()
        pages = block_table[seq_index.long(), pos // page].long()
        ok = pages >= 0
        k_cache[pages[ok], :, (pos % page)[ok]] = k[ok].to(k_cache.dtype)
        v_cache[pages[ok], :, :, (pos % page)[ok]] = v[ok].to(v_cache.dtype)     # values: (pages, Hkv, D, page)
    return qkv


def paged_attention(q, num_q_heads, k_cache, v_cache, block_table, cu_seqlens_q, kv_lens,
                    max_q_len, max_kv_len, scale, window=0, out=None, min_q_len=1, max_kv_len_of_many=None):
    T, Hq, D = q.shape
    Hkv, page = k_cache.shape[1], k_cache.shape[2]
    G = Hq // Hkv
    res = torch.zeros((T, Hq * D), dtype=torch.float32, device=q.device)
    cu = cu_seqlens_q.tolist()
    kvl = kv_lens.tolist()
    for b in range(len(kvl)):
        q0, q1 = cu[b], cu[b + 1]
        n, L = q1 - q0, kvl[b]
        if n == 0:
            continue
        nblk = -(-L // page)
        pages = block_table[b, :nblk].long().clamp(min=0)
        K = k_cache[pages].float().permute(1, 0, 2, 3).reshape(Hkv, nblk * page, D)[:, :L]
        V = v_cache[pages].float().permute(1, 0, 3, 2).reshape(Hkv, nblk * page, D)[:, :L]
        qpos = torch.arange(L - n, L, device=q.device)[:, None]
        kpos = torch.arange(L, device=q.device)[None, :]
        hidden = kpos > qpos
        if window > 0:
            hidden = hidden | (qpos - kpos >= window)
        qq = q[q0:q1].float()
        for h in range(Hq):
            s = (qq[:, h] @ K[h // G].T) * scale
            s = s.masked_fill(hidden, float("-inf"))
            p = torch.softmax(s, dim=-1)
            res[q0:q1, h * D:(h + 1) * D] = p @ V[h // G]
    res = res.to(q.dtype)
    if out is not None:
        out.copy_(res)
        return out
    return res


def decode_attention_takes(*args, **kwargs):
    return False            # the fused decoding kernel has no twin: its two halves above are the reference


def tile_weight(weight):
    return None


def linear(x, weight, out_dtype=None, out=None, tiled=None):
    res = (x.float() @ weight.float().T).to(out_dtype or x.dtype)
    if out is not None:
        out.copy_(res)
        return out
    return res


def linear_swiglu(x, weight, tiled=None):
    return swiglu(linear(x, weight))


def _uniform(seed, counter, n, device):
    # any fixed stream will do for the stand-in; the kernel's generator is tested on the GPU
    g = torch.Generator(device="cpu")
    g.manual_seed((int(seed) * 1000003 + int(counter)) & 0x7FFFFFFFFFFFFFFF)
    return torch.rand(n, generator=g).to(device)


def sample(logits, temperature, top_k, seed, counter, out=None, any_top_k=True):
    R, V = logits.shape
    res = torch.empty(R, dtype=torch.int32, device=logits.device)
    for r in range(R):
        row = logits[r]
        t = float(temperature[r])
        if t <= 0:
            res[r] = int(torch.argmax(row))
            continue
        z = row / t
        k = int(top_k[r])
        if 0 < k < V:
            kth = torch.topk(row, k).values[-1]
            z = z.masked_fill(row < kth, float("-inf"))
        u = _uniform(seed[r], counter[r], V, logits.device).clamp(1e-12, 1 - 1e-7)
        res[r] = int(torch.argmax(z - torch.log(-torch.log(u))))
    if out is not None:
        out.copy_(res)
        return out
    return res


ALL = ("embed_rows", "swiglu", "rmsnorm", "rope_table", "qk_norm_rope_store",
       "paged_attention", "decode_attention_takes", "linear", "linear_swiglu", "tile_weight", "sample")
