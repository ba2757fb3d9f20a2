"""The operations the model is made of, each a hand-written HIP kernel.

Every function checks its operands on the host (device, dtype, contiguity and
the shapes the kernel's grid assumes) and then launches on the current HIP
stream. Tensors must live on the GPU: there is no host implementation, and a
missing or unbuildable extension raises `ExtensionError`.

Activations and matrices are bfloat16 or float32 (the same for all operands of
one call unless stated); the residual stream, rotation tables, softmax
statistics and logits are float32 in both modes.
"""

import ctypes
import json
import os

import torch

from .build import ExtensionError, build_all, library, loaded_libraries

__all__ = [
    "ExtensionError",
    "build_all",
    "loaded_libraries",
    "embed_rows",
    "rmsnorm",
    "rope_table",
    "qk_norm_rope_store",
    "paged_attention",
    "decode_attention",
    "decode_attention_takes",
    "swiglu",
    "linear",
    "linear_plain",
    "linear_swiglu",
    "linear_residual_norm",
    "matmul_candidates",
    "matmul_kernels",
    "matmul_init",
    "matmul_table",
    "matmul_tuner",
    "matmul_rows_key",
    "matmul_fused_plan",
    "gemm_tiles",
    "gemm_tiles_configs",
    "gemm_tiles_splits",
    "matmul_plan",
    "stream_plan",
    "tile_weight",
    "sample",
    "measured_read_rate",
    "measured_matrix_rate",
]

_DT = {torch.float32: 0, torch.bfloat16: 1}
_UNSUPPORTED = 10002          # a launcher's refusal of a size it has no kernel for
_DECLINED = 1                 # the fused product of 17 to 128 rows did nothing: the plain product is faster here


class OperandError(ValueError):
    """An operand has a shape, dtype or placement the kernel does not take."""


def _ptr(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)   # the handle without a Stream object around it


def _stream():
    """The current device's current stream, as the launchers take it. Every operation asks, some
    hundreds of times in a step that is not a graph replay, so the short way is taken where this
    PyTorch has it (a fifth of such a step's host time otherwise)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(cond, message):
    if not cond:
        raise OperandError(message)


def _dev(*tensors):
    for t in tensors:
        if t is None:
            continue
        _need(t.is_cuda, "operands must be on the GPU; there is no host implementation")
        _need(t.is_contiguous(), "operands must be contiguous")


def _check(status, what):
    if status >= 20000:
        raise RuntimeError("%s failed: hipBLASLt status %d" % (what, status - 20000))
    if status != 0:
        raise RuntimeError("%s failed: HIP error %d" % (what, status))


_KINDS = {"plain": 0, "scaled": 1, "scaled_swiglu": 2, "residual": 3}
TABLE_FILE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "matmul_table.json")
_table_loaded = False


def _matmul():
    """The many-row product library, with the table of kernel choices loaded at its first use."""
    global _table_loaded
    lib = library("matmul")
    if not _table_loaded:
        _table_loaded = True
        if os.path.isfile(TABLE_FILE):
            with open(TABLE_FILE, encoding="utf-8") as fh:
                _add_to_table(lib, json.load(fh)["entries"])
    return lib


def _add_to_table(lib, entries):
    for e in entries:
        out = _DT[getattr(torch, e.get("out", "bfloat16"))]
        _check(lib.q3_matmul_table_add(_KINDS[e["kind"]], int(e["rows"]), int(e["N"]), int(e["K"]), out,
                                       int(e.get("library", 0)), int(e.get("own", -1)), int(e.get("splits", 1))),
               "matmul_table")


def matmul_init():
    """Allocate the many-row products' workspace and buffers on the current device now (a model
    being built calls this), so that no product inside a step allocates."""
    _check(_matmul().q3_matmul_init(), "matmul_init")


def matmul_table(entries, clear=False):
    """Load kernel choices: each entry {"kind": "plain" | "scaled" | "scaled_swiglu" | "residual",
    "rows": rounded rows (`matmul_rows_key`), "N", "K", "out": "bfloat16" | "float32",
    "library": the library's candidate number, or "own": tile shape and "splits": shares of K}.
    Sizes without an entry follow the rules of thumb. Sizes already met keep their kernel."""
    lib = _matmul()                      # the package's own table first, if it is not in yet
    if clear:
        _check(lib.q3_matmul_table_clear(), "matmul_table")
    _add_to_table(lib, entries)


def matmul_rows_key(kind, M):
    """The rows a table entry for `M` rows is filed under (sizes within a step of rows share one)."""
    return int(library("matmul").q3_matmul_rows_key(_KINDS[kind], int(M)))


def matmul_tuner(on):
    """With the tuner on, a product size first met outside a graph capture has its candidate
    kernels timed on the caller's operands and keeps the fastest for the life of the process
    (`matmul_plan`, `matmul_fused_plan` tell which): the way the table is made. Off (the
    default), kernels are chosen by the table and the rules alone, the same in every process."""
    _check(_matmul().q3_matmul_set_mode(1 if on else 0), "matmul_tuner")


def matmul_candidates(n):
    """How many of the vendor library's candidate kernels the tuner times for a new size."""
    _check(_matmul().q3_matmul_set_candidates(int(n)), "matmul_candidates")


def matmul_kernels(which):
    """Which kernels a product with many rows may go to: "both" (the table and the rules decide
    between the vendor library and the hand-written tiled kernel; the default), "library" (the
    library's first candidate), or "own" (the hand-written kernel wherever it takes the size: an
    inner size that is a multiple of 64). A change makes every size choose anew."""
    modes = {"both": 0, "library": 1, "own": 2}
    _need(which in modes, "which is one of %s" % ", ".join(sorted(modes)))
    _check(_matmul().q3_matmul_set_kernels(modes[which]), "matmul_kernels")


def matmul_plan(M, N, K, out_dtype=torch.bfloat16):
    """What serves a plain product of this size on the current device, or None if it has not
    been met: (candidates timed (1 without the tuner), index chosen, microseconds of the first
    candidate, of the chosen one, the hand-written kernel's tile shape if that serves it, else
    -1, over how many blocks it shares K out, the library's candidate number)."""
    info = (ctypes.c_float * 7)()
    if not _matmul().q3_matmul_plan(int(M), int(N), int(K), _DT[out_dtype], info):
        return None
    return int(info[0]), int(info[1]), float(info[2]), float(info[3]), int(info[4]), int(info[5]), int(info[6])


def matmul_fused_plan(kind, M, N, K):
    """What serves a product of 17 to 128 rows that carries a norm (`kind` "scaled",
    "scaled_swiglu" or "residual"): (tile shape or -1 for the library's product with the norm's
    work behind it, shares of K); None with the tuner on for a size it has not met."""
    info = (ctypes.c_int * 2)()
    if not _matmul().q3_matmul_fused_plan(_KINDS[kind], int(M), int(N), int(K), info):
        return None
    return int(info[0]), int(info[1])


def gemm_tiles_configs():
    """How many tile shapes the hand-written tiled product offers."""
    return int(library("matmul").q3_gemm_tiles_configs())


def gemm_tiles_splits(config, M, N, K):
    """Over how many blocks per tile the tiled product would share K out so that the chip is
    filled once (1: its tiles alone do)."""
    return int(library("matmul").q3_gemm_tiles_splits(int(config), int(M), int(N), int(K)))


def gemm_tiles(x, weight, config=0, out_dtype=None, swiglu=False, out=None, splits=1):
    """The hand-written tiled matrix-core product alone, with tile shape `config`: x (M, K) and
    weight (N, K) bfloat16, K a multiple of 64; out (M, N) bfloat16 or float32, or with `swiglu`
    (weight rows interleave gate and up) out (M, N / 2) bfloat16 = silu(gate) * up. With
    `splits` > 1 (N a multiple of 4) K is shared out over that many blocks per tile and their
    float32 partial products are added by a second kernel, which then also applies the activation."""
    _dev(x, weight, out)
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1], "x (M, K) and weight (N, K)")
    _need(x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16, "x and weight must be bfloat16")
    M, K = x.shape
    N = weight.shape[0]
    _need(M > 0 and K >= 64 and K % 64 == 0, "the inner size must be a multiple of 64")
    _need(0 <= config < gemm_tiles_configs(), "no such tile shape")
    out_dtype = out_dtype or torch.bfloat16
    _need(out_dtype in _DT and not (swiglu and (out_dtype != torch.bfloat16 or N % 2)),
          "out is bfloat16 or float32; with swiglu bfloat16 and an even number of weight rows")
    _need(1 <= splits <= min(64, K // 64) and (splits == 1 or N % 4 == 0),
          "K is shared out over 1 to min(64, K / 64) blocks, and then N is a multiple of 4")
    shape = (M, N // 2) if swiglu else (M, N)
    if out is None:
        out = torch.empty(shape, dtype=out_dtype, device=x.device)
    _need(out.shape == shape and out.dtype == out_dtype, "out must be %s of out_dtype" % (shape,))
    partials = torch.empty((splits * M * N,), dtype=torch.float32, device=x.device) if splits > 1 else None
    _check(library("matmul").q3_gemm_tiles(_ptr(x), _ptr(weight), _ptr(out), M, N, K, _DT[out_dtype],
                                           1 if swiglu else 0, int(config), int(splits), _ptr(partials), _stream()),
           "gemm_tiles")
    return out


def embed_rows(ids, table, out=None):
    """out[t, :] = float32(table[ids[t], :]). ids int32 (T,), table (V, H)."""
    _dev(ids, table, out)
    _need(ids.dtype == torch.int32 and ids.dim() == 1, "ids must be int32 (T,)")
    _need(table.dim() == 2 and table.dtype in _DT, "table must be (V, H) bfloat16 or float32")
    T, (V, H) = ids.shape[0], table.shape
    if out is None:
        out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    _need(out.shape == (T, H) and out.dtype == torch.float32, "out must be float32 (T, H)")
    if T:
        _check(library("elementwise").q3_embed_rows(
            _ptr(ids), _ptr(table), _ptr(out), T, H, V, _DT[table.dtype], _stream()), "embed_rows")
    return out


def swiglu(gate_up, out=None):
    """out[:, j] = silu(gate_up[:, 2j]) * gate_up[:, 2j + 1]: gate and up interleaved, (T, 2I) -> (T, I)."""
    _dev(gate_up, out)
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0 and gate_up.dtype in _DT,
          "gate_up must be (T, 2I) bfloat16 or float32")
    T, I = gate_up.shape[0], gate_up.shape[1] // 2
    if out is None:
        out = torch.empty((T, I), dtype=gate_up.dtype, device=gate_up.device)
    _need(out.shape == (T, I) and out.dtype == gate_up.dtype, "out must be (T, I) of the input's dtype")
    if T:
        _check(library("elementwise").q3_swiglu(
            _ptr(gate_up), _ptr(out), T, I, _DT[gate_up.dtype], _stream()), "swiglu")
    return out


def rmsnorm(x, weight, eps, out_dtype, delta=None, rows=None, write_back=True, out=None):
    """Root-mean-square norm of the float32 residual stream.

    For each output row r (source row s = rows[r], or r when rows is None):
    v = x[s] + delta[s] (delta optional), written back to x[s] if `write_back`
    and delta is given; out[r] = v * rsqrt(mean(v^2) + eps) * weight, rounded
    once to `out_dtype`. All arithmetic is float32.
    """
    _dev(x, weight, delta, rows, out)
    _need(x.dim() == 2 and x.dtype == torch.float32, "x must be float32 (T, H)")
    T, H = x.shape
    _need(weight.shape == (H,) and weight.dtype in _DT, "weight must be (H,) bfloat16 or float32")
    _need(out_dtype in _DT, "out_dtype must be bfloat16 or float32")
    if delta is not None:
        _need(delta.shape == (T, H) and delta.dtype == out_dtype,
              "delta must be (T, H) of the activation dtype")
    n_out = T
    if rows is not None:
        _need(rows.dtype == torch.int32 and rows.dim() == 1, "rows must be int32 (R,)")
        n_out = rows.shape[0]
    if out is None:
        out = torch.empty((n_out, H), dtype=out_dtype, device=x.device)
    _need(out.shape == (n_out, H) and out.dtype == out_dtype, "out must be (rows, H) of out_dtype")
    if n_out:
        _check(library("norm").q3_rmsnorm(
            _ptr(x), _ptr(delta), _ptr(weight), _ptr(rows), _ptr(out), n_out, T, H,
            ctypes.c_float(eps), _DT[out_dtype], _DT[weight.dtype],
            1 if (write_back and delta is not None) else 0, _stream()), "rmsnorm")
    return out


def rope_table(inv_freq, max_positions):
    """table[p] = [cos(p * inv_freq) | sin(p * inv_freq)], float32 (P, 2 * len(inv_freq))."""
    _dev(inv_freq)
    _need(inv_freq.dtype == torch.float32 and inv_freq.dim() == 1, "inv_freq must be float32 (D/2,)")
    half = inv_freq.shape[0]
    table = torch.empty((max_positions, 2 * half), dtype=torch.float32, device=inv_freq.device)
    _check(library("rotary").q3_rope_table(
        _ptr(inv_freq), _ptr(table), max_positions, half, _stream()), "rope_table")
    return table


def qk_norm_rope_store(qkv, num_q_heads, num_kv_heads, head_dim, positions, seq_index,
                       q_weight=None, k_weight=None, eps=0.0, table=None,
                       block_table=None, k_cache=None, v_cache=None,
                       cu_seqlens_q=None, kv_lens=None, max_q_len=0, max_kv_len=0):
    """Per-head RMSNorm of q and k, rotation by position, and the cache write, in one pass.

    qkv (T, (Hq + 2 Hkv) D) holds [q heads | k heads | v heads]. q heads are
    normalised with `q_weight`, rotated, and written back in place. k heads
    are normalised with `k_weight`, rotated, and stored; v heads are stored as
    they are. The store goes to page block_table[seq_index[t], pos // page] at
    slot pos % page of a key cache shaped (pages, Hkv, page, D) and a value
    cache shaped (pages, Hkv, D, page); entries below zero are skipped, and
    nothing is stored when no cache is given. Norm and
    rotation are each skipped when their operand is None. The rotation pairs
    element i with i + R/2 over the first R = table.shape[1] elements.
    `cu_seqlens_q`, `kv_lens` (after this step's write) and `max_q_len`
    describe the step's sequences; with them, bfloat16 steps use kernels with
    16-byte accesses that write values page by page. positions must then be
    kv_lens[b] - q_len[b] + i for row i of sequence b, as the step function
    makes them. `max_kv_len`: the step's last position + 1, if the caller knows it;
    a step that passes the end of the rotation table is refused (a position
    the table does not hold would go without its rotation).
    """
    _dev(qkv, positions, seq_index, q_weight, k_weight, table, block_table, k_cache, v_cache,
         cu_seqlens_q, kv_lens)
    if (cu_seqlens_q is None) != (kv_lens is None):
        raise OperandError("cu_seqlens_q and kv_lens are given together or not at all")
    if kv_lens is not None:
        _need(kv_lens.dtype == torch.int32 and cu_seqlens_q.dtype == torch.int32
              and cu_seqlens_q.shape == (kv_lens.shape[0] + 1,) and max_q_len > 0,
              "cu_seqlens_q int32 (B+1,), kv_lens int32 (B,), max_q_len > 0")
    Hq, Hkv, D = num_q_heads, num_kv_heads, head_dim
    _need(qkv.dim() == 2 and qkv.shape[1] == (Hq + 2 * Hkv) * D and qkv.dtype in _DT,
          "qkv must be (T, (Hq + 2 Hkv) D) bfloat16 or float32")
    T = qkv.shape[0]
    _need(1 <= D <= 512, "head_dim must be in 1..512")
    for t in (positions, seq_index):
        _need(t.dtype == torch.int32 and t.shape == (T,), "positions and seq_index must be int32 (T,)")
    w_dtype = 0
    if (q_weight is None) != (k_weight is None):
        raise OperandError("q_weight and k_weight are given together or not at all")
    if q_weight is not None:
        _need(q_weight.shape == (D,) and k_weight.shape == (D,) and q_weight.dtype in _DT
              and k_weight.dtype == q_weight.dtype, "norm weights must be (D,), same dtype")
        w_dtype = _DT[q_weight.dtype]
    rotary_dim, max_pos = 0, 0
    if table is not None:
        _need(table.dim() == 2 and table.dtype == torch.float32, "table must be float32 (P, R)")
        max_pos, rotary_dim = table.shape
        _need(rotary_dim % 2 == 0 and rotary_dim <= D, "rotary dim must be even and at most D")
        _need(max_kv_len <= max_pos, "the step reaches position %d, the rotation table ends at %d"
              % (max_kv_len - 1, max_pos - 1))
    page, stride = 0, 0
    if k_cache is not None:
        _need(v_cache is not None and block_table is not None, "a cache needs k, v and a block table")
        _need(k_cache.dim() == 4 and k_cache.shape[1] == Hkv and k_cache.shape[3] == D
              and v_cache.shape == (k_cache.shape[0], Hkv, D, k_cache.shape[2])
              and k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype,
              "caches must be keys (pages, Hkv, page, D) and values (pages, Hkv, D, page) of the activation dtype")
        _need(block_table.dim() == 2 and block_table.dtype == torch.int32, "block_table must be int32 (B, W)")
        page, stride = k_cache.shape[2], block_table.shape[1]
    if T:
        _check(library("rotary").q3_qk_norm_rope_store(
            _ptr(qkv), _ptr(q_weight), _ptr(k_weight), w_dtype, ctypes.c_float(eps),
            _ptr(table), rotary_dim, max_pos, _ptr(positions), _ptr(seq_index),
            _ptr(block_table), stride, 0 if block_table is None else block_table.shape[0],
            _ptr(k_cache), _ptr(v_cache), page, 0 if k_cache is None else k_cache.shape[0],
            T, Hq, Hkv, D, _DT[qkv.dtype], _ptr(cu_seqlens_q), _ptr(kv_lens),
            0 if kv_lens is None else kv_lens.shape[0], int(max_q_len), int(max_kv_len), _stream()),
            "qk_norm_rope_store")
    return qkv


def paged_attention(q, num_q_heads, k_cache, v_cache, block_table, cu_seqlens_q, kv_lens,
                    max_q_len, max_kv_len, scale, window=0, out=None, min_q_len=1, max_kv_len_of_many=None):
    """Causal softmax attention of packed query rows over paged keys and values.

    q is (T, Hq, D) seen through a row stride (a view of the qkv buffer is
    fine). Keys are cached as (pages, Hkv, page, D), values as
    (pages, Hkv, D, page). Sequence b owns rows cu_seqlens_q[b]..cu_seqlens_q[b+1]; its keys
    0..kv_lens[b]-1 lie in pages block_table[b, j // page]; its query row i sits
    at position kv_lens[b] - q_len + i and sees keys at positions <= its own
    and, if window > 0, fewer than `window` behind it. Query head h reads
    key head h // (Hq / Hkv). Softmax statistics and accumulation are float32.
    `max_q_len` and `min_q_len` bound the sequences' row counts (they choose
    between the kernels for few and for many rows; loose bounds cost time only).
    `max_kv_len_of_many`: the most keys of a sequence that brings many rows, if
    the caller knows it (it decides whether such sequences' keys are shared out
    over several blocks; `max_kv_len` stands in).

    bfloat16 with head size 64 or 128 and a page size that is a power of two from 16
    runs on the matrix cores; everything else (float32, other head sizes in
    steps of 16 up to 256, other page sizes) takes the general kernel.
    """
    _dev(k_cache, v_cache, block_table, cu_seqlens_q, kv_lens, out)
    _need(q.is_cuda and q.dim() == 3 and q.stride(2) == 1 and q.stride(1) == q.shape[2],
          "q must be (T, Hq, D) with contiguous heads")
    T, Hq, D = q.shape
    _need(Hq == num_q_heads, "q's head count differs from num_q_heads")
    _need(q.dtype in _DT and k_cache.dtype == q.dtype and v_cache.dtype == q.dtype,
          "q and the caches must share bfloat16 or float32")
    _need(k_cache.dim() == 4 and k_cache.shape[3] == D, "the key cache must be (pages, Hkv, page, D)")
    Hkv, page = k_cache.shape[1], k_cache.shape[2]
    _need(v_cache.shape == (k_cache.shape[0], Hkv, D, page), "the value cache must be (pages, Hkv, D, page)")
    _need(Hq % Hkv == 0, "query heads must be a multiple of key heads")
    _need(D % 16 == 0 and 16 <= D <= 256, "head_dim must be a multiple of 16 in 16..256, found %d" % D)
    B = kv_lens.shape[0]
    _need(cu_seqlens_q.dtype == torch.int32 and cu_seqlens_q.shape == (B + 1,), "cu_seqlens_q must be int32 (B+1,)")
    _need(kv_lens.dtype == torch.int32, "kv_lens must be int32 (B,)")
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.shape[0] >= B,
          "block_table must be int32 (B, W)")
    _need(block_table.shape[1] * page >= max_kv_len, "block_table is narrower than the longest sequence")
    _need(1 <= min_q_len <= max_q_len, "need 1 <= min_q_len <= max_q_len")
    if out is None:
        out = torch.empty((T, Hq * D), dtype=q.dtype, device=q.device)
    _need(out.shape == (T, Hq * D) and out.dtype == q.dtype, "out must be (T, Hq D)")
    if T and B:
        lib = library("attention")
        splits, workspace, prompt_splits, prompt_workspace = 1, None, 1, None
        if lib.q3_paged_attention_fast_path(Hq, Hkv, D, page, _DT[q.dtype]):
            if min_q_len * (Hq // Hkv) <= 16:
                splits = _splits(B, Hkv, max_kv_len)   # few rows per sequence: the keys go over several blocks
                if splits > 1:
                    lib.q3_paged_attention_workspace.restype = ctypes.c_long
                    n = lib.q3_paged_attention_workspace(B, Hkv, D, splits)
                    workspace = torch.empty((n,), dtype=torch.float32, device=q.device)
            if max_q_len * (Hq // Hkv) > 16:           # few long sequences over many keys: likewise
                longest = max_kv_len if max_kv_len_of_many is None else max_kv_len_of_many
                prompt_splits = lib.q3_paged_attention_prompt_splits(T, Hq, Hkv, int(longest))
                if prompt_splits > 1:
                    prompt_workspace = torch.empty((T * Hq * prompt_splits * (D + 2),), dtype=torch.float32,
                                                   device=q.device)
        _check(lib.q3_paged_attention(
            _ptr(q), q.stride(0), _ptr(out), _ptr(k_cache), _ptr(v_cache), k_cache.shape[0],
            _ptr(block_table), block_table.shape[1], _ptr(cu_seqlens_q), _ptr(kv_lens),
            B, T, Hq, Hkv, D, page, ctypes.c_float(scale), int(window), int(max_q_len), int(min_q_len),
            int(max_kv_len), _DT[q.dtype], splits, _ptr(workspace), prompt_splits, _ptr(prompt_workspace),
            _stream()),
            "paged_attention")
    return out


def _splits(B, Hkv, max_kv_len):
    """Into how many blocks a sequence's keys are split when a step has few rows per sequence:
    until the chip is full, two blocks a compute unit and no more (the blocks beyond 512 run when
    the others have ended: 24 requests of 8 key heads over 768 keys take 27 us in two parts and 31
    in three, 12 requests over 2,000 keys 30 us in five parts and 35 in six); beyond 32 parts the
    merge costs more than the split gains. Two corrections to that, both measured with 8 key heads
    of 128: with 8,192 keys or more a block's work dwarfs its start and what counts is that the
    blocks come in even rounds, so at least eight parts are taken up to 384 (sequence, key head)
    pairs and four beyond (33 sequences over 8,200 keys: 257 us whole, 199 in eight parts; 40: 272
    and 232; 24: 156 in two parts, 143 in eight; 48: 295 whole, 274 in four; over 32,000 keys 955
    and 713, 1,022 and 832, 557 and 511, 1,110 and 1,018); and 257 to 320 pairs over fewer keys are
    split in three (33 sequences over 2,100 keys: 78 us whole, 70 in three; 40: 85 and 78; from 48
    sequences on one part is the fastest there)."""
    pairs = B * Hkv
    splits = max(1, min(max_kv_len // 64, 512 // pairs, 32))
    if max_kv_len >= 8192 and pairs < 512:
        splits = max(splits, 8 if pairs <= 384 else 4)
    elif 256 < pairs <= 320 and max_kv_len >= 1024:
        splits = 3
    return splits


def decode_attention_takes(num_q_heads, num_kv_heads, head_dim, page_size, dtype, rotary_dim=0):
    """Whether `decode_attention` serves these sizes (the caller then skips `qk_norm_rope_store`)."""
    if dtype != torch.bfloat16:
        return False
    return bool(library("attention").q3_decode_attention_takes(
        num_q_heads, num_kv_heads, head_dim, page_size, _DT[dtype], int(rotary_dim)))


def decode_attention(qkv, num_q_heads, num_kv_heads, head_dim, k_cache, v_cache, block_table, cu_seqlens_q,
                     kv_lens, max_kv_len, scale, window=0, q_weight=None, k_weight=None, eps=0.0, table=None,
                     store=True):
    """`qk_norm_rope_store` and `paged_attention` of a step in which every sequence brings one
    token, in one kernel: qkv (B, (Hq + 2 Hkv) D) bfloat16 holds the raw projections of
    sequence b's token in row b; the new key and value go to position kv_lens[b] - 1 of the
    caches (unless `store` is false: a layer that reads another layer's cache) and the
    attention output (B, Hq D) is returned. qkv is left as it was."""
    _dev(qkv, k_cache, v_cache, block_table, cu_seqlens_q, kv_lens, q_weight, k_weight, table)
    Hq, Hkv, D = num_q_heads, num_kv_heads, head_dim
    B = kv_lens.shape[0]
    _need(qkv.dtype == torch.bfloat16 and qkv.shape == (B, (Hq + 2 * Hkv) * D), "qkv must be bfloat16 (B, (Hq + 2 Hkv) D)")
    _need(k_cache.dtype == torch.bfloat16 and v_cache.dtype == torch.bfloat16 and k_cache.dim() == 4
          and k_cache.shape[1] == Hkv and k_cache.shape[3] == D, "key cache must be bfloat16 (pages, Hkv, page, D)")
    page = k_cache.shape[2]
    _need(v_cache.shape == (k_cache.shape[0], Hkv, D, page), "value cache must be (pages, Hkv, D, page)")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.shape[0] >= B, "block table int32 (B, blocks)")
    _need(cu_seqlens_q.dtype == torch.int32 and cu_seqlens_q.shape == (B + 1,), "cu_seqlens_q int32 (B + 1,)")
    _need(kv_lens.dtype == torch.int32, "kv_lens int32 (B,)")
    _need((q_weight is None) == (k_weight is None), "q and k norm weights come together")
    w_dtype = 0
    if q_weight is not None:
        _need(q_weight.shape == (D,) and k_weight.shape == (D,) and q_weight.dtype == k_weight.dtype
              and q_weight.dtype in _DT, "norm weights (D,) of one dtype")
        w_dtype = _DT[q_weight.dtype]
    rotary_dim = max_pos = 0
    if table is not None:
        _need(table.dtype == torch.float32 and table.dim() == 2, "rotation table float32 (positions, rotary_dim)")
        max_pos, rotary_dim = table.shape
        _need(max_kv_len <= max_pos, "the step reaches position %d, the rotation table ends at %d"
              % (max_kv_len - 1, max_pos - 1))
    _need(decode_attention_takes(Hq, Hkv, D, page, qkv.dtype, rotary_dim), "sizes the decoding kernel does not take")
    out = torch.empty((B, Hq * D), dtype=qkv.dtype, device=qkv.device)
    if B:
        lib = library("attention")
        splits, workspace = _splits(B, Hkv, max_kv_len), None
        if splits > 1:
            lib.q3_paged_attention_workspace.restype = ctypes.c_long
            workspace = torch.empty((lib.q3_paged_attention_workspace(B, Hkv, D, splits),), dtype=torch.float32,
                                    device=qkv.device)
        _check(lib.q3_decode_attention(
            _ptr(qkv), _ptr(out), _ptr(k_cache), _ptr(v_cache), k_cache.shape[0], _ptr(block_table),
            block_table.shape[1], _ptr(cu_seqlens_q), _ptr(kv_lens), B, Hq, Hkv, D, page, ctypes.c_float(scale),
            int(window), splits, _ptr(workspace), _ptr(q_weight), _ptr(k_weight), w_dtype, ctypes.c_float(eps),
            _ptr(table), int(rotary_dim), int(max_pos), 1 if store else 0, int(max_kv_len), _stream()),
            "decode_attention")
    return out


def tile_weight(weight):
    """A copy of a bfloat16 matrix (N, K) in the order the few-row product kernel reads it:
    [N / 16 slabs][K / 32 steps][64 lanes][8], lane = (n % 16) + 16 * ((k % 32) // 8), rows
    padded with zeros to a multiple of 16. None if the matrix is not bfloat16 or K is not a
    multiple of 32 (the row-major kernel then serves it)."""
    if weight.dtype != torch.bfloat16 or weight.dim() != 2 or weight.shape[1] % 32:
        return None
    N, K = weight.shape
    N16 = -(-N // 16) * 16
    if N16 != N:
        weight = torch.cat((weight, weight.new_zeros((N16 - N, K))), dim=0)
    tiles = weight.view(N16 // 16, 16, K // 32, 4, 8).permute(0, 2, 3, 1, 4)   # slab, step, group, row, 8
    return tiles.contiguous().view(-1)


FEW_ROWS = 16                   # the few-row kernel's rows: one matrix instruction's worth of x
SMALL_WEIGHT_BYTES = 18 << 20   # up to this size the few-row kernel serves 32 rows, up to half of it 64


def few_rows_limit(weight):
    """Up to how many rows of x the few-row kernel serves a product with `weight` from its tiled
    copy: 16, or 32 or 64 for a small weight. The kernel works on 16 rows of x at a time; more
    rows are further sets of blocks that read the weight again. For a small weight that reading
    comes out of the caches and costs less than what the tiled kernel needs beyond 16 rows, a
    second kernel that adds its shares of K. Measured inside a graph, the product with its norm's
    work, few-row kernel against tiled kernel, in microseconds: 8 MB (4,096 x 1,024) at 24, 32, 48
    and 64 rows 5.8, 6.1, 8.4, 9.6 against 9.2, 9.6, 10.1, 10.9; 17 MB at 24, 32 and 48 rows 8.1,
    8.8, 11.9 against 9.9, 10.3, 11.5; 50 MB at 24 rows 20.0 against 15.0."""
    size = weight.numel() * weight.element_size()
    return FEW_ROWS * (4 if 2 * size <= SMALL_WEIGHT_BYTES else 2 if size <= SMALL_WEIGHT_BYTES else 1)


def sums_stride(M):
    """Columns of a tensor of rows' partial sums of squares for M rows (see `linear_residual_norm`)."""
    return -(-M // 16) * 16


def _tiled_ok(tiled, weight, M):
    if tiled is None or not 1 <= M <= few_rows_limit(weight):
        return False
    N, K = weight.shape
    _need(tiled.is_cuda and tiled.dtype == torch.bfloat16 and tiled.is_contiguous()
          and tiled.numel() == (-(-N // 16) * 16) * K and K % 32 == 0,
          "the tiled copy does not belong to this weight")
    return True


def _check_sums(sums, M):
    _dev(sums)
    _need(sums.dtype == torch.float32 and sums.dim() == 2 and sums.shape[1] == sums_stride(M) and sums.shape[0] > 0
          and sums.is_contiguous(), "row sums must be float32 (P, M rounded up to 16)")


def _row_sums_args(unscaled, M, K):
    """The few-row kernel's arguments for rows that still lack their 1 / rms factor: `unscaled` =
    (sums (P, M rounded up to 16) float32, eps, width) as `linear_residual_norm` leaves them."""
    if unscaled is None:
        return None, 0, ctypes.c_float(0.0), 0, 0
    sums, eps, width = unscaled
    _check_sums(sums, M)
    _need(width == K, "the rows' width must be the product's inner size")
    return _ptr(sums), sums.shape[0], ctypes.c_float(eps), int(width), sums.shape[1]


FUSED_ROWS_FEW, FUSED_ROWS_MOST = FEW_ROWS, 128


def fused_rows_take(weight, M):
    """Whether the tiled kernel carries a norm for `M` rows of a product with `weight` (N, K):
    more than 16 rows, at most 128 (beyond that the vendor library's products with the norms as
    kernels of their own are faster), bfloat16, K a multiple of 64 and N of 4. (Where the few-row
    kernel takes the rows too, a small weight's 17 to 32 or 64, that one is used.)"""
    return (FUSED_ROWS_FEW < M <= FUSED_ROWS_MOST and weight.dtype == torch.bfloat16 and weight.dim() == 2
            and weight.shape[1] % 64 == 0 and weight.shape[0] % 4 == 0 and weight.is_contiguous())


def _tiles_scaled(x, weight, out, unscaled, swiglu, what):
    sums, eps, width = unscaled
    M, K = x.shape
    _check_sums(sums, M)
    _need(width == K, "the rows' width must be the product's inner size")
    _need(x.is_contiguous() and out.is_contiguous(), "operands must be contiguous")
    _check(_matmul().q3_tiles_scaled(
        _ptr(x), _ptr(weight), _ptr(out), M, weight.shape[0], K, _DT[out.dtype], 1 if swiglu else 0, _ptr(sums),
        sums.shape[0], sums.shape[1], ctypes.c_float(eps), int(width), _stream()), what)
    return out


STREAM_ROWS_MOST = 96


STREAM_ROWS_LEAST = 9      # of a gate/up product that runs whole; every other product from 17 rows


def stream_plan(M, N, K, swiglu=False):
    """How the weight-streaming kernel for 17 to 96 rows (9 to 96 of a gate/up product with the
    activation) would serve a product with a tile-ordered weight of (N, K) under the current
    settings: the slabs of 16 weight rows per block (6 or 4), or None where it leaves the product
    to the other kernels (small weights, slabs that do not fill the chip in one round of blocks,
    `matmul_kernels` other than "both", the tuner on)."""
    ws = _matmul().q3_stream_plan(int(M), int(N), int(K), 1 if swiglu else 0)
    return int(ws) if ws else None


def _stream_product(x, weight, tiled, out, swiglu, unscaled, what):
    """The product by the weight-streaming kernel, if it takes it: True if `out` is written."""
    M, K = x.shape
    N = weight.shape[0]
    least = STREAM_ROWS_LEAST if swiglu else FEW_ROWS + 1
    if tiled is None or not least <= M <= STREAM_ROWS_MOST or K % 32 or not x.is_contiguous() or not out.is_contiguous():
        return False
    _need(tiled.is_cuda and tiled.dtype == torch.bfloat16 and tiled.is_contiguous()
          and tiled.numel() == (-(-N // 16) * 16) * K, "the tiled copy does not belong to this weight")
    sums, chunks, stride, eps, width = None, 0, 0, 0.0, 0
    if unscaled is not None:
        sums, eps, width = unscaled
        _check_sums(sums, M)
        _need(width == K, "the rows' width must be the product's inner size")
        chunks, stride = sums.shape
    status = _matmul().q3_stream_product(
        _ptr(x), _ptr(tiled), _ptr(out), M, N, K, _DT[out.dtype], 1 if swiglu else 0, _ptr(sums), chunks, stride,
        ctypes.c_float(eps), int(width), _stream())
    if status == _DECLINED:
        return False
    _check(status, what)
    return True


def linear(x, weight, out_dtype=None, out=None, tiled=None, unscaled=None):
    """out = x @ weight^T with float32 accumulation. x (M, K), weight (N, K).
    `tiled` is `tile_weight(weight)`, if the caller keeps one: few rows are then served from it.
    `unscaled` (see `linear_residual_norm`) says that x's rows still lack their 1 / rms factor;
    the product's rows receive it. Only the few-row kernel on a tiled weight does this.

    float32 operands take a float32 kernel with no reduced-precision mode;
    bfloat16 operands with at most 16 rows (32 or 64 with the tiled copy of a small
    weight, `few_rows_limit`) take a weight-streaming matrix-core kernel; bfloat16 with
    more rows is the vendor library's product or the tiled kernel's.
    """
    _dev(x, weight, out)
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1], "x (M, K) and weight (N, K)")
    _need(x.dtype in _DT and weight.dtype == x.dtype, "x and weight must share bfloat16 or float32")
    M, K = x.shape
    N = weight.shape[0]
    out_dtype = out_dtype or x.dtype
    _need(out_dtype in _DT, "out dtype must be bfloat16 or float32")
    _need(not (x.dtype == torch.float32 and out_dtype != torch.float32), "float32 inputs give float32 output")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=x.device)
    _need(out.shape == (M, N) and out.dtype == out_dtype, "out must be (M, N) of out_dtype")
    if M and x.dtype == torch.bfloat16 and _tiled_ok(tiled, weight, M):
        sums, sums_rows, eps, width, stride = _row_sums_args(unscaled, M, K)
        _check(library("gemm").q3_linear_tiled(
            _ptr(x), _ptr(tiled), _ptr(out), M, N, K, _DT[out_dtype], 0, sums, sums_rows, eps, width,
            None, None, 0, None, stride, _stream()), "linear")
        return out
    if M and x.dtype == torch.bfloat16 and (unscaled is None or fused_rows_take(weight, M)) \
            and _stream_product(x, weight, tiled, out, False, unscaled, "linear"):
        return out
    if unscaled is not None and x.dtype == torch.bfloat16 and fused_rows_take(weight, M):
        return _tiles_scaled(x, weight, out, unscaled, False, "linear")
    _need(unscaled is None, "unscaled rows need bfloat16 and few rows with a tiled weight (few_rows_limit), or 17 to "
          "128 rows with an inner size that is a multiple of 64")
    if M and x.dtype == torch.bfloat16 and not library("gemm").q3_linear_is_skinny(M, N, K, 1):
        # bfloat16 products with many rows go to the vendor library (hipBLASLt), as the
        # reference's engine uses its vendor library for them, or to the hand-written tiled
        # kernel, as a table of sizes and a rule of thumb say; accumulation is float32.
        # Few rows take the weight-streaming kernel below.
        _need(x.is_contiguous() and weight.is_contiguous() and out.is_contiguous(), "operands must be contiguous")
        status = _matmul().q3_matmul(_ptr(x), _ptr(weight), _ptr(out), M, N, K, _DT[out_dtype], _stream())
        if status == _UNSUPPORTED:
            # a size neither hipBLASLt nor the tiled kernel has a kernel for (an odd inner size,
            # say): plain multiply-adds with float32 sums
            linear_plain(x, weight, out)
        else:
            _check(status, "matmul")
    elif M:
        _check(library("gemm").q3_linear(
            _ptr(x), _ptr(weight), _ptr(out), M, N, K, _DT[x.dtype], _DT[out_dtype], _stream()), "linear")
    return out


def linear_plain(x, weight, out):
    """out = x @ weight^T by plain multiply-adds with float32 sums, for any size: what serves a
    bfloat16 product with more than 16 rows that neither the vendor library nor the tiled
    kernel takes, and every float32 product."""
    _dev(x, weight, out)
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1] and x.dtype in _DT
          and weight.dtype == x.dtype, "x (M, K) and weight (N, K) of one dtype")
    M, K = x.shape
    N = weight.shape[0]
    _need(out.shape == (M, N) and out.dtype in _DT and not (x.dtype == torch.float32 and out.dtype != torch.float32),
          "out must be (M, N); float32 inputs give float32 output")
    lib = library("gemm")
    _need(M > 16 or x.dtype == torch.float32 or not lib.q3_linear_is_skinny(M, N, K, 1),
          "bfloat16 products of up to 16 rows are the weight-streaming kernel's")
    if M:
        _check(lib.q3_linear(_ptr(x), _ptr(weight), _ptr(out), M, N, K, _DT[x.dtype], _DT[out.dtype], _stream()),
               "linear_plain")
    return out


def linear_swiglu(x, weight, tiled=None, unscaled=None):
    """swiglu(x @ weight^T) for a weight whose rows interleave gate and up (row 2i gate's, row
    2i + 1 up's): (M, K) x (2I, K) -> (M, I). With few bfloat16 rows the activation is the
    product kernel's epilogue; otherwise it is the product followed by `swiglu`.
    `unscaled`: as for `linear`."""
    _dev(x, weight)
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1] and weight.shape[0] % 2 == 0,
          "x (M, K) and weight (2I, K)")
    _need(x.dtype in _DT and weight.dtype == x.dtype, "x and weight must share bfloat16 or float32")
    M, K = x.shape
    N = weight.shape[0]
    if x.dtype == torch.bfloat16 and tiled is not None and STREAM_ROWS_LEAST <= M <= FEW_ROWS and N % 4 == 0:
        # a whole gate/up product of 9 to 16 rows: the streaming kernel, where it takes the size
        if unscaled is not None:
            _need(unscaled[0].dim() == 2 and unscaled[0].shape[1] == sums_stride(M), "row sums (P, M rounded up to 16)")
        out = torch.empty((M, N // 2), dtype=x.dtype, device=x.device)
        if _stream_product(x, weight, tiled, out, True, unscaled, "linear_swiglu"):
            return out
    if M and x.dtype == torch.bfloat16 and _tiled_ok(tiled, weight, M):
        out = torch.empty((M, N // 2), dtype=x.dtype, device=x.device)
        sums, sums_rows, eps, width, stride = _row_sums_args(unscaled, M, K)
        _check(library("gemm").q3_linear_tiled(
            _ptr(x), _ptr(tiled), _ptr(out), M, N, K, 1, 1, sums, sums_rows, eps, width,
            None, None, 0, None, stride, _stream()), "linear_swiglu")
        return out
    if M and x.dtype == torch.bfloat16 and tiled is not None and FEW_ROWS < M <= STREAM_ROWS_MOST \
            and (unscaled is None or fused_rows_take(weight, M)):
        out = torch.empty((M, N // 2), dtype=x.dtype, device=x.device)
        if _stream_product(x, weight, tiled, out, True, unscaled, "linear_swiglu"):
            return out
    if unscaled is not None and x.dtype == torch.bfloat16 and fused_rows_take(weight, M):
        out = torch.empty((M, N // 2), dtype=x.dtype, device=x.device)
        return _tiles_scaled(x, weight, out, unscaled, True, "linear_swiglu")
    _need(unscaled is None, "unscaled rows need bfloat16 and few rows with a tiled weight (few_rows_limit), or 17 to "
          "128 rows with an inner size that is a multiple of 64")
    if M and library("gemm").q3_linear_is_skinny(M, N, K, _DT[x.dtype]):
        out = torch.empty((M, N // 2), dtype=x.dtype, device=x.device)
        _check(library("gemm").q3_linear_swiglu(_ptr(x), _ptr(weight), _ptr(out), M, N, K, _DT[x.dtype], _stream()),
               "linear_swiglu")
        return out
    return swiglu(linear(x, weight, tiled=tiled))


def linear_residual_norm(x, weight, tiled, residual, norm_weight):
    """residual += x @ weight^T, and the next norm's input prepared in the same kernel.

    x (M, K) bfloat16, weight (N, K); residual (M, N) float32 is updated in place (the product
    is rounded to bfloat16 before the addition, as a product written out and added by the norm
    kernel would be). Returns (values, sums): values (M, N) bfloat16 = residual * norm_weight,
    and sums (P, M rounded up to 16) float32, the rows' sums of squares of the new residual in P
    partial sums (row m of the stream in column m). The norm's result is
    values * rsqrt(sum / N + eps) row by row; `linear` and `linear_swiglu` apply that factor to
    their products when given `unscaled=(sums, eps, N)`.

    Up to `few_rows_limit(weight)` rows, with the weight's tiled copy and N a multiple of 16, it
    is the few-row kernel's epilogue (P = N / 16, partial sums of 16 columns). With more rows, up
    to 128 (`fused_rows_take`; `tiled` is not used), the tiled kernel's partial products are added
    by a second kernel that does the same (P = ceil(N / 1024)). There the result is None, and
    nothing was done, for a size at which the plain product (`linear`) followed by the norm's own
    kernel is the faster way."""
    _dev(x, weight, tiled, residual, norm_weight)
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1], "x (M, K) and weight (N, K)")
    M, K = x.shape
    N = weight.shape[0]
    _need(residual.shape == (M, N) and residual.dtype == torch.float32 and residual.is_contiguous(),
          "residual must be float32 (M, N)")
    _need(norm_weight.shape == (N,) and norm_weight.dtype in _DT and norm_weight.is_contiguous(), "norm weight (N,)")
    values = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    few = x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and N % 16 == 0 and _tiled_ok(tiled, weight, M)
    if not few and x.dtype == torch.bfloat16 and fused_rows_take(weight, M):
        _need(x.is_contiguous(), "x must be contiguous")
        lib = _matmul()
        sums = torch.empty((lib.q3_tiles_residual_chunks(N), sums_stride(M)), dtype=torch.float32, device=x.device)
        status = lib.q3_tiles_residual(
            _ptr(x), _ptr(weight), M, N, K, _ptr(residual), _ptr(norm_weight), _DT[norm_weight.dtype], _ptr(values),
            _ptr(sums), sums.shape[1], _stream())
        if status == _DECLINED:
            return None
        _check(status, "linear_residual_norm")
        return values, sums
    _need(few, "bfloat16, a tiled weight with a width that is a multiple of 16 and no more rows than few_rows_limit, "
          "or 17 to 128 rows with an inner size that is a multiple of 64")
    sums = torch.empty((N // 16, sums_stride(M)), dtype=torch.float32, device=x.device)
    _check(library("gemm").q3_linear_tiled(
        _ptr(x), _ptr(tiled), _ptr(values), M, N, K, 1, 2, None, 0, ctypes.c_float(0.0), 0,
        _ptr(residual), _ptr(norm_weight), _DT[norm_weight.dtype], _ptr(sums), sums.shape[1], _stream()),
        "linear_residual_norm")
    return values, sums


def sample(logits, temperature, top_k, seed, counter, out=None, any_top_k=True):
    """One token per row of float32 logits (R, V).

    Row r: temperature[r] <= 0 takes the arg-max (lowest index among equals).
    Otherwise it draws from softmax(logits / temperature) restricted, when
    top_k[r] > 0, to logits not below the k-th largest; the draw is the
    arg-max of logits / temperature + Gumbel noise from a counter-based
    generator keyed by (seed[r], counter[r], column), so a request's tokens do
    not depend on what else is in the batch. `any_top_k=False` promises that no row has a
    top_k in effect, which saves the selection pass.
    """
    _dev(logits, temperature, top_k, seed, counter, out)
    _need(logits.dim() == 2 and logits.dtype == torch.float32, "logits must be float32 (R, V)")
    R, V = logits.shape
    _need(temperature.shape == (R,) and temperature.dtype == torch.float32, "temperature float32 (R,)")
    _need(top_k.shape == (R,) and top_k.dtype == torch.int32, "top_k int32 (R,)")
    _need(seed.shape == (R,) and seed.dtype == torch.int64, "seed int64 (R,)")
    _need(counter.shape == (R,) and counter.dtype == torch.int32, "counter int32 (R,)")
    if out is None:
        out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    _need(out.shape == (R,) and out.dtype == torch.int32, "out int32 (R,)")
    if R:
        lib = library("sampling")
        lib.q3_sample_workspace.restype = ctypes.c_long
        workspace = torch.empty((lib.q3_sample_workspace(R, V) + 7) // 8, dtype=torch.int64, device=logits.device)
        _check(lib.q3_sample(
            _ptr(logits), _ptr(temperature), _ptr(top_k), _ptr(seed), _ptr(counter), _ptr(out),
            R, V, 1 if any_top_k else 0, _ptr(workspace), _stream()), "sample")
    return out


def measured_read_rate(gigabytes=4.0, repeats=5):
    """Bytes per second at which a kernel reads a buffer of `gigabytes` that no cache holds (the
    fastest of `repeats` passes): what this GPU's memory delivers to a long, plain read."""
    lib = library("probes")
    count = int(gigabytes * 1e9) // 16 * 16
    buffer = torch.zeros(count, dtype=torch.uint8, device="cuda")
    sink = torch.zeros(1, dtype=torch.float32, device="cuda")
    best = 0.0
    for blocks in (2048, 4096, 8192):
        for _ in range(repeats):
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            begin.record()
            _check(lib.q3_probe_read(_ptr(buffer), ctypes.c_size_t(count), _ptr(sink), blocks, _stream()), "probe_read")
            end.record()
            end.synchronize()
            best = max(best, count / (begin.elapsed_time(end) * 1e-3))
    return best


def measured_matrix_rate(repeats=5, shape=None, blocks=256 * 8, iters=4096):
    """Floating-point operations per second of the bfloat16 matrix instructions with their
    operands in registers, all compute units busy: the better of v_mfma_f32_16x16x32_bf16 and
    v_mfma_f32_32x32x16_bf16 (`shape` 0 or 1 asks for one of them)."""
    lib = library("probes")
    sink = torch.zeros(1, dtype=torch.float32, device="cuda")
    flops = ctypes.c_double(0.0)
    best = 0.0
    for which in ((0, 1) if shape is None else (shape,)):
        for _ in range(repeats):
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            begin.record()
            _check(lib.q3_probe_mfma(int(blocks), int(iters), which, _ptr(sink), ctypes.byref(flops), _stream()),
                   "probe_mfma")
            end.record()
            end.synchronize()
            best = max(best, flops.value / (begin.elapsed_time(end) * 1e-3))
    return best
