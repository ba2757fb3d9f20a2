"""Each HIP kernel alone against its plain PyTorch twin, at sizes other than the
tiny models', in float32 (tight) and bfloat16 (against the float32 twin fed the
same bfloat16-representable inputs)."""

import math

import pytest
import torch

import torch_ops

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def _ops():
    from qwen3_from_scratch_amd import ops
    return ops


def _rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).cuda()


def _tol(dtype):
    return dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1.6e-2, atol=1e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,H,V", [(1, 40, 7), (37, 1000, 331), (5, 4096, 100)])
def test_embed_rows(dtype, T, H, V):
    table = _rand((V, H), dtype, 1)
    ids = torch.randint(0, V, (T,), dtype=torch.int32).cuda()
    got = _ops().embed_rows(ids, table)
    assert got.dtype == torch.float32
    assert torch.equal(got, torch_ops.embed_rows(ids, table))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,I", [(1, 24), (9, 1000), (130, 333)])
def test_swiglu(dtype, T, I):
    x = _rand((T, 2 * I), dtype, 2, scale=3.0)
    got = _ops().swiglu(x)
    want = torch_ops.swiglu(x.float())
    torch.testing.assert_close(got.float(), want, **_tol(dtype))
    zero = torch.zeros((3, 2 * I), dtype=dtype, device="cuda")
    assert torch.count_nonzero(_ops().swiglu(zero)) == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("wdtype", DTYPES)
@pytest.mark.parametrize("T,H", [(1, 16), (7, 1000), (33, 5120), (2, 13000), (3, 1001), (2, 20000), (5, 4096)])
def test_rmsnorm_plain_add_and_rows(dtype, wdtype, T, H):
    ops = _ops()
    x = _rand((T, H), torch.float32, 3, scale=2.0)
    w = (1 + 0.3 * _rand((H,), torch.float32, 4)).to(wdtype)
    d = _rand((T, H), dtype, 5)
    eps = 1e-3
    tol = _tol(dtype)
    torch.testing.assert_close(ops.rmsnorm(x.clone(), w, eps, dtype).float(),
                               torch_ops.rmsnorm(x.clone(), w, eps, torch.float32), **tol)
    x1, x2 = x.clone(), x.clone()
    got = ops.rmsnorm(x1, w, eps, dtype, delta=d)
    want = torch_ops.rmsnorm(x2, w, eps, torch.float32, delta=d)
    torch.testing.assert_close(got.float(), want, **tol)
    torch.testing.assert_close(x1, x2, rtol=0, atol=0)          # the stream was updated in place
    rows = torch.tensor([T - 1, 0, T // 2], dtype=torch.int32).cuda()
    x3 = x.clone()
    got = ops.rmsnorm(x3, w, eps, dtype, delta=d, rows=rows, write_back=False)
    want = torch_ops.rmsnorm(x.clone(), w, eps, torch.float32, delta=d, rows=rows, write_back=False)
    torch.testing.assert_close(got.float(), want, **tol)
    assert torch.equal(x3, x)                                    # and left alone here


def test_rope_table_matches_closed_form():
    # src/qwen3_from_scratch: test/models/test_rotary.py:19-54 (head 128, base 1e5, 1024 positions)
    D, base, P = 128, 100000.0, 1024
    inv = 1.0 / (base ** (torch.arange(0, D, 2, dtype=torch.float) / D))
    table = _ops().rope_table(inv.cuda(), P).cpu()
    freqs = torch.outer(torch.arange(P, dtype=torch.float), inv)
    assert table.shape == (P, D)
    torch.testing.assert_close(table[:, :D // 2], freqs.cos(), rtol=0, atol=1e-5)
    torch.testing.assert_close(table[:, D // 2:], freqs.sin(), rtol=0, atol=1e-5)
    # far positions: angles of tens of thousands of radians need full range reduction
    P = 40960
    table = _ops().rope_table(inv.cuda(), P).cpu()
    freqs = torch.outer(torch.arange(P, dtype=torch.float), inv)
    torch.testing.assert_close(table[-64:, :D // 2], freqs[-64:].cos(), rtol=0, atol=2e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("Hq,Hkv,D,R,page", [(4, 2, 16, 16, 16), (6, 3, 48, 48, 8), (5, 1, 80, 32, 4),
                                             (32, 8, 128, 128, 16), (2, 2, 256, 256, 16), (7, 1, 64, 64, 8),
                                             (8, 4, 32, 32, 32), (3, 3, 128, 128, 64)])
def test_qk_norm_rope_store(dtype, Hq, Hkv, D, R, page):
    ops = _ops()
    T, B, P = 23, 3, 300
    inv = 1.0 / (10000.0 ** (torch.arange(0, R, 2, dtype=torch.float) / R))
    table = torch_ops.rope_table(inv, P).cuda()
    qkv = _rand((T, (Hq + 2 * Hkv) * D), dtype, 6)
    qw = (1 + 0.2 * _rand((D,), torch.float32, 7)).to(dtype)
    kw = (1 + 0.2 * _rand((D,), torch.float32, 8)).to(dtype)
    seq = torch.tensor([0] * 9 + [1] * 1 + [2] * 13, dtype=torch.int32).cuda()
    pos = torch.tensor(list(range(40, 49)) + [77] + list(range(0, 13)), dtype=torch.int32).cuda()
    W = 100 // page + 1
    pages = torch.randperm(3 * W)[: 3 * W].view(3, W).to(torch.int32)
    pages[2, 1] = -1                                   # a page given back: nothing is stored there
    bt = pages.cuda()
    npages = 3 * W
    kc = torch.full((npages, Hkv, page, D), -7.0, dtype=dtype, device="cuda")
    vc = torch.full((npages, Hkv, D, page), -7.0, dtype=dtype, device="cuda")
    kc2, vc2 = kc.float(), vc.float()
    got = qkv.clone()
    ops.qk_norm_rope_store(got, Hq, Hkv, D, pos, seq, q_weight=qw, k_weight=kw, eps=1e-5, table=table,
                           block_table=bt, k_cache=kc, v_cache=vc)
    want = qkv.float().clone()
    torch_ops.qk_norm_rope_store(want, Hq, Hkv, D, pos, seq, q_weight=qw, k_weight=kw, eps=1e-5,
                                 table=table, block_table=bt, k_cache=kc2, v_cache=vc2)
    tol = _tol(dtype)
    torch.testing.assert_close(got.float()[:, :Hq * D], want[:, :Hq * D], **tol)
    assert torch.equal(got[:, Hq * D:], qkv[:, Hq * D:])            # k and v columns of qkv untouched
    torch.testing.assert_close(kc.float(), kc2, **tol)
    assert torch.equal(vc.float(), vc2)                             # values are copied bit for bit
    assert (kc2 == -7.0).any()                                      # untouched slots keep the sentinel
    # the same step described by its sequences: the kernels with 16-byte accesses where they apply
    cu = torch.tensor([0, 9, 10, 23], dtype=torch.int32).cuda()
    kvl = torch.tensor([49, 78, 13], dtype=torch.int32).cuda()
    kc3 = torch.full_like(kc, -7.0)
    vc3 = torch.full_like(vc, -7.0)
    got3 = qkv.clone()
    ops.qk_norm_rope_store(got3, Hq, Hkv, D, pos, seq, q_weight=qw, k_weight=kw, eps=1e-5, table=table,
                           block_table=bt, k_cache=kc3, v_cache=vc3, cu_seqlens_q=cu, kv_lens=kvl, max_q_len=13)
    torch.testing.assert_close(got3.float()[:, :Hq * D], want[:, :Hq * D], **tol)
    assert torch.equal(got3[:, Hq * D:], qkv[:, Hq * D:])
    torch.testing.assert_close(kc3.float(), kc2, **tol)
    assert torch.equal(vc3.float(), vc2)
    # and a step of few tokens per sequence (values go with the same launch)
    few_pos = torch.tensor([48, 77, 12], dtype=torch.int32).cuda()
    few_seq = torch.tensor([0, 1, 2], dtype=torch.int32).cuda()
    few = qkv[:3].clone()
    few_want = few.float().clone()
    kc4, vc4 = torch.full_like(kc, -7.0), torch.full_like(vc, -7.0)
    kc5, vc5 = kc4.float(), vc4.float()
    ops.qk_norm_rope_store(few, Hq, Hkv, D, few_pos, few_seq, q_weight=qw, k_weight=kw, eps=1e-5, table=table,
                           block_table=bt, k_cache=kc4, v_cache=vc4,
                           cu_seqlens_q=torch.tensor([0, 1, 2, 3], dtype=torch.int32).cuda(), kv_lens=kvl, max_q_len=1)
    torch_ops.qk_norm_rope_store(few_want, Hq, Hkv, D, few_pos, few_seq, q_weight=qw, k_weight=kw, eps=1e-5,
                                 table=table, block_table=bt, k_cache=kc5, v_cache=vc5)
    torch.testing.assert_close(few.float()[:, :Hq * D], few_want[:, :Hq * D], **tol)
    torch.testing.assert_close(kc4.float(), kc5, **tol)
    assert torch.equal(vc4.float(), vc5)
    # without norm, without rotation, without cache: q comes back as it went in
    same = qkv.clone()
    ops.qk_norm_rope_store(same, Hq, Hkv, D, pos, seq)
    assert torch.equal(same, qkv)


def _paged_case(dtype, B, Hq, Hkv, D, page, q_lens, kv_lens, seed, spread=True):
    g = torch.Generator().manual_seed(seed)
    T = sum(q_lens)
    W = max(-(-L // page) for L in kv_lens) + 1
    npages = B * W + 3
    perm = torch.randperm(npages, generator=g)[: B * W].view(B, W).to(torch.int32)
    for b in range(B):      # entries beyond the last page: the kernels may read them, but never the pages they name
        perm[b, -(-kv_lens[b] // page):] = -1
    kc = (torch.randn((npages, Hkv, page, D), generator=g)).to(dtype).cuda()
    vc = (torch.randn((npages, Hkv, D, page), generator=g)).to(dtype).cuda()   # values: transposed in the page
    q = (torch.randn((T, Hq, D), generator=g) * (2.0 if spread else 1.0)).to(dtype).cuda()
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32).cuda()
    kvl = torch.tensor(kv_lens, dtype=torch.int32).cuda()
    return q, kc, vc, perm.cuda(), cu, kvl


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("Hq,Hkv,D,page", [(4, 2, 16, 16), (8, 2, 32, 8), (6, 3, 48, 16), (5, 5, 80, 4),
                                           (32, 8, 128, 16), (3, 1, 256, 32), (16, 2, 64, 16),
                                           (40, 8, 128, 16), (64, 8, 128, 16), (14, 2, 64, 64), (9, 3, 128, 32),
                                           (8, 2, 128, 128), (6, 2, 64, 256), (4, 1, 48, 128)])
@pytest.mark.parametrize("window", [0, 19])
def test_paged_attention_mixed_batch(dtype, Hq, Hkv, D, page, window):
    ops = _ops()
    q_lens = [1, 37, 4, 1, 70]
    kv_lens = [16, 37, 20, 131, 200]
    q, kc, vc, bt, cu, kvl = _paged_case(dtype, 5, Hq, Hkv, D, page, q_lens, kv_lens, 9)
    scale = D ** -0.5
    got = ops.paged_attention(q, Hq, kc, vc, bt, cu, kvl, max(q_lens), max(kv_lens), scale, window=window)
    want = torch_ops.paged_attention(q.float(), Hq, kc.float(), vc.float(), bt, cu, kvl, max(q_lens),
                                     max(kv_lens), scale, window=window)
    tol = dict(rtol=1e-4, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(got.float(), want, **tol)


@pytest.mark.parametrize("Hq,Hkv,D,page", [(32, 8, 128, 16), (8, 1, 64, 32), (3, 3, 128, 64), (16, 1, 128, 16),
                                           (8, 2, 128, 128), (4, 1, 64, 256)])
@pytest.mark.parametrize("window", [0, 300])
def test_paged_attention_decoding_batches(Hq, Hkv, D, page, window):
    """Single tokens over contexts from one key to thousands: one split and many."""
    ops = _ops()
    for kv_lens in ([1, 2, 31, 32, 33, 255, 256, 257, 1000, 3001], [700] * 3, [4097], [15] * 70):
        B = len(kv_lens)
        q, kc, vc, bt, cu, kvl = _paged_case(torch.bfloat16, B, Hq, Hkv, D, page, [1] * B, kv_lens, 20 + B)
        scale = D ** -0.5
        got = ops.paged_attention(q, Hq, kc, vc, bt, cu, kvl, 1, max(kv_lens), scale, window=window)
        want = torch_ops.paged_attention(q.float(), Hq, kc.float(), vc.float(), bt, cu, kvl, 1, max(kv_lens),
                                         scale, window=window)
        torch.testing.assert_close(got.float(), want, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("Hq,Hkv,D,page", [(32, 8, 128, 16), (16, 2, 64, 16), (14, 2, 64, 64), (9, 3, 128, 32),
                                           (16, 1, 128, 16), (8, 2, 128, 128), (6, 2, 64, 256)])
@pytest.mark.parametrize("w_dtype", [torch.float32, torch.bfloat16, None])
@pytest.mark.parametrize("window,rotate,store", [(0, True, True), (23, True, True), (0, False, True), (0, True, False)])
def test_decode_attention_is_its_two_halves(Hq, Hkv, D, page, w_dtype, window, rotate, store):
    """A step of single tokens in one kernel gives what the preparation kernel followed by the
    attention kernel gives: the caches after the step to the bit, and the output to the bit
    where nothing is stored, else to the order in which the new key's share is added.
    Lengths are chosen so that the new key is a page's first and last slot, a tile's first
    key, and far into many splits."""
    ops = _ops()
    kv_lens = [1, page, page + 1, 33, 64, 65, 700, 2500]
    B = len(kv_lens)
    _, kc, vc, bt, cu, kvl = _paged_case(torch.bfloat16, B, Hq, Hkv, D, page, [1] * B, kv_lens, 77)
    qkv = _rand((B, (Hq + 2 * Hkv) * D), torch.bfloat16, 78, scale=1.5)
    qw = kw = None
    if w_dtype is not None:
        qw = (1.0 + _rand((D,), torch.float32, 79, scale=0.3)).to(w_dtype)
        kw = (1.0 + _rand((D,), torch.float32, 80, scale=0.3)).to(w_dtype)
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D))).cuda()
    table = ops.rope_table(inv_freq, 4096) if rotate else None
    positions = (kvl - 1).to(torch.int32)
    seq_index = torch.arange(B, dtype=torch.int32, device="cuda")
    scale = D ** -0.5
    assert ops.decode_attention_takes(Hq, Hkv, D, page, torch.bfloat16, D if rotate else 0)

    k1, v1, qkv1 = kc.clone(), vc.clone(), qkv.clone()
    ops.qk_norm_rope_store(qkv1, Hq, Hkv, D, positions, seq_index, q_weight=qw, k_weight=kw, eps=1e-6, table=table,
                           block_table=bt if store else None, k_cache=k1 if store else None,
                           v_cache=v1 if store else None, cu_seqlens_q=cu, kv_lens=kvl, max_q_len=1)
    q = qkv1[:, : Hq * D].unflatten(1, (Hq, D))
    want = ops.paged_attention(q, Hq, k1, v1, bt, cu, kvl, 1, max(kv_lens), scale, window=window)

    k2, v2, qkv2 = kc.clone(), vc.clone(), qkv.clone()
    got = ops.decode_attention(qkv2, Hq, Hkv, D, k2, v2, bt, cu, kvl, max(kv_lens), scale, window=window,
                               q_weight=qw, k_weight=kw, eps=1e-6, table=table, store=store)
    assert torch.equal(qkv2, qkv)                              # the raw projections are left alone
    assert torch.equal(k2, k1) and torch.equal(v2, v1)
    if not store:
        assert torch.equal(k2, kc) and torch.equal(v2, vc)
    if store:
        # the two-kernel path rounds the new key's probability to bfloat16 with all the others, the
        # fused one keeps it in float32: half a bfloat16 step of a probability times a value of size ~1
        torch.testing.assert_close(got.float(), want.float(), rtol=8e-3, atol=6e-3)
    else:
        assert torch.equal(got, want)
    # and against plain arithmetic
    ref = torch_ops.paged_attention(q.float(), Hq, k1.float(), v1.float(), bt, cu, kvl, 1, max(kv_lens), scale,
                                    window=window)
    torch.testing.assert_close(got.float().view(B, Hq, D), ref.view(B, Hq, D), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("Hq,Hkv,D,page", [(32, 8, 128, 16), (8, 2, 64, 32)])
@pytest.mark.parametrize("kv_lens", [[1, 17, 40, 64, 65], [700, 2500, 3]])
def test_nothing_past_a_sequences_end_is_read_into_the_result(Hq, Hkv, D, page, kv_lens):
    """Block tables that list real pages beyond a sequence's last one (a table that a graph
    keeps from a longer step, a page taken ahead), and slots at and past the sequence's end that
    hold NaN in keys and values, the slot the fused kernel writes among them: the decoding
    kernels look at whole tiles and whole tables before they know the length, and must mask
    what lies past it. One split and many, with and without a window."""
    ops = _ops()
    B = len(kv_lens)
    _, kc, vc, bt, cu, kvl = _paged_case(torch.bfloat16, B, Hq, Hkv, D, page, [1] * B, kv_lens, 91)
    W = bt.shape[1]
    spare = iter(sorted(set(range(kc.shape[0])) - set(bt[bt >= 0].tolist())) * W)
    clean_k, clean_v = kc.clone(), vc.clone()
    for b, L in enumerate(kv_lens):
        used = -(-L // page)
        for j in range(used, W):                      # real pages listed past the end, full of NaN
            pg = next(spare)
            bt[b, j] = pg
            kc[pg], vc[pg] = float("nan"), float("nan")
        last = int(bt[b, used - 1])
        first_free = (L - 1) % page                   # the new token's slot, and all slots after it
        kc[last, :, first_free:], vc[last, :, :, first_free:] = float("nan"), float("nan")
        clean_k[last, :, first_free:], clean_v[last, :, :, first_free:] = 0.0, 0.0
    qkv = _rand((B, (Hq + 2 * Hkv) * D), torch.bfloat16, 92, scale=1.5)
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D))).cuda()
    table = ops.rope_table(inv_freq, 4096)
    scale = D ** -0.5
    for window in (0, 50):
        k2, v2 = kc.clone(), vc.clone()
        got = ops.decode_attention(qkv.clone(), Hq, Hkv, D, k2, v2, bt, cu, kvl, max(kv_lens), scale, window=window,
                                   table=table)
        k1, v1, qkv1 = clean_k.clone(), clean_v.clone(), qkv.clone()
        ops.qk_norm_rope_store(qkv1, Hq, Hkv, D, (kvl - 1).to(torch.int32), torch.arange(B, dtype=torch.int32).cuda(),
                               table=table, block_table=bt, k_cache=k1, v_cache=v1, cu_seqlens_q=cu, kv_lens=kvl,
                               max_q_len=1)
        q = qkv1[:, : Hq * D].unflatten(1, (Hq, D))
        want = torch_ops.paged_attention(q.float(), Hq, k1.float(), v1.float(), bt, cu, kvl, 1, max(kv_lens), scale,
                                         window=window)
        assert torch.isfinite(got.float()).all(), window
        torch.testing.assert_close(got.float().view(B, Hq, D), want.view(B, Hq, D), rtol=2e-2, atol=2e-2)
        # the two-kernel path over the same poisoned caches (the new key and value written first)
        k3, v3 = kc.clone(), vc.clone()
        ops.qk_norm_rope_store(qkv.clone(), Hq, Hkv, D, (kvl - 1).to(torch.int32),
                               torch.arange(B, dtype=torch.int32).cuda(), table=table, block_table=bt, k_cache=k3,
                               v_cache=v3, cu_seqlens_q=cu, kv_lens=kvl, max_q_len=1)
        again = ops.paged_attention(q, Hq, k3, v3, bt, cu, kvl, 1, max(kv_lens), scale, window=window)
        assert torch.isfinite(again.float()).all(), window
        torch.testing.assert_close(again.float().view(B, Hq, D), want.view(B, Hq, D), rtol=2e-2, atol=2e-2)


def test_a_step_past_the_rotation_table_is_refused():
    """A position that the rotation table does not hold would go without its rotation: the
    operations refuse a step whose last position the caller says lies beyond the table."""
    ops = _ops()
    Hq, Hkv, D, page = 4, 2, 64, 16
    _, kc, vc, bt, cu, kvl = _paged_case(torch.bfloat16, 2, Hq, Hkv, D, page, [1, 1], [40, 41], 5)
    qkv = _rand((2, (Hq + 2 * Hkv) * D), torch.bfloat16, 6)
    table = ops.rope_table((1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D))).cuda(), 40)
    positions, seq = torch.tensor([39, 40], dtype=torch.int32).cuda(), torch.tensor([0, 1], dtype=torch.int32).cuda()
    with pytest.raises(ValueError, match="rotation table ends at 39"):
        ops.qk_norm_rope_store(qkv, Hq, Hkv, D, positions, seq, table=table, block_table=bt, k_cache=kc, v_cache=vc,
                               cu_seqlens_q=cu, kv_lens=kvl, max_q_len=1, max_kv_len=41)
    with pytest.raises(ValueError, match="rotation table ends at 39"):
        ops.decode_attention(qkv, Hq, Hkv, D, kc, vc, bt, cu, kvl, 41, D ** -0.5, table=table)
    # the launchers say the same to a caller that comes without the wrappers
    import ctypes

    from qwen3_from_scratch_amd.ops.build import library

    status = library("rotary").q3_qk_norm_rope_store(
        ctypes.c_void_p(qkv.data_ptr()), None, None, 0, ctypes.c_float(0.0), ctypes.c_void_p(table.data_ptr()), D, 40,
        ctypes.c_void_p(positions.data_ptr()), ctypes.c_void_p(seq.data_ptr()), None, 0, 0, None, None, 0, 0,
        2, Hq, Hkv, D, 1, None, None, 0, 0, 41, None)
    assert status != 0


@pytest.mark.parametrize("q_lens,kv_lens", [([512, 1, 100, 3, 33], [512, 900, 1100, 64, 2000]),
                                            ([700, 2], [3000, 50]), ([300], [9000]), ([40, 40, 40], [2100, 40, 700])])
@pytest.mark.parametrize("page", [16, 128])
def test_paged_attention_portions_over_long_prefixes(q_lens, kv_lens, page):
    """Portions of prompts with hundreds or thousands of cached keys before them, beside single
    tokens: few blocks of rows, whose keys are shared out over four blocks, over two, or not at all."""
    ops = _ops()
    Hq, Hkv, D = 32, 8, 128
    q, kc, vc, bt, cu, kvl = _paged_case(torch.bfloat16, len(q_lens), Hq, Hkv, D, page, q_lens, kv_lens, 31)
    scale = D ** -0.5
    got = ops.paged_attention(q, Hq, kc, vc, bt, cu, kvl, max(q_lens), max(kv_lens), scale, min_q_len=min(q_lens))
    want = torch_ops.paged_attention(q.float(), Hq, kc.float(), vc.float(), bt, cu, kvl, max(q_lens),
                                     max(kv_lens), scale)
    torch.testing.assert_close(got.float(), want, rtol=2e-2, atol=2e-2)
    for window in (0, 700):
        got = ops.paged_attention(q, Hq, kc, vc, bt, cu, kvl, max(q_lens), max(kv_lens), scale, window=window,
                                  min_q_len=min(q_lens))
        want = torch_ops.paged_attention(q.float(), Hq, kc.float(), vc.float(), bt, cu, kvl, max(q_lens),
                                         max(kv_lens), scale, window=window)
        torch.testing.assert_close(got.float(), want, rtol=2e-2, atol=2e-2)


def test_paged_attention_contexts_of_tens_of_thousands():
    """Contexts whose block tables are longer than what the prompt kernel keeps in shared memory
    at a time (508 pages: 8,128 keys of page 16), and that the decoding kernel cuts into its
    largest number of splits. A key on either side of such an edge is made to dominate the last
    row of a portion and a single token."""
    ops = _ops()
    Hq, Hkv, D, page = 8, 2, 128, 16
    G = Hq // Hkv
    q_lens, kv_lens = [300, 1, 40], [20000, 40000, 8200]
    scale = D ** -0.5
    for far in (8127, 8128, 16255, 16256, 19999 - 300):
        q, kc, vc, bt, cu, kvl = _paged_case(torch.bfloat16, 3, Hq, Hkv, D, page, q_lens, kv_lens, 50 + far % 7,
                                             spread=False)
        last_rows = (q_lens[0] - 1, q_lens[0])           # the portion's last row, the single token
        for b, row in enumerate(last_rows):
            pg = int(bt[b, far // page])
            kc[pg, :, far % page] = (q[row].view(Hkv, G, D)[:, 0] * 4).to(torch.bfloat16)
        got = ops.paged_attention(q, Hq, kc, vc, bt, cu, kvl, max(q_lens), max(kv_lens), scale, min_q_len=1)
        want = torch_ops.paged_attention(q.float(), Hq, kc.float(), vc.float(), bt, cu, kvl, max(q_lens),
                                         max(kv_lens), scale)
        torch.testing.assert_close(got.float(), want, rtol=2e-2, atol=2e-2)
        for b, row in enumerate(last_rows):
            v_far = vc[int(bt[b, far // page]), :, :, far % page].float()
            assert (got[row].float().view(Hq, D)[::G] - v_far).abs().max() < 0.2, (far, b)


@pytest.mark.parametrize("dtype", DTYPES)
def test_paged_attention_far_key_stands_out(dtype):
    """One key far back is made to dominate: a kernel that drops, repeats or
    misplaces a page shows at once."""
    ops = _ops()
    Hq, Hkv, D, page = 8, 2, 128, 16
    for L, far in [(1000, 3), (777, 400), (2049, 2048 - 17)]:
        q, kc, vc, bt, cu, kvl = _paged_case(dtype, 1, Hq, Hkv, D, page, [1], [L], 10 + L, spread=False)
        pg = int(bt[0, far // page])
        kc[pg, :, far % page] = (q[0].view(Hkv, Hq // Hkv, D)[:, 0] * 4).to(dtype)
        scale = D ** -0.5
        got = ops.paged_attention(q, Hq, kc, vc, bt, cu, kvl, 1, L, scale)
        want = torch_ops.paged_attention(q.float(), Hq, kc.float(), vc.float(), bt, cu, kvl, 1, L, scale)
        tol = dict(rtol=1e-4, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
        torch.testing.assert_close(got.float(), want, **tol)
        # the dominating key's value is (nearly) the answer for the first head of each group
        v_far = vc[pg, :, :, far % page].float()
        first = got.float().view(Hq, D)[:: Hq // Hkv]
        assert (first - v_far).abs().max() < 0.2


def test_paged_attention_first_token_returns_first_value():
    ops = _ops()
    q, kc, vc, bt, cu, kvl = _paged_case(torch.float32, 2, 4, 2, 32, 8, [1, 1], [1, 1], 11)
    got = ops.paged_attention(q, 4, kc, vc, bt, cu, kvl, 1, 1, 32 ** -0.5).view(2, 4, 32)
    for b in range(2):
        v0 = vc[int(bt[b, 0]), :, :, 0]
        torch.testing.assert_close(got[b], v0.repeat_interleave(2, dim=0), rtol=1e-6, atol=1e-6)


def test_paged_attention_ignores_garbage_beyond_the_sequence():
    ops = _ops()
    q, kc, vc, bt, cu, kvl = _paged_case(torch.float32, 2, 4, 2, 32, 8, [3, 1], [11, 21], 12)
    a = ops.paged_attention(q, 4, kc, vc, bt, cu, kvl, 3, 21, 0.2)
    # poison every slot past each sequence's end, and every page it does not own
    owned = set()
    for b, L in enumerate([11, 21]):
        for j in range(L):
            owned.add((int(bt[b, j // 8]), j % 8))
    for pg in range(kc.shape[0]):
        for s in range(8):
            if (pg, s) not in owned:
                kc[pg, :, s] = float("nan")
                vc[pg, :, :, s] = float("nan")
    b_ = ops.paged_attention(q, 4, kc, vc, bt, cu, kvl, 3, 21, 0.2)
    assert torch.equal(a, b_)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 64, 64), (2, 100, 72), (8, 331, 200), (33, 1000, 96), (64, 257, 1030),
                                   (130, 384, 224), (300, 129, 515)])
def test_linear(dtype, M, N, K):
    ops = _ops()
    x = _rand((M, K), dtype, 13)
    w = _rand((N, K), dtype, 14, scale=0.1)
    want = x.double() @ w.double().T
    got = ops.linear(x, w)
    assert got.dtype == dtype
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1.6e-2, atol=1e-2)
    torch.testing.assert_close(got.double(), want, **tol)
    got32 = ops.linear(x, w, out_dtype=torch.float32)
    assert got32.dtype == torch.float32
    torch.testing.assert_close(got32.double(), want, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (5, 6144, 4096), (8, 331, 200), (16, 1000, 2056), (3, 7, 12),
                                   (12, 50000, 256), (9, 4096, 12288), (4, 50, 515)])
def test_linear_float32_few_rows(M, N, K):
    """The float32 path's products when decoding: weights streamed once, a row's result the
    same whatever rows stand beside it."""
    ops = _ops()
    x = _rand((M, K), torch.float32, 51)
    w = _rand((N, K), torch.float32, 52, scale=0.05)
    got = ops.linear(x, w)
    torch.testing.assert_close(got.double(), x.double() @ w.double().T, rtol=1e-5, atol=1e-5)
    if K % 4 == 0:
        alone = ops.linear(x[M - 1:].contiguous(), w)
        assert torch.equal(alone[0], got[M - 1])


@pytest.mark.parametrize("M,N,K", [(1, 6144, 4096), (8, 4096, 4096), (5, 24576, 512), (16, 4096, 12288),
                                   (17, 1000, 2056), (32, 50000, 256), (48, 777, 4104), (64, 4096, 4096)])
def test_linear_few_rows_streams_weights(M, N, K):
    """The shapes of decoding: every way the kernel splits K and stacks row blocks."""
    ops = _ops()
    x = _rand((M, K), torch.bfloat16, 18)
    w = _rand((N, K), torch.bfloat16, 19, scale=0.05)
    want = x.float() @ w.float().T
    got = ops.linear(x, w, out_dtype=torch.float32)
    torch.testing.assert_close(got, want, rtol=2e-3, atol=2e-3)
    got16 = ops.linear(x, w)
    torch.testing.assert_close(got16.float(), want, rtol=1.6e-2, atol=1e-2)
    if M <= 16:
        # up to 16 rows share one way of splitting K: a row's result does not depend on its neighbours
        alone = ops.linear(x[:1].contiguous(), w, out_dtype=torch.float32)
        assert torch.equal(alone[0], got[0])


def _forget_choices(ops):
    ops.matmul_kernels("library")          # a change of setting makes every size choose anew
    ops.matmul_kernels("both")


@pytest.fixture
def rules_alone():
    """The table of kernel choices emptied for a test, and the package's own loaded again after it."""
    import json

    ops = _ops()
    ops.matmul_table([], clear=True)
    _forget_choices(ops)
    yield ops
    with open(ops.TABLE_FILE) as fh:
        ops.matmul_table(json.load(fh)["entries"], clear=True)
    _forget_choices(ops)


@pytest.mark.parametrize("M,N,K", [(17, 4096, 4096), (64, 6144, 4096), (200, 1000, 2056), (576, 5120, 1024),
                                   (2048, 768, 512), (33, 331, 72), (40, 129, 515), (300, 77, 100)])
def test_linear_many_rows_takes_its_kernel_by_rule(rules_alone, M, N, K):
    """More than 16 bfloat16 rows go to the vendor library's first candidate for the exact size
    (no stopwatch: the same kernel in every process), also inside a graph; a size it has no
    kernel for goes to the hand-written kernels."""
    ops = _ops()
    x = _rand((M, K), torch.bfloat16, 41)
    w = _rand((N, K), torch.bfloat16, 42, scale=0.05)
    want = x.double() @ w.double().T
    got = ops.linear(x, w, out_dtype=torch.float32)
    torch.testing.assert_close(got.double(), want, rtol=2e-3, atol=2e-3)
    got16 = ops.linear(x, w)
    torch.testing.assert_close(got16.double(), want, rtol=1.6e-2, atol=1e-2)
    plan = ops.matmul_plan(M, N, K)
    assert plan is not None and plan[0] == 1 and plan[2] == 0.0            # nothing was timed
    assert plan[4] == -1 and plan[6] == 0                                  # the library's first candidate
    assert torch.equal(ops.linear(x, w), got16)
    # the kernel for sizes that nothing else takes: plain multiply-adds, float32 sums
    plain = ops.linear_plain(x, w, torch.empty((M, N), dtype=torch.float32, device=x.device))
    torch.testing.assert_close(plain.double(), want, rtol=1e-4, atol=1e-4)
    plain16 = ops.linear_plain(x, w, torch.empty((M, N), dtype=torch.bfloat16, device=x.device))
    assert torch.equal(plain16, plain.bfloat16())
    # rows do not mix: a row's result is the same whatever its neighbours hold
    other = x.clone()
    other[1:] = _rand((M - 1, K), torch.bfloat16, 43)
    assert torch.equal(ops.linear(other, w)[0], got16[0])


def test_the_rule_for_few_tiles_and_a_long_inner_size(rules_alone):
    """A product with some hundreds of rows whose inner size is twice its width or more goes to
    the tiled kernel with K shared out; the same bits from two runs of the choice."""
    ops = rules_alone
    M, N, K = 200, 256, 1024
    x = _rand((M, K), torch.bfloat16, 61)
    w = _rand((N, K), torch.bfloat16, 62, scale=0.05)
    got = ops.linear(x, w)
    plan = ops.matmul_plan(M, N, K)
    assert plan[4] == 1 and plan[5] == ops.gemm_tiles_splits(1, M, N, K) > 1
    torch.testing.assert_close(got.double(), x.double() @ w.double().T, rtol=1.6e-2, atol=1e-2)
    _forget_choices(ops)
    assert torch.equal(ops.linear(x, w), got) and ops.matmul_plan(M, N, K) == plan


def test_the_table_decides_a_size():
    """A table entry sends a size to the library's second candidate or to a tile shape of the
    hand-written kernel with K shared out; sizes within the same step of rows follow it, others
    keep the rule; an entry the size cannot take (K no multiple of 64) is passed over."""
    ops = _ops()
    N, K = 1184, 640
    w = _rand((N, K), torch.bfloat16, 45, scale=0.05)
    rows = ops.matmul_rows_key("plain", 200)
    assert rows == 224 and ops.matmul_rows_key("plain", 50) == 56 and ops.matmul_rows_key("scaled", 50) == 56
    assert ops.matmul_rows_key("plain", 17) == 24 and ops.matmul_rows_key("plain", 64) == 64
    try:
        ops.matmul_table([{"kind": "plain", "rows": rows, "N": N, "K": K, "own": 1, "splits": 2},
                          {"kind": "plain", "rows": rows, "N": N, "K": K, "out": "float32", "library": 1},
                          {"kind": "plain", "rows": 64, "N": 96, "K": 72, "own": 0, "splits": 1}], clear=True)
        _forget_choices(ops)
        for M in (200, 195):
            x = _rand((M, K), torch.bfloat16, 46)
            got = ops.linear(x, w)
            assert ops.matmul_plan(M, N, K)[4:6] == (1, 2)
            assert torch.equal(got, ops.gemm_tiles(x, w, 1, splits=2))
            ops.linear(x, w, out_dtype=torch.float32)
            assert ops.matmul_plan(M, N, K, torch.float32)[4] == -1 and ops.matmul_plan(M, N, K, torch.float32)[6] in (0, 1)
        x = _rand((150, K), torch.bfloat16, 47)
        ops.linear(x, w)
        assert ops.matmul_plan(150, N, K)[4] == -1 and ops.matmul_plan(150, N, K)[6] == 0
        x3, w3 = _rand((64, 72), torch.bfloat16, 57), _rand((96, 72), torch.bfloat16, 58, scale=0.05)
        torch.testing.assert_close(ops.linear(x3, w3, out_dtype=torch.float32).double(), x3.double() @ w3.double().T,
                                   rtol=2e-3, atol=2e-3)
        # an entry that names a place the library's list for this size does not reach: its first candidate
        ops.matmul_table([{"kind": "plain", "rows": 320, "N": N, "K": K, "library": 63}])
        x4 = _rand((300, K), torch.bfloat16, 59)
        torch.testing.assert_close(ops.linear(x4, w).double(), x4.double() @ w.double().T, rtol=2e-2, atol=2e-2)
        offered = ops.matmul_plan(300, N, K)
        assert offered[4] == -1 and offered[6] in (0, 63)
    finally:
        import json
        with open(ops.TABLE_FILE) as fh:
            ops.matmul_table(json.load(fh)["entries"], clear=True)
        _forget_choices(ops)


def test_linear_many_rows_first_met_in_a_graph():
    """A size first met while a graph is captured gets its kernel there as anywhere (the choice
    needs no run); with the tuner on it runs untimed in the capture and is timed at its next
    eager call; the graph's replays keep giving the right product."""
    ops = _ops()
    M, N, K = 48, 1184, 608
    x = _rand((M, K), torch.bfloat16, 44)
    w = _rand((N, K), torch.bfloat16, 45, scale=0.05)
    ops.matmul_init()
    out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    assert ops.matmul_plan(M, N, K) is None
    ops.matmul_tuner(True)
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                ops.linear(x, w, out=out)
        torch.cuda.current_stream().wait_stream(side)
        assert ops.matmul_plan(M, N, K)[0] == 1
        want = x.double() @ w.double().T
        for seed in (46, 47, 48):
            out.zero_()
            graph.replay()
            torch.testing.assert_close(out.double(), want, rtol=1.6e-2, atol=1e-2)
            eager = ops.linear(x, w)                               # timed at the first of these
            torch.testing.assert_close(eager.double(), want, rtol=1.6e-2, atol=1e-2)
            x.copy_(_rand((M, K), torch.bfloat16, seed))
            want = x.double() @ w.double().T
        plan = ops.matmul_plan(M, N, K)
        assert plan[0] > 1 and 0 <= plan[1] < plan[0] and plan[3] <= plan[2]
        # a few rows fewer (the same step of rows): the same choice, asked of the library for the exact size
        M2 = 200
        x2 = _rand((M2, K), torch.bfloat16, 49)
        ops.linear(x2, w)
        fewer = ops.linear(x2[:M2 - 7].contiguous(), w, out_dtype=torch.float32)
        torch.testing.assert_close(fewer.double(), x2[:M2 - 7].double() @ w.double().T, rtol=2e-3, atol=2e-3)
    finally:
        ops.matmul_tuner(False)


@pytest.mark.parametrize("M,N,K", [(200, 304, 128), (513, 1000, 192), (77, 48, 64), (17, 2, 64), (300, 331, 4096),
                                   (1024, 1536, 1024), (150, 260, 640)])
def test_tiled_product_every_shape_and_epilogue(M, N, K):
    """The hand-written tiled matrix-core product: every tile shape, at sizes whose rows and
    columns end inside a tile, against a float64 product; float32 and bfloat16 outputs and the
    SwiGLU epilogue; one row's result does not depend on its neighbours."""
    ops = _ops()
    x = _rand((M, K), torch.bfloat16, 51)
    w = _rand((N, K), torch.bfloat16, 52, scale=0.05)
    want = x.double() @ w.double().T
    rounded = want.to(torch.bfloat16).double()
    gated = torch.nn.functional.silu(rounded[:, 0::2]) * rounded[:, 1::2] if N % 2 == 0 else None
    first = None
    for config in range(ops.gemm_tiles_configs()):
        got = ops.gemm_tiles(x, w, config, out_dtype=torch.float32)
        torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=1e-4)
        got16 = ops.gemm_tiles(x, w, config)
        torch.testing.assert_close(got16.double(), want, rtol=1.6e-2, atol=1e-2)
        # every shape adds a sum's terms in the same order (k ascending, 32 at a time)
        first = got if first is None else first
        assert torch.equal(got, first)
        if gated is not None:
            act = ops.gemm_tiles(x, w, config, swiglu=True)
            torch.testing.assert_close(act.double(), gated, rtol=3.2e-2, atol=2e-2)
        other = x.clone()
        other[1:] = _rand((M - 1, K), torch.bfloat16, 53)
        assert torch.equal(ops.gemm_tiles(other, w, config)[0], got16[0])
        # K shared out over several blocks per tile, their partial products added by a second kernel
        for splits in (2, 3, 5):
            if K // 64 >= splits and N % 4 == 0:
                shared = ops.gemm_tiles(x, w, config, out_dtype=torch.float32, splits=splits)
                torch.testing.assert_close(shared.double(), want, rtol=1e-4, atol=1e-4)
                shared16 = ops.gemm_tiles(x, w, config, splits=splits)
                torch.testing.assert_close(shared16.double(), want, rtol=1.6e-2, atol=1e-2)
                assert torch.equal(ops.gemm_tiles(other, w, config, splits=splits)[0], shared16[0])
    with pytest.raises(ops.OperandError):
        ops.gemm_tiles(x[:, :K - 8].contiguous(), w[:, :K - 8].contiguous())      # K no multiple of 64
    with pytest.raises(ops.OperandError):
        ops.gemm_tiles(x, w, 0, splits=K // 64 + 1)


def test_linear_many_rows_by_the_hand_written_kernel_alone():
    """Narrowed to the hand-written kernel, products with many rows are its:
    a size it takes, also first met inside a graph, and a size it does not take (the library's)."""
    ops = _ops()
    ops.matmul_init()
    ops.matmul_kernels("own")
    try:
        M, N, K = 150, 840, 320
        x = _rand((M, K), torch.bfloat16, 54)
        w = _rand((N, K), torch.bfloat16, 55, scale=0.05)
        want = x.double() @ w.double().T
        got = ops.linear(x, w, out_dtype=torch.float32)
        torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=1e-4)
        plan = ops.matmul_plan(M, N, K, torch.float32)
        assert plan[4] >= 0 and plan[0] >= 1
        assert torch.equal(got, ops.gemm_tiles(x, w, plan[4], out_dtype=torch.float32))
        # first met in a capture
        M2 = 90
        x2 = _rand((M2, K), torch.bfloat16, 56)
        out = torch.empty((M2, N), dtype=torch.bfloat16, device=x.device)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                ops.linear(x2, w, out=out)
        torch.cuda.current_stream().wait_stream(side)
        for _ in range(3):
            out.zero_()
            graph.replay()
            torch.testing.assert_close(out.double(), x2.double() @ w.double().T, rtol=1.6e-2, atol=1e-2)
            assert torch.equal(ops.linear(x2, w), out)
        assert ops.matmul_plan(M2, N, K)[4] >= 0
        # few tiles and many steps: K is shared out
        M4, N4, K4 = 300, 512, 4096
        assert ops.gemm_tiles_splits(1, M4, N4, K4) > 1
        x4, w4 = _rand((M4, K4), torch.bfloat16, 59), _rand((N4, K4), torch.bfloat16, 60, scale=0.05)
        torch.testing.assert_close(ops.linear(x4, w4, out_dtype=torch.float32).double(), x4.double() @ w4.double().T,
                                   rtol=1e-4, atol=1e-4)
        plan4 = ops.matmul_plan(M4, N4, K4, torch.float32)
        assert plan4[4] == 1 and plan4[5] == ops.gemm_tiles_splits(1, M4, N4, K4)
        # an inner size it does not take goes to the library
        x3, w3 = _rand((40, 72), torch.bfloat16, 57), _rand((96, 72), torch.bfloat16, 58, scale=0.05)
        torch.testing.assert_close(ops.linear(x3, w3, out_dtype=torch.float32).double(), x3.double() @ w3.double().T,
                                   rtol=2e-3, atol=2e-3)
        assert ops.matmul_plan(40, 96, 72, torch.float32)[4] == -1
    finally:
        ops.matmul_kernels("both")


@pytest.mark.parametrize("M,N,K", [(1, 6144, 4096), (8, 4096, 12288), (16, 1000, 96), (3, 331, 64), (9, 24, 2048),
                                   (5, 151936, 256), (12, 6144, 4096), (16, 24576, 512), (9, 6168, 160),
                                   (13, 6150, 4096), (9, 12312, 160), (11, 151936, 256), (16, 24576, 4096)])
def test_linear_from_the_tiled_copy(M, N, K):
    """The tile-ordered copy gives the very sums of the row-major kernel: the same numbers
    are added in the same order, only their addresses differ. That holds for the kernel that
    gives two slabs to a block too (more than eight rows, 384 slabs or more; also with an odd
    number of slabs and a last slab that is not whole; the vocabulary's 9,496 slabs)."""
    ops = _ops()
    x = _rand((M, K), torch.bfloat16, 23)
    w = _rand((N, K), torch.bfloat16, 24, scale=0.05)
    tiled = ops.tile_weight(w)
    assert tiled is not None and tiled.numel() == -(-N // 16) * 16 * K
    for out_dtype in (torch.bfloat16, torch.float32):
        assert torch.equal(ops.linear(x, w, out_dtype=out_dtype, tiled=tiled), ops.linear(x, w, out_dtype=out_dtype))
    if N % 2 == 0:
        act, want = ops.linear_swiglu(x, w, tiled=tiled), ops.linear_swiglu(x, w)
        if ops.stream_plan(M, N, K, swiglu=True) is None:
            assert torch.equal(act, want)
        else:       # a whole gate/up product of 9 to 16 rows is the streaming kernel's: another order of the sums
            torch.testing.assert_close(act.float(), want.float(), rtol=2e-2, atol=2e-2 * float(want.float().abs().max()))
    assert ops.tile_weight(_rand((8, 72), torch.bfloat16, 1)) is None       # K not a multiple of 32
    assert ops.tile_weight(w.float()) is None
    many = _rand((40, K), torch.bfloat16, 25)
    got, plain = ops.linear(many, w, tiled=tiled), ops.linear(many, w)
    if ops.stream_plan(40, N, K) is None:                                      # many rows of a small weight ignore the copy
        assert torch.equal(got, plain)
    else:                                                                      # a large one is streamed from it: other sums' order
        torch.testing.assert_close(got.float(), plain.float(), rtol=2e-2, atol=2e-2 * float(plain.float().abs().max()))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,I,K", [(1, 12288, 4096), (8, 100, 72), (16, 333, 200), (40, 64, 64)])
def test_linear_swiglu(dtype, M, I, K):
    ops = _ops()
    x = _rand((M, K), dtype, 21)
    w = _rand((2 * I, K), dtype, 22, scale=0.1)
    got = ops.linear_swiglu(x, w)
    assert got.shape == (M, I) and got.dtype == dtype
    want = torch_ops.swiglu((x.double() @ w.double().T).float())
    tol = dict(rtol=1e-4, atol=1e-4) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(got.float(), want, **tol)
    if dtype == torch.bfloat16:
        # fused or not, the result is the same to the bit
        assert torch.equal(got, ops.swiglu(ops.linear(x, w)))


@pytest.mark.parametrize("norm_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,H,K,N2", [(1, 4096, 4096, 6144), (8, 4096, 12288, 24576), (16, 96, 224, 160),
                                      (5, 992, 64, 330), (3, 32, 32, 48), (12, 4096, 1024, 24576),
                                      (16, 1024, 512, 6152),
                                      # small weights: 17 to 64 rows are two to four groups of the few-row kernel's blocks
                                      (17, 1024, 512, 6152), (24, 1024, 2048, 4096), (32, 96, 224, 160),
                                      (31, 1024, 4096, 8192), (20, 992, 64, 330), (48, 256, 128, 512),
                                      (64, 1024, 512, 2048), (33, 96, 224, 160), (50, 1024, 2048, 4096)])
def test_linear_residual_norm_and_unscaled_rows(M, H, K, N2, norm_dtype):
    """A product that adds itself into the residual stream and prepares the next norm, and the
    product after it, which applies the norm's division: together they give what the product,
    the norm kernel and the next product give one after the other."""
    ops = _ops()
    x = _rand((M, K), torch.bfloat16, 31)
    w1 = _rand((H, K), torch.bfloat16, 32, scale=0.05)
    w2 = _rand((N2, H), torch.bfloat16, 33, scale=0.05)
    nw = (1.0 + _rand((H,), torch.float32, 34, scale=0.2)).to(norm_dtype)
    residual = _rand((M, H), torch.float32, 35, scale=2.0)
    eps = 1e-5
    t1, t2 = ops.tile_weight(w1), ops.tile_weight(w2)

    # one after the other
    stream = residual.clone()
    delta = ops.linear(x, w1, tiled=t1)
    h = ops.rmsnorm(stream, nw, eps, torch.bfloat16, delta=delta)
    want = ops.linear(h, w2, out_dtype=torch.float32, tiled=t2)
    want_act = ops.linear_swiglu(h, w2, tiled=t2)

    fused_stream = residual.clone()
    values, sums = ops.linear_residual_norm(x, w1, t1, fused_stream, nw)
    assert torch.equal(fused_stream, stream)                      # the stream itself is the same to the bit
    assert sums.shape == (H // 16, ops.sums_stride(M))
    ms = (stream.double() ** 2).sum(dim=1)
    torch.testing.assert_close(sums.double().sum(dim=0)[:M], ms, rtol=1e-5, atol=1e-6)
    assert float(sums[:, M:].abs().max()) == 0.0 if M < sums.shape[1] else True
    torch.testing.assert_close(values.float(), (stream * nw.float()), rtol=8e-3, atol=1e-6)
    got = ops.linear(values, w2, out_dtype=torch.float32, tiled=t2, unscaled=(sums, eps, H))
    # both roundings of the norm's output are to bfloat16, of numbers that differ by the row's factor
    scale = float(want.abs().max())
    assert float((got - want).abs().max()) <= 6e-3 * scale
    exact = (stream.double() * torch.rsqrt((stream.double() ** 2).mean(dim=1, keepdim=True) + eps) * nw.double()) @ w2.double().T
    assert float((got.double() - exact).abs().max()) <= 6e-3 * scale
    got_act = ops.linear_swiglu(values, w2, tiled=t2, unscaled=(sums, eps, H))
    assert float((got_act.float() - want_act.float()).abs().max()) <= 2e-2 * max(1.0, float(want_act.float().abs().max()))
    # rows do not depend on their neighbours
    if M > 1:
        alone_stream = residual[:1].clone()
        v1, s1 = ops.linear_residual_norm(x[:1].contiguous(), w1, t1, alone_stream, nw)
        assert torch.equal(v1[0], values[0]) and torch.equal(s1[:, 0], sums[:, 0])
        a = ops.linear(v1, w2, out_dtype=torch.float32, tiled=t2, unscaled=(s1, eps, H))
        assert torch.equal(a[0], got[0])
    # what the kernel does not take is refused
    with pytest.raises(ops.OperandError):
        ops.linear(_rand((M + 16, H), torch.bfloat16, 1), w2, tiled=t2, unscaled=(sums, eps, H))
    if M <= 16:
        with pytest.raises(ops.OperandError):
            ops.linear(values, w2, unscaled=(sums, eps, H))


@pytest.mark.parametrize("norm_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,H,K,N2", [(17, 4096, 4096, 6144), (64, 4096, 12288, 24576), (40, 1024, 512, 6152),
                                      (33, 192, 64, 332), (64, 5120, 3200, 1000), (25, 1088, 17408, 128),
                                      (100, 4096, 4096, 24576), (128, 2048, 1024, 6144)])
def test_linear_residual_norm_and_unscaled_rows_beyond_sixteen(M, H, K, N2, norm_dtype):
    """The same pair of fusions for 17 to 128 rows, where the tiled kernel carries them: its
    partial products go through a second kernel that adds them into the stream, and the next
    product's epilogue (or the kernel that adds its partial products) divides by the rows' rms."""
    ops = _ops()
    x = _rand((M, K), torch.bfloat16, 41)
    w1 = _rand((H, K), torch.bfloat16, 42, scale=0.05)
    w2 = _rand((N2, H), torch.bfloat16, 43, scale=0.05)
    nw = (1.0 + _rand((H,), torch.float32, 44, scale=0.2)).to(norm_dtype)
    residual = _rand((M, H), torch.float32, 45, scale=2.0)
    residual[M // 2] *= 30.0                                       # a row whose factor is far from the others'
    eps = 1e-5
    assert ops.fused_rows_take(w1, M) and ops.fused_rows_take(w2, M)

    exact_delta = (x.double() @ w1.double().T)
    ops.matmul_init()
    try:
        # with the hand-written kernel alone the fusion is never declined
        ops.matmul_kernels("own")
        fused_stream = residual.clone()
        values, sums = ops.linear_residual_norm(x, w1, None, fused_stream, nw)
        # the stream: the product rounded to bfloat16 once, then added in float32
        stream = residual + exact_delta.float().bfloat16().float()
        differs = fused_stream != stream
        assert float(differs.float().mean()) < 0.02               # roundings at a bfloat16 tie aside
        torch.testing.assert_close(fused_stream, stream, rtol=0, atol=2 ** -7 * float(exact_delta.abs().max()))
        stream = fused_stream
        assert sums.shape == (-(-H // 1024), ops.sums_stride(M))
        torch.testing.assert_close(sums.double().sum(dim=0)[:M], (stream.double() ** 2).sum(dim=1), rtol=1e-5, atol=1e-6)
        assert torch.equal(values, (stream * nw.float()).bfloat16())
        # a second call gives the same bits (the choice of tile shape is kept, the additions are ordered)
        again_stream = residual.clone()
        v2, s2 = ops.linear_residual_norm(x, w1, None, again_stream, nw)
        assert torch.equal(again_stream, fused_stream) and torch.equal(v2, values) and torch.equal(s2[:, :M], sums[:, :M])

        h = ops.rmsnorm(stream.clone(), nw, eps, torch.bfloat16)
        want = ops.linear(h, w2, out_dtype=torch.float32)
        exact = (stream.double() * torch.rsqrt((stream.double() ** 2).mean(dim=1, keepdim=True) + eps)
                 * nw.double()) @ w2.double().T
        # the reader by the tiled kernel, by the library's product with the division behind it, and by
        # whichever of the two the table and the rule name; there the writer may leave the size to the plain product
        for which in ("own", "library", "both"):
            ops.matmul_kernels(which)
            got = ops.linear(values, w2, out_dtype=torch.float32, unscaled=(sums, eps, H))
            for m in range(M):                                     # row by row: their sizes differ
                scale = float(exact[m].abs().max())
                assert float((got[m] - want[m]).abs().max()) <= 6e-3 * scale, (which, m)
                assert float((got[m].double() - exact[m]).abs().max()) <= 6e-3 * scale, (which, m)
            assert torch.equal(ops.linear(values, w2, out_dtype=torch.float32, unscaled=(sums, eps, H)), got)
            got_bf16 = ops.linear(values, w2, unscaled=(sums, eps, H))
            torch.testing.assert_close(got_bf16.float(), got, rtol=8e-3, atol=1e-3)
            if N2 % 2 == 0:
                want_act = torch_ops.swiglu(exact.float().bfloat16().float())
                got_act = ops.linear_swiglu(values, w2, unscaled=(sums, eps, H))
                assert got_act.shape == (M, N2 // 2)
                assert float((got_act.float() - want_act).abs().max()) <= 2e-2 * max(1.0, float(want_act.abs().max()))
            other_stream = residual.clone()
            fused = ops.linear_residual_norm(x, w1, None, other_stream, nw)
            if fused is None:
                assert which != "own" and torch.equal(other_stream, residual)      # declined: nothing was done
            else:
                # another tile shape may serve this setting: other shares of K, other roundings
                torch.testing.assert_close(other_stream, fused_stream, rtol=0, atol=2 ** -7 * float(exact_delta.abs().max()))
                assert float((other_stream != fused_stream).float().mean()) < 0.02
        with pytest.raises(ops.OperandError):                      # sums of another number of rows
            ops.linear(values, w2, unscaled=(sums[:, :-1].contiguous(), eps, H))
    finally:
        ops.matmul_kernels("both")


@pytest.mark.parametrize("M", [17, 32, 33, 50, 64, 80, 96])
@pytest.mark.parametrize("N,K", [(24576, 4096), (20002, 1440), (16384, 1024), (12288, 4000)])
def test_weight_streaming_product_for_some_tens_of_rows(M, N, K):
    """17 to 96 rows against a weight of 24 MB or more whose slabs fill the chip in one round of blocks,
    from its tile-ordered copy: plain in bfloat16 and float32, with the rows' division by their rms, and
    with SwiGLU; K that is no multiple of a chunk (256) or of 64, N that is no multiple of 16, blocks of
    six slabs and of four. Against float64 sums."""
    ops = _ops()
    x = _rand((M, K), torch.bfloat16, 61)
    w = _rand((N, K), torch.bfloat16, 62, scale=0.05)
    tiled = ops.tile_weight(w)
    plan = ops.stream_plan(M, N, K)
    assert plan == {24576: 6, 20002: 6, 16384: 4, 12288: 4}[N]     # 256, 209, 256 and 192 blocks
    exact = x.double() @ w.double().T
    scale = float(exact.abs().max())
    got32 = ops.linear(x, w, out_dtype=torch.float32, tiled=tiled)
    assert float((got32.double() - exact).abs().max()) <= 1e-3 * scale
    got = ops.linear(x, w, tiled=tiled)
    assert torch.equal(got, ops.linear(x, w, tiled=tiled))         # the same bits every time
    torch.testing.assert_close(got.float(), got32, rtol=8e-3, atol=4e-3 * scale)
    # the streaming kernel served these, not the library: its sums are closer to exact than bfloat16 products
    # of the other kernels are to each other, and the plan says so; without the copy the others serve
    other = ops.linear(x, w, out_dtype=torch.float32)
    assert float((other.double() - exact).abs().max()) <= 1e-3 * scale
    # rows that still lack their norm's division, the sums of squares in chunks as the writer leaves them
    sums = torch.zeros((-(-K // 1024), ops.sums_stride(M)), dtype=torch.float32, device="cuda")
    sums[:, :M] = (torch.rand((sums.shape[0], M), device="cuda") + 0.5) * K / sums.shape[0]
    sums[:, M // 2] *= 900.0                                        # a row whose factor is far from the others'
    eps = 1e-5
    factor = torch.rsqrt(sums[:, :M].double().sum(dim=0) / K + eps)[:, None]
    if K % 64 == 0 and N % 4 == 0:
        scaled = ops.linear(x, w, out_dtype=torch.float32, tiled=tiled, unscaled=(sums, eps, K))
        for m in range(M):
            row = exact[m] * factor[m]
            assert float((scaled[m].double() - row).abs().max()) <= 2e-3 * float(row.abs().max()), m
        act = ops.linear_swiglu(x, w, tiled=tiled, unscaled=(sums, eps, K))
        want = torch_ops.swiglu((exact * factor).float().bfloat16().float())
        assert act.shape == (M, N // 2)
        assert float((act.float() - want).abs().max()) <= 2e-2 * max(1.0, float(want.abs().max()))
    plain_act = ops.linear_swiglu(x, w, tiled=tiled)
    want = torch_ops.swiglu(exact.float().bfloat16().float())
    assert float((plain_act.float() - want).abs().max()) <= 2e-2 * max(1.0, float(want.abs().max()))
    # asked for the other kernels alone, the streaming kernel steps aside
    try:
        ops.matmul_kernels("own")
        assert ops.stream_plan(M, N, K) is None
        if K % 64 == 0:
            torch.testing.assert_close(ops.linear(x, w, out_dtype=torch.float32, tiled=tiled), got32, rtol=2e-3,
                                       atol=1e-3 * scale)
    finally:
        ops.matmul_kernels("both")
    assert ops.stream_plan(16, N, K) is None and ops.stream_plan(97, N, K) is None
    assert ops.stream_plan(M, 1024, 4096) is None                  # a small weight: the other kernels' rows
    # slabs that would leave CUs idle (36 blocks) or need a second round (544, 1,583): the other kernels'
    assert ops.stream_plan(M, 3400, 4000) is None and ops.stream_plan(M, 34816, 5120) is None
    assert ops.stream_plan(M, 151936, 4096) is None


@pytest.mark.parametrize("M", [9, 12, 16])
@pytest.mark.parametrize("I,K,chunks", [(12288, 4096, 256), (9300, 2080, 130), (12288, 4096, 4)])
def test_gate_up_of_nine_to_sixteen_rows_by_the_streaming_kernel(M, I, K, chunks):
    """A whole gate/up product of 9 to 16 rows goes to the weight-streaming kernel, with the
    rows' sums of squares as the few-row kernel leaves them (a partial sum per slab of 16 columns:
    hundreds of them) or in a few chunks; the same product from the few-row kernel agrees."""
    ops = _ops()
    N = 2 * I
    x = _rand((M, K), torch.bfloat16, 71)
    w = _rand((N, K), torch.bfloat16, 72, scale=0.05)
    tiled = ops.tile_weight(w)
    assert ops.stream_plan(M, N, K, swiglu=True) == 6 and ops.stream_plan(M, N, K) is None
    assert ops.stream_plan(8, N, K, swiglu=True) is None and ops.stream_plan(M, 12000, 2080, swiglu=True) is None
    assert ops.stream_plan(M, 34816, 5120, swiglu=True) is None      # 363 blocks: more than one round
    sums = torch.zeros((chunks, 16), dtype=torch.float32, device="cuda")
    sums[:, :M] = (torch.rand((chunks, M), device="cuda") + 0.5) * K / chunks
    sums[:, M // 2] *= 400.0
    sums[:, M:] = float("nan")                                      # rows that are not there: never read into a result
    eps = 1e-6
    factor = torch.rsqrt(sums[:, :M].double().sum(dim=0) / K + eps)[:, None]
    exact = x.double() @ w.double().T
    for unscaled, truth in ((None, exact), ((sums, eps, K), exact * factor)):
        got = ops.linear_swiglu(x, w, tiled=tiled, unscaled=unscaled)
        want = torch_ops.swiglu(truth.float().bfloat16().float())
        assert got.shape == (M, I)
        assert float((got.float() - want).abs().max()) <= 2e-2 * max(1.0, float(want.abs().max()))
        assert torch.equal(got, ops.linear_swiglu(x, w, tiled=tiled, unscaled=unscaled))
        try:
            ops.matmul_kernels("own")                               # the few-row kernel serves it then
            other = ops.linear_swiglu(x, w, tiled=tiled, unscaled=unscaled)
        finally:
            ops.matmul_kernels("both")
        torch.testing.assert_close(got.float(), other.float(), rtol=2e-2, atol=2e-2 * max(1.0, float(want.abs().max())))


def test_linear_float32_is_true_float32():
    """Inputs whose products need all 24 bits: a matrix mode of reduced precision
    (bf16 or tf32-like splitting) would be off by far more than float32 rounding."""
    ops = _ops()
    g = torch.Generator().manual_seed(15)
    x = (1.0 + torch.rand((16, 512), generator=g) * 2 ** -10).cuda()
    w = (1.0 + torch.rand((24, 512), generator=g) * 2 ** -10).cuda()
    want = (x.double() @ w.double().T)
    got = ops.linear(x, w).double()
    assert ((got - want).abs() / want).max() < 2e-6


def test_sample_greedy_and_ties():
    ops = _ops()
    R, V = 5, 1000
    logits = _rand((R, V), torch.float32, 16)
    logits[2, 17] = logits[2, 900] = 50.0               # equal maxima: the lowest index wins
    z = torch.zeros(R, device="cuda")
    got = ops.sample(logits, z, torch.zeros(R, dtype=torch.int32, device="cuda"),
                     torch.zeros(R, dtype=torch.int64, device="cuda"),
                     torch.zeros(R, dtype=torch.int32, device="cuda"))
    assert got.tolist() == torch.argmax(logits, dim=-1).tolist()
    assert got[2] == 17


def test_sample_temperature_follows_softmax_and_seed():
    ops = _ops()
    V, R = 11, 40000
    base = torch.tensor([0.5, -1.0, 2.0, 0.0, 1.0, -3.0, 0.3, 1.7, -0.4, 0.9, 0.1])
    logits = base.repeat(R, 1).cuda().contiguous()
    T = 0.8
    temp = torch.full((R,), T, device="cuda")
    k0 = torch.zeros(R, dtype=torch.int32, device="cuda")
    seed = torch.full((R,), 1234, dtype=torch.int64, device="cuda")
    counter = torch.arange(R, dtype=torch.int32, device="cuda")
    got = ops.sample(logits, temp, k0, seed, counter)
    freq = torch.bincount(got.cpu().long(), minlength=V).double() / R
    p = torch.softmax(base.double() / T, dim=-1)
    chi2 = float((R * (freq - p) ** 2 / p).sum())
    assert chi2 < 40.0, chi2                              # 10 degrees of freedom; 40 is far in the tail
    # the same (seed, counter) gives the same token whatever else is in the batch
    again = ops.sample(logits[:100].contiguous(), temp[:100], k0[:100], seed[:100], counter[:100])
    assert torch.equal(again, got[:100])
    other = ops.sample(logits, temp, k0, seed + 1, counter)
    assert not torch.equal(other, got)
    # top-k: only the k best are ever drawn, with their renormalised frequencies
    k = 3
    got = ops.sample(logits, temp, torch.full((R,), k, dtype=torch.int32, device="cuda"), seed, counter)
    top = torch.topk(base, k).indices
    freq = torch.bincount(got.cpu().long(), minlength=V).double() / R
    assert set(torch.nonzero(freq).flatten().tolist()) == set(top.tolist())
    pk = torch.zeros(V, dtype=torch.double)
    pk[top] = torch.softmax(base[top].double() / T, dim=-1)
    chi2 = float((R * (freq[top] - pk[top]) ** 2 / pk[top]).sum())
    assert chi2 < 30.0, chi2
    # as the temperature goes to zero the draw becomes the arg-max
    cold = ops.sample(logits[:50].contiguous(), torch.full((50,), 1e-3, device="cuda"), k0[:50], seed[:50],
                      counter[:50])
    assert (cold == 2).all()


def test_sample_large_vocabulary_top_k():
    ops = _ops()
    R, V, k = 3, 151936, 40
    logits = _rand((R, V), torch.float32, 17, scale=3.0)
    temp = torch.ones(R, device="cuda")
    seed = torch.arange(R, dtype=torch.int64, device="cuda")
    allowed = [set(torch.topk(logits[r], k).indices.tolist()) for r in range(R)]
    for c in range(20):
        got = ops.sample(logits, temp, torch.full((R,), k, dtype=torch.int32, device="cuda"), seed,
                         torch.full((R,), c, dtype=torch.int32, device="cuda"))
        for r in range(R):
            assert int(got[r]) in allowed[r]


def test_operands_on_the_host_are_refused():
    ops = _ops()
    with pytest.raises(ValueError):
        ops.swiglu(torch.zeros(2, 8))


def test_measured_peaks_are_plausible():
    """The probes behind the benchmark's measured peaks: a read of a buffer no cache holds and the
    matrix instruction from registers reach a fair share of the published rates and do not pass them."""
    ops = _ops()
    read = ops.measured_read_rate(gigabytes=2.0, repeats=3)
    assert 2.0e12 < read < 8.0e12, read
    matrix = ops.measured_matrix_rate(repeats=3)
    assert 1.0e15 < matrix < 2.6e15, matrix
