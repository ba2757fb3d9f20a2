"""What fixes the plain implementation beside the reference's text: special cases
that reduce to a library routine, invariants, and vectors the reference's own
tests hold. Each is chosen so that a plausible mistake fails it."""

import math

import torch
import torch.nn.functional as F

import plain_qwen3 as plain


def test_rms_norm_is_the_library_routine():
    # test/models/test_rms_norm.py:25-44 holds the three implementations to 1e-5 of this
    g = torch.Generator().manual_seed(0)
    x = torch.randn(2, 128, 1024, generator=g)
    w = 1 + 0.1 * torch.randn(1024, generator=g)
    got = plain.rms_norm(x, w, 1e-5)
    torch.testing.assert_close(got, F.rms_norm(x, (1024,), w, 1e-5), rtol=1e-5, atol=1e-5)


def test_rms_norm_eps_inside_the_root_and_plain_weight():
    x = torch.ones(1, 8)
    w = torch.full((8,), 3.0)
    # all-ones input: w / sqrt(1 + eps); (1 + w) or eps outside the root would differ
    torch.testing.assert_close(plain.rms_norm(x, w, 0.5), w[None] / math.sqrt(1.5))
    # scale invariance as eps -> 0
    y = torch.randn(3, 16)
    torch.testing.assert_close(plain.rms_norm(y, torch.ones(16), 0.0), plain.rms_norm(7 * y, torch.ones(16), 0.0),
                               rtol=1e-5, atol=1e-6)


def test_rotary_angles_match_the_reference_table():
    # test/models/test_rotary.py:19-54: head 128, base 1e5, 1024 positions
    D, base, P = 128, 100000.0, 1024
    ang = plain.rotary_angles(torch.arange(P), D, base, torch.float32)
    inv = 1.0 / (base ** (torch.arange(0, D, 2, dtype=torch.float) / D))
    want = torch.outer(torch.arange(P, dtype=torch.float), inv)
    torch.testing.assert_close(ang.cos(), want.cos(), rtol=0, atol=1e-5)
    torch.testing.assert_close(ang.sin(), want.sin(), rtol=0, atol=1e-5)


def test_rotary_pairs_i_with_i_plus_half_as_complex_multiplication():
    g = torch.Generator().manual_seed(1)
    T, H, D = 7, 3, 16
    x = torch.randn(T, H, D, generator=g, dtype=torch.float64)
    pos = torch.tensor([0, 1, 2, 10, 11, 50, 200])
    ang = plain.rotary_angles(pos, D, 10000.0, torch.float64)
    got = plain.apply_rotary(x, ang)
    z = torch.complex(x[..., : D // 2], x[..., D // 2:]) * torch.polar(torch.ones_like(ang), ang)[:, None, :]
    torch.testing.assert_close(got, torch.cat((z.real, z.imag), dim=-1))
    # position 0 is the identity, and each pair keeps its length
    torch.testing.assert_close(got[0], x[0])
    torch.testing.assert_close((got[..., : D // 2] ** 2 + got[..., D // 2:] ** 2),
                               (x[..., : D // 2] ** 2 + x[..., D // 2:] ** 2))
    # interleaved pairing (2i, 2i+1) would give something else
    xi = x.view(T, H, D // 2, 2)
    wrong = torch.stack((xi[..., 0] * ang.cos()[:, None] - xi[..., 1] * ang.sin()[:, None],
                         xi[..., 1] * ang.cos()[:, None] + xi[..., 0] * ang.sin()[:, None]), dim=-1).view(T, H, D)
    assert not torch.allclose(wrong[1:], got[1:])


def test_rotary_scores_depend_on_distance_only():
    g = torch.Generator().manual_seed(2)
    D = 32
    q = torch.randn(1, 1, D, generator=g, dtype=torch.float64)
    k = torch.randn(1, 1, D, generator=g, dtype=torch.float64)

    def score(m, n):
        a = plain.apply_rotary(q, plain.rotary_angles(torch.tensor([m]), D, 1e4, torch.float64))
        b = plain.apply_rotary(k, plain.rotary_angles(torch.tensor([n]), D, 1e4, torch.float64))
        return float((a * b).sum())

    assert abs(score(5, 2) - score(105, 102)) < 1e-9
    assert abs(score(5, 2) - score(2, 5)) > 1e-6          # the sign of the distance matters


def test_attention_without_mask_window_or_groups_is_the_library_routine():
    g = torch.Generator().manual_seed(3)
    T, Hq, Hkv, D = 9, 6, 2, 16
    q = torch.randn(T, Hq, D, generator=g)
    k = torch.randn(T, Hkv, D, generator=g)
    v = torch.randn(T, Hkv, D, generator=g)
    got = plain.causal_attention(q, k, v, D ** -0.5)
    kk = k.repeat_interleave(Hq // Hkv, dim=1)            # grouped heads == repeated key heads
    vv = v.repeat_interleave(Hq // Hkv, dim=1)
    want = F.scaled_dot_product_attention(q.transpose(0, 1)[None], kk.transpose(0, 1)[None],
                                          vv.transpose(0, 1)[None], is_causal=True, scale=D ** -0.5)
    torch.testing.assert_close(got, want[0].transpose(0, 1), rtol=1e-5, atol=1e-5)
    # last row sees every key: plain softmax attention without any mask
    s = torch.softmax((q[-1, 0] @ k[:, 0].T) * D ** -0.5, dim=-1)
    torch.testing.assert_close(got[-1, 0], s @ v[:, 0], rtol=1e-5, atol=1e-5)
    # the first token's output is the first value
    torch.testing.assert_close(got[0], vv[0], rtol=1e-6, atol=1e-6)
    # a window of 1 returns each token's own value
    torch.testing.assert_close(plain.causal_attention(q, k, v, 1.0, window=1), vv, rtol=1e-6, atol=1e-6)


def test_swiglu_is_the_library_routine():
    # test/models/test_ffn.py:26-43 holds the reference to 1e-5 of this
    g = torch.Generator().manual_seed(4)
    H, I = 24, 40
    w = {"m.gate_proj.weight": torch.randn(I, H, generator=g), "m.up_proj.weight": torch.randn(I, H, generator=g),
         "m.down_proj.weight": torch.randn(H, I, generator=g)}
    x = torch.randn(5, H, generator=g)
    want = F.linear(F.silu(F.linear(x, w["m.gate_proj.weight"])) * F.linear(x, w["m.up_proj.weight"]),
                    w["m.down_proj.weight"])
    torch.testing.assert_close(plain.swiglu_mlp(x, w, "m"), want, rtol=1e-5, atol=1e-5)
    assert torch.count_nonzero(plain.swiglu_mlp(torch.zeros(2, H), w, "m")) == 0


def test_whole_model_invariants(model_folders):
    from helpers import random_tokens

    cfg, w = plain.read_model_folder(model_folders["B"], torch.float64)
    toks = random_tokens(20, cfg["vocab_size"], 9)
    full = plain.logits_of_sequence(cfg, w, toks)
    # causality: logits at t do not depend on tokens after t
    torch.testing.assert_close(plain.logits_of_sequence(cfg, w, toks[:11]), full[:11], rtol=1e-9, atol=1e-9)
    # a shift of all positions changes nothing: only distances count
    torch.testing.assert_close(plain.logits_of_sequence(cfg, w, toks, first_position=37), full,
                               rtol=1e-7, atol=1e-7)
    # q_norm and k_norm are distinct weights, applied before the rotation
    w2 = dict(w)
    w2["model.layers.0.self_attn.q_norm.weight"], w2["model.layers.0.self_attn.k_norm.weight"] = (
        w["model.layers.0.self_attn.k_norm.weight"], w["model.layers.0.self_attn.q_norm.weight"])
    assert not torch.allclose(plain.logits_of_sequence(cfg, w2, toks), full, atol=1e-6)
    # float32 agrees with float64 to rounding
    cfg32, w32 = plain.read_model_folder(model_folders["B"], torch.float32)
    torch.testing.assert_close(plain.logits_of_sequence(cfg32, w32, toks).double(), full, rtol=1e-4, atol=1e-5)


def test_tied_head_is_the_embedding(model_folders):
    cfg, w = plain.read_model_folder(model_folders["A"])
    assert cfg["tie_word_embeddings"] and "lm_head.weight" not in w
    cfg_b, w_b = plain.read_model_folder(model_folders["B"])
    assert not cfg_b["tie_word_embeddings"] and "lm_head.weight" in w_b


def test_head_norms_come_before_the_rotation():
    """With norm weights that differ between the two elements of a rotated pair, scores depend
    on the distance alone only if the norm comes first and the rotation last: the other order
    multiplies the halves of a rotated pair by different numbers and the property is gone."""
    g = torch.Generator().manual_seed(5)
    T, H, Hq, Hkv, D = 6, 24, 2, 1, 16
    cfg = dict(num_attention_heads=Hq, num_key_value_heads=Hkv, head_dim=D, rms_norm_eps=1e-6, rope_theta=100.0)
    w = {"a.%s_proj.weight" % n: torch.randn(rows, H, generator=g, dtype=torch.float64)
         for n, rows in (("q", Hq * D), ("k", Hkv * D), ("v", Hkv * D))}
    w["a.o_proj.weight"] = torch.randn(H, Hq * D, generator=g, dtype=torch.float64)
    gamma = torch.cat((torch.full((D // 2,), 0.3), torch.full((D // 2,), 2.5))).double()
    w["a.q_norm.weight"], w["a.k_norm.weight"] = gamma, 1.5 * gamma
    x = torch.randn(T, H, generator=g, dtype=torch.float64)
    here = plain.self_attention(x, w, "a", cfg, torch.arange(T))
    there = plain.self_attention(x, w, "a", cfg, torch.arange(T) + 1000)
    torch.testing.assert_close(here, there, rtol=1e-9, atol=1e-9)

    def other_order(positions):
        q = (x @ w["a.q_proj.weight"].T).view(T, Hq, D)
        k = (x @ w["a.k_proj.weight"].T).view(T, Hkv, D)
        v = (x @ w["a.v_proj.weight"].T).view(T, Hkv, D)
        ang = plain.rotary_angles(positions, D, 100.0, torch.float64)
        q = plain.rms_norm(plain.apply_rotary(q, ang), w["a.q_norm.weight"], 1e-6)
        k = plain.rms_norm(plain.apply_rotary(k, ang), w["a.k_norm.weight"], 1e-6)
        return plain.causal_attention(q, k, v, D ** -0.5).reshape(T, Hq * D) @ w["a.o_proj.weight"].T

    assert not torch.allclose(other_order(torch.arange(T)), other_order(torch.arange(T) + 1000), atol=1e-3)
    assert not torch.allclose(other_order(torch.arange(T)), here, atol=1e-3)


def _one_layer(g, zero):
    V, H, I, Hq, Hkv, D = 50, 24, 40, 2, 1, 16
    cfg = dict(num_hidden_layers=1, num_attention_heads=Hq, num_key_value_heads=Hkv, head_dim=D, rms_norm_eps=1e-5,
               rope_theta=1e4, tie_word_embeddings=False, vocab_size=V)
    shapes = {"model.embed_tokens.weight": (V, H), "lm_head.weight": (V, H),
              "model.layers.0.self_attn.q_proj.weight": (Hq * D, H), "model.layers.0.self_attn.k_proj.weight": (Hkv * D, H),
              "model.layers.0.self_attn.v_proj.weight": (Hkv * D, H), "model.layers.0.self_attn.o_proj.weight": (H, Hq * D),
              "model.layers.0.mlp.gate_proj.weight": (I, H), "model.layers.0.mlp.up_proj.weight": (I, H),
              "model.layers.0.mlp.down_proj.weight": (H, I)}
    w = {n: torch.randn(s, generator=g) * 0.3 for n, s in shapes.items()}
    for n in ("model.layers.0.input_layernorm.weight", "model.layers.0.post_attention_layernorm.weight",
              "model.norm.weight"):
        w[n] = 1 + 0.3 * torch.randn(H, generator=g)
    w["model.layers.0.self_attn.q_norm.weight"] = 1 + 0.3 * torch.randn(D, generator=g)
    w["model.layers.0.self_attn.k_norm.weight"] = 1 + 0.3 * torch.randn(D, generator=g)
    for n in zero:
        w[n] = torch.zeros_like(w[n])
    return cfg, w


def test_a_block_whose_parts_give_nothing_is_the_identity():
    """The norms sit before the parts and the stream is added outside them: with both output
    matrices zero a layer changes nothing, whatever the norms' weights; a norm on the stream
    itself (after the addition) would show."""
    g = torch.Generator().manual_seed(6)
    cfg, w = _one_layer(g, ("model.layers.0.self_attn.o_proj.weight", "model.layers.0.mlp.down_proj.weight"))
    x = torch.randn(7, 24, generator=g) * 5.0
    assert torch.equal(plain.decoder_layer(x, w, 0, cfg, torch.arange(7)), x)


def test_one_layer_without_attention_reduces_to_library_routines():
    """Embedding rows as they are (no factor), the second norm before the feed-forward, the sum
    outside it, the final norm, the head: with the attention's output matrix zero the whole
    model is a few library calls. A scaled embedding would change the balance between the
    stream and the feed-forward's addend, whose size does not depend on the stream's."""
    g = torch.Generator().manual_seed(7)
    cfg, w = _one_layer(g, ("model.layers.0.self_attn.o_proj.weight",))
    toks = [3, 17, 3, 44, 0, 49]
    x0 = F.embedding(torch.tensor(toks), w["model.embed_tokens.weight"])
    h = F.rms_norm(x0, (24,), w["model.layers.0.post_attention_layernorm.weight"], 1e-5)
    mlp = F.linear(F.silu(F.linear(h, w["model.layers.0.mlp.gate_proj.weight"]))
                   * F.linear(h, w["model.layers.0.mlp.up_proj.weight"]), w["model.layers.0.mlp.down_proj.weight"])
    want = F.linear(F.rms_norm(x0 + mlp, (24,), w["model.norm.weight"], 1e-5), w["lm_head.weight"])
    torch.testing.assert_close(plain.logits_of_sequence(cfg, w, toks), want, rtol=1e-5, atol=1e-5)
    scaled = F.linear(F.rms_norm(x0 * 24 ** 0.5 + mlp, (24,), w["model.norm.weight"], 1e-5), w["lm_head.weight"])
    assert not torch.allclose(scaled, want, atol=1e-2)


def test_peaked_weights_make_one_missing_key_show(model_folders, monkeypatch):
    """The tiny configurations with large weights and large query norms are there so that a key
    left out of the attention shows in the logits beyond the bound of the bfloat16 comparisons
    (a fiftieth of a row's spread), also for rows that have sixty other keys or more."""
    from helpers import random_tokens

    def worst_share(name, hidden_key):
        cfg, w = plain.read_model_folder(model_folders[name])
        toks = random_tokens(120, cfg["vocab_size"], 13)
        full = plain.logits_of_sequence(cfg, w, toks)
        whole = plain.causal_attention

        def without_one_key(q, k, v, scale, window=None):
            out = whole(q, k, v, scale, window)
            T = q.shape[0]
            keep = [j for j in range(T) if j != hidden_key]
            later = whole(q[keep], k[keep], v[keep], scale, window)     # the sequence as if that token's key were not there
            out = out.clone()
            for row, i in enumerate(keep):
                if i > hidden_key:
                    out[i] = later[row]
            return out

        monkeypatch.setattr(plain, "causal_attention", without_one_key)
        lacking = plain.logits_of_sequence(cfg, w, toks)
        monkeypatch.setattr(plain, "causal_attention", whole)
        spread = full.max(dim=1).values - full.min(dim=1).values
        share = (lacking - full).abs().max(dim=1).values / spread
        far = share[60:]                                               # rows with sixty keys or more
        return float(share.max()), float((far > 2e-2).float().mean())

    for name in ("DP", "EP"):
        worst, far_rows_over = worst_share(name, hidden_key=7)
        assert worst > 0.2 and far_rows_over > 0.3, (name, worst, far_rows_over)
