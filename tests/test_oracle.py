"""Pins the CPU oracle: golden vectors, PyTorch eager, and what the mathematics fixes."""

from __future__ import annotations

import numpy as np
import pytest
import torch
from torch import nn

from oracle import eager
from oracle import emmy_ops as O


def bf16_from_bits(bits):
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)


# -- golden vectors (reference test recipes) -------------------------------------


def test_rms_norm_golden(golden):
    x, w = golden["rms_sum_x"], golden["rms_sum_w"]
    np.testing.assert_allclose(O.rms_norm_sum(x, w, 1e-6), golden["rms_sum_y"], rtol=2e-6, atol=1e-7)
    np.testing.assert_allclose(O.rms_norm(x, w, 1e-6), golden["rms_mean_y"], rtol=2e-6, atol=1e-7)
    # the two variants differ exactly by the mean's 1/N inside the rsqrt
    assert not np.allclose(O.rms_norm(x, w, 1e-6), O.rms_norm_sum(x, w, 1e-6), rtol=1e-3)


@pytest.mark.parametrize("shape", ["4x8", "4x2048"])
def test_softmax_golden(golden, shape):
    np.testing.assert_allclose(O.softmax(golden[f"softmax_{shape}_x"]), golden[f"softmax_{shape}_y"], rtol=2e-6, atol=1e-10)


def test_linear_golden(golden):
    np.testing.assert_allclose(O.linear(golden["linear_f32_x"], golden["linear_f32_w"]), golden["linear_f32_y"], rtol=1e-6, atol=1e-6)


def test_config_goldens_match_current_torch(golden):
    """The committed vectors are what this container's eager produces for the seeded recipes."""
    np.testing.assert_allclose(eager.run_eager(eager.rms_norm_case(4, 2048)).numpy(), golden["c1_y"], rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(eager.run_eager(eager.softmax_case((1, 2, 8, 2048))).numpy(), golden["c2_y"], rtol=1e-6, atol=1e-10)
    got = eager.run_eager(eager.linear_case(32, 128, 96)).float()
    eager.assert_close(got, bf16_from_bits(golden["c3_y_bits"]).float(), 2e-2, 2e-2, "linear golden")
    got = eager.run_eager(eager.sdpa_case(1, 4, 2, 96, 128)).float()
    eager.assert_close(got, bf16_from_bits(golden["c4_y_bits"]).float(), 2e-2, 2e-2, "sdpa golden")


# -- restatement vs the library routine --------------------------------------------


def test_rms_norm_matches_torch():
    c = eager.rms_norm_case(rows=8, cols=512, seed=3)
    ref = eager.run_eager(c).numpy()
    got = O.rms_norm(c.inputs[0].numpy(), c.module.weight.detach().numpy(), 1e-6)
    np.testing.assert_allclose(got, ref, rtol=3e-6, atol=1e-7)


def test_rms_norm_invariant_unit_rms():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((5, 300)) * 7
    y = O.rms_norm(x, None, 0.0)
    np.testing.assert_allclose(np.sqrt((y * y).mean(-1)), 1.0, rtol=1e-12)


def test_softmax_properties():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((6, 77)) * 5
    y = O.softmax(x)
    np.testing.assert_allclose(y.sum(-1), 1.0, rtol=1e-13)
    np.testing.assert_allclose(O.softmax(x + 123.0), y, rtol=1e-12)  # shift invariance
    np.testing.assert_allclose(y, torch.softmax(torch.from_numpy(x), -1).numpy(), rtol=1e-12)


def test_silu_matches_torch():
    x = np.linspace(-20, 20, 401)
    np.testing.assert_allclose(O.silu(x), torch.nn.functional.silu(torch.from_numpy(x)).numpy(), rtol=1e-12, atol=1e-300)


def test_linear_brute_force():
    rng = np.random.default_rng(3)
    x, w = rng.standard_normal((3, 5)), rng.standard_normal((4, 5))
    want = np.array([[sum(x[i, k] * w[j, k] for k in range(5)) for j in range(4)] for i in range(3)])
    np.testing.assert_allclose(O.linear(x, w), want, rtol=1e-13)
    assert O.linear(x, w).shape == (3, 4)  # W is [out, in]: a transposed operand would not even broadcast


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("hq,hkv", [(4, 4), (4, 2), (6, 2)])
def test_sdpa_matches_torch(causal, hq, hkv):
    torch.manual_seed(5)
    q, k, v = torch.randn(2, hq, 9, 16, dtype=torch.float64), torch.randn(2, hkv, 9, 16, dtype=torch.float64), torch.randn(2, hkv, 9, 16, dtype=torch.float64)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=causal, enable_gqa=True).numpy()
    np.testing.assert_allclose(O.sdpa(q.numpy(), k.numpy(), v.numpy(), is_causal=causal), ref, rtol=1e-9, atol=1e-12)


def test_sdpa_gqa_head_mapping_brute_force():
    """kv head = q head // group (not modulo): distinguishable with 4 q heads over 2 kv heads."""
    rng = np.random.default_rng(7)
    q, k, v = rng.standard_normal((1, 4, 3, 8)), rng.standard_normal((1, 2, 3, 8)), rng.standard_normal((1, 2, 3, 8))
    got = O.sdpa(q, k, v, is_causal=True)
    for h in range(4):
        s = q[0, h] @ k[0, h // 2].T / np.sqrt(8)
        for i in range(3):
            p = np.exp(s[i, : i + 1] - s[i, : i + 1].max())
            np.testing.assert_allclose(got[0, h, i], (p / p.sum()) @ v[0, h // 2, : i + 1], rtol=1e-9)


# -- streaming carriers ------------------------------------------------------------------


@pytest.mark.parametrize("block", [1, 3, 7, 64])
def test_online_softmax_equals_softmax(block):
    rng = np.random.default_rng(11)
    x = rng.standard_normal((4, 50)) * 4
    np.testing.assert_allclose(O.online_softmax(x, block), O.softmax(x), rtol=1e-12)


def test_online_merge_is_associative_and_has_identity():
    rng = np.random.default_rng(12)
    parts = [(rng.standard_normal(5), rng.random(5) + 0.1) for _ in range(3)]
    a = O.online_softmax_merge(O.online_softmax_merge(parts[0], parts[1]), parts[2])
    b = O.online_softmax_merge(parts[0], O.online_softmax_merge(parts[1], parts[2]))
    np.testing.assert_allclose(a[0], b[0])
    np.testing.assert_allclose(a[1], b[1], rtol=1e-13)
    ident = (np.full(5, -1e30), np.zeros(5))
    m, d = O.online_softmax_merge(ident, parts[0])
    np.testing.assert_allclose(m, parts[0][0])
    np.testing.assert_allclose(d, parts[0][1])


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("block_kv", [1, 4, 5, 64])
def test_flash_equals_sdpa(causal, block_kv):
    rng = np.random.default_rng(13)
    q, k, v = rng.standard_normal((1, 4, 11, 8)), rng.standard_normal((1, 2, 11, 8)), rng.standard_normal((1, 2, 11, 8))
    want = O.sdpa(q, k, v, is_causal=causal)
    got = O.flash_attention(q, k, v, is_causal=causal, scale=1 / np.sqrt(8), block_kv=block_kv)
    np.testing.assert_allclose(got, want, rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("mask_shape", [(1, 1, 9, 13), (2, 1, 9, 13), (2, 4, 9, 13), (1, 4, 1, 13)])
def test_sdpa_additive_mask_matches_torch(mask_shape):
    """The mask is added to the *scaled* scores (a mask added before the scale, or multiplied in, fails), and
    broadcasts over batch, heads and queries; ``-inf`` entries drop a key."""
    torch.manual_seed(21)
    q, k, v = torch.randn(2, 4, 9, 16, dtype=torch.float64), torch.randn(2, 2, 13, 16, dtype=torch.float64), torch.randn(2, 2, 13, 16, dtype=torch.float64)
    mask = torch.randn(mask_shape, dtype=torch.float64) * 3
    mask[..., 5] = -float("inf")
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask, enable_gqa=True).numpy()
    np.testing.assert_allclose(O.sdpa(q.numpy(), k.numpy(), v.numpy(), is_causal=False, mask=mask.numpy()), ref, rtol=1e-9, atol=1e-12)
    for block_kv in (1, 4, 64):
        got = O.flash_attention(q.numpy(), k.numpy(), v.numpy(), is_causal=False, scale=0.25, block_kv=block_kv, mask=mask.numpy())
        np.testing.assert_allclose(got, ref, rtol=1e-9, atol=1e-12)


def test_sdpa_mask_replaces_the_causal_term():
    """A ``0 / -inf`` lower-triangular bias is the causal attention (closed form), and with a mask present the
    ``is_causal`` flag is not applied on top (decomposition/010_sdpa.py:91-101)."""
    rng = np.random.default_rng(22)
    q, k, v = rng.standard_normal((1, 2, 7, 8)), rng.standard_normal((1, 2, 7, 8)), rng.standard_normal((1, 2, 7, 8))
    tri = np.where(np.arange(7)[None, :] > np.arange(7)[:, None], -np.inf, 0.0)[None, None]
    np.testing.assert_allclose(O.sdpa(q, k, v, is_causal=False, mask=tri), O.sdpa(q, k, v, is_causal=True), rtol=1e-12)
    zero = np.zeros((1, 1, 7, 7))
    np.testing.assert_allclose(O.sdpa(q, k, v, is_causal=True, mask=zero), O.sdpa(q, k, v, is_causal=False), rtol=1e-12)


# -- bf16 carrier ------------------------------------------------------------------------------


def test_bf16_round_matches_torch_including_ties():
    rng = np.random.default_rng(17)
    x = np.concatenate([
        rng.standard_normal(4096).astype(np.float32) * 100,
        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, np.inf, -np.inf, 1e-40, 65504.0], dtype=np.float32),
        # exact ties: mantissa bit 16 set and nothing below (round to even both ways)
        np.array([0x3F808000, 0x3F818000, 0xBF808000, 0xBF818000], dtype=np.uint32).view(np.float32),
    ])
    want = torch.from_numpy(x).bfloat16().float().numpy()
    np.testing.assert_array_equal(O.bf16_round(x), want)
    assert np.isnan(O.bf16_round(np.array([np.nan], dtype=np.float32))[0])
    np.testing.assert_array_equal(O.from_bf16_bits(O.bf16_bits(x)), want)


def test_product_bf16_helpers_agree_with_oracle():
    from deplodock_amd.dtype import bf16_bits_from_f32, f32_from_bf16_bits

    x = (np.random.default_rng(19).standard_normal(1000) * 50).astype(np.float32)
    np.testing.assert_array_equal(bf16_bits_from_f32(x), O.bf16_bits(x))
    np.testing.assert_array_equal(f32_from_bf16_bits(O.bf16_bits(x)), O.bf16_round(x))


# -- block composition ------------------------------------------------------------------------------


def test_qwen3_block_restatement_matches_eager_fp32(golden):
    c = eager.qwen3_block_case(seq=32, dtype=torch.float32)
    x, cos, sin = (t.numpy() for t in c.inputs)
    got = O.qwen3_block(x, cos, sin, eager.block_weights(c), q_heads=16, kv_heads=8, head_dim=128, eps=1e-6)
    np.testing.assert_allclose(got, golden["c5_y_f32"], rtol=2e-4, atol=2e-4)
    np.testing.assert_allclose(eager.run_eager(c).numpy(), golden["c5_y_f32"], rtol=1e-5, atol=1e-5)


def test_rotate_half():
    x = np.arange(8.0)[None]
    np.testing.assert_array_equal(O.rotate_half(x), np.array([[-4.0, -5, -6, -7, 0, 1, 2, 3]]))


def test_deferred_rms_norm_identity():
    """What the fused block relies on when it defers a layer norm into the projections that read it:
    ``rms_norm(x, w) @ W^T == r * (x @ (W * w)^T)`` with ``r = rsqrt(mean x^2 + eps)`` per row, checked in
    float64 against the restated norm and linear (a wrong axis for ``w``, a missing ``eps`` or a ``mean``
    taken as a sum breaks it)."""
    rng = np.random.default_rng(7)
    x = rng.standard_normal((5, 96)) * 3.0
    w = 1.0 + 0.3 * rng.standard_normal(96)
    big_w = 0.05 * rng.standard_normal((40, 96))
    eps = 1e-6
    direct = O.linear(O.rms_norm(x, w, eps), big_w)
    r = 1.0 / np.sqrt((x * x).mean(-1, keepdims=True) + eps)
    deferred = r * O.linear(x, big_w * w[None, :])
    np.testing.assert_allclose(deferred, direct, rtol=1e-5, atol=1e-6)


# -- the scale-aware parity criteria themselves ----------------------------------------------------


def _attention_with_dropped_block(q, k, v, row_from: int, key0: int, key1: int):
    """fp32 causal attention in which rows >= ``row_from`` never see keys [key0, key1): what a flash loop
    that skips one key block for late rows computes (the block is missing from numerator and denominator)."""
    s = q.shape[-2]
    mask = torch.ones(s, s, dtype=torch.bool).tril()
    mask[row_from:, key0:key1] = False
    return nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask)


def test_row_relative_criterion_sees_a_dropped_key_block():
    """At S=2048 a late row's output is ~0.03 large, so the elementwise bound (rtol 2e-2 + atol 2e-2) hardly
    sees an output with a whole 32-key block missing from its late rows: with random V it leaves 99 % of the
    affected elements inside (only rows where the block held a dominant key stick out), and with
    position-coded V it accepts the result outright.  The row-relative criterion against fp32 eager rejects
    both, every affected row by a wide margin; V = 1 cannot see the omission at all (rows still sum to one)."""
    torch.manual_seed(0)
    s, d, row_from = 2048, 128, 1024
    q, k, v = (torch.randn(1, 2, s, d).bfloat16() for _ in range(3))
    qf, kf, vf = q.float(), k.float(), v.float()
    exact = nn.functional.scaled_dot_product_attention(qf, kf, vf, is_causal=True)
    bf16_eager = nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)
    wrong = _attention_with_dropped_block(qf, kf, vf, row_from=row_from, key0=256, key1=288).bfloat16()
    outside = (wrong.float() - exact).abs() > 2e-2 + 2e-2 * exact.abs()
    assert float(outside[:, :, row_from:].float().mean()) < 0.02  # the loose bound passes 98 % of what is wrong
    eager.assert_rows_within_baseline(bf16_eager, bf16_eager, exact, 1.5, "bf16 eager against itself")
    with pytest.raises(AssertionError, match="row-relative L2"):
        eager.assert_rows_within_baseline(wrong, bf16_eager, exact, 1.5, "dropped block")
    limit = 1.5 * float(eager.row_rel_l2(bf16_eager, exact).max())
    assert bool((eager.row_rel_l2(wrong, exact)[:, :, row_from:] > 5 * limit).all())  # every affected row, 5x over
    # the same omission under V = 1 is invisible, under position-coded V it is not
    ones = torch.ones_like(vf)
    assert float((_attention_with_dropped_block(qf, kf, ones, row_from, 256, 288) - 1).abs().max()) < 1e-5
    vpos = eager.position_coded_values(v)
    np.testing.assert_array_equal(vpos[0, 0, :, 0].float().numpy(), (torch.arange(s) / s).bfloat16().float().numpy())
    exact_p = nn.functional.scaled_dot_product_attention(qf, kf, vpos.float(), is_causal=True)
    eager_p = nn.functional.scaled_dot_product_attention(q, k, vpos, is_causal=True)
    wrong_p = _attention_with_dropped_block(qf, kf, vpos.float(), row_from, 256, 288).bfloat16()
    eager.assert_close(wrong_p, exact_p, 2e-2, 2e-2, "the loose bound accepts the wrong result")  # does not raise
    eager.assert_rows_within_baseline(eager_p, eager_p, exact_p, 1.5, "bf16 eager against itself, coded V")
    with pytest.raises(AssertionError, match="row-relative L2"):
        eager.assert_rows_within_baseline(wrong_p, eager_p, exact_p, 1.5, "dropped block, coded V")
    limit_p = 1.5 * float(eager.row_rel_l2(eager_p, exact_p).max())
    assert float((eager.row_rel_l2(wrong_p, exact_p)[:, :, row_from:] > limit_p).float().mean()) > 0.95


def test_mean_error_criterion_sees_a_wrong_norm_weight_pairing():
    """The block criterion: on out - x, our mean distance from the fp32 run may be at most 1.5 x bf16
    eager's.  A block whose post-attention norm weights are applied to the wrong columns (rolled by one)
    passes the elementwise bound atol 4e-2 on most elements and fails this one."""
    c = eager.qwen3_block_case(seq=64, norm_std=0.1, seed=3)
    exact = eager.run_eager_fp32(c)
    bf16 = eager.run_eager(c).float()
    x = c.inputs[0].float()
    eager.assert_mean_error_within_baseline(bf16 - x, bf16 - x, exact - x, 1.5, "bf16 eager against itself")
    import copy

    broken = copy.deepcopy(c)
    with torch.no_grad():
        w = broken.module.l.post_attention_layernorm.weight
        w.copy_(torch.roll(w, 1))
    wrong = eager.run_eager(broken).float()
    assert float(((wrong - bf16).abs() <= 4e-2 + 2e-2 * bf16.abs()).float().mean()) > 0.5  # the loose bound passes most of it
    with pytest.raises(AssertionError, match="exceeds"):
        eager.assert_mean_error_within_baseline(wrong - x, bf16 - x, exact - x, 1.5, "rolled norm weights")
    with pytest.raises(AssertionError, match="row-relative L2"):
        eager.assert_rows_within_baseline(wrong - x, bf16 - x, exact - x, 1.5, "rolled norm weights")
