"""Pins the oracle's restatement of the kernels around the attention (QGKV split, RMSNorm + RoPE,
sigmoid gate) to the known answers the reference's own tests hold, each recomputed here from the
closed form the reference test states -- not from the oracle's code."""
import math

import numpy as np

YARN = dict(factor=32.0, attention_factor=float(np.float32(1.0) + np.float32(0.1) * np.log(np.float32(32.0))),
            beta_fast=32.0, beta_slow=1.0, original_max_position_embeddings=8192, truncate=True)


def bf16_bits(oracle, values):
    return oracle.from_f32(np.asarray(values, np.float32), oracle.BF16)


def test_two_token_split_norm_rope_gate_closed_forms(oracle):
    """crates/inference-executor-metal/src/attn/gqa/backend.rs:883-1027: 1 Q head / 1 KV head of 2 dims,
    weights 1, positions 0 and 1, tolerance 2e-5."""
    rows = np.array([[1.0, 2.0, 0.5, -0.5, 3.0, 4.0, 5.0, 6.0], [2.0, 1.0, -1.0, 1.0, 4.0, 3.0, 6.0, 5.0]], np.float32)
    q, g, k, v = oracle.qgkv_split(rows.ravel(), 2, 1, 1, 2, oracle.F32)
    assert q.tolist() == [1, 2, 2, 1] and g.tolist() == [0.5, -0.5, -1, 1]
    assert k.tolist() == [3, 4, 4, 3] and v.tolist() == [5, 6, 6, 5]
    inv, factor, _ = oracle.rope_parameters(2, 1_000_000.0)
    assert inv.tolist() == [1.0] and factor == 1.0
    ones = bf16_bits(oracle, [1.0, 1.0])

    def norm_rope_2(row, position):
        inv_rms = 1.0 / math.sqrt((row[0] * row[0] + row[1] * row[1]) / 2.0 + 1.0e-6)
        x0, x1 = row[0] * inv_rms, row[1] * inv_rms
        return [x0 * math.cos(position) - x1 * math.sin(position), x0 * math.sin(position) + x1 * math.cos(position)]

    for t, name in ((q, "q"), (k, "k")):
        got = oracle.rms_norm_rope(t, ones, [0, 1], 1, 2, 2, 1e-6, inv, factor, oracle.F32)
        exp = norm_rope_2(t[:2], 0.0) + norm_rope_2(t[2:], 1.0)
        assert np.abs(got - np.array(exp)).max() <= 2e-5, name
    q_norm = oracle.rms_norm_rope(q, ones, [0, 1], 1, 2, 2, 1e-6, inv, factor, oracle.F32)
    gated = oracle.activation_gate(q_norm, g, oracle.F32)
    exp = [x / (1.0 + math.exp(-gate)) for x, gate in zip(q_norm.astype(np.float64), g.astype(np.float64))]
    assert np.abs(gated - np.array(exp)).max() <= 2e-5
    # inactive tokens keep their bytes: one active token of two
    q1, g1, k1, v1 = oracle.qgkv_split(rows.ravel(), 1, 1, 1, 2, oracle.F32)
    assert q1.tolist() == [1, 2] and v1.tolist() == [5, 6]


def test_yarn_correction_range(oracle):
    """rms_norm_rope.rs:377-393: (low, high) = (14, 29) for rope_dim 128, theta 1e7, beta 32 / 1, 8192."""
    _, factor, corr = oracle.rope_parameters(128, 10_000_000.0, YARN)
    assert corr == (14.0, 29.0)
    assert factor == np.float32(1.0) + np.float32(0.1) * np.log(np.float32(32.0))


def test_f32_yarn_long_context_closed_form(oracle):
    """rms_norm_rope.rs:395-470: one head of 128 dims at position 262143, tolerance 1e-3."""
    x = np.array([((i * 37 % 29) - 14.0) / 8.0 for i in range(128)], np.float32)
    w = np.array([0.75 + (i % 11) / 20.0 for i in range(128)], np.float32)
    w_bits = bf16_bits(oracle, w)
    w_f = oracle.to_f32(w_bits, oracle.BF16).astype(np.float64)
    inv, factor, corr = oracle.rope_parameters(128, 10_000_000.0, YARN)
    got = oracle.rms_norm_rope(x, w_bits, [262143], 1, 128, 128, 1e-6, inv, factor, oracle.F32)
    inv_rms = 1.0 / math.sqrt(float((x.astype(np.float64) ** 2).sum()) / 128 + 1e-6)
    exp = np.zeros(128)
    for d in range(64):
        ramp = min(max((d - corr[0]) / (corr[1] - corr[0]), 0.0), 1.0)
        inv_freq = np.float32(np.float32(10_000_000.0) ** np.float32(-(d / 64.0))) * np.float32(1.0 + ramp * (1.0 / 32.0 - 1.0))
        theta = float(np.float32(262143.0) * np.float32(inv_freq))
        first, second = w_f[d] * x[d] * inv_rms, w_f[d + 64] * x[d + 64] * inv_rms
        exp[d] = factor * (first * math.cos(theta) - second * math.sin(theta))
        exp[d + 64] = factor * (first * math.sin(theta) + second * math.cos(theta))
    assert np.abs(got - exp).max() < 1e-3


def test_bf16_norm_rounding_order_is_bit_exact(oracle):
    """rms_norm_rope.rs:472-517: head_dim 4, rope_dim 2, position 0: every element equals
    bf16(w * bf16(x * inv_rms)), bit for bit (the rotation at angle 0 is the identity)."""
    x_bits = bf16_bits(oracle, [0.73046875, -1.171875, 0.43945313, 2.03125])
    w_bits = bf16_bits(oracle, [1.296875, 0.8984375, 1.1015625, 0.703125])
    inv, factor, _ = oracle.rope_parameters(2, 1_000_000.0)
    got = oracle.rms_norm_rope(x_bits, w_bits, [0], 1, 4, 2, 1e-6, inv, factor, oracle.BF16)
    x = oracle.to_f32(x_bits, oracle.BF16)
    w = oracle.to_f32(w_bits, oracle.BF16)
    inv_rms = np.float32(1.0) / np.sqrt(np.float32((x * x).sum(dtype=np.float32) / np.float32(4.0) + np.float32(1e-6)))
    normalized = oracle.to_f32(bf16_bits(oracle, x * inv_rms), oracle.BF16)
    exp = bf16_bits(oracle, w * normalized)
    assert got.tolist() == exp.tolist()


def test_bf16_gate_rounds_after_every_step(oracle):
    """gqa_activation_gate.metal:13-27: |x| -> exp(-|x|) -> 1 + e -> 1 / d -> (1 - y for x < 0), each
    rounded to bf16, then one bf16 product; checked against the same chain in numpy on 4096 values."""
    rng = np.random.default_rng(5)
    a_bits = bf16_bits(oracle, rng.normal(0, 1, 4096))
    g_bits = bf16_bits(oracle, rng.normal(0, 3, 4096))
    got = oracle.activation_gate(a_bits, g_bits, oracle.BF16)

    def r(v):
        return oracle.to_f32(bf16_bits(oracle, v), oracle.BF16)

    a, g = oracle.to_f32(a_bits, oracle.BF16), oracle.to_f32(g_bits, oracle.BF16)
    y = r(np.float32(1.0) / r(np.float32(1.0) + r(np.exp(-np.abs(g), dtype=np.float32))))
    s = np.where(g < 0, r(np.float32(1.0) - y), y)
    exp = bf16_bits(oracle, a * s)
    # numpy's and libm's expf may differ in the last place, which a bf16 rounding occasionally shows
    assert (got != exp).mean() < 0.01
    assert np.abs(oracle.to_f32(got, oracle.BF16) - oracle.to_f32(exp, oracle.BF16)).max() <= 2 ** -6
    # sigmoid symmetry and limits in f32
    big = oracle.activation_gate(np.ones(3, np.float32), np.array([-100.0, 0.0, 100.0], np.float32), oracle.F32)
    assert big.tolist() == [0.0, 0.5, 1.0]


def test_split_is_a_permutation(oracle):
    """Every input slot lands in exactly one output slot, for bf16 storage too."""
    hq, hkv, d, t = 6, 2, 8, 5
    width = 2 * hq * d + 2 * hkv * d
    src = np.arange(t * width, dtype=np.uint16)
    q, g, k, v = oracle.qgkv_split(src, t, hq, hkv, d, oracle.BF16)
    assert sorted(np.concatenate([q, g, k, v]).tolist()) == src.tolist()
    row = src.reshape(t, width)
    assert (q.reshape(t, hq, d)[:, 1] == row[:, 2 * d:3 * d]).all()      # second pair, q half
    assert (g.reshape(t, hq, d)[:, 1] == row[:, 3 * d:4 * d]).all()      # second pair, g half
    assert (k.reshape(t, hkv * d) == row[:, 2 * hq * d:2 * hq * d + hkv * d]).all()
