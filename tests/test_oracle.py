"""Pins the CPU oracle before anything is compared with it: the reference's own known answers
(tests/golden/reference_vectors.json), closed forms, a float64 brute force written independently
with numpy, invariants a wrong index or a dropped term would break, and independent library
conversions (torch bfloat16, numpy float16) for the storage formats."""
import json
import math
import os

import numpy as np
import pytest

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))


# ------------------------------------------------------------------ softmax


def test_softmax_closed_form(oracle):
    g = GOLDEN["softmax"]
    out = oracle.softmax(np.log(np.array(g["logits_ln"], np.float64)).astype(np.float32))
    assert np.abs(out - np.array(g["expected"])).max() <= g["tolerance"]


def test_softmax_properties(oracle):
    rng = np.random.default_rng(0)
    x = rng.normal(size=37).astype(np.float32) * 5
    p = oracle.softmax(x)
    assert abs(float(p.sum()) - 1) < 1e-6 and (p > 0).all()
    assert np.abs(oracle.softmax(x + 3.5) - p).max() < 1e-6  # shift invariance
    assert np.allclose(oracle.softmax(np.full(8, 2.0, np.float32)), 1 / 8)
    ref = np.exp(x.astype(np.float64) - x.max())
    assert np.abs(p - ref / ref.sum()).max() < 1e-6
    assert oracle.softmax(np.array([-1e4, 0.0], np.float32)).tolist() == [0.0, 1.0]  # underflow, not NaN


def test_softmax_rejects_non_finite(oracle):
    with pytest.raises(ValueError):
        oracle.softmax(np.array([0.0, np.nan], np.float32))
    with pytest.raises(ValueError):
        oracle.softmax(np.array([np.inf, 0.0], np.float32))


# ------------------------------------------------------------------ attention


def test_causal_two_token_known_answer(oracle):
    g = GOLDEN["causal_two_tokens"]
    out = oracle.projected_gqa_reference(g["num_q_heads"], g["num_kv_heads"], g["head_dim"], g["scale"],
                                         g["cu_tokens"], g["token_indices"], np.array(g["q"], np.float32),
                                         [np.array(g["context_k"], np.float32)], [np.array(g["context_v"], np.float32)])
    # the reference forms the expectation in f32 as well (an f32 ulp at 17.6 is 1.9e-6)
    first = np.exp(np.float32(-2.0))
    total = np.float32(first + np.float32(1.0))
    w1, w2 = np.float32(first / total), np.float32(np.float32(1.0) / total)
    expected = np.array(g["expected_first_token"] + [np.float32(10) * w1, np.float32(20) * w2] * 2, np.float32)
    assert np.abs(out - expected).max() < g["tolerance"]
    w = math.exp(-2) / (1 + math.exp(-2))
    assert np.abs(out[4:] - np.array([10 * w, 20 * (1 - w)] * 2)).max() < 2e-6


def brute_force(hq, hkv, d, scale, cu, starts, q, ks, vs):
    """Independent float64 statement: token i of request r sits at position starts[r] + i and sees
    keys [0, position]; query head h reads KV head h // (hq / hkv)."""
    group = hq // hkv
    out = np.zeros((cu[-1], hq, d))
    q = np.asarray(q, np.float64).reshape(cu[-1], hq, d)
    for r, start in enumerate(starts):
        k = np.asarray(ks[r], np.float64).reshape(-1, hkv, d)
        v = np.asarray(vs[r], np.float64).reshape(-1, hkv, d)
        for i in range(cu[r + 1] - cu[r]):
            t = cu[r] + i
            visible = start + i + 1
            for h in range(hq):
                logits = k[:visible, h // group] @ q[t, h] * scale
                p = np.exp(logits - logits.max())
                out[t, h] = (p / p.sum()) @ v[:visible, h // group]
    return out.reshape(-1)


@pytest.mark.parametrize("seed", range(8))
def test_against_float64_brute_force(oracle, seed):
    rng = np.random.default_rng(seed)
    hkv = int(rng.choice([1, 2, 3]))
    group = int(rng.choice([1, 2, 6]))
    hq, d = hkv * group, int(rng.choice([2, 8, 16]))
    counts = rng.integers(1, 4, size=int(rng.integers(1, 4)))
    starts = [int(s) for s in rng.integers(0, 20, size=len(counts))]
    cu = [0] + np.cumsum(counts).tolist()
    scale = float(rng.uniform(0.1, 1.0))
    q = rng.normal(size=cu[-1] * hq * d).astype(np.float32)
    ks = [rng.normal(size=(starts[r] + counts[r]) * hkv * d).astype(np.float32) for r in range(len(counts))]
    vs = [rng.normal(size=k.size).astype(np.float32) for k in ks]
    out = oracle.projected_gqa_reference(hq, hkv, d, scale, cu, starts, q, ks, vs)
    assert np.abs(out - brute_force(hq, hkv, d, scale, cu, starts, q, ks, vs)).max() < 2e-5


def _one(oracle, hq, hkv, d, scale, start, n, q, k, v, threads=1):
    return oracle.projected_gqa_reference(hq, hkv, d, scale, [0, n], [start], q, [k], [v], num_threads=threads)


def test_uniform_keys_give_the_mean_of_values(oracle):
    rng = np.random.default_rng(1)
    hq, hkv, d, ctx = 4, 2, 8, 33
    k = np.tile(rng.normal(size=(1, hkv, d)), (ctx, 1, 1)).astype(np.float32)
    v = rng.normal(size=(ctx, hkv, d)).astype(np.float32)
    q = rng.normal(size=(1, hq, d)).astype(np.float32)
    out = _one(oracle, hq, hkv, d, 0.7, ctx - 1, 1, q, k, v).reshape(hq, d)
    for h in range(hq):
        assert np.abs(out[h] - v[:, h // 2].mean(axis=0)).max() < 1e-5


def test_value_linearity_and_scale_equivalence(oracle):
    rng = np.random.default_rng(2)
    hq, hkv, d, ctx = 6, 1, 16, 50
    q = rng.normal(size=(2, hq, d)).astype(np.float32)
    k = rng.normal(size=(ctx, hkv, d)).astype(np.float32)
    v1 = rng.normal(size=(ctx, hkv, d)).astype(np.float32)
    v2 = rng.normal(size=(ctx, hkv, d)).astype(np.float32)
    a = _one(oracle, hq, hkv, d, 0.25, ctx - 2, 2, q, k, v1)
    b = _one(oracle, hq, hkv, d, 0.25, ctx - 2, 2, q, k, v2)
    c = _one(oracle, hq, hkv, d, 0.25, ctx - 2, 2, q, k, v1 + v2)
    assert np.abs(a + b - c).max() < 1e-5
    # scaling q by 2 and halving the scale is the same computation up to rounding
    e = _one(oracle, hq, hkv, d, 0.125, ctx - 2, 2, q * 2, k, v1)
    assert np.abs(a - e).max() < 1e-5


def test_causality_and_position_dependence(oracle):
    rng = np.random.default_rng(3)
    hq, hkv, d, start, n = 2, 2, 8, 10, 3
    q = rng.normal(size=(n, hq, d)).astype(np.float32)
    k = rng.normal(size=(start + n, hkv, d)).astype(np.float32)
    v = rng.normal(size=(start + n, hkv, d)).astype(np.float32)
    base = _one(oracle, hq, hkv, d, 0.5, start, n, q, k, v).reshape(n, -1)
    k2, v2 = k.copy(), v.copy()
    k2[start + 1:] += 3.0  # keys the first token must not see
    v2[start + 1:] -= 5.0
    moved = _one(oracle, hq, hkv, d, 0.5, start, n, q, k2, v2).reshape(n, -1)
    assert np.array_equal(base[0], moved[0])
    assert not np.allclose(base[1], moved[1]) and not np.allclose(base[2], moved[2])
    k3 = k.copy()
    k3[start] += 3.0  # the token's own key is visible to it
    assert not np.allclose(base[0], _one(oracle, hq, hkv, d, 0.5, start, n, q, k3, v).reshape(n, -1)[0])


def test_kv_head_mapping(oracle):
    """Query heads [g*G, (g+1)*G) read KV head g and nothing else."""
    rng = np.random.default_rng(4)
    hq, hkv, d, ctx = 6, 3, 4, 9
    q = rng.normal(size=(1, hq, d)).astype(np.float32)
    k = rng.normal(size=(ctx, hkv, d)).astype(np.float32)
    v = rng.normal(size=(ctx, hkv, d)).astype(np.float32)
    base = _one(oracle, hq, hkv, d, 1.0, ctx - 1, 1, q, k, v).reshape(hq, d)
    v2 = v.copy()
    v2[:, 1] += 1.0
    moved = _one(oracle, hq, hkv, d, 1.0, ctx - 1, 1, q, k, v2).reshape(hq, d)
    assert np.array_equal(base[[0, 1, 4, 5]], moved[[0, 1, 4, 5]])
    assert np.abs(moved[[2, 3]] - base[[2, 3]] - 1.0).max() < 1e-5


def test_threads_do_not_change_a_bit(oracle):
    rng = np.random.default_rng(5)
    hq, hkv, d = 8, 2, 32
    cu, starts = [0, 3, 4, 9], [100, 0, 57]
    q = rng.normal(size=cu[-1] * hq * d).astype(np.float32)
    ks = [rng.normal(size=(starts[r] + cu[r + 1] - cu[r]) * hkv * d).astype(np.float32) for r in range(3)]
    vs = [rng.normal(size=k.size).astype(np.float32) for k in ks]
    a = oracle.projected_gqa_reference(hq, hkv, d, 0.3, cu, starts, q, ks, vs, num_threads=1)
    b = oracle.projected_gqa_reference(hq, hkv, d, 0.3, cu, starts, q, ks, vs, num_threads=4)
    assert np.array_equal(a, b)


def test_rejects_malformed_batches(oracle):
    q = np.zeros(4, np.float32)
    k = np.zeros(4, np.float32)
    with pytest.raises((ValueError, AssertionError)):
        oracle.projected_gqa_reference(3, 2, 2, 1.0, [0, 1], [0], q, [k], [k])  # heads not divisible
    with pytest.raises((ValueError, AssertionError)):
        oracle.projected_gqa_reference(2, 1, 2, 1.0, [1, 2], [0], q, [k], [k])  # cu must start at 0


# ------------------------------------------------------------------ storage formats


def test_bf16_round_trip_is_exhaustive_and_matches_torch(oracle):
    import torch

    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    f = oracle.to_f32(bits, oracle.BF16)
    assert np.array_equal(f.view(np.uint32), bits.astype(np.uint32) << 16)
    back = oracle.from_f32(f, oracle.BF16)
    nan = np.isnan(f)
    assert np.array_equal(back[~nan], bits[~nan])
    assert np.isnan(oracle.to_f32(back[nan], oracle.BF16)).all()
    rng = np.random.default_rng(6)
    x = np.concatenate([rng.normal(size=200000).astype(np.float32) * 10,
                        (rng.integers(0, 2**32, size=200000, dtype=np.uint64).astype(np.uint32)).view(np.float32)])
    x = x[np.isfinite(x)]
    ours = oracle.from_f32(x, oracle.BF16)
    theirs = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(ours, theirs)


def test_bf16_ties_round_to_even(oracle):
    def enc(v):
        return int(oracle.from_f32(np.array([v], np.float32), oracle.BF16)[0])

    assert enc(1.0) == 0x3F80
    assert enc(1.0 + 2.0**-8) == 0x3F80  # exact tie, even mantissa below
    assert enc(1.0 + 3 * 2.0**-8) == 0x3F82  # exact tie, odd mantissa below rounds up
    assert enc(1.0 + 2.0**-8 + 2.0**-20) == 0x3F81  # just above the tie
    assert enc(-0.0) == 0x8000 and enc(np.inf) == 0x7F80
    assert enc(3.3895313892515355e38) == 0x7F7F  # largest finite bf16
    assert enc(3.4028234663852886e38) == 0x7F80  # f32 max rounds up into infinity


def test_f16_round_trip_is_exhaustive_and_matches_numpy(oracle):
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    f = oracle.to_f32(bits, oracle.F16)
    expected = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(expected)
    assert np.array_equal(f[~nan], expected[~nan]) and np.isnan(f[nan]).all()
    back = oracle.from_f32(f, oracle.F16)
    assert np.array_equal(back[~nan], bits[~nan])
    rng = np.random.default_rng(7)
    x = np.concatenate([rng.normal(size=200000).astype(np.float32) * 100,
                        rng.normal(size=50000).astype(np.float32) * 1e-6,  # subnormal range
                        np.array([65504.0, 65519.9, 65520.0, 1e9, -1e9, 5.96e-8, 2.98e-8, 2.99e-8], np.float32)])
    with np.errstate(over="ignore"):
        assert np.array_equal(oracle.from_f32(x, oracle.F16), x.astype(np.float16).view(np.uint16))


# ------------------------------------------------------------------ pages


def test_page_write_known_answers(oracle):
    g = GOLDEN["page_write_single_token"]
    for dtype, np_t in ((oracle.BF16, np.uint16), (oracle.F16, np.uint16), (oracle.F32, np.float32)):
        pages = np.zeros(g["page_elements"], np_t)
        oracle.kv_page_write(pages, np.array(g["flat_k"], np_t), np.array(g["flat_v"], np_t), g["req_slots"],
                             g["flat_token_indices"], g["page_ids"], 1, 0, g["layout"], g["num_kv_heads"],
                             g["head_dim"], g["page_elements"] * pages.itemsize, dtype)
        assert pages.tolist() == g["expected_page"]


def test_page_write_bucketed_canary(oracle):
    g = GOLDEN["page_write_bucketed_canary"]
    n = g["page_elements"]
    for active, untouched in ((3, True), (4, False)):
        pages = np.full(2 * n, g["sentinel"], np.uint16)
        oracle.kv_page_write(pages, np.array(g["flat_k"], np.uint16), np.array(g["flat_v"], np.uint16),
                             g["req_slots"], g["flat_token_indices"], g["page_ids"], active, 0, g["layout"],
                             g["num_kv_heads"], g["head_dim"], n * 2, oracle.BF16)
        assert (pages[n:] == g["sentinel"]).all() == untouched
        # page 0: K rows of tokens 0..2 then one untouched K row, V likewise ([K|V][head][token][dim])
        assert pages[:6].tolist() == [10, 11, 12, 13, 14, 15] and pages[8:14].tolist() == [20, 21, 22, 23, 24, 25]
        assert pages[6:8].tolist() == [g["sentinel"]] * 2
    assert pages[n:n + 2].tolist() == [16, 17] and pages[n + 8:n + 10].tolist() == [26, 27]


def pack_pages(k, v, page_ids, tokens_per_page, num_pages):
    """Independent statement of the page layout: page = [K|V][kv_head][token_in_page][dim]."""
    ctx, hkv, d = k.shape
    pages = np.zeros((num_pages, 2, hkv, tokens_per_page, d), k.dtype)
    for t in range(ctx):
        page = page_ids[t // tokens_per_page]
        pages[page, 0, :, t % tokens_per_page] = k[t]
        pages[page, 1, :, t % tokens_per_page] = v[t]
    return pages.reshape(-1)


@pytest.mark.parametrize("ids_per_block", [1, 2, 4])
def test_gather_and_write_agree_with_an_independent_packer(oracle, ids_per_block):
    rng = np.random.default_rng(8 + ids_per_block)
    hkv, d, p, ctx, layers, slots = 2, 8, 4, 37, 2, 3
    blocks = -(-(-(-ctx // p)) // ids_per_block)
    layout = (slots, layers, blocks, ids_per_block)
    num_pages = 40
    k = rng.normal(size=(ctx, hkv, d)).astype(np.float32)
    v = rng.normal(size=(ctx, hkv, d)).astype(np.float32)
    ids = rng.permutation(num_pages)[: blocks * ids_per_block].astype(np.uint32)
    table = np.zeros(slots * layers * blocks * ids_per_block, np.uint32)
    slot, layer = 2, 1
    base = ((slot * layers + layer) * blocks) * ids_per_block
    table[base:base + len(ids)] = ids
    expected = pack_pages(k, v, ids, p, num_pages)
    page_bytes = 2 * hkv * p * d * 4
    gk, gv = oracle.gather_context(expected, table, slot, layer, ctx, layout, hkv, d, page_bytes, oracle.F32)
    assert np.array_equal(gk, k.reshape(-1)) and np.array_equal(gv, v.reshape(-1))
    pages = np.zeros_like(expected)
    oracle.kv_page_write(pages, k.reshape(-1), v.reshape(-1), [slot] * ctx, list(range(ctx)), table, ctx, layer,
                         layout, hkv, d, page_bytes, oracle.F32)
    assert np.array_equal(pages, expected)


def test_paged_attention_ignores_where_pages_live(oracle):
    rng = np.random.default_rng(11)
    hq, hkv, d, p = 4, 2, 16, 4
    ctxs, layers = [19, 5, 33], 1
    blocks = max(-(-c // p) for c in ctxs)
    layout = (len(ctxs), layers, blocks, 1)
    num_pages = 64
    page_bytes = 2 * hkv * p * d * 2
    ks = [oracle.to_f32(oracle.from_f32(rng.normal(size=(c, hkv, d)), oracle.BF16), oracle.BF16) for c in ctxs]
    vs = [oracle.to_f32(oracle.from_f32(rng.normal(size=(c, hkv, d)), oracle.BF16), oracle.BF16) for c in ctxs]
    q = oracle.from_f32(rng.normal(size=(len(ctxs), hq, d)), oracle.BF16)
    outs = []
    for trial in range(2):
        perm = rng.permutation(num_pages).astype(np.uint32)
        table = np.zeros(len(ctxs) * blocks, np.uint32)
        pages = np.zeros(num_pages * page_bytes // 2, np.uint16)
        cursor = 0
        for r, c in enumerate(ctxs):
            n = -(-c // p)
            ids = perm[cursor:cursor + n]
            cursor += n
            table[r * blocks:r * blocks + n] = ids
            packed = pack_pages(oracle.from_f32(ks[r], oracle.BF16).reshape(c, hkv, d),
                                oracle.from_f32(vs[r], oracle.BF16).reshape(c, hkv, d), ids, p, num_pages)
            pages = np.where(packed != 0, packed, pages)
        outs.append(oracle.paged_gqa(hq, hkv, d, 0.25, page_bytes, oracle.BF16, layout, 0, [0, 1, 2],
                                     [c - 1 for c in ctxs], [0, 1, 2, 3], q, pages, table))
    assert np.array_equal(outs[0], outs[1])
    dense = oracle.projected_gqa_reference(hq, hkv, d, 0.25, [0, 1, 2, 3], [c - 1 for c in ctxs],
                                           oracle.to_f32(q, oracle.BF16), ks, vs)
    assert np.array_equal(outs[0], dense)
