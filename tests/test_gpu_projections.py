"""GPU parity of the kernels around the attention (QGKV split, RMSNorm + RoPE, sigmoid gate), alone
and fused into the append / the combine, against the CPU oracle through the C ABI.

Tolerances.  The split and the V lines of the fused append are bit copies.  RMSNorm + RoPE differs from the
oracle in the summation order of the squares and in the sin / cos implementation: f32 outputs within 2e-5
(1e-3 at position 262143, the reference's own bounds), 2-byte outputs within one unit in the last place on at
most 2 % of the elements.  The gate follows the reference's rounding chain; exp implementations may differ in
the last place, which a 2-byte rounding shows on well under 1 % of the elements."""
import math

import numpy as np
import pytest

from parity_util import importlib_workloads, layout_tuple, oracle_dtype, oracle_step

pytestmark = pytest.mark.gpu


def storage(psi, dtype):
    return np.float32 if dtype == psi.Dtype.Float32 else np.uint16


def to_storage(oracle, psi, values, dtype):
    return oracle.from_f32(np.asarray(values, np.float32), int(dtype)) if dtype != psi.Dtype.Float32 else \
        np.asarray(values, np.float32)


def host(t, np_dtype):
    a = t.cpu().numpy()
    return a.view(np_dtype) if a.dtype != np_dtype else a


def ulp_report(oracle, got, exp, dtype_id):
    """(fraction of differing elements, largest difference in units of the last place) for 2-byte storage."""
    diff = got != exp
    if not diff.any():
        return 0.0, 0
    # monotone integer key of the bit patterns
    def key(bits):
        b = bits.astype(np.int32)
        return np.where(b & 0x8000, -(b & 0x7fff), b & 0x7fff)
    return float(diff.mean()), int(np.abs(key(got) - key(exp)).max())


def test_two_token_pipeline_known_answer_with_poisoned_tail(psi, device):
    """crates/inference-executor-metal/src/attn/gqa/backend.rs:883-1027 through the C ABI: split -> Q / K norm +
    rope -> gate on two tokens of (1 Q head, 1 KV head, 2 dims), active counts 1, 2, 1, outputs pre-filled
    with -777; inactive rows keep the fill, active rows match the closed forms to 2e-5."""
    import torch

    rows = np.array([[1.0, 2.0, 0.5, -0.5, 3.0, 4.0, 5.0, 6.0], [2.0, 1.0, -1.0, 1.0, 4.0, 3.0, 6.0, 5.0]], np.float32)
    split = psi.GQAQGKVSplitKernel(device, 1, 1, 2, psi.Dtype.Float32)
    norm = psi.RMSNormRopeKernel(device, psi.RMSNormRopeConfig(1, 2, 2, 1e-6, 1_000_000.0, psi.Dtype.Float32))
    gate = psi.GQAActivationGateKernel(device, 1, 2, psi.Dtype.Float32)
    ones = device.from_numpy(np.array([0x3f80, 0x3f80], np.uint16))

    def norm_rope_2(row, position):
        inv_rms = 1.0 / math.sqrt((row[0] * row[0] + row[1] * row[1]) / 2.0 + 1.0e-6)
        x0, x1 = row[0] * inv_rms, row[1] * inv_rms
        return [x0 * math.cos(position) - x1 * math.sin(position), x0 * math.sin(position) + x1 * math.cos(position)]

    for active in (1, 2, 1):
        values = rows.copy()
        positions = np.array([0, 1], np.uint32)
        if active == 1:
            values[1] = np.nan
            positions[1] = 0xFFFFFFFF
        qgkv = device.from_numpy(values.ravel())
        pos = device.from_numpy(positions)
        bufs = [torch.full((4,), -777.0, dtype=torch.float32, device=device.torch_device) for _ in range(7)]
        q, g, k, v, q_norm, k_norm, gated = bufs
        split.invoke_bucketed(2, qgkv, q, g, k, v, active)
        norm.invoke_bucketed(2, q, ones, pos, q_norm, active)
        norm.invoke_bucketed(2, k, ones, pos, k_norm, active)
        gate.invoke_bucketed(2, q_norm, g, gated, active)
        device.sync()
        n = 2 * active
        exp_q, exp_g = rows[:active, 0:2].ravel(), rows[:active, 2:4].ravel()
        exp_k, exp_v = rows[:active, 4:6].ravel(), rows[:active, 6:8].ravel()
        exp_qn = np.array(sum((norm_rope_2(exp_q[2 * t:2 * t + 2], float(t)) for t in range(active)), []))
        exp_kn = np.array(sum((norm_rope_2(exp_k[2 * t:2 * t + 2], float(t)) for t in range(active)), []))
        exp_gated = exp_qn / (1.0 + np.exp(-exp_g.astype(np.float64)))
        for buf, exp in ((q, exp_q), (g, exp_g), (k, exp_k), (v, exp_v), (q_norm, exp_qn), (k_norm, exp_kn),
                         (gated, exp_gated)):
            got = buf.cpu().numpy()
            assert np.abs(got[:n] - exp).max() <= 2e-5
            assert (got[n:] == -777.0).all()


def test_f32_yarn_long_context_known_answer(psi, device):
    """components/rms_norm_rope.rs:395-470: 128 dims at position 262143 under Yarn, tolerance 1e-3."""
    factor = float(np.float32(1.0) + np.float32(0.1) * np.log(np.float32(32.0)))
    cfg = psi.RMSNormRopeConfig(1, 128, 128, 1e-6, 10_000_000.0, psi.Dtype.Float32,
                                psi.RopeScaling.Yarn(32.0, factor, 32.0, 1.0, 8192, True))
    x = np.array([((i * 37 % 29) - 14.0) / 8.0 for i in range(128)], np.float32)
    w = np.array([0.75 + (i % 11) / 20.0 for i in range(128)], np.float32)
    import torch

    w_t = torch.tensor(w).to(torch.bfloat16)
    w_f = w_t.to(torch.float32).numpy().astype(np.float64)
    out = device.from_numpy(np.zeros(128, np.float32))
    psi.RMSNormRopeKernel(device, cfg).invoke(1, device.from_numpy(x), w_t.to(device.torch_device),
                                              device.from_numpy(np.array([262143], np.uint32)), out)
    device.sync()
    inv_rms = 1.0 / math.sqrt(float((x.astype(np.float64) ** 2).sum()) / 128 + 1e-6)
    exp = np.zeros(128)
    for d in range(64):
        ramp = min(max((d - 14.0) / (29.0 - 14.0), 0.0), 1.0)
        inv_freq = np.float32(np.float32(10_000_000.0) ** np.float32(-(d / 64.0))) * np.float32(1.0 + ramp * (1.0 / 32.0 - 1.0))
        theta = float(np.float32(262143.0) * np.float32(inv_freq))
        first, second = w_f[d] * x[d] * inv_rms, w_f[d + 64] * x[d + 64] * inv_rms
        exp[d] = factor * (first * math.cos(theta) - second * math.sin(theta))
        exp[d + 64] = factor * (first * math.sin(theta) + second * math.cos(theta))
    assert np.abs(out.cpu().numpy() - exp).max() < 1e-3


def test_bf16_norm_rounding_order_known_answer(psi, oracle, device):
    """components/rms_norm_rope.rs:472-517: bf16(w * bf16(x * inv_rms)), bit for bit."""
    x_bits = oracle.from_f32(np.array([0.73046875, -1.171875, 0.43945313, 2.03125], np.float32), oracle.BF16)
    w_bits = oracle.from_f32(np.array([1.296875, 0.8984375, 1.1015625, 0.703125], np.float32), oracle.BF16)
    cfg = psi.RMSNormRopeConfig(1, 4, 2, 1e-6, 1_000_000.0, psi.Dtype.Bfloat16)
    out = device.from_numpy(np.zeros(4, np.uint16))
    psi.RMSNormRopeKernel(device, cfg).invoke(1, device.from_numpy(x_bits), device.from_numpy(w_bits),
                                              device.from_numpy(np.array([0], np.uint32)), out)
    device.sync()
    x, w = oracle.to_f32(x_bits, oracle.BF16), oracle.to_f32(w_bits, oracle.BF16)
    inv_rms = np.float32(1.0) / np.sqrt(np.float32((x * x).sum(dtype=np.float32) / np.float32(4.0) + np.float32(1e-6)))
    normalized = oracle.to_f32(oracle.from_f32(x * inv_rms, oracle.BF16), oracle.BF16)
    exp = oracle.from_f32(w * normalized, oracle.BF16)
    assert host(out, np.uint16).tolist() == exp.tolist()


@pytest.mark.parametrize("dtype_name,heads,head_dim,rope_dim,yarn", [
    ("Bfloat16", 24, 256, 64, False),   # the partial-rotary shape of the gated layers
    ("Bfloat16", 4, 256, 256, True),
    ("Float32", 6, 128, 128, True),
    ("Float16", 3, 96, 32, False),      # head_dim not a multiple of 64
    ("Float32", 2, 40, 8, False),
])
def test_rms_norm_rope_against_oracle(psi, oracle, device, dtype_name, heads, head_dim, rope_dim, yarn):
    dtype = getattr(psi.Dtype, dtype_name)
    rng = np.random.default_rng(11)
    tokens, active = 9, 7
    scaling = psi.RopeScaling.Yarn(8.0, 1.2, 32.0, 1.0, 4096, True) if yarn else psi.RopeScaling()
    cfg = psi.RMSNormRopeConfig(heads, head_dim, rope_dim, 1e-6, 1_000_000.0, dtype, scaling)
    x = to_storage(oracle, psi, rng.normal(0, 2, tokens * heads * head_dim), dtype)
    w = oracle.from_f32(rng.uniform(0.5, 1.5, head_dim).astype(np.float32), oracle.BF16)
    positions = rng.integers(0, 40000, tokens).astype(np.uint32)
    fill = to_storage(oracle, psi, np.full(x.size, -777.0), dtype)
    out = device.from_numpy(fill.copy())
    psi.RMSNormRopeKernel(device, cfg).invoke_bucketed(tokens, device.from_numpy(x), device.from_numpy(w),
                                                      device.from_numpy(positions), out, active)
    device.sync()
    got = host(out, storage(psi, dtype))
    inv, factor, _ = cfg.kernel_parameters()
    exp = oracle.rms_norm_rope(x[:active * heads * head_dim], w, positions[:active], heads, head_dim, rope_dim, 1e-6,
                               inv, factor, int(dtype))
    n = active * heads * head_dim
    assert (got[n:] == fill[n:]).all(), "rows of inactive tokens were written"
    if dtype == psi.Dtype.Float32:
        assert np.abs(got[:n] - exp).max() <= 2e-5
    else:
        frac, ulps = ulp_report(oracle, got[:n], exp, int(dtype))
        assert ulps <= 1 and frac <= 0.02, (frac, ulps)


def test_norm_rope_reads_the_projection_output_in_place(psi, oracle, device):
    """Strided input: the Q rows inside [q_0|g_0|q_1|g_1|...|k|v] give the same result as the split copy."""
    hq, hkv, d, tokens = 6, 2, 128, 5
    rng = np.random.default_rng(12)
    width = 2 * (hq + hkv) * d
    qgkv = oracle.from_f32(rng.normal(0, 1, tokens * width).astype(np.float32), oracle.BF16)
    q, _, _, _ = oracle.qgkv_split(qgkv, tokens, hq, hkv, d, oracle.BF16)
    w = oracle.from_f32(rng.uniform(0.5, 1.5, d).astype(np.float32), oracle.BF16)
    pos = device.from_numpy(np.arange(100, 100 + tokens, dtype=np.uint32))
    kern = psi.RMSNormRopeKernel(device, psi.RMSNormRopeConfig(hq, d, 64, 1e-6, 1e6, psi.Dtype.Bfloat16))
    dense_out = device.from_numpy(np.zeros(tokens * hq * d, np.uint16))
    strided_out = device.from_numpy(np.zeros(tokens * hq * d, np.uint16))
    kern.invoke(tokens, device.from_numpy(q), device.from_numpy(w), pos, dense_out)
    kern.invoke_bucketed(tokens, device.from_numpy(qgkv), device.from_numpy(w), pos, strided_out, tokens,
                         input_token_stride=width, input_head_stride=2 * d)
    device.sync()
    assert host(dense_out, np.uint16).tolist() == host(strided_out, np.uint16).tolist()


@pytest.mark.parametrize("dtype_name,p", [("Bfloat16", 16), ("Float32", 8), ("Float16", 32)])
def test_fused_append_matches_norm_rope_then_page_write(psi, oracle, device, dtype_name, p):
    """K lines of the pages equal RMSNorm + RoPE of the raw K rows at each token's position (oracle), V lines
    are bit copies, every other byte of the arena keeps its content."""
    wl = importlib_workloads(psi)
    dtype = getattr(psi.Dtype, dtype_name)
    w = wl.make_workload(21, [300, 17, 64, 5], 8, 2, 128, dtype, p, q_lens=[3, 1, 2, 5], num_page_ids_per_block=2)
    norm = psi.RMSNormRopeConfig(2, 128, 64, 1e-6, 1_000_000.0, dtype)
    rng = np.random.default_rng(22)
    weight = oracle.from_f32(rng.uniform(0.5, 1.5, 128).astype(np.float32), oracle.BF16)
    dw = wl.DeviceWorkload(device, w)
    before = dw.pages_host().copy()
    write = psi.GQAKVPageWrite(device, psi.GQAKVPageWriteConfig(w.num_kv_heads, w.head_dim, w.page_bytes, dtype))
    m = dw.meta
    write.invoke_norm_rope_bucketed(
        dw.write_shape, psi.GQAKVPageWriteBuffers(dw.pages, dw.flat_k, dw.flat_v, m.d_req_slots,
                                                  m.d_flat_token_indices, dw.page_ids),
        norm, device.from_numpy(weight), dw.shape.num_tokens, w.layer)
    device.sync()
    got = dw.pages_host()
    flat_pos = np.concatenate([w.token_indices[r] + np.arange(n, dtype=np.uint32)
                               for r, n in enumerate(np.diff(w.cu_tokens))]).astype(np.uint32)
    flat_slots = np.repeat(w.req_slots, np.diff(w.cu_tokens))
    inv, factor, _ = norm.kernel_parameters()
    k_normed = oracle.rms_norm_rope(w.flat_k.reshape(-1), weight, flat_pos, 2, 128, 64, 1e-6, inv, factor, int(dtype))
    exp = before.copy()
    oracle.kv_page_write(exp, k_normed, w.flat_v, flat_slots, flat_pos, w.page_ids, w.num_tokens, w.layer,
                         layout_tuple(w), w.num_kv_heads, w.head_dim, w.page_bytes, oracle_dtype(oracle, w))
    got, exp, before = got.reshape(-1), exp.reshape(-1), before.reshape(-1)
    touched = exp.view(np.uint8).reshape(exp.size, -1) != before.view(np.uint8).reshape(before.size, -1)
    untouched = ~touched.any(axis=1)
    assert (got[untouched].view(np.uint8) == before[untouched].view(np.uint8)).all(), "bytes outside the appended lines changed"
    if dtype == psi.Dtype.Float32:
        assert np.abs(got - exp).max() <= 2e-5
    else:
        frac, ulps = ulp_report(oracle, got, exp, int(dtype))
        assert ulps <= 1 and frac <= 0.02 * w.num_tokens * 2 * 128 / got.size + 1e-9, (frac, ulps)
    # the attention that follows sees the same pages as the unfused sequence would produce
    dw.map()
    dw.reduce()


@pytest.mark.parametrize("dtype_name", ["Bfloat16", "Float32", "Float16"])
def test_gate_against_oracle(psi, oracle, device, dtype_name):
    dtype = getattr(psi.Dtype, dtype_name)
    rng = np.random.default_rng(31)
    hq, d, tokens, active = 6, 64, 11, 8
    a = to_storage(oracle, psi, rng.normal(0, 1, tokens * hq * d), dtype)
    g = to_storage(oracle, psi, rng.normal(0, 3, tokens * hq * d), dtype)
    fill = to_storage(oracle, psi, np.full(a.size, -777.0), dtype)
    out = device.from_numpy(fill.copy())
    psi.GQAActivationGateKernel(device, hq, d, dtype).invoke_bucketed(tokens, device.from_numpy(a),
                                                                      device.from_numpy(g), out, active)
    device.sync()
    got = host(out, storage(psi, dtype))
    n = active * hq * d
    exp = oracle.activation_gate(a[:n], g[:n], int(dtype))
    assert (got[n:] == fill[n:]).all()
    if dtype == psi.Dtype.Float32:
        assert np.abs(got[:n] - exp).max() <= 1e-6
    else:
        frac, ulps = ulp_report(oracle, got[:n], exp, int(dtype))
        assert ulps <= 1 and frac <= 0.01, (frac, ulps)


@pytest.mark.parametrize("q_len,in_place", [(1, False), (1, True), (3, False)])
def test_gate_fused_into_the_combine(psi, oracle, device, q_len, in_place):
    """The combine with a gate equals the combine followed by the stand-alone gate kernel, bit for bit (the same
    device functions in the same order), and matches the oracle's attention then gate within the gate's bound.
    `in_place`: the gate is read from inside a [q|g] interleaved projection output through strides."""
    import torch

    wl = importlib_workloads(psi)
    hq, hkv, d = 12, 2, 256
    w = wl.make_workload(41, [700, 33, 260], hq, hkv, d, psi.Dtype.Bfloat16, 16, q_lens=q_len)
    rng = np.random.default_rng(42)
    tokens = w.num_tokens
    gates = oracle.from_f32(rng.normal(0, 2, tokens * hq * d).astype(np.float32), oracle.BF16)
    if in_place:
        width = 2 * (hq + hkv) * d
        qgkv = np.zeros(tokens * width, np.uint16)
        qgkv.reshape(tokens, width)[:, :2 * hq * d].reshape(tokens, hq, 2, d)[:, :, 1, :] = gates.reshape(tokens, hq, d)
        gate = psi.OutputGate(device.from_numpy(qgkv), width, 2 * d, offset=d)
    else:
        gate = psi.OutputGate(device.from_numpy(gates), hq * d, d)
    dw = wl.DeviceWorkload(device, w, partition_tokens=256, longest_first=True)
    dw.step()
    plain = dw.output.clone()
    gated_two_step = torch.zeros_like(plain)
    psi.GQAActivationGateKernel(device, hq, d, psi.Dtype.Bfloat16).invoke_bucketed(
        tokens, plain, device.from_numpy(gates), gated_two_step, tokens)
    m, s = dw.meta, dw.shape
    if dw.variant.is_tiled():
        dw.kernels.invoke_reduce_bucketed(dw.scratch, m.d_q_token_tiles, m.d_cu_kv_splits, dw.output,
                                          s.num_q_token_tiles, partial_row_index=m.d_partial_row_index, gate=gate)
    else:
        dw.kernels.invoke_reduce_bucketed(dw.scratch, m.d_cu_kv_splits, dw.output, s.num_tokens,
                                          partial_row_index=m.d_partial_row_index, gate=gate)
    device.sync()
    fused = host(dw.output.view(torch.int16), np.uint16)
    assert fused.tolist() == host(gated_two_step.view(torch.int16), np.uint16).tolist()
    _, attn = oracle_step(oracle, w)
    exp = oracle.activation_gate(oracle.from_f32(attn.reshape(-1), oracle.BF16), gates, oracle.BF16)
    got_f, exp_f = oracle.to_f32(fused, oracle.BF16), oracle.to_f32(exp, oracle.BF16)
    assert np.abs(got_f - exp_f).max() <= 2e-3 and np.sqrt(((got_f - exp_f) ** 2).sum() / (exp_f ** 2).sum()) <= 6e-3


def test_single_launch_prepare_equals_the_separate_kernels(psi, oracle, device):
    """Q norm + rope and the fused append as one launch, reading the projection output in place:
    the Q buffer and the page arena equal, bit for bit, what the two separate entry points write."""
    import torch

    wl = importlib_workloads(psi)
    hq, hkv, d = 12, 2, 256
    w = wl.make_workload(51, [130, 17, 700], hq, hkv, d, psi.Dtype.Bfloat16, 16, q_lens=[2, 1, 4])
    rng = np.random.default_rng(52)
    tokens, width = w.num_tokens, 2 * (hq + hkv) * d
    qgkv = device.from_numpy(oracle.from_f32(rng.normal(0, 1, tokens * width).astype(np.float32), oracle.BF16))
    wq = device.from_numpy(oracle.from_f32(rng.uniform(0.5, 1.5, d).astype(np.float32), oracle.BF16))
    wk = device.from_numpy(oracle.from_f32(rng.uniform(0.5, 1.5, d).astype(np.float32), oracle.BF16))
    q_norm = psi.RMSNormRopeConfig(hq, d, 64, 1e-6, 1e7, psi.Dtype.Bfloat16)
    k_norm = psi.RMSNormRopeConfig(hkv, d, 64, 2e-6, 1e7, psi.Dtype.Bfloat16)
    results = []
    for single_launch in (False, True):
        dw = wl.DeviceWorkload(device, w)
        m = dw.meta
        q_out = torch.zeros(tokens * hq * d, dtype=torch.int16, device=device.torch_device)
        buffers = psi.GQAKVPageWriteBuffers(dw.pages, qgkv[2 * hq * d:], qgkv[(2 * hq + hkv) * d:], m.d_req_slots,
                                            m.d_flat_token_indices, dw.page_ids)
        if single_launch:
            dw.write.invoke_prepare_bucketed(dw.write_shape, buffers, dw.cfg, q_norm, k_norm, qgkv, wq, q_out, wk,
                                             tokens, w.layer, q_token_stride=width, q_head_stride=2 * d,
                                             k_token_stride=width, v_token_stride=width)
        else:
            psi.RMSNormRopeKernel(device, q_norm).invoke_bucketed(tokens, qgkv, wq, m.d_flat_token_indices, q_out,
                                                                  tokens, input_token_stride=width,
                                                                  input_head_stride=2 * d)
            dw.write.invoke_norm_rope_bucketed(dw.write_shape, buffers, k_norm, wk, tokens, w.layer,
                                               k_token_stride=width, v_token_stride=width)
        device.sync()
        results.append((q_out.cpu().numpy().copy(), dw.pages_host().copy()))
    assert np.array_equal(results[0][0], results[1][0]) and results[0][0].any()
    assert np.array_equal(results[0][1].view(np.uint8), results[1][1].view(np.uint8))
    mismatch = psi.RMSNormRopeConfig(hkv, d, 128, 2e-6, 1e7, psi.Dtype.Bfloat16)
    with pytest.raises(psi.PsiHipError) as err:
        dw.write.invoke_prepare_bucketed(dw.write_shape, buffers, dw.cfg, q_norm, mismatch, qgkv, wq, q_out, wk, tokens,
                                         w.layer, q_token_stride=width, q_head_stride=2 * d, k_token_stride=width,
                                         v_token_stride=width)
    assert "must share rope_dim" in str(err.value)
