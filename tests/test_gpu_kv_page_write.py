"""KV append on the GPU: the reference's known answers and canary cases
(crates/inference-backend-metal/src/components/gqa_kv_page_write.rs:283-364), through the C ABI."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _run(psi, device, dtype, pages_np, k_np, v_np, req_slots, positions, page_ids, layout, hkv, d, page_bytes,
         total, active, layer=0):
    pages = device.from_numpy(pages_np)
    cfg = psi.GQAKVPageWriteConfig(hkv, d, page_bytes, dtype)
    shape = psi.GQAKVPageWriteShape(total, layout)
    kernel = psi.GQAKVPageWrite(device, cfg)
    bufs = psi.GQAKVPageWriteBuffers(pages, device.from_numpy(k_np), device.from_numpy(v_np),
                                     device.from_numpy(np.asarray(req_slots, np.uint32)),
                                     device.from_numpy(np.asarray(positions, np.uint32)),
                                     device.from_numpy(np.asarray(page_ids, np.uint32)))
    kernel.invoke_bucketed(shape, bufs, active, layer)
    device.sync()
    return pages.cpu().numpy()


def test_fixed_u16_and_f32(psi, device):
    layout = psi.GQAPageTableLayout(1, 1, 1, 1)
    out = _run(psi, device, psi.Dtype.Bfloat16, np.zeros(8, np.uint16), np.array([10, 11], np.uint16),
               np.array([20, 21], np.uint16), [0], [1], [0], layout, 1, 2, 16, 1, 1)
    assert out.view(np.uint16).tolist() == [0, 0, 10, 11, 0, 0, 20, 21]
    out = _run(psi, device, psi.Dtype.Float32, np.zeros(8, np.float32), np.array([10, 11], np.float32),
               np.array([20, 21], np.float32), [0], [1], [0], layout, 1, 2, 32, 1, 1)
    assert out.tolist() == [0.0, 0.0, 10.0, 11.0, 0.0, 0.0, 20.0, 21.0]


def test_bucketed_replay_preserves_inactive_kv_page(psi, device):
    sentinel, page_values = 0x7777, 16
    layout = psi.GQAPageTableLayout(2, 1, 1, 1)
    k = np.arange(10, 18, dtype=np.uint16)
    v = np.arange(20, 28, dtype=np.uint16)
    args = dict(req_slots=[0, 0, 0, 1], positions=[0, 1, 2, 0], page_ids=[0, 1], layout=layout, hkv=1, d=2,
                page_bytes=page_values * 2, total=4)
    out = _run(psi, device, psi.Dtype.Bfloat16, np.full(2 * page_values, sentinel, np.uint16), k, v, active=3,
               **args).view(np.uint16)
    assert (out[page_values:] == sentinel).all()
    # page 0 holds 4 tokens of K then 4 of V, D=2
    assert out[:6].tolist() == [10, 11, 12, 13, 14, 15] and out[8:14].tolist() == [20, 21, 22, 23, 24, 25]
    assert out[6:8].tolist() == [sentinel] * 2 and out[14:16].tolist() == [sentinel] * 2
    out = _run(psi, device, psi.Dtype.Bfloat16, np.full(2 * page_values, sentinel, np.uint16), k, v, active=4,
               **args).view(np.uint16)
    assert out[page_values:page_values + 2].tolist() == [16, 17]
    assert out[page_values + 8:page_values + 10].tolist() == [26, 27]


def test_contract_violations_are_reported(psi, device):
    layout = psi.GQAPageTableLayout(1, 1, 1, 1)
    with pytest.raises(psi.PsiHipError, match="exceeds the shader u32 count domain"):
        _run(psi, device, psi.Dtype.Bfloat16, np.zeros(8, np.uint16), np.zeros(2, np.uint16), np.zeros(2, np.uint16),
             [0], [0], [0], layout, 2, 2, 16, 1 << 30, 1)
    with pytest.raises(psi.PsiHipError, match="page-table index exceeds layer count"):
        _run(psi, device, psi.Dtype.Bfloat16, np.zeros(8, np.uint16), np.zeros(2, np.uint16), np.zeros(2, np.uint16),
             [0], [0], [0], layout, 1, 2, 16, 1, 1, layer=1)
    with pytest.raises(psi.PsiHipError, match="divisible by the K/V bytes per token"):
        psi.GQAKVPageWriteConfig(1, 2, 10, psi.Dtype.Bfloat16).num_tokens_per_page()


@pytest.mark.parametrize("dtype_name", ["Bfloat16", "Float16", "Float32"])
def test_random_append_matches_oracle_bit_exact(psi, oracle, device, dtype_name):
    """Multi-layer table, two page IDs per block, several tokens per request, ragged positions."""
    import importlib

    wl = importlib.import_module(psi.__name__ + ".workloads")
    from parity_util import layout_tuple, oracle_dtype

    dtype = getattr(psi.Dtype, dtype_name)
    w = wl.make_workload(23, [40, 7, 65, 16, 3], 8, 4, 128, dtype, 8, q_lens=[4, 1, 3, 2, 3], num_gqa_layers=3,
                         layer=2, num_page_ids_per_block=2)
    dw = wl.DeviceWorkload(device, w)
    dw.append()
    got = dw.pages_host()
    exp = w.pages.copy()
    flat_slots = np.repeat(w.req_slots, np.diff(w.cu_tokens))
    flat_pos = np.concatenate([w.token_indices[r] + np.arange(n, dtype=np.uint32)
                               for r, n in enumerate(np.diff(w.cu_tokens))]).astype(np.uint32)
    oracle.kv_page_write(exp, w.flat_k, w.flat_v, flat_slots, flat_pos, w.page_ids, w.num_tokens, w.layer,
                         layout_tuple(w), w.num_kv_heads, w.head_dim, w.page_bytes, oracle_dtype(oracle, w))
    assert got.tobytes() == exp.tobytes()
    assert got.tobytes() != w.pages.tobytes()
