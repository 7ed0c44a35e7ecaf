"""Selected state gathered on the device and restored: the payload is the concatenation of the selected entries'
bytes (numpy slicing of the same buffer is the expected value), a restore touches nothing outside the selection,
and a snapshot of the KV cache taken after one decode step lets a fresh arena and page table reproduce the next
step bit for bit."""
import importlib

import numpy as np
import pytest

from parity_util import importlib_workloads

pytestmark = pytest.mark.gpu


def _expected(host_bytes, ranges, entry_bytes):
    parts = [host_bytes[b * entry_bytes:e * entry_bytes] for b, e in ranges]
    return np.concatenate(parts) if parts else np.zeros(0, np.uint8)


@pytest.mark.parametrize("entry_bytes,offset", [(32768, 0), (4096, 0), (24, 0), (4, 4), (6, 0), (7, 1)])
def test_pack_equals_slicing_and_unpack_restores(psi, device, entry_bytes, offset):
    import torch

    snap = importlib.import_module(psi.__name__ + ".state_snapshot")
    rng = np.random.default_rng(entry_bytes)
    entries = 700
    host = rng.integers(0, 256, size=entries * entry_bytes + 16, dtype=np.uint8)
    backing = device.from_numpy(host)
    buf = backing[offset:offset + entries * entry_bytes]  # the narrow units are used when the base is not 16-aligned
    view = host[offset:offset + entries * entry_bytes]
    # 300 ranges (more than one launch's worth), of very different lengths
    cuts = np.sort(rng.choice(np.arange(1, entries), size=599, replace=False))
    ranges = [(int(cuts[i]), int(cuts[i + 1])) for i in range(0, 598, 2)]
    ranges = [(b, e) for b, e in ranges if e > b]
    ranges = [r for i, r in enumerate(ranges) if i == 0 or ranges[i - 1][1] < r[0]]
    assert len(ranges) > 128
    payload = snap.pack_selected(device, buf, ranges, entry_bytes)
    device.sync()
    want = _expected(view, ranges, entry_bytes)
    assert np.array_equal(payload.cpu().numpy(), want)

    fresh_host = rng.integers(0, 256, size=host.size, dtype=np.uint8)
    fresh_backing = device.from_numpy(fresh_host)
    fresh = fresh_backing[offset:offset + entries * entry_bytes]
    snap.unpack_selected(device, fresh, ranges, entry_bytes, payload)
    device.sync()
    got = fresh_backing.cpu().numpy()
    exp = fresh_host.copy()
    for b, e in ranges:
        exp[offset + b * entry_bytes:offset + e * entry_bytes] = view[b * entry_bytes:e * entry_bytes]
    assert np.array_equal(got, exp)  # selected entries restored, every other byte (and the guard bytes) kept


def test_one_long_range_and_the_empty_selection(psi, device):
    snap = importlib.import_module(psi.__name__ + ".state_snapshot")
    rng = np.random.default_rng(5)
    host = rng.integers(0, 256, size=96 << 20, dtype=np.uint8)  # 3072 pages of 32 KiB
    buf = device.from_numpy(host)
    payload = snap.pack_selected(device, buf, [(1, 3071)], 32768)
    device.sync()
    assert np.array_equal(payload.cpu().numpy(), host[32768:3071 * 32768])
    empty = snap.pack_selected(device, buf, [], 32768)
    assert empty.numel() == 0
    snap.unpack_selected(device, buf, [], 32768, empty)
    with pytest.raises(psi.PsiHipError, match="file length mismatch: expected=65536 actual=32768"):
        snap.unpack_selected(device, buf, [(4, 6)], 32768, payload[:32768])
    with pytest.raises(psi.PsiHipError, match="out of bounds"):
        snap.pack_selected(device, buf, [(3000, 3073)], 32768)


def test_snapshot_of_selected_requests_resumes_decoding(psi, oracle, device):
    """Two of five requests survive a stop: their pages (as page-ID ranges) and page-table rows are written out,
    read back into a zeroed arena and table, and the next decode step of those requests equals the step on the
    original state bit for bit."""
    import torch

    snap = importlib.import_module(psi.__name__ + ".state_snapshot")
    wl = importlib_workloads(psi)
    w = wl.make_workload(151, [700, 33, 1500, 512, 64], 24, 4, 256, psi.Dtype.Bfloat16, 16)
    dw = wl.DeviceWorkload(device, w, partition_tokens=512)
    dw.step()
    device.sync()
    base_out = dw.output.clone()
    keep = [0, 2]  # requests that survive
    layout = w.layout
    row = layout.num_gqa_layers * layout.num_blocks * layout.num_page_ids_per_block
    table_host = w.page_ids.reshape(layout.num_req_slots, row)
    slots = sorted(int(w.req_slots[r]) for r in keep)
    pages_needed = sorted({int(p) for r in keep
                           for p in table_host[int(w.req_slots[r])][:-(-int(w.context_lens[r]) // 16)]})

    def canonical(ids):
        out = []
        for i in ids:
            if out and out[-1][1] == i:
                out[-1][1] = i + 1
            else:
                out.append([i, i + 1])
        return [tuple(r) for r in out]

    page_ranges, slot_ranges = canonical(pages_needed), canonical(slots)
    table = psi.GQARequestPageTable(device, layout)
    table.page_ids.copy_(dw.page_ids.view(torch.int32))
    arena_bytes = snap.PageArenaState(device, dw.pages, w.page_bytes).write_selected_state(page_ranges)
    table_bytes = snap.RequestPageTableState(table).write_selected_state(slot_ranges)
    assert arena_bytes.size == len(pages_needed) * w.page_bytes and table_bytes.size == len(slots) * row * 4

    # a fresh process: zeroed arena and table, then the restore
    new_pages = torch.zeros_like(dw.pages)
    new_table = psi.GQARequestPageTable(device, layout)
    snap.PageArenaState(device, new_pages, w.page_bytes).read_selected_state(page_ranges, arena_bytes)
    snap.RequestPageTableState(new_table).read_selected_state(slot_ranges, table_bytes)
    device.sync()
    got_table = new_table.page_ids.cpu().numpy().view(np.uint32).reshape(layout.num_req_slots, row)
    for s in range(layout.num_req_slots):
        assert np.array_equal(got_table[s], table_host[s] if s in slots else np.zeros(row, np.uint32))

    # attention of the surviving requests over the restored state (the append already happened before the stop)
    dw.pages, dw.page_ids = new_pages, new_table.page_ids
    dw.output.zero_()
    dw.map()
    dw.reduce()
    device.sync()
    width = w.num_q_heads * w.head_dim
    for r in keep:
        assert torch.equal(dw.output[r * width:(r + 1) * width].view(torch.int16),
                           base_out[r * width:(r + 1) * width].view(torch.int16)), f"request {r}"
