"""Selected state of the KV cache for a snapshot: page-ID ranges of the page arena and request-slot ranges of
the GQA page table, gathered on the device into one payload and restored from it.

Mirrors `SelectedStateIO` of the reference (crates/inference-executor-metal/src/model/state_snapshot.rs:249-304,
:533-591; model/page_arena/file_io.rs:28-49; attn/gqa/request_page_table/file_io.rs:28-59): the payload is the
concatenation of the selected entries' bytes, ranges are half-open `(begin, end)` pairs in canonical form (non-empty,
sorted, disjoint, not adjacent).  Files, manifest and publishing are the caller's; a payload is handed over as one
pinned host array so that the host link is crossed once."""
import ctypes
from typing import Sequence, Tuple

import numpy as np

from . import _lib as L
from .gqa import Device, GQARequestPageTable, _nbytes, _ptr

Ranges = Sequence[Tuple[int, int]]


def _ranges_array(entry_ranges: Ranges):
    flat = [int(v) for r in entry_ranges for v in r]
    if len(flat) != 2 * len(entry_ranges):
        raise ValueError("entry ranges must be (begin, end) pairs")
    return L.u32_array(flat), len(entry_ranges)


def selected_payload_bytes(entry_ranges: Ranges, entry_bytes: int, buffer_bytes: int) -> int:
    """Size of the payload of a selection; raises `PsiHipError` with the reference's message when the ranges are
    not canonical or leave the buffer."""
    arr, n = _ranges_array(entry_ranges)
    out = ctypes.c_uint64()
    L.check(L.load().psi_hip_selected_ranges_payload_bytes(arr, n, entry_bytes, buffer_bytes, ctypes.byref(out)))
    return out.value


def pack_selected(device: Device, buffer, entry_ranges: Ranges, entry_bytes: int):
    """`write_selected_buffer`: the selected entries of a device tensor as one device payload (uint8 tensor)."""
    import torch

    arr, n = _ranges_array(entry_ranges)
    size = selected_payload_bytes(entry_ranges, entry_bytes, _nbytes(buffer))
    payload = torch.empty(size, dtype=torch.uint8, device=device.torch_device)
    L.check(device.lib.psi_hip_buffer_pack_selected(device.ctx, _ptr(buffer), _nbytes(buffer), arr, n, entry_bytes,
                                                    _ptr(payload) if size else None, size))
    return payload


def unpack_selected(device: Device, buffer, entry_ranges: Ranges, entry_bytes: int, payload) -> None:
    """`read_selected_buffer`: a device payload written back over the selected entries; the rest of the buffer
    keeps its bytes."""
    arr, n = _ranges_array(entry_ranges)
    L.check(device.lib.psi_hip_buffer_unpack_selected(device.ctx, _ptr(buffer), _nbytes(buffer), arr, n, entry_bytes,
                                                      _ptr(payload) if _nbytes(payload) else None, _nbytes(payload)))


def _to_host(device: Device, payload) -> np.ndarray:
    import torch

    device.sync()  # the gather ran on the library's stream, the copy below runs on torch's
    host = torch.empty(payload.numel(), dtype=torch.uint8, pin_memory=payload.numel() > 0)
    host.copy_(payload)
    torch.cuda.current_stream().synchronize()
    return host.numpy()


def _to_device(device: Device, payload_bytes: np.ndarray):
    import torch

    host = torch.from_numpy(np.ascontiguousarray(payload_bytes, dtype=np.uint8))
    on_device = host.to(device.torch_device)
    torch.cuda.current_stream().synchronize()  # the scatter runs on the library's stream
    return on_device


class PageArenaState:
    """`SelectedStateIO for PageArena`: entries are pages, IDs are page IDs."""

    def __init__(self, device: Device, pages, page_bytes: int):
        if page_bytes <= 0 or _nbytes(pages) % page_bytes:
            raise ValueError("the arena must hold whole pages")
        self.device, self.pages, self.page_bytes = device, pages, page_bytes

    def write_selected_state(self, page_id_ranges: Ranges) -> np.ndarray:
        return _to_host(self.device, pack_selected(self.device, self.pages, page_id_ranges, self.page_bytes))

    def read_selected_state(self, page_id_ranges: Ranges, payload_bytes: np.ndarray) -> None:
        unpack_selected(self.device, self.pages, page_id_ranges, self.page_bytes,
                        _to_device(self.device, payload_bytes))


class RequestPageTableState:
    """`SelectedStateIO for GQARequestPageTable`: entries are the rows of request slots."""

    def __init__(self, table: GQARequestPageTable):
        self.device, self.table = table.device, table
        layout = table.layout
        self.entry_bytes = layout.num_gqa_layers * layout.num_blocks * layout.num_page_ids_per_block * 4

    def write_selected_state(self, request_slot_ranges: Ranges) -> np.ndarray:
        return _to_host(self.device, pack_selected(self.device, self.table.page_ids, request_slot_ranges,
                                                   self.entry_bytes))

    def read_selected_state(self, request_slot_ranges: Ranges, payload_bytes: np.ndarray) -> None:
        unpack_selected(self.device, self.table.page_ids, request_slot_ranges, self.entry_bytes,
                        _to_device(self.device, payload_bytes))
