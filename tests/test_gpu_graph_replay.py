"""A decode layer-step (append -> map -> combine) captured into a HIP graph and replayed: every
replay, with the program's own eager work and synchronisations in between, must reproduce the
eager result bit for bit on the inputs current at replay time.  The library's launches take their
active counts as kernel arguments and use no memset, so a captured step is self-contained."""
import numpy as np
import pytest

from parity_util import importlib_workloads

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("q_len", [1, 2])
def test_captured_layer_step_replays(psi, device, q_len):
    import torch

    wl = importlib_workloads(psi)
    w = wl.make_workload(101 + q_len, [700, 33, 1500, 512, 64], 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=q_len)
    dw = wl.DeviceWorkload(device, w, partition_tokens=512)
    pristine = dw.pages.clone()

    def eager():
        dw.pages.copy_(pristine)
        dw.step()
        device.sync()
        return dw.output.clone()

    base = eager()
    side = torch.cuda.Stream()
    main = device.stream
    graph = torch.cuda.CUDAGraph()
    try:
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            device.use_stream(side)
            dw.pages.copy_(pristine)
            dw.step()  # warm-up on the capture stream
            side.synchronize()
            with torch.cuda.graph(graph, stream=side):
                dw.step()
    finally:
        device.use_stream(main)
    torch.cuda.synchronize()

    rng = np.random.default_rng(7)
    for replay in range(4):
        # new inputs each time: queries and the new tokens' K/V change, the history is restored
        dw.pages.copy_(pristine)
        if replay:
            for t in (dw.q, dw.flat_k, dw.flat_v):
                t.copy_(device.from_numpy(wl.to_storage(rng.standard_normal(t.numel(), dtype=np.float32),
                                                       w.dtype)))
        expected = eager()
        dw.pages.copy_(pristine)
        dw.output.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(dw.output.view(torch.int16), expected.view(torch.int16)), f"replay {replay}"
        if replay == 0:
            assert torch.equal(dw.output.view(torch.int16), base.view(torch.int16))
        # eager work of the program between replays
        _ = (dw.output.float() * 2).sum().item()
