"""Seeded sweep over shapes and launch modes: every case is one layer-step through the C ABI checked against the
oracle (pages bit-exact, outputs within the tolerance).  The cases mix what the dedicated tests cover one at a
time: head groupings, head_dim 128/256, page sizes, both 2-byte types, ragged batches with one-token and
page-boundary contexts, one or several new tokens per request, and the launch modes (row per workgroup, longest
first, balanced plan, append folded into the map)."""
import numpy as np
import pytest

from parity_util import importlib_workloads, run_and_check

pytestmark = pytest.mark.gpu

HEADS = [(24, 4), (16, 2), (32, 8), (8, 8), (5, 1), (14, 2), (12, 4), (64, 8)]


def _case(seed):
    rng = np.random.default_rng(1000 + seed)
    hq, hkv = HEADS[int(rng.integers(len(HEADS)))]
    d = int(rng.choice([128, 256]))
    p = int(rng.choice([8, 16, 32]))
    dtype_name = str(rng.choice(["Bfloat16", "Float16"]))
    batch = int(rng.integers(1, 10))
    special = [1, 2, p, p + 1, 511, 512, 513, 1024]
    ctx = [int(rng.choice(special)) if rng.random() < 0.4 else int(rng.integers(1, 3000)) for _ in range(batch)]
    tiled = bool(rng.random() < 0.4)
    if tiled:
        q_lens = [int(rng.integers(1, 9)) for _ in range(batch)]
    else:
        q_lens = [int(rng.integers(1, 4)) if rng.random() < 0.3 else 1 for _ in range(batch)]
    ctx = [max(c, q) for c, q in zip(ctx, q_lens)]
    mode = str(rng.choice(["rows", "longest_first", "balanced", "balanced_fused", "fused"]))
    partition = int(rng.choice([256, 512, 1024]))
    return hq, hkv, d, p, dtype_name, ctx, q_lens, tiled, mode, partition


@pytest.mark.parametrize("seed", range(32))
def test_seeded_shape_and_mode(psi, oracle, device, seed):
    hq, hkv, d, p, dtype_name, ctx, q_lens, tiled, mode, partition = _case(seed)
    wl = importlib_workloads(psi)
    dtype = getattr(psi.Dtype, dtype_name)
    w = wl.make_workload(2000 + seed, ctx, hq, hkv, d, dtype, p, q_lens=q_lens)
    group = min(hq // hkv, 8)
    if tiled:
        variant = psi.GQASplitKVVariant.TiledQ(8, 16 if p >= 8 else 4, group)
    else:
        variant = psi.GQASplitKVVariant.SingleQ(256, 256, group)
    how = dict(balanced=mode.startswith("balanced"), longest_first=mode == "longest_first",
               fused_append=mode.endswith("fused") and not tiled)
    what = f"seed {seed}: {dtype_name} {hq}/{hkv}/{d} P={p} ctx={ctx} q={q_lens} {'tiled' if tiled else 'single'} {mode}"
    print(what, flush=True)
    run_and_check(psi, oracle, device, w, what, partition_tokens=partition, variant=variant, max_tokens=128,
                  check_rounded=False, **how)
