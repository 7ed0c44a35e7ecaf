"""Full-size workloads, checked through properties that do not need the scalar oracle to finish:
  * split-count invariance: any partition of [0, ctx) gives the same attention output;
  * page-placement invariance: moving pages in the arena and rewriting the table changes nothing,
    bit for bit;
  * a sampled oracle check: a few requests of the full batch recomputed on the CPU.
Plus the long-context / large-magnitude-K case at a length the oracle still covers."""
import numpy as np
import pytest

from parity_util import (assert_appended_lines, assert_outputs_close, importlib_workloads, layout_tuple, oracle_dtype,
                         oracle_sample, run_and_check)

pytestmark = pytest.mark.gpu


def _full_c2(psi, device, partition, f32_output=True, seed=2, **how):
    wl = importlib_workloads(psi)
    w = wl.config_c2(seed=seed, batch=32, host_pages=False)
    return wl, w, wl.DeviceWorkload(device, w, partition_tokens=partition, f32_output=f32_output, **how)


def test_c2_full_batch_split_count_invariance(psi, device):
    """Batch 32, contexts 1024..8192 (592 MB of K/V): 512-, 2048-token partitions and one split per
    token must agree to f32 rounding."""
    outs = []
    for partition in (512, 2048, 1 << 20):
        _, w, dw = _full_c2(psi, device, partition)
        dw.step()
        outs.append(dw.output_f32())
        del dw
    assert np.isfinite(outs[0]).all()
    scale = np.sqrt((outs[2] ** 2).mean())
    assert np.abs(outs[0] - outs[2]).max() < 2e-5 and np.abs(outs[1] - outs[2]).max() < 2e-5
    assert np.sqrt(((outs[0] - outs[2]) ** 2).mean()) / scale < 1e-5


def test_c2_full_batch_page_placement_invariance(psi, device):
    import torch

    wl, w, dw = _full_c2(psi, device, 512, f32_output=False)
    dw.step()
    base = dw.output.clone()
    # move every page: new arena[perm[i]] = old arena[i], table entries follow
    page_elems = 2 * w.num_kv_heads * w.tokens_per_page * w.head_dim
    gen = torch.Generator(device="cpu")
    gen.manual_seed(5)
    perm = torch.randperm(w.num_pages, generator=gen).to(device.torch_device)
    moved = torch.empty_like(dw.pages)
    moved.view(w.num_pages, page_elems)[perm] = dw.pages.view(w.num_pages, page_elems)
    dw.pages = moved
    dw.page_ids = perm[dw.page_ids.long()].to(torch.int32)
    dw.output.zero_()
    dw.map()
    dw.reduce()
    device.sync()
    assert torch.equal(dw.output.view(torch.int16), base.view(torch.int16))


@pytest.mark.parametrize("how", [{}, {"balanced": True, "fused_append": True}], ids=["row per workgroup", "bench default"])
def test_c2_full_batch_sampled_against_oracle(psi, oracle, device, how):
    """Three of the 32 requests (shortest, median, longest context) recomputed by the scalar oracle
    from the device's own pages.  `bench default`: the balanced worker plan with the append folded into the
    map launch, as `bench.py` runs the step."""
    wl, w, dw = _full_c2(psi, device, 512, **how)
    dw.step()
    if how:
        plain = _full_c2(psi, device, 512)[2]
        plain.step()
        assert np.abs(plain.output_f32() - dw.output_f32()).max() < 2e-5
        assert np.array_equal(plain.pages_host(), dw.pages_host())
        assert dw.shape.num_sdpa_map_task_templates <= dw.meta.num_workers + 32
        del plain
    got = dw.output_f32().reshape(32, w.num_q_heads * w.head_dim)
    pages = dw.pages_host()
    order = np.argsort(w.context_lens)
    picks = [int(order[0]), int(order[16]), int(order[-1])]
    dt = oracle_dtype(oracle, w)
    exp = oracle.paged_gqa(w.num_q_heads, w.num_kv_heads, w.head_dim, w.scale, w.page_bytes, dt, layout_tuple(w),
                           w.layer, w.req_slots[picks], w.token_indices[picks], np.arange(4, dtype=np.uint32),
                           w.q.reshape(32, -1)[picks].reshape(-1), pages, w.page_ids, num_threads=16)
    assert_outputs_close(got[picks].reshape(-1), exp, "C2 sampled")


def test_long_context_with_large_keys(psi, oracle, device):
    """C3's geometry (16 Q / 2 KV, D=256, bf16) with K outliers of 8 sigma at rate 1e-4, partitions
    from 4096 down to 256 tokens, at 16384 tokens per sequence (the oracle's reach)."""
    wl = importlib_workloads(psi)
    w = wl.make_workload(3, [16384, 16384], 16, 2, 256, psi.Dtype.Bfloat16, 16, outlier_rate=1e-4, outlier_sigma=8.0)
    first = None
    for partition in (4096, 512, 256):
        stats, dw = run_and_check(psi, oracle, device, w, f"long ctx partition {partition}",
                                  partition_tokens=partition, check_rounded=False)
        out = dw.output_f32()
        if first is None:
            first = out
        assert np.abs(out - first).max() < 2e-5


# How `bench.py` launches a decode step (balanced worker plan, append inside the map launch) and a verify step
# (balanced worker plan), next to the plain launch (one workgroup per plan row, separate append).
DECODE_MODES = [pytest.param({}, id="row per workgroup"),
                pytest.param({"balanced": True, "longest_first": True, "fused_append": True}, id="bench default")]
VERIFY_MODES = [pytest.param({}, id="row per workgroup"), pytest.param({"balanced": True}, id="bench default")]


def _sampled_check(oracle, dw, picks, what):
    """Oracle on the picked requests from the device's own pages; appended K/V lines bit-exact for every token."""
    exp, rows = oracle_sample(oracle, dw, picks)
    got = dw.output_f32().reshape(dw.w.num_tokens, -1)[rows]
    stats = assert_outputs_close(got.reshape(-1), exp.reshape(-1), what)
    assert_appended_lines(dw)
    return stats


@pytest.mark.parametrize("how", DECODE_MODES)
def test_c3_full_length_with_outliers(psi, oracle, device, how):
    """4 x 131072 tokens (1.07 GB of K/V), 16 Q / 2 KV heads, K outliers of 8 sigma at rate 1e-4 across the whole
    arena: 32 vs 256 partitions per sequence agree to f32 rounding, and one whole sequence (all 16 heads over
    131072 keys) matches the scalar oracle run on the device's pages."""
    import torch

    wl = importlib_workloads(psi)
    w = wl.make_workload(33, [131072] * 4, 16, 2, 256, psi.Dtype.Bfloat16, 16, host_pages=False, outlier_rate=1e-4,
                         outlier_sigma=8.0)
    outs = []
    for partition in (4096, 512):
        dw = wl.DeviceWorkload(device, w, partition_tokens=partition, f32_output=True, **how)
        dw.step()
        outs.append(dw.output_f32())
        if partition == 512:
            k_half = dw.pages.view(w.num_pages, 2, -1)[:256, 0].float().abs()
            rate = float((k_half >= 7.9).float().mean())
            assert 0.5e-4 < rate < 2e-4, f"outlier rate {rate:.2e}"
            _sampled_check(oracle, dw, [2], "C3 sampled sequence")
        del dw
    assert np.isfinite(outs[0]).all()
    assert np.abs(outs[0] - outs[1]).max() < 2e-5


@pytest.mark.parametrize("q_len", [2, 4])
@pytest.mark.parametrize("how", VERIFY_MODES)
def test_c4_verify_full_batch(psi, oracle, device, how, q_len):
    """C4's batch (64 sequences, contexts 2048..16384, 24 Q / 4 KV heads) with one and with three drafts per
    sequence, causal among the new tokens: 512- and 4096-token partitions agree to f32 rounding, the shortest,
    median and longest sequence match the scalar oracle, every appended line is in its page slot."""
    wl = importlib_workloads(psi)
    ctx = wl.config_c2_context_lens(4, 64, 2048, 16384) + q_len
    w = wl.make_workload(4, ctx, 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=q_len, host_pages=False)
    outs = []
    for partition in (512, 4096):
        dw = wl.DeviceWorkload(device, w, partition_tokens=partition, f32_output=True, **how)
        assert dw.variant.is_tiled() and dw.balanced == bool(how)
        dw.step()
        outs.append(dw.output_f32())
        if partition == 512:
            order = np.argsort(w.context_lens)
            _sampled_check(oracle, dw, [int(order[0]), int(order[32]), int(order[-1])], f"C4 q_len {q_len} sampled")
        del dw
    assert np.isfinite(outs[0]).all()
    assert np.abs(outs[0] - outs[1]).max() < 2e-5


@pytest.mark.parametrize("hq", [32, 28])
def test_c4_verify_with_eight_tokens_and_64_columns_through_row_groups(psi, oracle, device, hq):
    """C4's batch with 8 (and 7) heads per KV head and eight new tokens per sequence: 64 (56) query columns per tile.
    The row-group map with the planned partition (tables written narrow: a work item serves all the heads of its KV
    head), the same with 512-token partitions and the plain multi-query map agree to f32 rounding; the shortest,
    median and longest sequence match the scalar oracle, every appended line is in its page slot."""
    wl = importlib_workloads(psi)
    ctx = wl.config_c2_context_lens(4, 64, 2048, 16384) + 8
    w = wl.make_workload(4, ctx, hq, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=8, host_pages=False)
    variant = psi.GQASplitKVVariant.TiledQ(8, 16, hq // 4)
    outs = {}
    for name, partition, grouped in (("planned", "auto", True), ("grouped 512", 512, True), ("plain 512", 512, False)):
        dw = wl.DeviceWorkload(device, w, partition_tokens=partition, f32_output=True, grouped=grouped, variant=variant)
        assert (dw.meta.num_row_groups > 0) == grouped
        if grouped:
            assert dw.meta.group_tiles == 4  # 4 tiles x 8 tokens x 8 heads = 256 columns: no head subsets
        dw.step()
        outs[name] = dw.output_f32()
        if name == "planned":
            assert dw.partition_tokens >= 2048
            order = np.argsort(w.context_lens)
            _sampled_check(oracle, dw, [int(order[0]), int(order[32]), int(order[-1])], f"C4 q_len 8, {hq} heads, sampled")
        del dw
    assert np.isfinite(outs["planned"]).all()
    assert np.abs(outs["planned"] - outs["grouped 512"]).max() < 1e-4
    assert np.abs(outs["planned"] - outs["plain 512"]).max() < 1e-4


def test_c5_prefill_chunk_full_size(psi, oracle, device):
    """C5's chunk: 2048 new tokens on a 4096-token prefix, 24 Q / 4 KV heads.  The row-group map and
    the plain multi-query map agree to rounding on the whole chunk, partition lengths do not matter,
    and sampled query tokens (first, a partition boundary, middle, last) match the scalar oracle run
    on the device's own pages."""
    wl = importlib_workloads(psi)
    w = wl.make_workload(5, [4096 + 2048], 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=2048, host_pages=False)
    variant = psi.GQASplitKVVariant.TiledQ(8, 16, 6)
    outs = {}
    for name, partition, grouped in (("grouped 2048", 2048, True), ("grouped 512", 512, True), ("plain 2048", 2048, False)):
        dw = wl.DeviceWorkload(device, w, partition_tokens=partition, f32_output=True, grouped=grouped, variant=variant)
        assert (dw.meta.num_row_groups > 0) == grouped
        dw.step()
        outs[name] = dw.output_f32().reshape(2048, -1)
        if name == "grouped 2048":
            pages = dw.pages_host()
        del dw
    assert np.isfinite(outs["grouped 2048"]).all()
    assert np.abs(outs["grouped 2048"] - outs["grouped 512"]).max() < 1e-4
    assert np.abs(outs["grouped 2048"] - outs["plain 2048"]).max() < 1e-4
    picks = np.array([0, 1, 511, 512, 1023, 2040, 2047])
    dt = oracle_dtype(oracle, w)
    exp = oracle.paged_gqa(w.num_q_heads, w.num_kv_heads, w.head_dim, w.scale, w.page_bytes, dt, layout_tuple(w),
                           w.layer, np.repeat(w.req_slots, len(picks)), (w.token_indices[0] + picks).astype(np.uint32),
                           np.arange(len(picks) + 1, dtype=np.uint32), w.q.reshape(2048, -1)[picks].reshape(-1), pages,
                           w.page_ids, num_threads=16)
    assert_outputs_close(outs["grouped 2048"][picks].reshape(-1), exp, "C5 chunk sampled")


def test_prefill_chunk_full_size_on_the_reference_geometry(psi, oracle, device):
    """The same chunk on the geometry of the reference's published figures and TiledQ profile (128, 8)
    (gqa_split_kv_tiled_q.rs:66-76): 40 Q / 8 KV heads of 128, 8-token pages.  Row-group map against the plain
    multi-query map on the whole chunk, and sampled query tokens against the scalar oracle."""
    wl = importlib_workloads(psi)
    w = wl.make_workload(5, [4096 + 2048], 40, 8, 128, psi.Dtype.Bfloat16, 8, q_lens=2048, host_pages=False)
    variant = psi.GQASplitKVVariant.TiledQ(8, 16, 5)
    outs = {}
    for name, partition, grouped in (("grouped 4096", 4096, True), ("plain 2048", 2048, False)):
        dw = wl.DeviceWorkload(device, w, partition_tokens=partition, f32_output=True, grouped=grouped, variant=variant)
        assert (dw.meta.num_row_groups > 0) == grouped
        dw.step()
        outs[name] = dw.output_f32().reshape(2048, -1)
        if grouped:
            pages = dw.pages_host()
        del dw
    assert np.isfinite(outs["grouped 4096"]).all()
    assert np.abs(outs["grouped 4096"] - outs["plain 2048"]).max() < 1e-4
    picks = np.array([0, 1, 47, 48, 1023, 2040, 2047])
    dt = oracle_dtype(oracle, w)
    exp = oracle.paged_gqa(w.num_q_heads, w.num_kv_heads, w.head_dim, w.scale, w.page_bytes, dt, layout_tuple(w),
                           w.layer, np.repeat(w.req_slots, len(picks)), (w.token_indices[0] + picks).astype(np.uint32),
                           np.arange(len(picks) + 1, dtype=np.uint32), w.q.reshape(2048, -1)[picks].reshape(-1), pages,
                           w.page_ids, num_threads=16)
    assert_outputs_close(outs["grouped 4096"][picks].reshape(-1), exp, "head_dim 128 chunk sampled")


@pytest.mark.parametrize("how", DECODE_MODES)
def test_c5_decode_batch_full_size(psi, oracle, device, how):
    """C5's decode side: 128 sequences with contexts 512..32768 (about 8.7 GB of K/V).  512- and 4096-token
    partitions agree to f32 rounding; the shortest, median and longest sequence match the scalar oracle."""
    wl = importlib_workloads(psi)
    ctx = wl.config_c2_context_lens(55, 128, 512, 32768)
    w = wl.make_workload(55, ctx, 24, 4, 256, psi.Dtype.Bfloat16, 16, host_pages=False)
    outs = []
    for partition in (512, 4096):
        dw = wl.DeviceWorkload(device, w, partition_tokens=partition, f32_output=True, **how)
        dw.step()
        outs.append(dw.output_f32())
        if partition == 512:
            order = np.argsort(w.context_lens)
            _sampled_check(oracle, dw, [int(order[0]), int(order[64]), int(order[-1])], "C5 decode sampled")
        del dw
    assert np.isfinite(outs[0]).all()
    assert np.abs(outs[0] - outs[1]).max() < 2e-5


def test_c5_mixed_step(psi, oracle, device):
    """C5 as one step: a 2048-token prefill chunk on a 4096-token prefix and 128 decode sequences with contexts
    512..32768 over one arena and one page table -- the chunk through the row-group map, the decode tokens
    through the balanced decode map, both appends included.  Sampled against the scalar oracle on the device's
    pages: chunk tokens at the start, at a 512 boundary, in the middle and at the end; the shortest, median and
    longest decode sequence.  Every appended line is in its page slot."""
    wl = importlib_workloads(psi)
    w = wl.config_c5()
    step = wl.MixedStep(device, w, f32_output=True)
    plan = step.mixed_plan
    assert (plan.num_chunk_reqs, plan.num_chunk_tokens) == (1, 2048)
    assert step.chunk_meta.num_row_groups > 0 and step.chunk_meta.split_kv_variant().is_tiled()
    assert step.decode_meta.num_workers > 0 and not step.decode_meta.split_kv_variant().is_tiled()
    step.step()
    got = step.output_f32().reshape(w.num_tokens, -1)
    assert np.isfinite(got).all()
    assert device.take_device_error() == 0
    # decode side: whole requests
    order = 1 + np.argsort(w.context_lens[1:])
    picks = [int(order[0]), int(order[64]), int(order[-1])]
    exp, rows = oracle_sample(oracle, step, picks)
    assert_outputs_close(got[rows].reshape(-1), exp.reshape(-1), "C5 mixed, decode side")
    assert_appended_lines(step)  # both parts' new tokens
    # chunk side: single query tokens of the chunk, each as a one-token request at its own position
    import dataclasses

    tokens = np.array([0, 1, 511, 512, 1023, 2040, 2047])
    probe_w = dataclasses.replace(w, req_slots=np.repeat(w.req_slots[:1], len(tokens)),
                                  token_indices=(w.token_indices[0] + tokens).astype(np.uint32),
                                  cu_tokens=np.arange(len(tokens) + 1, dtype=np.uint32),
                                  q=w.q.reshape(w.num_tokens, -1)[tokens].reshape(-1))

    class _Probe:  # what oracle_sample reads of a device workload
        w, pages, page_ids, device = probe_w, step.pages, step.page_ids, step.device

    exp, _ = oracle_sample(oracle, _Probe, list(range(len(tokens))))
    assert_outputs_close(got[tokens].reshape(-1), exp.reshape(-1), "C5 mixed, chunk side")


def test_c4_batch_accept_rollback_cycle(psi, oracle, host_oracle, device):
    """C4 end to end on its full batch: 64 requests with 2048..16384 cached tokens, the library's allocator and
    token window next to the Python restatement of the reference's (`oracle/host_oracle.py`), three drafts per
    request.  Two verify steps (4 new tokens per request through the multi-query kernels, balanced plan): after
    each, a seeded accept mask commits a prefix of the drafts, so the next step starts at the first rejected
    position and overwrites it.  Checked: every query, block hand-over and token window of the two bookkeepers
    agree at every step, the device page table equals the restatement's table bit for bit after the rollbacks,
    cached lengths advance by 1 + accepted, no page is freed below block granularity, the appended lines are in
    their page slots, and sampled sequences match the scalar oracle on the device's pages (so a step sees the
    accepted history and none of the rejected drafts)."""
    import dataclasses
    import importlib

    import torch
    from test_runtime_blocks import OracleImpl, ProductImpl, public

    wl = importlib_workloads(psi)
    hq, hkv, d, p, spec = 24, 4, 256, 16, 3
    rng = np.random.default_rng(404)
    cached0 = wl.config_c2_context_lens(4, 64, 2048, 16384)
    n_req = len(cached0)
    blocks_per_req = [-(-(int(c) + 2 * (spec + 1) + p) // p) for c in cached0]
    num_pages = sum(blocks_per_req) + 8
    max_blocks = max(blocks_per_req)
    layout = psi.GQAPageTableLayout(n_req, 1, max_blocks, 1)
    table = psi.GQARequestPageTable(device, layout)
    oracle_table = np.zeros(layout.num_page_ids(), np.uint32)
    o, lib = OracleImpl(host_oracle), ProductImpl(psi)
    ao, al = o.allocator(num_pages), lib.allocator(num_pages)
    both = []

    def sync(r, bo, bl):
        so, sl = bo.prepare_blocks(), bl.prepare_blocks()
        assert so == sl, f"request {r}: block hand-over differs"
        for i, ids in enumerate(sl[1][0]):
            table.write_page_ids(r, 0, sl[0] + i, ids, num_cache_pages=num_pages)
            oracle_table[r * max_blocks + so[0] + i] = so[1][0][i][0]

    for r, c in enumerate(cached0):
        prompt = [100000 * r + i for i in range(int(c) + 1)]  # c cached tokens after the prefill + the decode input
        bo, bl = o.blocks(ao, p, 1, 1, prompt), lib.blocks(al, p, 1, 1, prompt)
        while True:
            so, sl = bo.init(), bl.init()
            assert so == sl
            if so >= int(c):
                break
        qo, ql = bo.prepare(int(c)), bl.prepare(int(c))
        assert public(qo) == public(ql) and qo["kind"] == "Prefill" and qo["token_index"] == 0
        sync(r, bo, bl)
        bo.commit_prefill(qo), bl.commit_prefill(ql)
        drafts = [50000 + 10 * r + j for j in range(spec)]
        bo.set_spec(drafts), bl.set_spec(drafts)
        both.append((bo, bl))
    assert (ao.used(), ao.free()) == (al.used(), al.free())

    page_elems = 2 * hkv * p * d
    base = wl.make_workload(44, [32] * 2, hq, hkv, d, psi.Dtype.Bfloat16, p, host_pages=False)  # a template
    pages, accepted_total, used_before = None, 0, al.used()
    for step in range(2):
        queries = []
        for r, (bo, bl) in enumerate(both):
            _, _, _, ready, queued, drafts = bl.state()
            budget = len(ready) + len(queued) + len(drafts)
            while bl.b.ready_token_slots() < budget:
                so, sl = bo.init(), bl.init()
                assert so == sl and so != "ResourceLimitExceeded"
            qo, ql = bo.prepare(budget), bl.prepare(budget)
            assert public(qo) == public(ql)
            assert ql["kind"] == "Decode" and len(ql["tokens"]) == 1 and len(ql["spec_tokens"]) == spec
            sync(r, bo, bl)
            queries.append((qo, ql))
        starts = np.array([ql["token_index"] for _, ql in queries], np.uint32)
        q_len = 1 + spec
        total = n_req * q_len
        w = dataclasses.replace(
            base, layout=layout, num_pages=num_pages, req_slots=np.arange(n_req, dtype=np.uint32),
            token_indices=starts, cu_tokens=(np.arange(n_req + 1) * q_len).astype(np.uint32),
            page_ids=oracle_table.copy(), pages=None, seed=404,
            q=wl.to_storage(rng.standard_normal((total, hq, d), dtype=np.float32), psi.Dtype.Bfloat16).reshape(-1),
            flat_k=wl.to_storage(rng.standard_normal((total, hkv, d), dtype=np.float32), psi.Dtype.Bfloat16).reshape(-1),
            flat_v=wl.to_storage(rng.standard_normal((total, hkv, d), dtype=np.float32), psi.Dtype.Bfloat16).reshape(-1))
        # the device table is the one the library's hand-overs wrote; it must equal the restatement's
        device.sync()
        assert np.array_equal(table.page_ids_buffer().cpu().numpy().view(np.uint32), oracle_table), f"step {step}"
        if pages is None:
            pages = wl.device_pages(device, w)  # random history in every page
        dw = wl.DeviceWorkload(device, w, partition_tokens=512, f32_output=True, balanced=True, pages=pages,
                               page_ids=table.page_ids_buffer())
        assert dw.variant.is_tiled()
        dw.step()
        order = np.argsort(w.context_lens)
        _sampled_check(oracle, dw, [int(order[0]), int(order[31]), int(order[-1])], f"C4 cycle step {step}")
        del dw
        for r, ((bo, bl), (qo, ql)) in enumerate(zip(both, queries)):
            accept = int(rng.integers(0, spec + 1))  # seeded accept mask: a prefix of the drafts
            accepted_total += accept
            before = len(bl.b.cached_tokens())
            sampled = 70000 + 100 * step + r
            new_drafts = [60000 + 100 * step + 10 * r + j for j in range(spec)]
            bo.commit_decode(qo, qo["spec_tokens"][:accept], sampled, new_drafts)
            bl.commit_decode(ql, ql["spec_tokens"][:accept], sampled, new_drafts)
            assert len(bl.b.cached_tokens()) == before + 1 + accept
            if r % 16 == 0:
                assert bo.state() == bl.state()
            assert bo.counts() == bl.counts()
        # rejected drafts free nothing: pages are owned per block, and no block was released
        assert al.used() >= used_before and (ao.used(), ao.free()) == (al.used(), al.free())
    assert 0 < accepted_total < 2 * n_req * spec
    assert o.bitmap(ao) == lib.bitmap(al)
    for bo, bl in both:
        bo.drop(), bl.drop()
    assert (ao.used(), al.used()) == (0, 0)
