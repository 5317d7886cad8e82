"""The decode entry point that allocates nothing (``areno_hip_paged_decode_static``: split-KV partials in a buffer
built into the library) against ``areno_hip_paged_decode`` with a caller workspace, through the C ABI: outputs and
the appended cache rows must be bit-identical (same kernels, same layout of the partials), on two calls in a row of
which the second is the smaller one, so that whatever the first call left in the shared buffer is still there."""

import pytest
import torch

from areno_amd import workloads
from areno_amd.accel import cabi
from tests.gpu_util import DEV, assert_close, expected_decode, gpu_quantize, tolerances

pytestmark = pytest.mark.gpu


def _pools(w):
    return tuple(t for t in (w.k_cache, w.v_cache, w.k_scale, w.v_scale) if t is not None)


def _both_ways(w, **kw):
    """Run the workload through both entry points from the same starting cache; returns (static out, workspace out)."""
    start = tuple(t.clone() for t in _pools(w))
    b, hq, _, d, bs = w.shape
    cache = cabi.describe_cache(w.k_cache, w.v_cache, w.k_scale, w.v_scale)
    out_static = torch.full_like(w.q, float("nan"))
    rc = cabi.paged_decode_static(cache, w.q, w.k_update, w.v_update, out_static, w.block_table, w.cache_seqlens,
                                  softmax_scale=w.softmax_scale, **kw)  # fmt: skip
    cabi.check(rc, "areno_hip_paged_decode_static")
    torch.cuda.synchronize()
    after_static = tuple(t.clone() for t in _pools(w))
    for dst, src in zip(_pools(w), start):
        dst.copy_(src)
    workspace = torch.empty(cabi.decode_workspace_bytes(b, hq, d, bs, w.block_table.shape[1]), dtype=torch.uint8, device=DEV)
    out_ws = torch.full_like(w.q, float("nan"))
    cabi.paged_decode(cache, w.q, w.k_update, w.v_update, out_ws, w.block_table, w.cache_seqlens, workspace,
                      softmax_scale=w.softmax_scale, **kw)  # fmt: skip
    torch.cuda.synchronize()
    for a, b_ in zip(after_static, _pools(w)):
        assert torch.equal(a.view(torch.uint8), b_.view(torch.uint8)), "the appended rows differ between the entry points"
    return out_static, out_ws


def test_static_scratch_decode_matches_the_workspace_entry_point_twice_in_a_row():
    big = workloads.cfg2_qwen7b_int8(device=DEV, quantize_fn=gpu_quantize)  # 64 rows, contexts to 4096, 16 MB of partials
    got, want = _both_ways(big)
    assert torch.equal(got, want), "first call (64 rows, int8 pages)"
    assert_close(got, expected_decode(big), *tolerances("int8"), what="static entry point, cfg 2, vs oracle")
    small = workloads.cfg0_tiny("bf16", device=DEV)  # 4 rows, contexts to 300: reuses the front of the same buffer
    got, want = _both_ways(small)
    assert torch.equal(got, want), "second, smaller call (4 rows, bf16 pages)"
    assert_close(got, expected_decode(small), *tolerances("bf16"), what="static entry point, cfg 0, vs oracle")
    # once more with a window and fp8 pages on the dirty buffer
    third = workloads.cfg0_tiny("fp8", device=DEV, quantize_fn=gpu_quantize)
    got, want = _both_ways(third, window_left=40)
    assert torch.equal(got, want), "third call (window, fp8 pages)"
    assert_close(got, expected_decode(third, window_left=40), *tolerances("fp8"), what="static entry point, window")


def test_static_scratch_decode_refuses_shapes_beyond_its_buffer():
    capacity = int(cabi.lib().areno_hip_paged_decode_static_capacity())
    assert capacity == 64 << 20
    w = workloads.cfg0_tiny("bf16", device=DEV)
    cache = cabi.describe_cache(w.k_cache, w.v_cache)
    # 1024 rows x 64 q heads x 64 dims: (1024 + 1024) slots x 64 heads x 66 floats = 35 MB fits ...
    assert cabi.decode_workspace_bytes(1024, 64, 64, 16, 32) <= capacity
    # ... the same with 128 q heads does not; the check comes before any launch, so the pointers are never used
    assert cabi.decode_workspace_bytes(1024, 128, 64, 16, 32) > capacity
    q = torch.zeros(1024, 128, 64, dtype=torch.bfloat16, device=DEV)
    table = torch.zeros(1024, 32, dtype=torch.int32, device=DEV)
    lens = torch.zeros(1024, dtype=torch.int32, device=DEV)
    before = w.k_cache.clone()
    rc = cabi.paged_decode_static(cache, q, None, None, torch.empty_like(q), table, lens)
    assert rc == cabi.ERR_WORKSPACE
    message = cabi.lib().areno_hip_last_error().decode()
    assert "built-in buffer holds 67108864" in message and "areno_hip_paged_decode" in message
    torch.cuda.synchronize()
    assert torch.equal(before, w.k_cache)


def test_static_scratch_decode_allocates_nothing_and_replays_from_a_graph():
    """What the entry point exists for: no device memory is allocated by a call (free bytes unchanged), and it can be
    recorded into a HIP graph; every replay must give the eager result."""
    w = workloads.cfg0_tiny("int8", device=DEV, quantize_fn=gpu_quantize)
    cache = cabi.describe_cache(w.k_cache, w.v_cache, w.k_scale, w.v_scale)
    out = torch.empty_like(w.q)

    def call(stream=None):
        return cabi.paged_decode_static(cache, w.q, w.k_update, w.v_update, out, w.block_table, w.cache_seqlens,
                                        softmax_scale=w.softmax_scale, stream=stream)  # fmt: skip

    cabi.check(call(), "warm call")  # the first call on a device looks the buffer's address up
    torch.cuda.synchronize()
    eager = out.clone()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        cabi.check(call(), "static call")
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "a static call changed the device's free memory"
    assert torch.equal(out, eager)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        cabi.check(call(torch.cuda.current_stream().cuda_stream), "static call under capture")
    for replay in range(3):
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {replay} differs from the eager call"
        cabi.check(call(), "eager call between replays")  # the program's own work between the replays
        torch.cuda.synchronize()
