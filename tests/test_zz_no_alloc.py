"""The decode entry point that allocates nothing (`tyr_hip_gqa_decode_static`): called through the
C ABI, twice in a row (the second call on a smaller input, so it finds the first call's partials in
the shared scratch array), each result compared bit for bit with `tyr_hip_gqa_decode` on the same
inputs -- both run the same kernels, so integer equality of the bf16 / f32 patterns is the bar --
and against the CPU checker at the decode tolerance."""
import math

import numpy as np
import pytest
import torch

import oracle
from oracle import libtorch_path as lt
from tests.util import bits, from_bits, max_abs

pytestmark = pytest.mark.gpu
TOL = 2e-2


def _call_pair(L_, q, k, v, splits, kv_len):
    """(o, lse) of the static entry point and of the workspace entry point on the same inputs."""
    B, Hq, _, D = q.shape
    Hkv, Lmax = k.shape[1], k.shape[2]
    sc = 1 / math.sqrt(D)
    stream = torch.cuda.current_stream().cuda_stream
    o_s = torch.full_like(q, float("nan"))
    lse_s = torch.full((B, Hq), float("nan"), device="cuda")
    rc = L_.tyr_hip_gqa_decode_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), o_s.data_ptr(), lse_s.data_ptr(),
                                      B, Hq, Hkv, kv_len, D, Lmax, sc, splits, stream)
    assert rc == 0, L_.tyr_hip_strerror(rc)
    o_w = torch.full_like(q, float("nan"))
    lse_w = torch.full((B, Hq), float("nan"), device="cuda")
    nbytes = L_.tyr_hip_gqa_decode_workspace_bytes(B, Hq, Hkv, kv_len, D, splits)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
    rc = L_.tyr_hip_gqa_decode(q.data_ptr(), k.data_ptr(), v.data_ptr(), o_w.data_ptr(), lse_w.data_ptr(),
                               B, Hq, Hkv, kv_len, D, Lmax, sc, splits, ws.data_ptr(), ws.numel(), stream)
    assert rc == 0, L_.tyr_hip_strerror(rc)
    torch.cuda.synchronize()
    return (o_s, lse_s), (o_w, lse_w)


def test_static_decode_two_calls_match_workspace_entry_point():
    from tyr_amd import _lib
    L_ = _lib.load()
    # first call: 4 sequences, 5 splits of a ragged length; second call: smaller in every extent
    cases = [((4, 32, 8, 1500, 128), 5, 1403), ((2, 8, 2, 300, 128), 3, 300)]
    for i, ((B, Hq, Hkv, Lmax, D), splits, kv_len) in enumerate(cases):
        q, = lt.make_inputs(900 + i, (B, Hq, 1, D))
        k, v = lt.make_inputs(910 + i, (B, Hkv, Lmax, D), (B, Hkv, Lmax, D))
        (o_s, lse_s), (o_w, lse_w) = _call_pair(L_, q.cuda(), k.cuda(), v.cuda(), splits, kv_len)
        assert np.array_equal(bits(o_s), bits(o_w)), f"call {i}: O differs from tyr_hip_gqa_decode"
        assert np.array_equal(lse_s.cpu().numpy().view(np.uint32), lse_w.cpu().numpy().view(np.uint32))
        want_o, want_lse = oracle.gqa_decode(bits(q), bits(k), bits(v), 1 / math.sqrt(D), splits, kv_len=kv_len)
        assert max_abs(o_s.cpu().float(), from_bits(want_o).float()) <= TOL
        assert max_abs(lse_s.cpu(), want_lse) <= 1e-3


def test_static_decode_single_split_and_auto():
    from tyr_amd import _lib
    L_ = _lib.load()
    for i, splits in enumerate((1, 0)):
        B, Hq, Hkv, Lmax, D = 3, 16, 4, 2048, 128
        q, = lt.make_inputs(920 + i, (B, Hq, 1, D))
        k, v = lt.make_inputs(930 + i, (B, Hkv, Lmax, D), (B, Hkv, Lmax, D))
        (o_s, lse_s), (o_w, lse_w) = _call_pair(L_, q.cuda(), k.cuda(), v.cuda(), splits, Lmax)
        assert np.array_equal(bits(o_s), bits(o_w))
        assert np.array_equal(lse_s.cpu().numpy().view(np.uint32), lse_w.cpu().numpy().view(np.uint32))


def test_static_decode_rejects_oversized_request():
    from tyr_amd import _lib
    L_ = _lib.load()
    B, Hq, Hkv, Lmax, D, splits = 64, 64, 8, 64 * 512, 128, 64      # 64*64*64*130*4 B = 136 MB of partials
    assert L_.tyr_hip_gqa_decode_workspace_bytes(B, Hq, Hkv, Lmax, D, splits) > (8 << 20)
    # the size check comes first: the (tiny, wrong-sized) tensors are never touched
    t = torch.zeros(16, dtype=torch.bfloat16, device="cuda")
    rc = L_.tyr_hip_gqa_decode_static(t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), None,
                                      B, Hq, Hkv, Lmax, D, Lmax, 0.1, splits, None)
    assert rc == -5 and b"workspace" in L_.tyr_hip_strerror(rc)


def _free_device_bytes():
    free, _total = torch.cuda.mem_get_info()
    return free


def test_static_decode_allocates_nothing_and_replays_from_a_captured_graph():
    """The entry point takes no memory from the device or from the caching allocator (outputs are the caller's), and --
    after one warm-up call, which resolves the address of the static array -- it can be recorded into a HIP graph: three
    replays with eager work in between, each equal to the eager result of the workspace entry point."""
    from tyr_amd import _lib
    L_ = _lib.load()
    B, Hq, Hkv, Lmax, D, splits = 2, 8, 2, 900, 128, 4
    sc = 1 / math.sqrt(D)
    q, = lt.make_inputs(940, (B, Hq, 1, D))
    k, v = lt.make_inputs(941, (B, Hkv, Lmax, D), (B, Hkv, Lmax, D))
    q, k, v = q.cuda(), k.cuda(), v.cuda()
    (o_s, lse_s), (o_w, lse_w) = _call_pair(L_, q, k, v, splits, Lmax)           # warm-up + reference result
    o = torch.zeros_like(q)
    lse = torch.zeros((B, Hq), device="cuda")
    torch.cuda.synchronize()

    def call(stream):
        rc = L_.tyr_hip_gqa_decode_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(),
                                          B, Hq, Hkv, Lmax, D, Lmax, sc, splits, stream)
        assert rc == 0, L_.tyr_hip_strerror(rc)

    before = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), _free_device_bytes())
    for _ in range(3):
        call(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    after = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), _free_device_bytes())
    assert before == after, (before, after)
    assert torch.equal(o, o_w) and torch.equal(lse, lse_w)

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(torch.cuda.current_stream().cuda_stream)
    for replay in range(3):
        o.zero_(); lse.zero_()                                                   # eager work between the replays
        junk = torch.full((1 << 18,), float(replay), device="cuda")
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(o, o_w) and torch.equal(lse, lse_w), replay
        del junk
