"""The entry points only launch kernels on the caller's stream (no allocation, no memset, no host
synchronisation), so a decode step can be captured in a HIP graph.  The graph is replayed several times
with eager work and synchronisations in between, and every replay is checked against the eager result."""
import math

import pytest
import torch

from oracle import libtorch_path as lt

pytestmark = pytest.mark.gpu


def test_decode_step_replays_from_a_captured_graph():
    import tyr_amd
    B, Hq, Hkv, L, D = 2, 8, 2, 700, 128           # few (batch, kv head) groups: the split + combine path
    q, = lt.make_inputs(3, (B, Hq, 1, D))
    kn, vn = lt.make_inputs(4, (B, Hkv, 1, D), (B, Hkv, 1, D))
    k0, v0 = lt.make_inputs(5, (B, Hkv, L, D), (B, Hkv, L, D))
    cos_t, sin_t = lt.compute_rotary_freqs(L, D)
    pos = L - 1
    cos, sin = cos_t[pos:pos + 1].contiguous().cuda(), sin_t[pos:pos + 1].contiguous().cuda()
    q, kn, vn = q.cuda(), kn.cuda(), vn.cuda()
    sc = 1.0 / math.sqrt(D)

    def step(kc, vc):
        qr = tyr_amd.decode_rope_append(q, kn, vn, cos, sin, kc, vc, pos)
        return tyr_amd.gqa_decode(qr, kc, vc, scale=sc, kv_len=L)

    ke, ve = k0.cuda().clone(), v0.cuda().clone()
    want_o, want_lse = step(ke, ve)
    torch.cuda.synchronize()

    kg, vg = k0.cuda().clone(), v0.cuda().clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(kg, vg)                                  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        got_o, got_lse = step(kg, vg)
    for replay in range(4):
        kg.copy_(k0.cuda()); vg.copy_(v0.cuda())     # eager work between the replays
        got_o.zero_(); got_lse.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got_o, want_o) and torch.equal(got_lse, want_lse), replay
        assert torch.equal(kg, ke) and torch.equal(vg, ve), replay


def test_calls_on_a_side_stream_allocate_on_that_stream():
    # Outputs and scratch of a call with `stream=` must belong to that stream (the caching allocator reuses a
    # freed block on the stream it was allocated on): the scratch of a backward or split-decode call queued on a
    # side stream is dropped at return while its kernels are still pending, and current-stream allocations that
    # follow must not be handed that block.  Results must equal those of the same calls on the current stream.
    import tyr_amd
    B, H, N, D = 2, 4, 600, 128
    q, k, v, g = (t.cuda() for t in lt.make_inputs(8, (B, H, N, D), (B, H, N, D), (B, H, N, D), (B, H, N, D)))
    qd, = lt.make_inputs(9, (B, 8, 1, D))
    kd, vd = (t.cuda() for t in lt.make_inputs(10, (B, 2, 3000, D), (B, 2, 3000, D)))
    qd = qd.cuda()
    o, lse = tyr_amd.flash_attn_fwd(q, k, v, causal=True)
    want = tyr_amd.flash_attn_bwd(q, k, v, o, lse, g, causal=True)
    want_d = tyr_amd.gqa_decode(qd, kd, vd, num_splits=6)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    for handle in (side, side.cuda_stream):          # a torch stream object and a raw hipStream_t handle
        got = tyr_amd.flash_attn_bwd(q, k, v, o, lse, g, causal=True, stream=handle)
        got_d = tyr_amd.gqa_decode(qd, kd, vd, num_splits=6, stream=handle)
        # churn on the current stream while the side stream is still busy
        junk = [torch.full((1 << 20,), float(i), device="cuda") for i in range(8)]
        side.synchronize()
        for a, b in zip(got + got_d, want + want_d):
            assert torch.equal(a, b)
        del junk
