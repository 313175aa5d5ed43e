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
