"""Stage lifetimes of the kernels that fill LDS by global->LDS requests (no registers in between).

Every such kernel keeps tiles in a small ring of LDS stages.  Two things must hold for every stage, whatever the
relative speed of the waves of a workgroup:

  read-after-write   a fragment read of tile v from a stage comes after a workgroup barrier that every wave reached
                     after waiting for its own share of the requests of tile v (a wave only waits for its own requests);
  write-after-read   a request that overwrites a stage is issued after a workgroup barrier that follows, in every
                     wave's program order, the last read of the tile the stage held (LDS reads have returned at a
                     barrier: the compiler waits for them in front of it).

The checker below works on the order of events of one wave -- requests, waits, barriers, reads, the epilogue's plain
stores -- which this file restates for each kernel from its source (same loop structure, same stage arithmetic), for
every wave of a workgroup and a range of trip counts.  Barriers cut a wave's events into intervals; events of two waves
in the same interval are concurrent, events in different intervals are ordered.  A read of version v of a stage in
interval i is safe iff the request of v completed at a barrier <= i and the next request into the same stage is issued
in an interval > i.

The forward kernel once lacked the barrier between its prologue's reads of K stage 0 and the first step's request into
that stage; `test_the_checker_catches_the_forward_kernels_old_race` runs that event order and demands a violation.
"""
import pytest


class Trace:
    """Event recorder for one wave."""

    def __init__(self):
        self.interval = 0
        self.events = []          # (kind, interval, stage, version)
        self.pending = []         # requests of this wave not yet waited for: indices into self.requests
        self.requests = []        # [stage, version, issued_interval, completed_barrier or None]

    def dma(self, stage, version):
        self.requests.append([stage, version, self.interval, None])
        self.pending.append(len(self.requests) - 1)

    def wait(self, keep_newest=0):
        """s_waitcnt vmcnt: everything but the newest `keep_newest` requests has landed (for this wave)."""
        done = self.pending[:len(self.pending) - keep_newest] if keep_newest else self.pending
        for i in done:
            self.requests[i][3] = "waited"
        self.pending = self.pending[len(done):]

    def bar(self):
        self.interval += 1
        for r in self.requests:
            if r[3] == "waited":
                r[3] = self.interval          # visible to every wave from this interval on

    def read(self, stage, version):
        self.events.append(("read", self.interval, stage, version))

    def store(self, stage, version="scratch"):
        """A plain LDS store by this wave (epilogue staging): overwrites the stage at once."""
        self.requests.append([stage, version, self.interval, self.interval])


def violations(traces):
    """traces: one Trace per wave of a workgroup.  Returns a list of human-readable violations."""
    out = []
    skeleton = [(r[0], r[1], r[2], r[3]) for r in traces[0].requests]
    for t in traces[1:]:
        if [(r[0], r[1], r[2], r[3]) for r in t.requests] != skeleton:
            out.append("waves disagree on the order of requests, waits and barriers")
            return out
    by_stage = {}
    for stage, version, issued, completed in skeleton:
        by_stage.setdefault(stage, []).append((version, issued, completed))
    for w, t in enumerate(traces):
        for _, at, stage, version in t.events:
            reqs = by_stage.get(stage, [])
            idx = [i for i, r in enumerate(reqs) if r[0] == version]
            if not idx:
                out.append(f"wave {w}: reads {version} from {stage}, which nobody requested")
                continue
            # the request this read means: the last one of that version issued before the read's interval ends
            i = max(j for j in idx if reqs[j][1] <= at) if any(reqs[j][1] <= at for j in idx) else idx[0]
            version_, issued, completed = reqs[i]
            if completed is None or not isinstance(completed, int) or completed > at:
                out.append(f"wave {w}: reads {version} from {stage} in interval {at} before its request completed ({completed})")
            if i + 1 < len(reqs) and reqs[i + 1][1] <= at:
                out.append(f"wave {w}: reads {version} from {stage} in interval {at}, but {reqs[i + 1][0]} is requested into it "
                           f"in interval {reqs[i + 1][1]}")
    return out


# ------------------------------------------------------------------ flash_attn_fwd_kernel (tyr_amd/csrc/flash_attn_fwd.hip)
def forward_wave(passes, wave, barrier_after_prologue=True):
    """passes: list of (nkv, nkv_w per wave, overlap_next).  Stages K0 K1 V0 V1; tile j of pass p is version (p, 'K'|'V', j).
    The epilogue stages O through the V stages (each wave its own quarter of them)."""
    t = Trace()
    preloaded = False
    for p, (nkv, nkv_ws, overlap_next) in enumerate(passes):
        nkv_w = nkv_ws[wave]
        if not preloaded:
            t.dma("K0", (p, "K", 0))
            t.dma("V0", (p, "V", 0))
            if nkv > 1:
                t.dma("K1", (p, "K", 1))
        else:
            t.dma("V0", (p, "V", 0))
        t.wait()
        t.bar()
        t.read("K0", (p, "K", 0))                       # S(0)
        if barrier_after_prologue:
            t.bar()
        for j in range(nkv):
            if j + 2 < nkv:
                t.dma(f"K{j & 1}", (p, "K", j + 2))
            elif overlap_next:
                t.dma(f"K{j & 1}", (p + 1, "K", j + 2 - nkv))
            if j >= nkv_w and j + 1 < nkv:
                t.dma(f"V{(j + 1) & 1}", (p, "V", j + 1))
            if j < nkv_w:
                if j + 1 < nkv:                          # (on the last tile these reads hit stale data and are unused)
                    t.read(f"K{(j + 1) & 1}", (p, "K", j + 1))
                if j + 1 < nkv:
                    t.dma(f"V{(j + 1) & 1}", (p, "V", j + 1))
                t.read(f"V{j & 1}", (p, "V", j))
            t.wait()
            t.bar()
        t.store("V0", (p, "O"))
        t.store("V1", (p, "O"))
        t.read("V0", (p, "O"))
        t.read("V1", (p, "O"))
        t.bar()
        preloaded = overlap_next
    return t


def forward_passes(nkvs):
    """Consecutive tiles of one workgroup (a pair, or a persistent workgroup's jobs): tile p hands over to tile p+1 through
    overlap_next when its tile count is even (the stage parity the kernel asks for)."""
    out = []
    for i, nkv in enumerate(nkvs):
        # causal: waves 0, 1 see one tile less than waves 2, 3 when the tile count is even (128 query rows, 64-row tiles)
        nkv_w = [max(1, nkv - 1), max(1, nkv - 1), nkv, nkv]
        out.append((nkv, nkv_w, i + 1 < len(nkvs) and nkv % 2 == 0))
    return out


@pytest.mark.parametrize("nkvs", [[1], [2], [3], [2, 2], [64, 2], [6, 4, 2, 8], [5, 4], [4, 1, 2], [2, 3, 2], [8, 8, 8]])
def test_forward_kernel(nkvs):
    traces = [forward_wave(forward_passes(nkvs), w) for w in range(4)]
    assert violations(traces) == []


def test_the_checker_catches_the_forward_kernels_old_race():
    traces = [forward_wave(forward_passes([4]), w, barrier_after_prologue=False) for w in range(4)]
    v = violations(traces)
    assert v and all("K0" in x for x in v), v


# ------------------------------------------------------------------ flash_attn_bwd_dq_kernel (tyr_amd/csrc/flash_attn_bwd.hip)
def dq_wave(passes, wave):
    """Stages KV0 KV1 (K and V of a tile are requested together); the epilogue stages dQ through the front of the LDS
    block, which overlaps both stages."""
    t = Trace()
    for p, (nkv, nkv_ws) in enumerate(passes):
        t.dma("KV0", (p, 0))
        t.wait()
        t.bar()
        for j in range(nkv):
            if j + 1 < nkv:
                t.dma(f"KV{(j + 1) & 1}", (p, j + 1))
            if j < nkv_ws[wave]:
                t.read(f"KV{j & 1}", (p, j))
            t.wait()
            t.bar()
        t.store("KV0", (p, "dQ"))
        t.store("KV1", (p, "dQ"))
        t.read("KV0", (p, "dQ"))
        t.read("KV1", (p, "dQ"))
        t.bar()
    return t


@pytest.mark.parametrize("nkvs", [[1], [2], [3], [64, 2], [7, 4], [1, 1]])
def test_backward_dq_kernel(nkvs):
    passes = [(n, [max(1, n - 1), max(1, n - 1), n, n]) for n in nkvs]
    assert violations([dq_wave(passes, w) for w in range(4)]) == []


# ------------------------------------------------------------------ flash_attn_bwd_dkv_kernel
def dkv_wave(ntile, heads, wave, causal=True, stages=4):
    """Stages T0..T3: tile t (Q, dO and the (lse, delta) pairs of 64 query rows) lives in stage t % 4, three tiles are in
    flight.  Sub-tile u = 2t + T; a step on u reads tile t and, ahead, the sub-tiles u+1 and u+2 (tile t or t+1); reads past
    the last tile are dropped.  A causal wave skips the sub-tiles above its diagonal but keeps the tile boundaries."""
    t = Trace()
    nsub = 2 * ntile
    u0 = wave if causal else 0

    def rd(h, tile):
        if tile < ntile:
            t.read(f"T{tile % stages}", (h, tile))

    for h in range(heads):
        for k in range(3):
            t.dma(f"T{k % stages}", (h, k))
        t.wait(keep_newest=2)
        t.bar()

        def tile_boundary(u):
            if u % 2 == 0 and u // 2 + 1 < ntile:
                t.wait(keep_newest=1)
                t.bar()
                t.dma(f"T{(u // 2 + 3) % stages}", (h, u // 2 + 3))

        u = 0
        while u < u0 and u < nsub:
            tile_boundary(u)
            u += 1
        if u < nsub:                                     # first_scores: sub-tile u and the row fragments of u+1
            rd(h, u // 2)
            rd(h, (u + 1) // 2)
        while u < nsub:
            tile_boundary(u)
            rd(h, u // 2)                                # transposed fragments of u
            rd(h, (u + 1) // 2)                          # pairs of u+1
            rd(h, (u + 2) // 2)                          # row fragments of u+2
            u += 1
        t.wait()
        t.bar()
    for s in range(stages):
        t.store(f"T{s}", "dKdV")                        # the epilogue's staging area overlaps the front stages
        t.read(f"T{s}", "dKdV")
    return t


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("ntile,heads", [(1, 1), (2, 1), (3, 2), (4, 1), (5, 1), (8, 4), (64, 1)])
def test_backward_dkv_kernel(ntile, heads, causal):
    assert violations([dkv_wave(ntile, heads, w, causal) for w in range(4)]) == []


def test_three_stages_would_not_be_enough_for_the_dkv_kernel():
    # with tile t+3 requested into the stage of tile t (a ring of three), the steps that still read tile t collide with it
    assert violations([dkv_wave(6, 1, w, True, stages=3) for w in range(4)])


# ------------------------------------------------------------------ gemm_bf16_fast_kernel / gemm_fp8_fast_kernel
def gemm_wave(KT, ksteps):
    """Two stages S0 S1, each an A and a B slice.  Slice kt+1 is requested during the first k-steps of slice kt; the
    fragments of k-step s+1 are read under the products of k-step s; inside the last k-step (bf16: after its second product
    row, fp8: before its last) the workgroup waits, synchronises and reads the first fragments of the next slice.  The request and the reads past the
    last slice touch the idle stage and are never used (modelled: the request, as it is really issued; not the reads).
    The epilogue stages C through the front of the LDS block (stage 0)."""
    t = Trace()
    t.dma("S0", 0)
    t.wait()
    t.bar()
    t.read("S0", 0)
    for kt in range(KT):
        st = kt & 1
        for s in range(ksteps):
            if s < ksteps - 1:
                if s < 2:
                    t.dma(f"S{st ^ 1}", kt + 1)          # the two halves of the next slice (bf16: k-steps 0, 1; fp8: both in 0)
                t.read(f"S{st}", kt)
            else:
                t.wait()
                t.bar()
                if kt + 1 < KT:
                    t.read(f"S{st ^ 1}", kt + 1)
    t.store("S0", "C")
    t.read("S0", "C")
    return t


# eight waves; bf16: four k-steps of 16 per 64-wide slice; fp8: two k-steps of 64 per 128-byte slice
@pytest.mark.parametrize("ksteps,waves", [(4, 8), (2, 8)])
@pytest.mark.parametrize("KT", [1, 2, 3, 4, 63, 64])
def test_gemm_fast_kernels(KT, ksteps, waves):
    assert violations([gemm_wave(KT, ksteps) for _ in range(waves)]) == []
