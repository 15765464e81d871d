"""Assertions that depend on wall-clock behaviour, kept apart from the parity files and collected after all of them
(a busy or throttled box can fail these with no defect in the code, and the suite stops at its first failure):

* the library's default tile choice is within 15 % of the best forced variant's time on products outside the GPT-3
  family (shapes and operands of tests/test_gpu_chooser.py, whose own test checks the results);
* a watcher on a second stream sees chunks of a counted LS / RS call complete before the kernel has ended
  (tests/test_gpu_signal.py checks that what it then reads is the finished chunk);
* one gated and counted LS / RS launch, its slices arriving 150 us apart on a producer stream, has chunk 0 complete
  before the last slice has been flagged (tests/test_zx_gpu_gate.py checks the results of such calls);
* the fp32 kernel's tile choice is within 15 % of the best of its five tiles forced.

Times are sustained wall-clock means (warm-up, then a loop between two synchronisations), the best of two rounds per
candidate, so that one host hiccup does not decide the comparison.  Marked ``perf`` besides ``gpu``:
``-m "gpu and not perf"`` runs the suite without them."""
import time

import pytest
import torch

from meshslice_amd import _lib
import test_gpu_chooser as chooser
import test_gpu_signal as signal_tests

pytestmark = [pytest.mark.gpu, pytest.mark.perf]
SLACK = 1.15
LAST_VARIANT = 14


def _sustained(f, warm=10, steps=25):
    for _ in range(warm):
        f()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        f()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


@pytest.mark.parametrize("flow", ["os", "ls", "rs"])
@pytest.mark.parametrize("shape", chooser.SHAPES, ids=["x".join(map(str, s)) for s in chooser.SHAPES])
def test_default_choice_is_close_to_the_best_variant(flow, shape):
    lib = _lib.load()
    run, _check = chooser.operands(flow, shape)
    times = {}
    try:
        for rnd in range(2):
            for v in range(0, LAST_VARIANT + 1):
                assert lib.ms_set_variant(v) == 0
                t = _sustained(run)
                times[v] = min(times.get(v, t), t)
                if v == 0:
                    picked = (int(lib.ms_query(_lib.MS_QUERY_LAST_VARIANT)), int(lib.ms_query(_lib.MS_QUERY_LAST_SPLITS)),
                              int(lib.ms_query(_lib.MS_QUERY_LAST_LAUNCHES)))
    finally:
        lib.ms_set_variant(0)
    best_v = min(range(1, LAST_VARIANT + 1), key=lambda v: times[v])
    if times[0] > SLACK * times[best_v]:
        # a host hiccup during the default's loops reads like a bad choice: time the two again before judging
        try:
            for v in (0, best_v, 0, best_v):
                assert lib.ms_set_variant(v) == 0
                times[v] = min(times[v], _sustained(run))
        finally:
            lib.ms_set_variant(0)
    assert times[0] <= SLACK * times[best_v], (
        f"default (variant {picked[0]}, {picked[1]} split(s), {picked[2]} launch(es)) {times[0] * 1e6:.0f} us; "
        f"variant {best_v} {times[best_v] * 1e6:.0f} us; all: " + " ".join(f"{v}:{t * 1e6:.0f}" for v, t in times.items()))


@pytest.mark.parametrize("shape", [(2048, 3072, 2048), (3072, 3072, 2048), (2048, 6144, 1024), (4096, 4096, 1024), (2048, 2048, 4096), (1024, 2048, 2048),
                                   (1536, 1536, 4096)], ids=lambda s: "x".join(map(str, s)))
def test_fp32_default_tile_is_close_to_the_best_tile(shape):
    """The fp32 kernel's tile choice (rounds x tile area x fitted cost) against each of its five tiles forced."""
    lib = _lib.load()
    m, n, k = shape
    g = torch.Generator(device="cuda").manual_seed(3)
    A = torch.randn((m, k), generator=g, device="cuda"); B = torch.randn((k, n), generator=g, device="cuda")
    C = torch.empty((m, n), device="cuda")
    import meshslice_amd as ms
    run = lambda: ms.gemm_os([A], [B], out=C)
    times = {}
    try:
        for rnd in range(2):
            for v in (0, 21, 22, 23, 24, 25):
                assert lib.ms_set_variant(v) == 0
                t = _sustained(run)
                times[v] = min(times.get(v, t), t)
                if v == 0:
                    picked = int(lib.ms_query(_lib.MS_QUERY_LAST_VARIANT))
    finally:
        lib.ms_set_variant(0)
    best = min((21, 22, 23, 24, 25), key=lambda v: times[v])
    assert times[0] <= SLACK * times[best], f"default (tile {picked}) {times[0] * 1e6:.0f} us; " + " ".join(f"{v}:{t * 1e6:.0f}" for v, t in times.items())


@pytest.mark.parametrize("flow", ["ls", "rs"])
def test_a_watcher_sees_chunks_complete_before_the_kernel_ends(flow):
    S, m, n, k, BAND = 8, 8192, 1536, 8192, 48      # about 1.3 ms of kernel: room for some tens of polls
    ops = signal_tests._operands(flow, m, n, k, S, torch.bfloat16)
    out = [torch.zeros((m, n), dtype=torch.bfloat16, device="cuda") for _ in range(S)]
    early = []
    for attempt in range(5):                  # the first call also loads the kernel's code: it may end before the first poll
        tiles, final, h, copied, _bands = signal_tests._watch_once(flow, ops, out, S, m, n, BAND)
        early = sorted(s for s, r in copied.items() if r)
        if early and len(h) > 2:
            break
    assert early, "no chunk was seen complete before the kernel had ended"


@pytest.mark.parametrize("flow", ["ls", "rs"])
def test_one_launch_with_both_ends_open_hands_on_chunk_0_before_the_last_slice_has_arrived(flow):
    """ms_gemm_ls_gated / ms_gemm_rs_gated with completion counters: the product is enqueued first, a producer stream
    then delivers slice after slice about 150 us apart (a copy, a delay, the flag), and a watcher polls flags and
    counters from the host.  Chunk 0 must be seen complete while the last flag is still down: the launch multiplies what
    has arrived while the rest is on its way, and says which chunks may already be handed on."""
    import meshslice_amd as ms
    S, m, n, k = 8, 8192, 1536, 8192
    lib = _lib.load()
    src = signal_tests._operands(flow, m, n, k, S, torch.bfloat16)
    which = 1 if flow == "ls" else 0
    ops = list(src)
    ops[which] = [torch.zeros_like(t) for t in src[which]]
    gated = ms.gemm_ls_gated if flow == "ls" else ms.gemm_rs_gated
    ready = torch.zeros(S + 1, dtype=torch.int32, device="cuda")
    done = torch.zeros(S, dtype=torch.int32, device="cuda")
    seen_ready = torch.zeros(S + 1, dtype=torch.int32).pin_memory()
    seen_done = torch.zeros(S, dtype=torch.int32).pin_memory()
    compute, producer, watch = torch.cuda.Stream(), torch.cuda.Stream(), torch.cuda.Stream()
    try:
        assert lib.ms_set_reserved_cus(32) == 0        # the producer's copies and the watcher's need compute units beside the product
        want = signal_tests._plain(flow, src, torch.bfloat16)
    finally:
        lib.ms_set_reserved_cus(0)
    early = []
    for attempt in range(4):          # the first call also loads code and sets up the streams: it may be over before the first poll
        for t in ops[which]:
            t.zero_()
        ready.zero_(); done.zero_()
        torch.cuda.synchronize()
        try:
            assert lib.ms_set_reserved_cus(32) == 0
            with torch.cuda.stream(compute):
                got, tiles = gated(*ops, ready, out_dtype=torch.bfloat16, chunk_done=done, timeout_ms=1500)
        finally:
            lib.ms_set_reserved_cus(0)
        with torch.cuda.stream(producer):
            for s_ in range(S):
                ops[which][s_].copy_(src[which][s_])
                torch.cuda._sleep(300000)                   # about 150 us
                ms.signal_set(ready, s_)
        history = []
        with torch.cuda.stream(watch):
            for poll in range(2000):                        # bounded: the watcher gives up, it never waits for the kernel
                seen_ready.copy_(ready, non_blocking=True)  # (flags first: a chunk seen complete after a flag seen down was complete before the flag went up)
                seen_done.copy_(done, non_blocking=True)
                watch.synchronize()
                history.append((seen_ready.tolist(), seen_done.tolist()))
                if history[-1][1] == [tiles] * S or history[-1][0][S]:
                    break
        torch.cuda.synchronize()
        if ms.gate_timed_out(ready):
            pytest.skip("the producer's copies did not run beside the waiting product on this machine")
        assert done.tolist() == [tiles] * S
        for s_ in range(S):
            assert torch.equal(got[s_], want[s_])
        early = [i for i, (r, d) in enumerate(history) if d[0] == tiles and r[S - 1] == 0]
        if early:
            break
    assert early, f"chunk 0 was never seen complete while the last flag was down ({len(history)} polls)"
    first = history[early[0]]
    print(f"\n{flow}: {len(history)} polls; chunk 0 first seen complete with {sum(first[0][:S])} of {S} slices flagged and {sum(d == tiles for d in first[1])} chunks complete")
