"""``oa_h2d_async`` / ``oa_d2h_async``: host<->device copies on a fixed SDMA engine per
direction, issued by the library through the ROCr runtime and fenced inside a HIP
stream (include/offload_adam_hip.h, csrc/link_copies.hip), through the C ABI.

What has to hold is the contract of ``hipMemcpyAsync`` on the stream: the copy sees
everything the stream was given before it, everything given after it sees the copy,
events recorded behind it complete after it - whatever else runs on other streams,
from whichever thread, and for more copies than the signal ring has slots.  Every
wait in these tests is bounded: a copy that never completes fails the test instead
of hanging it.
"""

import ctypes
import threading
import time
from ctypes import c_size_t, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu


def _lib():
    from offload_adam_amd import _lib as kernels

    return kernels, kernels.load()


def _done(stream, seconds=30.0):
    """True once the stream has drained; False after ``seconds`` (never blocks for good)."""
    t0 = time.monotonic()
    while time.monotonic() - t0 < seconds:
        if stream.query():
            return True
        time.sleep(0.0005)
    return False


def _status(lib):
    h2d, d2h = ctypes.c_uint(0), ctypes.c_uint(0)
    a, b, c = ctypes.c_ulonglong(0), ctypes.c_ulonglong(0), ctypes.c_ulonglong(0)
    rc = lib.oa_link_copy_status(ctypes.byref(h2d), ctypes.byref(d2h), ctypes.byref(a),
                                 ctypes.byref(b), ctypes.byref(c))
    return rc, h2d.value, d2h.value, a.value, b.value, c.value


def _h2d(lib, dst, src, stream, wait=None, record=None):
    return lib.oa_h2d_async(c_void_p(dst.data_ptr()), c_void_p(src.data_ptr()),
                            c_size_t(src.numel() * src.element_size()),
                            c_void_p(stream.cuda_stream), wait, record)


def _d2h(lib, dst, src, stream, wait=None, record=None):
    return lib.oa_d2h_async(c_void_p(dst.data_ptr()), c_void_p(src.data_ptr()),
                            c_size_t(src.numel() * src.element_size()),
                            c_void_p(stream.cuda_stream), wait, record)


def test_fixed_engine_copies_are_in_effect_and_keep_stream_order():
    from offload_adam_amd.pinned_alloc import zeros_pinned

    kernels, lib = _lib()
    torch.cuda.init()
    rc, e_up, e_down, up0, down0, fell0 = _status(lib)
    assert rc == 0, kernels.error_string(rc)
    assert (e_up, e_down) == (1, 2)
    n = 6 << 20
    host_in = zeros_pinned((n,), torch.int32, numa_node=None)
    host_out = zeros_pinned((n,), torch.int32, numa_node=None)
    host_in.copy_(torch.arange(n, dtype=torch.int32))
    up, down = torch.cuda.Stream(), torch.cuda.Stream()
    main = torch.cuda.current_stream()
    for rep in range(6):
        dev = torch.empty(n, dtype=torch.int32, device="cuda")
        # kernels before the copy on the same stream: the copy must come after them
        with torch.cuda.stream(up):
            dev.fill_(-1)
        assert _h2d(lib, dev, host_in, up) == 0
        # work after the copy on the same stream must see it
        with torch.cuda.stream(up):
            dev.add_(rep)
        main.wait_stream(up)
        dev.mul_(2)
        down.wait_stream(main)
        assert _d2h(lib, host_out, dev, down) == 0
        dev.record_stream(down)
        assert _done(down), "the write-back never completed"
        assert torch.equal(host_out, (host_in + rep) * 2), rep
    rc, _, _, up1, down1, fell1 = _status(lib)
    assert rc == 0 and up1 - up0 == 6 and down1 - down0 == 6 and fell1 == fell0


def test_events_passed_in_are_waited_for_and_recorded():
    from offload_adam_amd.pinned_alloc import zeros_pinned

    _, lib = _lib()
    n = 4 << 20
    host = zeros_pinned((n,), torch.float32, numa_node=None)
    back = zeros_pinned((n,), torch.float32, numa_node=None)
    host.copy_(torch.linspace(0, 1, n))
    side = torch.cuda.Stream()
    main = torch.cuda.current_stream()
    dev = torch.zeros(n, dtype=torch.float32, device="cuda")
    busy = torch.zeros(64 << 20, dtype=torch.float32, device="cuda")
    for _ in range(20):
        busy.add_(1.0)  # keeps the main stream busy for a few milliseconds
    dev.fill_(3.0)
    ready = torch.cuda.Event()
    ready.record(main)
    arrived = torch.cuda.Event()
    arrived.record(side)  # gives the event a handle; it is recorded again by the copy
    # the write-back waits for `ready` (main stream's fill) although it runs on `side`
    assert _d2h(lib, back, dev, side, c_void_p(ready.cuda_event), c_void_p(arrived.cuda_event)) == 0
    t0 = time.monotonic()
    while not arrived.query():
        assert time.monotonic() - t0 < 30, "the event behind the copy never completed"
        time.sleep(0.0005)
    assert bool((back == 3.0).all())
    # zero bytes: events are still honoured, nothing is copied
    again = torch.cuda.Event()
    again.record(side)
    assert lib.oa_h2d_async(None, None, c_size_t(0), c_void_p(side.cuda_stream), None,
                            c_void_p(again.cuda_event)) == 0
    assert _done(side)
    assert lib.oa_h2d_async(None, c_void_p(host.data_ptr()), c_size_t(16),
                            c_void_p(side.cuda_stream), None, None) == -1


def test_more_copies_than_ring_slots_from_two_threads():
    """3000 small copies per direction (the ring has 1024 slots), issued from two
    threads on two streams at once, each checked against its source."""
    from offload_adam_amd.pinned_alloc import zeros_pinned

    _, lib = _lib()
    chunk, count = 4096, 3000
    host_src = zeros_pinned((count, chunk), torch.int32, numa_node=None)
    host_dst = zeros_pinned((count, chunk), torch.int32, numa_node=None)
    host_src.copy_(torch.arange(count * chunk, dtype=torch.int32).view(count, chunk))
    dev_a = torch.zeros(count, chunk, dtype=torch.int32, device="cuda")
    dev_b = (torch.arange(count * chunk, dtype=torch.int32, device="cuda") * 3).view(count, chunk)
    torch.cuda.synchronize()
    up, down = torch.cuda.Stream(), torch.cuda.Stream()
    errors = []

    def worker(h2d):
        try:
            torch.cuda.set_device(0)
            for i in range(count):
                rc = (_h2d(lib, dev_a[i], host_src[i], up) if h2d
                      else _d2h(lib, host_dst[i], dev_b[i], down))
                if rc:
                    errors.append((h2d, i, rc))
                    return
        except Exception as exc:  # noqa: BLE001 - reported by the main thread
            errors.append(repr(exc))

    threads = [threading.Thread(target=worker, args=(flag,)) for flag in (True, False)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(120)
        assert not t.is_alive(), "a thread is stuck issuing copies"
    assert not errors, errors[:3]
    assert _done(up) and _done(down), "copies never completed"
    assert torch.equal(dev_a.cpu(), host_src)
    assert torch.equal(host_dst, dev_b.cpu())


def test_a_batch_is_one_unit_in_the_streams_order():
    """oa_link_copy_batch: 700 copies (more than one unit of 256) of ragged sizes, some
    empty, behind a kernel that produces their source; events recorded behind chosen
    copies complete in order and only once their copy has landed."""
    from offload_adam_amd.pinned_alloc import zeros_pinned

    kernels, lib = _lib()
    count = 700
    sizes = [0 if i % 97 == 5 else 4 * (1000 + 37 * i) for i in range(count)]
    offsets = [sum(sizes[:i]) for i in range(count)]
    total = sum(sizes)
    host = zeros_pinned((total,), torch.uint8, numa_node=None)
    dev = torch.zeros(total, dtype=torch.uint8, device="cuda")
    side = torch.cuda.Stream()
    main = torch.cuda.current_stream()
    pattern = (torch.arange(total, device="cuda") % 251).to(torch.uint8)
    side.wait_stream(main)
    with torch.cuda.stream(side):
        for _ in range(8):
            dev.zero_()
        dev.copy_(pattern)  # the copies below must see this, not the zeros
    events = {i: torch.cuda.Event() for i in (0, 5, 255, 256, 699)}
    for e in events.values():
        e.record(side)  # gives each a handle
    dsts = (ctypes.c_uint64 * count)(*[host.data_ptr() + o for o in offsets])
    srcs = (ctypes.c_uint64 * count)(*[dev.data_ptr() + o for o in offsets])
    nbytes = (ctypes.c_size_t * count)(*sizes)
    recs = (ctypes.c_uint64 * count)(*[events[i].cuda_event if i in events else 0
                                       for i in range(count)])
    rc = lib.oa_link_copy_batch(count, dsts, srcs, nbytes, kernels.OA_COPY_D2H,
                                c_void_p(side.cuda_stream), recs)
    assert rc == 0, kernels.error_string(rc)
    t0 = time.monotonic()
    while not events[699].query():
        assert time.monotonic() - t0 < 30, "the last event never completed"
        time.sleep(0.0005)
    assert all(e.query() for e in events.values())
    assert torch.equal(host, pattern.cpu())
    # the other direction, no events, then arguments the library rejects
    dev.zero_()
    side.wait_stream(main)
    rc = lib.oa_link_copy_batch(count, srcs, dsts, nbytes, kernels.OA_COPY_H2D,
                                c_void_p(side.cuda_stream), None)
    assert rc == 0 and _done(side)
    assert torch.equal(dev.cpu(), pattern.cpu())
    assert lib.oa_link_copy_batch(count, srcs, dsts, nbytes, kernels.OA_COPY_D2D,
                                  c_void_p(side.cuda_stream), None) == -1
    assert lib.oa_link_copy_batch(-1, srcs, dsts, nbytes, kernels.OA_COPY_H2D,
                                  c_void_p(side.cuda_stream), None) == -1
    assert lib.oa_link_copy_batch(0, None, None, None, kernels.OA_COPY_H2D,
                                  c_void_p(side.cuda_stream), None) == 0
    bad = (ctypes.c_uint64 * count)(*([0] + list(srcs)[1:]))
    assert lib.oa_link_copy_batch(count, bad, dsts, nbytes, kernels.OA_COPY_H2D,
                                  c_void_p(side.cuda_stream), None) == -1
    assert _done(side)


def test_the_optimizer_uses_them_and_the_old_path_gives_the_same_bits(monkeypatch):
    """``OffloadAdam``'s transfers go through the fixed-engine entry points by default;
    with them switched off (hipMemcpyAsync + tools library) the results are identical."""
    import random
    import warnings

    from offload_adam_amd import OffloadAdam
    from offload_adam_amd import offload_adam as oa_mod

    _, lib = _lib()
    monkeypatch.setattr(random, "getrandbits", lambda k: 0x1234_5678_9ABC_DEF0)

    def run(fixed):
        monkeypatch.setattr(oa_mod, "_FIXED_ENGINE_COPIES", fixed)
        torch.manual_seed(0)
        model = torch.nn.Sequential(torch.nn.Linear(256, 512), torch.nn.GELU(),
                                    torch.nn.Linear(512, 256)).to(device="cuda", dtype=torch.bfloat16)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            opt = OffloadAdam(model, lr=1e-2, inplace_param_threshold=1000)
        g = torch.Generator().manual_seed(1)
        for step in range(3):
            for mb in range(2):
                opt.ready_for_optimizer_step = mb == 1
                x = torch.randn(32, 256, generator=g).to(device="cuda", dtype=torch.bfloat16)
                model(x).float().square().mean().backward()
            opt.step()
        torch.cuda.synchronize()
        return [p.detach().clone() for p in model.parameters()], opt

    before = _status(lib)
    fixed, opt = run(True)
    after = _status(lib)
    assert after[3] > before[3] and after[4] > before[4], "the optimizer did not use them"
    assert after[5] == before[5]
    plain, _ = run(False)
    assert _status(lib)[3:5] == after[3:5]
    for a, b in zip(fixed, plain):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))


def test_bounded_wait_reports_a_copy_that_outlasts_it_and_recovers():
    """The stream-side wait of a copy is bounded (``oa_link_wait_limit``): with a bound of
    one poll and a 256 MB copy (about 5 ms on the link) the wait gives up while the
    engine is still copying, the stream goes on, and every later copy call returns
    OA_ELINKTIMEOUT until the caller clears the mark.  The condition is forced from the
    host; every kernel involved exits by itself and the copy completes normally."""
    from offload_adam_amd.pinned_alloc import zeros_pinned

    kernels, lib = _lib()
    OA_ELINKTIMEOUT = -7
    rc = _status(lib)[0]
    assert rc == 0, kernels.error_string(rc)
    n = 64 << 20
    host = zeros_pinned((n,), torch.int32, numa_node=None)
    host.copy_(torch.arange(n, dtype=torch.int32))
    dev = torch.zeros(n, dtype=torch.int32, device="cuda")
    small_host = zeros_pinned((1024,), torch.int32, numa_node=None)
    small_dev = torch.arange(1024, dtype=torch.int32, device="cuda")
    s = torch.cuda.Stream()
    torch.cuda.synchronize()
    assert lib.oa_link_wait_limit(1 << 40, 0) == -3  # OA_ERANGE: beyond 2^32 - 1
    assert lib.oa_link_wait_limit(1, 0) == 0
    try:
        assert _h2d(lib, dev, host, s) == 0
        assert _done(s, 10.0), "the bounded wait did not let the stream go on"
        # the mark is up: nothing more is issued on this GPU's link
        assert _d2h(lib, small_host, small_dev, s) == OA_ELINKTIMEOUT
        assert lib.oa_link_wait_limit(0, 0) == OA_ELINKTIMEOUT
        assert "time limit" in kernels.error_string(OA_ELINKTIMEOUT)
        from offload_adam_amd import offload_adam as oa_mod

        if oa_mod._fixed_engine_copies():
            with pytest.raises(RuntimeError, match="time limit"):
                oa_mod._copy_async(small_host, small_dev, kernels.OA_COPY_D2H, s)
        # the copy itself was never lost: wait, by the clock, until all of it has landed
        t0 = time.monotonic()
        landed = False
        while time.monotonic() - t0 < 20.0 and not landed:
            time.sleep(0.05)
            landed = bool((dev[-4096:].cpu() == host[-4096:]).all()) and int(dev[0].item()) == 0 \
                and int(dev[n // 2].item()) == n // 2
        assert landed
        time.sleep(0.2)
        assert torch.equal(dev.cpu(), host)
    finally:
        # (nothing is outstanding any more: the one copy issued under the mark has landed)
        assert lib.oa_link_wait_limit(0, 1) in (0, OA_ELINKTIMEOUT)
    assert lib.oa_link_wait_limit(0, 0) == 0
    assert _d2h(lib, small_host, small_dev, s) == 0
    assert _done(s)
    assert torch.equal(small_host, small_dev.cpu())
