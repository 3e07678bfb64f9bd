"""Calls from several host threads on their own streams: the library keeps no mutable state between calls (the
reference's autograd backward runs on another thread than the forward), so concurrent calls give the bits that the same
calls give one after the other."""
import threading

import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(gpu, seed, B, H, Lq, Lkv, d):
    g = torch.Generator(device=gpu).manual_seed(seed)
    rn = lambda L, s: (torch.randn((B, H, L, d), generator=g, device=gpu) * s).to(torch.bfloat16)
    return rn(Lq, 1.0), rn(Lkv, 1.0), rn(Lkv, 1.0), rn(Lq, 0.1), rn(Lkv, 0.1), rn(Lkv, 0.1), rn(Lq, 1.0)


def _work(pkg, args):
    q, k, v, tq, tk, tv, dout = args
    o, to, lse = pkg.fwd_jvp(q, k, v, tq, tk, tv)
    dq, dk, dv = pkg.bwd(q, k, v, o, lse, dout)
    return o, to, lse, dq, dk, dv


def test_concurrent_calls_from_threads_match_serial_calls(pkg, gpu):
    shapes = [(1, 4, 1000, 1000, 128), (2, 2, 640, 333, 64), (1, 3, 2048, 512, 128), (1, 2, 515, 999, 32)]
    cases = [_inputs(gpu, 100 + i, *shp) for i, shp in enumerate(shapes)]
    serial = [_work(pkg, c) for c in cases]
    torch.cuda.synchronize()
    results, errors = [None] * len(cases), []

    def run(i):
        try:
            stream = torch.cuda.Stream(device=gpu)
            stream.wait_stream(torch.cuda.default_stream(gpu))
            with torch.cuda.stream(stream):
                out = None
                for _ in range(5):
                    out = _work(pkg, cases[i])
            stream.synchronize()
            results[i] = out
        except Exception as e:  # surfaced below: an exception in a thread would otherwise pass silently
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=run, args=(i,)) for i in range(len(cases))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a worker thread did not finish"
    assert not errors, errors
    torch.cuda.synchronize()
    for i, (want, got) in enumerate(zip(serial, results)):
        for name, a, b in zip(("o", "to", "lse", "dq", "dk", "dv"), want, got):
            assert torch.equal(a, b), f"case {i} ({shapes[i]}): {name} differs between serial and concurrent calls"
