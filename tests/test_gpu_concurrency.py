"""Two host threads, each on a stream of its own, run forward + backward of the one-stage Function at the same
time with different launch options: the library keeps no per-call state outside the caller's buffers (launch options
travel with the call, the per-device caches are guarded), so every result must equal the one the same thread gets
when it runs alone."""
import threading

import pytest
import torch

from forms import tiny_case

pytestmark = pytest.mark.gpu


def _step(F1, t, dev):
    v, d, loc, a = [t[k].to(dev).requires_grad_() for k in ("value", "dist", "loc", "attn")]
    out, score = F1.apply(v, d, t["shapes3"].to(dev), t["lsi"].to(dev), loc, a, 64)
    grads = torch.autograd.grad(out, [v, d, loc, a], t["grad_out"].to(dev))
    return [out.detach(), score.detach(), *grads]


def test_two_threads_on_two_streams():
    from dfa3D import _lib
    from dfa3D.functional import MultiScale3DDeformableAttnFunction as F1
    dev = torch.device("cuda:0")
    cases = [tiny_case(90, B=2, C=32, M=8, Q=900, P=8, D=16, levels=((37, 52), (19, 26), (7, 9)), dtype=torch.float32),
             tiny_case(91, B=3, C=16, M=5, Q=700, P=4, D=32, levels=((21, 30), (9, 11)), dtype=torch.float32)]
    options = [dict(), dict(tile=404, chunk=256)]
    alone = []
    for t, o in zip(cases, options):
        with _lib.launch_options(**o):
            alone.append([x.cpu() for x in _step(F1, t, dev)])
    torch.cuda.synchronize()

    results, errors = [None, None], []
    start = threading.Barrier(2)

    def work(i):
        try:
            stream = torch.cuda.Stream()                   # default priority
            with torch.cuda.stream(stream), _lib.launch_options(**options[i]):
                start.wait(timeout=60)
                for _ in range(5):
                    got = _step(F1, cases[i], dev)
                stream.synchronize()
            results[i] = [x.cpu() for x in got]
        except Exception as e:                             # reported by the main thread
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=120)
    assert not any(th.is_alive() for th in threads), "a worker thread did not finish"
    assert not errors, errors
    for i in range(2):
        for k, (got, want) in enumerate(zip(results[i], alone[i])):
            if k < 2 or k >= 4:                            # output, scores, per-point gradients: same arithmetic
                assert torch.equal(got, want), f"thread {i}, result {k}"
            else:                                          # tile flushes: summation order may differ
                torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-4)
