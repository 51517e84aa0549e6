"""Host threads: the library keeps no per-call state of its own (partitions are functions of the shapes, scratch and
streams are the caller's), so threads that bring their own stream and
workspace may call it at the same time (turboexl3 src/root.zig:155-160 keeps its caches behind spinlocks to the same
end). Four threads issue mixed calls on their own streams; every result must equal the single-threaded one."""
import threading

import numpy as np
import pytest
import torch

from tests.gpu_util import MCG, bytes_of, dev_f16_bits, dev_u16, make_x
from tests.test_gpu_moe import dev_bank, routing

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def t3():
    from turboexl3_amd import api
    return api


def test_threads_with_their_own_streams_and_workspaces(oracle, t3):
    rng = np.random.default_rng(0x7EAD)
    in_f, out_f, n = 1024, 512, 64
    trellis, suh, svh = oracle.synth_linear(rng, in_f, out_f, n)
    d_t, d_suh, d_svh = dev_u16(trellis), dev_f16_bits(suh), dev_f16_bits(svh)
    hidden, inter, experts, topk = 512, 256, 8, 4
    bank = dev_bank(t3, oracle.synth_bank(rng, experts, hidden, inter, 48))
    dec = t3.Decode(MCG, 16)
    w_hat = t3.dequant(d_t, dec)
    workers = 4
    inputs = []
    for w in range(workers):
        xd, _ = make_x(rng, 600, in_f, torch.bfloat16)
        xm, _ = make_x(rng, 20, hidden, torch.bfloat16)
        s, sc = routing(rng, 20, topk, experts)
        inputs.append((xd, xm.reshape(1, 20, hidden), torch.from_numpy(s).cuda().reshape(1, 20, topk),
                       torch.from_numpy(sc).cuda().reshape(1, 20, topk)))

    def calls(w, stream):
        xd, xm, s, sc = inputs[w]
        out = []
        for rows in (1, 7, 40, 600):  # one launch, chain, trellis GEMM, W_hat + the plain f16 GEMM
            out.append(t3.linear(xd[:rows], d_t, d_suh, d_svh, dec, stream=stream))
        out.append(t3.linear_resident(xd[:90], w_hat, d_suh, d_svh, stream=stream))
        out.append(t3.moe_clamped(xm[:, :3], bank, s[:, :3], sc[:, :3], dec, 7, stream=stream))
        out.append(t3.moe_clamped(xm, bank, s, sc, dec, 7, stream=stream))
        return out

    want = []
    for w in range(workers):
        want.append([bytes_of(y) for y in calls(w, None)])
    torch.cuda.synchronize()

    got = [None] * workers
    errors = []

    def worker(w):
        try:
            torch.cuda.set_device(0)
            stream = torch.cuda.Stream()
            mine = []
            with torch.cuda.stream(stream):  # torch's allocations of the outputs follow the thread's stream
                for _ in range(10):
                    mine = calls(w, stream)
            stream.synchronize()
            got[w] = [bytes_of(y) for y in mine]
        except Exception as e:  # surfaced by the main thread
            errors.append((w, repr(e)))

    threads = [threading.Thread(target=worker, args=(w,)) for w in range(workers)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(100)
    assert not errors, errors
    for w in range(workers):
        assert got[w] is not None, f"thread {w} did not finish"
        for i, (g, e) in enumerate(zip(got[w], want[w])):
            assert g == e, f"thread {w} call {i} differs from the single-threaded result"
