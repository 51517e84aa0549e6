"""The entry points under HIP graph capture: they allocate nothing, synchronise nothing and leave their arrival
counters as they found them, so a serving loop can hold a decode step (or a prefill chunk) as one graph. A captured
sequence of calls is replayed several times, with new inputs and eager work between the replays, and every replay must
give the bytes of the same calls made eagerly."""
import numpy as np
import pytest
import torch

from tests.gpu_util import MCG, MUL1, bytes_of, dev_f16_bits, dev_u16, make_x
from tests.test_gpu_moe import dev_bank, routing

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def t3():
    from turboexl3_amd import api
    return api


def test_captured_calls_replay_to_the_eager_bytes(oracle, t3):
    rng = np.random.default_rng(0x64A9)
    in_f, out_f, n = 1024, 512, 64
    trellis, suh, svh = oracle.synth_linear(rng, in_f, out_f, n)
    d_t, d_suh, d_svh = dev_u16(trellis), dev_f16_bits(suh), dev_f16_bits(svh)
    hidden, inter, experts, topk = 512, 256, 8, 4
    bank = dev_bank(t3, oracle.synth_bank(rng, experts, hidden, inter, 48))
    dec = t3.Decode(MCG, 16)

    # static inputs, as a captured step keeps them; the rows of each call are views of one buffer a kind
    x_dense = torch.zeros(530, in_f, dtype=torch.float16, device="cuda")
    w_hat = t3.dequant(d_t, dec)
    w_std, _ = t3.unrot_weight(d_t, d_suh, d_svh, dec, torch.float16)
    x_moe = torch.zeros(1, 20, hidden, dtype=torch.bfloat16, device="cuda")
    slots = torch.zeros(1, 20, topk, dtype=torch.int32, device="cuda")
    scores = torch.zeros(1, 20, topk, dtype=torch.float32, device="cuda")

    def step():
        return [
            t3.linear(x_dense[:1], d_t, d_suh, d_svh, dec),          # one launch, its finish by the last arriver
            t3.linear(x_dense[:8], d_t, d_suh, d_svh, dec),          # the three-launch chain
            t3.linear(x_dense[:40], d_t, d_suh, d_svh, dec),         # 40 rows: the trellis GEMM
            t3.linear(x_dense, d_t, d_suh, d_svh, dec),              # 530 rows: W_hat decoded, the f16 GEMM with its finish
            t3.linear_resident(x_dense[:100], w_hat, d_suh, d_svh),  # the same GEMM over a kept W_hat
            t3.linear_unrot(x_dense[:100], w_std),                   # the plain product over the un-rotated weight
            t3.linear_unrot_parts(x_dense[:100], w_std),             # the same with K shared out: planes, then their sum
            t3.linear_static(x_dense[:3], d_t, d_suh, d_svh, dec),   # scratch in the library's own device array
            t3.moe_clamped(x_moe[:, :2], bank, slots[:, :2], scores[:, :2], dec, 7),   # two arriving launches
            t3.moe_clamped(x_moe, bank, slots, scores, dec, 7),      # 20 rows: route, GEMMs, combine
            t3.linear(x_dense[:1], d_t, d_suh, d_svh, t3.Decode(MUL1, 16)),
        ]

    def new_inputs(seed):
        r = np.random.default_rng(seed)
        xd, _ = make_x(r, 530, in_f, torch.float16, outliers=True)
        xm, _ = make_x(r, 20, hidden, torch.bfloat16)
        s, w = routing(r, 20, topk, experts)
        x_dense.copy_(xd)
        x_moe.copy_(xm.reshape(1, 20, hidden))
        slots.copy_(torch.from_numpy(s).reshape(1, 20, topk))
        scores.copy_(torch.from_numpy(w).reshape(1, 20, topk))

    new_inputs(1)
    step()  # sizes the harness's workspace before anything is captured
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            captured = step()
    torch.cuda.synchronize()
    for seed in (2, 3, 4, 5):
        new_inputs(seed)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [bytes_of(y) for y in captured]
        want = [bytes_of(y) for y in step()]  # the program's own eager work between the replays
        torch.cuda.synchronize()
        for i, (g, w) in enumerate(zip(got, want)):
            assert g == w, f"replay with inputs {seed}: call {i} differs from the eager call"


def test_the_grouped_routed_form_under_capture(oracle, t3):
    """The six-launch grouped form (its grouping launch builds the table on the device from the call's ids): captured once,
    replayed on new activations AND new routings, every replay the eager bytes."""
    rng = np.random.default_rng(0x64AA)
    hidden, inter, experts, topk, rows = 512, 256, 6, 3, 12
    bank = dev_bank(t3, oracle.synth_bank(rng, experts, hidden, inter, 64))
    dec = t3.Decode(MCG, 16)
    x = torch.zeros(1, rows, hidden, dtype=torch.bfloat16, device="cuda")
    slots = torch.zeros(1, rows, topk, dtype=torch.int32, device="cuda")
    scores = torch.zeros(1, rows, topk, dtype=torch.float32, device="cuda")

    def new_inputs(seed):
        r = np.random.default_rng(seed)
        xm, _ = make_x(r, rows, hidden, torch.bfloat16)
        s, w = routing(r, rows, topk, experts)
        s[seed % rows, 0] = -1  # a skipped id, somewhere else every time
        x.copy_(xm.reshape(1, rows, hidden))
        slots.copy_(torch.from_numpy(s).reshape(1, rows, topk))
        scores.copy_(torch.from_numpy(w).reshape(1, rows, topk))

    t3.configure(decode_form=6)
    try:
        new_inputs(1)
        t3.moe_clamped(x, bank, slots, scores, dec, 7)
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                captured = t3.moe_clamped(x, bank, slots, scores, dec, 7)
        torch.cuda.synchronize()
        for seed in (2, 3, 4):
            new_inputs(seed)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            got = bytes_of(captured)
            want = bytes_of(t3.moe_clamped(x, bank, slots, scores, dec, 7))
            torch.cuda.synchronize()
            assert got == want, f"replay with inputs {seed} differs from the eager call"
    finally:
        t3.configure()
