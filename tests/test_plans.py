"""The library's launch partitions, read through t3_linear_plan_of / t3_moe_plan_of without a GPU (nothing is launched
and no pointer is followed): the benchmark configurations' partitions, the rule every byte equality rests on (the K
split of a matrix never depends on the rows of a call), and the path a call takes by its rows."""
import ctypes as C

import pytest

from turboexl3_amd import _lib
from turboexl3_amd._lib import Array, Bank, Config, Decode, LinearPlan, MoePlan, Proj

F32, F16, BF16, U16, I16, U32, I32 = range(7)
FAKE = 0x10000  # an aligned non-null address: the plan queries read descriptors only


def arr(dtype, *shape):
    a = Array()
    a.data, a.ndim, a.dtype = FAKE, len(shape), dtype
    for i, d in enumerate(shape):
        a.shape[i] = d
    return a


@pytest.fixture(scope="module")
def lib():
    return _lib.lib()


def linear_plan(lib, rows, in_f, out_f, n, dtype=F16):
    p = LinearPlan()
    st = lib.t3_linear_plan_of(C.byref(arr(dtype, rows, in_f)), C.byref(arr(U16, in_f // 16, out_f // 16, n)),
                               Decode(1, 16), C.byref(p))
    assert st == 0, lib.t3_error_name(st)
    return p


def bank_of(experts, hidden, inter, n_gu, n_dn):
    def proj(i, o, n):
        return Proj(arr(U16, experts, i // 16, o // 16, n), arr(F16, experts, i), arr(F16, experts, o))
    return Bank(proj(hidden, inter, n_gu), proj(hidden, inter, n_gu), proj(inter, hidden, n_dn))


def moe_plan(lib, rows, experts, hidden, inter, topk, n_gu, n_dn, shared=None):
    p = MoePlan()
    bank = bank_of(experts, hidden, inter, n_gu, n_dn)
    st = lib.t3_moe_plan_of(C.byref(arr(BF16, 1, rows, hidden)), C.byref(bank), C.byref(arr(I32, 1, rows, topk)),
                            C.byref(shared) if shared is not None else None, C.byref(p))
    assert st == 0, lib.t3_error_name(st)
    return p


def test_config2_qkv_partition(lib):
    # in 4096, out 12288: K3 and K4 take eight tiles a load (a tile row's 8 x 2n bytes fit one 1 KB load), K5 four;
    # 768 workgroups either way, one launch at one row
    for k, bt, ks in ((3, 8, 8), (4, 8, 8), (5, 4, 4)):
        p = linear_plan(lib, 1, 4096, 12288, 16 * k)
        assert (p.path, p.launches) == (0, 1)
        assert (p.tiles_a_load, p.k_slices, p.workgroups) == (bt, ks, 768), (k, p.tiles_a_load, p.k_slices)
        assert p.tiles_a_wave * 4 * p.k_slices == 4096 // 16
        assert p.code_bytes == (4096 // 16) * (12288 // 16) * 16 * k * 2
    assert linear_plan(lib, 1, 4096, 12288, 64).code_bytes == 25165824


def test_the_k_split_never_depends_on_the_rows(lib):
    for in_f, out_f, n in ((4096, 12288, 64), (4096, 151936, 96), (2048, 2048, 64), (512, 256, 36), (7168, 2048, 32)):
        one = linear_plan(lib, 1, in_f, out_f, n)
        for rows in (2, 3, 4, 5, 16, 17, 32):
            p = linear_plan(lib, rows, in_f, out_f, n)
            assert (p.k_slices, p.tiles_a_load, p.tiles_a_wave) == (one.k_slices, one.tiles_a_load, one.tiles_a_wave)


def test_dense_path_by_rows(lib):
    paths = {rows: linear_plan(lib, rows, 4096, 12288, 64).path for rows in (1, 2, 3, 4, 5, 32, 33, 511)}
    assert paths == {1: 0, 2: 0, 3: 0, 4: 0, 5: 2, 32: 2, 33: 3, 511: 3}
    assert linear_plan(lib, 2, 4096, 12288, 80).path == 0          # above four bits a weight: up to two rows
    assert linear_plan(lib, 3, 4096, 12288, 80).path == 2
    assert linear_plan(lib, 1, 4096, 151936, 96).path == 1         # 64 tiles a wave: prepare launch + arriving GEMV
    assert linear_plan(lib, 1, 4096, 151936, 96).code_bytes == 466747392
    cfg = Config()
    lib.t3_config_default(C.byref(cfg))
    cfg.dec_one = 0
    assert lib.t3_configure(C.byref(cfg)) == 0
    try:
        assert linear_plan(lib, 1, 4096, 12288, 64).path == 2
    finally:
        lib.t3_config_default(C.byref(cfg))
        assert lib.t3_configure(C.byref(cfg)) == 0


def test_few_rows_share_the_tile_rows_out(lib):
    # the trellis GEMM at 64 rows: one item, 56 workgroup columns spread over the dies, eight K parts of sixteen steps
    p = linear_plan(lib, 64, 4096, 14336, 64, BF16)
    assert (p.path, p.launches, p.k_slices) == (3, 3, 8)
    assert p.workgroups == 56 * 8
    q = linear_plan(lib, 300, 4096, 14336, 64, BF16)   # three items: 168 workgroups a part, two parts fit the 512 resident
    assert (q.path, q.k_slices) == (3, 2)
    # from dense_gemm_rows (513) rows the W_hat form serves: decode once, prepare, the f16 GEMM that ends with the finish
    # (or, over few tiles, shares K out and leaves the finish to a launch of its own): five 128-row items or more
    w = linear_plan(lib, 600, 4096, 14336, 64, BF16)
    assert (w.path, w.launches, w.k_slices) == (4, 3, 1)
    assert [linear_plan(lib, r, 4096, 14336, 64, BF16).path for r in (512, 513)] == [3, 4]
    assert [linear_plan(lib, r, 7168, 2048, 48, BF16).path for r in (512, 1024, 4096)] == [3, 4, 4]
    few = linear_plan(lib, 1024, 7168, 2048, 48, BF16)      # 4 x 8 tiles: eight K parts of 28 steps fill the 256 compute units
    assert (few.k_slices, few.launches, few.workgroups) == (8, 4, 256)
    cfg = Config()
    lib.t3_config_default(C.byref(cfg))
    cfg.dense_gemm_rows = 0
    assert lib.t3_configure(C.byref(cfg)) == 0
    try:
        assert linear_plan(lib, 600, 4096, 14336, 64, BF16).k_slices == 1   # kept on the trellis GEMM: five items, 280 workgroups
    finally:
        lib.t3_config_default(C.byref(cfg))
        assert lib.t3_configure(C.byref(cfg)) == 0


def test_config3_routed_partition(lib):
    shared = bank_of(1, 2048, 512, 48, 48)
    for rows in (1, 8, 16):
        p = moe_plan(lib, rows, 512, 2048, 512, 10, 48, 48, shared)
        assert (p.path, p.launches) == (0, 2)
        assert p.row_slots == rows * 11 and p.shared_slots == 1
        # up to four rows the gate|up launch takes four tiles a load (twice the workgroups of half the length); the K
        # partition, and so a row's sums, are the same at every row count
        assert (p.tiles_a_wave_gu, p.k_slices_gu, p.tiles_a_load_gu) == (8, 4, 4 if rows <= 4 else 8)
        assert (p.tiles_a_wave_dn, p.k_slices_dn, p.tiles_a_load_dn) == (8, 1, 8)
        assert p.expert_code_bytes == 1179648
    p = moe_plan(lib, 17, 512, 2048, 512, 10, 48, 48, shared)
    assert (p.path, p.launches) == (3, 9)


def test_down_slices_a_workgroup(lib):
    # a down projection of two K slices (inter 513..1024): one workgroup of eight waves holds both while those workgroups
    # are resident at once (512 of them); 512 experts of 2560 x 640 top-10 have 20 column blocks x 10 r
    plans = [moe_plan(lib, rows, 512, 2560, 640, 10, 48, 48) for rows in (1, 2, 3, 4, 8)]
    assert [p.k_slices_dn for p in plans] == [2] * 5               # the sums' partition does not move
    assert [p.k_slices_a_workgroup_dn for p in plans] == [2, 2, 1, 1, 1]
    # four tiles a load (K5): twice the column workgroups
    assert [moe_plan(lib, rows, 512, 2560, 640, 10, 80, 80).k_slices_a_workgroup_dn for rows in (1, 2)] == [2, 1]
    # one slice, or four: a workgroup a slice
    assert moe_plan(lib, 1, 512, 2048, 512, 10, 48, 48).k_slices_a_workgroup_dn == 1
    assert moe_plan(lib, 1, 64, 4096, 2048, 8, 64, 64).k_slices_a_workgroup_dn == 1


def test_config4_prefill_items(lib):
    p = moe_plan(lib, 2048, 256, 7168, 2048, 8, 32, 48)
    assert p.path == 3 and p.row_slots == 16384
    assert p.item_rows == 96                       # 64 rows an expert on average, 64 + 3 sqrt(64) = 88 within 96
    assert p.max_items == 256 + 16384 // 96
    q = moe_plan(lib, 4096, 256, 7168, 2048, 8, 32, 48)
    assert q.item_rows == 128                      # 128 rows an expert: the full shape
    assert [moe_plan(lib, t, 256, 7168, 2048, 8, 32, 48).item_rows for t in (512, 1024, 1280, 1344)] == [32, 64, 64, 96]
    assert p.expert_code_bytes == 2 * 3670016 + 5505024
    # the cut that leaves no more items an expert than the other (a uniform routing's counts scatter like sqrt(mean)), the
    # 96-row kernel's speed allowed for: 512 experts of 2560 x 640, top-10, at 160 / 120 / 80 / 200 rows an expert
    assert [moe_plan(lib, t, 512, 2560, 640, 10, 64, 64).item_rows for t in (8192, 6144, 4096, 10240)] == [96, 128, 96, 128]


def test_decode_forms_by_configuration(lib):
    cfg = Config()
    # the reference's values (src/core/config.zig:140), each mapped to one of this library's forms
    for form, path, launches in ((3, 2, 5), (7, 2, 5), (8, 1, 4), (5, 4, 6), (6, 4, 6), (9, 0, 2)):
        lib.t3_config_default(C.byref(cfg))
        cfg.decode_form = form
        assert lib.t3_configure(C.byref(cfg)) == 0
        try:
            p = moe_plan(lib, 4, 12, 512, 256, 4, 64, 64)
            assert (p.path, p.launches) == (path, launches)
        finally:
            lib.t3_config_default(C.byref(cfg))
            assert lib.t3_configure(C.byref(cfg)) == 0


def test_decode_form_by_the_gate_up_launch_size(lib):
    # two launches while the gate|up launch stays within 8192 workgroups (column groups x row-slots x 2 x K slices); past
    # that the five launches behind a grouping launch, six in all: 4096 x 2048 K4 top-8 has 16 x 8 r x 2 x 8 = 2048 r
    for rows, launches in ((1, 2), (3, 2), (5, 6), (16, 6)):
        assert moe_plan(lib, rows, 64, 4096, 2048, 8, 64, 64).launches == launches
    # 7168 x 2048 K3 top-8: 16 x 8 r x 2 x 14 = 3584 r
    assert [moe_plan(lib, rows, 256, 7168, 2048, 8, 48, 48).launches for rows in (1, 2, 3)] == [2, 2, 6]
    # four tiles a load (K5) doubles the column groups: 4096 x 1024 has 16 x 8 r x 2 x 8 = 2048 r as well
    assert [moe_plan(lib, rows, 64, 4096, 1024, 8, 80, 80).launches for rows in (3, 5)] == [2, 6]
    # one row of a top-k wide enough to pass the bound has nothing to group: the five launches
    assert moe_plan(lib, 1, 64, 8192, 4096, 32, 64, 64).launches == 5
    # below the bound the grouped form serves where a uniform routing is expected to save more than ~1400 gate|up
    # workgroups: 16 experts of 2048 x 1024, top-4, at 16 rows (4096 workgroups, 15.8 groups of 64 row-slots: 3084 saved),
    # not at 8 (2048, 14.4 of 32: 1126); 64 experts of 4096 x 2048 top-8 at 4 rows (8192, 26.5 of 32: 1412)
    assert [moe_plan(lib, rows, 16, 2048, 1024, 4, 64, 64).launches for rows in (4, 8, 16)] == [2, 2, 6]
    assert moe_plan(lib, 4, 64, 4096, 2048, 8, 64, 64).launches == 6
    assert moe_plan(lib, 16, 128, 2048, 768, 8, 64, 64).launches == 6      # 6144 workgroups, 82 groups of 128: 2200 saved


def test_plan_refusals(lib):
    p = LinearPlan()
    st = lib.t3_linear_plan_of(C.byref(arr(F16, 1, 4000)), C.byref(arr(U16, 256, 768, 64)), Decode(1, 16), C.byref(p))
    assert lib.t3_error_name(st).decode() == "BadExl3Shape"
    st = lib.t3_linear_plan_of(C.byref(arr(F16, 1, 4096)), C.byref(arr(U16, 256, 768, 64)), Decode(1, 16), None)
    assert lib.t3_error_name(st).decode() == "BadArgs"
    m = MoePlan()
    bank = bank_of(8, 512, 256, 64, 64)
    st = lib.t3_moe_plan_of(C.byref(arr(BF16, 1, 2, 512)), C.byref(bank), C.byref(arr(I32, 1, 2, 33)), None, C.byref(m))
    assert st != 0


def test_sizes_beyond_the_launches_arithmetic_are_refused_by_name(lib):
    # widths and row counts past what the launches index (a 16-bit grid dimension over in / 16, 32-bit element offsets over
    # rows x width) refuse before anything is launched or any pointer followed; misaligned arrays are bad arguments
    name = lambda st: lib.t3_error_name(st).decode()
    p = LinearPlan()
    wide_in = 16 * 65536   # in / 16 one past a grid's y
    st = lib.t3_linear_plan_of(C.byref(arr(F16, 1, wide_in)), C.byref(arr(U16, wide_in // 16, 8, 16)), Decode(1, 16), C.byref(p))
    assert name(st) == "Exl3EngineNotImplemented"
    st = lib.t3_linear_plan_of(C.byref(arr(BF16, 1 << 21, 4096)), C.byref(arr(U16, 256, 256, 64)), Decode(1, 16), C.byref(p))
    assert name(st) == "Exl3EngineNotImplemented"   # 2^21 rows x 4096 columns: 2^33 elements
    assert lib.t3_linear_plan_of(C.byref(arr(BF16, 1 << 16, 4096)), C.byref(arr(U16, 256, 256, 64)), Decode(1, 16), C.byref(p)) == 0
    st = lib.t3_dequant(None, C.byref(arr(U16, wide_in // 16, 8, 16)), Decode(1, 16), C.byref(arr(F16, wide_in, 128)))
    assert name(st) == "Exl3EngineNotImplemented"
    odd = arr(U16, 8, 8, 16)
    odd.data = FAKE + 2
    assert name(lib.t3_dequant(None, C.byref(odd), Decode(1, 16), C.byref(arr(F16, 128, 128)))) == "BadArgs"
    bias = arr(F16, 128)
    bias.data = FAKE + 6
    st = lib.t3_linear_bias(None, C.byref(arr(F16, 1, 128)), C.byref(arr(U16, 8, 8, 16)), C.byref(arr(F16, 128)),
                            C.byref(arr(F16, 128)), C.byref(bias), Decode(1, 16), C.byref(arr(F16, 1, 128)), FAKE, 1 << 20)
    assert name(st) == "BadArgs"


def test_configure_publishes_whole_snapshots(lib):
    # a call reads one whole configuration, also while another thread configures: many writers, one reader of plans
    import threading
    stop = threading.Event()

    def writer(rows_alone):
        cfg = Config()
        lib.t3_config_default(C.byref(cfg))
        cfg.dense_rows_alone, cfg.dense_gemm_rows = rows_alone, 513 if rows_alone == 0 else 0
        while not stop.is_set():
            assert lib.t3_configure(C.byref(cfg)) == 0

    threads = [threading.Thread(target=writer, args=(v,)) for v in (0, 1)]
    for t in threads:
        t.start()
    try:
        for _ in range(2000):
            p = linear_plan(lib, 600, 4096, 14336, 64, BF16)
            assert (p.path, p.k_slices) in ((4, 1), (3, 1)), (p.path, p.k_slices)   # never a mix of the two settings
    finally:
        stop.set()
        for t in threads:
            t.join()
        cfg = Config()
        lib.t3_config_default(C.byref(cfg))
        assert lib.t3_configure(C.byref(cfg)) == 0


def test_a_process_that_never_configures_runs_the_defaults():
    """The configuration a library starts with is the one t3_config_default hands out: a fresh process that asks for a
    plan without ever configuring gets the default's paths (the W_hat form only where its GEMM's tiles fill the GPU)."""
    import subprocess
    import sys
    code = (
        "import ctypes as C\n"
        "from tests.test_plans import linear_plan, BF16\n"
        "from turboexl3_amd import _lib\n"
        "lib = _lib.lib()\n"
        "print(linear_plan(lib, 512, 4096, 4096, 64, BF16).path, linear_plan(lib, 600, 4096, 14336, 64, BF16).path)\n"
    )
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, cwd=root, timeout=120)
    assert out.returncode == 0, out.stderr
    assert out.stdout.split() == ["3", "4"]
