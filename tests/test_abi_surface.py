"""CPU-side checks of the C ABI: the library loads, exports every symbol include/turboexl3_hip.h declares,
and its host-only entry points (names, admission rules, configuration) behave as the reference's do.
No kernel runs here."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from turboexl3_amd import _lib, build
    if not os.path.exists(_lib.LIB_PATH):
        build.build()
    return _lib.lib()


def test_every_declared_symbol_is_exported_and_bound(lib):
    from turboexl3_amd import _lib
    header = open(os.path.join(ROOT, "include", "turboexl3_hip.h")).read()
    declared = set(re.findall(r"\b(t3_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found"
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert declared == set(_lib.SYMBOLS), declared ^ set(_lib.SYMBOLS)


def test_error_names_are_the_reference_names(lib):
    from turboexl3_amd import _lib
    for status, name in enumerate(_lib.STATUS_NAMES):
        assert lib.t3_error_name(status).decode() == name
    assert lib.t3_error_name(999).decode() == "UnknownStatus"


def test_rate_topk_and_trellis_admission(lib):
    # src/core/format.zig:96-100, src/core/spec.zig:75-88
    assert [n for n in range(10, 140) if lib.t3_rate_admitted(n)] == list(range(16, 130, 2))
    assert lib.t3_admit_topk(32) == 0
    assert lib.t3_error_name(lib.t3_admit_topk(33)).decode() == "Exl3TopKExceedsReduceBank"
    shape = (C.c_int64 * 4)(8, 160, 40, 64)
    assert lib.t3_trellis_admitted(shape, 4, 8, 2560, 640, 64) == 1
    assert lib.t3_trellis_admitted(shape, 4, 8, 2560, 640, 48) == 0      # over the config's rate
    assert lib.t3_trellis_admitted(shape, 4, 8, 2560, 640, 80) == 1      # under it
    assert lib.t3_trellis_admitted(shape, 3, 8, 2560, 640, 64) == 0
    assert lib.t3_trellis_admitted(shape, 4, 9, 2560, 640, 64) == 0
    odd = (C.c_int64 * 4)(8, 160, 40, 63)
    assert lib.t3_trellis_admitted(odd, 4, 8, 2560, 640, 64) == 0


def test_configure_refuses_unserved_values(lib):
    from turboexl3_amd._lib import Config
    cfg = Config()
    lib.t3_config_default(C.byref(cfg))
    assert (cfg.decode_form, cfg.dec_one, cfg.prefill, cfg.mcg_pair, cfg.mul1_defer, cfg.dense_gemm_rows,
            cfg.dense_rows_alone) == (9, 1, 1, 0, 1, 513, 0)
    # src/core/config.zig:191-192,245: 3, 5, 6, 7, 8 and 9 are served, 0, 4 and 10 refused
    for form in (0, 4, 10):
        cfg.decode_form = form
        assert lib.t3_error_name(lib.t3_configure(C.byref(cfg))).decode() == "InvalidTurboexl3Config"
    for form in (3, 5, 6, 7, 8, 9):
        cfg.decode_form = form
        assert lib.t3_configure(C.byref(cfg)) == 0
    cfg.decode_form, cfg.dense_gemm_rows = 9, -1
    assert lib.t3_error_name(lib.t3_configure(C.byref(cfg))).decode() == "InvalidTurboexl3Config"
    cfg.dense_gemm_rows = 513
    cfg.decode_form = 3
    assert lib.t3_configure(C.byref(cfg)) == 0
    cfg.decode_form = 9
    cfg.dec_one = 2
    assert lib.t3_error_name(lib.t3_configure(C.byref(cfg))).decode() == "InvalidTurboexl3Config"
    lib.t3_config_default(C.byref(cfg))
    assert lib.t3_configure(C.byref(cfg)) == 0


def test_null_arguments_are_bad_args(lib):
    from turboexl3_amd._lib import Decode
    need = C.c_size_t(0)
    assert lib.t3_error_name(lib.t3_linear_workspace_bytes(None, None, Decode(1, 16), C.byref(need))).decode() == "BadArgs"
    assert lib.t3_error_name(lib.t3_test_codebooks(None, None, None, None)).decode() == "BadArgs"


def test_hand_written_wide_stores_keep_their_wait_states():
    """A vector-memory store of more than 64 bits reads its data registers over several cycles; the compiler keeps two
    wait states between such a store and a vector write of those registers for its own stores, not for one inside an
    `asm` statement. Every hand-written wide store in the kernels carries them in the same statement."""
    src = os.path.join(ROOT, "turboexl3_amd", "csrc")
    wide = re.compile(r"(global|buffer|flat)_store_(dwordx[34]|b96|b128)")
    found = 0
    for name in sorted(os.listdir(src)):
        text = open(os.path.join(src, name)).read()
        for m in re.finditer(r"\basm\b[^;]*?\(([^;]*?)\)\s*;", text, re.S):
            body = m.group(1)
            if wide.search(body):
                found += 1
                assert re.search(r"_store_\w+[^\"]*\\n\\ts_nop [1-9]", body), f"{name}: a wide store without wait states behind it"
    assert found >= 1  # store_coherent4 (t3_common.hpp)
