"""The C-ABI library loads and exports exactly what include/sah.h declares (no compute)."""
import ctypes
import os
import re

import pytest

from sparse_attention_hub_amd import _native as N

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "sah.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(?:int|int64_t|const char\*)\s+(sah_\w+)\s*\(", text)))


def test_library_is_built_and_loads():
    assert N.library_path().exists(), "build it with python sparse-attention-hub_amd/build.py"
    lib = N.lib()
    assert lib.sah_version() == N.ABI_VERSION == 4


def test_a_library_of_another_layout_generation_is_refused(monkeypatch):
    """The argument structures of another SAH_VERSION would be read past their end: the binding refuses to load."""
    monkeypatch.setattr(N, "_lib", None)
    monkeypatch.setattr(N, "ABI_VERSION", N.ABI_VERSION + 1)
    with pytest.raises(N.NativeLibraryError, match="layout generation"):
        N.lib()
    monkeypatch.undo()
    assert N.lib().sah_version() == N.ABI_VERSION


def test_every_declared_symbol_is_exported_and_bound():
    declared = _declared_functions()
    assert len(declared) >= 15
    handle = ctypes.CDLL(str(N.library_path()))
    for name in declared:
        assert hasattr(handle, name), f"{name} declared in include/sah.h but not exported"
    assert sorted(N.EXPECTED_SYMBOLS) == declared


def test_argument_errors_are_reported_without_a_gpu():
    # NULL args never launch anything; the error string names the entry point
    lib = N.lib()
    assert lib.sah_sparse_attention(None) == -2
    assert b"sah_sparse_attention" in lib.sah_last_error()
    assert lib.sah_select_topk(None) == -2
    # whole rows per workgroup (many short rows): no workspace; few or long rows: (m, l, acc[D]) per split
    assert N.work_floats(256, 2688, 128) == 0
    # split form: rows x splits x (D + 2) floats, where the library chooses the split count: never more than 64
    # splits, never more splits than 256-key chunks, no tile of a longest row beyond 11 chunks, and enough
    # workgroups to cover the chip while the row still has chunks to hand out
    for n_rows, max_cnt, D in ((128, 2278, 128), (512, 131072, 128), (64, 2688, 64), (32, 1500, 128), (1, 70000, 128)):
        floats = N.work_floats(n_rows, max_cnt, D)
        # fewer rows than compute units: also room for the one-kernel selection + attention, which gives a row
        # min(8, 256 // rows) workgroups - their partial results
        parts = min(8, 256 // n_rows) if n_rows < 192 else 1
        fused = n_rows * parts * (D + 2) if parts > 1 else 0
        assert floats >= fused
        if floats == fused:
            continue
        assert floats > 0 and floats % (n_rows * (D + 2)) == 0
        n_split = floats // (n_rows * (D + 2))
        chunks = -(-max_cnt // 256)
        assert 1 <= n_split <= min(64, chunks)
        assert -(-chunks // n_split) <= 11 or n_split == 64
        assert n_rows * n_split >= 2048 or 2 * n_split > min(64, chunks)
    assert N.work_floats(32, 300, 128) == 32 * 8 * 130  # short rows: whole-row form, or the one-kernel form
    assert N.work_floats(0, 100, 128) == 0 and N.work_floats(16, 100, 0) == 0
    for fn in ("sah_hash_decode_topk", "sah_adaptive_budget", "sah_adaptive_sample", "sah_pq_adc_scores"):
        assert getattr(lib, fn)(None) == -2 and fn.encode() in lib.sah_last_error()
    assert lib.sah_pq_adc_lut_bytes(4, 32, 8, 1, 16, 256, 1) == 4 * 8 * 1 * 16 * 256 * 8


def test_struct_layouts_match_header_sizes():
    # sah_rows: 4 pointers + 4 int32
    assert ctypes.sizeof(N.Rows) == 4 * 8 + 4 * 4
    assert ctypes.sizeof(N.SinkLocalArgs) == ctypes.sizeof(N.Rows) + 5 * 4 + 4 + 8


def test_every_entry_point_refuses_null_and_names_itself():
    """Every `int sah_*(const args*)` entry point checks its argument block before touching the device."""
    lib = N.lib()
    one_arg = ["sah_sink_local_indices", "sah_rows_from_dense", "sah_rows_to_dense", "sah_hash_signatures", "sah_hamming_topk",
               "sah_hamming_scores", "sah_qk_scores", "sah_select_topk", "sah_pq_keys_absmax", "sah_pq_kmeans_assign",
               "sah_pq_kmeans_update", "sah_pq_adc_scores", "sah_sparse_attention", "sah_sparse_attention_static",
               "sah_attention_weights", "sah_adaptive_budget", "sah_adaptive_sample", "sah_hash_decode_topk",
               "sah_hash_compact_codes", "sah_run_chain", "sah_amask_classify"]
    for fn in one_arg:
        assert getattr(lib, fn)(None) == -2, fn
        assert fn.replace("_static", "").encode() in lib.sah_last_error() or fn.encode() in lib.sah_last_error(), fn
    assert lib.sah_hash_signatures_pair(None, None) == -2
    assert lib.sah_hash_decode_attention(None, None, None) == -2
    assert lib.sah_select_topk_attention(None, None, None) == -2
    # whatever takes an argument block is in one of the two lists above
    plain = {"sah_version", "sah_last_error", "sah_timing_enable", "sah_timing_collect", "sah_pq_adc_lut_bytes",
             "sah_sparse_attention_work_floats"}
    assert set(one_arg) | {"sah_hash_signatures_pair", "sah_hash_decode_attention", "sah_select_topk_attention"} | plain == set(_declared_functions())


def test_bad_argument_blocks_are_refused_with_the_documented_codes():
    """Validation happens on the host, before any launch: the codes of include/sah.h (no GPU needed)."""
    lib = N.lib()
    buf = ctypes.create_string_buffer(4096)          # stands for device memory: never dereferenced by the checks
    ptr = ctypes.addressof(buf)

    def rows(n_rows=4, n_keys=100, cap=16, n_words=None):
        return N.Rows(ptr, ptr, None, ptr, n_rows, cap, n_keys, (n_keys + 31) // 32 if n_words is None else n_words)

    # rows: empty, inconsistent bitmap width, missing arrays
    a = N.SinkLocalArgs(rows(n_rows=0), 1, 4, 4, 1, 0, None)
    assert lib.sah_sink_local_indices(ctypes.byref(a)) == -1
    a = N.SinkLocalArgs(rows(n_words=1), 1, 4, 4, 1, 0, None)
    assert lib.sah_sink_local_indices(ctypes.byref(a)) == -1 and b"n_words" in lib.sah_last_error()
    r = rows()
    r.cnt = None
    a = N.SinkLocalArgs(r, 1, 4, 4, 1, 0, None)
    assert lib.sah_sink_local_indices(ctypes.byref(a)) == -2
    # selection: key width other than 16 / 32 bits, capacity below active + k
    sel = N.SelectTopkArgs(rows(), ptr, 104, 8, 100, 0, 5, 0, 0, 0, 0, None)
    assert lib.sah_select_topk(ctypes.byref(sel)) < 0 and b"sah_select_topk" in lib.sah_last_error()
    sel = N.SelectTopkArgs(rows(cap=6), ptr, 104, 16, 100, 0, 50, 0, 1, 4, 4, None)   # fresh rows: sink + window do not fit
    assert lib.sah_select_topk(ctypes.byref(sel)) == -4
    sel = N.SelectTopkArgs(rows(), ptr, 104, 16, 100, 50, 5, 0, 0, 0, 0, None)         # candidates beyond the row
    assert lib.sah_select_topk(ctypes.byref(sel)) == -1
    sel = N.SelectTopkArgs(rows(), ptr, 96, 16, 100, 0, 5, 0, 0, 0, 0, None)           # key rows shorter than the candidates
    assert lib.sah_select_topk(ctypes.byref(sel)) == -1
    # what the no-allocation attention refuses is more than its built-in buffer holds
    assert N.work_floats(1024, 131072, 128) > 4 * 1024 * 1024 >= N.work_floats(512, 131072, 128)
    # the remainders of a scoring pass: 16-bit scores only
    al = (ptr + 63) // 64 * 64
    qk = N.QkScoresArgs(al, 128, 128, 128, al, 128, 128, 128, None, 0, 0, 0, 0, 1, 1, 1, 1, 8, 128, al, 64, None, al)
    assert lib.sah_qk_scores(ctypes.byref(qk)) == -1 and b"resid_out" in lib.sah_last_error()
    # additive-mask classification: empty shape, too many rows, unknown dtype
    amc = N.AmaskClassifyArgs(ptr, 0, 0, 0, 1, 2, 1, 1, 0, ptr, None)
    assert lib.sah_amask_classify(ctypes.byref(amc)) == -1
    amc = N.AmaskClassifyArgs(ptr, 0, 0, 0, 1, 70000, 1, 1, 8, ptr, None)
    assert lib.sah_amask_classify(ctypes.byref(amc)) == -3
    amc = N.AmaskClassifyArgs(ptr, 0, 0, 0, 1, 2, 1, 1, 8, None, None)
    assert lib.sah_amask_classify(ctypes.byref(amc)) == -2
