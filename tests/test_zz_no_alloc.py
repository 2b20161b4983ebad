"""`sah_sparse_attention_static`, the attention entry point that allocates nothing: through the C ABI against
`sah_sparse_attention` with a caller-provided workspace, on two calls in a row, the second on a smaller input.
Same kernels, same order of sums, so the outputs must agree bit for bit."""
import ctypes as C

import pytest
import torch

from _util import make_qkv

pytestmark = pytest.mark.gpu


def _rows_and_args(N, cuda, B, Hq, Hkv, Lk, D, n_sel, dtype, seed, work, sinks=None, stats=None):
    """A mask of `n_sel` random distinct columns per row in the kernels' layout, and the argument block of an
    attention call over it (out buffer included). `work` = None leaves the workspace fields empty."""
    from sparse_attention_hub_amd.sparse_attention.utils.mask_attention_utils import unit_inverse_weight

    q, k, v = make_qkv(B, Hq, Hkv, 1, Lk, D, dtype, seed=seed, device=cuda)
    n_rows = B * Hq
    g = torch.Generator().manual_seed(seed + 100)
    cols = torch.stack([torch.randperm(Lk, generator=g)[:n_sel] for _ in range(n_rows)]).to(torch.int32).to(cuda)
    cnt = torch.full((n_rows,), n_sel, dtype=torch.int32, device=cuda)
    cnt[0] = n_sel // 3                     # ragged rows: the splits of a short row must still be merged correctly
    bitmap = torch.zeros((n_rows, (Lk + 31) // 32), dtype=torch.int32, device=cuda)
    rows = N.Rows(cols.data_ptr(), cnt.data_ptr(), None, bitmap.data_ptr(), n_rows, n_sel, Lk, (Lk + 31) // 32)
    out = torch.zeros((B, 1, Hq, D), dtype=dtype, device=cuda)
    args = N.AttentionArgs(
        rows,
        q.data_ptr(), q.stride(0), q.stride(1), q.stride(2),
        k.data_ptr(), k.stride(0), k.stride(1), k.stride(2),
        v.data_ptr(), v.stride(0), v.stride(1), v.stride(2),
        None, 0, 0, 0, None if sinks is None else sinks.data_ptr(),
        N.dtype_code(dtype), B, Hq, Hkv, 1, Lk, D,
        float(D ** -0.5), unit_inverse_weight(dtype), 0, 0, 0, 0, n_sel,
        out.data_ptr(),
        None if work is None else work.data_ptr(), 0 if work is None else work.numel(),
        None, None if stats is None else stats.data_ptr(), N.stream_ptr(cuda),
    )
    return args, out, (q, k, v, cols, cnt, bitmap)


def test_static_workspace_entry_point_matches_the_allocating_one(cuda):
    from sparse_attention_hub_amd import _native as N

    lib = N.lib()
    limit = 4 * 1024 * 1024
    shapes = [  # (B, Hq, Hkv, Lk, D, entries per row, dtype): split form (few rows), then a smaller call
        (2, 32, 8, 20000, 128, 5000, torch.bfloat16),
        (1, 8, 2, 3000, 64, 1200, torch.float32),
        (8, 32, 8, 4000, 128, 2688, torch.bfloat16),      # whole-row form: no workspace at all
    ]
    for i, (B, Hq, Hkv, Lk, D, n_sel, dtype) in enumerate(shapes):
        floats = N.work_floats(B * Hq, n_sel, D)
        assert floats <= limit
        assert (floats > 0) == (i < 2)
        work = torch.full((max(floats, 1),), float("nan"), dtype=torch.float32, device=cuda)
        # the second shape also carries sink logits and asks for the (max, denominator) pairs
        sinks = torch.linspace(-0.5, 0.5, Hq, device=cuda) if i == 1 else None
        st1 = torch.zeros((B * Hq, 2), dtype=torch.float32, device=cuda) if i == 1 else None
        st2 = torch.zeros((B * Hq, 2), dtype=torch.float32, device=cuda) if i == 1 else None
        a1, out1, keep1 = _rows_and_args(N, cuda, B, Hq, Hkv, Lk, D, n_sel, dtype, 7 + i, work, sinks, st1)
        a2, out2, keep2 = _rows_and_args(N, cuda, B, Hq, Hkv, Lk, D, n_sel, dtype, 7 + i, None, sinks, st2)
        N.call("sah_sparse_attention", a1)
        if i == 0:
            # the first call on a device looks the built-in buffer's address up; a caller that must not even do that
            # (stream capture) makes one warm-up call first, as here
            N.call("sah_sparse_attention_static", a2)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        allocs_before = torch.cuda.memory_stats()["allocation.all.allocated"]
        N.call("sah_sparse_attention_static", a2)
        torch.cuda.synchronize()
        # what the entry point exists for: no device memory is allocated around the call
        assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == allocs_before
        assert bool(torch.isfinite(out1.float()).all()) and float(out1.float().abs().max()) > 0
        assert torch.equal(out1, out2), f"call {i}: outputs differ"
        if i == 1:
            assert torch.equal(st1, st2) and bool((st1[:, 1] > 0).all())
    # a call that needs more than the built-in buffer is refused before anything is launched
    B, Hq, Hkv, Lk, D, n_sel = 32, 32, 8, 131072, 128, 131072
    assert N.work_floats(B * Hq, n_sel, D) > limit
    n_rows = B * Hq
    cnt = torch.zeros((n_rows,), dtype=torch.int32, device=cuda)
    bitmap = torch.zeros((n_rows, Lk // 32), dtype=torch.int32, device=cuda)
    cols = torch.zeros((n_rows, 8), dtype=torch.int32, device=cuda)
    q = torch.zeros((B, Hq, 1, D), dtype=torch.bfloat16, device=cuda)
    kv = torch.zeros((B, Hkv, 8, D), dtype=torch.bfloat16, device=cuda)   # never read: the call is refused
    out = torch.zeros((B, 1, Hq, D), dtype=torch.bfloat16, device=cuda)
    big = N.AttentionArgs(
        N.Rows(cols.data_ptr(), cnt.data_ptr(), None, bitmap.data_ptr(), n_rows, n_sel, Lk, Lk // 32),
        q.data_ptr(), q.stride(0), q.stride(1), q.stride(2),
        kv.data_ptr(), kv.stride(0), kv.stride(1), kv.stride(2),
        kv.data_ptr(), kv.stride(0), kv.stride(1), kv.stride(2),
        None, 0, 0, 0, None, N.dtype_code(torch.bfloat16), B, Hq, Hkv, 1, Lk, D, 1.0, 1.0, 0, 0, 0, 0, n_sel,
        out.data_ptr(), None, 0, None, None, N.stream_ptr(cuda))
    rc = lib.sah_sparse_attention_static(C.addressof(big))
    assert rc == -4 and b"built-in buffer holds" in lib.sah_last_error()
    assert lib.sah_sparse_attention_static(None) == -2
