"""Device buffers of the kernels' sparse-mask layout (see include/sah.h, `sah_rows`).

One row per (batch, query head, query position):
    cols   int32 [n_rows, cap]      active key columns, unordered
    cnt    int32 [n_rows]           valid entries per row
    w      float32 [n_rows, cap]    entry weights, or None when every weight is 1.0
    bitmap int32 [n_rows, n_words]  bit j set <=> column j active
The host keeps `max_cnt`, an upper bound of every cnt[r] that is known without
reading device memory, and `uniform_cnt` when every row is known to hold exactly
that many entries (true for Sink/Local/top-k chains), so that neither capacity
planning nor the conversion to the reference's indices/ptr form needs a device
synchronisation.
"""
from __future__ import annotations

from typing import Optional

import torch

from ... import _native as N


class NativeRows:
    __slots__ = (
        "cols", "cnt", "w", "bitmap", "n_rows", "cap", "n_keys", "n_words",
        "max_cnt", "uniform_cnt", "fresh", "device",
    )

    def __init__(self, n_rows: int, n_keys: int, cap: int, device: torch.device, weighted: bool = False):
        if n_rows <= 0 or n_keys <= 0:
            raise ValueError(f"rows need positive dimensions, got n_rows={n_rows}, n_keys={n_keys}")
        cap = max(1, min(int(cap), n_keys))
        self.n_rows = n_rows
        self.n_keys = n_keys
        self.n_words = (n_keys + 31) // 32
        self.cap = cap
        self.device = device
        self.cols = torch.empty((n_rows, cap), dtype=torch.int32, device=device)
        self.cnt = torch.empty((n_rows,), dtype=torch.int32, device=device)
        self.bitmap = torch.empty((n_rows, self.n_words), dtype=torch.int32, device=device)
        self.w: Optional[torch.Tensor] = (
            torch.empty((n_rows, cap), dtype=torch.float32, device=device) if weighted else None
        )
        self.max_cnt = 0
        self.uniform_cnt: Optional[int] = 0
        # cnt and bitmap hold garbage until a kernel initialises them (fresh rows = empty mask)
        self.fresh = True

    # -- state ---------------------------------------------------------------
    def zero_if_fresh(self) -> None:
        """Make fresh rows a valid empty mask for kernels that cannot initialise them."""
        if self.fresh:
            self.cnt.zero_()
            self.bitmap.zero_()
            self.fresh = False

    def note_added(self, per_row: int, exact: bool) -> None:
        """Record that a kernel appended at most (`exact`: exactly) `per_row` entries per row."""
        self.max_cnt = min(self.n_keys, self.max_cnt + per_row)
        if exact and self.uniform_cnt is not None:
            self.uniform_cnt = self.uniform_cnt + per_row
        else:
            self.uniform_cnt = None
        self.fresh = False

    def reserve(self, extra: int) -> None:
        """Ensure room for `extra` more entries in every row (copies the lists when growing)."""
        need = min(self.n_keys, self.max_cnt + int(extra))
        if need <= self.cap:
            return
        new_cap = need
        cols = torch.empty((self.n_rows, new_cap), dtype=torch.int32, device=self.device)
        if not self.fresh and self.max_cnt > 0:
            cols[:, : self.max_cnt] = self.cols[:, : self.max_cnt]
        self.cols = cols
        if self.w is not None:
            w = torch.empty((self.n_rows, new_cap), dtype=torch.float32, device=self.device)
            if not self.fresh and self.max_cnt > 0:
                w[:, : self.max_cnt] = self.w[:, : self.max_cnt]
            self.w = w
        self.cap = new_cap

    def make_weighted(self) -> None:
        """Attach a weight array (ones for the existing entries)."""
        if self.w is None:
            self.w = torch.ones((self.n_rows, self.cap), dtype=torch.float32, device=self.device)

    def clone(self) -> "NativeRows":
        other = NativeRows.__new__(NativeRows)
        for name in self.__slots__:
            val = getattr(self, name)
            setattr(other, name, val.clone() if isinstance(val, torch.Tensor) else val)
        return other

    # -- FFI -------------------------------------------------------------------
    def as_struct(self) -> N.Rows:
        return N.Rows(
            self.cols.data_ptr(),
            self.cnt.data_ptr(),
            None if self.w is None else self.w.data_ptr(),
            self.bitmap.data_ptr(),
            self.n_rows,
            self.cap,
            self.n_keys,
            self.n_words,
        )

    # -- conversions (plumbing, not on the decode path) ---------------------------
    def sorted_entries(self):
        """(cols_sorted int64 [R,cap], weights [R,cap] or None, cnt int64 [R]) with padding pushed right."""
        self.zero_if_fresh()
        cnt = self.cnt.to(torch.int64).clamp_(max=self.cap)
        pos = torch.arange(self.cap, device=self.device).unsqueeze(0)
        valid = pos < cnt.unsqueeze(1)
        big = torch.full_like(self.cols, self.n_keys)
        keyed = torch.where(valid, self.cols, big).to(torch.int64)
        order = torch.argsort(keyed, dim=1, stable=True)
        cols_sorted = torch.gather(keyed, 1, order)
        w_sorted = None if self.w is None else torch.gather(self.w, 1, order)
        return cols_sorted, w_sorted, cnt
