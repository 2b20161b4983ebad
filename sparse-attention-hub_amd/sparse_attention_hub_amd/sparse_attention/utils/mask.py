"""`Mask`: the attention-mask value type of the ResearchAttention path.

Same public surface as the reference `Mask` (sparse_attention/utils/mask.py:10-1077):
a mask over a tensor of shape (..., n) whose entries are *weights* (0 = inactive,
w > 0 = active with inclusion probability w) held in one of these forms

  * empty  (`is_empty`)  — no masker has run; consumers treat it as "no masking";
  * full   (`is_full`)   — every entry 1.0;
  * dense  (`from_dense_mask`, `.mask`);
  * index  (`from_index`, `.indices` flat int64 row*n+col, `.ptr` int64 rows+1,
            `.data` weights or None meaning 1.0);
  * rows   (`from_rows`, `.rows`) — the kernels' own layout (NativeRows: int32
            column lists + counts + membership bitmap), which is what the
            MI355X maskers produce and the attention kernel consumes.

The dense and index forms are plain tensor containers (torch indexing, any
device); they exist so that callers written against the reference keep working
and are never touched on the decode path, where the chain stays in rows form.
"""
from __future__ import annotations

import warnings
from typing import Literal, Optional, Tuple

import numpy as np
import torch

from ... import _native as N
from .native_rows import NativeRows


def _numel(shape: Tuple[int, ...]) -> int:
    return int(np.prod(shape)) if len(shape) else 1


class Mask:
    def __init__(
        self,
        shape: Tuple[int, ...],
        dtype: torch.dtype,
        device: torch.device,
        mask: Optional[torch.Tensor] = None,
        indices: Optional[torch.Tensor] = None,
        ptr: Optional[torch.Tensor] = None,
        data: Optional[torch.Tensor] = None,
        from_dense_mask: bool = False,
        from_index: bool = False,
        is_full: bool = False,
        is_empty: bool = False,
        rows: Optional[NativeRows] = None,
    ):
        self.shape = tuple(shape)
        self.dtype = dtype
        self.device = device
        self.from_dense_mask = False
        self.from_index = False
        self.from_rows = False
        self.is_full = False
        self.is_empty = False
        self.mask: Optional[torch.Tensor] = None
        self.indices: Optional[torch.Tensor] = None
        self.ptr: Optional[torch.Tensor] = None
        self.data: Optional[torch.Tensor] = None
        self.rows: Optional[NativeRows] = None

        if is_full or is_empty:
            if device is None:
                raise ValueError("device must be specified for full masks" if is_full else "device must be specified for empty masks")
            self.is_full, self.is_empty = bool(is_full), bool(is_empty) and not is_full
        elif rows is not None:
            self.rows = rows
            self.from_rows = True
            self.device = rows.device
        elif from_dense_mask and mask is not None:
            self.mask = mask.to(dtype)
            self.device = mask.device
            self.from_dense_mask = True
        elif from_index and indices is not None and ptr is not None:
            self.indices, self.ptr, self.data = indices, ptr, data
            self.device = indices.device
            self.from_index = True
        else:
            raise ValueError(
                "Must specify either from_dense_mask with mask, from_index with indices and ptr, is_full=True, or is_empty=True"
            )

    # ------------------------------------------------------------------ state
    def _become(self, other: "Mask") -> "Mask":
        for name in ("from_dense_mask", "from_index", "from_rows", "is_full", "is_empty",
                     "mask", "indices", "ptr", "data", "rows", "device"):
            setattr(self, name, getattr(other, name))
        return self

    def _detect_full_mask(self, only_check_flag: bool = True) -> bool:
        if self.is_full:
            return True
        if self.is_empty or only_check_flag:
            return False
        if self.from_dense_mask:
            return bool(torch.all(self.mask == 1.0).item())
        if self.from_index:
            if self.indices.numel() != _numel(self.shape):
                return False
            return True if self.data is None else bool(torch.all(self.data == 1.0).item())
        if self.from_rows:
            return bool(torch.all(self.get_dense_mask() == 1.0).item())
        return False

    def _detect_empty_mask(self, only_check_flag: bool = True) -> bool:
        if self.is_empty:
            return True
        if self.is_full or only_check_flag:
            return False
        if self.from_dense_mask:
            return bool(torch.all(self.mask == 0.0).item())
        if self.from_index:
            return int(self.indices.numel()) == 0
        if self.from_rows:
            self.rows.zero_if_fresh()
            return bool((self.rows.cnt == 0).all().item())
        return False

    def is_full_mask(self) -> bool:
        return self.is_full

    def is_empty_mask(self) -> bool:
        return self.is_empty

    def __repr__(self) -> str:
        return (
            f"Mask(shape={self.shape}, dtype={self.dtype}, from_dense_mask={self.from_dense_mask}, "
            f"from_index={self.from_index}, from_rows={self.from_rows}, is_full={self.is_full}, is_empty={self.is_empty})"
        )

    # ----------------------------------------------------------- constructors
    @classmethod
    def create_empty_mask(cls, shape, dtype: torch.dtype, device: torch.device) -> "Mask":
        return cls(shape=shape, dtype=dtype, device=device, is_empty=True)

    @classmethod
    def create_full_mask(cls, shape, dtype: torch.dtype, device: torch.device) -> "Mask":
        return cls(shape=shape, dtype=dtype, device=device, is_full=True)

    @classmethod
    def create_mask_from_rows(cls, shape, rows: NativeRows, dtype: torch.dtype) -> "Mask":
        """Wrap kernel-layout rows; `shape` is (..., n_keys) with prod(shape[:-1]) == rows.n_rows."""
        if _numel(shape[:-1]) != rows.n_rows or shape[-1] != rows.n_keys:
            raise ValueError(f"rows ({rows.n_rows} x {rows.n_keys}) do not match mask shape {tuple(shape)}")
        return cls(shape=shape, dtype=dtype, device=rows.device, rows=rows)

    @classmethod
    def create_mask_from_indices(cls, shape, indices: torch.Tensor, ptr: torch.Tensor,
                                 data: Optional[torch.Tensor], dtype: torch.dtype) -> "Mask":
        expected = _numel(shape[:-1]) + 1
        if ptr.numel() != expected:
            raise ValueError(f"ptr.numel() must be {expected}, got {ptr.numel()}")
        return cls(shape=shape, dtype=dtype, device=indices.device, indices=indices, ptr=ptr, data=data, from_index=True)

    @classmethod
    def create_mask_from_dense_mask(cls, shape, mask: torch.Tensor, dtype: torch.dtype) -> "Mask":
        if tuple(mask.shape) != tuple(shape):
            raise ValueError(f"mask.shape must be {tuple(shape)}, got {tuple(mask.shape)}")
        return cls(shape=shape, dtype=dtype, device=mask.device, mask=mask, from_dense_mask=True)

    @classmethod
    def create_from_row_wise_idx(cls, shape, row_wise_idx: torch.Tensor, data: torch.Tensor,
                                 mask_type: Literal["index", "dense"], dtype: torch.dtype,
                                 use_padding: bool = False, mode: Literal["sparse", "dense"] = "dense") -> "Mask":
        if mode == "sparse":
            if mask_type == "dense":
                warnings.warn("Creating dense mask in sparse mode is SLOW. Unless you know what you are doing, use dense mode instead.",
                              UserWarning, stacklevel=2)
            return cls.create_from_row_wise_idx_sparse(shape, row_wise_idx, data, mask_type, dtype, use_padding)
        if mode == "dense":
            if mask_type == "index":
                warnings.warn("Creating index mask in dense mode is SLOW. Unless you know what you are doing, use sparse mode instead.",
                              UserWarning, stacklevel=2)
            return cls.create_from_row_wise_idx_dense(shape, row_wise_idx, data, mask_type, dtype, use_padding)
        raise ValueError(f"Invalid mode: {mode}")

    @staticmethod
    def _check_row_wise(shape, row_wise_idx: torch.Tensor, data: torch.Tensor) -> None:
        if len(shape) < 1:
            raise ValueError("shape must have at least one dimension")
        if row_wise_idx.shape[-1] <= 0:
            raise ValueError("row_wise_idx must have at least one column")
        want = tuple(shape[:-1]) + (row_wise_idx.shape[-1],)
        if tuple(row_wise_idx.shape) != want:
            raise ValueError(f"row_wise_idx.shape must be {want}, got {tuple(row_wise_idx.shape)}")
        if data.shape != row_wise_idx.shape:
            raise ValueError(f"data.shape must match row_wise_idx.shape {tuple(row_wise_idx.shape)}, got {tuple(data.shape)}")

    @classmethod
    def create_from_row_wise_idx_dense(cls, shape, row_wise_idx, data, mask_type, dtype, use_padding: bool = False) -> "Mask":
        cls._check_row_wise(shape, row_wise_idx, data)
        assert not use_padding, "use_padding is not supported for dense mode; use sparse mode instead"
        if mask_type not in ("dense", "index"):
            raise ValueError(f"type must be 'index' or 'dense', got {mask_type}")
        dense = torch.zeros(tuple(shape), dtype=dtype, device=row_wise_idx.device)
        dense.scatter_(-1, row_wise_idx, data.to(dtype))  # duplicates: last write wins
        return cls.create_mask_from_dense_mask(shape, dense, dtype=dtype)

    @classmethod
    def create_from_row_wise_idx_sparse(cls, shape, row_wise_idx, data, mask_type, dtype, use_padding: bool = False) -> "Mask":
        cls._check_row_wise(shape, row_wise_idx, data)
        if mask_type not in ("dense", "index"):
            raise ValueError(f"type must be 'index' or 'dense', got {mask_type}")
        n = shape[-1]
        n_rows = _numel(shape[:-1])
        k = row_wise_idx.shape[-1]
        idx = row_wise_idx.reshape(n_rows, k)
        val = data.reshape(n_rows, k)
        dev = idx.device
        flat = idx + torch.arange(n_rows, device=dev).unsqueeze(1) * n
        if use_padding:
            keep = idx >= 0
            indices = flat[keep]
            values = val[keep]
            ptr = torch.zeros(n_rows + 1, dtype=torch.long, device=dev)
            ptr[1:] = torch.cumsum(keep.sum(dim=1), dim=0)
        else:
            indices = flat.reshape(-1)
            values = val.reshape(-1)
            ptr = torch.arange(0, n_rows * k + 1, k, dtype=torch.long, device=dev)
        sparse = cls.create_mask_from_indices(shape, indices, ptr, values, dtype=dtype)
        if mask_type == "dense":
            return cls.create_mask_from_dense_mask(shape, sparse.get_dense_mask(), dtype=dtype)
        return sparse

    # ------------------------------------------------------------ conversions
    def get_index_mask(self) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """(indices, ptr, data): flat int64 indices (ascending inside a row), row pointers, weights."""
        n_rows = _numel(self.shape[:-1])
        n = self.shape[-1]
        dev = self.device
        if self.is_full:
            total = n_rows * n
            return (torch.arange(total, dtype=torch.long, device=dev),
                    torch.arange(0, total + 1, n, dtype=torch.long, device=dev),
                    torch.ones(total, dtype=self.dtype, device=dev))
        if self.is_empty:
            return (torch.empty(0, dtype=torch.long, device=dev),
                    torch.zeros(n_rows + 1, dtype=torch.long, device=dev),
                    torch.empty(0, dtype=self.dtype, device=dev))
        if self.from_index:
            if self.indices is None or self.ptr is None:
                raise RuntimeError("Sparse mask indices or ptr is None")
            data = self.data if self.data is not None else torch.ones(self.indices.numel(), dtype=self.dtype, device=self.indices.device)
            return self.indices, self.ptr, data
        if self.from_dense_mask:
            if self.mask is None:
                raise RuntimeError("Dense mask is None")
            flat = self.mask.reshape(-1)
            indices = torch.nonzero(flat, as_tuple=False).squeeze(-1)
            ptr = torch.zeros(n_rows + 1, dtype=torch.long, device=flat.device)
            ptr[1:] = torch.cumsum(torch.count_nonzero(self.mask.reshape(n_rows, n), dim=1), dim=0)
            return indices, ptr, flat[indices]
        if self.from_rows:
            rows = self.rows
            cols, w, cnt = rows.sorted_entries()
            base = torch.arange(n_rows, device=dev, dtype=torch.long).unsqueeze(1) * n
            if rows.uniform_cnt is not None:
                u = rows.uniform_cnt
                indices = (cols[:, :u] + base).reshape(-1)
                ptr = torch.arange(0, n_rows * u + 1, max(u, 1), dtype=torch.long, device=dev) if u > 0 else torch.zeros(n_rows + 1, dtype=torch.long, device=dev)
                data = torch.ones(n_rows * u, dtype=self.dtype, device=dev) if w is None else w[:, :u].reshape(-1).to(self.dtype)
                return indices, ptr, data
            valid = torch.arange(rows.cap, device=dev).unsqueeze(0) < cnt.unsqueeze(1)
            indices = (cols + base)[valid]
            ptr = torch.zeros(n_rows + 1, dtype=torch.long, device=dev)
            ptr[1:] = torch.cumsum(cnt, dim=0)
            data = torch.ones(indices.numel(), dtype=self.dtype, device=dev) if w is None else w[valid].to(self.dtype)
            return indices, ptr, data
        raise RuntimeError("Mask object is in an invalid state")

    def get_dense_mask(self) -> torch.Tensor:
        if self.is_full:
            return torch.ones(self.shape, dtype=self.dtype, device=self.device)
        if self.is_empty:
            return torch.zeros(self.shape, dtype=self.dtype, device=self.device)
        if self.from_dense_mask:
            if self.mask is None:
                raise RuntimeError("Dense mask is None")
            return self.mask
        if self.from_index:
            if self.indices is None or self.ptr is None:
                raise RuntimeError("Sparse mask indices or ptr is None")
            dense = torch.zeros(self.shape, dtype=self.dtype, device=self.indices.device)
            if self.indices.numel() > 0:
                dense.view(-1)[self.indices] = 1.0 if self.data is None else self.data.to(self.dtype)
            return dense
        if self.from_rows:
            rows = self.rows
            rows.zero_if_fresh()
            dense = torch.zeros(self.shape, dtype=self.dtype, device=rows.device)
            args = N.DenseRowsArgs(rows.as_struct(), dense.data_ptr(), N.dtype_code(self.dtype), N.stream_ptr(rows.device))
            N.call("sah_rows_to_dense", args)
            return dense
        raise RuntimeError("Mask object is in an invalid state")

    def to_rows(self, extra: int = 0, weighted: Optional[bool] = None) -> NativeRows:
        """Kernel-layout rows of this mask with room for `extra` more entries per row.

        Rows-form masks hand out their own buffers (later kernels extend them in
        place, as the reference's maskers mutate the dense tensor they alias,
        utils/mask.py:591-594); other forms are converted with sah_rows_from_dense.
        """
        n = self.shape[-1]
        n_rows = _numel(self.shape[:-1])
        if self.is_full:
            raise ValueError("a full mask has no row form; callers short-circuit on is_full_mask()")
        if self.from_rows:
            rows = self.rows
            rows.reserve(extra)
            if weighted:
                rows.zero_if_fresh()
                rows.make_weighted()
            return rows
        if self.is_empty:
            return NativeRows(n_rows, n, max(1, extra), self.device, weighted=bool(weighted))
        dense = self.get_dense_mask().reshape(n_rows, n).contiguous()
        N.require_device(dense, "mask")
        nz = dense != 0
        population = int(nz.sum(dim=1).max().item())
        has_weights = bool((nz & (dense != 1)).any().item()) or bool(weighted)
        rows = NativeRows(n_rows, n, max(1, population + extra), dense.device, weighted=has_weights)
        args = N.DenseRowsArgs(rows.as_struct(), dense.data_ptr(), N.dtype_code(dense.dtype), N.stream_ptr(dense.device))
        N.call("sah_rows_from_dense", args)
        rows.fresh = False
        rows.max_cnt = population
        rows.uniform_cnt = None
        return rows

    # ------------------------------------------------------------- apply mask
    def _check_input(self, input_tensor: torch.Tensor) -> None:
        if tuple(input_tensor.shape) != self.shape:
            raise ValueError(f"input_tensor.shape must be {self.shape}, got {tuple(input_tensor.shape)}")

    def apply_mask(self, input_tensor: torch.Tensor, mode: Literal["sparse", "dense"] = "dense") -> torch.Tensor:
        if mode == "sparse":
            return self.apply_mask_sparse(input_tensor)
        if mode == "dense":
            return self.apply_mask_dense(input_tensor)
        raise ValueError(f"Invalid mode: {mode}")

    def apply_mask_dense(self, input_tensor: torch.Tensor) -> torch.Tensor:
        self._check_input(input_tensor)
        if self.is_full or self.is_empty:
            return input_tensor
        return input_tensor * self.get_dense_mask()

    def apply_mask_sparse(self, input_tensor: torch.Tensor) -> torch.Tensor:
        self._check_input(input_tensor)
        if self.is_full or self.is_empty:
            return input_tensor
        indices, _, data = self.get_index_mask()
        out = torch.zeros_like(input_tensor)
        if indices.numel() > 0:
            out.view(-1)[indices] = input_tensor.reshape(-1)[indices] * data
        return out

    def apply_inv_mask(self, input_tensor: torch.Tensor, mode: Literal["sparse", "dense"] = "dense") -> torch.Tensor:
        if mode == "sparse":
            return self.apply_inv_mask_sparse(input_tensor)
        if mode == "dense":
            return self.apply_inv_mask_dense(input_tensor)
        raise ValueError(f"Invalid mode: {mode}")

    def apply_inv_mask_dense(self, input_tensor: torch.Tensor) -> torch.Tensor:
        """x * 1/(w + 1e-6) where w != 0, else 0 (reference: utils/mask.py:718-740)."""
        self._check_input(input_tensor)
        if self.is_full or self.is_empty:
            return input_tensor
        dense = self.get_dense_mask()
        return input_tensor * (1.0 / (dense + 1e-6) * (dense != 0))

    def apply_inv_mask_sparse(self, input_tensor: torch.Tensor) -> torch.Tensor:
        self._check_input(input_tensor)
        if self.is_full or self.is_empty:
            return input_tensor
        indices, _, data = self.get_index_mask()
        out = torch.zeros_like(input_tensor)
        if indices.numel() > 0:
            out.view(-1)[indices] = input_tensor.reshape(-1)[indices] * (1.0 / (data + 1e-6))
        return out

    # ------------------------------------------------------------------ merge
    def merge_mask(self, other_mask: "Mask", inplace: bool, mode: Literal["sparse", "dense"] = "dense") -> "Mask":
        if mode == "dense":
            return self.merge_mask_dense(other_mask, inplace)
        if mode == "sparse":
            return self.merge_mask_sparse(other_mask, inplace)
        raise ValueError(f"Invalid mode: {mode}")

    def _merge_trivial(self, other: "Mask", inplace: bool, as_index: bool) -> Optional["Mask"]:
        """Full / empty algebra shared by both merge modes; None when a real merge is needed."""
        if self.shape != other.shape:
            raise ValueError(f"Cannot merge masks with different shapes: {self.shape} vs {other.shape}")
        if self.is_full or other.is_full:
            full = Mask.create_full_mask(self.shape, self.dtype, self.device)
            return self._become(full) if inplace else full
        if self.is_empty and other.is_empty:
            return self if inplace else Mask.create_empty_mask(self.shape, self.dtype, self.device)
        if self.is_empty or other.is_empty:
            src = other if self.is_empty else self
            if inplace:
                return self if src is self else self._become(src)
            if as_index:
                i, p, d = src.get_index_mask()
                return Mask.create_mask_from_indices(self.shape, i, p, d, dtype=self.dtype)
            return Mask.create_mask_from_dense_mask(self.shape, src.get_dense_mask(), dtype=self.dtype)
        return None

    def merge_mask_dense(self, other_mask: "Mask", inplace: bool) -> "Mask":
        """clamp(m1 + m2, 0, 1) (reference: utils/mask.py:809-891)."""
        done = self._merge_trivial(other_mask, inplace, as_index=False)
        if done is not None:
            return done
        merged = torch.clamp(self.get_dense_mask() + other_mask.get_dense_mask(), 0.0, 1.0)
        out = Mask.create_mask_from_dense_mask(self.shape, merged, dtype=self.dtype)
        return self._become(out) if inplace else out

    def merge_mask_sparse(self, other_mask: "Mask", inplace: bool) -> "Mask":
        """Union of the index sets, weights added and clamped to [0, 1] (utils/mask.py:893-1062)."""
        done = self._merge_trivial(other_mask, inplace, as_index=True)
        if done is not None:
            return done
        i1, p1, d1 = self.get_index_mask()
        i2, p2, d2 = other_mask.get_index_mask()
        n_rows = _numel(self.shape[:-1])
        n = self.shape[-1]
        if i1.numel() == 0 and i2.numel() == 0:
            dev = self.device
            idx = torch.empty(0, dtype=torch.long, device=dev)
            dat = torch.empty(0, dtype=self.dtype, device=dev)
            ptr = torch.zeros(n_rows + 1, dtype=torch.long, device=dev)
        elif i1.numel() == 0:
            idx, dat, ptr = i2, torch.clamp(d2, 0.0, 1.0), p2
        elif i2.numel() == 0:
            idx, dat, ptr = i1, torch.clamp(d1, 0.0, 1.0), p1
        else:
            dev = i1.device
            both = torch.cat([i1, i2])
            vals = torch.cat([d1.to(self.dtype), d2.to(self.dtype)])
            both, order = torch.sort(both)
            idx, inverse = torch.unique_consecutive(both, return_inverse=True)
            dat = torch.zeros(idx.numel(), dtype=self.dtype, device=dev)
            dat.scatter_add_(0, inverse, vals[order])
            dat = torch.clamp(dat, 0.0, 1.0)
            per_row = torch.zeros(n_rows, dtype=torch.long, device=dev)
            per_row.scatter_add_(0, idx // n, torch.ones_like(idx))
            ptr = torch.zeros(n_rows + 1, dtype=torch.long, device=dev)
            ptr[1:] = torch.cumsum(per_row, dim=0)
        out = Mask.create_mask_from_indices(self.shape, idx, ptr, dat, dtype=self.dtype)
        return self._become(out) if inplace else out

    # ---------------------------------------------------------------- density
    def get_density(self) -> float:
        if self.is_full:
            return 1.0
        if self.is_empty:
            return 0.0
        if self.from_dense_mask:
            return float(torch.sum(self.mask > 0) / self.mask.numel())
        if self.from_index:
            return float(len(self.indices)) / float(_numel(self.shape))
        if self.from_rows:
            self.rows.zero_if_fresh()
            return float(self.rows.cnt.clamp(max=self.rows.cap).sum().item()) / float(_numel(self.shape))
        raise RuntimeError("Mask object is in an invalid state")
