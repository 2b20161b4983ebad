"""Cached launch plan for the common decode chains.

`ResearchAttention.custom_attention` (reference: research_attention/base.py:63-170) walks
its maskers in Python and then calls the masked attention. For the chains every decode
benchmark of this path uses —

    Sink, Local [, HashAttentionTopK | OracleTopK | PQCache]      (no additive mask, no sink
                                                                    logits, weights not requested)

— the same kernels can be driven from argument blocks that are built once and patched per
step (tensor pointers, key count), then handed to `sah_run_chain` in ONE native call. The
results are those of the masker-by-masker path (same kernels, same order); what goes away
is the per-step Python: Mask objects, row-buffer allocation, five ctypes dispatches.

Anything the plan does not cover (first call of a layer that has to hash every key or run
k-means, a full-mask short-circuit, an additive attention mask, ...) returns None and the
caller takes the general path.
"""
from __future__ import annotations

import ctypes as C
from typing import Any, Dict, Optional, Tuple

import torch

from ... import _native as N
from ..utils.mask_attention_utils import _workspace, unit_inverse_weight
from .maskers.fixed.base import sortable_key_of
from .maskers.fixed.implementations.basic_fixed import LocalMasker, SinkMasker
from .maskers.fixed.implementations.hashattention_top_k import HashAttentionTopKMasker, PackedSignatureCache
from .maskers.fixed.implementations.oracle_top_k import OracleTopK
from .maskers.fixed.implementations.pq_top_k import PQCache, PQCodebook, adc_lut_buffer

_MAX_NEW_KEYS = 64  # more than this many unseen keys => not a decode step, take the general path
_COMPACT_CODES = True  # HashAttention decode: the kernel scans 4-byte sign planes + an exception list instead of 8-byte codes
_HASH_BLOCK = 64    # HashAttention decode: new keys are hashed this many at a time (never more than the local window)


def plan_kind(maskers) -> Optional[str]:
    """'fixed' | 'hash' | 'oracle' | 'pq' if the masker list is a chain the plan covers."""
    if len(maskers) < 2 or type(maskers[0]) is not SinkMasker or type(maskers[1]) is not LocalMasker:
        return None
    if len(maskers) == 2:
        return "fixed"
    if len(maskers) == 3:
        t = type(maskers[2])
        if t is HashAttentionTopKMasker:
            return "hash"
        if t is OracleTopK:
            return "oracle"
        if t is PQCache and maskers[2].metric == "euclidean":  # "ip" augments the keys first: masker path
            return "pq"
    return None


class _LayerBlocks:
    """Per-layer argument blocks (signature weights differ per layer)."""

    __slots__ = ("sig_a", "sig_b", "weights_key")

    def __init__(self):
        self.sig_a = None
        self.sig_b = None
        self.weights_key = None


class DecodePlan:
    def __init__(self, maskers, kind: str, q: torch.Tensor, k: torch.Tensor):
        self.kind = kind
        self.sink_masker, self.local_masker = maskers[0], maskers[1]
        self.top = maskers[2] if len(maskers) == 3 else None
        self.device = q.device
        self.dtype = q.dtype
        self.dt = N.dtype_code(q.dtype)
        self.B, self.Hq, self.Lq, self.D = q.shape
        self.Hkv = k.shape[1]
        self.n_rows = self.B * self.Hq * self.Lq
        self.es = q.element_size()
        self.key_bits = 32 if q.dtype == torch.float32 else 16
        self.cap = 0
        self.words_alloc = 0
        self.cols = self.cnt = self.bitmap = None
        self.qcodes = None
        self.keybuf = None
        self.residbuf = None
        self.keybuf_pitch = 0
        self.layers: Dict[int, _LayerBlocks] = {}
        self.sink_local = N.SinkLocalArgs()
        self.hamming = N.HammingTopkArgs()
        self.hash_decode = N.HashDecodeArgs()
        self.compact = N.HashCompactArgs()
        self.qk = N.QkScoresArgs()
        self.pq_assign = N.PqAssignArgs()
        self.pq_adc = N.PqAdcArgs()
        self.adc_lut = None
        self.select = N.SelectTopkArgs()
        self.att = N.AttentionArgs()
        self.chain = N.ChainArgs()
        self.unit = unit_inverse_weight(q.dtype)
        # arrival counters of the one-kernel selection + attention (zero between calls: the kernel puts them back)
        self.tickets = torch.zeros((self.n_rows,), dtype=torch.int32, device=self.device)
        self._excluded_min = sortable_key_of(torch.finfo(q.dtype).min, q.dtype)

    def signature(self, q: torch.Tensor, k: torch.Tensor) -> Tuple:
        return (q.device, q.dtype, tuple(q.shape), k.shape[1])

    # ------------------------------------------------------------------ buffers
    def _ensure_rows(self, cap: int, n_keys: int) -> None:
        words = (n_keys + 31) // 32
        if cap > self.cap or self.cols is None:
            self.cap = cap + 64
            self.cols = torch.empty((self.n_rows, self.cap), dtype=torch.int32, device=self.device)
            self.cnt = torch.empty((self.n_rows,), dtype=torch.int32, device=self.device)
        if words > self.words_alloc or self.bitmap is None:
            self.words_alloc = words + 256
            self.bitmap = torch.empty((self.n_rows * self.words_alloc,), dtype=torch.int32, device=self.device)

    def _rows_struct(self, n_keys: int) -> N.Rows:
        return N.Rows(self.cols.data_ptr(), self.cnt.data_ptr(), None, self.bitmap.data_ptr(), self.n_rows, self.cap,
                      n_keys, (n_keys + 31) // 32)

    def _ensure_keybuf(self, n_cols: int) -> None:
        if self.keybuf is None or n_cols > self.keybuf_pitch:
            self.keybuf_pitch = (n_cols + 4096 + 63) // 64 * 64
            kdt = torch.int32 if self.dtype == torch.float32 else torch.int16
            self.keybuf = torch.empty((self.n_rows, self.keybuf_pitch), dtype=kdt, device=self.device)
            # exact scores (OracleTopK) of 16-bit tensors: what their rounding took away goes beside the keys, and the
            # attention takes its logits from the two instead of reading K again
            self.residbuf = (torch.empty_like(self.keybuf)
                             if self.kind == "oracle" and kdt == torch.int16 and self.D in (64, 128) else None)

    # --------------------------------------------------------------------- run
    def run(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scaling: float,
            sparse_meta_data: Dict[Any, Any], layer_idx: Optional[int]) -> Optional[torch.Tensor]:
        """One layer-step; returns the attention output (B, Lq, Hq, D) or None if not applicable."""
        Lk = k.shape[2]
        Lq = self.Lq
        sink = self.sink_masker._calculate_effective_sink_size(Lk)
        window = self.local_masker._calculate_effective_window_size(Lk)
        if sink <= 0 or window <= 0 or Lk <= sink or Lk <= window + Lq:
            return None
        k_eff = 0
        top = self.top
        if top is not None:
            if layer_idx is None and self.kind in ("hash", "pq"):
                return None  # the general path raises the reference's ValueError
            k_eff = top._calculate_effective_size(top.heavy_size, Lk)
            if k_eff <= 0 or Lk <= k_eff:
                return None
        if q.stride(3) != 1 or k.stride(3) != 1 or v.stride(3) != 1 or v.shape[2] != Lk:
            return None
        stream = N.stream_ptr(self.device)
        cap = sink + window + k_eff
        self._ensure_rows(cap, Lk)
        rows = self._rows_struct(Lk)
        chain = self.chain
        es = self.es
        # what this step adds to the persistent caches (keys hashed, compacted, quantised) is recorded only after
        # the native call has returned without an error: a refused call must not leave a cache that claims codes
        # nobody wrote
        commit = []

        sl = self.sink_local
        sl.rows, sl.lq, sl.sink, sl.window, sl.fresh, sl.clear_future, sl.stream = rows, Lq, sink, window, 1, 1, stream
        chain.sink_local = C.addressof(sl)
        chain.sig_a = chain.sig_b = chain.hamming = chain.qk = chain.pq_assign = chain.pq_adc = chain.select = None
        chain.hash_decode = chain.compact = None

        if self.kind == "hash":
            cache = sparse_meta_data.get("key", {}).get(layer_idx)
            if not isinstance(cache, PackedSignatureCache) or Lk < cache.n or Lk - cache.n > _MAX_NEW_KEYS:
                return None
            if cache.codes.shape[0] != self.B or cache.codes.shape[1] != self.Hq:
                return None
            blocks = self.layers.get(layer_idx)
            wkey = (id(top.hat_weights), layer_idx)
            if blocks is None or blocks.weights_key != wkey:
                blocks = _LayerBlocks()
                blocks.weights_key = wkey
                blocks.sig_a = top._hash_args(k, self.Hkv, self.Hq, 0, 1, layer_idx, "key", cache.codes, cache.capacity, 0)
                if self.qcodes is None:
                    self.qcodes = torch.empty((self.n_rows, 2), dtype=torch.int32, device=self.device)
                blocks.sig_b = top._hash_args(q, self.Hq, self.Hq, 0, Lq, layer_idx, "query", self.qcodes, Lq, 0)
                self.layers[layer_idx] = blocks
            n_new = Lk - cache.n
            cache.reserve(Lk)
            # One query per row: this step can only select columns below Lk - window, so the codes of keys still
            # inside the local window are not needed yet. They are hashed a block at a time (one bulk launch
            # every `lag` steps) instead of one key per step; `cache.n` is the number of keys hashed so far.
            lag = min(window, _HASH_BLOCK) if Lq == 1 else 1
            hash_now = n_new >= lag
            if n_new > 0 and hash_now:
                a = blocks.sig_a
                a.x = k.data_ptr() + cache.n * k.stride(2) * es
                a.xs_b, a.xs_h, a.xs_l = k.stride(0), k.stride(1), k.stride(2)
                a.L = n_new
                a.codes, a.code_pitch, a.code_offset, a.stream = cache.codes.data_ptr(), cache.capacity, cache.n, stream
                chain.sig_a = C.addressof(a)
            bq = blocks.sig_b
            bq.x = q.data_ptr()
            bq.xs_b, bq.xs_h, bq.xs_l, bq.stream = q.stride(0), q.stride(1), q.stride(2), stream
            chain.sig_b = C.addressof(bq)
            if Lq == 1:
                # the whole mask-building half of the step as one entry point (one kernel when shapes allow);
                # a single new key is hashed inside it, a block of them by one launch in front of it
                hd = self.hash_decode
                hd.rows, hd.sink, hd.window = rows, sink, window
                hd.query_sig = chain.sig_b
                use_compact = _COMPACT_CODES
                hd.key_sig = chain.sig_a if n_new == 1 and not use_compact else None
                hd.pos_codes = hd.exc = hd.exc_cnt = None
                if use_compact:
                    # keys hashed since the compact form was last brought up to date (by this step's launch in
                    # front of the kernel, by the first call of the layer, by the general path) are added to it
                    cache.ensure_compact_buffers()
                    hashed = Lk if hash_now else cache.n
                    if hashed > cache.n_compact:
                        cp = self.compact
                        cp.codes, cp.code_pitch, cp.n_rows = cache.codes.data_ptr(), cache.capacity, self.n_rows
                        cp.from_, cp.to = cache.n_compact, hashed
                        cp.pos_codes, cp.pos_pitch = cache.pos.data_ptr(), cache.pos.shape[2]
                        cp.exc, cp.exc_cap, cp.exc_cnt = cache.exc.data_ptr(), cache.exc.shape[2], cache.exc_cnt.data_ptr()
                        cp.full_plane, cp.stream = cache.full_plane, stream
                        chain.compact = C.addressof(cp)
                        commit.append((cache, "n_compact", hashed))
                    hd.pos_codes, hd.pos_pitch = cache.pos.data_ptr(), cache.pos.shape[2]
                    hd.exc, hd.exc_cap, hd.exc_cnt = cache.exc.data_ptr(), cache.exc.shape[2], cache.exc_cnt.data_ptr()
                    hd.full_plane = cache.full_plane
                hd.kcodes, hd.code_pitch, hd.k, hd.stream = cache.codes.data_ptr(), cache.capacity, k_eff, stream
                hd.skip_bitmap = 1  # only the attention kernel reads these rows, and it reads the column lists
                chain.hash_decode = C.addressof(hd)
                chain.sink_local = chain.sig_b = None
                if hd.key_sig is not None:
                    chain.sig_a = None  # hashed inside the kernel
            else:
                hm = self.hamming
                hm.rows, hm.kcodes, hm.code_pitch = rows, cache.codes.data_ptr(), cache.capacity
                hm.qcodes, hm.lq, hm.k, hm.stream = self.qcodes.data_ptr(), Lq, k_eff, stream
                chain.hamming = C.addressof(hm)
            if hash_now:
                commit.append((cache, "n", Lk))
        elif self.kind == "oracle":
            self._ensure_keybuf(Lk)
            qa = self.qk
            qa.q, qa.qs_b, qa.qs_h, qa.qs_l = q.data_ptr(), q.stride(0), q.stride(1), q.stride(2)
            qa.k, qa.ks_b, qa.ks_h, qa.ks_l = k.data_ptr(), k.stride(0), k.stride(1), k.stride(2)
            qa.amask = None
            qa.dtype, qa.B, qa.Hq, qa.Hkv, qa.Lq, qa.Lk, qa.D = self.dt, self.B, self.Hq, self.Hkv, Lq, Lk, self.D
            qa.keys_out, qa.key_pitch, qa.stream = self.keybuf.data_ptr(), self.keybuf_pitch, stream
            qa.resid_out = None if self.residbuf is None else self.residbuf.data_ptr()
            chain.qk = C.addressof(qa)
            se = self.select
            se.rows, se.keys, se.key_pitch, se.key_bits = rows, self.keybuf.data_ptr(), self.keybuf_pitch, self.key_bits
            se.n_cand, se.col_offset, se.k, se.excluded_key, se.stream = Lk, 0, k_eff, self._excluded_min, stream
            se.skip_bitmap = 1  # only the attention reads these rows, and it reads the column lists
            chain.select = C.addressof(se)
            if Lq == 1:
                # one query per row: the selection kernel writes the sink + local rows itself
                se.fresh, se.fresh_sink, se.fresh_window = 1, sink, window
                chain.sink_local = None
            else:
                se.fresh = 0
        elif self.kind == "pq":
            off = top.init_offset
            if Lk <= k_eff + off + Lq + 2 ** top.pq_bits:
                return None
            book = sparse_meta_data.get("pq_codebook", {}).get(layer_idx)
            cf32 = sparse_meta_data.get("pq_centroids_f32", {}).get(layer_idx)
            if not isinstance(book, PQCodebook) or cf32 is None:
                return None
            current = Lk - off
            if current < book.n or current - book.n > _MAX_NEW_KEYS or book.codes.shape[0] != self.B:
                return None
            n_sub, d_sub, n_cent = top._geometry(k)
            book.reserve(current)
            # One query per row: only columns below Lk - window can be selected, so the code of a key that is still
            # inside the local window is not needed yet. New keys are quantised a block at a time (one launch every
            # `lag` steps); `book.n` is the number of keys quantised so far and the scoring pass covers exactly those,
            # which always include every column outside the window.
            lag = min(window, _HASH_BLOCK) if Lq == 1 else 1
            if current - book.n >= lag:
                pa = self.pq_assign
                pa.k, pa.ks_b, pa.ks_h, pa.ks_l = k.data_ptr(), k.stride(0), k.stride(1), k.stride(2)
                pa.dtype, pa.B, pa.Hkv, pa.n_sub, pa.d_sub, pa.n_cent = self.dt, self.B, self.Hkv, n_sub, d_sub, n_cent
                pa.key_offset, pa.n_keys = off + book.n, current - book.n
                pa.centres, pa.codes, pa.code_pitch, pa.code_offset = cf32.data_ptr(), book.codes.data_ptr(), book.capacity, book.n
                pa.sums = pa.counts = pa.skip_flag = None
                pa.round_dist, pa.stream = 1, stream
                chain.pq_assign = C.addressof(pa)
                commit.append((book, "n", current))
            else:
                current = book.n
            self._ensure_keybuf(current)
            ad = self.pq_adc
            ad.q, ad.qs_b, ad.qs_h, ad.qs_l = q.data_ptr(), q.stride(0), q.stride(1), q.stride(2)
            ad.dtype, ad.B, ad.Hq, ad.Hkv, ad.Lq = self.dt, self.B, self.Hq, self.Hkv, Lq
            ad.n_sub, ad.d_sub, ad.n_cent = n_sub, d_sub, n_cent
            ad.centres, ad.codes, ad.code_pitch, ad.n_cand = cf32.data_ptr(), book.codes.data_ptr(), book.capacity, current
            ad.keys_out, ad.key_pitch, ad.stream = self.keybuf.data_ptr(), self.keybuf_pitch, stream
            if self.adc_lut is None:
                self.adc_lut = adc_lut_buffer(self.B, self.Hq, self.Hkv, Lq, n_sub, n_cent, self.dtype, self.device)
            ad.lut, ad.lut_bytes = self.adc_lut.data_ptr(), self.adc_lut.numel()
            narrow = sparse_meta_data.get("pq_centroids", {}).get(layer_idx)
            ad.centres_narrow = (narrow.data_ptr() if narrow is not None and narrow.dtype == self.dtype and narrow.is_contiguous()
                                 and narrow.shape[-1] == d_sub and narrow.dtype != torch.float32 else None)
            chain.pq_adc = C.addressof(ad)
            se = self.select
            se.rows, se.keys, se.key_pitch, se.key_bits = rows, self.keybuf.data_ptr(), self.keybuf_pitch, self.key_bits
            se.n_cand, se.col_offset, se.k, se.excluded_key, se.stream = current, off, k_eff, self._excluded_min, stream
            se.skip_bitmap = 1  # only the attention reads these rows, and it reads the column lists
            chain.select = C.addressof(se)
            if Lq == 1:
                # one query per row: the selection kernel writes the sink + local rows itself
                se.fresh, se.fresh_sink, se.fresh_window = 1, sink, window
                chain.sink_local = None
            else:
                se.fresh = 0

        out = torch.empty((self.B, Lq, self.Hq, self.D), dtype=self.dtype, device=self.device)
        work = _workspace(self.device, N.work_floats(self.n_rows, cap, self.D))
        at = self.att
        at.rows = rows
        at.q, at.qs_b, at.qs_h, at.qs_l = q.data_ptr(), q.stride(0), q.stride(1), q.stride(2)
        at.k, at.ks_b, at.ks_h, at.ks_l = k.data_ptr(), k.stride(0), k.stride(1), k.stride(2)
        at.v, at.vs_b, at.vs_h, at.vs_l = v.data_ptr(), v.stride(0), v.stride(1), v.stride(2)
        at.amask = None
        at.sinks = None
        at.dtype, at.B, at.Hq, at.Hkv, at.Lq, at.Lk, at.D = self.dt, self.B, self.Hq, self.Hkv, Lq, Lk, self.D
        at.scaling, at.unit_inv_w, at.dense, at.max_cnt = float(scaling), self.unit, 0, cap
        at.out, at.work, at.work_floats = out.data_ptr(), work.data_ptr(), work.numel()
        at.logits_out = at.stats_out = None
        at.closed_form = 0
        # an exact scoring pass came before: its 16-bit keys are the attention's logits, K is not read again
        at.score_keys, at.score_resid, at.score_pitch = None, None, 0
        if self.kind == "oracle" and self.residbuf is not None:
            at.score_keys, at.score_resid, at.score_pitch = self.keybuf.data_ptr(), self.residbuf.data_ptr(), self.keybuf_pitch
        if self.kind == "fixed" and Lq == 1:
            # Sink + Local alone: the attention kernel takes the columns in closed form, no row is ever written
            at.closed_form, at.closed_sink, at.closed_window = 1, sink, window
            chain.sink_local = None
        at.stream = stream
        chain.attention = C.addressof(at)
        chain.tickets = self.tickets.data_ptr()
        N.call("sah_run_chain", chain)
        for obj, name, value in commit:
            setattr(obj, name, value)
        return out
