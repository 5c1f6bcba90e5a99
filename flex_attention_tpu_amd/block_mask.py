"""Block-sparsity maps: the GPU builder (flexattn_build_block_mask) and its host-side handle.

The reference evaluates ``block_mask_fn(q_block, kv_block)`` at every grid step and again inside
the K/V index maps (flex_attention_kernel.py:97-106, 231-236).  Here the same predicate is
evaluated once per (mask, shape, tile) by a small HIP kernel into a device-resident map that the
attention kernels walk; maps are cached (bounded, least recently used) because they depend on
nothing but the mask specification.
"""
from __future__ import annotations

import collections
import ctypes as C
from typing import Callable, Optional

import torch

from . import _lib
from .masks import DocIds, MaskSpec

_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def raw_stream(device) -> int:
    """Handle of the current stream of `device` (the lookup that builds no Stream object where torch has one: the
    launch path of a small call is a few tens of microseconds in all)."""
    if _raw_stream is not None:
        idx = device.index
        return _raw_stream(torch.cuda.current_device() if idx is None else idx)
    return torch.cuda.current_stream(device).cuda_stream


class LRU:
    """Small least-recently-used cache: holds at most ``maxsize`` entries (each may pin device
    tensors), so a training loop with a new document layout every batch does not grow it."""

    def __init__(self, maxsize: int):
        self.maxsize = maxsize
        self._d = collections.OrderedDict()

    def get(self, key):
        v = self._d.get(key)
        if v is not None:
            self._d.move_to_end(key)
        return v

    def put(self, key, value):
        self._d[key] = value
        self._d.move_to_end(key)
        while len(self._d) > self.maxsize:
            self._d.popitem(last=False)

    def clear(self):
        self._d.clear()

    def __len__(self):
        return len(self._d)


class BlockMap:
    """Device-resident block map at (block_q x block_k) granularity.

    state[qb, kb]: 0 skip, 1 partial, 2 full.  kv_idx[qb, :kv_cnt[qb]] / q_idx[kb, :q_cnt[kb]] are
    the ascending lists of blocks to visit per q-block row / kv-block column.
    """

    def __init__(self, spec: MaskSpec, Sq: int, Sk: int, block_q: int, block_k: int, device):
        self.spec, self.Sq, self.Sk, self.block_q, self.block_k = spec, Sq, Sk, block_q, block_k
        self.nq, self.nk = Sq // block_q, Sk // block_k
        self.state = torch.empty(self.nq, self.nk, dtype=torch.uint8, device=device)
        self.kv_cnt = torch.empty(self.nq, dtype=torch.int32, device=device)
        self.kv_idx = torch.empty(self.nq, self.nk, dtype=torch.int32, device=device)
        self.q_cnt = torch.empty(self.nk, dtype=torch.int32, device=device)
        self.q_idx = torch.empty(self.nk, self.nq, dtype=torch.int32, device=device)
        self.built_on = None   # stream the builder kernel was launched on
        self.ready = None      # event recorded behind it
        self._ds_index = None  # (col, rank, pairs) of the dS exchange buffer, built at first use
        self._partial_share = None

    def _tensors(self):
        t = [self.state, self.kv_cnt, self.kv_idx, self.q_cnt, self.q_idx]
        if self._ds_index is not None:
            t += [self._ds_index[0], self._ds_index[1]]
        return t

    def wait_ready(self, device) -> None:
        """Makes the current stream wait for the builder kernel if that ran on another stream, and tells the
        caching allocator that the map is in use on this stream too (a map evicted from the cache must not be
        handed out again while a kernel on this stream still walks it)."""
        if self.ready is None or raw_stream(device) == self.built_on:
            return
        cur = torch.cuda.current_stream(device)
        if cur.cuda_stream != self.built_on:
            cur.wait_event(self.ready)
            for t in self._tensors():
                t.record_stream(cur)

    def ds_index(self):
        """(col int32 [nk + 1], rank int32 [nq, nk], pairs) of flexattn_build_ds_index for this map: the order of
        the dS exchange buffer's blocks over the kept tile pairs.  Built once per map (one 4-byte copy to the
        host for the number of pairs)."""
        if self._ds_index is None:
            dev = self.state.device
            col = torch.empty(self.nk + 1, dtype=torch.int32, device=dev)
            rank = torch.empty(self.nq, self.nk, dtype=torch.int32, device=dev)
            lib = _lib.load()
            with torch.cuda.device(dev):
                self.wait_ready(dev)
                cmap = self.as_c()
                _lib.check(lib.flexattn_build_ds_index(C.byref(cmap), col.data_ptr(), rank.data_ptr(),
                                                       torch.cuda.current_stream(dev).cuda_stream), lib)
                pairs = int(col[-1].item())
            self._ds_index = (col, rank, pairs)
        return self._ds_index

    def partial_share(self) -> float:
        """Share of the tiles that run which are partly masked (read back from the device once per map)."""
        if self._partial_share is None:
            self.wait_ready(self.state.device)
            run = int((self.state != 0).sum().item())
            self._partial_share = (int((self.state == 1).sum().item()) / run) if run else 0.0
        return self._partial_share

    def ds_index_c(self) -> _lib.DsIndexC:
        col, rank, pairs = self.ds_index()
        return _lib.DsIndexC(col.data_ptr(), rank.data_ptr(), pairs)

    def as_c(self) -> _lib.BlockMapC:
        return _lib.BlockMapC(self.state.data_ptr(), self.kv_cnt.data_ptr(), self.kv_idx.data_ptr(),
                              self.q_cnt.data_ptr(), self.q_idx.data_ptr(), self.nq, self.nk,
                              self.block_q, self.block_k)

    def run_mask(self) -> torch.Tensor:
        """bool [nq, nk]: tile must run (the quantity the reference's block closures return)."""
        return self.state != 0


# Bounded caches (least recently used entries are dropped; a dropped map is simply rebuilt):
MAP_CACHE_SIZE = 64
DOC_CACHE_SIZE = 64
_doc_cache = LRU(DOC_CACHE_SIZE)   # (DocIds, device) -> int32 device array
_map_cache = LRU(MAP_CACHE_SIZE)   # (spec, Sq, Sk, block_q, block_k, device) -> BlockMap


def doc_ids_on(doc: Optional[DocIds], device) -> Optional[torch.Tensor]:
    """int32 device copy of the document ids (cached per device)."""
    if doc is None:
        return None
    key = (doc, str(device))
    t = _doc_cache.get(key)
    if t is None:
        t = torch.from_numpy(doc.array.copy()).to(device)  # (pageable host memory: the copy is synchronous)
        _doc_cache.put(key, t)
    return t


_rows_cache = LRU(DOC_CACHE_SIZE)   # (DocIds, B) -> DocIds with B rows


def _rows_of(doc: DocIds, B: int) -> DocIds:
    """`doc` with one row per batch entry (a shared row repeated; cached)."""
    if doc.batches == B and doc.array.ndim == 2:
        return doc
    key = (doc, B)
    d = _rows_cache.get(key)
    if d is None:
        d = DocIds(doc.rows(B))
        _rows_cache.put(key, d)
    return d


_range_cache = LRU(DOC_CACHE_SIZE)  # (DocIds, DocIds of the other side, device) -> int32 [n, 2] device array or False


def doc_ranges_on(doc: DocIds, other: DocIds, device) -> Optional[torch.Tensor]:
    """Device copy of ``doc.ranges_in(other)`` (cached per device), or None when ``other`` is not sorted."""
    key = (doc, other, str(device))
    t = _range_cache.get(key)
    if t is None:
        r = doc.ranges_in(other)
        t = torch.from_numpy(r).to(device) if r is not None else False
        _range_cache.put(key, t)
    return t if t is not False else None


def mask_spec_c(spec: MaskSpec, Sq: int, Sk: int, device) -> _lib.MaskSpecC:
    """C view of a MaskSpec; validates the document array lengths."""
    doc_q = doc_k = range_q = range_k = None
    doc_batches = 0
    if spec.flags & _lib.MASK_DOC:
        if spec.doc_ids is None:
            raise ValueError("document mask without document ids")
        ids_k = spec.doc_ids_k if spec.doc_ids_k is not None else spec.doc_ids
        if len(spec.doc_ids) < Sq or len(ids_k) < Sk:
            raise ValueError(f"document ids cover {len(spec.doc_ids)} q / {len(ids_k)} kv positions, need {Sq} / {Sk}")
        # a row per batch entry on either side: both sides go to the kernels as [B, S] (doc_batches = B)
        batches = max(spec.doc_ids.batches, ids_k.batches)
        ids_q = spec.doc_ids
        if batches > 1:
            if len(ids_q) != Sq or len(ids_k) != Sk:   # (the kernels step from row to row by the sequence lengths)
                raise ValueError(f"document ids per batch entry must have exactly {Sq} q / {Sk} kv positions")
            ids_q, ids_k = _rows_of(ids_q, batches), _rows_of(ids_k, batches)
        tq, tk = doc_ids_on(ids_q, device), doc_ids_on(ids_k, device)
        cur = torch.cuda.current_stream(device)
        tq.record_stream(cur)   # (cached arrays may be evicted while a kernel on this stream still reads them)
        tk.record_stream(cur)
        doc_q, doc_k = tq.data_ptr(), tk.data_ptr()
        # sorted ids (the usual case: documents packed one after the other): the interval of the other side's
        # positions with a position's id, from which the kernels mask partial tiles without comparing ids
        if len(ids_q) == Sq and len(ids_k) == Sk:
            rq, rk = doc_ranges_on(ids_q, ids_k, device), doc_ranges_on(ids_k, ids_q, device)
            if rq is not None:
                rq.record_stream(cur)
                range_q = rq.data_ptr()
            if rk is not None:
                rk.record_stream(cur)
                range_k = rk.data_ptr()
        doc_batches = batches
    return _lib.MaskSpecC(spec.flags, spec.window, spec.stride, doc_batches, doc_q, doc_k, range_q, range_k)


def build_block_map(spec: MaskSpec, Sq: int, Sk: int, block_q: int, block_k: int, device,
                    cache: bool = True, score_code=None) -> BlockMap:
    """Runs the GPU block-mask builder (or returns the cached map for this specification).  A compiled
    mask closure is built by the functor library that holds it (`score_code`: the compiled score closure of
    the same call, if any, so that one library serves both)."""
    device = torch.device(device)
    key = (spec, Sq, Sk, block_q, block_k, str(device))
    if cache:
        hit = _map_cache.get(key)
        if hit is not None:
            hit.wait_ready(device)
            return hit
    if Sq % block_q or Sk % block_k:
        raise ValueError(f"Sq={Sq} / Sk={Sk} not divisible by blocks {block_q} / {block_k}")
    lib = _lib.load_for(score_code if spec.custom is not None else None, spec.custom)
    bm = BlockMap(spec, Sq, Sk, block_q, block_k, device)
    mc = mask_spec_c(spec, Sq, Sk, device)
    stream = torch.cuda.current_stream(device).cuda_stream
    with torch.cuda.device(device):
        _lib.check(lib.flexattn_build_block_mask(
            C.byref(mc), Sq, Sk, block_q, block_k, bm.state.data_ptr(), bm.kv_cnt.data_ptr(),
            bm.kv_idx.data_ptr(), bm.q_cnt.data_ptr(), bm.q_idx.data_ptr(), stream), lib)
        bm.built_on = stream
        bm.ready = torch.cuda.Event()
        bm.ready.record(torch.cuda.current_stream(device))
    if cache:
        _map_cache.put(key, bm)
    return bm


def create_block_mask(mask_fns, Sq: int, Sk: int, block_q: int, block_k: int, device="cuda") -> BlockMap:
    """Block map of a ``(mask_fn, block_mask_fn)`` pair (or a MaskSpec) at the given granularity."""
    spec = mask_fns if isinstance(mask_fns, MaskSpec) else spec_of(mask_fns[0], mask_fns[1])
    return build_block_map(spec, Sq, Sk, block_q, block_k, device)


def spec_of(mask_fn: Optional[Callable], block_mask_fn: Optional[Callable]) -> MaskSpec:
    """MaskSpec carried by the closures: those of this package's factories, or of compiler.compile_mask_fn
    for arbitrary element predicates.  Untagged closures are rejected."""
    spec = None
    for f in (mask_fn, block_mask_fn):
        if f is None:
            continue
        s = getattr(f, "spec", None)
        if s is None:
            raise NotImplementedError(
                "mask_fn/block_mask_fn must come from flex_attention_tpu_amd.masks factories or from "
                "flex_attention_tpu_amd.compiler.compile_mask_fn (which compiles a Python predicate into the kernels)")
        if spec is not None and s != spec:
            raise ValueError("mask_fn and block_mask_fn describe different masks")
        spec = s
    return spec if spec is not None else MaskSpec()


def host_block_map(block_mask_fn: Callable, nq: int, nk: int) -> torch.Tensor:
    """bool [nq, nk] by calling the Python block closure on every tile (CPU; used by tests)."""
    out = torch.empty(nq, nk, dtype=torch.bool)
    for qb in range(nq):
        for kb in range(nk):
            out[qb, kb] = bool(block_mask_fn(qb, kb))
    return out
