"""Paged KV cache with the two side structures the decode path reads: the INT4 K shadow and the
Quest page metadata. Storage only — every computation is a call into ``twilight_amd.kernel``."""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib
from .kernel import kv_append, kv_shadow_build, meta_planes_build

PAGE = _lib.PAGE
HEAD_DIM = _lib.HEAD_DIM


class PagedKVCache:
    """K / V pages ``[num_pages, 16, Hkv, 128]`` (fp16 or bf16) plus ``k_int4``
    ``[num_pages, Hkv, 1280]`` and ``meta`` ``[num_pages, Hkv, 512]`` (uint8 records), and the
    CSR page table of the current batch (``kv_page_indices``, ``kv_page_indptr``,
    ``kv_last_page_len``; the layout benchmark/efficiency/bench_gemv.py:425-431 builds)."""

    def __init__(self, num_pages: int, num_kv_heads: int, dtype: torch.dtype, device):
        if dtype not in (torch.float16, torch.bfloat16):
            raise RuntimeError("PagedKVCache dtype must be float16 or bfloat16")
        self.num_pages, self.num_kv_heads, self.dtype = num_pages, num_kv_heads, dtype
        self.device = torch.device(device)
        shape = (num_pages, PAGE, num_kv_heads, HEAD_DIM)
        self.k_cache = torch.zeros(shape, dtype=dtype, device=self.device)
        self.v_cache = torch.zeros(shape, dtype=dtype, device=self.device)
        self.k_int4 = torch.zeros((num_pages, num_kv_heads, _lib.INT4_RECORD_BYTES),
                                  dtype=torch.uint8, device=self.device)
        self.meta = torch.zeros((num_pages, num_kv_heads, _lib.META_RECORD_BYTES),
                                dtype=torch.uint8, device=self.device)
        self.kv_page_indices: Optional[torch.Tensor] = None
        self.kv_page_indptr: Optional[torch.Tensor] = None
        self.kv_last_page_len: Optional[torch.Tensor] = None
        self.max_pages_per_req = 0
        self._seq_lens = None  # host copy, for append bookkeeping
        self._room = 0         # appends that surely fit every request's last page
        self._append_key = None
        self._table_cap = 0    # pages per request of a fixed-address page table (0: not fixed)
        # Quest metadata in plane layout [slots, Hkv, 128, 2, cap] (see enable_planes) and the
        # slot of every request of the batch (None: slot = position in the batch)
        self.meta_planes: Optional[torch.Tensor] = None
        self.plane_slots: Optional[torch.Tensor] = None

    # ---- page table ---------------------------------------------------------------------------
    def set_page_table(self, kv_page_indices: torch.Tensor, kv_page_indptr: torch.Tensor,
                       kv_last_page_len: torch.Tensor) -> None:
        self.kv_page_indices = kv_page_indices.to(self.device, torch.int32).contiguous()
        self.kv_page_indptr = kv_page_indptr.to(self.device, torch.int32).contiguous()
        self.kv_last_page_len = kv_last_page_len.to(self.device, torch.int32).contiguous()
        ip = kv_page_indptr.cpu().long()
        npg = ip[1:] - ip[:-1]
        self.max_pages_per_req = int(npg.max().item())
        self._seq_lens = ((npg - 1) * PAGE + kv_last_page_len.cpu().long()).tolist()
        # host mirrors of the table: append() never reads the device copies back
        ids = kv_page_indices.cpu().tolist()
        ipl = ip.tolist()
        self._per_req = [ids[ipl[b]:ipl[b + 1]] for b in range(len(ipl) - 1)]
        self._last = kv_last_page_len.cpu().tolist()
        self._room = PAGE - max(self._last) if self._last else 0
        self._append_key = None
        self._table_cap = 0

    def reserve_page_table(self, cap_pages: int) -> None:
        """Fix the addresses of the page table for requests of up to ``cap_pages`` pages: from
        here on ``append`` rewrites ``kv_page_indices`` / ``kv_page_indptr`` in place when a
        request takes a new page, and ``max_pages_per_req`` stays at ``cap_pages`` (the kernels
        take it as an upper bound; the pages a request really has come from the table). A decode
        step whose launches were recorded into a HIP graph therefore stays valid while the
        requests grow."""
        if cap_pages < self.max_pages_per_req:
            raise RuntimeError(f"cap_pages {cap_pages} is below the longest request "
                               f"({self.max_pages_per_req} pages)")
        if self.meta_planes is not None and cap_pages > self.meta_planes.size(4):
            raise RuntimeError("reserve_page_table: the plane buffer is smaller than cap_pages")
        buf = torch.zeros(self.batch * cap_pages, dtype=torch.int32, device=self.device)
        buf[:self.kv_page_indices.numel()] = self.kv_page_indices
        self.kv_page_indices = buf
        self._table_cap = int(cap_pages)
        self.max_pages_per_req = int(cap_pages)
        self._append_key = None

    @property
    def batch(self) -> int:
        return self.kv_page_indptr.numel() - 1

    # ---- filling ------------------------------------------------------------------------------
    @property
    def max_seq_len(self) -> int:
        """Longest request of the batch in tokens (host-side count, no device read)."""
        return max(self._seq_lens) if self._seq_lens else 0

    def rebuild_shadow(self, page_ids: Optional[torch.Tensor] = None,
                       valid_len: Optional[torch.Tensor] = None) -> None:
        """(Re)build INT4 records and Quest metadata of ``page_ids`` (default: every page, all 16
        tokens valid), and the plane-layout metadata of the whole page table when enabled."""
        kv_shadow_build(self.k_cache, self.k_int4, self.meta, page_ids, valid_len)
        self.rebuild_planes()

    def enable_planes(self, cap_pages: Optional[int] = None, num_slots: Optional[int] = None,
                      slots: Optional[torch.Tensor] = None) -> None:
        """Keep the Quest metadata also in plane layout (per request slot, kv head and channel the
        page minima contiguously, then the maxima), sized for requests of up to ``cap_pages`` pages
        (default: the current longest request). The one-launch selector then reads half the
        metadata bytes. Needs a page table. ``num_slots`` (default: the batch size) is the number
        of requests the buffer can hold; ``slots`` int32 [batch] names the slot of each request of
        the current batch (default: its position), see :meth:`set_plane_slots`."""
        if self.kv_page_indptr is None:
            raise RuntimeError("enable_planes needs a page table (set_page_table)")
        cap = max(int(cap_pages or 0), self.max_pages_per_req, 8)
        # the library needs a multiple of 8; a multiple of 128 pages keeps every run 256-byte
        # aligned, so that a wavefront's 256-byte load touches two cache lines, not three
        cap = (cap + 127) // 128 * 128
        n = max(int(num_slots or 0), self.batch)
        self.meta_planes = torch.zeros((n, self.num_kv_heads, HEAD_DIM, 2, cap),
                                       dtype=self.dtype, device=self.device)
        self.plane_slots = None
        if slots is not None:
            self.set_plane_slots(slots, rebuild=False)
        self.rebuild_planes()

    def set_plane_slots(self, slots: Optional[torch.Tensor], rebuild: bool = False) -> None:
        """Name the plane slot of every request of the current batch (int32 [batch], distinct
        values in [0, slots of the buffer)); ``None`` goes back to slot = position. When the batch
        changes composition (a request leaves, the others move up) the page table and this table
        change and the planes stay where they are; ``rebuild`` refills the named slots from the
        records (for requests that are new to the buffer)."""
        if slots is not None:
            host = [int(x) for x in slots.cpu().tolist()]
            n = 0 if self.meta_planes is None else self.meta_planes.size(0)
            if len(host) != self.batch or len(set(host)) != len(host) or \
                    any(x < 0 or x >= n for x in host):
                raise RuntimeError("plane slots must be distinct, one per request, inside the buffer")
            slots = slots.to(self.device, torch.int32).contiguous()
        self.plane_slots = slots
        if rebuild:
            self.rebuild_planes()

    def rebuild_planes(self) -> None:
        """Refill the plane-layout metadata from the records, for the pages of the page table."""
        if self.meta_planes is None or self.kv_page_indptr is None:
            return
        fits = (self.batch <= self.meta_planes.size(0) if self.plane_slots is None
                else self.plane_slots.numel() == self.batch)
        if not fits or self.max_pages_per_req > self.meta_planes.size(4):
            raise RuntimeError("the page table no longer fits the plane buffer: call enable_planes "
                               "(or set_plane_slots for the new batch)")
        meta_planes_build(self.meta, self.kv_page_indices, self.kv_page_indptr,
                          self.max_pages_per_req, self.meta_planes, self.plane_slots)

    @classmethod
    def from_dense(cls, k: torch.Tensor, v: torch.Tensor, device, page_perm: Optional[torch.Tensor] = None,
                   spare_pages: int = 0, plane_pages: Optional[int] = None) -> "PagedKVCache":
        """Page dense ``k`` / ``v`` [B, Hkv, N, 128] (prefill fill). ``page_perm`` (a permutation of
        ``B*ceil(N/16)`` ids) scatters logical pages over physical slots."""
        B, Hkv, N, D = k.shape
        assert D == HEAD_DIM and v.shape == k.shape
        npg = (N + PAGE - 1) // PAGE
        total = B * npg
        c = cls(total + spare_pages, Hkv, k.dtype, device)
        if page_perm is None:
            page_perm = torch.arange(total)
        page_perm = page_perm.long()

        def paged(x):
            pad = npg * PAGE - N
            if pad:
                x = torch.nn.functional.pad(x, (0, 0, 0, pad))
            return x.reshape(B, Hkv, npg, PAGE, D).permute(0, 2, 3, 1, 4).reshape(total, PAGE, Hkv, D)

        perm_dev = page_perm.to(c.device)
        c.k_cache[perm_dev] = paged(k).to(c.device)
        c.v_cache[perm_dev] = paged(v).to(c.device)
        last = N - (npg - 1) * PAGE
        c.set_page_table(page_perm.to(torch.int32), (torch.arange(B + 1) * npg).to(torch.int32),
                         torch.full((B,), last, dtype=torch.int32))
        # valid tokens per physical page: 16 everywhere except each request's last page
        valid = torch.full((total + spare_pages,), PAGE, dtype=torch.int32)
        last_pages = page_perm.reshape(B, npg)[:, -1]
        valid[last_pages] = last
        ids = torch.arange(total + spare_pages, dtype=torch.int32)
        c.rebuild_shadow(ids.to(c.device), valid.to(c.device))
        if plane_pages is not None:
            c.enable_planes(plane_pages)
        return c

    def append(self, k_new: torch.Tensor, v_new: torch.Tensor, free_pages: Optional[list] = None) -> None:
        """Decode append of one token per request: ``k_new`` / ``v_new`` [B, Hkv, 128]. Extends the
        page table when a request's last page is full (taking ids from ``free_pages``; host-side
        bookkeeping only, nothing is read back from the device), then one kernel writes the token
        and updates the shadow records and the lengths. The two halves are also callable on their
        own: :meth:`advance_host` every step before a recorded step is replayed,
        :meth:`append_device` inside the recorded step."""
        self.advance_host(free_pages)
        self.append_device(k_new, v_new)

    def advance_host(self, free_pages: Optional[list] = None) -> None:
        """Host half of :meth:`append`: make room for one more token per request (a new page from
        ``free_pages`` where the last one is full) and count the token."""
        B = self.batch
        per_req, last = self._per_req, self._last
        grew = False
        if self._room <= 0:  # some request may have filled its last page
            for b in range(B):
                if last[b] == PAGE:
                    if not free_pages:
                        raise RuntimeError("PagedKVCache.append: no free page left")
                    per_req[b].append(int(free_pages.pop(0)))
                    last[b] = 0
                    grew = True
            self._room = PAGE - max(last)
        if grew:  # a request took a new page: the CSR arrays change shape, lengths are re-sent
            flat = [p for r in per_req for p in r]
            ptr = [0]
            for r in per_req:
                ptr.append(ptr[-1] + len(r))
            if self._table_cap:
                if max(len(r) for r in per_req) > self._table_cap:
                    raise RuntimeError("PagedKVCache.append: request outgrew reserve_page_table")
                self.kv_page_indices[:len(flat)].copy_(torch.tensor(flat, dtype=torch.int32))
                self.kv_page_indptr.copy_(torch.tensor(ptr, dtype=torch.int32))
            else:
                self.kv_page_indices = torch.tensor(flat, dtype=torch.int32, device=self.device)
                self.kv_page_indptr = torch.tensor(ptr, dtype=torch.int32, device=self.device)
                self.max_pages_per_req = max(len(r) for r in per_req)
            if self.meta_planes is not None and self.max_pages_per_req > self.meta_planes.size(4):
                raise RuntimeError("PagedKVCache.append: request outgrew the plane buffer "
                                   "(enable_planes with a larger cap_pages)")
            # same tensor object every step, so cached argument blocks of the layer stay valid
            self.kv_last_page_len.copy_(torch.tensor(last, dtype=torch.int32))
        self._room -= 1
        for b in range(B):
            last[b] += 1
            self._seq_lens[b] += 1

    def append_device(self, k_new: torch.Tensor, v_new: torch.Tensor) -> None:
        """Device half of :meth:`append`: one launch writes the token of every request at the
        position the device-side lengths give (and adds one to them), its INT4 codes and the
        min/max fold. :meth:`advance_host` must have made room for it."""
        B = self.batch
        if k_new.device != self.device or k_new.dtype != self.dtype:
            k_new = k_new.to(self.device, self.dtype)
        if v_new.device != self.device or v_new.dtype != self.dtype:
            v_new = v_new.to(self.device, self.dtype)
        if k_new.stride(-1) != 1 or v_new.stride() != k_new.stride():
            k_new, v_new = k_new.contiguous(), v_new.contiguous()
        # one launch: rows, INT4 codes, min/max metadata, and the device-side lengths + 1. The
        # operands are checked (kv_append) when any of them changes; between such changes the
        # call goes straight to the library with the checked shapes.
        planes = self.meta_planes
        slots = self.plane_slots if planes is not None else None
        key = (tuple(k_new.shape), k_new.stride(), k_new.dtype, self.k_cache.data_ptr(),
               self.v_cache.data_ptr(), self.kv_page_indices.data_ptr(),
               self.kv_page_indptr.data_ptr(), self.kv_last_page_len.data_ptr(),
               self.k_int4.data_ptr(), self.meta.data_ptr(),
               0 if planes is None else planes.data_ptr(), 0 if slots is None else slots.data_ptr())
        if key != self._append_key:
            kv_append(k_new, v_new, self.k_cache, self.v_cache, self.kv_page_indices,
                      self.kv_page_indptr, self.kv_last_page_len, self.k_int4, self.meta, planes, slots)
            self._append_key = key
        else:
            ks = self.k_cache.stride()
            with torch.cuda.device(self.device):
                rc = _lib.lib().twl_kv_append(
                    k_new.data_ptr(), v_new.data_ptr(), _lib.TWL_F16 if self.dtype == torch.float16
                    else _lib.TWL_BF16, k_new.stride(0), k_new.stride(1), self.k_cache.data_ptr(),
                    self.v_cache.data_ptr(), ks[0], ks[1], ks[2], self.kv_page_indices.data_ptr(),
                    self.kv_page_indptr.data_ptr(), self.kv_last_page_len.data_ptr(), B,
                    self.num_kv_heads, self.k_int4.data_ptr(), self.meta.data_ptr(),
                    0 if planes is None else planes.data_ptr(),
                    0 if planes is None else planes.size(4),
                    0 if slots is None else slots.data_ptr(),
                    0 if planes is None else planes.size(0),
                    torch.cuda.current_stream(self.device).cuda_stream)
            _lib.check(rc, "KvAppend")
