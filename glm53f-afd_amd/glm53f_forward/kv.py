"""Device side of snapshot marks: a slot's positional state saved into pages of the pool and loaded back
(reference: crates/glm53f-forward/src/kv.rs:385-478 `copy_mark`, :482-545 `mark` / `rewind`, :618-720 host
images). Each part's whole pages move by one scatter (save) or gather (load) launch of the HIP library, its
last partial page by a device copy. Device memory is torch's; every copy runs on the current stream.
"""
from typing import List, Optional

import numpy as np
import torch

from . import ffi
from .kvplan import TAIL, KvLayout, OutOfMemory, PageAlloc


class KvError(Exception):
    """An argument the reference rejects as invalid."""


def _ptr(t: torch.Tensor, byte: int = 0) -> int:
    return t.data_ptr() + byte


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _launched(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what}: hipError {rc}")


class KvPool:
    """The arenas (kv.rs:120-150): `pages` [pages][page_bytes]; per slot `state` [slots][kda_state_bytes],
    `conv` [slots][conv_bytes], `tails` [slots][max(tails_bytes, 16)]; the device list of a mark's pages."""

    def __init__(self, layout: KvLayout, slots: int, pages: int, device: str = "cuda:0"):
        self.layout, self.max_slots, self.device = layout, slots, torch.device(device)
        u8 = dict(dtype=torch.uint8, device=self.device)
        self.pages = torch.zeros(pages * layout.page_bytes, **u8)
        self.state = torch.zeros(slots * layout.kda_state_bytes(), **u8)
        self.conv = torch.zeros(slots * layout.conv_bytes(), **u8)
        self.tails = torch.zeros(slots * max(layout.tails_bytes(), 16), **u8)
        self.mark_index = torch.zeros(max(layout.mark_pages(), 1), dtype=torch.int32, device=self.device)
        self.alloc = PageAlloc(pages)
        self._free_slots = list(range(slots - 1, -1, -1))

    def free_pages(self) -> int:
        return self.alloc.free()

    def slot(self) -> "GlmKv":
        if not self._free_slots:
            raise OutOfMemory("no free slot")
        return GlmKv(self, self._free_slots.pop())


class KvMark:
    """The pool pages holding a saved state, the three parts in order; `release()` gives them back (the
    reference's Drop, kv.rs:229-236)."""

    def __init__(self, pool: KvPool, tokens: int, pages: List[int]):
        self.pool, self.tokens, self._pages = pool, tokens, pages

    def bytes(self) -> int:
        return self.pool.layout.mark_bytes()

    def pages(self) -> int:
        return len(self._pages)

    def page_list(self) -> List[int]:
        return list(self._pages)

    def release(self) -> None:
        for p in self._pages:
            self.pool.alloc.release(p)
        self._pages = []


class GlmKv:
    """One request's positional state (the paged rows of the DSA layers are not part of this path)."""

    def __init__(self, pool: KvPool, slot: int):
        self.pool, self.slot, self.tokens, self.pending = pool, slot, 0, 0

    # ---- regions (kv.rs:387-397)
    def state_at(self) -> int:
        return self.slot * self.pool.layout.kda_state_bytes()

    def conv_at(self) -> int:
        return self.slot * self.pool.layout.conv_bytes()

    def tails_at(self) -> int:
        return self.slot * max(self.pool.layout.tails_bytes(), 16)

    def clear_state(self) -> None:
        l, p = self.pool.layout, self.pool
        p.state[self.state_at():self.state_at() + l.kda_state_bytes()].zero_()
        p.conv[self.conv_at():self.conv_at() + l.conv_bytes()].zero_()
        p.tails[self.tails_at():self.tails_at() + l.tails_bytes()].zero_()

    def _arenas(self):
        p = self.pool
        return [(p.state, self.state_at()), (p.conv, self.conv_at()), (p.tails, self.tails_at())]

    def copy_mark(self, mark: KvMark, save: bool) -> None:
        """Copy the positional state into the mark's pages (save) or out of them into the slot (kv.rs:412-478)."""
        if mark.pool is not self.pool:
            raise KvError("a mark of another pool")
        l, p = self.pool.layout, self.pool
        pb = l.page_bytes
        pages = mark.page_list()
        # the list buffer is reused in stream order
        p.mark_index[:len(pages)].copy_(torch.tensor(pages, dtype=torch.int32))
        first = 0
        for (arena, at), (_, n, count) in zip(self._arenas(), l.mark_regions()):
            full, rem = divmod(n, pb)
            if full > 0:
                idx = _ptr(p.mark_index, 4 * first)
                if save:
                    rc = ffi.glm53f_fwd_scatter_rows(_ptr(arena, at), pb, idx, _ptr(p.pages), pb, full, pb, _stream())
                else:
                    rc = ffi.glm53f_fwd_gather_rows(_ptr(p.pages), pb, idx, _ptr(arena, at), pb, full, pb, _stream())
                _launched(rc, "mark pages")
            if rem > 0:
                page = pages[first + full] * pb
                if save:
                    p.pages[page:page + rem].copy_(arena[at + full * pb:at + full * pb + rem])
                else:
                    arena[at + full * pb:at + full * pb + rem].copy_(p.pages[page:page + rem])
            first += count

    def mark(self) -> KvMark:
        """Save the positional state at the current position in pages of the pool; OutOfMemory (nothing
        allocated) when too few are free (kv.rs:482-510)."""
        if self.pending != 0:
            raise KvError("mark inside an uncommitted verify window")
        need, a = self.pool.layout.mark_pages(), self.pool.alloc
        if a.free() < need:
            raise OutOfMemory(f"a snapshot mark takes {need} pages of the KV pool, {a.free()} are free")
        pages = sorted(a.alloc() for _ in range(need))
        mark = KvMark(self.pool, self.tokens, pages)
        self.copy_mark(mark, True)
        return mark

    def rewind(self, to: int, mark: KvMark) -> None:
        """Go back to `to` tokens, where `mark` was taken in this slot's history (kv.rs:513-541)."""
        if mark.tokens != to or to > self.tokens:
            raise KvError(f"rewind to {to} with a mark at {mark.tokens} (the slot holds {self.tokens})")
        self.copy_mark(mark, False)
        self.tokens, self.pending = to, 0

    def fork(self, src: "GlmKv", to: int, mark: KvMark) -> None:
        """Become `src`'s first `to` tokens at `mark`: the mark's state loaded (kv.rs:545-575)."""
        if self.pool is not src.pool:
            raise KvError("fork across pools")
        if mark.tokens != to or to > src.tokens:
            raise KvError(f"fork of {to} tokens with a mark at {mark.tokens} from a slot of {src.tokens}")
        self.clear_state()
        self.copy_mark(mark, False)
        self.tokens, self.pending = to, 0

    # ---- host images (kv.rs:618-720)
    def state_bytes(self) -> int:
        return self.pool.layout.mark_bytes()

    def export_state(self, mark: KvMark) -> np.ndarray:
        """The mark's positional state as a host image [states | conv windows | tails]; tail slots past each
        tail's count are zeroed, so the image depends only on the committed tokens (kv.rs:618-662)."""
        if mark.pool is not self.pool:
            raise KvError("the mark is another pool's")
        l, p = self.pool.layout, self.pool
        pb = l.page_bytes
        dst = np.zeros(l.mark_bytes(), dtype=np.uint8)
        pages, first = mark.page_list(), 0
        for off, n, count in l.mark_regions():
            k = 0
            while k < count:
                run = 1
                while k + run < count and pages[first + k + run] == pages[first + k] + run:
                    run += 1
                nbytes = min(n - k * pb, run * pb)
                at = pages[first + k] * pb
                dst[off + k * pb:off + k * pb + nbytes] = p.pages[at:at + nbytes].cpu().numpy()
                k += run
            first += count
        base = l.kda_state_bytes() + l.conv_bytes()
        for j in range(l.dsa_layers):
            t = dst[base + j * TAIL:base + (j + 1) * TAIL]
            n = min(int(t[:4].view("<u4")[0]), 3)
            t[16 + n * 512:] = 0
        return dst

    def import_state(self, tokens: int, src: np.ndarray) -> None:
        """Finish a restore of `tokens` tokens: load the positional state image (kv.rs:697-720)."""
        l, p = self.pool.layout, self.pool
        if tokens != self.tokens or src.size != l.mark_bytes() or src.dtype != np.uint8:
            raise KvError(f"import_state({tokens}) after {self.tokens} imported rows, {src.size} bytes")
        s, c = l.kda_state_bytes(), l.conv_bytes()
        img = torch.from_numpy(np.ascontiguousarray(src))
        p.state[self.state_at():self.state_at() + s].copy_(img[:s])
        p.conv[self.conv_at():self.conv_at() + c].copy_(img[s:s + c])
        p.tails[self.tails_at():self.tails_at() + l.tails_bytes()].copy_(img[s + c:])

    # ---- typed views of this slot's regions, for the KDA kernels
    def state_view(self) -> torch.Tensor:
        l = self.pool.layout
        raw = self.pool.state[self.state_at():self.state_at() + l.kda_state_bytes()]
        return raw.view(torch.bfloat16 if l.kda_state_bf16 else torch.float32)

    def conv_view(self) -> torch.Tensor:
        l = self.pool.layout
        return self.pool.conv[self.conv_at():self.conv_at() + l.conv_bytes()].view(torch.bfloat16)
