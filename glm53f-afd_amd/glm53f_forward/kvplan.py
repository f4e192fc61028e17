"""Byte layout of the device KV and the page accounting, on the host (reference:
crates/glm53f-forward/src/kvplan.rs:1-200; constants from crates/glm53f-dsa/src/cache.rs:48-64 and
crates/glm53f-forward/src/shape.rs).

Pages: one physical page holds 64 tokens of every DSA layer, 35,904 bytes per layer. Positional state, per slot:
the KDA states [kda_layers][64][128 v][128 k] in f32 or bf16, the bf16 conv windows [kda_layers][3][24,576], and
the DSA tails [dsa_layers][1,552 B]. A mark saves all three in pages of the pool, each part from a page of its
own.
"""
from dataclasses import dataclass, replace

LAYER_PAGE_BYTES = 35_904     # 64 latent records of 528 B, 16 pooled keys of 128 B, 16 f32 scales
PAGE = 64                     # tokens per page
TAIL = 1_552                  # bytes of one DSA layer's tail
KDA_HEADS = 64
KDA_DIM = 128
KDA_QKV = 3 * KDA_HEADS * KDA_DIM
KDA_WINDOW = 3
# GLM-5.3-Flash (crates/glm53f-forward/tests/kv_plan.rs:43-67)
FULL_KDA_LAYERS = 34
FULL_DSA_LAYERS = 11


class OutOfMemory(Exception):
    """The pool has too few free pages (the reference's Error::OutOfMemory)."""


@dataclass(frozen=True)
class KvLayout:
    kda_layers: int = FULL_KDA_LAYERS
    dsa_layers: int = FULL_DSA_LAYERS
    draft_kv_bytes: int = 0
    kda_state_bf16: bool = False

    @property
    def page_bytes(self) -> int:
        """Every DSA layer's 64-token block (kvplan.rs:61)."""
        return max(self.dsa_layers, 1) * LAYER_PAGE_BYTES

    def with_kda_state_bf16(self, bf16: bool) -> "KvLayout":
        return replace(self, kda_state_bf16=bf16)

    @staticmethod
    def state_elems_per_layer() -> int:
        return KDA_HEADS * KDA_DIM * KDA_DIM

    def kda_state_elem_bytes(self) -> int:
        return 2 if self.kda_state_bf16 else 4

    @staticmethod
    def conv_elems_per_layer() -> int:
        return KDA_WINDOW * KDA_QKV

    def kda_state_bytes(self) -> int:
        return self.kda_layers * self.state_elems_per_layer() * self.kda_state_elem_bytes()

    def conv_bytes(self) -> int:
        return self.kda_layers * self.conv_elems_per_layer() * 2

    def tails_bytes(self) -> int:
        return self.dsa_layers * TAIL

    def mark_bytes(self) -> int:
        """A mark's positional state, also the size of its host image (kvplan.rs:104-108)."""
        return self.kda_state_bytes() + self.conv_bytes() + self.tails_bytes()

    def mark_regions(self):
        """The three parts as (offset in the host image, bytes, pool pages) (kvplan.rs:110-125)."""
        pb = self.page_bytes
        s, c, t = self.kda_state_bytes(), self.conv_bytes(), self.tails_bytes()
        return [(0, s, -(-s // pb)), (s, c, -(-c // pb)), (s + c, t, -(-t // pb))]

    def mark_pages(self) -> int:
        return sum(r[2] for r in self.mark_regions())

    def slot_fixed_bytes(self) -> int:
        return self.mark_bytes() + self.draft_kv_bytes

    @staticmethod
    def pages_for(tokens: int) -> int:
        return -(-tokens // PAGE)

    def paged_bytes(self, tokens: int) -> int:
        return self.pages_for(tokens) * self.page_bytes


class PageAlloc:
    """Reference counts and the free list of a pool of physical pages (kvplan.rs:150-200): the lowest free page
    is handed out first; a released page goes back on top of the list."""

    def __init__(self, pages: int):
        self._free = list(range(pages - 1, -1, -1))
        self._refs = [0] * pages

    def total(self) -> int:
        return len(self._refs)

    def free(self) -> int:
        return len(self._free)

    def refs(self, page: int) -> int:
        return self._refs[page]

    def alloc(self):
        if not self._free:
            return None
        p = self._free.pop()
        assert self._refs[p] == 0
        self._refs[p] = 1
        return p

    def share(self, page: int) -> None:
        assert self._refs[page] > 0, "sharing a free page"
        self._refs[page] += 1

    def release(self, page: int) -> bool:
        assert self._refs[page] > 0, "releasing a free page"
        self._refs[page] -= 1
        if self._refs[page] == 0:
            self._free.append(page)
            return True
        return False
