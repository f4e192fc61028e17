"""CPU tests of the snapshot path's host side: the layout's known answers (the reference's
crates/glm53f-forward/tests/kv_plan.rs:28-105), the page allocator's order (kvplan.rs:150-200), the oracle of the
row gather/scatter against the reference's own vector (crates/glm53f-forward/tests/gemv.rs:333-358) and brute
force, and the C ABI of include/glm53f_fwd_rows.h as a boundary (symbols and prototypes; no compute call)."""
import os
import re

import numpy as np
import pytest

from glm53f_forward import ffi as rows_ffi
from glm53f_forward.kvplan import LAYER_PAGE_BYTES, PAGE, TAIL, KvLayout, PageAlloc
from oracle import rows_oracle as ro

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_layout_known_answers_full_model():
    l = KvLayout()
    assert l.page_bytes == 394_944 == 64 * 6_171
    assert l.kda_state_bytes() == 136 << 20
    assert l.conv_bytes() == 34 * 3 * 24_576 * 2
    assert l.tails_bytes() == 17_072
    regions = l.mark_regions()
    assert [r[2] for r in regions] == [362, 13, 1]
    assert [r[0] for r in regions] == [0, l.kda_state_bytes(), l.kda_state_bytes() + l.conv_bytes()]
    assert sum(r[1] for r in regions) == l.mark_bytes()
    assert l.mark_pages() == 376
    assert l.mark_pages() * l.page_bytes >= l.mark_bytes()
    for tokens in (1, 63, 64, 65, 4096, 262_144):
        assert l.paged_bytes(tokens) == -(-tokens // PAGE) * l.page_bytes
    assert l.slot_fixed_bytes() == l.mark_bytes()
    assert KvLayout(draft_kv_bytes=1 << 20).slot_fixed_bytes() == l.mark_bytes() + (1 << 20)


def test_layout_known_answers_layer_prefix_and_bf16_states():
    s5 = KvLayout(kda_layers=4, dsa_layers=1)
    assert s5.page_bytes == LAYER_PAGE_BYTES == 35_904
    assert s5.mark_pages() == 468 + 17 + 1
    f = KvLayout()
    b = f.with_kda_state_bf16(True)
    assert (f.kda_state_elem_bytes(), b.kda_state_elem_bytes()) == (4, 2)
    assert b.kda_state_bytes() == 68 << 20
    assert b.conv_bytes() == f.conv_bytes()
    assert b.mark_bytes() == f.mark_bytes() - (68 << 20)
    assert [r[2] for r in b.mark_regions()] == [181, 13, 1]
    assert b.mark_pages() == 195
    assert b.mark_pages() * b.page_bytes >= b.mark_bytes()
    # no DSA layer: a page still has one layer's bytes, and the tails take no page
    k = KvLayout(kda_layers=2, dsa_layers=0)
    assert k.page_bytes == LAYER_PAGE_BYTES and k.tails_bytes() == 0 and k.mark_regions()[2][2] == 0
    assert TAIL == 1_552


def test_page_alloc_order_and_counts():
    a = PageAlloc(4)
    assert (a.total(), a.free()) == (4, 4)
    assert [a.alloc() for _ in range(3)] == [0, 1, 2]
    a.share(1)
    assert a.refs(1) == 2
    assert not a.release(1) and a.release(1)
    assert a.alloc() == 1                       # a released page is the next one out
    assert a.alloc() == 3 and a.alloc() is None
    with pytest.raises(AssertionError):
        PageAlloc(1).release(0)


def test_oracle_on_the_reference_vector():
    src = np.array([(i * 7) % 251 for i in range(10 * 64)], dtype=np.uint8)
    idx = [7, 2, 9]
    got = np.zeros(3 * 48, dtype=np.uint8)
    assert ro.gather_rows(src, 64, idx, got, 48, 3, 48) == 0
    back = np.zeros(10 * 64, dtype=np.uint8)
    assert ro.scatter_rows(got, 48, idx, back, 64, 3, 48) == 0
    for i, row in enumerate(idx):
        assert (got[i * 48:(i + 1) * 48] == src[row * 64:row * 64 + 48]).all()
        assert (back[row * 64:row * 64 + 48] == src[row * 64:row * 64 + 48]).all()
    touched = np.zeros(10 * 64, dtype=bool)
    for row in idx:
        touched[row * 64:row * 64 + 48] = True
    assert (back[~touched] == 0).all()          # nothing else is written


def test_oracle_against_byte_loops_and_argument_checks():
    rng = np.random.default_rng(5)
    src = rng.integers(0, 256, 9 * 80, dtype=np.uint8)
    idx = rng.permutation(9)[:5]
    got = np.full(5 * 96, 0xEE, dtype=np.uint8)
    assert ro.gather_rows(src, 80, idx, got, 96, 5, 32) == 0
    for i in range(5):
        for b in range(96):
            want = src[idx[i] * 80 + b] if b < 32 else 0xEE
            assert got[i * 96 + b] == want
    d = np.zeros(16, dtype=np.uint8)
    assert ro.gather_rows(src, 80, idx, d, 16, 0, 16) == 0          # no rows
    assert ro.gather_rows(src, 80, idx, d, 16, 1, 0) == 0           # no bytes
    assert ro.gather_rows(src, 80, idx, d, 16, -1, 16) == ro.INVALID
    assert ro.gather_rows(src, 80, idx, d, 16, 1, 24) == ro.INVALID  # bytes not a multiple of 16
    assert ro.gather_rows(src, 72, idx, d, 16, 1, 16) == ro.INVALID  # stride not a multiple of 16
    assert ro.gather_rows(src, 16, idx, d, 32, 1, 32) == ro.INVALID  # stride below the row size
    assert ro.scatter_rows(src, 80, None, d, 16, 1, 16) == ro.INVALID


def test_oracle_mark_round_trip():
    l = KvLayout(kda_layers=1, dsa_layers=1, kda_state_bf16=True)
    rng = np.random.default_rng(9)
    pool_pages = l.mark_pages() + 5
    pages = np.zeros(pool_pages * l.page_bytes, dtype=np.uint8)
    sizes = [l.kda_state_bytes(), l.conv_bytes(), l.tails_bytes()]
    arenas = [(rng.integers(0, 256, 2 * n, dtype=np.uint8), n) for n in sizes]   # slot 1 of 2
    before = [a.copy() for a, _ in arenas]
    mark_pages = sorted(rng.permutation(pool_pages)[:l.mark_pages()].tolist())
    ro.copy_mark(l.mark_regions(), l.page_bytes, mark_pages, pages, arenas, True)
    for a, at in arenas:
        a[at:] = 0
    ro.copy_mark(l.mark_regions(), l.page_bytes, mark_pages, pages, arenas, False)
    for (a, _), b in zip(arenas, before):
        assert (a == b).all()
    # the pages hold the parts in order, each from a page of its own
    first = 0
    for (a, at), (_, n, count) in zip(arenas, l.mark_regions()):
        img = np.concatenate([pages[p * l.page_bytes:(p + 1) * l.page_bytes] for p in mark_pages[first:first + count]])
        assert (img[:n] == a[at:at + n]).all()
        first += count


def declarations():
    text = open(os.path.join(ROOT, "include", "glm53f_fwd_rows.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = {}
    for m in re.finditer(r"\bint32_t\s+(glm53f_fwd_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        out[m.group(1)] = len(m.group(2).split(","))
    return out


def test_library_exports_the_declared_row_entry_points():
    decl = declarations()
    assert set(decl) == {"glm53f_fwd_gather_rows", "glm53f_fwd_scatter_rows"} <= set(rows_ffi.PROTOTYPES)
    lib = rows_ffi.lib()
    for name, nargs in decl.items():
        assert hasattr(lib, name), name
        assert len(rows_ffi.PROTOTYPES[name][1]) == nargs == 8, name
