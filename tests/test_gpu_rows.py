"""The row gather/scatter through the C ABI and snapshot marks on the device, bit for bit:

* the reference's own vector (crates/glm53f-forward/tests/gemv.rs:333-358) and seeded cases against the oracle,
  over every lanes-per-row choice of the short-row kernel, the long-row kernel's full and partial spans, strides
  above the row size, more than 65,535 rows, and bytes next to the rows left alone;
* the argument checks of crates/glm53f-forward/kernels/glue.cu:221-233;
* a mark of the full model's layout (376 pages in f32, 195 with bf16 KDA states; kv_plan.rs:59-97): its pages
  against the oracle's, rewind after the slot is overwritten, host images out and in (kv.rs:618-720);
* the snapshot as an operation of the engine (crates/glm53f-forward/tests/snapshot.rs:66-140): decode rounds of
  the KDA kernels on the pool's arenas continue bit for bit after a rewind and in a forked slot.
"""
import numpy as np
import pytest
import torch

from glm53f_forward import ffi as rf
from glm53f_forward.kv import GlmKv, KvError, KvPool
from glm53f_forward.kvplan import TAIL, KvLayout, OutOfMemory
from glm53f_kda import DK, WINDOW, channels, ffi, state_len
from oracle import kda_oracle as o
from oracle import rows_oracle as ro

import harness as hs

pytestmark = pytest.mark.gpu
DEV = hs.DEV


def dev(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a).to(DEV)


def run(fn, src, src_stride, idx, dst, dst_stride, rows, nbytes):
    d_src, d_dst = dev(src), dev(dst)
    d_idx = dev(np.asarray(idx, dtype=np.int32)) if idx is not None and len(idx) else torch.zeros(1, dtype=torch.int32, device=DEV)
    rc = fn(hs.ptr(d_src), src_stride, hs.ptr(d_idx), hs.ptr(d_dst), dst_stride, rows, nbytes, None)
    hs.sync()
    return rc, d_dst.cpu().numpy()


def test_reference_vector():
    src = np.array([(i * 7) % 251 for i in range(10 * 64)], dtype=np.uint8)
    idx = [7, 2, 9]
    rc, got = run(rf.glm53f_fwd_gather_rows, src, 64, idx, np.zeros(3 * 48, dtype=np.uint8), 48, 3, 48)
    assert rc == 0
    rc, back = run(rf.glm53f_fwd_scatter_rows, got, 48, idx, np.zeros(10 * 64, dtype=np.uint8), 64, 3, 48)
    assert rc == 0
    for i, row in enumerate(idx):
        assert (got[i * 48:(i + 1) * 48] == src[row * 64:row * 64 + 48]).all()
        assert (back[row * 64:row * 64 + 48] == src[row * 64:row * 64 + 48]).all()


# (pieces per row, rows moved, rows on the indexed side, extra stride pieces src, dst)
CASES = [(1, 7, 20, 0, 0), (1, 70_000, 70_000, 0, 1), (3, 300, 1000, 1, 0), (5, 33, 40, 2, 3), (17, 257, 300, 0, 0),
         (100, 64, 64, 4, 0), (255, 9, 12, 0, 1), (256, 10, 10, 0, 0), (1000, 6, 9, 3, 0), (1023, 5, 5, 0, 0),
         (1024, 5, 8, 0, 2), (2048, 4, 4, 0, 0), (2049, 3, 6, 1, 1), (24_684, 11, 14, 0, 0), (5000, 40, 50, 0, 0)]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"{c[0]}x16B-{c[1]}rows")
def test_gather_and_scatter_match_the_oracle(case):
    chunks, rows, n_indexed, pad_s, pad_d = case
    rng = np.random.default_rng(chunks * 31 + rows)
    nbytes = 16 * chunks
    idx = rng.permutation(n_indexed)[:rows].astype(np.int32)
    # gather: src is the indexed side
    s_stride, d_stride = nbytes + 16 * pad_s, nbytes + 16 * pad_d
    src = rng.integers(0, 256, n_indexed * s_stride, dtype=np.uint8)
    dst = rng.integers(0, 256, rows * d_stride, dtype=np.uint8)
    want = dst.copy()
    assert ro.gather_rows(src, s_stride, idx, want, d_stride, rows, nbytes) == 0
    rc, got = run(rf.glm53f_fwd_gather_rows, src, s_stride, idx, dst, d_stride, rows, nbytes)
    assert rc == 0 and np.array_equal(got, want)
    # scatter: dst is the indexed side
    src2 = rng.integers(0, 256, rows * d_stride, dtype=np.uint8)
    dst2 = rng.integers(0, 256, n_indexed * s_stride, dtype=np.uint8)
    want2 = dst2.copy()
    assert ro.scatter_rows(src2, d_stride, idx, want2, s_stride, rows, nbytes) == 0
    rc, got2 = run(rf.glm53f_fwd_scatter_rows, src2, d_stride, idx, dst2, s_stride, rows, nbytes)
    assert rc == 0 and np.array_equal(got2, want2)
    # scatter undoes gather on the indexed rows
    rc, back = run(rf.glm53f_fwd_scatter_rows, got, d_stride, idx, np.zeros_like(src), s_stride, rows, nbytes)
    assert rc == 0
    for i in idx[:50]:
        assert np.array_equal(back[i * s_stride:i * s_stride + nbytes], src[i * s_stride:i * s_stride + nbytes])


def test_argument_checks():
    buf = torch.zeros(4096, dtype=torch.uint8, device=DEV)
    idx = torch.zeros(4, dtype=torch.int32, device=DEV)
    p, q, ix = hs.ptr(buf), hs.ptr(buf, 2048), hs.ptr(idx)
    for fn in (rf.glm53f_fwd_gather_rows, rf.glm53f_fwd_scatter_rows):
        assert fn(p, 64, ix, q, 64, 0, 64, None) == 0            # no rows: nothing to do
        assert fn(p, 64, ix, q, 64, 2, 0, None) == 0             # no bytes
        assert fn(None, 64, None, None, 64, 0, 64, None) == 0     # the empty case is accepted before the pointers
        assert fn(p, 64, ix, q, 64, -1, 64, None) == 1
        assert fn(p, 64, ix, q, 64, 1, -16, None) == 1
        assert fn(p, 64, ix, q, 64, 1, 24, None) == 1            # bytes % 16
        assert fn(p, 72, ix, q, 64, 1, 64, None) == 1            # src stride % 16
        assert fn(p, 64, ix, q, 40, 1, 32, None) == 1            # dst stride % 16
        assert fn(p, 32, ix, q, 64, 1, 64, None) == 1            # src stride below the row
        assert fn(p, 64, ix, q, 32, 1, 64, None) == 1            # dst stride below the row
        assert fn(p + 8, 64, ix, q, 64, 1, 64, None) == 1        # src not 16-byte aligned
        assert fn(p, 64, ix, q + 4, 64, 1, 64, None) == 1        # dst not 16-byte aligned
        assert fn(p, 64, None, q, 64, 1, 64, None) == 1          # no index
        assert fn(None, 64, ix, q, 64, 1, 64, None) == 1
    hs.sync()
    assert int(buf.sum()) == 0


def fill_slot(kv: GlmKv, seed: int) -> None:
    """Seeded bytes in the slot's three regions; the tails get a plausible count word first."""
    l, p = kv.pool.layout, kv.pool
    g = torch.Generator(device=DEV).manual_seed(seed)
    for arena, at, n in ((p.state, kv.state_at(), l.kda_state_bytes()), (p.conv, kv.conv_at(), l.conv_bytes()),
                         (p.tails, kv.tails_at(), l.tails_bytes())):
        arena[at:at + n] = torch.randint(0, 256, (n,), device=DEV, generator=g, dtype=torch.uint8)
    for j in range(l.dsa_layers):
        count = torch.tensor([(seed + j) % 4, 0, 0, 0], dtype=torch.uint8, device=DEV)
        p.tails[kv.tails_at() + j * TAIL:kv.tails_at() + j * TAIL + 4] = count


def slot_image(kv: GlmKv) -> np.ndarray:
    l, p = kv.pool.layout, kv.pool
    return torch.cat([p.state[kv.state_at():kv.state_at() + l.kda_state_bytes()],
                      p.conv[kv.conv_at():kv.conv_at() + l.conv_bytes()],
                      p.tails[kv.tails_at():kv.tails_at() + l.tails_bytes()]]).cpu().numpy()


@pytest.mark.parametrize("bf16", [True, False], ids=["bf16-states-195-pages", "f32-states-376-pages"])
def test_full_model_mark_pages_rewind_and_host_images(bf16):
    l = KvLayout().with_kda_state_bf16(bf16)
    assert l.mark_pages() == (195 if bf16 else 376)
    pool = KvPool(l, slots=2, pages=l.mark_pages() + 7)
    spare = [pool.alloc.alloc() for _ in range(3)]      # so that the mark's pages are not 0..n-1
    _ = pool.slot()
    kv = pool.slot()                                    # slot 1
    assert kv.slot == 1
    pool.alloc.release(spare[1])                        # a hole: the page list is not one run
    fill_slot(kv, 11)
    kv.tokens = 72
    image = slot_image(kv)
    free0 = pool.free_pages()
    m = kv.mark()
    hs.sync()
    assert (m.tokens, m.pages(), m.bytes()) == (72, l.mark_pages(), l.mark_bytes())
    assert pool.free_pages() == free0 - l.mark_pages()
    pages = m.page_list()
    assert pages == sorted(pages) and pages[0] == 1 and pages[1] == 3
    # the pool's pages against the oracle's copy of the same slot into the same pages
    want_pages = np.zeros(pool.pages.numel(), dtype=np.uint8)
    s, c = l.kda_state_bytes(), l.conv_bytes()
    host_arenas = [(image[:s].copy(), 0), (image[s:s + c].copy(), 0), (image[s + c:].copy(), 0)]
    ro.copy_mark(l.mark_regions(), l.page_bytes, pages, want_pages, host_arenas, True)
    assert np.array_equal(pool.pages.cpu().numpy(), want_pages)
    # the slot moves on, then goes back
    kv.tokens = 80
    fill_slot(kv, 12)
    assert not np.array_equal(slot_image(kv), image)
    with pytest.raises(KvError):
        kv.rewind(71, m)
    kv.rewind(72, m)
    hs.sync()
    assert kv.tokens == 72 and np.array_equal(slot_image(kv), image)
    # host image: the slot's bytes but for the tail slots past each count
    want = image.copy()
    base = s + c
    for j in range(l.dsa_layers):
        n = min(int(want[base + j * TAIL]), 3)
        want[base + j * TAIL + 16 + n * 512:base + (j + 1) * TAIL] = 0
    exported = kv.export_state(m)
    assert np.array_equal(exported, want)
    # a restore into another slot re-exports the same image; the first slot is untouched
    other = GlmKv(pool, 0)
    other.tokens = 72
    other.import_state(72, exported)
    with pytest.raises(KvError):
        other.import_state(71, exported)
    with pytest.raises(OutOfMemory):
        other.mark()                                    # the pool has too few pages for a second mark
    m.release()
    assert pool.free_pages() == free0
    m2 = other.mark()
    hs.sync()
    assert np.array_equal(other.export_state(m2), want)
    assert np.array_equal(slot_image(kv), image)


H, L = 64, 2
C, N, CW = channels(H), state_len(H), WINDOW * channels(H)
P_COLS, WIDTH = C + H, H * DK


def decode_round(pool: KvPool, layers, weights, slots, p_rows, ag_rows):
    """One decode row per slot through every layer on the pool's arenas (chain in place, then the conv shift);
    returns the layers' outputs."""
    meta = hs.BatchMeta([1] * len(slots), [s * L * CW for s in slots], [s * L * N for s in slots], None)
    state = pool.state.view(torch.bfloat16)
    conv = pool.conv.view(torch.bfloat16)
    outs = []
    for j in range(L):
        p, ag, w = p_rows[j], ag_rows[j], weights[j]
        out = torch.zeros(meta.total, WIDTH, device=DEV, dtype=torch.bfloat16)
        st_l, cv_l = hs.ptr(state, j * N), hs.ptr(conv, j * CW)
        hs.check(ffi.glm53f_kda_chain_batch_bf16state(
            H, meta.batch, hs.ptr(meta.cu_rows), hs.ptr(p), P_COLS, C, hs.ptr(ag), 2 * WIDTH, hs.ptr(ag, WIDTH),
            2 * WIDTH, cv_l, hs.ptr(meta.conv_off), hs.ptr(w.conv_w), st_l, st_l, hs.ptr(meta.state_off), *w.args(),
            hs.ptr(out), WIDTH, None, None, None, None, None), "chain")
        hs.check(ffi.glm53f_kda_conv_shift_batch(C, 1, meta.batch, hs.ptr(meta.cu_rows), hs.ptr(meta.keep), cv_l, 0,
                                                 hs.ptr(meta.conv_off), hs.ptr(p), 0, P_COLS, None), "conv shift")
        outs.append(out)
    hs.sync()
    return outs


def test_decode_continues_bit_for_bit_after_rewind_and_in_a_fork():
    l = KvLayout(kda_layers=L, dsa_layers=1, kda_state_bf16=True)
    pool = KvPool(l, slots=3, pages=2 * l.mark_pages() + 2)
    a, b, c = pool.slot(), pool.slot(), pool.slot()
    g = torch.Generator(device=DEV).manual_seed(77)
    pool.state.view(torch.bfloat16)[:] = (torch.randn(3 * L * N, device=DEV, generator=g) * 0.05).to(torch.bfloat16)
    pool.conv.view(torch.bfloat16)[:] = torch.randn(3 * L * CW, device=DEV, generator=g).to(torch.bfloat16)
    layers = [o.synth_layer(H, 300 + j) for j in range(L)]
    weights = [hs.Weights(p) for p in layers]

    def rows(n):
        return ([torch.randn(n, P_COLS, device=DEV, generator=g).to(torch.bfloat16) for _ in range(L)],
                [torch.randn(n, 2 * WIDTH, device=DEV, generator=g).to(torch.bfloat16) for _ in range(L)])

    # two rounds on slots a and c, a mark of a, three more rounds
    for _ in range(2):
        decode_round(pool, layers, weights, [a.slot, c.slot], *rows(2))
    a.tokens = 2
    m = a.mark()
    c_before = slot_image(c)
    later = [rows(1) for _ in range(3)]
    first = [decode_round(pool, layers, weights, [a.slot], *r) for r in later]
    a.tokens = 5
    after5 = slot_image(a)
    # back to the mark: the same rows give the same bits
    a.rewind(2, m)
    again = [decode_round(pool, layers, weights, [a.slot], *r) for r in later]
    for x, y in zip(first, again):
        for j in range(L):
            assert torch.equal(x[j], y[j])
    assert np.array_equal(slot_image(a), after5)
    # a fork of the mark into slot b continues the same way; slot c never moved
    b.fork(a, 2, m)
    forked = [decode_round(pool, layers, weights, [b.slot], *r) for r in later]
    for x, y in zip(first, forked):
        for j in range(L):
            assert torch.equal(x[j], y[j])
    assert np.array_equal(slot_image(b), after5)
    assert np.array_equal(slot_image(c), c_before)
    with pytest.raises(KvError):
        b.fork(a, 3, m)
