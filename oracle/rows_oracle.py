"""CPU restatement of the row gather/scatter and of a snapshot mark's page copies, in numpy.

TEST INFRASTRUCTURE ONLY: imported by tests, the smoke check and the benchmark's CPU-baseline leg, never by the
product path.

Follows the reference's crates/glm53f-forward/kernels/glue.cu:101-110 (the copy) and :221-244 (the argument
checks), and crates/glm53f-forward/src/kv.rs:412-478 (`copy_mark`: whole pages by one gather or scatter, the last
partial page by a copy, each part of the mark from a page of its own).

Pinned by: the reference's own vector (crates/glm53f-forward/tests/gemv.rs:333-358: ten 64-byte rows holding
i * 7 % 251, rows 7, 2, 9 gathered as 48-byte rows and scattered back), brute-force byte loops on small cases,
and the identity scatter(gather(x)) == x on the indexed rows (tests/test_rows.py).
"""
import numpy as np

INVALID = 1


def _check(src, src_stride, idx, dst, dst_stride, rows, nbytes):
    if (rows < 0 or nbytes < 0 or nbytes % 16 or src_stride % 16 or dst_stride % 16 or src_stride < nbytes
            or dst_stride < nbytes):
        return INVALID
    if rows == 0 or nbytes == 0:
        return 0
    if src is None or dst is None or idx is None:
        return INVALID
    return None


def gather_rows(src: np.ndarray, src_stride: int, idx, dst: np.ndarray, dst_stride: int, rows: int, nbytes: int) -> int:
    """dst[i] = src[idx[i]] for i < rows, on flat uint8 arrays (glue.cu:101-110 with scatter = 0)."""
    rc = _check(src, src_stride, idx, dst, dst_stride, rows, nbytes)
    if rc is not None:
        return rc
    for i in range(rows):
        s = int(idx[i]) * src_stride
        dst[i * dst_stride:i * dst_stride + nbytes] = src[s:s + nbytes]
    return 0


def scatter_rows(src: np.ndarray, src_stride: int, idx, dst: np.ndarray, dst_stride: int, rows: int, nbytes: int) -> int:
    """dst[idx[i]] = src[i] for i < rows (glue.cu:101-110 with scatter = 1)."""
    rc = _check(src, src_stride, idx, dst, dst_stride, rows, nbytes)
    if rc is not None:
        return rc
    for i in range(rows):
        d = int(idx[i]) * dst_stride
        dst[d:d + nbytes] = src[i * src_stride:i * src_stride + nbytes]
    return 0


def copy_mark(regions, page_bytes: int, mark_pages, pages: np.ndarray, arenas, save: bool) -> None:
    """kv.rs:412-478 on host arrays. `regions`: (offset, bytes, pool pages) of the three parts; `arenas`: one
    (flat uint8 array, byte offset of the slot's region) per part; `mark_pages`: the mark's pool pages, the parts
    in order; `pages`: the pool's flat page arena."""
    pb, first = page_bytes, 0
    for (arena, at), (_, n, count) in zip(arenas, regions):
        full, rem = divmod(n, pb)
        idx = list(mark_pages[first:first + full])
        if full > 0:
            if save:
                scatter_rows(arena[at:], pb, idx, pages, pb, full, pb)
            else:
                gather_rows(pages, pb, idx, arena[at:], pb, full, pb)
        if rem > 0:
            page = mark_pages[first + full] * pb
            if save:
                pages[page:page + rem] = arena[at + full * pb:at + full * pb + rem]
            else:
                arena[at + full * pb:at + full * pb + rem] = pages[page:page + rem]
        first += count
