"""
CPU model of the 16-byte loads of the one-read cross-entropy kernel (csrc/cross_entropy.hip,
ce_row_kernel): every lane issues CACHE_VECS loads without a branch, a lane with no vector at
its position reading the aligned 16 bytes that hold the first element of its row.  Whatever the
row width, dtype and alignment of the tensor, each such load must be 16-byte aligned and stay
inside the pages the tensor occupies (a load outside them is a GPU memory fault, not an error).
"""

import pytest

SHAPES = [(12288, 1), (5, 7), (8096, 32), (48, 50257), (9, 12345), (4, 131075), (1, 8000), (3, 8),
          (64, 33), (37, 129), (512, 4099), (2, 2), (7, 3), (3, 32768), (3, 32776), (2, 65536), (2, 49153)]


def check(batch, feat, elem_size, base):
    vec = 16 // elem_size
    # the launcher's choice: 512 lanes and up to 8 vectors per lane, 1024 lanes beyond 4096 vectors
    max_vecs = -(-feat // vec)
    block = 1024 if max_vecs > 512 * 8 else 512
    per_lane = -(-max_vecs // block)
    cache_vecs = next(c for c in ((6, 7, 8) if block == 1024 else (2, 4, 8)) if per_lane <= c) if max_vecs <= 8192 else 0
    first_page = base // 4096 * 4096
    end = base + batch * feat * elem_size
    last_page_end = (end + 4095) // 4096 * 4096
    for row in range(batch):
        row_addr = base + row * feat * elem_size
        off = (row_addr & 15) // elem_size
        head_n = min(vec - off, feat) if off else 0
        n_int = (feat - head_n) // vec
        interior = row_addr + head_n * elem_size
        safe = row_addr - off * elem_size
        if n_int:
            assert interior % 16 == 0
        for tid in (0, 1, block - 1):
            for i in range(cache_vecs):
                v = tid + i * block
                addr = interior + v * 16 if v < n_int else safe
                assert addr % 16 == 0, (row, tid, i)
                assert first_page <= addr and addr + 16 <= last_page_end, (row, tid, i)
                if v < n_int:
                    assert row_addr <= addr and addr + 16 <= row_addr + feat * elem_size


@pytest.mark.parametrize('base_offset', [0, 2, 4, 6, 8, 14])
@pytest.mark.parametrize('elem_size', [2, 4])
def test_every_vector_load_is_aligned_and_inside_the_tensor(base_offset, elem_size) -> None:
    if base_offset % elem_size:
        pytest.skip('a tensor is aligned to its element size')
    for batch, feat in SHAPES:
        check(min(batch, 40), feat, elem_size, 4096 * 10 + base_offset)
