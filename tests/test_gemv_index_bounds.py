"""Host mirror of the index arithmetic of the v_dot2 decode GEMV's activation staging and weight
requests (llmopt_amd/csrc/kernels/w4a16_gemv.hip: x_source, x_store, issue_item, the launch's
LDS size), run over every thread of a workgroup for the shapes the GPU tests use.

Every address the ring variants request must lie inside its buffer and every LDS index inside the
bytes the launch asks for - for the 256-thread workgroups the kernel is built with.  The same
arithmetic with 1024-thread workgroups (a variant that was tried and faulted on the GPU) is
enumerated too: it overruns the LDS block whenever rows x chunks is not a multiple of four, which
is why the kernel now refuses such a block size at compile time."""
import itertools

import pytest

K_CHUNK = 2048          # K values one wave-wide 16-byte load covers
X_AHEAD = 8             # activation vectors per thread requested ahead of the ring


def staging_indices(m_rows, m_template, k, threads):
    """(global 16-byte vector offsets into x, LDS uint4 indices) the staging touches."""
    segs = k // 32
    chunks = (segs + 63) // 64
    vectors_per_row = chunks * 256
    x_vectors = m_template * vectors_per_row
    reads, writes = [], []
    for thread in range(threads):
        ahead = [thread + n * threads for n in range(X_AHEAD) if n * threads < x_vectors]
        rest = list(range(thread + X_AHEAD * threads, x_vectors, threads))
        for i in ahead + rest:
            m, kk = divmod(i, vectors_per_row)
            valid = m < m_rows and kk < k // 8
            reads.append(((m if valid else 0) * k) // 8 + (kk if valid else 0))
            seg, j = kk >> 2, kk & 3
            writes.append(((m * chunks + (seg >> 6)) * 4 + j) * 64 + (seg & 63))
    lds_vectors = m_template * chunks * 256          # what the launch allocates for the activation
    return reads, writes, lds_vectors, x_vectors


def weight_requests(n, k, rows_per_tile, tiles_requested):
    """Byte offsets of the 16-byte weight loads and 2-byte scale loads of one wave's items."""
    segs = k // 32
    chunks = (segs + 63) // 64
    tiles = (n + rows_per_tile - 1) // rows_per_tile
    out = []
    for tile, item, lane in itertools.product(tiles_requested, range(chunks), range(64)):
        real = tile < tiles
        seg = item * 64 + lane
        safe = seg if (real and seg < segs) else 0
        for r in range(rows_per_tile):
            col = min((tile if real else 0) * rows_per_tile + r, n - 1)
            out.append((col * (k // 2) + safe * 16, col * (k // 64) * 2 + (safe >> 1) * 2))
    return out


SHAPES = [(1, 1, 576), (1, 1, 4096), (2, 2, 576), (2, 2, 4096), (2, 2, 14336), (1, 2, 64), (2, 2, 1024), (1, 1, 14336)]


@pytest.mark.parametrize("m_rows,m_template,k", SHAPES)
def test_staging_of_256_thread_workgroups_stays_inside_its_buffers(m_rows, m_template, k):
    reads, writes, lds_vectors, x_vectors = staging_indices(m_rows, m_template, k, 256)
    assert x_vectors % 256 == 0
    assert max(reads) * 8 + 8 <= m_rows * k          # halves of x
    assert max(writes) < lds_vectors
    assert sorted(writes) == list(range(lds_vectors))  # every vector of the LDS copy written exactly once


@pytest.mark.parametrize("n,k,rows", [(512, 4096, 2), (33, 14336, 1), (1, 64, 2), (1536, 576, 2), (4096, 14336, 1)])
def test_weight_and_scale_requests_stay_inside_the_matrix(n, k, rows):
    tiles = (n + rows - 1) // rows
    requests = weight_requests(n, k, rows, [0, tiles - 1, tiles, tiles + 5000])  # the last two: past the end
    assert max(w for w, _ in requests) + 16 <= n * k // 2
    assert max(s for _, s in requests) + 2 <= n * (k // 64) * 2


def test_1024_thread_workgroups_would_overrun_the_lds_copy():
    """rows x chunks = 2 (two rows of K = 576): 512 vectors for 1024 threads.  Threads 512..1023
    compute row indices 2 and 3 and store zeros past the block the launch allocated."""
    reads, writes, lds_vectors, x_vectors = staging_indices(2, 2, 576, 1024)
    assert x_vectors % 1024 != 0
    assert max(reads) * 8 + 8 <= 2 * 576             # the global side is clamped: no stray reads
    assert max(writes) >= lds_vectors                # the LDS side is not
    # where rows x chunks is a multiple of four the same block size is in bounds
    _, writes, lds_vectors, x_vectors = staging_indices(2, 2, 4096, 1024)
    assert x_vectors % 1024 == 0 and max(writes) < lds_vectors
