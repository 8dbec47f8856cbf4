"""Host-side restatement of the index arithmetic of the grouped 256-row GEMM form (lowbit_gemm_kernel.h:
grouped_tile, dma_x_grouped, the LDS piece layout), checked for what must hold whatever the rows per group:
every (group, row tile, column tile) is worked on exactly once; every byte the LDS-DMA fetches lies inside x
(the rows of the last 32-row block are clamped to the group's last row); every LDS piece that the MFMAs of the
computed blocks read has been filled with the row it stands for."""
import numpy as np
import pytest

ROWS = 256


def grouped_tile(offs, tiles_n, b):
    n = len(offs) - 1
    full = sum((offs[e + 1] - offs[e]) // ROWS for e in range(n))
    part = sum(((offs[e + 1] - offs[e]) % ROWS) != 0 for e in range(n))
    want_full = True
    if b < full * tiles_n:
        idx, tn = b % full, b // full
    else:
        b -= full * tiles_n
        if b >= part * tiles_n:
            return None
        want_full, tn = False, b // part
        idx = (b + tn) % part             # groups rotate over the XCDs (workgroup id % 8) from column to column
    for e in range(n):
        r0, r1 = offs[e], offs[e + 1]
        f = (r1 - r0) // ROWS
        if want_full:
            if idx < f:
                return e, r0 + idx * ROWS, r1, tn
            idx -= f
        elif (r1 - r0) % ROWS:
            if idx == 0:
                return e, r0 + f * ROWS, r1, tn
            idx -= 1
    return None


def check(counts, k, tiles_n=3):
    offs = [0] + [int(v) for v in np.cumsum(counts)]
    total = offs[-1]
    n_wg = tiles_n * (total // ROWS + len(counts))
    x_bytes = total * k * 2
    seen = set()
    for b in range(n_wg):
        t = grouped_tile(offs, tiles_n, b)
        if t is None:
            continue
        e, m0, m_end, tn = t
        assert (e, m0, tn) not in seen
        seen.add((e, m0, tn))
        assert offs[e] <= m0 < m_end <= offs[e + 1] and (m0 - offs[e]) % ROWS == 0
        rows_here = min(m_end - m0, ROWS)
        mbc = min((m_end - m0 + 31) // 32, 8)
        lds = {}
        for wave in range(4):
            h = wave >> 1
            tile_base = (m0 * k + h * 64) * 2
            for j in range(2 * mbc):
                tail = j >= 2 * (mbc - 1)
                piece_row = 8 * (2 * j + (wave & 1))
                for lane in range(64):
                    if tail:
                        row = min(piece_row + (lane & 7), rows_here - 1)
                        src = tile_base + row * k * 2 + (lane >> 3) * 16
                    else:
                        row = piece_row + (lane & 7)
                        src = tile_base + piece_row * k * 2 + (lane & 7) * k * 2 + (lane >> 3) * 16
                    assert 0 <= src and src + 16 <= x_bytes
                    assert row == min(piece_row + (lane & 7), rows_here - 1)
                    assert src - (m0 + row) * k * 2 == h * 128 + (lane >> 3) * 16
                piece = h * 32 + 2 * j + (wave & 1)
                assert piece not in lds and piece < 64
                lds[piece] = piece_row
        for half in range(2):
            for mb in range(mbc):
                for q in range(4):
                    piece = half * 32 + 4 * mb + q
                    assert lds.get(piece) == 8 * (4 * mb + q)
    assert len(seen) == sum((c + ROWS - 1) // ROWS for c in counts) * tiles_n


CASES = [[160] * 8, [136, 108, 150, 121, 132, 111, 130, 136], [1, 0, 255, 257, 33, 7, 129, 342], [256] * 8, [0, 0, 5],
         [513], list(range(1, 40)), [31, 32, 33, 63, 64, 65, 95, 96, 97, 127, 128, 129, 159, 160, 161, 191, 192, 193,
                                     223, 224, 225, 255, 256]]


@pytest.mark.parametrize("case", range(len(CASES)))
def test_fixed_row_counts(case):
    for k in (128, 4096, 14336):
        check(CASES[case], k)


def test_random_row_counts():
    rng = np.random.default_rng(0)
    for _ in range(25):
        check([int(v) for v in rng.integers(0, 600, size=rng.integers(1, 9))], 4096, tiles_n=2)
