"""Host-side restatement of the index arithmetic of the grouped 256-row GEMM form (lowbit_gemm_kernel.h:
grouped_tile, dma_x_grouped, the LDS piece layout), checked for what must hold whatever the rows per group:
every (group, row tile, column tile) is worked on exactly once; every byte the LDS-DMA fetches lies inside x
(the rows of the last 32-row block are clamped to the group's last row); every 16-byte operand that the MFMAs of
the computed blocks read from LDS has been filled with the row and columns it stands for; loads take whole cache
lines per eight lanes and operand reads spread over all LDS banks.  At the end: the dense 128-row form's line of tiles,
dealt to the XCDs whole or in 64-row halves, covers every row of every column tile exactly once."""
import numpy as np
import pytest

ROWS = 256


def grouped_tile(offs, tiles_n, chunk, b):
    """Cells of `chunk` column tiles of one row tile, dealt to the XCDs (b % 8) in turn; an XCD walks its cells in
    order.  Whole row tiles first, then the groups' partly filled ones."""
    n = len(offs) - 1
    full = sum((offs[e + 1] - offs[e]) // ROWS for e in range(n))
    part = sum(((offs[e + 1] - offs[e]) % ROWS) != 0 for e in range(n))
    per_row_tile = (tiles_n + chunk - 1) // chunk
    cells = (full + part) * per_row_tile
    i, ci = b >> 3, b & 7
    while True:
        if ci >= cells:
            return None
        q = ci % per_row_tile
        size = min(chunk, tiles_n - q * chunk)
        if i < size:
            break
        i -= size
        ci += 8
    tn = q * chunk + i
    idx = ci // per_row_tile
    want_full = idx < full
    if not want_full:
        idx -= full
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


def grouped_tile_lanes(offs, tiles_n, chunk, b):
    """The same answer found the way a wave finds it for up to 64 groups (grouped_tile_lanes): lane e holds group
    e's offsets, an inclusive prefix sum over the lanes counts whole row tiles, a ballot marks the groups with a
    partly filled one, and the group comes out of a ballot over 'my range of row tiles holds idx'."""
    n = len(offs) - 1
    assert n <= 64
    lanes = range(64)
    r0 = [offs[l] if l < n else 0 for l in lanes]
    r1 = [offs[l + 1] if l < n else 0 for l in lanes]
    rows = [max(r1[l] - r0[l], 0) for l in lanes]
    f = [rows[l] // ROWS for l in lanes]
    p = [rows[l] % ROWS != 0 for l in lanes]
    incl = list(f)
    d = 1
    while d < 64:                                   # shuffle-up scan: lane l adds what lane l - d held before the step
        prev = list(incl)
        for l in lanes:
            if l >= d:
                incl[l] = prev[l] + prev[l - d]
        d <<= 1
    full = incl[63]
    pm = sum(1 << l for l in lanes if p[l])
    per_row_tile = (tiles_n + chunk - 1) // chunk
    cells = (full + bin(pm).count("1")) * per_row_tile
    i, ci = b >> 3, b & 7
    while True:
        if ci >= cells:
            return None
        q = ci % per_row_tile
        size = min(chunk, tiles_n - q * chunk)
        if i < size:
            break
        i -= size
        ci += 8
    tn = q * chunk + i
    idx = ci // per_row_tile
    want_full = idx < full
    if want_full:
        hit = [l for l in lanes if incl[l] - f[l] <= idx < incl[l]]
    else:
        idx -= full
        hit = [l for l in lanes if p[l] and bin(pm & ((1 << l) - 1)).count("1") == idx]
    if not hit:
        return None
    g = hit[0]
    m0 = r0[g] + ((idx - (incl[g] - f[g])) if want_full else f[g]) * ROWS
    return g, m0, r1[g], tn


def grouped_grid(row_tiles, tiles_n, chunk):
    cells = row_tiles * ((tiles_n + chunk - 1) // chunk)
    return 8 * ((cells + 7) // 8) * chunk


def lane_row_chunk(lane, parity):
    """Row (0..7) and 16-byte chunk (0..7) of its piece that a lane fetches: eight consecutive lanes take the eight
    chunks of one row (one cache line), permuted so that the MFMA's reads spread over the LDS banks."""
    r = (lane >> 3) ^ parity
    return r, (lane & 7) ^ r


def operand_offset(lane, t):
    """Byte offset, within the four pieces of a 32-row block, of the MFMA operand of `lane` for 16-column step
    t = ks % 4 of a half row (lowbit_gemm_kernel.h: xlane[t])."""
    kg, i32 = lane >> 5, lane & 31
    p, r = i32 >> 3, i32 & 7
    return p * 1024 + ((r ^ (p & 1)) * 8 + ((2 * t + kg) ^ r)) * 16


def check(counts, k, tiles_n=3, chunk=None, waves=4):
    offs = [0] + [int(v) for v in np.cumsum(counts)]
    total = offs[-1]
    chunk = chunk or (tiles_n + 7) // 8
    n_wg = grouped_grid(total // ROWS + len(counts), tiles_n, chunk)
    x_bytes = total * k * 2
    seen = set()
    hw = waves // 2                                # waves per half row
    idle_seen = [False] * 8
    for b in range(n_wg):
        t = grouped_tile(offs, tiles_n, chunk, b)
        if t is None:
            idle_seen[b & 7] = True
            continue
        assert not idle_seen[b & 7], "an idle workgroup ahead of a working one on the same XCD"
        e, m0, m_end, tn = t
        assert (e, m0, tn) not in seen
        seen.add((e, m0, tn))
        assert offs[e] <= m0 < m_end <= offs[e + 1] and (m0 - offs[e]) % ROWS == 0
        rows_here = min(m_end - m0, ROWS)
        mbc = min((m_end - m0 + 31) // 32, 8)
        half_row = 32                                # pieces per half row of an x buffer
        lds = {}                                  # 16-byte slot -> (row of the tile, byte column of the K step) it holds
        for wave in range(waves):
            h = wave // hw
            tile_base = (m0 * k + h * 64) * 2
            for j in range(4 // hw * mbc):
                tail = j >= 4 // hw * (mbc - 1)
                piece_row = 8 * (hw * j + wave % hw)
                piece = h * half_row + hw * j + wave % hw
                assert piece % 2 == wave & 1 and piece < 2 * half_row
                for lane in range(64):
                    r, c = lane_row_chunk(lane, wave & 1)
                    if tail:
                        row = min(piece_row + r, rows_here - 1)
                        src = tile_base + row * k * 2 + c * 16
                    else:
                        row = piece_row + r
                        src = tile_base + piece_row * k * 2 + r * k * 2 + c * 16
                    assert 0 <= src and src + 16 <= x_bytes
                    assert row == min(piece_row + r, rows_here - 1)
                    assert src - (m0 + row) * k * 2 == h * 128 + c * 16
                    slot = piece * 1024 + lane * 16          # LDS-DMA writes the lanes in lane order
                    assert slot not in lds
                    lds[slot] = (row, h * 128 + c * 16)
        # every operand the MFMAs of the computed blocks read holds the row and columns it stands for
        for ks in range(8):
            for mb in range(mbc):
                for lane in range(64):
                    kg, i32 = lane >> 5, lane & 31
                    slot = ((ks // 4) * half_row + 4 * mb) * 1024 + operand_offset(lane, ks % 4)
                    want_row = min(32 * mb + i32, rows_here - 1)
                    assert lds.get(slot) == (want_row, (ks * 16 + kg * 8) * 2), (ks, mb, lane)
    assert len(seen) == sum((c + ROWS - 1) // ROWS for c in counts) * tiles_n


def test_operand_reads_cover_all_lds_banks():
    """A wave-wide 16-byte read is served 16 lanes at a time; the 64 banks are 4 bytes wide.  Each group of 16
    lanes must touch every bank once, for every 16-column step."""
    for t in range(4):
        for g in range(4):
            banks = []
            for lane in range(16 * g, 16 * g + 16):
                o = operand_offset(lane, t)
                banks += [((o + 4 * i) // 4) % 64 for i in range(4)]
            assert sorted(banks) == list(range(64)), (t, g)


def test_loads_fetch_whole_cache_lines():
    """Eight consecutive lanes of a load cover one 128-byte line of one row."""
    for parity in (0, 1):
        for s8 in range(8):
            rc = [lane_row_chunk(8 * s8 + i, parity) for i in range(8)]
            assert len({r for r, _ in rc}) == 1 and sorted(c for _, c in rc) == list(range(8))
        assert sorted(lane_row_chunk(l, parity)[0] for l in range(0, 64, 8)) == list(range(8))


CASES = [[160] * 8, [136, 108, 150, 121, 132, 111, 130, 136], [1, 0, 255, 257, 33, 7, 129, 342], [256] * 8, [0, 0, 5],
         [513], list(range(1, 40)), [31, 32, 33, 63, 64, 65, 95, 96, 97, 127, 128, 129, 159, 160, 161, 191, 192, 193,
                                     223, 224, 225, 255, 256]]


@pytest.mark.parametrize("waves", [4, 8])
@pytest.mark.parametrize("case", range(len(CASES)))
def test_fixed_row_counts(case, waves):
    for k in (128, 4096, 14336):
        check(CASES[case], k, waves=waves)


def test_random_row_counts():
    rng = np.random.default_rng(0)
    for _ in range(25):
        tiles_n = int(rng.integers(1, 20))
        check([int(v) for v in rng.integers(0, 600, size=rng.integers(1, 9))], 4096, tiles_n=tiles_n,
              chunk=[None, tiles_n, 1, 3][int(rng.integers(0, 4))], waves=int(rng.choice([4, 8])))


def test_tile_order_keeps_an_xcd_on_few_row_tiles_and_shares_even():
    """Eight groups of uneven size, 112 column tiles (the fused gate/up launch of a Mixtral layer): every XCD gets 14
    column tiles of every group, and 32 consecutive workgroups of an XCD touch at most four groups."""
    counts = [141, 124, 137, 122, 123, 151, 116, 110]
    offs = [0] + [int(v) for v in np.cumsum(counts)]
    tiles_n, chunk = 112, 14
    per_xcd = [[] for _ in range(8)]
    for b in range(grouped_grid(sum(counts) // ROWS + len(counts), tiles_n, chunk)):
        t = grouped_tile(offs, tiles_n, chunk, b)
        if t is not None:
            per_xcd[b & 7].append(t[0])
    for seq in per_xcd:
        assert sorted(seq) == sorted(list(range(8)) * 14)
        assert max(len(set(seq[i:i + 32])) for i in range(len(seq))) <= 4
    # a launch of a single round (the down projection: 16 column tiles): a group's column tiles share an XCD
    for b in range(grouped_grid(12, 16, 16)):
        t = grouped_tile(offs, 16, 16, b)
        assert t is None or t[0] == b & 7


# ---- dense 128-row form: the line of tiles dealt to the XCDs, whole or in 64-row halves (lowbit_gemm_kernel.h,
# the !GROUPED branch at the top of gemm_mfma_kernel; gemm.hip: band_rows, split_tail_tiles and the grid)

def _band_rows(tiles_m):
    bands = 1
    while bands * 2 <= 8 and bands * 2 <= tiles_m:
        bands *= 2
    return (tiles_m + bands - 1) // bands


def _dense_rows_covered(M, tiles_n, split_tail):
    """rows of y that each (row, column tile) receives, from every workgroup of the launch"""
    GM = 128
    tiles_m = (M + GM - 1) // GM
    T = tiles_m * tiles_n
    band_m = _band_rows(tiles_m)
    grid = 8 * ((T + 7) // 8 + split_tail)
    hits = np.zeros((M, tiles_n), dtype=np.int32)
    for b in range(grid):
        xcd, slot = b & 7, b >> 3
        first = T * xcd // 8
        count = T * (xcd + 1) // 8 - first
        idx, half = slot, -1
        whole = count - min(split_tail, count)
        if slot >= whole:
            idx = whole + ((slot - whole) >> 1)
            half = (slot - whole) & 1
        if idx >= count:
            continue
        line = first + idx
        per_band = band_m * tiles_n
        band, r = divmod(line, per_band)
        rows_b = min(tiles_m - band * band_m, band_m)
        tile_n = r // rows_b
        m0 = (band * band_m + r % rows_b) * GM
        m_end = M
        if half >= 0:
            m0 += (GM // 2) * half
            if m0 >= M:
                continue
            m_end = min(M, m0 + GM // 2)
        else:
            m_end = min(M, m0 + GM)
        assert 0 <= tile_n < tiles_n and 0 <= m0 < M
        hits[m0:m_end, tile_n] += 1
    return hits


def test_dense_tile_line_with_half_tiles_covers_every_row_once():
    rng = np.random.default_rng(5)
    cases = [(65, 2), (128, 8), (129, 3), (192, 48), (193, 24), (64, 5), (1, 1), (2048, 43), (1000, 12)]
    cases += [(int(rng.integers(1, 1500)), int(rng.integers(1, 50))) for _ in range(40)]
    for M, tiles_n in cases:
        T = (M + 127) // 128 * tiles_n
        for split_tail in (0, T // 8 + 1, 3):          # none, all (what the launcher passes), a few at each share's end
            hits = _dense_rows_covered(M, tiles_n, split_tail)
            assert (hits == 1).all(), (M, tiles_n, split_tail)


@pytest.mark.parametrize("n_groups", [1, 8, 63, 64])
def test_lane_lookup_agrees_with_the_walk_over_the_offsets(n_groups):
    rng = np.random.default_rng(n_groups)
    for trial in range(6):
        counts = rng.integers(0, 3 * ROWS, n_groups)
        counts[rng.random(n_groups) < 0.3] = 0
        if trial == 0:
            counts[:] = ROWS                        # whole tiles only
        if trial == 1:
            counts[:] = 0                           # nothing at all
        offs = [0] + [int(v) for v in np.cumsum(counts)]
        for tiles_n, chunk in ((3, 1), (16, 2), (5, 5)):
            row_tiles = sum(int(c) // ROWS + (int(c) % ROWS != 0) for c in counts)
            n_wg = grouped_grid(offs[-1] // ROWS + n_groups, tiles_n, chunk)
            got = [grouped_tile_lanes(offs, tiles_n, chunk, b) for b in range(n_wg)]
            assert got == [grouped_tile(offs, tiles_n, chunk, b) for b in range(n_wg)]
            assert sum(g is not None for g in got) == row_tiles * tiles_n
