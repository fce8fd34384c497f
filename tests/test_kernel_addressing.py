"""Host models of the addresses four kernels form, checked against their buffers' bounds.

A wild address on the GPU can end more than the test that made it, so the index arithmetic of
the kernels whose launches the host plans most freely is restated here in Python and swept
over shapes, plans and cache states on the CPU: the tiled product (``csrc/gemm_tiled.hip``:
what a thread fetches, where it stages it in LDS, which fragments a wavefront reads, where the
sums go), the product of steps of many rows (``csrc/gemm_wide.hip``: the same, with its
numbering of workgroups over weight tiles, ranges of K and tiles of activation rows), the decode attention (``csrc/attention_mfma.hip``, ``decode_kernel``: which page and
key every lane reads for every split, with pages given back below a window and table entries
that are padding) and the 32-row prefill attention (``prefill_wide_kernel``: the block-table
look-ups of its pipeline, five windows ahead, self-fed and fed, whole blocks and shares of a
block, and the slots the shares' partial sums go to).  The models follow the kernels line by
line and must be changed with them.
"""

from __future__ import annotations

import random

import pytest

DEPTH, LDS_ROW, THREADS, ROW_PIECES = 128, 136, 256, 16  # gemm_tiled.hip's constants


def tiled_tile(m: int) -> tuple[int, int]:
    """(MB, activation rows of the tile) that ``launch_tiled`` picks for ``m`` rows."""
    if m <= 16:
        return 1, 16
    if m <= 32:
        return 1, 32
    return (2, 64) if m <= 64 else (4, 128)


def check_tiled(m, n, k, tile, per_split, splits, gated, x_stride):
    mb, xrows = tiled_tile(m)
    nt = 32 * tile
    stage = (nt + xrows) * LDS_ROW
    w_pieces, x_pieces = nt * ROW_PIECES // THREADS, xrows * ROW_PIECES // THREADS
    assert w_pieces * THREADS == nt * ROW_PIECES and x_pieces * THREADS == xrows * ROW_PIECES
    x_size = (m - 1) * x_stride + k
    total = -(-k // DEPTH)
    shared = xrows == 16
    blocks = -(-n // nt)
    for bx in sorted({0, blocks // 2, blocks - 1}):
        n_base = bx * nt
        for split in sorted({0, splits - 1}):
            first = split * per_split
            last = min(first + per_split, total)
            if first >= last:
                continue
            for tid in range(THREADS):
                piece_k, piece_row = 8 * (tid % ROW_PIECES), tid // ROW_PIECES
                for it in sorted({first, last - 1, last, last + 1}):  # the loop fetches two iterations past the range
                    k0 = min(min(it, last - 1) * DEPTH + piece_k, k - 8)
                    assert k0 >= 0
                    for i in range(w_pieces):
                        at = min(n_base + piece_row + 16 * i, n - 1) * k + k0
                        assert 0 <= at and at + 8 <= n * k
                    for i in range(x_pieces):
                        at = min(piece_row + 16 * i, m - 1) * x_stride + k0
                        assert 0 <= at and at + 8 <= x_size
                dst = piece_row * LDS_ROW + piece_k
                for buf in (0, 1):
                    assert all(buf * stage + dst + (nt + 16 * i) * LDS_ROW + 8 <= (buf + 1) * stage for i in range(x_pieces))
                    assert all(buf * stage + dst + 16 * i * LDS_ROW + 8 <= buf * stage + nt * LDS_ROW for i in range(w_pieces))
                lane, wave = tid % 64, tid // 64
                lane16, group, wave_n, wave_m = lane % 16, lane // 16, wave >> 1, wave & 1
                base = lane16 * LDS_ROW + 8 * group
                for step in range(DEPTH // 32):
                    for b in range(mb):
                        assert base + (nt + (0 if shared else 16 * mb * wave_m) + 16 * b) * LDS_ROW + 32 * step + 8 <= stage
                    for a in range(tile):
                        assert base + (wave_n * tile + a) * 16 * LDS_ROW + 32 * step + 8 <= nt * LDS_ROW
                if shared and wave_m:
                    continue
                for a in range(tile):
                    nrow = n_base + (wave_n * tile + a) * 16 + 4 * group
                    if nrow >= n:
                        continue
                    for b in range(mb):
                        row = (0 if shared else 16 * mb * wave_m) + 16 * b + lane16
                        if row >= m:
                            continue
                        if gated:
                            width = 2 if nrow + 3 < n else (1 if nrow + 1 < n else 0)
                            assert row * (n // 2) + nrow // 2 + width <= m * (n // 2)
                        else:
                            width = 4 if (nrow + 3 < n and n % 4 == 0) else min(4, n - nrow)
                            assert (split * m + row) * n + nrow + width <= splits * m * n


@pytest.mark.parametrize("m", [1, 9, 16, 17, 32, 33, 64, 65, 128])
def test_tiled_product_stays_inside_its_buffers(m):
    rng = random.Random(m)
    for n, k in ((97, 72), (5003, 200), (160, 48), (48, 40), (64, 264), (161, 128), (256, 1096), (6, 16)):
        iters = -(-k // DEPTH)
        for tile in (2, 4, 5, 8):
            if tile == 8 and m > 32:
                continue  # tiles of 256 weight rows take up to 32 rows
            for want in sorted({1, 2, iters}):
                per_split = -(-iters // min(want, iters))
                splits = -(-iters // per_split)
                check_tiled(m, n, k, tile, per_split, splits, False, k + 8 * rng.randint(0, 3))
                if splits == 1 and n % 2 == 0:
                    check_tiled(m, n, k, tile, per_split, splits, True, k)


WINDOW_KEYS = 32  # attention_mfma.hip


def check_decode(ctx, window, shift, table, splits, keys_per_split, device_context=None):
    """Every page a lane of ``decode_kernel`` selects is a live one, and the splits cover the
    keys lo..ctx-1 exactly."""
    if device_context is not None:  # a recorded launch sizes the splits on the device
        span = device_context
        if window and span > window + WINDOW_KEYS - 1:
            span = window + WINDOW_KEYS - 1
        per = (span + WINDOW_KEYS - 1 + splits - 1) // splits
        keys_per_split = -(-per // WINDOW_KEYS) * WINDOW_KEYS
    p = ctx - 1
    lo = max(0, p - window + 1) if window else 0
    covered = set()
    for split in range(splits):
        begin = (lo & ~31) + split * keys_per_split
        end = min(begin + keys_per_split, ctx)
        for w in range(begin, end, WINDOW_KEYS):
            first = w >> shift
            pages = [table[min(first + i, len(table) - 1)] for i in range(4)]
            for lane16 in range(16):
                for t in range(2):
                    key = w + 8 * (lane16 >> 2) + 4 * t + (lane16 & 3)
                    live = min(max(key, max(w, lo)), min(w + 31, p))
                    assert pages[(live - w) >> shift] >= 0, (ctx, window, 1 << shift, split, w, key)
                    if lo <= key <= p:
                        assert key not in covered
                        covered.add(key)
            for group in range(4):
                chunk = w + 8 * group
                live = chunk + 7 >= lo and chunk <= p
                key = chunk if live else (min(max(chunk, max(w, lo)), min(w + 31, p)) & ~7)
                assert pages[(key - w) >> shift] >= 0, (ctx, window, 1 << shift, split, w, chunk)
    assert covered == set(range(lo, ctx)), (ctx, window, splits, keys_per_split)


def test_decode_attention_reads_live_pages_only():
    rng = random.Random(2)
    for _ in range(3000):
        shift = rng.choice([3, 4, 5, 6])
        page = 1 << shift
        ctx = rng.choice([1, 2, 31, 32, 33, 63, 64, 65, 100, 257, 600, 1000, rng.randint(1, 5000)])
        window = rng.choice([0, 0, 1, 12, 16, 33, 70, 300, 1025])
        needed = -(-ctx // page)
        width = needed + rng.choice([0, 1, 5])
        table = [rng.randint(0, 500) for _ in range(needed)] + [-1] * (width - needed)
        if window:  # pages wholly below the window's lower bound were given back
            for i in range(max(0, ctx - window) // page):
                table[i] = -1
        bound = rng.choice([ctx, min(ctx + 50, width * page), width * page])  # what the host knows of the longest context
        span = bound if not window else min(bound, window + 31)
        for splits_wanted in (1, 2, rng.randint(1, 64), 256):
            splits = max(1, min(splits_wanted, -(-span // 32)))
            keys_per_split = -(-(-(-(span + 31) // splits)) // 32) * 32
            splits = -(-(span + 31) // keys_per_split)
            check_decode(ctx, window, shift, table, splits, keys_per_split)
            check_decode(ctx, window, shift, table, splits, keys_per_split, device_context=ctx)


def check_prefill_wide(pos0, cols, window, shift, table, fed, share=None):
    """``prefill_wide_kernel``'s block-table look-ups for one block of ``cols`` rows whose first
    row is at ``pos0``: every index lies inside the row, every page a load is formed from is a
    live one, and a window whose scores are used is fetched from its own pages.  ``share``:
    (first window, windows) of a block whose keys are shared out."""
    width = len(table)
    p_last = pos0 + cols - 1
    lo_first = max(0, pos0 - window + 1) if window else 0
    lo_last = max(0, p_last - window + 1) if window else 0
    begin, end = lo_first & ~31, p_last + 1
    if share is not None and share[1] > 0:
        begin += share[0] * WINDOW_KEYS
        end = min(end, begin + share[1] * WINDOW_KEYS)
    if begin >= end:
        return 0
    rounds = (end - begin + WINDOW_KEYS - 1) // WINDOW_KEYS
    last_window = (end - 1) & ~31
    steady_from = (lo_last - begin + WINDOW_KEYS - 1) // WINDOW_KEYS
    steady_to = min((pos0 + 1 - begin) // WINDOW_KEYS - 6, rounds - 1) if cols == 32 else -1
    if fed:
        assert shift >= 4, "the fed form wants pages of 16 keys or more"
    pieces = [0, 2] if fed else [0, 1, 2, 3]  # the pieces whose page a wavefront looks up (fed: one per half window)

    def window_at(i):
        return min(begin + i * WINDOW_KEYS, last_window)

    def page_of_chunk(w, piece):
        index = min((w + 8 * piece) >> shift, width - 1)
        assert 0 <= index < width
        return table[index]

    def fetch(w, pages, inside, used):
        """Keys or values of window ``w`` with the page ids looked up earlier (per looked-up piece)."""
        if inside or (w >= lo_first and w + 31 <= p_last):
            for piece, page in zip(pieces, pages):
                assert page >= 0, (pos0, cols, window, 1 << shift, share, w, piece)
                if used:
                    assert page == table[(w + 8 * piece) >> shift]
                    if fed:  # the half window's other piece lies on the same page
                        assert (w + 8 * piece + 8) >> shift == (w + 8 * piece) >> shift
        else:  # a window at the edge looks its pages up per lane
            for key in range(w, w + 32):
                live = min(max(key, max(w, lo_first)), min(w + 31, p_last))
                assert 0 <= live >> shift < width and table[live >> shift] >= 0, (pos0, cols, window, 1 << shift, share, w, key)

    page = [[page_of_chunk(window_at(k), piece) for piece in pieces] for k in range(5)]
    fetch(window_at(0), page[0], False, True)
    fetch(window_at(1), page[1], False, rounds > 1)
    fetch(window_at(2), page[2], False, rounds > 2)
    page = page[1:]  # page1 .. page4
    order = []
    i = 0
    while i < rounds and i < steady_from:
        order.append((i, False))
        if i + 1 < rounds:
            order.append((i + 1, False))
        i += 2
    while i + 1 <= steady_to:
        order += [(i, True), (i + 1, True)]
        i += 2
    while i < rounds:
        order.append((i, False))
        if i + 1 < rounds:
            order.append((i + 1, False))
        i += 2
    assert [r for r, _ in order] == list(range(rounds))
    for i, steady in order:
        w = begin + i * WINDOW_KEYS

        def at(k, w=w, i=i, steady=steady):
            return w + k * WINDOW_KEYS if steady else window_at(i + k)

        if steady:  # nothing is tested or clamped: the windows must lie inside what every column sees
            assert w >= lo_last and at(5) + 31 <= pos0
        fetch(at(3), page[2], steady, i + 3 < rounds)
        fetch(at(1), page[0], steady, i + 1 < rounds)
        page = page[1:] + [[page_of_chunk(at(5), piece) for piece in pieces]]
    return rounds


def test_prefill_attention_looks_up_live_pages_only():
    """Blocks of the 32-row prefill attention kernel over random contexts, windows, page sizes and
    shares: whole prompts, portions at the end of long contexts, blocks of fewer than 32 rows,
    tables with padding behind a request's pages and pages given back below a window."""
    from turboserve_amd.kernels.ops import prefill_block_windows, prefill_share_list

    rng = random.Random(5)
    for _ in range(1500):
        shift = rng.choice([3, 4, 5, 6])
        page = 1 << shift
        window = rng.choice([0, 0, 0, 1, 12, 33, 70, 300])
        count = rng.choice([2, 5, 31, 32, 33, 64, 100, 257, rng.randint(2, 700)])
        before = rng.choice([0, 0, 7, 32, 45, 1000, rng.randint(0, 3000)])
        context = before + count
        needed = -(-context // page)
        table = [rng.randint(0, 500) for _ in range(needed)] + [-1] * rng.choice([0, 0, 1, 3])
        if window:  # pages wholly below the lowest key the portion's first row sees were given back
            for i in range(max(0, before - window + 1) // page):
                table[i] = -1
        fed = shift >= 4 and rng.random() < 0.5
        for offset in range(0, count, 32):
            check_prefill_wide(before + offset, min(32, count - offset), window, shift, table, fed)
        # the same blocks with their keys shared out, as the planner would for an idle device
        blocks, ranges, combine = prefill_share_list([count], [context], 32, window, 1, 4096, rng.choice([1, 2, 16]), combine_cost=0)
        slots = sum(entry[3] for entry in combine)
        seen = set()
        for (_, row), (first, windows, slot) in zip(blocks, ranges):
            cols = min(32, count - row)
            assert windows == 0 or first + windows <= prefill_block_windows(before + row, cols, window)
            check_prefill_wide(before + row, cols, window, shift, table, fed, (first, windows))
            if slot >= 0:
                assert slot < slots and slot not in seen  # every share writes a partial slot of its own
                seen.add(slot)
        for row, rows, first_slot, shares in combine:
            assert 0 <= row and row + rows <= count and 0 <= first_slot and first_slot + shares <= slots
            assert set(range(first_slot, first_slot + shares)) <= seen


def check_wide(m, n, k, tile, x_rows, waves, depth, per_split, splits, mode, x_stride):
    """``gemm_wide_kernel`` (``csrc/gemm_wide.hip``): the workgroup numbering covers every (weight
    tile, range of K, tile of activation rows) exactly once, and every address a thread forms,
    in global memory and in LDS, lies inside its buffer."""
    wm = waves // 2
    threads = 64 * waves
    lds_row, row_pieces = depth, depth // 8  # rows are not padded: the pieces of a row are swizzled
    piece_rows = threads // row_pieces

    def key(row):
        return (row >> 1) & 7 if row_pieces == 8 else row & 15

    def banks(element):  # the four 4-byte banks (of 64) a 16-byte piece at this element offset lies in
        return {(element // 2 + i) % 64 for i in range(4)}

    # sixteen lanes of a write (consecutive pieces of one or two rows) and of a read (one piece of
    # sixteen consecutive rows) touch every bank at most once
    for first in range(0, threads, 16):
        touched = [banks((t // row_pieces) * lds_row + 8 * ((t % row_pieces) ^ key(t // row_pieces))) for t in range(first, first + 16)]
        assert sum(len(b) for b in touched) == len(set().union(*touched)) == 64
    for piece in range(row_pieces):
        touched = [banks(r * lds_row + 8 * (piece ^ key(r))) for r in range(16)]
        assert sum(len(b) for b in touched) == len(set().union(*touched)) == 64
    nt = 32 * tile
    mb = x_rows // (16 * wm)
    assert mb >= 1 and 16 * wm * mb == x_rows and x_rows % piece_rows == 0
    w_pieces, x_pieces = -(-nt // piece_rows), x_rows // piece_rows
    stage = (nt + x_rows) * lds_row
    assert 2 * stage * 2 <= 160 * 1024
    n_tiles, m_tiles = -(-n // nt), -(-m // x_rows)
    units = n_tiles * splits
    ids = -(-units // 8) * 8 * m_tiles
    total = -(-k // depth)
    x_size = (m - 1) * x_stride + k
    seen = set()
    for block in range(ids):
        die, turn = block % 8, block // 8
        m_tile, unit = turn % m_tiles, (turn // m_tiles) * 8 + die
        if unit >= units:
            continue
        assert (unit, m_tile) not in seen
        seen.add((unit, m_tile))
    assert len(seen) == units * m_tiles
    for unit, m_tile in sorted({(0, 0), (units - 1, m_tiles - 1), (units // 2, m_tiles // 2)}):
        n_base, split, m_base = (unit % n_tiles) * nt, unit // n_tiles, m_tile * x_rows
        first = split * per_split
        last = min(first + per_split, total)
        if first >= last:
            continue
        for tid in range(threads):
            piece_k, piece_row = 8 * (tid % row_pieces), tid // row_pieces
            for it in sorted({first, last - 1, last, last + 2}):  # loads are issued up to three iterations past the range
                k0 = min(min(it, last - 1) * depth + piece_k, k - 8)
                assert k0 >= 0
                for i in range(w_pieces):
                    at = min(n_base + min(piece_row + piece_rows * i, nt - 1), n - 1) * k + k0
                    assert 0 <= at and at + 8 <= n * k
                for i in range(x_pieces):
                    at = min(m_base + piece_row + piece_rows * i, m - 1) * x_stride + k0
                    assert 0 <= at and at + 8 <= x_size
            dst = piece_row * lds_row + 8 * ((tid % row_pieces) ^ key(piece_row))
            for buf in (0, 1):
                for i in range(x_pieces):
                    at = buf * stage + dst + (nt + piece_rows * i) * lds_row
                    assert buf * stage + nt * lds_row <= at and at + 8 <= (buf + 1) * stage
                for i in range(w_pieces):
                    if nt % piece_rows == 0 or piece_row + piece_rows * i < nt:
                        at = buf * stage + dst + piece_rows * i * lds_row
                        assert buf * stage <= at and at + 8 <= buf * stage + nt * lds_row
            lane, wave = tid % 64, tid // 64
            lane16, group, wave_n, wave_m = lane % 16, lane // 16, wave // wm, wave % wm
            base = lane16 * lds_row
            for step in range(depth // 32):
                piece = 8 * ((4 * step + group) ^ key(lane16))
                assert 0 <= piece and piece + 8 <= lds_row
                for b in range(mb):
                    at = base + (nt + 16 * mb * wave_m + 16 * b) * lds_row + piece
                    assert nt * lds_row <= at and at + 8 <= stage
                for a in range(tile):
                    assert base + (wave_n * tile + a) * 16 * lds_row + piece + 8 <= nt * lds_row
            for a in range(tile):
                nrow = n_base + (wave_n * tile + a) * 16 + 4 * group
                if nrow >= n:
                    continue
                for b in range(mb):
                    row = m_base + 16 * mb * wave_m + 16 * b + lane16
                    if row >= m:
                        continue
                    if mode == 2:
                        width = 2 if nrow + 3 < n else (1 if nrow + 1 < n else 0)
                        assert row * (n // 2) + nrow // 2 + width <= m * (n // 2)
                    elif mode == 1:
                        width = 4 if (nrow + 3 < n and n % 4 == 0) else min(4, n - nrow)
                        assert (split * m + row) * n + nrow + width <= splits * m * n
                    else:
                        width = 4 if (nrow + 3 < n and n % 4 == 0) else min(4, n - nrow)
                        assert row * n + nrow + width <= m * n


WIDE_SHAPES = [(2, 128, 4, 64), (5, 256, 4, 64), (4, 128, 8, 64), (5, 128, 8, 64), (2, 256, 8, 64), (5, 256, 8, 64), (8, 256, 8, 64),
               (8, 128, 8, 64), (2, 64, 8, 64), (5, 64, 8, 64), (8, 64, 8, 64), (2, 64, 8, 128), (4, 64, 8, 128), (5, 64, 8, 128)]


@pytest.mark.parametrize("tile,x_rows,waves,depth", WIDE_SHAPES)
def test_wide_product_stays_inside_its_buffers(tile, x_rows, waves, depth):
    rng = random.Random(tile * x_rows + depth)
    for m, n, k in ((130, 97, 72), (300, 500, 200), (513, 640, 1096), (17, 1000, 40), (64, 161, 264), (257, 6, 16), (1, 48, 8)):
        iters = -(-k // depth)
        for want in sorted({1, 2, iters}):
            per_split = -(-iters // min(want, iters))
            splits = -(-iters // per_split)
            check_wide(m, n, k, tile, x_rows, waves, depth, per_split, splits, 1, k + 8 * rng.randint(0, 3))
            if splits == 1:
                check_wide(m, n, k, tile, x_rows, waves, depth, per_split, splits, 0, k)
                if n % 2 == 0:
                    check_wide(m, n, k, tile, x_rows, waves, depth, per_split, splits, 2, k)
