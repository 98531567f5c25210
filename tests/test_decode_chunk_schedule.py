"""CPU model of the matrix-core split kernel's chunk schedule (csrc/swa_decode_mfma.hip): which
chunks a split treats as edge / interior, which tiles it looks up in the block table and which
rows it reads. Invariants: every visible chunk is computed exactly once; the unclamped interior
loader (and its block-table lookups) only ever touches tiles wholly inside [lo, hi); the edge
loader only touches clamped tiles and rows. A lookup outside [first_tile, last_tile] would read
past the sequence's block-table row on the GPU."""
import itertools


def check(hi, wl, key_lo, n_split, depth, fused):
    lo = max(0, hi - 1 - wl) if wl >= 0 else 0
    lo = max(lo, key_lo)
    visible = hi > lo
    first_tile = lo >> 4
    last_tile = (hi - 1) >> 4 if visible else first_tile
    first_chunk = first_tile >> 1
    n_chunks = (last_tile >> 1) - first_chunk + 1 if visible else 0
    cps = (n_chunks + n_split - 1) // n_split

    def tile_base(t):
        assert first_tile <= t <= last_tile, (t, first_tile, last_tile, hi, wl, n_split)

    def clamp_tile(t):
        return min(max(t, first_tile), last_tile)

    def clamp_row(tc, row):
        r = min(max((tc << 4) + row, lo), hi - 1) - (tc << 4)
        assert 0 <= r < 16, (tc, row, r, lo, hi)

    def load_edge(cc):
        for t in (clamp_tile(2 * cc), clamp_tile(2 * cc + 1)):
            tile_base(t)
            for row in range(16):
                clamp_row(t, row)

    computed, newest_seen = [], 0
    for split in range(n_split):
        cb = first_chunk + split * cps
        ce = min(cb + cps, first_chunk + n_chunks)
        if cb >= ce:
            continue

        def is_edge(cc):
            return (cc << 5) < lo or (cc << 5) + 32 > hi or (fused and cc == ((hi - 1) >> 5))

        e_head = is_edge(cb)
        e_tail = (ce - 1 > cb) and is_edge(ce - 1)
        ib, ie = cb + (1 if e_head else 0), ce - (1 if e_tail else 0)
        if ib < ie:
            lastc = ie - 1

            def locate(cc):
                assert ib <= cc <= lastc
                assert (cc << 5) >= lo and (cc << 5) + 32 <= hi          # interior loader: no clamping
                assert not (fused and cc == ((hi - 1) >> 5))             # never reads the unappended row
                tile_base(2 * cc)
                tile_base(2 * cc + 1)

            ch = ib
            locate(ch)
            for u in range(depth):
                locate(min(ch + u + 1, lastc))
            load_edge(cb)
            load_edge(ce - 1)
            if e_head:
                computed.append(cb)
            while ch < ie:
                locate(min(ch + depth + 1, lastc))
                computed.append(ch)
                ch += 1
        else:
            load_edge(cb)
            load_edge(ce - 1)
            if e_head:
                computed.append(cb)
        if e_tail:
            computed.append(ce - 1)
        if visible and ce == first_chunk + n_chunks:
            newest_seen += 1                                             # the split that stores the new row
    assert sorted(computed) == list(range(first_chunk, first_chunk + n_chunks)), (computed, hi, wl, n_split)
    assert newest_seen == (1 if visible else 0)


def test_chunk_schedule_invariants():
    lengths = list(range(0, 100)) + [127, 128, 129, 200, 257, 4096, 4097, 4100]
    windows = [-1, 0, 1, 15, 16, 31, 32, 37, 64, 4096]
    n = 0
    for hi, wl, klo, ns, fused in itertools.product(lengths, windows, [0, 40], [1, 2, 3, 4, 7], [False, True]):
        check(hi, wl, klo, ns, 1, fused)
        n += 1
    for hi, wl, ns in itertools.product([1, 33, 64, 200, 4097], [64, 4096], [1, 3, 4]):
        for depth in (2, 3):
            check(hi, wl, 0, ns, depth, True)
    assert n > 20000
