"""Generates so3_fused64_items.h: which ITEM every thread of the per-volume 64^3 kernels holds in each of its 7 rounds.

    python s2cnn_amd/csrc/gen_fused64_items.py          # rewrites so3_fused64_items.h beside this file

An item is (c, a, n): the four degrees l = 4c..4c+3 of the two spectral columns (m = +a, n) and (m = -a, n), a, n >= 0;
it exists for c >= cmin(a, n) = max(a, n) // 4, c < 8: 3264 items for 7 x 512 places (round, thread).  The kernels work
for ANY assignment of items to places (everything that depends on it is derived from the table), but two things make one
assignment better than another:

 * truncated spectra skip whole rounds: all items with c <= 5 (degrees l < 24) must sit in rounds 0-2, all items with
   c <= 6 (l < 28) in rounds 0-5;
 * a thread whose consecutive rounds hold the SAME column (a, n) reads the transformed bins of that column once per beta
   step instead of once per item (analysis), and sums the shares of those items in registers before they leave for the
   plane (synthesis).  A RUN is a maximal sequence of consecutive rounds of a thread with the same column.  The analysis
   reads whenever ANY lane of a wave starts a run, so the lanes of a wave should start their runs in the same rounds; the
   synthesis adds the runs of a column from a staging area with two places per column, so a column may be cut into at
   most TWO runs over all threads.

The layout below, by thread (waves of 64):
   threads   0-255 (waves 0-3)  rounds 0-4: c = 3..7 of a column with cmin <= 3 (the 16 x 16 block a, n < 16)
   threads 256-399              round 0: a single item; rounds 1-4: c = 4..7 of a column with cmin = 4
   threads 400-415              rounds 0-2: c = 0, 1, 2 of a column with cmin = 0;       rounds 3-4: a pair (c = 6, 7)
   threads 416-463              round 0: a single item; rounds 1-2: c = 1, 2 of a column with cmin = 1; rounds 3-4: a pair
   threads 464-511              rounds 0-1: single items (or nothing);                      rounds 3-4: a pair
   rounds 5-6: a pair (c = 6, 7 of a column with cmin = 5 or 6) in 272 threads, c = 7 of a column with cmin = 7 in the others
single items: c = 2 of the columns with cmin = 2 and c = 5 of those with cmin = 5.  Every column is cut into at most two
runs.  The kernels have one copy of their loop for waves 0-3 and one for waves 4-7, each with the rounds in which some
lane of those waves starts a run as a compile-time mask (FRESH_LO, FRESH_HI below): rounds 0 and 5 for waves 0-3, rounds
0, 1, 3 and 5 for waves 4-7, instead of all 7.

Entry format (uint16): bits 0-4 n, 5-9 a, 10-12 c, 13 the place holds an item, 14 which of the column's two runs this one
is, 15 the run ends with this round.  Places without an item carry the column of the round before them (no new run).
"""
import os

THREADS, NIT = 512, 7
HERE = os.path.dirname(os.path.abspath(__file__))


def cmin(a, n):
    return max(a, n) // 4


def build():
    cols = {k: [(a, n) for a in range(32) for n in range(32) if cmin(a, n) == k] for k in range(8)}
    place = [[None] * NIT for _ in range(THREADS)]          # place[t][round] = (c, a, n)
    used = set()

    def put(t, r, c, a, n):
        assert place[t][r] is None and (c, a, n) not in used and 8 > c >= cmin(a, n), (t, r, c, a, n)
        place[t][r] = (c, a, n)
        used.add((c, a, n))

    # waves 0-3: the block a, n < 16 (cmin <= 3), row-major: c = 3..7 in rounds 0-4
    main = [(a, n) for a in range(16) for n in range(16)]
    for t, (a, n) in enumerate(main):
        for r, c in enumerate((3, 4, 5, 6, 7)):
            put(t, r, c, a, n)
    # threads 256-399: columns with cmin = 4: c = 4..7 in rounds 1-4
    assert len(cols[4]) == 144
    for i, (a, n) in enumerate(cols[4]):
        for r, c in zip((1, 2, 3, 4), (4, 5, 6, 7)):
            put(256 + i, r, c, a, n)
    # threads 400-415: c = 0, 1, 2 of the columns with cmin = 0
    for i, (a, n) in enumerate(cols[0]):
        for r, c in enumerate((0, 1, 2)):
            put(400 + i, r, c, a, n)
    # threads 416-463: c = 1, 2 of the columns with cmin = 1
    for i, (a, n) in enumerate(cols[1]):
        put(416 + i, 1, 1, a, n)
        put(416 + i, 2, 2, a, n)
    # single items: c = 2 of cmin = 2 (80), c = 5 of cmin = 5 (176), into round 0 of threads 256-399 and 416-463 and
    # rounds 0-1 of 464-511, in that order
    singles = [(5, a, n) for (a, n) in cols[5]] + [(2, a, n) for (a, n) in cols[2]]
    holes = [(t, 0) for t in range(256, 400)] + [(t, 0) for t in range(416, 464)] + [(t, r) for r in range(2) for t in range(464, 512)]
    assert len(singles) <= len(holes)
    for (c, a, n), (t, r) in zip(singles, holes):
        put(t, r, c, a, n)
    # pairs (c = 6, 7) of the columns with cmin = 5 and 6: rounds 3-4 of threads 400-511, rounds 5-6 of 272 threads
    pairs = cols[6] + cols[5]
    pair_places = [(t, 5) for t in range(0, 272)] + [(t, 3) for t in range(400, 512)]
    assert len(pairs) == len(pair_places) == 384
    for (a, n), (t, r) in zip(pairs, pair_places):
        put(t, r, 6, a, n)
        put(t, r + 1, 7, a, n)
    # c = 7 of the columns with cmin = 7: round 5 of the other 240 threads
    assert len(cols[7]) == 240
    for (a, n), t in zip(cols[7], range(272, 512)):
        put(t, 5, 7, a, n)

    every = {(c, a, n) for a in range(32) for n in range(32) for c in range(cmin(a, n), 8)}
    assert used == every and len(every) == 3264
    for t in range(THREADS):
        for r in range(NIT):
            if place[t][r] is not None:
                c = place[t][r][0]
                assert (c > 5 or r <= 2) and (c > 6 or r <= 5), (t, r, place[t][r])      # what the truncated kernels rely on
    return place


def encode(place):
    """uint16 entries [round][thread] with run structure; checks that no column has more than two runs."""
    col = [[None] * NIT for _ in range(THREADS)]
    for t in range(THREADS):
        last = (0, 0)
        for r in range(NIT):
            if place[t][r] is not None:
                last = place[t][r][1:]
            else:                               # an empty place continues the column before it (or the one after it, in front)
                nxt = next((place[t][q][1:] for q in range(r + 1, NIT) if place[t][q] is not None), last)
                last = last if r > 0 else nxt
            col[t][r] = last
    runs = {}                                   # column -> number of runs so far
    table = [[0] * THREADS for _ in range(NIT)]
    starts = [[False] * THREADS for _ in range(NIT)]
    for t in range(THREADS):
        r = 0
        while r < NIT:
            e = r
            while e + 1 < NIT and col[t][e + 1] == col[t][r]:
                e += 1
            has_item = any(place[t][q] is not None for q in range(r, e + 1))
            part = 0
            if has_item:
                part = runs.get(col[t][r], 0)
                runs[col[t][r]] = part + 1
            starts[r][t] = True
            for q in range(r, e + 1):
                a, n = col[t][q]
                c = place[t][q][0] if place[t][q] is not None else 0
                table[q][t] = n | (a << 5) | (c << 10) | ((place[t][q] is not None) << 13) | (part << 14) | ((q == e) << 15)
            r = e + 1
    assert max(runs.values()) <= 2, max(runs.values())
    fresh = [sum(1 << r for r in range(NIT) if any(starts[r][t] for t in range(lo, lo + 256))) for lo in (0, 256)]
    return table, fresh


def main():
    table, fresh = encode(build())
    lines = ["// GENERATED by gen_fused64_items.py - do not edit; see that script for the layout and what it is chosen for.",
             "// ITEM_TABLE[round * 512 + thread]: bits 0-4 n, 5-9 a, 10-12 c, 13 the place holds an item, 14 which of the column's",
             "// two runs this one is, 15 the run ends with this round.",
             "// FRESH_LO / FRESH_HI: bit r = some thread of waves 0-3 / waves 4-7 starts a run (another column) in round r.",
             "#pragma once", "#include <stdint.h>", "namespace fused64 {",
             "constexpr unsigned FRESH_LO = 0x%02x, FRESH_HI = 0x%02x;" % tuple(fresh),
             "#define S2CNN_FUSED64_ITEMS \\"]
    flat = [table[r][t] for r in range(NIT) for t in range(THREADS)]
    for i in range(0, len(flat), 16):
        lines.append("  " + ", ".join("0x%04x" % v for v in flat[i:i + 16]) + (", \\" if i + 16 < len(flat) else ""))
    lines += ["static const uint16_t ITEM_TABLE_HOST[%d] = {S2CNN_FUSED64_ITEMS};" % len(flat),
              "__device__ static const uint16_t ITEM_TABLE[%d] = {S2CNN_FUSED64_ITEMS};" % len(flat),
              "#undef S2CNN_FUSED64_ITEMS", "}  // namespace fused64", ""]
    with open(os.path.join(HERE, "so3_fused64_items.h"), "w") as f:
        f.write("\n".join(lines))
    print("rounds that start a run: waves 0-3 %s, waves 4-7 %s" % tuple(bin(f) for f in fresh))


if __name__ == "__main__":
    main()
