"""Known answers for the reference's random pattern generator (src/format/format_sr_nm.cpp:151-237), derived without
running any C++: glibc's rand() (the additive-feedback generator of stdlib/random_r.c, TYPE_3, seeded by srand(1) as a
process that never calls srand is) and libstdc++'s std::random_shuffle (bits/stl_algo.h: for i = 1 .. len-1 swap
element i with element rand() % (i + 1)) are restated here in pure Python, and the generator's draws are walked in
the reference's order:

  * metadata, per 32-row block i, per complete tile j of 8 kept columns (4 complete groups), per row pair k: one
    word, built from 8 draws "shuffle the persistent array {0,1,2,3}, sort its first two entries" (:157-177); then,
    only when K % m != 0, per row pair one word from `resto / m` draws per row of the pair plus the fixed pair (0, 1)
    for the partial group (:179-210).  Complete groups beyond the last complete tile get NO draw when K % m == 0:
    their words stay zero;
  * column-loc, after ALL metadata draws, per V-row block, per group: "shuffle the persistent array {0..m-1}, sort its
    first four entries" (:213-229); a partial last group gets 0, 1, 2, 3 (:230-235).

Both arrays persist across draws (they are never reset), which is what makes the stream order observable.

A second file pins the benchmark's fills and the order in which one `benchmark_spmm --sparsity-type n-to-m` run consumes
the stream: the K x N entries of B first (src/dataset/dataset.cpp:81 -> src/util/matrix_utils.h:88-97), then the pattern
(src/format/format_sr_nm.cpp:62), then the rows x Ksp stored values of A in storage order (:64-68); every fill entry is
`rand() % 9 - 4` (C's remainder of a non-negative int, so Python's % agrees).

    python tests/golden/make_random_mask_kat.py      # rewrites tests/golden/random_mask_kat.json and benchmark_draw_order_kat.json
"""
import json
import os


def glibc_rand_stream(seed, count):
    r = [0] * (344 + count)
    r[0] = seed
    for i in range(1, 31):
        hi, lo = divmod(r[i - 1], 127773)
        w = 16807 * lo - 2836 * hi
        r[i] = w + 2147483647 if w < 0 else w
    for i in range(31, 34):
        r[i] = r[i - 31]
    for i in range(34, 344 + count):
        r[i] = (r[i - 31] + r[i - 3]) & 0xffffffff
    return [r[i + 344] >> 1 for i in range(count)]


class Stream:
    def __init__(self, seed=1):
        self.values = glibc_rand_stream(seed, 1 << 16)
        self.pos = 0

    def rand(self):
        v = self.values[self.pos]
        self.pos += 1
        return v

    def shuffle(self, a):
        for i in range(1, len(a)):
            j = self.rand() % (i + 1)
            if i != j:
                a[i], a[j] = a[j], a[i]


def round_up(x, y):
    return -(-x // y) * y


def random_mask(rows, cols, m, v, stream, n=2, mbrow=32):
    ncol = (cols // m) * n                  # kept columns of the complete groups (:53)
    ncol_pad = -(-cols // m) * n            # ... counting a partial last group (:54)
    ksp = round_up(ncol_pad, 16)            # row length of the value array (:55)
    meta = [0] * ((rows // 2) * (ksp // 8))
    arr = [0, 1, 2, 3]
    for i in range(rows // mbrow):
        full = ncol // 8
        for j in range(full):
            for k in range(mbrow // 2):
                word = 0
                for g in range(8):
                    stream.shuffle(arr)
                    arr[:n] = sorted(arr[:n])
                    for w in range(n):
                        word |= arr[w] << (g * 4 + w * 2)
                meta[i * (mbrow // 2) * (ksp // 8) + j * (mbrow // 2) + k] = word
        if ncol_pad > ncol:
            resto = cols - 4 * m * full
            for k in range(mbrow // 2):
                word = 0
                for t in range(2):
                    g = 0
                    while g < resto // m:
                        stream.shuffle(arr)
                        arr[:n] = sorted(arr[:n])
                        for w in range(n):
                            word |= arr[w] << ((g + t * 4) * 4 + w * 2)
                        g += 1
                    if resto % m > 0:
                        for w in range(n):
                            word |= w << ((g + t * 4) * 4 + w * 2)
                meta[i * (mbrow // 2) * (ksp // 8) + full * (mbrow // 2) + k] = word
    columns = [0] * ((rows // v) * (ksp // 2) * 4)
    arr2 = list(range(m))
    resto = cols - (ncol // n) * m
    for i in range(rows // v):
        for j in range(ncol // n):
            stream.shuffle(arr2)
            arr2[:4] = sorted(arr2[:4])
            columns[i * (ksp // 2) * 4 + j * 4:i * (ksp // 2) * 4 + j * 4 + 4] = arr2[:4]
        if resto > 0:
            j = ncol // n
            columns[i * (ksp // 2) * 4 + j * 4:i * (ksp // 2) * 4 + j * 4 + 4] = [0, 1, 2, 3]
    return meta, columns


CASES = [
    # rows, cols, m, v  -- drawn one after another from ONE stream, as consecutive matrices of one process would be
    (32, 32, 8, 32),      # one complete tile, no tail
    (64, 48, 8, 32),      # 6 complete groups: groups 4, 5 lie beyond the complete tile and K % m == 0 -> words stay zero
    (64, 44, 8, 32),      # 5 complete groups + 4 columns: tail words (one draw per row + the fixed pair); two 32-row blocks
    (128, 168, 16, 64),   # m = 16: two complete tiles, then two drawn groups + a partial one per row; two V blocks
    (64, 32, 4, 64),      # plain 2:4
]


def fill_small_ints(count, stream):
    return [stream.rand() % 9 - 4 for _ in range(count)]


def benchmark_inputs(rows, cols, ncolsB, m, v, stream):
    """What one run of the reference benchmark draws, in its order: B, pattern, values of A."""
    B = fill_small_ints(cols * ncolsB, stream)
    meta, columns = random_mask(rows, cols, m, v, stream)
    ksp = round_up(-(-cols // m) * 2, 16)
    values = fill_small_ints(rows * ksp, stream)
    return dict(rows=rows, cols=cols, ncolsB=ncolsB, m=m, v=v, B=B, metadata=meta, columns=columns, values=values,
                draws=stream.pos)


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    d = Stream(1)
    head = fill_small_ints(6, d)
    assert head == [-3, 3, -4, 3, 1, 3]       # 1804289383 % 9 - 4, 846930886 % 9 - 4, ...: worked by hand from the stream's head
    d = Stream(1)
    runs = [benchmark_inputs(32, 32, 8, 8, 32, d),      # 256 draws for B, 32 words x 8 x 3, 8 groups x 7, 512 values
            benchmark_inputs(64, 44, 16, 8, 32, d)]     # a second run of the same process: K % m != 0, two V blocks
    with open(os.path.join(here, "benchmark_draw_order_kat.json"), "w") as f:
        json.dump(dict(fill_head=head, runs=runs), f, separators=(",", ":"))
    print("wrote benchmark_draw_order_kat.json", [r["draws"] for r in runs])
    s = Stream(1)
    assert s.values[:4] == [1804289383, 846930886, 1681692777, 1714636915]      # the published head of glibc's stream
    out = []
    for rows, cols, m, v in CASES:
        start = s.pos
        meta, columns = random_mask(rows, cols, m, v, s)
        out.append(dict(rows=rows, cols=cols, m=m, v=v, draws_before=start, draws_after=s.pos, metadata=meta, columns=columns))
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "random_mask_kat.json")
    with open(path, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print("wrote", path, [c["draws_after"] for c in out])


if __name__ == "__main__":
    main()
