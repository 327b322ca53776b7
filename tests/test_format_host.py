"""The library's host format builder (venom_amd/csrc/vnm_format.cpp through the C ABI)
against the reference's golden vectors and against the CPU oracle.  Bit-exact."""
import numpy as np
import pytest

import oracle
from helpers import golden_cases, ksp_of, numpy_decode, random_conforming
from venom_amd import _lib
from venom_amd import format as F


@pytest.mark.parametrize("path", golden_cases(), ids=lambda p: p.split("vnm_")[-1][:-4])
def test_library_matches_reference_vectors(path):
    z = np.load(path)
    d, n, m, v = z["dense"], int(z["n"]), int(z["m"]), int(z["v"])
    rows, cols = d.shape
    g = F.geometry(rows, cols, n, m, v)
    assert (g.ksp, g.n_values, g.n_metadata, g.n_columns) == (int(z["ksp"]), z["values"].size, z["metadata"].size, z["columns"].size)
    if "fixed" not in path:
        masks, columns = F.select_columns(np.abs(d), n, m, v)
        assert np.array_equal(masks, z["masks"])
        assert np.array_equal(columns, z["columns"])
    if bool(z["encode_defined"]):
        vals, meta = F.encode((d * z["masks"]).astype(np.float32), z["columns"], n, m, v, mask=z["masks"])
        assert np.array_equal(vals, z["values"])
        assert np.array_equal(meta, z["metadata"].view(np.uint32))
        back = F.decode(z["values"], z["metadata"], z["columns"], rows, cols, n, m, v)
        assert np.array_equal(back, z["decoded"])


SHAPES = [(64, 64, 8, 32), (128, 96, 8, 64), (128, 256, 16, 128), (64, 40, 4, 32), (64, 70, 8, 32), (96, 75, 8, 32),
          (256, 512, 32, 128), (64, 33, 8, 32), (512, 1024, 8, 128)]


@pytest.mark.parametrize("rows,cols,m,v", SHAPES)
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_encode_decode_equal_oracle(rows, cols, m, v, dtype):
    dense, mask, columns = random_conforming(rows, cols, 2, m, v, seed=rows * 7 + cols, dtype=dtype)
    for mk in (None, mask):
        vals, meta = F.encode(dense, columns, 2, m, v, mask=mk)
        ovals, ometa = oracle.encode(dense, columns, 2, m, v, mask=mk)
        assert np.array_equal(vals.view(np.uint8), ovals.view(np.uint8)) and np.array_equal(meta, ometa)
    back = F.decode(vals, meta, columns, rows, cols, 2, m, v)
    if cols % m != 1:
        # (a one-column tail gets the reference's explicit zero entry on the same position as the
        # kept one, and its decoder then lets the zero win: no round trip there, by construction)
        assert np.array_equal(back, dense)
    assert np.array_equal(back, oracle.decode(vals, meta, columns, rows, cols, 2, m, v))
    assert np.array_equal(back, numpy_decode(vals, meta, columns, rows, cols, 2, m, v))
    # threads do not change the result
    v1, m1 = F.encode(dense, columns, 2, m, v, threads=1)
    assert np.array_equal(v1.view(np.uint8), vals.view(np.uint8)) and np.array_equal(m1, meta)


def test_decode_arbitrary_arrays_equals_oracle():
    # non-conforming metadata (both slots on one position, descending pairs) decodes like the reference loops
    rng = np.random.default_rng(11)
    rows, cols, m, v = 128, 104, 8, 64
    g = F.geometry(rows, cols, 2, m, v)
    vals = rng.standard_normal(g.n_values).astype(np.float32)
    meta = rng.integers(0, 2 ** 32, g.n_metadata, dtype=np.uint64).astype(np.uint32)
    columns = rng.integers(0, m, g.n_columns).astype(np.uint32)
    assert np.array_equal(F.decode(vals, meta, columns, rows, cols, 2, m, v),
                          oracle.decode(vals, meta, columns, rows, cols, 2, m, v))


def test_encode_fewer_than_n_kept_is_defined_and_roundtrips():
    rows, cols, m, v = 64, 64, 8, 32
    dense, mask, columns = random_conforming(rows, cols, 2, m, v, seed=4)
    # drop one kept entry in some rows, all kept entries in others
    dense2 = dense.copy()
    r, c = np.nonzero(dense2)
    dense2[r[::3], c[::3]] = 0.0
    dense2[5, :] = 0.0
    vals, meta = F.encode(dense2, columns, 2, m, v)
    assert np.array_equal(F.decode(vals, meta, columns, rows, cols, 2, m, v), dense2)
    assert np.array_equal(oracle.decode(vals, meta, columns, rows, cols, 2, m, v), dense2)
    # pairs stay ascending and distinct
    from helpers import slot_maps
    _, wi, sh = slot_maps(rows, ksp_of(cols, 2, m))
    nib = (meta[wi] >> sh.astype(np.uint32)) & 0xF
    assert ((nib & 3) < (nib >> 2)).all()


def test_encode_more_than_n_kept_is_an_error():
    rows, cols, m, v = 64, 64, 8, 32
    dense, mask, columns = random_conforming(rows, cols, 2, m, v, seed=4)
    cq = columns.reshape(rows // v, -1, 4)
    dense[0, cq[0, 0]] = 1.0           # four non-zeros among the four selected columns
    with pytest.raises(_lib.SpathaError) as e:
        F.encode(dense, columns, 2, m, v)
    assert e.value.status == 1


@pytest.mark.parametrize("rows,cols,m,v", [(64, 64, 8, 32), (64, 67, 8, 32), (64, 70, 8, 32), (128, 66, 8, 64),
                                           (64, 64, 16, 32), (32, 64, 32, 32), (64, 32, 4, 32)])
@pytest.mark.parametrize("kind", ["gauss", "ties", "sparse"])
def test_selector_equals_oracle(rows, cols, m, v, kind):
    rng = np.random.default_rng(rows + cols * 3 + m)
    if kind == "gauss":
        d = np.abs(rng.standard_normal((rows, cols))).astype(np.float32)
    elif kind == "ties":
        d = rng.integers(0, 3, size=(rows, cols)).astype(np.float32)
    else:
        d = np.abs(rng.standard_normal((rows, cols))).astype(np.float32) * (rng.random((rows, cols)) < 0.3)
        d[:, :m] = 0
    masks, columns = F.select_columns(d, 2, m, v)
    omasks, ocolumns = oracle.select_columns(d, 2, m, v)
    assert np.array_equal(columns, ocolumns)
    assert np.array_equal(masks, omasks)
    m1, c1 = F.select_columns(d, 2, m, v, threads=1)
    assert np.array_equal(m1, masks) and np.array_equal(c1, columns)


@pytest.mark.parametrize("rows,cols,m,v", [(128, 128, 8, 64), (128, 136, 8, 64), (64, 140, 8, 32), (64, 75, 10, 32),
                                           (128, 100, 20, 128), (64, 64, 4, 64)])
def test_random_pattern_equals_oracle_stream(rows, cols, m, v):
    oracle.srand(1)
    ometa, ocols = oracle.random_mask(rows, cols, 2, m, v)
    ovals = oracle.fill_rand_ints(64)
    oracle.srand(1)                       # same C library stream in this process
    meta, columns = F.random_pattern(rows, cols, 2, m, v)
    vals = F.fill_rand_small_ints(64)
    assert np.array_equal(meta, ometa) and np.array_equal(columns, ocols)
    assert np.array_equal(vals.astype(np.float32), ovals)


def test_random_pattern_known_answers():
    """The library's generator against answers derived without it and without the oracle: five matrices drawn one after
    another from the C library's stream (tests/golden/make_random_mask_kat.py walks glibc's rand() and libstdc++'s
    random_shuffle in the order of src/format/format_sr_nm.cpp:151-237)."""
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "random_mask_kat.json")) as f:
        kat = json.load(f)
    oracle.srand(1)
    for c in kat:
        meta, columns = F.random_pattern(c["rows"], c["cols"], 2, c["m"], c["v"])
        assert np.array_equal(meta, np.array(c["metadata"], np.uint32)), (c["rows"], c["cols"])
        assert np.array_equal(columns, np.array(c["columns"], np.uint32)), (c["rows"], c["cols"])


def _golden_json(name):
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", name)) as f:
        return json.load(f)


def test_small_int_fill_known_answers():
    """`rand() % 9 - 4` after srand(1): glibc's stream starts 1804289383, 846930886, 1681692777, 1714636915, 1957747793,
    424238335, i.e. -3, 3, -4, 3, 1, 3 (reference fill: src/format/format_sr_nm.cpp:64-68, src/util/matrix_utils.h:88-97).
    Literals, not a second evaluation of the formula."""
    want = [-3.0, 3.0, -4.0, 3.0, 1.0, 3.0]
    assert _golden_json("benchmark_draw_order_kat.json")["fill_head"] == want
    oracle.srand(1)
    assert oracle.fill_rand_ints(6).tolist() == want
    oracle.srand(1)
    got = F.fill_rand_small_ints(6)
    assert got.dtype == np.float16 and got.astype(np.float32).tolist() == want
    assert got.view(np.uint16).tolist() == [0xC200, 0x4200, 0xC400, 0x4200, 0x3C00, 0x4200]


def test_benchmark_draw_order_known_answers():
    """One benchmark run consumes rand() as B, then pattern, then values (src/dataset/dataset.cpp:70-90,
    src/format/format_sr_nm.cpp:62-68).  The driver draws through spatha_benchmark_inputs_f16; its output is held against
    a pure-Python walk of glibc's stream (tests/golden/make_random_mask_kat.py), two runs of one process in a row."""
    kat = _golden_json("benchmark_draw_order_kat.json")
    first = kat["runs"][0]
    assert first["B"][:3] == [-3, 3, -4] and first["draws"] == 256 + 16 * 8 * 3 + 4 * 7 + 32 * 16
    oracle.srand(1)
    for c in kat["runs"]:
        B, meta, columns, vals = F.benchmark_inputs(c["rows"], c["cols"], c["ncolsB"], 2, c["m"], c["v"])
        assert B.astype(np.int64).reshape(-1).tolist() == c["B"]
        assert meta.tolist() == c["metadata"] and columns.tolist() == c["columns"]
        assert vals.astype(np.int64).tolist() == c["values"]
    # the oracle's pieces called in that order agree as well
    oracle.srand(1)
    for c in kat["runs"]:
        oB = oracle.fill_rand_ints(c["cols"] * c["ncolsB"])
        ometa, ocols = oracle.random_mask(c["rows"], c["cols"], 2, c["m"], c["v"])
        ovals = oracle.fill_rand_ints(len(c["values"]))
        assert oB.tolist() == c["B"] and ometa.tolist() == c["metadata"] and ocols.tolist() == c["columns"]
        assert ovals.tolist() == c["values"]


def test_meta_blob_layout():
    meta = np.arange(1, 12, dtype=np.uint32)          # 11 words -> column-loc starts at word 16
    columns = np.arange(100, 105, dtype=np.uint32)
    blob, off = F.pack_meta_blob(meta, columns)
    assert off == 16 and blob.size == 24
    assert np.array_equal(blob[:11], meta) and (blob[11:16] == 0).all()
    assert np.array_equal(blob[16:21], columns) and (blob[21:] == 0).all()


def test_bad_shapes_are_reported_not_fatal():
    with pytest.raises(_lib.SpathaError) as e:
        F.geometry(100, 64, 2, 8, 64)        # rows % V
    assert e.value.status == 2
    with pytest.raises(_lib.SpathaError) as e:
        F.geometry(96, 64, 2, 8, 48)         # V % 32
    assert e.value.status == 2
    with pytest.raises(_lib.SpathaError) as e:
        F.geometry(64, 64, 3, 8, 32)         # n != 2
    assert e.value.status == 1
    with pytest.raises(_lib.SpathaError) as e:
        F.geometry(64, 64, 2, 3, 32)         # m < 4
    assert e.value.status == 1


def test_file_container_round_trip_and_rejects_damage(tmp_path):
    rows, cols, n, m, v = 128, 100, 2, 8, 64
    vals, meta, columns = F.synthetic_vnm(rows, cols, n, m, v, seed=3, value_std=1.0)
    path = tmp_path / "a.vnm"
    F.save(path, vals, meta, columns, rows, cols, n, m, v)
    v2, m2, c2, g = F.load(path)
    assert (g.rows, g.cols, g.n, g.m, g.v) == (rows, cols, n, m, v)
    assert v2.dtype == np.float16 and np.array_equal(v2.view(np.uint16), vals.view(np.uint16))
    assert np.array_equal(m2, meta.view(np.uint32)) and np.array_equal(c2, columns.reshape(-1))
    # fp32 values keep their width
    F.save(path, vals.astype(np.float32), meta, columns, rows, cols, n, m, v)
    assert F.load(path)[0].dtype == np.float32
    raw = bytearray(path.read_bytes())
    for damage in ("flip", "truncate", "append", "magic", "shape"):
        bad = bytearray(raw)
        if damage == "flip":
            bad[64 + 10] ^= 1                      # one payload bit: checksum
        elif damage == "truncate":
            bad = bad[:-4]
        elif damage == "append":
            bad += b"\0"
        elif damage == "magic":
            bad[0] = ord("X")
        else:
            bad[12] ^= 64                          # rows no longer match the stored array lengths
        p2 = tmp_path / (damage + ".vnm")
        p2.write_bytes(bytes(bad))
        with pytest.raises(_lib.SpathaError) as e:
            F.load(p2)
        assert e.value.status == 7, damage
    with pytest.raises(_lib.SpathaError) as e:
        F.load(tmp_path / "missing.vnm")
    assert e.value.status == 7
