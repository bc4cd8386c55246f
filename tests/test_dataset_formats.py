"""On-disk formats: the oracle's restatement of the reference readers is pinned by exact rational
arithmetic and by the file's definition; the library's readers (host code of libntship.so, no GPU
involved) are then compared with the oracle bit for bit.

Files are written the way data/generate_nts_dataset.py writes them: np.savetxt("%.4f") with the row
index put in front (write_to_file, :354-368), "i label", "i count idx ...", "i word" and the binary
edge list of 4-byte ids (edge2bin, :340-345)."""
import ctypes
import os
from fractions import Fraction

import numpy as np
import pytest

import oracle
from neutronbench_amd import dataset
from neutronbench_amd.abi import NtsError, call


def nearest_f32(token):
    """Nearest float32 (ties to even) of a decimal string, decided in exact rational arithmetic."""
    exact = Fraction(token)
    guess = np.float32(float(exact))
    with np.errstate(over="ignore"):
        cands = [guess, np.nextafter(guess, np.float32(np.inf)), np.nextafter(guess, np.float32(-np.inf))]
    best = None
    for c in cands:
        if not np.isfinite(c):
            continue
        err = abs(Fraction(float(c)) - exact)
        key = (err, int(np.float32(c).view(np.uint32)) & 1)  # even mantissa wins a tie
        if best is None or key < best[0]:
            best = (key, np.float32(c))
    out = best[1]
    if out == 0 and token.strip().startswith("-"):
        out = np.float32(-0.0)
    return out


def write_feature_file(path, ids, rows, fmt="%.4f", sep=" ", eol="\n"):
    with open(path, "w", newline="") as f:
        for i, r in zip(ids, rows):
            f.write(str(int(i)) + sep + sep.join(fmt % v for v in r) + eol)


def write_simple(path, ids, words):
    with open(path, "w") as f:
        for i, w in zip(ids, words):
            f.write(f"{int(i)} {w}\n")


def library_read(tmp, V, F, classes=1, threads=0):
    d = dataset.GNNDatum(V, F, classes, pinned=False)
    d.readFeature_Label_Mask(tmp / "g.feat", tmp / "g.label", tmp / "g.mask", threads=threads)
    return d


def assert_same_tables(d, o):
    assert np.array_equal(d.local_feature.view(np.uint32), o["local_feature"].view(np.uint32))
    for k in ("local_label", "global_label", "local_mask", "global_mask"):
        assert np.array_equal(getattr(d, k), o[k]), k


TOKENS = ["0.0130", "-0.0000", "12.3456", "1", "+2.5", "16777215", "16777216", "16777217", "16777219", "0.1",
          "0.3333333333333333148", "1e-3", "-4.25E+2", "3.4028234e38", "1.17549435e-38", "1e-45", "7.0e-46",
          "123456789.125", "0.000000059604644775390625", "9007199254740993", "0.0000000001", "33554434.0",
          "8388608.5", "8388609.5", "0.100000001490116119384765625", "1.00000005960464477539"]


def test_oracle_and_library_parse_tokens_to_the_nearest_float(tmp_path):
    # One record holding every token: what the text means is fixed by mathematics (nearest float32
    # of the decimal, ties to even), independent of either implementation.
    F = len(TOKENS)
    (tmp_path / "g.feat").write_text("0 " + " ".join(TOKENS) + "\n")
    (tmp_path / "g.label").write_text("0 3\n")
    (tmp_path / "g.mask").write_text("0 train\n")
    want = np.array([nearest_f32(t) for t in TOKENS], dtype=np.float32)
    o = oracle.read_feature_label_mask(tmp_path / "g.feat", tmp_path / "g.label", tmp_path / "g.mask", 1, F)
    assert np.array_equal(o["local_feature"][0].view(np.uint32), want.view(np.uint32))
    d = library_read(tmp_path, 1, F)
    assert np.array_equal(d.local_feature[0].view(np.uint32), want.view(np.uint32))


def test_random_decimal_tokens_match_exact_rounding(tmp_path):
    rng = np.random.default_rng(5)
    toks = []
    for _ in range(3000):
        kind = rng.integers(0, 4)
        x = float(rng.standard_normal() * 10.0 ** rng.integers(-6, 7))
        toks.append(["%.4f" % x, "%.9g" % x, "%.17g" % x, "%e" % x][kind])
    F = len(toks)
    (tmp_path / "g.feat").write_text("0\t" + "\n".join(toks) + "\n")  # the record spans many lines
    (tmp_path / "g.label").write_text("0 1\n")
    (tmp_path / "g.mask").write_text("0 val\n")
    want = np.array([nearest_f32(t) for t in toks], dtype=np.float32)
    o = oracle.read_feature_label_mask(tmp_path / "g.feat", tmp_path / "g.label", tmp_path / "g.mask", 1, F)
    assert np.array_equal(o["local_feature"][0].view(np.uint32), want.view(np.uint32))
    d = library_read(tmp_path, 1, F, threads=3)
    assert np.array_equal(d.local_feature[0].view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("threads", [1, 8])
@pytest.mark.parametrize("shuffled", [False, True])
def test_generator_format_round_trip(tmp_path, threads, shuffled):
    # Definition pin: a table printed with "%.4f" reads back as float32(round(x, 4)) placed by id;
    # labels and masks by their definition.
    rng = np.random.default_rng(11)
    V, F = 3000, 37
    x = rng.standard_normal((V, F)).astype(np.float32)
    labels = rng.integers(0, 40, V)
    words = rng.choice(["train", "val", "eval", "test", "unknown"], V)
    ids = rng.permutation(V) if shuffled else np.arange(V)
    write_feature_file(tmp_path / "g.feat", ids, x[ids])
    write_simple(tmp_path / "g.label", ids, labels[ids])
    write_simple(tmp_path / "g.mask", ids, words[ids])
    want = np.array([[nearest_f32("%.4f" % v) for v in row] for row in x[:50]], dtype=np.float32)
    code = {"train": 0, "val": 1, "eval": 1, "test": 2, "unknown": 3}
    o = oracle.read_feature_label_mask(tmp_path / "g.feat", tmp_path / "g.label", tmp_path / "g.mask", V, F)
    assert np.array_equal(o["local_feature"][:50].view(np.uint32), want.view(np.uint32))
    assert np.allclose(o["local_feature"], np.round(x.astype(np.float64), 4), atol=1e-6)
    assert np.array_equal(o["local_label"], labels) and np.array_equal(o["global_label"], labels)
    assert np.array_equal(o["local_mask"], [code[w] for w in words])
    assert np.array_equal(o["global_mask"], o["local_mask"])
    d = library_read(tmp_path, V, F, threads=threads)
    assert_same_tables(d, o)


def test_label_and_mask_follow_the_feature_file_position_not_their_own_id(tmp_path):
    # The k-th label / mask record goes to the vertex of the k-th feature record (local tables);
    # the global tables use the label / mask file's own id.
    V, F = 4, 2
    (tmp_path / "g.feat").write_text("2 1 2\n0 3 4\n3 5 6\n")
    (tmp_path / "g.label").write_text("0 7\n1 8\n2 9\n")
    (tmp_path / "g.mask").write_text("0 test\n1 train\n2 foo\n")
    o = oracle.read_feature_label_mask(tmp_path / "g.feat", tmp_path / "g.label", tmp_path / "g.mask", V, F)
    assert o["local_feature"].tolist() == [[3, 4], [0, 0], [1, 2], [5, 6]]
    assert o["local_label"].tolist() == [8, 0, 7, 9] and o["global_label"].tolist() == [7, 8, 9, 0]
    assert o["local_mask"].tolist() == [0, 0, 2, 3] and o["global_mask"].tolist() == [2, 0, 3, 0]
    assert_same_tables(library_read(tmp_path, V, F), o)


def test_multi_label_tabs_and_crlf(tmp_path):
    rng = np.random.default_rng(3)
    V, F, C = 200, 5, 12
    ids = rng.permutation(V)
    x = rng.standard_normal((V, F)).astype(np.float32)
    write_feature_file(tmp_path / "g.feat", ids, x[ids], fmt="%.6e", sep="\t", eol="\r\n")
    want = np.zeros((V, C), dtype=np.int64)
    with open(tmp_path / "g.label", "w") as f:
        for i in ids:
            idx = rng.choice(C, rng.integers(0, 5), replace=False)
            want[i, idx] = 1
            f.write(f"{i} {len(idx)} " + " ".join(map(str, idx)) + "\n")
    write_simple(tmp_path / "g.mask", ids, rng.choice(["train", "val", "test"], V))
    o = oracle.read_feature_label_mask(tmp_path / "g.feat", tmp_path / "g.label", tmp_path / "g.mask", V, F, C)
    assert np.array_equal(o["local_label"].reshape(V, C), want)
    assert np.array_equal(o["global_label"].reshape(V, C), want)
    assert_same_tables(library_read(tmp_path, V, F, C, threads=4), o)


def test_ids_outside_the_partition_are_skipped(tmp_path):
    # Single-label files only: for a skipped vertex the reference consumes two label tokens whatever
    # the label layout is (core/ntsDataloador.hpp:337-346), which is only in step for "id label".
    rng = np.random.default_rng(13)
    V, F = 150, 4
    ids = rng.permutation(V + 30)
    x = rng.standard_normal((V + 30, F)).astype(np.float32)
    labels = rng.integers(0, 9, V + 30)
    write_feature_file(tmp_path / "g.feat", ids, x[ids])
    write_simple(tmp_path / "g.label", ids, labels[ids])
    write_simple(tmp_path / "g.mask", ids, rng.choice(["train", "val", "test"], V + 30))
    o = oracle.read_feature_label_mask(tmp_path / "g.feat", tmp_path / "g.label", tmp_path / "g.mask", V, F)
    assert np.array_equal(o["local_label"], labels[:V])
    assert_same_tables(library_read(tmp_path, V, F, threads=2), o)


def test_large_file_thread_counts_agree(tmp_path):
    rng = np.random.default_rng(8)
    V, F = 20000, 64
    x = rng.standard_normal((V, F)).astype(np.float32)
    np.savetxt(tmp_path / "raw", x, fmt="%.4f")
    with open(tmp_path / "raw") as src, open(tmp_path / "g.feat", "w") as out:
        for i, line in enumerate(src):
            out.write(str(i) + " " + line)
    write_simple(tmp_path / "g.label", range(V), rng.integers(0, 7, V))
    write_simple(tmp_path / "g.mask", range(V), rng.choice(["train", "val", "test"], V))
    o = oracle.read_feature_label_mask(tmp_path / "g.feat", tmp_path / "g.label", tmp_path / "g.mask", V, F)
    for threads in (1, 5, 16):
        assert_same_tables(library_read(tmp_path, V, F, threads=threads), o)


def test_ogb_csv_variant(tmp_path):
    rng = np.random.default_rng(2)
    V, F = 500, 9
    x = rng.standard_normal((V, F))
    with open(tmp_path / "feat.csv", "w") as f:
        for r in x:
            f.write(",".join(repr(float(v)) for v in r) + "\n")
    labels = rng.integers(0, 47, V)
    (tmp_path / "label.csv").write_text("\n".join(map(str, labels)) + "\n")
    perm = rng.permutation(V)
    os.mkdir(tmp_path / "split")
    for name, part in (("train.csv", perm[:300]), ("valid.csv", perm[300:400]), ("test.csv", perm[400:])):
        (tmp_path / "split" / name).write_text("\n".join(map(str, part)) + "\n")
    o = oracle.read_feature_label_mask_ogb(tmp_path / "feat.csv", tmp_path / "label.csv", tmp_path / "split", V, F)
    # atof then narrowing: float32(float64(text)); repr() round-trips the float64 exactly
    assert np.array_equal(o["local_feature"], x.astype(np.float32))
    assert np.array_equal(o["local_label"], labels)
    want_mask = np.zeros(V, dtype=np.int32)
    want_mask[perm[300:400]] = 1
    want_mask[perm[400:]] = 2
    assert np.array_equal(o["local_mask"], want_mask)
    d = dataset.GNNDatum(V, F, pinned=False)
    d.readFeature_Label_Mask_OGB(tmp_path / "feat.csv", tmp_path / "label.csv", tmp_path / "split", threads=3)
    assert np.array_equal(d.local_feature.view(np.uint32), o["local_feature"].view(np.uint32))
    assert np.array_equal(d.local_label, o["local_label"]) and np.array_equal(d.local_mask, o["local_mask"])


def test_edge_file_round_trip(tmp_path):
    rng = np.random.default_rng(4)
    pairs = rng.integers(0, 1000, (12345, 2)).astype(np.uint32)
    # the generator's writer: every id as 4 bytes in host byte order, src then dst
    with open(tmp_path / "g.edge", "wb") as f:
        f.writelines(int(v).to_bytes(4, byteorder=__import__("sys").byteorder) for v in pairs.flatten())
    src, dst = oracle.read_edges(tmp_path / "g.edge")
    assert np.array_equal(src, pairs[:, 0]) and np.array_equal(dst, pairs[:, 1])
    assert dataset.edge_file_count(tmp_path / "g.edge") == 12345
    got = dataset.read_edge_file(tmp_path / "g.edge", vertices=1000)
    assert np.array_equal(got, pairs)
    with pytest.raises(ValueError):
        dataset.read_edge_file(tmp_path / "g.edge", vertices=int(pairs.max()))
    part = np.empty((100, 2), dtype=np.uint32)
    call("nts_edge_file_read", os.fsencode(tmp_path / "g.edge"), part.ctypes.data, 200, 100, None)
    assert np.array_equal(part, pairs[200:300])
    (tmp_path / "empty.edge").write_bytes(b"")
    assert dataset.read_edge_file(tmp_path / "empty.edge").shape == (0, 2)


def test_binary_table_round_trip(tmp_path):
    rng = np.random.default_rng(6)
    d = dataset.GNNDatum(321, 17, pinned=False)
    d.local_feature[...] = rng.standard_normal((321, 17)).astype(np.float32)
    d.write_feature_table(tmp_path / "t.bin")
    e = dataset.GNNDatum(321, 17, pinned=False)
    e.read_feature_table(tmp_path / "t.bin")
    assert np.array_equal(e.local_feature.view(np.uint32), d.local_feature.view(np.uint32))
    part = np.empty((10, 17), dtype=np.float32)
    call("nts_table_bin_read", os.fsencode(tmp_path / "t.bin"), part.ctypes.data, 300, 10)
    assert np.array_equal(part, d.local_feature[300:310])
    with pytest.raises(NtsError):
        call("nts_table_bin_read", os.fsencode(tmp_path / "t.bin"), part.ctypes.data, 315, 10)
    with pytest.raises(ValueError):
        dataset.GNNDatum(321, 16, pinned=False).read_feature_table(tmp_path / "t.bin")
    (tmp_path / "bad.bin").write_bytes(b"x" * 64)
    with pytest.raises(NtsError):
        dataset.GNNDatum(321, 17, pinned=False).read_feature_table(tmp_path / "bad.bin")


def test_reader_errors(tmp_path):
    (tmp_path / "g.label").write_text("0 1\n")
    (tmp_path / "g.mask").write_text("0 train\n")
    with pytest.raises(NtsError):  # missing file
        library_read(tmp_path, 2, 2)
    (tmp_path / "g.feat").write_text("0 1.0 2.0\n1 3.0\n")  # incomplete last record
    with pytest.raises(NtsError):
        library_read(tmp_path, 2, 2)
    (tmp_path / "g.feat").write_text("0 1.0 abc\n")
    with pytest.raises(NtsError):
        library_read(tmp_path, 2, 2)
    (tmp_path / "g.feat").write_text("x 1.0 2.0\n")
    with pytest.raises(NtsError):
        library_read(tmp_path, 2, 2)
    (tmp_path / "g.feat").write_text("")  # an empty file holds no records
    d = library_read(tmp_path, 2, 2)
    assert not d.local_feature.any()
