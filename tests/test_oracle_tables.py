"""Pins the truth-table file format and index order (reference: tf2/src/approx_ops_types.h:99-122,205-216;
tf2/README.md:104-117) with the reference's own tables and its own C multiplier models."""
import hashlib
import json
import os

import numpy as np
import pytest


def _sha(b):
    return hashlib.sha256(b).hexdigest()


def test_committed_tables_match_recorded_hashes(golden_dir):
    sums = json.load(open(os.path.join(golden_dir, "table_sha256.json")))
    tdir = os.path.join(golden_dir, "tables")
    names = sorted(os.listdir(tdir))
    assert len(names) == 7
    for n in names:
        assert _sha(open(os.path.join(tdir, n), "rb").read()) == sums[n]
    assert len(sums) == 37


def test_reference_models_reproduce_every_table_hash(golden_dir):
    """f(a, b) of each reference C model, a outer / b inner, little-endian uint16 == the .bin file.
    The hashes on both sides were recorded from the reference tree by tests/golden/make_fixtures.py."""
    tables = json.load(open(os.path.join(golden_dir, "table_sha256.json")))
    models = json.load(open(os.path.join(golden_dir, "ref_models_sha256.json")))
    assert len(models) == 36
    for name, h in models.items():
        assert tables[name] == h, name


def test_live_reference_models_when_built(oracle, golden_dir):
    if not oracle.have_ref_models():
        pytest.skip("oracle/_ref not built (reference tree absent)")
    for name in ("L40", "2AC", "KEM", "1JFF"):
        t = oracle.ref_model_table(name)
        disk = oracle.table_load(os.path.join(golden_dir, "tables", "mul8u_%s.bin" % name))
        assert np.array_equal(t, disk), name


def test_test_table_is_exact_products(oracle, golden_dir, pkg):
    t = oracle.table_load(os.path.join(golden_dir, "tables", "test_mul_table.bin"))
    a = np.arange(256)[:, None]
    b = np.arange(256)[None, :]
    assert np.array_equal(t.reshape(256, 256), (a * b).astype(np.uint16))
    assert np.array_equal(oracle.table_exact(), t)
    assert np.array_equal(pkg.synth.table_exact(), t)


def test_index_order_is_input_major(oracle, golden_dir):
    """Only 4 of the reference tables are symmetric; L40 is not, so the order is observable:
    entry [a*256+b] of the file is model(a, b), not model(b, a)."""
    t = oracle.table_load(os.path.join(golden_dir, "tables", "mul8u_L40.bin")).reshape(256, 256)
    assert not np.array_equal(t, t.T)
    raw = np.fromfile(os.path.join(golden_dir, "tables", "mul8u_L40.bin"), dtype="<u2")
    assert raw[3 * 256 + 200] == t[3, 200] and raw[200 * 256 + 3] == t[200, 3]


def test_tables_with_nonzero_zero_row(oracle, golden_dir):
    """mul8u_2AC has T[0][b] != 0 for some b: padding taps (code = zero point) must be looked up, not skipped."""
    t = oracle.table_load(os.path.join(golden_dir, "tables", "mul8u_2AC.bin")).reshape(256, 256)
    assert t[0].any()


def test_short_or_missing_file_is_invalid_argument(oracle, tmp_path):
    p = tmp_path / "short.bin"
    p.write_bytes(b"\x00" * 1000)
    with pytest.raises(ValueError, match="Couldn't read the lookup table"):
        oracle.table_load(str(p))
    with pytest.raises(ValueError):
        oracle.table_load(str(tmp_path / "missing.bin"))
