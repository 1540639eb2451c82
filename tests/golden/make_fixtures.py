"""Regenerates the committed fixtures under tests/golden/.

Run in the build container, where the reference tree is mounted:
    python tests/golden/make_fixtures.py

What it writes
  tables/*.bin            six of the reference's truth tables (data files from
                          tf2/examples/axmul_8x8/, byte-for-byte) plus its test table
  table_sha256.json       sha256 of all 37 reference tables (36 multipliers + the test table)
  ref_models_sha256.json  sha256 of the table each of the reference's 36 C multiplier models
                          (tf1/axqconv/axmult/*.c, compiled by oracle/Makefile) produces when
                          called as f(a, b), a outer, b inner -- must equal table_sha256.json
  config1_oracle.npz      seeded config-1 tensors with the oracle's int32 sums and float outputs
                          (regression vectors made by this repository's oracle, not by the reference)
"""
import hashlib
import json
import os
import shutil
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402
import __graft_entry__ as entry  # noqa: E402
synth = entry.load_package().synth

REF = "/root/reference"
KEEP = ["1JFF", "L40", "2AC", "KEM", "QKX", "17C8"]


def sha(b):
    return hashlib.sha256(b).hexdigest()


def main():
    os.makedirs(os.path.join(HERE, "tables"), exist_ok=True)
    sums = {}
    for name in oracle.MULTIPLIER_NAMES:
        p = os.path.join(REF, "tf2/examples/axmul_8x8", "mul8u_%s.bin" % name)
        sums["mul8u_%s.bin" % name] = sha(open(p, "rb").read())
        if name in KEEP:
            shutil.copyfile(p, os.path.join(HERE, "tables", "mul8u_%s.bin" % name))
    p = os.path.join(REF, "tf2/test/test_mul_table.bin")
    sums["test_mul_table.bin"] = sha(open(p, "rb").read())
    shutil.copyfile(p, os.path.join(HERE, "tables", "test_mul_table.bin"))
    json.dump(sums, open(os.path.join(HERE, "table_sha256.json"), "w"), indent=1, sort_keys=True)

    oracle.build()
    models = {}
    for name in oracle.MULTIPLIER_NAMES:
        t = oracle.ref_model_table(name)
        models["mul8u_%s.bin" % name] = sha(t.astype("<u2").tobytes())
    json.dump(models, open(os.path.join(HERE, "ref_models_sha256.json"), "w"), indent=1, sort_keys=True)

    case = synth.config1(seed=1)
    out = {}
    for tname, table in (("exact", synth.table_exact()), ("noisy", synth.table_noisy(seed=7))):
        rc, y, acc = oracle.conv2d(table, case["x"], case["f"], *case["minmax"], strides=(1, 1), padding="SAME")
        assert rc == 0
        out["y_" + tname] = y
        out["acc_" + tname] = acc
    np.savez_compressed(os.path.join(HERE, "config1_oracle.npz"), x=case["x"], f=case["f"],
                        minmax=np.array(case["minmax"], np.float32), **out)
    print("fixtures written")


if __name__ == "__main__":
    main()
