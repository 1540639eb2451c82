"""Truth-table files in the reference's format (tf2/README.md:104-117): 65536 little-endian uint16,
entry [a * 256 + b] = approximate product of input code a and filter code b.

    python tables.py exact out.bin
    python tables.py truncated 4 out.bin        # a*b - (a*b mod 2^k)
    python tables.py noisy SEED out.bin         # clamp(a*b + round(N(0, 0.02*a*b)))
    python tables.py uniform SEED out.bin       # clamp(a*b + U(-64, 64))
    python tables.py tune in.bin out.bin        # the tf1 AxTune column remap (needs the built library)
    python tables.py info in.bin                # error statistics against exact multiplication
"""
import sys

import numpy as np


def write_table(path, table):
    t = np.ascontiguousarray(table).reshape(-1)
    if t.size != 65536:
        raise ValueError("a table holds 256 x 256 entries")
    if t.min() < 0 or t.max() > 65535:
        raise ValueError("entries must fit uint16")
    t.astype("<u2").tofile(path)


def read_table(path):
    t = np.fromfile(path, dtype="<u2")
    if t.size != 65536:
        raise ValueError("%s: expected 131072 bytes, got %d" % (path, t.size * 2))
    return t.astype(np.uint16)


def table_from_function(fn):
    """fn(a, b) -> product, evaluated for a outer, b inner (the order of the reference's generator)."""
    a = np.arange(256, dtype=np.int64)[:, None]
    b = np.arange(256, dtype=np.int64)[None, :]
    return np.clip(np.broadcast_to(fn(a, b), (256, 256)), 0, 65535).astype(np.uint16).reshape(-1)


def error_stats(table):
    t = np.asarray(table, np.int64).reshape(256, 256)
    exact = np.arange(256, dtype=np.int64)[:, None] * np.arange(256, dtype=np.int64)[None, :]
    err = t - exact
    return {"mean_abs_error": float(np.abs(err).mean()), "max_abs_error": int(np.abs(err).max()),
            "mean_error": float(err.mean()), "wrong_entries": int((err != 0).sum()),
            "symmetric": bool(np.array_equal(t, t.T))}


def main(argv):
    from . import synth
    if len(argv) < 3:
        print(__doc__)
        return 2
    kind = argv[1]
    if kind == "exact":
        write_table(argv[2], synth.table_exact())
    elif kind == "truncated":
        write_table(argv[3], synth.table_truncated(int(argv[2])))
    elif kind == "noisy":
        write_table(argv[3], synth.table_noisy(int(argv[2])))
    elif kind == "uniform":
        write_table(argv[3], synth.table_uniform_error(int(argv[2])))
    elif kind == "tune":
        from . import ops
        write_table(argv[3], ops.tune_table(read_table(argv[2])))
    elif kind == "info":
        for k, v in error_stats(read_table(argv[2])).items():
            print("%-16s %s" % (k, v))
    else:
        print(__doc__)
        return 2
    return 0


if __name__ == "__main__":
    import importlib.util
    import os
    here = os.path.dirname(os.path.abspath(__file__))
    spec = importlib.util.spec_from_file_location("tf_approximate_amd", os.path.join(here, "__init__.py"),
                                                  submodule_search_locations=[here])
    pkg = importlib.util.module_from_spec(spec)
    sys.modules["tf_approximate_amd"] = pkg
    spec.loader.exec_module(pkg)
    from tf_approximate_amd import tables as _self
    sys.exit(_self.main(sys.argv))
