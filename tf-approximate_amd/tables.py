"""Truth-table files in the reference's format (tf2/README.md:104-117): 65536 little-endian uint16,
entry [a * 256 + b] = approximate product of input code a and filter code b.

    python tables.py exact out.bin
    python tables.py truncated 4 out.bin        # a*b - (a*b mod 2^k)
    python tables.py noisy SEED out.bin         # clamp(a*b + round(N(0, 0.02*a*b)))
    python tables.py uniform SEED out.bin       # clamp(a*b + U(-64, 64))
    python tables.py tune in.bin out.bin        # the tf1 AxTune column remap (needs the built library)
    python tables.py info in.bin                # error statistics against exact multiplication
    python tables.py cmodel model.c FUNC out.bin [u64|u8]
                                                # compile a C model of a multiplier with gcc and tabulate FUNC(a, b);
                                                # u64 (default): uint64_t FUNC(uint64_t, uint64_t), the EvoApproxLib
                                                # form; u8: uint16_t FUNC(uint8_t, uint8_t)
"""
import os
import subprocess
import sys
import tempfile

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


_DRIVER = """#include <stdint.h>
#include <stdio.h>
%(proto)s;
int main(int argc, char **argv)
{
    FILE *f = fopen(argv[1], "wb");
    if (!f)
        return 1;
    for (unsigned a = 0; a < 256; a++)          /* input code outer, filter code inner: tf2/README.md:104-117 */
        for (unsigned b = 0; b < 256; b++) {
            uint16_t v = (uint16_t)%(func)s(a, b);
            if (fwrite(&v, sizeof v, 1, f) != 1)
                return 1;
        }
    return fclose(f) ? 1 : 0;
}
"""


def table_from_c_model(source, func, proto="u64", cc="gcc"):
    """Tabulates a C model of an 8x8 multiplier the way the reference's recipe does (tf2/README.md:104-117):
    compiles `source` together with a generated driver and returns the 65536 products FUNC(a, b), a outer.
    proto "u64": uint64_t FUNC(uint64_t, uint64_t) (the form of the EvoApproxLib models); "u8":
    uint16_t FUNC(uint8_t, uint8_t)."""
    if not func.isidentifier():
        raise ValueError("not a C identifier: %r" % (func,))
    protos = {"u64": "uint64_t %s(uint64_t, uint64_t)", "u8": "uint16_t %s(uint8_t, uint8_t)"}
    if proto not in protos:
        raise ValueError("proto must be u64 or u8")
    with tempfile.TemporaryDirectory() as tmp:
        driver = os.path.join(tmp, "driver.c")
        with open(driver, "w") as f:
            f.write(_DRIVER % {"proto": protos[proto] % func, "func": func})
        exe = os.path.join(tmp, "tabulate")
        r = subprocess.run([cc, "-O2", "-o", exe, driver, os.path.abspath(source)], stdout=subprocess.PIPE,
                           stderr=subprocess.STDOUT, text=True)
        if r.returncode != 0:
            raise RuntimeError("compiling %s failed:\n%s" % (source, r.stdout))
        out = os.path.join(tmp, "table.bin")
        subprocess.run([exe, out], check=True)
        return read_table(out)


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
    elif kind == "cmodel":
        if len(argv) < 5:
            print(__doc__)
            return 2
        write_table(argv[4], table_from_c_model(argv[2], argv[3], argv[5] if len(argv) > 5 else "u64"))
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
