"""Builds libaxconv_hip.so (gfx950 only) in-tree with hipcc."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libaxconv_hip.so")
SOURCES = ["axconv_api.hip", "lutgemm_kernel.hip", "lutgemm_px_kernel.hip", "prepass_kernels.hip", "depthwise_kernel.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # -Wno-inline-asm: the generated phase bodies name m0, which they write, in their clobber lists, and clang
    # warns about every reserved register it sees there
    "-Wall", "-Wno-unused-command-line-argument", "-Wno-inline-asm",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
]


def generate():
    """Writes csrc/lookup_asm.inc, the generated inline assembly of the lookup phase."""
    gen = os.path.join(CSRC, "gen_lookup_asm.py")
    text = subprocess.run([sys.executable, gen], stdout=subprocess.PIPE, text=True, check=True).stdout
    with open(os.path.join(CSRC, "lookup_asm.inc"), "w") as f:
        f.write(text)


def build(verbose=False, extra=()):
    generate()
    cmd = ["hipcc"] + FLAGS + list(extra) + [os.path.join(CSRC, s) for s in SOURCES] + ["-o", LIB]
    if verbose:
        print(" ".join(cmd))
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the packed-fp32 target feature and says so; that line is noise
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    build_harness(verbose)
    return LIB


SHELL = os.path.join(HERE, "shell")
HARNESS = os.path.join(HERE, "axconv_harness")


def build_harness(verbose=False):
    """The TensorFlow-free op shell plus the standalone C++ harness, linked against the library."""
    cmd = ["hipcc", "--offload-arch=gfx950", "-O2", "-std=c++17", "-Wall", "-Wno-unused-command-line-argument",
           "-I", os.path.join(ROOT, "include"), "-I", SHELL,
           os.path.join(SHELL, "approx_conv2d_op.cc"), os.path.join(SHELL, "axconv_harness.cc"),
           "-L", HERE, "-laxconv_hip", "-Wl,-rpath,$ORIGIN", "-o", HARNESS]
    if verbose:
        print(" ".join(cmd))
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed (harness):\n" + res.stdout)
    return HARNESS


if __name__ == "__main__":
    build(verbose=True, extra=sys.argv[1:])
    print("built", LIB)
