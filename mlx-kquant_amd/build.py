"""Builds libkq.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

    python mlx-kquant_amd/build.py            # rebuild everything
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "lib", "libkq.so")
BLOB = os.path.join(HERE, "data", "kq_iq_grids.bin")

# (source, extra flags[, object name]).  kq_generic.hip holds the bit-exact decoders: no FMA contraction.
SOURCES = [
    ("kq_api.cpp", ["-x", "hip"]),
    ("kq_encode.cpp", ["-x", "hip"]),
    ("kq_generic.hip", ["-ffp-contract=off"]),
    ("kq_mfma.hip", []),
    ("kq_nt.hip", ["-ffp-contract=off"]),
    # one source, two objects: the dense and the gathered launchers instantiate their kernels in parallel
    ("kq_stream.hip", ["-Wno-inline-asm", "-DKQ_STREAM_PART=1"], "kq_stream_dense"),
    ("kq_stream.hip", ["-Wno-inline-asm", "-DKQ_STREAM_PART=2"], "kq_stream_gather"),
    ("kq_gemm.hip", []),
    ("kq_gemm2.hip", ["-Wno-inline-asm"]),
    ("kq_gemm3.hip", ["-Wno-inline-asm"]),
    ("kq_gemm3b.hip", ["-Wno-inline-asm"]),
    ("kq_gemm3f.hip", ["-Wno-inline-asm"]),
    ("kq_gemm3i.hip", ["-Wno-inline-asm", "-ffp-contract=off"]),
    ("kq_moe.hip", []),
    ("kq_anymma.hip", ["-ffp-contract=off"]),
    # one source, three objects: its kernel families are instantiated in parallel
    ("kq_codes.hip", ["-DKQ_CODES_PART=1"], "kq_codes_dense"),
    ("kq_codes.hip", ["-DKQ_CODES_PART=2"], "kq_codes_gather"),
    ("kq_codes.hip", ["-DKQ_CODES_PART=3"], "kq_codes_grouped"),
    ("kq_fp4.hip", []),
    ("kq_router.hip", ["-ffp-contract=off"]),
    # the device encoder must round exactly like the host one: no fused multiply-adds
    ("kq_encode_dev.hip", ["-ffp-contract=off"]),
]
COMMON = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
    # packed-FP32 VALU forms are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-fno-strict-aliasing",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC, "-I", OBJ,
]
GRID_INC = os.path.join(OBJ, "kq_iq_grids.inc")


def _write_grid_inc():
    """The IQ codebook data file as a C byte list (initialiser of the __device__ array in kq_api.cpp)."""
    data = open(BLOB, "rb").read()
    lines = [",".join(str(b) for b in data[i:i + 32]) + "," for i in range(0, len(data), 32)]
    text = "\n".join(lines) + "\n"
    if not os.path.exists(GRID_INC) or open(GRID_INC).read() != text:
        with open(GRID_INC, "w") as f:
            f.write(text)



def _hipcc():
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.isabs(c) and os.path.exists(c) or not os.path.isabs(c)):
            return c
    raise RuntimeError("hipcc not found")


def _compile(item):
    src, extra = item[0], item[1]
    out = os.path.join(OBJ, (item[2] if len(item) > 2 else os.path.splitext(src)[0]) + ".o")
    cmd = [_hipcc()] + COMMON + extra + ["-c", os.path.join(CSRC, src), "-o", out]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    log = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, log))
    if log.strip():
        print(log)
    return out


def build_all(verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    _write_grid_inc()
    with ThreadPoolExecutor(max_workers=6) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build_all()
    sys.exit(0)
