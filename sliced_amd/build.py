"""Builds the gfx950 libraries in-tree with hipcc (cross-compiles without a GPU).

    python -m sliced_amd.build            # libsliced_hip.so (kernels + C ABI) and libsliced_host.so

Flags:
  --offload-arch=gfx950       the only target; there is no other code path
  -ffp-contract=off           elementwise arithmetic rounds op by op, like the reference's scalar loops
  -Xclang -target-feature -Xclang -packed-fp32-ops
                              do not form packed-fp32 VALU instructions
"""
import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "_build")
LIB_HIP = os.path.join(HERE, "libsliced_hip.so")
LIB_HOST = os.path.join(HERE, "libsliced_host.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
KERNEL_SOURCES = ["runtime.hip", "elementwise.hip", "ew_program.hip", "reduce.hip", "softmax.hip", "transpose.hip", "gemm.hip", "gemm_spread.hip", "gemm_wide.hip", "gemm_skinny.hip", "gemm_tall.hip", "gemm_bits.hip", "bcast_ops.hip", "loss.hip", "mlp_step.hip"]
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function",
    "-Wno-unknown-warning-option", "-Wno-unused-command-line-argument",
]
HOST_SOURCES = [os.path.join("host", "host_api.cpp")]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wall", "-I", os.path.join(HERE, "..", "include")]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_kernels(verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    jobs = []
    for src in KERNEL_SOURCES:
        obj = os.path.join(OBJ, src.replace(".hip", ".o"))
        jobs.append([HIPCC, *HIP_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj])
    with cf.ThreadPoolExecutor(max_workers=min(8, len(jobs))) as ex:
        for out in ex.map(_run, jobs):
            if verbose and out:
                print(out)
    objs = [j[-1] for j in jobs]
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_HIP, *objs])
    return LIB_HIP


def build_host(verbose=False):
    srcs = [os.path.join(CSRC, s) for s in HOST_SOURCES]
    if not all(os.path.exists(s) for s in srcs):
        return None
    out = _run(["g++", *HOST_FLAGS, "-shared", "-o", LIB_HOST, *srcs, "-L", HERE, "-lsliced_hip",
                "-Wl,-rpath,$ORIGIN"])
    if verbose and out:
        print(out)
    return LIB_HOST


CONSUMER_SRC = os.path.join(HERE, "..", "tests", "abi_consumer", "consumer.c")
CONSUMER = os.path.join(OBJ, "abi_consumer")


def build_consumer(verbose=False):
    """The plain-C caller of the ABI that the tests run (C99, -pedantic -Werror: the header has to be C)."""
    if not os.path.exists(CONSUMER_SRC):
        return None
    os.makedirs(OBJ, exist_ok=True)
    out = _run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-O1", "-I", os.path.join(HERE, "..", "include"),
                CONSUMER_SRC, "-o", CONSUMER, "-L", HERE, "-lsliced_hip", "-lm", "-Wl,-rpath,$ORIGIN/.."])
    if verbose and out:
        print(out)
    return CONSUMER


def build_all(verbose=False):
    libs = [build_kernels(verbose)]
    h = build_host(verbose)
    if h:
        libs.append(h)
    build_consumer(verbose)
    return libs


if __name__ == "__main__":
    for lib in build_all(verbose=True):
        print("built", lib)
    sys.exit(0)
