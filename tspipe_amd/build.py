"""Builds libtspipe_amd.so (gfx950) from tspipe_amd/csrc with hipcc.

Run as ``python -m tspipe_amd.build``.  The library is written next to this
file so it travels with the source tree; nothing is installed.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(HERE, "libtspipe_amd.so")
SOURCES = ["misc.cpp", "plan.cpp", "ema_copy.hip", "losses.hip", "kd.hip", "bn.hip", "infonce.hip", "infonce_general.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -packed-fp32-ops off: the compiler's automatic v_pk_*_f32 forms are not
# trusted on this hardware pool.
DEVICE_FLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
COMMON_FLAGS = ["-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function", "-x", "hip"]


def _compile(src: str, defines=(), obj_dir: str = OBJ_DIR) -> str:
    obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *COMMON_FLAGS, *DEVICE_FLAGS, *["-D" + d for d in defines], "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(_compile, SOURCES))
    tmp = LIB_PATH + ".tmp"
    cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", *objs, "-o", tmp]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH}")
    return LIB_PATH


# Measurement variants: the library with one source rebuilt under a macro, for
# A/B runs against the default build (TSPIPE_AMD_LIBRARY selects the file that
# tspipe_amd loads).  None of them is loaded unless asked for.
VARIANTS = {
    # long 16-bit KD rows parked in LDS instead of registers between the walks
    "kd-rows-in-lds": ("kd.hip", ["TS_KD_ROWS_IN_LDS"]),
}


def build_variant(name: str, verbose: bool = True) -> str:
    """Builds libtspipe_amd.<name>.so: the objects of the default build (built
    first if missing) with the variant's source recompiled under its macros."""
    src, defines = VARIANTS[name]
    if not all(os.path.exists(os.path.join(OBJ_DIR, os.path.splitext(s)[0] + ".o")) for s in SOURCES):
        build(verbose=False)
    var_dir = os.path.join(OBJ_DIR, name)
    os.makedirs(var_dir, exist_ok=True)
    var_obj = _compile(src, defines, var_dir)
    objs = [var_obj if s == src else os.path.join(OBJ_DIR, os.path.splitext(s)[0] + ".o") for s in SOURCES]
    out = os.path.join(HERE, f"libtspipe_amd.{name}.so")
    res = subprocess.run([HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", *objs, "-o", out],
                         capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    if verbose:
        print(f"built {out}")
    return out


HOST_DIR = os.path.join(HERE, "csrc_host")
HOST_NAME = "_ts_hostlist"


def build_host(verbose: bool = False) -> str:
    """Builds the optional host-side list helper (plain C++ against torch's
    headers, no GPU code) into tspipe_amd/csrc_host/.  The adapters work
    without it, only with more Python overhead per call."""
    from torch.utils import cpp_extension
    os.makedirs(os.path.join(HOST_DIR, "build"), exist_ok=True)
    cpp_extension.load(name=HOST_NAME, sources=[os.path.join(HOST_DIR, "hostlist.cpp")],
                       build_directory=os.path.join(HOST_DIR, "build"), extra_cflags=["-O2"], verbose=verbose)
    built = os.path.join(HOST_DIR, "build", HOST_NAME + ".so")
    final = os.path.join(HERE, HOST_NAME + ".so")
    import shutil
    shutil.copyfile(built, final + ".tmp")
    os.replace(final + ".tmp", final)
    return final


CONSUMER_SRC = os.path.join(os.path.dirname(HERE), "tests", "cabi", "consumer.cpp")
CONSUMER_BIN = os.path.join(os.path.dirname(HERE), "tests", "cabi", "build", "consumer")


def build_consumer(verbose: bool = False) -> str:
    """Builds the stand-alone C++ consumer of the C ABI (tests/cabi): host code
    only, linked against the library with an rpath, no Python or torch."""
    os.makedirs(os.path.dirname(CONSUMER_BIN), exist_ok=True)
    cmd = [HIPCC, "-O2", "-std=c++17", "-Wall", "--offload-arch=gfx950", CONSUMER_SRC, "-o", CONSUMER_BIN,
           "-L" + HERE, "-ltspipe_amd", "-Wl,-rpath,$ORIGIN/../../../tspipe_amd"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"building the C-ABI consumer failed:\n{res.stderr}")
    if verbose:
        print(f"built {CONSUMER_BIN}")
    return CONSUMER_BIN


if __name__ == "__main__":
    if len(sys.argv) > 2 and sys.argv[1] == "--variant":
        build_variant(sys.argv[2])
    else:
        build()
        build_host()
        build_consumer()
