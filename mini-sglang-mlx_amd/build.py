"""Compile the HIP sources under ``csrc/`` into ``lib/libmsgl_paged_attention.so`` (gfx950).

Usage: ``python build.py [--force]``.  hipcc cross-compiles, so this runs without a GPU.
Each ``.hip`` file is compiled to an object on its own (in parallel) and the objects are
linked into one shared library whose only exported symbols are the ``msgl_*`` C ABI of
``include/msgl_paged_attention.h``, ``include/msgl_radix_cache.h`` and
``include/msgl_state_pool.h``.
"""
from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(LIB_DIR, "libmsgl_paged_attention.so")
SOURCES = ["api.hip", "store_kv_cache.hip", "paged_splitkv.hip", "paged_prefill.hip", "paged_prefill_d256.hip",
           "build_metadata.hip", "qk_norm_rope_store.hip",
           "gdn_state.hip", "radix_cache.hip", "state_slots.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# Packed fp32 VALU forms are switched off for every device compile on this target.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
]


def _newer(src_paths, target) -> bool:
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(s) > t for s in src_paths)


def _compile(src: str, save_temps: bool) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    if save_temps:
        cmd.insert(1, "--save-temps=obj")
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the device feature flag; that warning is expected
    err = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(force: bool = False, save_temps: bool = False) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    headers.append(os.path.join(HERE, "..", "include", "msgl_paged_attention.h"))
    headers.append(os.path.join(HERE, "..", "include", "msgl_radix_cache.h"))
    headers.append(os.path.join(HERE, "..", "include", "msgl_state_pool.h"))
    todo = []
    for src in SOURCES:
        obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
        if force or _newer([os.path.join(CSRC, src), *headers], obj):
            todo.append(src)
    with concurrent.futures.ThreadPoolExecutor(max_workers=4) as ex:
        list(ex.map(lambda s: _compile(s, save_temps), todo))
    objs = [os.path.join(OBJ_DIR, os.path.splitext(s)[0] + ".o") for s in SOURCES]
    if todo or force or _newer(objs, LIB_PATH):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB_PATH]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"link failed:\n{proc.stderr}")
    return LIB_PATH


if __name__ == "__main__":
    path = build(force="--force" in sys.argv, save_temps="--save-temps" in sys.argv)
    print(path)
