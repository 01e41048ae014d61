"""Builds ``libtracea.so`` (HIP kernels for gfx950 + the C ABI) in-tree.

Usage: ``python -m tracea_amd.build [--force] [-j N]``.  hipcc cross-compiles
without a GPU, so this runs on any machine with ROCm installed.  Each line of
``csrc/contraction_variants.def`` becomes one translation unit compiled from
``csrc/contraction_variant.hip`` with the tile shape passed as -D flags.
"""
import argparse
import concurrent.futures
import hashlib
import json
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
# TRACEA_BUILD_CSRC / TRACEA_BUILD_OUT redirect the build to another source tree / output
# directory (kernel experiments); by default everything stays inside the package.
CSRC = os.environ.get("TRACEA_BUILD_CSRC") or os.path.join(HERE, "csrc")
_OUT = os.environ.get("TRACEA_BUILD_OUT") or HERE
OBJ = os.path.join(_OUT, "_obj")
LIB_DIR = os.path.join(_OUT, "lib")
LIB = os.path.join(LIB_DIR, "libtracea.so")
BIN_DIR = os.path.join(_OUT, "bin")
TUNER_BIN = os.path.join(BIN_DIR, "tracea-tuner")

ARCH = "gfx950"
# -packed-fp32-ops: keep the compiler from forming packed fp32 VALU instructions.
DEVICE_FLAGS = ["--offload-arch=" + ARCH, "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
INCLUDE = os.path.normpath(os.path.join(HERE, "..", "include"))
COMMON = ["-I" + INCLUDE, "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wall", "-Wno-unused-command-line-argument",
          "-Wno-pass-failed"]

HOST_SOURCES = ["abi.cpp", "tuner_abi.cpp", "graph_abi.cpp", "plan_abi.cpp", "ttg_abi.cpp", "host/tile_graph.cpp", "host/execution_plan.cpp", "contraction_registry.cpp", "host/dispatch.cpp", "host/tuning.cpp",
                "host/pipeline_config.cpp", "host/gaussian_process.cpp", "host/autotuner.cpp",
                "host/graph_fusion.cpp"]
DEVICE_SOURCES = ["support_kernels.hip", "conv_transpose_kernels.hip", "graph_kernels.hip", "attention_kernels.hip"]


def hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def variants():
    text = open(os.path.join(CSRC, "contraction_variants.def")).read()
    out = []
    for m in re.finditer(r"^TRACEA_VARIANT\(([^)]*)\)", text, re.M):
        f = [x.strip() for x in m.group(1).split(",")]
        out.append(dict(name=f[0], bm=f[1], bn=f[2], bk=f[3], wm=f[4], wn=f[5], stages=f[6], direct=f[7]))
    return out


def _headers_digest():
    h = hashlib.sha1()
    for root, _, files in os.walk(CSRC):
        for fn in sorted(files):
            if fn.endswith((".hpp", ".h", ".def")):
                h.update(open(os.path.join(root, fn), "rb").read())
    h.update(open(os.path.join(INCLUDE, "tracea.h"), "rb").read())
    return h.hexdigest()


def _jobs():
    jobs = []
    for v in variants():
        defs = ["-DV_NAME=" + v["name"], "-DV_BM=" + v["bm"], "-DV_BN=" + v["bn"], "-DV_BK=" + v["bk"],
                "-DV_WM=" + v["wm"], "-DV_WN=" + v["wn"], "-DV_STAGES=" + v["stages"],
                "-DV_DIRECT=" + v["direct"]]
        jobs.append((os.path.join(CSRC, "contraction_variant.hip"),
                     os.path.join(OBJ, "variant_" + v["name"] + ".o"), DEVICE_FLAGS + defs))
    for s in DEVICE_SOURCES:
        jobs.append((os.path.join(CSRC, s), os.path.join(OBJ, s.replace("/", "_") + ".o"), DEVICE_FLAGS))
    for s in HOST_SOURCES:
        jobs.append((os.path.join(CSRC, s), os.path.join(OBJ, s.replace("/", "_") + ".o"), []))
    return jobs


def _compile(job, digest, force):
    src, obj, flags = job
    stamp = obj + ".stamp"
    device = "--offload-arch=" + ARCH in flags
    key = hashlib.sha1((digest + open(src, "rb").read().hex() + " ".join(flags)).encode()).hexdigest()
    if (not force and os.path.exists(obj) and os.path.exists(stamp) and open(stamp).read() == key and
            (not device or os.path.exists(obj + ".resources.json"))):
        return obj, False
    cmd = [hipcc()] + COMMON + flags + (["-Rpass-analysis=kernel-resource-usage"] if device else []) + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("compile failed: %s\n%s" % (" ".join(cmd), r.stderr[-4000:]))
    if device:
        with open(obj + ".resources.json", "w") as f:
            json.dump(_kernel_resources(r.stderr), f)
    open(stamp, "w").write(key)
    return obj, True


_REMARK = re.compile(r"remark:\s+(Function Name|VGPRs|AGPRs|ScratchSize \[bytes/lane\]|VGPRs Spill|"
                     r"LDS Size \[bytes/block\]|Occupancy \[waves/SIMD\]): (\S+)")
_FIELDS = {"VGPRs": "vgprs", "AGPRs": "agprs", "ScratchSize [bytes/lane]": "scratch_bytes", "VGPRs Spill": "vgpr_spills",
           "LDS Size [bytes/block]": "lds_bytes", "Occupancy [waves/SIMD]": "waves_per_simd"}


def _kernel_resources(remarks):
    """What the compiler reports per kernel (-Rpass-analysis=kernel-resource-usage): registers,
    scratch bytes per lane, static LDS.  A kernel of this library that needs scratch memory has
    always been a mistake in its source (a run-time index into registers or into the argument
    block), costing a factor of two: the numbers are kept so that a test can watch them."""
    out, cur = [], None
    for m in _REMARK.finditer(remarks):
        key, val = m.group(1), m.group(2)
        if key == "Function Name":
            cur = {"name": val}
            out.append(cur)
        elif cur is not None:
            cur[_FIELDS[key]] = int(val)
    return out


def build(force=False, jobs=None, verbose=True):
    """Compile every translation unit and link ``lib/libtracea.so``."""
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    digest = _headers_digest()
    todo = _jobs()
    jobs = jobs or min(8, os.cpu_count() or 4)
    objs, rebuilt = [], 0
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        for obj, did in ex.map(lambda j: _compile(j, digest, force), todo):
            objs.append(obj)
            rebuilt += int(did)
    # per-kernel resource usage of everything that goes into the library, next to it
    resources = {}
    for obj in objs:
        if os.path.exists(obj + ".resources.json"):
            for k in json.load(open(obj + ".resources.json")):
                resources[k["name"]] = {f: v for f, v in k.items() if f != "name"}
    with open(os.path.join(LIB_DIR, "kernel_resources.json"), "w") as f:
        json.dump(resources, f, indent=0, sort_keys=True)
    if rebuilt or force or not os.path.exists(LIB):
        cmd = [hipcc(), "-shared", "-fPIC", "--offload-arch=" + ARCH, "-o", LIB] + objs
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stderr[-4000:])
    # command-line tuner: plain C++ over the public headers, linked against the library
    os.makedirs(BIN_DIR, exist_ok=True)
    src = os.path.join(CSRC, "tools", "tuner_main.cpp")
    if (rebuilt or force or not os.path.exists(TUNER_BIN)
            or os.path.getmtime(TUNER_BIN) < os.path.getmtime(src)):
        cmd = ["g++", "-std=c++17", "-O2", "-Wall", "-I", INCLUDE, src, "-o", TUNER_BIN, "-L", LIB_DIR, "-ltracea",
               "-Wl,-rpath,$ORIGIN/../lib"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("tuner link failed:\n" + r.stderr[-4000:])
    if verbose:
        print("libtracea.so: %d of %d objects rebuilt -> %s" % (rebuilt, len(todo), LIB))
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("-j", type=int, default=None)
    a = ap.parse_args()
    try:
        build(force=a.force, jobs=a.j)
    except RuntimeError as e:
        sys.stderr.write(str(e) + "\n")
        sys.exit(1)
