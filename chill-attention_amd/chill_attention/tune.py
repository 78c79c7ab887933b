"""Tile sweep for the static MI355X tile table — the counterpart of the reference's
``benchmark/spills.py`` and ``benchmark/gen_configs.py``, which time every Triton tile shape and
record register spills to fill ``autotune.py``'s default tables.

Here a tile shape is a compile-time property of a library, so a candidate is a BUILD of the library
with the table overridden (``CHILL_TUNE_*`` macros of ``csrc/chill_tiles.h``):

    python -m chill_attention.tune resources            # registers / LDS / spills of every kernel of the shipped table
    python -m chill_attention.tune build                 # compile all candidate libraries (no GPU needed)
    python -m chill_attention.tune time [C3 C2 ...]      # time every built candidate on the GPU, print a table

``build`` and ``time`` are separate because compiling belongs on the CPU and timing on the GPU box.
The shipped table takes, per mask class and head dim, the row that wins on the BASELINE workloads.
"""

from __future__ import annotations

import json
import os
import re
import subprocess
import sys
import tempfile

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_PKG_DIR)
CSRC_DIR = os.path.join(_ROOT, "csrc")
TUNE_LIB_DIR = os.path.join(_ROOT, "lib", "tune")
TUNE_BUILD_DIR = os.path.join(_ROOT, "build", "tune")

# (name, {macro: value}): forward and dQ shapes for 16-bit inputs with head dim <= 128
CANDIDATES = [
    ("shipped", {}),  # the table as it ships
    ("w8_s64", {"CHILL_TUNE_FWD_WAVES": 8, "CHILL_TUNE_DQ_WAVES": 8, "CHILL_TUNE_FWD_STREAMED": 64,
                "CHILL_TUNE_DQ_STREAMED": 64, "CHILL_TUNE_FWD_STAGES": 3, "CHILL_TUNE_DQ_STAGES": 3}),
    ("w8_s32", {"CHILL_TUNE_FWD_WAVES": 8, "CHILL_TUNE_DQ_WAVES": 8, "CHILL_TUNE_FWD_STREAMED": 32,
                "CHILL_TUNE_DQ_STREAMED": 32, "CHILL_TUNE_FWD_STAGES": 3, "CHILL_TUNE_DQ_STAGES": 3}),
    ("w8_s128", {"CHILL_TUNE_FWD_WAVES": 8, "CHILL_TUNE_DQ_WAVES": 8, "CHILL_TUNE_FWD_STREAMED": 128,
                 "CHILL_TUNE_DQ_STREAMED": 128, "CHILL_TUNE_FWD_STAGES": 2, "CHILL_TUNE_DQ_STAGES": 2}),
    # 4 waves, one workgroup per CU (three LDS stages)
    ("w4_s64", {"CHILL_TUNE_FWD_WAVES": 4, "CHILL_TUNE_DQ_WAVES": 4, "CHILL_TUNE_FWD_STREAMED": 64,
                "CHILL_TUNE_DQ_STREAMED": 64, "CHILL_TUNE_FWD_STAGES": 3, "CHILL_TUNE_DQ_STAGES": 3}),
    # 4 waves, two workgroups per CU (two or three LDS stages of half the size)
    ("w4_s64_n2", {"CHILL_TUNE_FWD_WAVES": 4, "CHILL_TUNE_DQ_WAVES": 4, "CHILL_TUNE_FWD_STREAMED": 64,
                   "CHILL_TUNE_DQ_STREAMED": 64, "CHILL_TUNE_FWD_STAGES": 2, "CHILL_TUNE_DQ_STAGES": 2}),
    ("w4_s32_n3", {"CHILL_TUNE_FWD_WAVES": 4, "CHILL_TUNE_DQ_WAVES": 4, "CHILL_TUNE_FWD_STREAMED": 32,
                   "CHILL_TUNE_DQ_STREAMED": 32, "CHILL_TUNE_FWD_STAGES": 3, "CHILL_TUNE_DQ_STAGES": 3}),
]

_HIPFLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-Wno-unused-value",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def candidate_library(name: str) -> str:
    return os.path.join(TUNE_LIB_DIR, name, "libchill_attention_hip.so")


def build_candidates(jobs: int = 8) -> None:
    for name, macros in CANDIDATES:
        extra = " ".join(f"-D{k}={v}" for k, v in macros.items() if k != "__flags__")
        cmd = ["make", "-C", CSRC_DIR, f"-j{jobs}", f"EXTRA={extra}", f"HIPEXTRA={macros.get('__flags__', '')}",
               f"BUILD={os.path.join(TUNE_BUILD_DIR, name)}", f"LIBDIR={os.path.dirname(candidate_library(name))}"]
        print("building", name, extra, flush=True)
        subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL)


def kernel_resources(elem: str = "bf16", dim: int = 128, macros: dict | None = None) -> list:
    """Per-kernel register, LDS and spill figures of one (element type, head dim) translation unit
    pair, read from the code-object metadata hipcc writes (``-S``)."""
    rows = []
    with tempfile.TemporaryDirectory() as tmp:
        # (at head dim 128 only the backward has such kernels)
        for unit in ("chill_fwd_inst.hip", "chill_bwd_inst.hip") if dim == 256 else ("chill_bwd_inst.hip",):
            out = os.path.join(tmp, unit + ".s")
            cmd = ["hipcc", *_HIPFLAGS, f"-I{os.path.join(_ROOT, '..', 'include')}",
                   f"-DCHILL_ELEM={elem}_t", f"-DCHILL_ELEM_NAME={elem}", f"-DCHILL_HEAD_DIM={dim}",
                   *[f"-D{k}={v}" for k, v in (macros or {}).items() if k != "__flags__"],
                   *(macros or {}).get("__flags__", "").split(),
                   "--cuda-device-only", "-S", os.path.join(CSRC_DIR, unit), "-o", out]
            subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
            text = open(out).read()
            for block in re.findall(r"- \.agpr_count:.*?\.wavefront_size:", text, flags=re.S):
                get = lambda key: int(re.search(rf"\.{key}:\s+(\d+)", block).group(1))  # noqa: E731
                name = re.search(r"\.name:\s+(\S+)", block).group(1)
                demangled = subprocess.run(["c++filt", name], capture_output=True, text=True).stdout.strip()
                rows.append({
                    "kernel": re.sub(r"\(.*", "", demangled).replace("void chill::", ""),
                    "vgpr": get("vgpr_count"), "agpr": get("agpr_count"), "sgpr": get("sgpr_count"),
                    "lds_static": get("group_segment_fixed_size"),
                    "vgpr_spill": get("vgpr_spill_count"), "sgpr_spill": get("sgpr_spill_count"),
                    "scratch": get("private_segment_fixed_size"),
                })
    return rows


def check_hand_managed_registers(macros: dict | None = None) -> None:
    """Raise RuntimeError unless, in every kernel that names accumulation registers itself (16-bit inputs:
    the three kernels of head dim 256, dK/dV with register-resident K at head dims 64 and 128, dQ with register-resident Q and dO at head dim 128), the compiler stays
    below the registers the kernel names.  Spilled registers are accepted only where the compiler touches
    no accumulation register at all (they are in scratch memory then, not parked in accumulation
    registers).  The check reads the assembly hipcc writes for the given build (``macros`` as for the
    library build); it covers register overlap and spills, nothing else.  Part of every build of the library."""
    for elem in ("bf16", "f16"):
        for dim in (256, 128, 64):
            rows = hand_managed_registers(elem, dim, macros)
            if not rows:
                raise RuntimeError(f"no hand-managed kernel found for {elem} head dim {dim}")
            for name, compiler_max, hand_min, spilled in rows:
                if compiler_max >= hand_min or (spilled and compiler_max >= 0):
                    raise RuntimeError(
                        f"kernel {name}: the compiler uses accumulation registers up to a{compiler_max} (the kernel "
                        f"manages a{hand_min} and above itself) or spills ({spilled} registers): this build is unsound")


def hand_managed_registers(elem: str = "bf16", dim: int = 256, macros: dict | None = None) -> list:
    """Kernels that name accumulation registers themselves (fwd_regs_kernel, dq_regs_kernel, dkdv_regs_kernel) rely on the compiler
    keeping out of them.  Compiles the translation units of (elem, dim) to assembly and
    returns, per such kernel, (name, highest accumulation register the COMPILER uses or -1, lowest one
    the kernel's own asm statements name, spilled registers): sound iff the first is below the second
    and nothing is spilled."""
    text = ""
    with tempfile.TemporaryDirectory() as tmp:
        # (at head dim 128 only the backward has such kernels)
        for unit in ("chill_fwd_inst.hip", "chill_bwd_inst.hip") if dim == 256 else ("chill_bwd_inst.hip",):
            out = os.path.join(tmp, unit + ".s")
            cmd = ["hipcc", *_HIPFLAGS, f"-I{os.path.join(_ROOT, '..', 'include')}",
                   f"-DCHILL_ELEM={elem}_t", f"-DCHILL_ELEM_NAME={elem}", f"-DCHILL_HEAD_DIM={dim}",
                   *[f"-D{k}={v}" for k, v in (macros or {}).items() if k != "__flags__"],
                   *(macros or {}).get("__flags__", "").split(),
                   "--cuda-device-only", "-S", os.path.join(CSRC_DIR, unit), "-o", out]
            subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
            text += open(out).read()
    spills = {}
    for block in re.findall(r"- \.agpr_count:.*?\.wavefront_size:", text, flags=re.S):
        name = re.search(r"\.name:\s+(\S+)", block).group(1)
        spills[name] = int(re.search(r"\.vgpr_spill_count:\s+(\d+)", block).group(1))
    rows, cur, in_asm = {}, None, False
    for line in text.splitlines():
        m = re.match(r"^(_ZN5chill\w+):", line)
        if m:
            cur = m.group(1) if re.search(r"_regs\d*_kernel", m.group(1)) else None
            if cur:
                rows[cur] = {"compiler": -1, "hand": 1 << 30}
            continue
        if line.startswith(".Lfunc_end"):
            cur = None
        if cur is None:
            continue
        if "#ASMSTART" in line:
            in_asm = True
            continue
        if "#ASMEND" in line:
            in_asm = False
            continue
        code = line.split(";")[0]
        used = [int(x) for x in re.findall(r"\ba(\d+)\b", code)]
        for lo, hi in re.findall(r"\ba\[(0x[0-9a-f]+|\d+)(?::(0x[0-9a-f]+|\d+))?\]", code):
            used += [int(lo, 0), int(hi, 0) if hi else int(lo, 0)]
        if used:
            if in_asm:
                rows[cur]["hand"] = min(rows[cur]["hand"], min(used))
            else:
                rows[cur]["compiler"] = max(rows[cur]["compiler"], max(used))
    return [(k, v["compiler"], v["hand"], spills.get(k, -1)) for k, v in rows.items()]


def time_candidates(workloads) -> list:
    """Kernel times of every built candidate on the given bench workloads (needs the GPU).  Each
    candidate runs in a process of its own, because a process binds one build of the library."""
    results = []
    bench = os.path.join(_ROOT, "..", "bench.py")
    for name, _ in CANDIDATES:
        lib = candidate_library(name)
        if not os.path.exists(lib):
            print(f"{name}: not built, skipped")
            continue
        for w in workloads:
            env = dict(os.environ, CHILL_ATTENTION_LIB=lib)
            res = subprocess.run([sys.executable, bench, "--workload", w, "--steps", "10", "--warmup", "3",
                                  "--no-cpu-baseline"], env=env, capture_output=True, text=True)
            if res.returncode != 0:
                print(f"{name} {w}: failed\n{res.stderr[-500:]}")
                continue
            line = json.loads(res.stdout.strip().splitlines()[-1])
            results.append({"candidate": name, "workload": w, "tflops": line["value"], **line["kernel_ms"]})
            print(f"{name:8s} {w:4s} " + "  ".join(f"{k[6:]} {v:.3f} ms" for k, v in line["kernel_ms"].items())
                  + f"  -> {line['value']:.1f} TFLOP/s", flush=True)
    return results


def main(argv) -> None:
    what = argv[0] if argv else "resources"
    if what == "resources":
        for row in kernel_resources():
            print(row)
    elif what == "build":
        build_candidates()
    elif what == "time":
        time_candidates(argv[1:] or ["C3"])
    else:
        raise SystemExit(__doc__)


if __name__ == "__main__":
    main(sys.argv[1:])
