"""Build recipe for the gfx950 backend: compiles csrc/*.hip into zigrad_amd/libzg_hip.so.

hipcc cross-compiles for gfx950 without a GPU present.  Objects are cached by source mtime unless
`force` is set; the link step always runs when any object changed.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
OBJ_DIR = PKG_DIR / "build"
LIB_PATH = PKG_DIR / "libzg_hip.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -ffp-contract=off: elementwise/reduction kernels must round a*b+c like the host loops they replace.
# packed-fp32 code generation is disabled on purpose (compiler-formed v_pk_*_f32 are not trusted here).
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
    "-Wno-unused-command-line-argument",
]


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _headers_mtime() -> float:
    hdrs = list(CSRC.glob("*.h")) + [PKG_DIR.parent / "include" / "zg_hip.h"]
    return max(h.stat().st_mtime for h in hdrs)


def _compile(src: Path, force: bool) -> tuple[Path, bool]:
    obj = OBJ_DIR / (src.stem + ".o")
    newest = max(src.stat().st_mtime, _headers_mtime())
    if not force and obj.exists() and obj.stat().st_mtime >= newest:
        return obj, False
    cmd = [HIPCC, *FLAGS, "-c", str(src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError(f"hipcc failed for {src.name}")
    # the host pass warns that it does not know the packed-fp32 feature; anything else is shown
    noise = ("packed-fp32-ops", "warning generated", "warnings generated")
    for line in (res.stdout + res.stderr).splitlines():
        if line.strip() and not any(n in line for n in noise):
            sys.stderr.write(line + "\n")
    return obj, True


def build(force: bool = False, jobs: int | None = None) -> Path:
    OBJ_DIR.mkdir(exist_ok=True)
    srcs = sources()
    jobs = jobs or min(8, len(srcs))
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(lambda s: _compile(s, force), srcs))
    objs = [o for o, _ in results]
    changed = any(c for _, c in results)
    if changed or force or not LIB_PATH.exists():
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB_PATH), *map(str, objs)]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            sys.stderr.write(res.stdout + res.stderr)
            raise RuntimeError("link of libzg_hip.so failed")
    return LIB_PATH


C_HARNESS_SRC = PKG_DIR.parent / "examples" / "c_caller" / "mlp_step.c"
C_HARNESS_BIN = C_HARNESS_SRC.with_suffix("")
C_DQN_SRC = PKG_DIR.parent / "examples" / "c_caller" / "dqn_step.c"
C_DQN_BIN = C_DQN_SRC.with_suffix("")
C_GCN_SRC = PKG_DIR.parent / "examples" / "c_caller" / "gcn_step.c"
C_GCN_BIN = C_GCN_SRC.with_suffix("")


def build_c_harness() -> Path:
    """The plain-C callers of the C ABI (examples/c_caller/*.c), linked against the library in its tree."""
    for src, out in ((C_HARNESS_SRC, C_HARNESS_BIN), (C_DQN_SRC, C_DQN_BIN), (C_GCN_SRC, C_GCN_BIN)):
        cmd = ["gcc", "-std=c11", "-O2", "-Wall", "-Werror", "-D_POSIX_C_SOURCE=199309L", f"-I{PKG_DIR.parent / 'include'}",
               str(src), "-o", str(out), f"-L{PKG_DIR}", "-lzg_hip", "-Wl,-rpath,$ORIGIN/../../zigrad_amd"]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            sys.stderr.write(res.stdout + res.stderr)
            raise RuntimeError(f"gcc failed for {src}")
    return C_HARNESS_BIN


if __name__ == "__main__":
    p = build(force="--force" in sys.argv)
    build_c_harness()
    print(p)
