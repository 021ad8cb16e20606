"""The shared library loads and exports every entry point include/zg_hip.h declares (no GPU calls)."""
import ctypes

from zigrad_amd._lib import LIB_PATH, Library, parse_header


def test_header_declares_expected_surface():
    protos = parse_header()
    # every DeviceReference op of the hot path has an entry point
    for op in ["add", "sub", "mul", "div", "dot", "matvec", "matmul", "bmm_acc", "outer", "transpose", "axpy", "sum",
               "scale", "nrm2", "clip_nrm2", "pow_fwd", "pow_bwd", "sqrt_fwd", "sqrt_bwd", "rsqrt_fwd", "rsqrt_bwd",
               "exp_fwd", "exp_bwd", "relu_fwd", "relu_bwd", "relu_inplace_bwd", "tanh_fwd", "tanh_bwd",
               "tanh_inplace_bwd", "sigm_fwd", "sigm_bwd", "sigm_inplace_bwd", "max_fwd", "max_bwd", "clamp_fwd",
               "clamp_bwd", "unbroadcast", "broadcast", "sum_along", "max_along", "argmax_along", "scatter_add",
               "scatter_gcn_deg_scaled", "scatter_gcn_deg_scaled_bwd", "index_select_fwd", "index_select_bwd",
               "smce_fwd", "smce_bwd", "smce_label_fwd", "smce_label_bwd", "smooth_l1_fwd", "smooth_l1_bwd", "mse_fwd",
               "mse_bwd", "sgd_step", "adam_step", "mem_fill", "mem_sequence", "mem_take", "mem_random",
               "mem_cache_alloc", "mem_cache_free", "mem_scratch", "memcpy_h2d", "memcpy_d2h", "memcpy_d2d", "sync"]:
        assert "zg_hip_" + op in protos, op
    assert len(protos) >= 90


def test_library_exports_every_declared_symbol():
    assert LIB_PATH.exists(), "build the library first: python -m zigrad_amd.build"
    lib = Library()
    for name in lib.protos:
        assert hasattr(lib.cdll, name), name


def test_argument_errors_are_reported_without_a_gpu():
    lib = Library()
    # a null context is rejected on the host before anything touches a device
    rc = lib.cdll.zg_hip_sync(None)
    assert rc == 1
    assert b"null context" in lib.cdll.zg_hip_last_error()
    n = ctypes.c_int(-1)
    assert lib.cdll.zg_hip_device_count(ctypes.byref(n)) == 0
    assert n.value >= 0


def _zig_calls(text):
    """(name, number of arguments) of every `c.zg_hip_*( ... )` call in Zig source, comments stripped."""
    import re

    text = re.sub(r"//[^\n]*", "", text)
    for m in re.finditer(r"\bc\.(zg_hip_\w+)\s*\(", text):
        depth, args, i, seen = 1, 0, m.end(), False
        while depth:
            ch = text[i]
            if ch in "([{":
                depth += 1
            elif ch in ")]}":
                depth -= 1
            elif ch == "," and depth == 1:
                args += 1
            if depth and not ch.isspace():
                seen = True
            i += 1
        # a trailing comma before the closing parenthesis is Zig's multi-line call style, not another argument
        body = text[m.end(): i - 1].rstrip()
        if body.endswith(","):
            args -= 1
        yield m.group(1), (args + 1 if seen else 0)


def test_zig_veneer_calls_match_the_header():
    """zig/hip_device.zig binds the library through @cImport of include/zg_hip.h: every entry point it calls must be
    declared there with the number of arguments the call passes (no Zig toolchain here to compile it)."""
    from pathlib import Path

    protos = parse_header()
    text = (Path(__file__).resolve().parents[1] / "zig" / "hip_device.zig").read_text()
    calls = list(_zig_calls(text))
    assert len({n for n, _ in calls}) >= 80
    for name, n_args in calls:
        assert name in protos, f"{name} is called by the veneer but not declared in zg_hip.h"
        assert n_args == len(protos[name][1]), f"{name}: veneer passes {n_args} arguments, header declares {len(protos[name][1])}"


def test_zig_veneer_uses_only_what_the_reference_allocators_export():
    """The binding imports src/allocators.zig: every `allocators.<name>` it names must be a `pub` declaration of
    that file, and it must not reach into the allocator objects (no `self.cache.<method>` that the reference's
    CachingAllocator lacks: the binding keeps no allocator object at all)."""
    import re
    from pathlib import Path

    import pytest

    text = (Path(__file__).resolve().parents[1] / "zig" / "hip_device.zig").read_text()
    text = re.sub(r"//[^\n]*", "", text)
    assert not re.search(r"\bself\.cache\b", text), "the binding is meant to go through zg_hip_mem_cache_* only"
    used = set(re.findall(r"\ballocators\.(\w+)", text)) - {"zig"}  # "../allocators.zig" is the import itself
    assert used, "the binding no longer imports src/allocators.zig?"
    ref = Path("/root/reference/src/allocators.zig")
    if not ref.exists():
        pytest.skip("the reference checkout is not present on this machine")
    exported = set(re.findall(r"(?m)^pub (?:const|fn) (\w+)", ref.read_text()))
    assert used <= exported, f"not exported by the reference's src/allocators.zig: {sorted(used - exported)}"
    # the members of the DataHandler contract (src/allocators/block_pool.zig:103-173) are all present
    handler = text[text.index("pub const DataHandler = struct"):]
    handler = handler[:handler.index("\n};")]
    for member in ("min_split_size", "fn map(", "fn unmap(", "fn alloc(", "fn free(", "fn page_size(", "fn reset(", "fn deinit("):
        assert member in handler, member


def test_header_is_plain_c_and_links_from_a_c_program(tmp_path):
    """include/zg_hip.h compiles as C11 with gcc (no C++ in the boundary) and a C program linked against the library
    can call it: device count and the error string, nothing that needs a GPU."""
    import subprocess
    from pathlib import Path

    root = Path(__file__).resolve().parents[1]
    src = tmp_path / "probe.c"
    src.write_text(
        '#include <stdio.h>\n#include "zg_hip.h"\n'
        "int main(void) {\n"
        "    int n = -1;\n"
        "    if (zg_hip_device_count(&n) != 0 || n < 0) return 2;\n"
        "    if (zg_hip_sync(NULL) == 0) return 3; /* a null context must be refused */\n"
        '    printf("%d %s\\n", n, zg_hip_last_error());\n'
        "    return 0;\n}\n")
    exe = tmp_path / "probe"
    cc = ["gcc", "-std=c11", "-Wall", "-Werror", "-pedantic", f"-I{root / 'include'}", str(src), "-o", str(exe),
          f"-L{LIB_PATH.parent}", "-lzg_hip", f"-Wl,-rpath,{LIB_PATH.parent}"]
    built = subprocess.run(cc, capture_output=True, text=True)
    assert built.returncode == 0, built.stderr
    ran = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert ran.returncode == 0, (ran.returncode, ran.stdout, ran.stderr)
    assert "null context" in ran.stdout
