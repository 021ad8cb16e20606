"""Static checks of the Zig side (zig/hip_device.zig, zig/opspec_additions.zig, zig/enabled_devices.patch) that need no
Zig toolchain: every `c.zg_hip_*` call passes arguments of the KIND the header declares (pointer / integer / float,
and no const slice where the C side writes), every `p.<field>` an op method reads exists in the parameter struct of that
name (the reference's src/device/opspec.zig or the additions file), with the type the use implies, and the patch applies
to the reference's files.  The binding has never been compiled; these checks are what can be verified without a
compiler (the reference's own device-parameterised tests, tests/src/main.zig:14-27, are what will exercise it)."""
from __future__ import annotations

import re
import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
VENEER = ROOT / "zig" / "hip_device.zig"
ADDITIONS = ROOT / "zig" / "opspec_additions.zig"
PATCH = ROOT / "zig" / "enabled_devices.patch"
REF = Path("/root/reference")


# ---------------------------------------------------------------------------------------------------------------
# the header: parameter kinds
# ---------------------------------------------------------------------------------------------------------------
def header_kinds():
    """{name: [(param name, kind, pointee-is-const)]}; kind is 'ptr', 'int' or 'float'."""
    text = (ROOT / "include" / "zg_hip.h").read_text()
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    out = {}
    for m in re.finditer(r"(?m)^[ \t]*[A-Za-z_][\w \t\*]*?\b(zg_hip_\w+)\s*\(([^;{}]*?)\)\s*;", text):
        name, params = m.group(1), m.group(2).strip()
        plist = []
        if params and params != "void":
            for p in params.split(","):
                pm = re.match(r"(.*?)(\w+)$", p.strip())
                decl, pname = pm.group(1).strip(), pm.group(2)
                if "*" in decl:
                    # `const float *x`: the pointee is const; `float *const *params`: the outer pointee (a pointer) is const
                    pointee = decl[: decl.rindex("*")].strip()
                    plist.append((pname, "ptr", pointee.endswith("const") or (pointee.startswith("const") and "*" not in pointee)))
                elif decl in ("float", "double"):
                    plist.append((pname, "float", False))
                else:
                    assert decl in ("int", "size_t", "uint64_t", "uint8_t", "int64_t"), (name, decl)
                    plist.append((pname, "int", False))
        out[name] = plist
    return out


# ---------------------------------------------------------------------------------------------------------------
# opspec structs: {op name: {field: zig type}}
# ---------------------------------------------------------------------------------------------------------------
def opspec_structs(text):
    text = re.sub(r"//[^\n]*", "", text)
    out = {}
    for m in re.finditer(r"pub fn (\w+)\(T: type\) type \{\s*return struct \{(.*?)\n    \};", text, flags=re.S):
        fields = {}
        for fm in re.finditer(r"(?m)^\s*(\w+):\s*([^,=\n]+?)(?:\s*=\s*[^,\n]+)?,\s*$", m.group(2)):
            fields[fm.group(1)] = fm.group(2).strip()
        out[m.group(1)] = fields
    return out


def all_structs():
    structs = opspec_structs(ADDITIONS.read_text())
    ref = REF / "src" / "device" / "opspec.zig"
    have_ref = ref.exists()
    if have_ref:
        for k, v in opspec_structs(ref.read_text()).items():
            assert k not in structs, f"{k} is declared by the reference already; the additions must not repeat it"
            structs[k] = v
    return structs, have_ref


def field_kind(ztype):
    """What a field of this Zig type is when passed on: ('slice', const) / ('optslice', const) / 'float' / 'int' / 'bool' /
    ('ptr', const)."""
    t = ztype.replace(" ", "")
    if t.startswith("?[]"):
        return ("optslice", t.startswith("?[]const"))
    if t.startswith("[]"):
        return ("slice", t.startswith("[]const"))
    if t.startswith("*"):
        return ("ptr", t.startswith("*const"))
    if t in ("T", "f32", "f64"):
        return "float"
    if t in ("usize", "u64", "u32", "i32", "c_int"):
        return "int"
    if t == "bool":
        return "bool"
    return "other"


# ---------------------------------------------------------------------------------------------------------------
# the veneer: op methods and the calls in them
# ---------------------------------------------------------------------------------------------------------------
def split_args(body):
    args, depth, cur = [], 0, ""
    for ch in body:
        if ch in "([{":
            depth += 1
        elif ch in ")]}":
            depth -= 1
        if ch == "," and depth == 0:
            args.append(cur.strip())
            cur = ""
        else:
            cur += ch
    if cur.strip():
        args.append(cur.strip())
    return args


def veneer_functions():
    """[(fn name, opspec struct name or None, body text, {parameter: type})] for every function of the binding."""
    text = re.sub(r"//[^\n]*", "", VENEER.read_text())
    out = []
    for m in re.finditer(r"(?m)^(?:    )?(?:pub )?fn (\w+)\(", text):
        depth, i = 1, m.end()
        while depth:                      # the parameter list, parentheses balanced (`p: opspec.add(T)`)
            depth += {"(": 1, ")": -1}.get(text[i], 0)
            i += 1
        params_text = text[m.end(): i - 1]
        j = text.index("{", i)
        if "\n" in text[i:j] or ";" in text[i:j]:
            continue                      # a prototype or a function type, not a definition
        depth, k = 1, j + 1
        while depth:
            depth += {"{": 1, "}": -1}.get(text[k], 0)
            k += 1
        params = {}
        for part in split_args(params_text):
            if ":" in part:
                n, t = part.split(":", 1)
                params[n.strip().replace("comptime ", "")] = t.strip()
        spec = re.fullmatch(r"opspec\.(\w+)\(T\)", params.get("p", ""))
        out.append((m.group(1), spec.group(1) if spec else None, text[j + 1: k - 1], params))
    return out


def calls_in(body):
    for m in re.finditer(r"\bc\.(zg_hip_\w+)\s*\(", body):
        depth, i = 1, m.end()
        while depth:
            depth += {"(": 1, ")": -1}.get(body[i], 0)
            i += 1
        yield m.group(1), split_args(body[m.end(): i - 1])


def local_types(body):
    """{name: zig type} of the typed locals (`const bias: ?[*]const T = ...`, `var status: c_int = 0`)."""
    return {m.group(1): m.group(2).strip() for m in re.finditer(r"\b(?:const|var) (\w+): ([^=;]+?)\s*=", body)}


def classify(arg, fields, locals_, fn_params):
    """-> (kind, const) with kind in ptr / int / float / unknown; raises AssertionError on a use that cannot compile."""
    a = arg.strip()
    m = re.fullmatch(r"@ptrCast\((.*)\)", a)
    cast = bool(m)
    if m:
        a = m.group(1).strip()
    m = re.fullmatch(r"@constCast\((.*)\)", a)
    if m:
        inner = classify(m.group(1), fields, locals_, fn_params)
        return ("ptr", False) if inner[0] == "ptr" else inner
    if a in ("self.ctx", "ctx", "device.ctx"):
        return ("ptr", False)
    if a == "null":
        return ("ptr", True)
    m = re.fullmatch(r"p\.(\w+)\.ptr", a)
    if m:
        assert m.group(1) in fields, f"p.{m.group(1)}: no such field"
        k = field_kind(fields[m.group(1)])
        assert isinstance(k, tuple) and k[0] == "slice", f"p.{m.group(1)}.ptr on a field of type {fields[m.group(1)]}"
        return ("ptr", k[1])
    m = re.fullmatch(r"p\.(\w+)\.len", a)
    if m:
        assert m.group(1) in fields, f"p.{m.group(1)}: no such field"
        k = field_kind(fields[m.group(1)])
        assert isinstance(k, tuple) and k[0] == "slice", f"p.{m.group(1)}.len on a field of type {fields[m.group(1)]}"
        return ("int", False)
    m = re.fullmatch(r"p\.plan\.plan", a)
    if m:
        assert "plan" in fields
        return ("ptr", True)
    m = re.fullmatch(r"@intFromBool\(p\.(\w+)\)", a)
    if m:
        assert m.group(1) in fields, f"p.{m.group(1)}: no such field"
        assert field_kind(fields[m.group(1)]) == "bool", f"@intFromBool of p.{m.group(1)}: {fields[m.group(1)]}"
        return ("int", False)
    if re.fullmatch(r"@intFromBool\(.*\)", a) or re.fullmatch(r"@intCast\(.*\)", a):
        return ("int", False)
    m = re.fullmatch(r"p\.(\w+)", a)
    if m:
        assert m.group(1) in fields, f"p.{m.group(1)}: no such field"
        k = field_kind(fields[m.group(1)])
        if isinstance(k, tuple) and k[0] == "ptr":      # a single-item pointer field (axpy's alpha: *const T)
            return k
        assert k in ("float", "int"), f"p.{m.group(1)} ({fields[m.group(1)]}) passed as it is: a slice needs .ptr/.len, a bool @intFromBool"
        return (k, False)
    m = re.fullmatch(r"&(\w+)", a)
    if m:
        return ("ptr", False)
    if re.fullmatch(r"\w+", a):
        t = locals_.get(a) or fn_params.get(a)
        if t:
            t = t.replace(" ", "")
            if t.startswith("?[*]") or t.startswith("[*]") or t.startswith("?*") or t.startswith("*"):
                return ("ptr", "const" in t.split("]")[-1][:6] or t.lstrip("?").startswith("*const") or "]const" in t)
            if t in ("c_int", "usize", "u64", "u32", "u8"):
                return ("int", False)
            if t == "f32":
                return ("float", False)
            if t == "T":    # a generic memory routine (mem_fill switches on T): the element type decides
                return ("unknown", None)
            if t.startswith("[]"):
                raise AssertionError(f"slice `{a}` passed without .ptr / .len")
    m = re.fullmatch(r"(\w+)\.ptr", a)
    if m:
        t = (locals_.get(m.group(1)) or fn_params.get(m.group(1)) or "").replace(" ", "")
        if t.startswith("[]"):
            return ("ptr", t.startswith("[]const"))
        return ("ptr", None)
    m = re.fullmatch(r"(\w+)\.len(\s*\*.*)?", a)
    if m:
        return ("int", False)
    if re.fullmatch(r"[\w.]+\s*\*\s*@sizeOf\(\w+\)", a) or re.fullmatch(r"\d+", a):
        return ("int", False)
    if re.fullmatch(r"if \(.*\) .* else .*", a):
        return ("unknown", None)
    return ("unknown", None)


def test_every_call_passes_the_kinds_the_header_declares():
    kinds = header_kinds()
    structs, _ = all_structs()
    n_calls = n_args = n_unknown = 0
    for fn, spec, body, fn_params in veneer_functions():
        fields = structs.get(spec, {}) if spec else {}
        locals_ = local_types(body)
        for name, args in calls_in(body):
            assert name in kinds, f"{fn}: {name} is not declared in zg_hip.h"
            want = kinds[name]
            assert len(args) == len(want), f"{fn}: {name} takes {len(want)} arguments, the call passes {len(args)}"
            n_calls += 1
            for arg, (pname, kind, c_const) in zip(args, want):
                try:
                    got, z_const = classify(arg, fields, locals_, fn_params)
                except AssertionError as e:
                    raise AssertionError(f"{fn}: {name}({pname} = {arg}): {e}") from None
                n_args += 1
                if got == "unknown":
                    n_unknown += 1
                    continue
                assert got == kind, f"{fn}: {name}: parameter `{pname}` is a {kind}, the call passes `{arg}` (a {got})"
                if kind == "ptr" and z_const is True and not c_const and arg.strip() != "null":
                    raise AssertionError(f"{fn}: {name}: `{arg}` is const on the Zig side but `{pname}` is written by the C side")
    assert n_calls >= 110 and n_args >= 600
    assert n_unknown <= 0.05 * n_args, f"{n_unknown} of {n_args} arguments could not be classified"


def test_every_op_method_names_a_parameter_struct_that_exists_and_reads_only_its_fields():
    structs, have_ref = all_structs()
    seen = 0
    for fn, spec, body, _ in veneer_functions():
        if spec is None:
            continue
        seen += 1
        assert spec == fn, f"method {fn} takes opspec.{spec}: DeviceReference.dispatch finds methods by __name__"
        if spec not in structs:
            if not have_ref:
                continue    # a struct of the reference's own opspec.zig, which is not on this machine
            raise AssertionError(f"opspec.{spec} exists neither in the reference's opspec.zig nor in the additions")
        used = set(re.findall(r"\bp\.(\w+)", body))
        missing = used - set(structs[spec])
        assert not missing, f"{fn}: reads p.{sorted(missing)} which opspec.{spec} does not have ({sorted(structs[spec])})"
    assert seen >= 70
    # every struct of the additions file has its method, and carries the reference's two declarations
    add_text = ADDITIONS.read_text()
    methods = {fn for fn, spec, _, _ in veneer_functions() if spec}
    for name in opspec_structs(add_text):
        assert name in methods, f"opspec_additions.{name} has no HipDevice method"
        assert f'pub const __name__ = "{name}";' in add_text
    assert add_text.count("pub const __type__ = T;") == len(opspec_structs(add_text))


def test_the_additions_cover_every_lifted_entry_point():
    """Each entry point that stands for a host loop of the reference has a parameter struct whose array fields match the
    entry point's pointer parameters by name."""
    kinds = header_kinds()
    adds = opspec_structs(ADDITIONS.read_text())
    for name, fields in adds.items():
        cname = "zg_hip_" + name
        assert cname in kinds, name
        for pname, kind, _ in kinds[cname][1:]:
            if kind == "ptr" and pname not in ("status", "plan"):
                assert pname in fields, f"{name}: C parameter `{pname}` has no field"


@pytest.mark.skipif(not REF.exists(), reason="the reference checkout is not present on this machine")
def test_the_patch_applies_to_the_reference_files(tmp_path):
    if shutil.which("patch") is None:
        pytest.skip("no patch tool")
    text = PATCH.read_text()
    files = re.findall(r"(?m)^\+\+\+ b/(\S+)", text)
    assert set(files) >= {"build.zig", "src/device/enabled_devices.zig", "src/device.zig", "src/zigrad.zig", "tests/src/main.zig"}
    for f in files:
        (tmp_path / f).parent.mkdir(parents=True, exist_ok=True)
        shutil.copy(REF / f, tmp_path / f)
    res = subprocess.run(["patch", "-p1", "--batch"], cwd=tmp_path, input=text, capture_output=True, text=True)
    assert res.returncode == 0, res.stdout + res.stderr
    enabled = (tmp_path / "src/device/enabled_devices.zig").read_text()
    assert '.name = "hip"' in enabled and "*HipDevice" in enabled and "build_options.enable_hip" in enabled
    assert "enable_hip" in (tmp_path / "build.zig").read_text()
    assert "hip.reference()" in (tmp_path / "tests/src/main.zig").read_text()
