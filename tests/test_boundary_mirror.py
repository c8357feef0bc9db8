"""The host layer is written against an API-compatible mirror of mllm's core (mllm_amd/csrc/host/mllm_core.hpp).  Where the
reference checkout is mounted this test reads the reference's own headers AS TEXT and compares what the boundary depends
on: the virtual interface of Allocator / Backend / BaseOp / BaseOpFactory / LinearOp (names, parameter types, constness),
the option struct and enum values the Linear op is created with, the numeric ids of the op / device slots, and the plugin
descriptor's field list.  A drift in the mirror then fails here instead of in a maintainer's build.  Skipped where the
reference is absent (the GPU box)."""
import os
import re

import pytest

REF = "/root/reference"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
MIRROR = os.path.join(ROOT, "mllm_amd", "csrc", "host", "mllm_core.hpp")

pytestmark = pytest.mark.skipif(not os.path.isdir(os.path.join(REF, "mllm")), reason="reference checkout not mounted")


def _strip_comments(txt):
    txt = re.sub(r"/\*.*?\*/", " ", txt, flags=re.S)
    return re.sub(r"//[^\n]*", " ", txt)


def _body(txt, kind, name):
    """text between the braces of `class|struct name ... { ... };` (first definition, not a forward declaration)"""
    for m in re.finditer(r"\b%s\s+%s\b[^;{]*\{" % (kind, re.escape(name)), txt):
        depth, i = 1, m.end()
        while depth and i < len(txt):
            depth += {"{": 1, "}": -1}.get(txt[i], 0)
            i += 1
        return txt[m.end():i - 1]
    raise AssertionError("%s %s not found" % (kind, name))


def _statements(body):
    """top-level statements of a class body: nested braces (inline bodies) removed, split at ';'"""
    out, depth, cur = [], 0, []
    for ch in body:
        if ch == "{":
            depth += 1
            if depth == 1:
                cur.append(" {} ")
            continue
        if ch == "}":
            depth -= 1
            if depth == 0:  # an inline body ends the statement like a ';' does
                out.append("".join(cur))
                cur = []
            continue
        if depth:
            continue
        if ch == ";":
            out.append("".join(cur))
            cur = []
        else:
            cur.append(ch)
    return [" ".join(s.split()) for s in out if s.strip()]


def _param_type(p):
    p = " ".join(p.split())
    p = re.sub(r"\s*=.*$", "", p)  # default argument
    m = re.match(r"^(.*[\s&*>])([A-Za-z_]\w*)$", p)
    if m and m.group(1).strip() not in ("const", "unsigned", "signed", "struct"):
        p = m.group(1)
    return re.sub(r"\s*([&*<>,])\s*", r"\1", p.strip())


def _virtuals(body, include_overrides=False):
    """{method name: set of (return type, (parameter types), const?)} for the virtual (or overriding) member functions"""
    res = {}
    for st in _statements(body):
        st = re.sub(r"\[\[[^\]]*\]\]", " ", st)
        st = re.sub(r"^(public|protected|private)\s*:\s*", "", st.strip())
        is_virtual = re.search(r"\bvirtual\b", st) is not None
        is_override = re.search(r"\boverride\b", st) is not None
        if not (is_virtual or (include_overrides and is_override)) or "~" in st:
            continue
        st = re.sub(r"\b(virtual|inline|explicit)\b", " ", st)
        m = re.match(r"^\s*(.*?)\s*\b([A-Za-z_]\w*)\s*\((.*)\)\s*(const)?\s*(override|final)?\s*(=\s*0)?\s*(\{\})?\s*$", st)
        assert m, "cannot parse member function: %r" % st
        ret, name, params, const = m.group(1), m.group(2), m.group(3), bool(m.group(4))
        ptypes = tuple(_param_type(p) for p in _split_params(params)) if params.strip() else ()
        res.setdefault(name, set()).add((re.sub(r"\s*([&*<>,])\s*", r"\1", " ".join(ret.split())), ptypes, const))
    return res


def _split_params(s):
    out, depth, cur = [], 0, []
    for ch in s:
        depth += {"<": 1, "(": 1, ">": -1, ")": -1}.get(ch, 0)
        if ch == "," and depth == 0:
            out.append("".join(cur))
            cur = []
        else:
            cur.append(ch)
    out.append("".join(cur))
    return out


def _read(path):
    return _strip_comments(open(path).read())


def _enum(txt, name):
    """{enumerator: value} of `enum [class] name [: type] { ... }` with C++ implicit numbering and references to earlier names"""
    m = re.search(r"\benum\s+(?:class\s+)?%s\b[^{;]*\{(.*?)\}" % re.escape(name), txt, flags=re.S)
    assert m, name
    vals, nxt = {}, 0
    for item in m.group(1).split(","):
        item = item.strip()
        if not item:
            continue
        if "=" in item:
            k, expr = (x.strip() for x in item.split("=", 1))
            expr = re.sub(r"[A-Za-z_]\w*", lambda mm: str(vals[mm.group(0)]) if mm.group(0) in vals else mm.group(0), expr)
            nxt = int(eval(expr, {"__builtins__": {}}))  # integer literals and + only, after substitution
        else:
            k = item
        vals[k] = nxt
        nxt += 1
    return vals


MIR = _read(MIRROR)


@pytest.mark.parametrize("ref_file,kind,name", [
    ("mllm/backends/base/Allocator.hpp", "class", "Allocator"),
    ("mllm/backends/base/Backend.hpp", "class", "Backend"),
    ("mllm/core/BaseOp.hpp", "class", "BaseOp"),
    ("mllm/core/BaseOp.hpp", "struct", "BaseOpFactory"),
    ("mllm/core/BaseOp.hpp", "class", "TypedOpFactory"),
])
def test_virtual_interface_matches_the_reference(ref_file, kind, name):
    ref = _virtuals(_body(_read(os.path.join(REF, ref_file)), kind, name))
    mir = _virtuals(_body(MIR, kind, name))
    assert ref, "no virtual functions found in %s" % ref_file
    assert set(ref) == set(mir), (sorted(ref), sorted(mir))
    for fn in ref:
        assert ref[fn] == mir[fn], (fn, ref[fn], mir[fn])


def test_linear_op_overrides_and_options_match_the_reference():
    rtxt = _read(os.path.join(REF, "mllm/core/aops/LinearOp.hpp"))
    ref = _virtuals(_body(rtxt, "class", "LinearOp"), include_overrides=True)
    mir = _virtuals(_body(MIR, "class", "LinearOp"), include_overrides=True)
    # the mirror leaves trace() to the base class (IR tracing is not part of this backend); everything it overrides must
    # have the reference's signature, and it must override what the dispatcher calls
    assert set(mir) <= set(ref) and {"load", "forward", "reshape", "setup", "getParams"} <= set(mir)
    for fn in mir:
        assert mir[fn] == ref[fn], (fn, ref[fn], mir[fn])
    # option struct: the reference's fields, in order, with the same types (the QNN-only field is not mirrored)
    def fields(body):
        out = []
        for st in _statements(body):
            m = re.match(r"^([\w:<>]+)\s+(\w+)(\s*=.*)?$", st)
            if m:
                out.append((m.group(1), m.group(2)))
        return out
    rf = [f for f in fields(_body(rtxt, "struct", "LinearOpOptions")) if f[1] != "qnn_impl_type"]
    mf = fields(_body(MIR, "struct", "LinearOpOptions"))
    assert rf == mf, (rf, mf)
    # enumerators the mirror declares carry the reference's values (the impl type travels through the options by value)
    re_, me = _enum(rtxt, "LinearImplTypes"), _enum(MIR, "LinearImplTypes")
    for k, v in me.items():
        if k != "kLinearImplTypes_End":
            assert re_[k] == v, (k, re_[k], v)


def test_op_and_device_ids_match_the_reference():
    ro, mo = _enum(_read(os.path.join(REF, "mllm/core/OpTypes.hpp")), "OpTypes"), _enum(MIR, "OpTypes")
    for k, v in mo.items():
        assert ro[k] == v, (k, ro[k], v)
    rd, md = _enum(_read(os.path.join(REF, "mllm/core/DeviceTypes.hpp")), "DeviceTypes"), _enum(MIR, "DeviceTypes")
    for k, v in md.items():
        if k not in ("kHIP", "kDeviceTypes_End"):  # kHIP is this backend's own id in the range reserved for plug-in devices
            assert rd[k] == v, (k, rd[k], v)
    assert md["kHIP"] > rd["kDynamicDeviceType_Start"]


def test_plugin_descriptor_fields_match_the_reference():
    def desc(txt):
        body = _body(txt, "struct", "PluginOpPackageDescriptor")
        out = []
        for st in _statements(body):
            m = re.match(r"^([\w:]+)\s+(\w+)((?:\s*\[[^\]]+\])*)(\s*=.*)?$", st)
            assert m, st
            out.append((m.group(1), m.group(2), re.sub(r"\s", "", m.group(3))))
        return out
    rtxt = _read(os.path.join(REF, "mllm/backends/base/PluginInterface.hpp"))
    assert desc(rtxt) == desc(MIR)
    for macro in ("MLLM_PLUGIN_OP_PACKAGE_DESCRIPTOR_VERSION", "MLLM_PLUGIN_OP_PACKAGE_NAME_LEN", "MLLM_PLUGIN_OP_PACKAGE_DESCRIPTOR_LEN"):
        r = re.search(r"#define\s+%s\s+(\d+)" % macro, rtxt)
        m = re.search(r"#define\s+%s\s+(\d+)" % macro, MIR)
        assert r and m and r.group(1) == m.group(1), macro
    # both pack the struct to 4 bytes
    assert re.search(r"#pragma\s+pack\(push,\s*4\)\s*struct\s+PluginOpPackageDescriptor", rtxt)
    assert re.search(r"#pragma\s+pack\(push,\s*4\)\s*struct\s+PluginOpPackageDescriptor", MIR)
