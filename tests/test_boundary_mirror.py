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


# ---- model-file schema ---------------------------------------------------------------------------------------------
# The V1 / V2 reader and writer (mllm_amd/csrc/host/mllm_core.cpp) restate the reference's packed structs; the tests of the
# reader otherwise only see files that this repository's own tests write.  Here the reference's schema headers are read as
# text: magic numbers, version, array lengths, the field lists (type, name, order) and the sizes their static_asserts state.
CORE_CPP = os.path.join(ROOT, "mllm_amd", "csrc", "host", "mllm_core.cpp")
_WIDTH = {"int32_t": 4, "uint32_t": 4, "uint64_t": 8, "size_t": 8, "char": 1}


def _macros(txt):
    return {m.group(1): int(m.group(2), 0) for m in re.finditer(r"#define\s+(\w+)\s+(0x[0-9A-Fa-f]+|\d+)\b", txt)}


def _struct_body(txt, struct):
    """like _body, for `struct [__attribute__((packed))] name { ... }`; also returns the text between `struct` and the name"""
    m = re.search(r"\bstruct\s+((?:__attribute__\s*\(\(\s*packed\s*\)\)\s*)?)%s\s*\{" % re.escape(struct), txt)
    assert m, "struct %s not found" % struct
    depth, i = 1, m.end()
    while depth and i < len(txt):
        depth += {"{": 1, "}": -1}.get(txt[i], 0)
        i += 1
    return txt[m.end():i - 1], m.group(1)


def _fields(txt, struct, macros=None):
    """[(type, name, array length or None)] of a packed struct's data members, in order"""
    out = []
    for st in _statements(_struct_body(txt, struct)[0]):
        m = re.fullmatch(r"(\w+)\s+(\w+(?:\[\w+\])?(?:\s*,\s*\w+(?:\[\w+\])?)*)", st)
        if not m:
            continue  # member functions
        for decl in m.group(2).split(","):  # `int32_t magic_number, version;` declares two members
            d = re.fullmatch(r"\s*(\w+)(?:\[(\w+)\])?\s*", decl)
            n = d.group(2)
            if n is not None:
                n = int(n, 0) if re.fullmatch(r"0x[0-9A-Fa-f]+|\d+", n) else (macros or {})[n]
            out.append((m.group(1), d.group(1), n))
    return out


def _sizeof(fields):
    return sum(_WIDTH[t] * (n or 1) for t, _, n in fields)


def _asserted_sizes(txt):
    return {m.group(1): int(m.group(2)) for m in re.finditer(r"static_assert\(sizeof\((\w+)\)\s*==\s*(\d+)", txt)}


def test_model_file_v2_schema_matches_the_reference_header():
    ref = _strip_comments(open(os.path.join(REF, "mllm/core/schema/ModelFileV2.hpp")).read())
    mine = _strip_comments(open(CORE_CPP).read())
    mac = _macros(ref)
    consts = {m.group(1): int(m.group(2), 0) for m in re.finditer(r"\b(k\w+)\s*=\s*(0x[0-9A-Fa-f]+|\d+)", mine)}
    assert consts["kV2Magic"] == mac["MLLM_MODEL_FILE_V2_MAGIC_NUMBER"] == 0x519A
    assert consts["kV2Version"] == mac["MLLM_MODEL_FILE_V2_VERSION"]
    assert consts["kV2ModelName"] == mac["MLLM_MODEL_FILE_V2_MODEL_NAME_LENGTH"]
    assert consts["kV2ParamName"] == mac["MLLM_MODEL_FILE_V2_PARAMS_NAME_LENGTH"]
    assert consts["kV2ShapeLen"] == mac["MLLM_MODEL_FILE_V2_TENSOR_SHAPE_LENGTH"]
    sizes_ref, sizes_mine = _asserted_sizes(ref), {}
    m = re.search(r"static_assert\(sizeof\(V2Header\)\s*==\s*(\d+)\s*&&\s*sizeof\(V2Param\)\s*==\s*(\d+)", mine)
    assert m, "the mirror states its struct sizes"
    sizes_mine = {"V2Header": int(m.group(1)), "V2Param": int(m.group(2))}
    for theirs, ours in (("ModelFileV2Descriptor", "V2Header"), ("ModelFileV2ParamsDescriptor", "V2Param")):
        fr, fm = _fields(ref, theirs, mac), _fields(mine, ours, consts)
        assert "packed" in _struct_body(ref, theirs)[1] and "packed" in _struct_body(mine, ours)[1]
        # same names in the same order, same widths (size_t in the reference is 8 bytes on every 64-bit target it builds for)
        assert [(n, _WIDTH[t], a) for t, n, a in fr] == [(n, _WIDTH[t], a) for t, n, a in fm], (theirs, fr, fm)
        assert _sizeof(fr) == sizes_ref[theirs] == sizes_mine[ours] == _sizeof(fm)


def test_model_file_v1_schema_matches_the_reference_header():
    ref = _strip_comments(open(os.path.join(REF, "mllm/core/schema/ModelFileV1.hpp")).read())
    mine = _strip_comments(open(CORE_CPP).read())
    assert _macros(ref)["MLLM_MODEL_FILE_V1_MAGIC_NUMBER"] == int(re.search(r"kV1Magic\s*=\s*(\d+)", mine).group(1)) == 20012
    assert "packed" in _struct_body(ref, "ModelFileV1Descriptor")[1] and "packed" in _struct_body(ref, "ModelFileV1ParamsDescriptor")[1]
    head = _fields(ref, "ModelFileV1Descriptor")
    assert [(n, _WIDTH[t]) for t, n, _ in head] == [("magic_number", 4), ("parameter_desc_offset", 8)]
    assert _sizeof(head) == _asserted_sizes(ref)["ModelFileV1Descriptor"] == 12
    # the reader takes the header as 4 + 8 bytes at offsets 0 and 4 and the descriptors from byte 12 on
    assert re.search(r"bytes\(0,\s*4,\s*&magic\)", mine) and re.search(r"bytes\(4,\s*8,\s*&desc_bytes\)", mine)
    assert re.search(r"bytes\(12,\s*desc_bytes", mine)
    # per tensor: name_len, the name, then data_len, offset, dtype with the reference's widths, in the reference's order
    per = _fields(ref, "ModelFileV1ParamsDescriptor")
    assert [(n, _WIDTH[t]) for t, n, _ in per] == [("name_len", 4), ("data_len", 8), ("offset", 8), ("dtype", 4)]
    v1 = mine[mine.index("version == ModelFileVersion::kV1"):]
    v1 = v1[:v1.index("items.push_back")]
    takes = re.findall(r"(\w+)\s*=\s*take<(\w+)>", v1)
    assert [(_WIDTH[t]) for _, t in takes] == [4, 8, 8, 4], takes
    assert [n.split(".")[-1] for n, _ in takes] == ["name_len", "len", "offset", "dtype"]
    # ... and the writer emits the same sequence
    sv = mine[mine.index("void save("):]
    sv = sv[sv.index("version == ModelFileVersion::kV1"):sv.index("} else {")]
    writes = re.findall(r"out\.write\((?:reinterpret_cast<const char\*>\(&(\w+)\)|(\w+)\.data\(\)),\s*(\w+)\)", sv)
    assert [(a or b, n) for a, b, n in writes] == [("kV1Magic", "4"), ("desc_bytes", "8"), ("name_len", "4"), ("name", "name_len"),
                                                    ("len", "8"), ("offset", "8"), ("dtype", "4")], writes
