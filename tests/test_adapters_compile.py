"""The lc0-side adapters (lc0_amd/lc0_adapter/*.cc: the actual drop-in, REGISTER_NETWORK and
BackendManager::Register) are not part of liblc0mi.so; they need lc0's headers. Where the reference tree is
present (the build container) they are syntax- and type-checked against those headers: every override must
match src/neural/network.h:56-126, src/neural/backend.h:75-125 and src/neural/factory.h:111-142 as they are
today. proto/net.pb.h, which lc0's headers include and lc0's build generates, is written here as a
declaration-only header from the text of proto/net.proto (messages, nested enums, accessors in the naming of lc0's
generator); nothing from the reference tree is executed. A syntax check does not link: running the adapters inside
a real lc0 build is not covered."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference"
ADAPTERS = ["network_mi355x.cc", "backend_mi355x.cc"]


SCALARS = {"float": "float", "double": "double", "int32": "std::int32_t", "int64": "std::int64_t",
           "uint32": "std::uint32_t", "uint64": "std::uint64_t", "sint32": "std::int32_t", "sint64": "std::int64_t",
           "fixed32": "std::uint32_t", "fixed64": "std::uint64_t", "sfixed32": "std::int32_t",
           "sfixed64": "std::int64_t", "bool": "bool", "string": "std::string", "bytes": "std::string"}


def _proto_stub_header(proto_text):
    """Declaration-only C++ for the messages of a .proto file: one class per message (nested where the proto nests),
    enums with their enumerators in class scope, has_/get/mutable_/set_/add_/_size accessors per field."""
    import re
    text = re.sub(r"//[^\n]*", "", proto_text)
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    tokens = re.findall(r"[A-Za-z_][A-Za-z0-9_.]*|-?\d+|[{};=\[\]]", text)
    pos = 0

    def parse_block(kind, name):
        nonlocal pos
        node = {"kind": kind, "name": name, "children": [], "fields": [], "values": []}
        while tokens[pos] != "}":
            t = tokens[pos]
            if t in ("message", "enum") and tokens[pos + 2] == "{":
                child_kind, child_name = t, tokens[pos + 1]
                pos += 3
                node["children"].append(parse_block(child_kind, child_name))
            elif kind == "message" and t in ("optional", "repeated", "required"):
                node["fields"].append((t, tokens[pos + 1], tokens[pos + 2]))
                while tokens[pos] != ";":
                    pos += 1
                pos += 1
            elif kind == "enum" and tokens[pos + 1] == "=":
                node["values"].append((t, tokens[pos + 2]))
                while tokens[pos] != ";":
                    pos += 1
                pos += 1
            else:
                pos += 1
        pos += 1
        return node

    top = []
    while pos < len(tokens):
        if tokens[pos] in ("message", "enum") and pos + 2 < len(tokens) and tokens[pos + 2] == "{":
            kind, name = tokens[pos], tokens[pos + 1]
            pos += 3
            top.append(parse_block(kind, name))
        else:
            pos += 1

    def emit(node, indent):
        pad = "  " * indent
        if node["kind"] == "enum":
            vals = ", ".join("%s = %s" % v for v in node["values"])
            return ["%senum %s { %s };" % (pad, node["name"], vals)]
        out = ["%sclass %s : public lczero::ProtoMessage {" % (pad, node["name"]), pad + " public:"]
        for child in node["children"]:
            if child["kind"] == "message":
                out.append("%s  class %s;" % (pad, child["name"]))
        for child in node["children"]:
            out += emit(child, indent + 1)
        for label, typ, name in node["fields"]:
            ctype = SCALARS.get(typ, typ.replace(".", "::"))
            by_value = typ in SCALARS and typ not in ("string", "bytes")
            ret = ctype if by_value else "const %s&" % ctype
            if label == "repeated":
                out += ["%s  int %s_size() const;" % (pad, name), "%s  %s %s(int index) const;" % (pad, ret, name),
                        "%s  const std::vector<%s>& %s() const;" % (pad, ctype, name),
                        "%s  std::vector<%s>* mutable_%s();" % (pad, ctype, name),
                        "%s  %s* add_%s();" % (pad, ctype, name)]
            else:
                out += ["%s  bool has_%s() const;" % (pad, name), "%s  %s %s() const;" % (pad, ret, name),
                        "%s  %s* mutable_%s();" % (pad, ctype, name), "%s  void set_%s(%s value);" % (pad, name, ret)]
        out += ["%s  void Clear() override;" % pad, "%s  std::string OutputAsString() const override;" % pad,
                "%s  std::string OutputAsJson() const override;" % pad, pad + "};"]
        return out

    lines = ["// Declarations only: written by tests/test_adapters_compile.py from the text of proto/net.proto.",
             "#pragma once", "#include <cstdint>", "#include <string>", "#include <vector>",
             '#include "utils/protomessage.h"', "namespace pblczero {"]
    for node in top:
        if node["kind"] == "message":
            lines.append("class %s;" % node["name"])
    for node in top:
        lines += emit(node, 0)
    lines.append("}  // namespace pblczero")
    return "\n".join(lines) + "\n"


@pytest.fixture(scope="module")
def generated_headers(tmp_path_factory):
    if not os.path.isdir(os.path.join(REF, "src")):
        pytest.skip("the reference tree is absent: lc0's headers are needed to compile the adapters")
    out = tmp_path_factory.mktemp("gen")
    os.makedirs(os.path.join(str(out), "proto"))
    header = _proto_stub_header(open(os.path.join(REF, "proto", "net.proto")).read())
    assert "enum InputFormat" in header and "class Net " in header
    open(os.path.join(str(out), "proto", "net.pb.h"), "w").write(header)
    return str(out)


@pytest.mark.parametrize("source", ADAPTERS)
def test_adapter_compiles_against_lc0_headers(source, generated_headers):
    cmd = ["g++", "-std=c++20", "-fsyntax-only", "-Wall", "-Werror=overloaded-virtual", "-Wno-unused",
           "-I" + os.path.join(REF, "src"), "-I" + generated_headers, "-I" + os.path.join(ROOT, "include"),
           os.path.join(ROOT, "lc0_amd", "lc0_adapter", source)]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert res.returncode == 0, res.stdout[-4000:]


def test_adapters_use_only_declared_entry_points():
    """Every lc0mi_* symbol the adapters call is declared in include/lc0mi.h (and so exported by the library,
    which tests/test_cabi_cpu.py checks)."""
    import re
    header = open(os.path.join(ROOT, "include", "lc0mi.h")).read()
    declared = set(re.findall(r"\b(lc0mi_[a-z0-9_]+)\s*\(", header))
    for source in ADAPTERS:
        text = open(os.path.join(ROOT, "lc0_amd", "lc0_adapter", source)).read()
        used = set(re.findall(r"\b(lc0mi_[a-z0-9_]+)\s*\(", text))
        assert used and used <= declared, (source, used - declared)
