"""Extracts (message, field name) -> field number of proto/net.proto from the reference's text into
net_proto_fields.json. Run in the build container: python tests/golden/make_net_proto_fields.py"""
import json
import os
import re
import sys

SRC = sys.argv[1] if len(sys.argv) > 1 else "/root/reference/proto/net.proto"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "net_proto_fields.json")


def main():
    text = re.sub(r"//[^\n]*", "", open(SRC).read())
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    tokens = re.findall(r"[A-Za-z_][A-Za-z0-9_.]*|\d+|[{};=\[\]]", text)
    fields, stack, i = {}, [], 0
    while i < len(tokens):
        t = tokens[i]
        if t in ("message", "enum") and tokens[i + 2] == "{":
            stack.append((t, tokens[i + 1]))
            i += 3
            continue
        if t == "}":
            stack.pop()
            i += 1
            continue
        if stack and stack[-1][0] == "message" and t in ("optional", "repeated", "required"):
            # <label> <type> <name> = <number> [options] ;
            name, number = tokens[i + 2], int(tokens[i + 4])
            fields.setdefault(stack[-1][1], {})[name] = {"number": number, "type": tokens[i + 1], "label": t}
            while tokens[i] != ";":
                i += 1
        i += 1
    json.dump(fields, open(OUT, "w"), indent=1, sort_keys=True)
    print(OUT, sum(len(v) for v in fields.values()), "fields")


if __name__ == "__main__":
    main()
