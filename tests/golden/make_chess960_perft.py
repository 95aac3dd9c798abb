"""Extracts the Chess960 perft known answers held by the reference's own test
(src/chess/board_test.cc, table kChess960Positions; commented-out rows are
skipped) into chess960_perft.json.  Data only: FEN strings and node counts.
Run once in the build container:  python tests/golden/make_chess960_perft.py
"""
import json, os, re, sys

src = sys.argv[1] if len(sys.argv) > 1 else "/root/reference/src/chess/board_test.cc"
text = open(src).read()
start = text.index("kChess960Positions[] = {")
end = text.index("};", start)
body = "\n".join(l for l in text[start:end].splitlines() if not l.strip().startswith("//"))
rows = re.findall(r'\{\s*"([^"]+)"\s*,\s*\{([^}]*)\}\s*\}', body)
out = [{"fen": fen, "perft": [int(x) for x in nums.split(",")]} for fen, nums in rows]
dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "chess960_perft.json")
json.dump(out, open(dst, "w"), indent=0)
print(len(out), "rows ->", dst)
