"""Regenerates op_table_op-mem-{cuda,ompsimd}.json from the reference's generated op lists
(docs/executor/op-mem-*/list.md, the output of TfFactory::print_markdown).  The lists are data the
reference holds; this script only re-tabulates them.  Run where the reference checkout is mounted:

    python tests/golden/make_op_tables.py [/root/reference]
"""
import json
import os
import sys


def parse(path):
    rows, tftype = [], None
    for line in open(path, encoding="utf-8"):
        line = line.rstrip("\n")
        if line.startswith("### "):
            tftype = line[4:].strip()
            continue
        if not line.startswith("|") or tftype is None:
            continue
        # cells are separated by " | "; a bare "|" inside a cell is a precision union (float64|float32)
        cells = [c.strip() for c in line.strip().strip("|").split(" | ")]
        if len(cells) != 4 or cells[0] in ("Operation", "") or set(cells[0]) <= set("-"):
            continue
        rows.append({"tftype": tftype, "name": cells[0], "author": cells[1], "formula": cells[2], "ir": cells[3]})
    return rows


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    here = os.path.dirname(os.path.abspath(__file__))
    for executor in ("op-mem-cuda", "op-mem-ompsimd"):
        source = f"docs/executor/{executor}/list.md"
        out = {"source": source, "rows": parse(os.path.join(ref, source))}
        with open(os.path.join(here, f"op_table_{executor}.json"), "w", encoding="utf-8") as f:
            json.dump(out, f, indent=1, ensure_ascii=False)
            f.write("\n")
        print(executor, len(out["rows"]), "rows")


if __name__ == "__main__":
    main()
