#!/usr/bin/env python3
"""Extract the region tuner's polygon data into a flat numeric table.

The region tuner of aws-ofi-nccl (src/tuner/nccl_ofi_regions.cpp:295-1882)
defines, per platform, per communicator shape (ranks == 8*nodes, 2*nodes or
nodes) and per collective, an ordered list of polygons in (bytes, ranks)
space.  Some vertices are "extended" points: the intersection of the line
through two anchor points with the bounding box (TUNER_MAX_SIZE,
TUNER_MAX_RANKS); the reference computes those at init time in log2 space
(nccl_ofi_regions.cpp:254-289).

This script reads that source file *as text* and writes the same numbers in
this project's own flat layout (region_tables.inc): four arrays (sets,
polygons, vertices, extension anchors) that both the HIP tuner kernels and
the CPU oracle index.  Only numbers are carried over; the extension arithmetic
is re-done by the consumers of the table.

usage: gen_region_tables.py <path-to-nccl_ofi_regions.cpp> [out.inc]
       (with no out path the table is written to stdout)
"""
import re
import sys

PLATFORM_OF_FUNC = {
    "region_init_internal_p5_p5e": 0,
    "region_init_internal_p5en": 1,
    "region_init_internal_p6": 2,
    "region_init_internal_p6_b300": 3,
}
COLL = {"ncclFuncBroadcast": 0, "ncclFuncReduce": 1, "ncclFuncAllGather": 2,
        "ncclFuncReduceScatter": 3, "ncclFuncAllReduce": 4}
ALGO = {"NCCL_ALGO_TREE": 0, "NCCL_ALGO_RING": 1, "NCCL_ALGO_COLLNET_DIRECT": 2,
        "NCCL_ALGO_COLLNET_CHAIN": 3, "NCCL_ALGO_NVLS": 4, "NCCL_ALGO_NVLS_TREE": 5,
        "NCCL_ALGO_PAT": 6}
PROTO = {"NCCL_PROTO_LL": 0, "NCCL_PROTO_LL128": 1, "NCCL_PROTO_SIMPLE": 2}
MAX_SIZE = 100.0 * 1024 * 1024 * 1024
MAX_RANKS = 1024.0 * 1024


def strip_comments(text):
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    return re.sub(r"//[^\n]*", " ", text)


def number(tok):
    """Evaluate a numeric constant expression (digits, '.', '*', 'e', ULL suffixes)."""
    t = tok.strip()
    t = t.replace("TUNER_MAX_SIZE", repr(MAX_SIZE)).replace("TUNER_MAX_RANKS", repr(MAX_RANKS))
    t = re.sub(r"\(double\)", "", t)
    t = re.sub(r"(?<=\d)(ULL|UL|LL|L|U)\b", "", t)
    if not re.fullmatch(r"[0-9eE+\-.* ()]+", t):
        raise ValueError("not a numeric constant: %r" % tok)
    return float(eval(t, {"__builtins__": {}}))  # arithmetic on literals only


def split_top(s):
    """Split s on commas that are not nested inside braces or parentheses."""
    out, depth, cur = [], 0, []
    for ch in s:
        if ch in "{(":
            depth += 1
        elif ch in "})":
            depth -= 1
        if ch == "," and depth == 0:
            out.append("".join(cur).strip())
            cur = []
        else:
            cur.append(ch)
    last = "".join(cur).strip()
    if last:
        out.append(last)
    return out


def matching(s, start):
    """Index of the brace that closes the one at s[start]."""
    depth = 0
    for i in range(start, len(s)):
        if s[i] == "{":
            depth += 1
        elif s[i] == "}":
            depth -= 1
            if depth == 0:
                return i
    raise ValueError("unbalanced braces")


def inner(s):
    s = s.strip()
    assert s[0] == "{" and s[-1] == "}", s
    return s[1:-1]


def parse_point(tok):
    m = re.fullmatch(r"\(\s*nccl_ofi_tuner_point_t\s*\)\s*(\{.*\})", tok.strip(), flags=re.S)
    if not m:
        raise ValueError("not a point literal: %r" % tok)
    xy = split_top(inner(m.group(1)))
    assert len(xy) == 2, tok
    return number(xy[0]), number(xy[1])


def parse_coord(tok, ext_names):
    """-> (kind, value): kind 0 literal, 1+2*e ext e's x, 2+2*e ext e's y."""
    tok = tok.strip()
    m = re.fullmatch(r"(\w+)\.(x|y)", tok)
    if m and m.group(1) in ext_names:
        e = ext_names.index(m.group(1))
        return (1 + 2 * e if m.group(2) == "x" else 2 + 2 * e), 0.0
    return 0, number(tok)


def parse_chunk(chunk):
    """One `collType = ...; ... set_regions(...)` block -> (coll, exts, regions)."""
    coll = COLL[re.match(r"\s*(\w+)\s*;", chunk).group(1)]
    exts, ext_names = [], []
    for m in re.finditer(r"nccl_ofi_tuner_point_t\s+(\w+)\s*=\s*extend_region\s*\(", chunk):
        # arguments run to the matching ')'
        i, depth = m.end(), 1
        while depth:
            depth += {"(": 1, ")": -1}.get(chunk[i], 0)
            i += 1
        args = split_top(chunk[m.end():i - 1])
        assert len(args) == 3, args
        a, b, z = (parse_point(t) for t in args)
        assert z == (MAX_SIZE, MAX_RANKS), z
        ext_names.append(m.group(1))
        exts.append((a, b))
    m = re.search(r"regions\s*\[\s*\]\s*=\s*\{", chunk)
    start = m.end() - 1
    body = inner(chunk[start:matching(chunk, start) + 1])
    regions = []
    for ent in split_top(body):
        fields = {}
        for f in split_top(inner(ent)):
            k, v = f.split("=", 1)
            fields[k.strip()] = v.strip()
        verts = []
        for v in split_top(inner(fields[".vertices"])):
            if v in ext_names:
                e = ext_names.index(v)
                verts.append((1 + 2 * e, 0.0, 2 + 2 * e, 0.0))
            else:
                xy = split_top(inner(v))
                assert len(xy) == 2, v
                xk, xv = parse_coord(xy[0], ext_names)
                yk, yv = parse_coord(xy[1], ext_names)
                verts.append((xk, xv, yk, yv))
        nv = int(number(fields[".num_vertices"]))
        assert nv == len(verts), (nv, len(verts), ent)
        regions.append((ALGO[fields[".algorithm"]], PROTO[fields[".protocol"]], verts))
    return coll, exts, regions


def parse(path):
    text = strip_comments(open(path).read())
    sets = []
    funcs = list(re.finditer(r"static\s+ncclResult_t\s+(region_init_internal_\w+)\s*\(", text))
    for n, fm in enumerate(funcs):
        name = fm.group(1)
        if name not in PLATFORM_OF_FUNC:
            continue
        end = funcs[n + 1].start() if n + 1 < len(funcs) else len(text)
        # the last platform function is followed by non-table code; cut at its 'exit:' label
        body = text[fm.end():end]
        body = body[:body.index("exit:")]
        # split by communicator shape
        shape_iter = list(re.finditer(r"if\s*\(\s*nRanks\s*==\s*(?:(\d+)\s*\*\s*)?nNodes\s*\)", body))
        for k, sm in enumerate(shape_iter):
            ppn = int(sm.group(1)) if sm.group(1) else 1
            s_end = shape_iter[k + 1].start() if k + 1 < len(shape_iter) else len(body)
            sbody = body[sm.end():s_end]
            parts = re.split(r"collType\s*=", sbody)[1:]
            for chunk in parts:
                coll, exts, regions = parse_chunk(chunk)
                sets.append((PLATFORM_OF_FUNC[name], ppn, coll, exts, regions))
    sets.sort(key=lambda s: (s[0], -s[1], s[2]))
    return sets


def fmt(v):
    r = repr(float(v))
    return r if ("e" in r or "." in r or "inf" in r) else r + ".0"


def emit(sets, out):
    w = out.write
    w("/* Region tuner polygon data in flat form.  Generated by gen_region_tables.py from the\n")
    w(" * vertex lists in aws-ofi-nccl src/tuner/nccl_ofi_regions.cpp:295-1882; do not edit.\n")
    w(" * Coordinates are in linear (bytes, ranks) space.  kind 0 = literal value,\n")
    w(" * kind 1+2e / 2+2e = x / y of extension point e of the same set. */\n")
    ext_rows, vtx_rows, poly_rows, set_rows = [], [], [], []
    for plat, ppn, coll, exts, regions in sets:
        set_rows.append((plat, ppn, coll, len(poly_rows), len(regions), len(ext_rows), len(exts)))
        for (a, b) in exts:
            ext_rows.append((a[0], a[1], b[0], b[1]))
        for algo, proto, verts in regions:
            poly_rows.append((algo, proto, len(vtx_rows), len(verts)))
            vtx_rows.extend(verts)
    w("#define OFI_REGION_NUM_SETS %d\n#define OFI_REGION_NUM_POLYS %d\n" % (len(set_rows), len(poly_rows)))
    w("#define OFI_REGION_NUM_VERTS %d\n#define OFI_REGION_NUM_EXTS %d\n" % (len(vtx_rows), len(ext_rows)))
    w("/* {platform, ranks_per_node, collective, first_poly, num_polys, first_ext, num_exts} */\n")
    w("static const int ofi_region_sets[OFI_REGION_NUM_SETS][7] = {\n")
    for r in set_rows:
        w("\t{%s},\n" % ", ".join(str(x) for x in r))
    w("};\n/* {algorithm, protocol, first_vertex, num_vertices} */\n")
    w("static const int ofi_region_polys[OFI_REGION_NUM_POLYS][4] = {\n")
    for r in poly_rows:
        w("\t{%s},\n" % ", ".join(str(x) for x in r))
    w("};\n/* {x_kind, y_kind} and {x, y} per vertex */\n")
    w("static const int ofi_region_vert_kind[OFI_REGION_NUM_VERTS][2] = {\n")
    for i in range(0, len(vtx_rows), 8):
        w("\t" + " ".join("{%d,%d}," % (v[0], v[2]) for v in vtx_rows[i:i + 8]) + "\n")
    w("};\nstatic const double ofi_region_vert_xy[OFI_REGION_NUM_VERTS][2] = {\n")
    for i in range(0, len(vtx_rows), 3):
        w("\t" + " ".join("{%s, %s}," % (fmt(v[1]), fmt(v[3])) for v in vtx_rows[i:i + 3]) + "\n")
    w("};\n/* extension anchors {ax, ay, bx, by}; the third point is always (max size, max ranks) */\n")
    w("static const double ofi_region_exts[OFI_REGION_NUM_EXTS][4] = {\n")
    for r in ext_rows:
        w("\t{%s},\n" % ", ".join(fmt(x) for x in r))
    w("};\n")


def main(argv):
    if len(argv) < 2:
        sys.stderr.write(__doc__)
        return 2
    sets = parse(argv[1])
    if len(argv) > 2:
        with open(argv[2], "w") as f:
            emit(sets, f)
    else:
        emit(sets, sys.stdout)
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
