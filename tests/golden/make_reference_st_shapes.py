"""Collects the shapes the reference's own system tests drive through the V operators, as data.

Reads (as text; nothing of the reference is imported or run) the test cases of
    test/st/algorithm/testcase/alltoallv_testcase.cc      sendCountMatrix + data type(s) per TEST_F
    test/st/algorithm/testcase/alltoallvc_testcase.cc     the same
    test/st/algorithm/testcase/all_gather_v_testcase.cc   counts / displs + data type per TEST_F
    test/st/algorithm/testcase/reduce_scatter_v_testcase.cc, reduce_scatter_v_testcase_a3.cc   counts / displs / type / op
    test/st/algorithm/testcase/broadcast_testcase.cc      rank count, count, type, root per TEST_F
    test/st/algorithm/testcase/scatter_testcase.cc        root, count (per rank), type per TEST_F
(cases whose numbers are written out; the few that build them in loops or helper functions, the 32- and 128-rank
"pairwise" matrices among them, are left out)
and writes tests/golden/reference_st_shapes.json: one entry per test case with its name, the file and line it starts
on, the rank count, the data type names and the numbers; for the cases that only assert the entry point's return code,
that code ("expect") and whether the call was in place.  The reference checks these cases with a simulated world and
a verifier of the data flow, not with values; here tests/test_wide_gpu_reference_st_shapes.py replays the shapes (scaled
down where a count is in the millions) against the oracle.

Usage (in the container that holds /root/reference):  python tests/golden/make_reference_st_shapes.py
"""
import json
import os
import re

REF = "/root/reference/test/st/algorithm/testcase"
HERE = os.path.dirname(os.path.abspath(__file__))


def cases_of(path):
    text = open(path, encoding="utf-8", errors="replace").read()
    for m in re.finditer(r"TEST_F\(\s*\w+\s*,\s*(\w+)\s*\)\s*\{", text):
        start = m.end()
        depth, i = 1, start
        while depth and i < len(text):
            depth += {"{": 1, "}": -1}.get(text[i], 0)
            i += 1
        yield m.group(1), text.count("\n", 0, m.start()) + 1, text[start:i - 1]


def numbers(body, name):
    m = re.search(name + r"\s*=\s*\{(.*?)\}\s*;", body, re.S)
    if not m:
        return None
    inner = re.sub(r"//[^\n]*", "", m.group(1))
    vals = [v for v in re.split(r"[,\s]+", inner) if v]
    return [int(v.rstrip("uUlL")) for v in vals] if all(re.fullmatch(r"\d+[uUlL]*", v) for v in vals) else None


def product(expr):
    """An element count written as a number or a product of numbers, casts allowed: `(uint64_t)1024 * 1024 * 4`."""
    expr = re.sub(r"\(\s*(uint64_t|u64)\s*\)|static_cast<\w+>", "", expr).replace("(", "").replace(")", "")
    factors = [f.strip() for f in expr.split("*")]
    if not all(re.fullmatch(r"\d+[uUlL]*", f) for f in factors):
        return None
    value = 1
    for f in factors:
        value *= int(f.rstrip("uUlL"))
    return value


def ranks_of(body):
    """Rank count of the topology a case builds: the devices listed in `TopoMeta topoMeta{{{..}, {..}}}`, or the
    product of the three numbers of `GenTopoMeta(topoMeta, pods, servers, devices)`."""
    m = re.search(r"TopoMeta\s+topoMeta\s*\{(.*?)\}\s*;", body, re.S)
    if m:
        return len(re.findall(r"\d+", m.group(1)))
    m = re.search(r"GenTopoMeta\(\s*topoMeta\s*,\s*(\d+)\s*,\s*(\d+)\s*,\s*(\d+)\s*\)", body)
    return int(m.group(1)) * int(m.group(2)) * int(m.group(3)) if m else None


def rooted_cases(out):
    # broadcast_testcase.cc: either named locals (rankSize, count, dataType, root) or the arguments written into the call
    fn = "broadcast_testcase.cc"
    for name, line, body in cases_of(os.path.join(REF, fn)):
        body = re.sub(r"//[^\n]*", "", body)
        types = re.findall(r"HCCL_DATA_TYPE_(\w+)", body)
        call = re.search(r"RunBroadcastTest\(\s*topoMeta\s*,\s*([^,]+),\s*([^,]+),\s*[\w:]+\s*,\s*([^,]+),", body)
        if not (types and call):
            continue
        local = {k: re.search(r"\b%s\s*=\s*([^;]+);" % k, body) for k in ("rankSize", "count", "root")}
        arg = [local[k].group(1) if local[k] and a.strip() == k else a for k, a in zip(("rankSize", "count", "root"), call.groups())]
        ranks, count, root = (product(a) for a in arg)
        if None in (ranks, count, root) or ranks != ranks_of(body):
            continue
        out.append({"kind": "broadcast", "name": name, "source": "%s:%d" % (fn, line), "ranks": ranks,
                    "types": [types[0]], "count": count, "root": root})
    # scatter_testcase.cc: RunScatterTest(root, topoMeta, count, type)
    fn = "scatter_testcase.cc"
    for name, line, body in cases_of(os.path.join(REF, fn)):
        body = re.sub(r"//[^\n]*", "", body)
        call = re.search(r"RunScatterTest\w*\(\s*(\d+)\s*,\s*topoMeta\s*,\s*([^,]+),\s*HcclDataType::HCCL_DATA_TYPE_(\w+)\s*\)", body)
        ranks = ranks_of(body)
        if not call or ranks is None or product(call.group(2)) is None:
            continue
        out.append({"kind": "scatter", "name": name, "source": "%s:%d" % (fn, line), "ranks": ranks,
                    "types": [call.group(3)], "count": product(call.group(2)), "root": int(call.group(1))})


def main():
    out = []
    for fn, kind in (("alltoallv_testcase.cc", "all_to_all_v"), ("alltoallvc_testcase.cc", "all_to_all_vc")):
        for name, line, body in cases_of(os.path.join(REF, fn)):
            matrix = numbers(body, "sendCountMatrix")
            types = re.findall(r"HCCL_DATA_TYPE_(\w+)", body)
            n = int(round(len(matrix) ** 0.5)) if matrix else 0
            if matrix and n * n == len(matrix) and types:
                out.append({"kind": kind, "name": name, "source": "%s:%d" % (fn, line), "ranks": n,
                            "types": sorted(set(types), key=types.index), "matrix": matrix})
    for fn in ("all_gather_v_testcase.cc", "reduce_scatter_v_testcase.cc", "reduce_scatter_v_testcase_a3.cc"):
        kind = "all_gather_v" if fn.startswith("all_gather") else "reduce_scatter_v"
        path = os.path.join(REF, fn)
        if not os.path.exists(path):
            continue
        for name, line, body in cases_of(path):
            counts, displs = numbers(body, r"\.counts"), numbers(body, r"\.displs")
            made = re.search(r"MakeVDataDes\(\s*\{([^{}]*)\}\s*,\s*\{([^{}]*)\}\s*,", body)
            if made and not counts:   # the helper form: MakeVDataDes({counts}, {displs}, type)
                counts, displs = ([int(v) for v in re.findall(r"\d+", made.group(k))] for k in (1, 2))
            types = re.findall(r"HCCL_DATA_TYPE_(\w+)", body)
            ops = re.findall(r"HCCL_REDUCE_(\w+)", body)
            if counts and displs and len(counts) == len(displs) and types:
                entry = {"kind": kind, "name": name, "source": "%s:%d" % (fn, line), "ranks": len(counts),
                         "types": sorted(set(types), key=types.index), "counts": counts, "displs": displs}
                if ops:
                    entry["ops"] = sorted(set(ops), key=ops.index)
                # cases that only assert the entry point's return code: (in place?, expected code)
                m = re.search(r"EXPECT_EQ\(\s*Run\w+\(\s*\w+\s*,\s*\w+\s*,\s*(true|false)\s*\)\s*,\s*HCCL_(\w+)\s*\)", body)
                if m:
                    entry["in_place"] = m.group(1) == "true"
                    entry["expect"] = m.group(2)
                out.append(entry)
    rooted_cases(out)
    path = os.path.join(HERE, "reference_st_shapes.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=None, separators=(",", ":"))
        f.write("\n")
    by_kind = {}
    for e in out:
        by_kind[e["kind"]] = by_kind.get(e["kind"], 0) + 1
    print(path, by_kind)


if __name__ == "__main__":
    main()
