"""Collects the shapes the reference's own system tests drive through AllReduce, ReduceScatter, Reduce, AllGather and
AlltoAll, as data.

Reads (as text; nothing of the reference is imported or run) the TEST_F cases of
    test/st/algorithm/testcase/all_reduce_testcase.cc, all_reduce_multilevel_testcase.cc, all_reduce_parallel_testcase.cc
    test/st/algorithm/testcase/reduce_scatter_testcase.cc, reduce_scatter_aicpu_testcase.cc, ..._testcase2.cc, ..._testcase3.cc,
        reduce_scatter_3level_testcase.cc, reduce_scatter_meshchunk_concur_testcase.cc
    test/st/algorithm/testcase/reduce_testcase.cc, reduce_aicpu_testcase.cc, reduce_3level_testcase.cc, reduce_sequence_testcase.cc
    test/st/algorithm/testcase/all_gather_aicpu_testcase.cc, all_gather_3level_testcase.cc, alltoall_testcase.cc
and writes tests/golden/reference_st_reduce_shapes.json: one entry per case whose numbers are written out and whose
world has at most 64 ranks, with its name, the file and line it starts on, the servers of its topology (ranks per
server) and its pods (servers per pod), the element count (the file's constants folded in), the data type, the reduce
operation, the root (Reduce) and the HCCL_ALGO string the case, or its fixture's SetUp, sets, if any.  The reference checks these cases on a simulated task graph; tests/test_wide_gpu_reference_st_reduce_shapes.py
replays the shapes (counts scaled down, remainders kept) against the oracle.

Usage (in the container that holds /root/reference):  python tests/golden/make_reference_st_reduce_shapes.py
"""
import json
import os
import re

REF = "/root/reference/test/st/algorithm/testcase"
HERE = os.path.dirname(os.path.abspath(__file__))
FILES = {
    "all_reduce": ["all_reduce_testcase.cc", "all_reduce_multilevel_testcase.cc", "all_reduce_parallel_testcase.cc"],
    "reduce_scatter": ["reduce_scatter_testcase.cc", "reduce_scatter_aicpu_testcase.cc", "reduce_scatter_aicpu_testcase2.cc",
                       "reduce_scatter_aicpu_testcase3.cc", "reduce_scatter_3level_testcase.cc",
                       "reduce_scatter_meshchunk_concur_testcase.cc"],
    "reduce": ["reduce_testcase.cc", "reduce_aicpu_testcase.cc", "reduce_3level_testcase.cc", "reduce_sequence_testcase.cc"],
    "all_gather": ["all_gather_aicpu_testcase.cc", "all_gather_3level_testcase.cc"],
    "all_to_all": ["alltoall_testcase.cc"],
}
SIZES = {"INT8": 1, "UINT8": 1, "INT16": 2, "UINT16": 2, "FP16": 2, "BFP16": 2, "INT32": 4, "UINT32": 4, "FP32": 4,
         "INT64": 8, "UINT64": 8, "FP64": 8, "HIF8": 1, "FP8E4M3": 1, "FP8E5M2": 1, "FP8E8M0": 1}


def cases_of(text):
    for m in re.finditer(r"TEST_F\(\s*\w+\s*,\s*(\w+)\s*\)\s*\{", text):
        start = m.end()
        depth, i = 1, start
        while depth and i < len(text):
            depth += {"{": 1, "}": -1}.get(text[i], 0)
            i += 1
        yield m.group(1), text.count("\n", 0, m.start()) + 1, text[start:i - 1]


def strip_comments(body):
    return re.sub(r"//[^\n]*", "", body)


def value_of(expr, names):
    """An element count written with numbers, the file's constants, + - * /, std::max / std::min and casts."""
    e = re.sub(r"sizeof\(\s*HcclDataType::\w+\s*\)", "4", expr)   # the size of the enumeration, as the case writes it
    e = re.sub(r"static_cast<\s*\w+\s*>", "", e)
    e = re.sub(r"\(\s*(u64|uint64_t|u32)\s*\)", "", e)
    e = e.replace("std::max", "max").replace("std::min", "min")
    e = re.sub(r"(\d+)[uUlL]+\b", r"\1", e)
    e = e.replace("/", "//")
    if not re.fullmatch(r"[\w\s()+\-*/,<>]*", e) or "__" in e:
        return None
    allowed = dict(names, max=max, min=min)
    if any(w not in allowed for w in re.findall(r"[A-Za-z_]\w*", e)):
        return None
    try:
        v = eval(e, {"__builtins__": {}}, allowed)
    except Exception:
        return None
    return int(v) if isinstance(v, int) and v >= 0 else None


def topology(body):
    """(ranks per server, servers per pod) of a case: TopoMeta is a list of pods of servers of device ids."""
    m = re.search(r"TopoMeta\s+\w+\s*\{(.*?)\}\s*;", body, re.S)
    if m:
        text = m.group(1)
        servers, pods, depth, inPod = [], [], 0, 0
        for k, ch in enumerate(text):
            if ch == "{":
                depth += 1
                if depth == 1:
                    inPod = 0
                elif depth == 2:
                    end = text.index("}", k)
                    size = len([x for x in text[k + 1:end].split(",") if x.strip()])
                    if size:
                        servers.append(size)
                        inPod += 1
            elif ch == "}":
                if depth == 1 and inPod:
                    pods.append(inPod)
                depth -= 1
        return (servers, pods) if servers else None
    m = re.search(r"GenTopoMeta\(\s*\w+\s*,\s*(\d+)\s*,\s*(\d+)\s*,\s*(\d+)\s*\)", body)
    if m:
        pods, servers, ranks = int(m.group(1)), int(m.group(2)), int(m.group(3))
        return [ranks] * (pods * servers), [servers] * pods
    return None


def main():
    out = []
    skipped = 0
    large = 0
    for kind, files in FILES.items():
        for name in files:
            text = open(os.path.join(REF, name), encoding="utf-8", errors="replace").read()
            consts = {}
            for m in re.finditer(r"constexpr\s+(?:u64|uint64_t|u32|uint32_t|size_t)\s+(\w+)\s*=\s*([^;]+);", text):
                v = value_of(m.group(2), consts)
                if v is not None:
                    consts[m.group(1)] = v
            tokens = dict(re.findall(r'constexpr\s+char\s+(\w+)\[\]\s*=\s*"([^"]+)"\s*;', text))
            tokens.update(re.findall(r'constexpr\s+const\s+char\s*\*\s*(\w+)\s*=\s*"([^"]+)"\s*;', text))
            # a string the fixture's SetUp puts into HCCL_ALGO holds for every case of the file
            fixture = re.search(r'void\s+SetUp\(\)[^{]*\{[^}]*setenv\(\s*"HCCL_ALGO"\s*,\s*"([^"]+)"', text, re.S)
            for case, line, raw in cases_of(text):
                body = strip_comments(raw)
                topo = topology(body)
                servers, pods = topo if topo else (None, None)
                dtype = re.search(r"HCCL_DATA_TYPE_(\w+)", body)
                op = re.search(r"HCCL_REDUCE_(\w+)", body)
                names = dict(consts)
                if dtype and dtype.group(1) in SIZES:
                    names["dataTypeSize"] = SIZES[dtype.group(1)]
                count = None
                m = re.search(r"\b(?:dataCount|recvCount|sendCount|sendDataCount|count)\s*=\s*([^;]+);", body)
                call = re.search(r"\bRun\w+\(\s*(\w+)\s*,(.*?)\)\s*;", body, re.S)
                args = [a.strip() for a in re.split(r",(?![^()]*\))", call.group(2))] if call else []
                if m:
                    count = value_of(m.group(1), names)
                elif args:
                    count = value_of(args[0], names)
                config = None
                m = re.search(r'"([a-z_]+:[A-Za-z_]+\{[^"]*\})"', body)
                if m:
                    config = m.group(1)
                else:
                    m = re.search(r'setenv\(\s*"HCCL_ALGO"\s*,\s*(\w+)\s*,', body)
                    if m and m.group(1) in tokens:
                        config = tokens[m.group(1)]
                    elif fixture:
                        config = fixture.group(1)
                root = None
                if kind == "reduce":
                    m = re.search(r"\broot\s*=\s*(\d+)\s*;", body)
                    if m:
                        root = int(m.group(1))
                    elif args and re.fullmatch(r"\d+", args[-1]):
                        root = int(args[-1])
                if not servers or not dtype or count is None or (kind == "reduce" and root is None):
                    skipped += 1
                    continue
                if sum(servers) > 64:
                    large += 1
                    continue
                out.append({"kind": kind, "name": case, "source": "%s:%d" % (name, line), "servers": servers,
                            "pods": pods, "count": count, "type": dtype.group(1), "op": op.group(1) if op else "SUM",
                            "root": root, "hccl_algo": config})
    with open(os.path.join(HERE, "reference_st_reduce_shapes.json"), "w") as f:
        json.dump(out, f, indent=0)
        f.write("\n")
    print(len(out), "cases written,", skipped, "left out (numbers built by helpers or loops),", large,
          "for worlds of more than 64 ranks")


if __name__ == "__main__":
    main()
