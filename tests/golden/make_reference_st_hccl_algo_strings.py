"""Collects every HCCL_ALGO string the reference's own system tests set, as data.

Reads (as text; nothing of the reference is imported or run) test/st/algorithm/testcase/*.cc and writes
tests/golden/reference_st_hccl_algo_strings.json: one entry per distinct string with the places it is used
(file:line).  These are configurations the reference's parser of this device generation accepts (the cases run
with them); tests/test_two_level_and_hccl_algo.py checks that the library's parser accepts every one of them.

Usage (in the container that holds /root/reference):  python tests/golden/make_reference_st_hccl_algo_strings.py
"""
import glob
import json
import os
import re

REF = "/root/reference/test/st/algorithm/testcase"
HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    found = {}
    for path in sorted(glob.glob(os.path.join(REF, "*.cc")) + glob.glob(os.path.join(REF, "*.h"))):
        for no, line in enumerate(open(path, encoding="utf-8", errors="replace"), 1):
            for m in re.finditer(r'"([a-z_]+:[A-Za-z_]+\{[^"]*\})"', line):
                found.setdefault(m.group(1), []).append("%s:%d" % (os.path.basename(path), no))
    out = [{"config": k, "used_at": v} for k, v in sorted(found.items())]
    with open(os.path.join(HERE, "reference_st_hccl_algo_strings.json"), "w") as f:
        json.dump(out, f, indent=1)
        f.write("\n")
    print(len(out), "distinct strings,", sum(len(v) for v in found.values()), "uses")


if __name__ == "__main__":
    main()
