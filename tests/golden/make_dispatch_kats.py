"""Extracts the dispatcher known-answer data the reference holds into dispatch_kats.json.

Run in the authoring container only (needs the reference checkout; the fixture it writes is
committed and is all the tests read):

    python tests/golden/make_dispatch_kats.py [/root/reference]

For every tuned artefact directory under experiment/dtas_tuned/ it records DATA, not source:
  * from host.cc: the call_table rows ({launch_args...}, kernel name), the index_table and the
    index statement that the reference's Engine emitted;
  * from data_base/best_record.json: per bucket, the range and the winning config dict;
  * from data_base/tuning_record.py: per bucket, the candidate config dicts that were emitted
    (the "#range:" / "#config:" comment lines only).
These pin generate_range_list, merge_same_configs, get_index_table and the config emitters.
"""
import ast
import json
import os
import re
import sys

ROOT = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
BASE = os.path.join(ROOT, "experiment", "dtas_tuned")

ROW = re.compile(r"\{\{([^}]*)\},\s*\w+,\s*\"([^\"]+)\"\}")
RANGE = re.compile(r"<(\w+): Range\((\d+), (\d+)\)>")


def parse_host(path):
    text = open(path).read()
    out = {}
    m = re.search(r"kernel_entry_info call_table\[\] = \{(.*?)\n\s*\};", text, re.S)
    if m:
        rows = []
        for args, name in ROW.findall(m.group(1)):
            # an entry is a literal "(int64_t)320" or a dynamic extent such as "n" (grid = rows)
            vals = []
            for tok in args.split(","):
                m2 = re.search(r"\(int64_t\)(\d+)", tok)
                vals.append(int(m2.group(1)) if m2 else tok.strip().strip("()"))
            rows.append({"launch_args": vals, "name": name})
        out["call_table"] = rows
    m = re.search(r"int64_t index_table\[\] = \{([^}]*)\};", text)
    if m:
        out["index_table"] = [int(x) for x in m.group(1).split(",") if x.strip()]
    m = re.search(r"int64_t index = ([^;]*);", text)
    if m:
        out["index_stmt"] = "  int64_t index = " + m.group(1).strip() + ";\n"
    m = re.search(r"TVM_DLL int32_t (\w+)\(", text)
    if m:
        out["func"] = m.group(1)
    if "call_table" not in out:
        # static-shape path: a single kernel, launch arguments pushed as literals
        out["single_kernel"] = sorted(set(re.findall(r"\"(\w+_kernel)\"", text)))
        out["literal_launch_args"] = [int(x) for x in re.findall(r"v_int64\) = \(\(int64_t\)(\d+)\);", text)]
    return out


def parse_best(path):
    recs = []
    for rec in json.load(open(path)):
        for key, val in rec.items():
            ranges = [[v, int(a), int(b)] for v, a, b in RANGE.findall(key)]
            recs.append({"key_prefix": key.split("_<")[0], "ranges": ranges, "config": val["config"][0]})
    return recs


def parse_tuning(path):
    buckets = []
    cur = None
    for line in open(path, errors="replace"):
        if line.startswith("#range:"):
            ranges = [[v, int(a), int(b)] for v, a, b in RANGE.findall(line)]
            if cur is None or cur["ranges"] != ranges:
                cur = {"ranges": ranges, "configs": []}
                buckets.append(cur)
        elif line.startswith("#config:") and cur is not None:
            kind, _, body = line[len("#config:"):].strip().partition(": ")
            cur["configs"].append({"kind": kind, "config": ast.literal_eval(body)})
    return buckets


def main():
    kats = {}
    for dirpath, _, files in sorted(os.walk(BASE)):
        if "host.cc" not in files:
            continue
        rel = os.path.relpath(dirpath, ROOT)
        entry = {"host": parse_host(os.path.join(dirpath, "host.cc"))}
        best = os.path.join(dirpath, "data_base", "best_record.json")
        if os.path.exists(best):
            entry["best_record"] = parse_best(best)
        tun = os.path.join(dirpath, "data_base", "tuning_record.py")
        if os.path.exists(tun):
            entry["candidates"] = parse_tuning(tun)
        kats[rel] = entry
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "dispatch_kats.json")
    with open(out, "w") as f:
        json.dump(kats, f, indent=1, sort_keys=True)
    print(f"wrote {out}: {len(kats)} artefact dirs")


if __name__ == "__main__":
    main()
