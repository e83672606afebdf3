"""Makes launch_table_cover.json: a smallest set of (shape, setting) runs of
tests/test_gpu_launch_table.py that between them launch every kernel build
the full sweep launches.

Two steps, on a machine with the GPU (from the repository root):

  1. the full sweep under a kernel trace, with this file loaded as a pytest
     plugin, which launches a marker (oslo_copy_probe with a grid size of its
     own) before every run of a shape under a setting and writes the list of
     runs to marks.json:

       cd /tmp && export TMPDIR=/tmp && cd <repository root>
       PYTHONPATH=tests/golden OSLO_LAUNCH_TABLE=full OSLO_COVER_MARKS=<dir>/marks.json \\
       rocprofv3 --kernel-trace -M --output-format csv -d <dir> -o t -- \\
           python3 -m pytest -p make_launch_table_cover tests/test_gpu_launch_table.py -m gpu -q

  2. the cover: the trace is cut at the markers, every kernel of the library
     (mangled name, i.e. with its template arguments) is attributed to the
     runs that launched it, and runs are picked greedily, the one that adds
     the most kernels first, until every kernel is launched:

       python3 tests/golden/make_launch_table_cover.py <dir> <dir>/marks.json

The table only has to be made again when a launch rule, a launch table or the
sweep itself changes; tests/test_gpu_launch_table.py reads it at collection.
"""
import collections
import csv
import glob
import gzip
import json
import os
import re
import sys

# ---------------------------------------------------------------------------
# step 1: pytest plugin
# ---------------------------------------------------------------------------
_state = {"item": None, "marks": [], "buffers": None}


def pytest_runtest_call(item):
    _state["item"] = item.nodeid


def pytest_collection_finish(session):
    table = sys.modules.get("test_gpu_launch_table")
    if table is None:
        return
    import torch
    from oslo_amd.torch import _C

    lib = _C.load_library()

    def marked(settings, run):
        done = 0
        for setting in settings:
            for key in table.KEYS:
                _C.tune(key, 0)
            if _state["buffers"] is None:
                _state["buffers"] = tuple(torch.zeros(32 << 20, dtype=torch.uint8, device="cuda") for _ in range(2))
            src, dst = _state["buffers"]
            index = len(_state["marks"])
            nbytes = 16 * 256 * (index + 1)          # index + 1 workgroups of 256 lanes
            assert nbytes <= src.numel(), "more runs than the marker can number"
            assert lib.oslo_copy_probe(src.data_ptr(), dst.data_ptr(), nbytes,
                                       torch.cuda.current_stream().cuda_stream) == 0
            torch.cuda.synchronize()
            _state["marks"].append([index, _state["item"], setting])
            for key, value in setting.items():
                _C.tune(key, value)
            try:
                run(setting)
            except RuntimeError as e:
                if not setting or not any(s in str(e) for s in ("no kernel", "needs a workgroup", "built for")):
                    raise
                continue
            torch.cuda.synchronize()
            done += 1
        return done

    table._under_each = marked


def pytest_sessionfinish(session, exitstatus):
    if _state["marks"]:
        with open(os.environ.get("OSLO_COVER_MARKS", "marks.json"), "w") as f:
            json.dump(_state["marks"], f)


# ---------------------------------------------------------------------------
# step 2: the cover
# ---------------------------------------------------------------------------
def kernels_per_mark(trace_dir):
    rows = []
    for path in glob.glob(os.path.join(trace_dir, "**", "*kernel_trace.csv*"), recursive=True):
        opener = gzip.open if path.endswith(".gz") else open
        with opener(path, "rt", newline="") as f:
            for row in csv.DictReader(f):
                name = row.get("Kernel_Name") or ""
                if "oslo" in name:
                    rows.append((int(row["Start_Timestamp"]), name, int(row["Grid_Size_X"])))
    rows.sort()
    per_mark, current = collections.defaultdict(set), -1
    for _, name, grid in rows:
        if "copy_probe_kernel" in name:
            current = grid // 256 - 1
        elif current >= 0:
            per_mark[current].add(name[:-3] if name.endswith(".kd") else name)
    return per_mark


def greedy_cover(per_mark):
    remaining = set().union(*per_mark.values())
    chosen = []
    while remaining:
        best = max(per_mark, key=lambda m: (len(per_mark[m] & remaining), -m))
        gain = per_mark[best] & remaining
        if not gain:
            break
        chosen.append(best)
        remaining -= gain
    return chosen


def main(trace_dir, marks_path):
    marks = {m[0]: m for m in json.load(open(marks_path))}
    per_mark = kernels_per_mark(trace_dir)
    chosen = greedy_cover(per_mark)
    family = {"test_softmax_launch_table": "softmax", "test_norm_launch_table": "norm",
              "test_elementwise_launch_table": "eltwise"}
    table = {name: collections.defaultdict(list) for name in family.values()}
    for m in chosen:
        _, nodeid, setting = marks[m][:3]
        test, params = re.match(r".*::(\w+)\[(.*)\]", nodeid).groups()
        dtype, size = params.rsplit("-", 1)          # "f32-f16-4096" -> "f32-f16", "4096"
        table[family[test]]["%s:%s" % (dtype, size)].append(setting)

    def shape_order(key):
        dtype, size = key.split(":")
        return dtype, int(size)

    out = {fam: {k: sorted(v, key=lambda d: json.dumps(d, sort_keys=True)) for k, v in sorted(t.items(), key=lambda kv: shape_order(kv[0]))}
           for fam, t in table.items()}
    lines = ["{"]
    for i, (fam, shapes) in enumerate(out.items()):
        lines.append(' "%s": {' % fam)
        items = list(shapes.items())
        for j, (key, settings) in enumerate(items):
            lines.append('  "%s": %s%s' % (key, json.dumps(settings, sort_keys=True), "," if j + 1 < len(items) else ""))
        lines.append(" }" + ("," if i + 1 < len(out) else ""))
    lines.append("}")
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "launch_table_cover.json")
    with open(path, "w") as f:
        f.write("\n".join(lines) + "\n")
    kernels = set().union(*per_mark.values())
    print("%d runs in the sweep, %d kernels launched, %d runs chosen over %d shapes -> %s"
          % (len(marks), len(kernels), len(chosen), sum(len(t) for t in out.values()), path))


if __name__ == "__main__":
    main(sys.argv[1], sys.argv[2])
