"""The cover table of the launch-table sweep and the tool that makes it, without a GPU."""
import csv
import importlib.util
import json
import os

HERE = os.path.dirname(__file__)


def _tool():
    spec = importlib.util.spec_from_file_location("make_launch_table_cover",
                                                  os.path.join(HERE, "golden", "make_launch_table_cover.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_trace_is_cut_at_the_markers_and_covered_greedily(tmp_path):
    tool = _tool()
    rows = [
        # (timestamp, kernel, grid): marker i has a grid of 256 * (i + 1) lanes
        (5, "_ZN4oslo9early_kernelEv.kd", 64),                       # before the first marker: ignored
        (10, "_ZN4oslo17copy_probe_kernelEPKDv4_jPS0_l.kd", 256),    # run 0
        (11, "_ZN4oslo1aEv.kd", 64), (12, "_ZN4oslo1bEv.kd", 64),
        (20, "_ZN4oslo17copy_probe_kernelEPKDv4_jPS0_l.kd", 512),    # run 1
        (21, "_ZN4oslo1bEv.kd", 64),
        (30, "_ZN4oslo17copy_probe_kernelEPKDv4_jPS0_l.kd", 768),    # run 2
        (31, "_ZN4oslo1cEv.kd", 64), (32, "_ZN2at6nativeEv.kd", 64),
    ]
    with open(tmp_path / "t_kernel_trace.csv", "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(["Kernel_Name", "Start_Timestamp", "Grid_Size_X"])
        for ts, name, grid in reversed(rows):                         # (the file need not be in time order)
            w.writerow([name, ts, grid])
    per_mark = tool.kernels_per_mark(str(tmp_path))
    assert dict(per_mark) == {0: {"_ZN4oslo1aEv", "_ZN4oslo1bEv"}, 1: {"_ZN4oslo1bEv"}, 2: {"_ZN4oslo1cEv"}}
    assert sorted(tool.greedy_cover(per_mark)) == [0, 2]             # run 1 adds nothing


def test_cover_table_names_shapes_and_overrides_of_the_sweep():
    with open(os.path.join(HERE, "golden", "launch_table_cover.json")) as f:
        cover = json.load(f)
    assert set(cover) == {"softmax", "norm", "eltwise"}
    src = open(os.path.join(HERE, "test_gpu_launch_table.py")).read()
    for family, shapes in cover.items():
        assert shapes, family
        for key, settings in shapes.items():
            dtype, size = key.split(":")
            assert all(d in ("f32", "f16", "bf16") for d in dtype.split("-")) and int(size) > 0
            assert settings and all(isinstance(s, dict) for s in settings)
            for s in settings:
                for knob, value in s.items():
                    assert '"%s"' % knob in src and isinstance(value, int)   # a knob the sweep resets afterwards
