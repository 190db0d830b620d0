"""Host side of the calibration flow (no GPU): consolidation of profiler runs,
the quantisation-parameter rules and the C table writer, checked on hand-worked
records against the rules of the reference's driver script
(utils/halo_pgq.py:241-332 of the reference tree).
"""
import re

import numpy as np


def _profile():
    rec = lambda op, mn, mx, cmin, cmax, shape: {"op_type": op, "shape": shape, "channels": len(cmin), "min_value": mn,
                                                 "max_value": mx, "channels_min": cmin, "channels_max": cmax}
    return {"ProfilingResults": {
        "a.jpg": {"conv": rec("odla_Conv", -1.0, 3.0, [-1.0, -0.5], [3.0, 1.0], [1, 2, 4, 4]),
                  "relu": rec("odla_Relu", 0.0, 3.0, [], [], [1, 2, 4, 4]),
                  "bad": {"op_type": "odla_Add", "shape": [2], "channels": 3, "min_value": 0, "max_value": 1,
                          "channels_min": [0], "channels_max": [1]}},
        "b.jpg": {"conv": rec("odla_Conv", -2.0, 2.5, [-2.0, 0.25], [2.5, 0.5], [1, 2, 4, 4]),
                  "relu": rec("odla_Relu", 0.0, 5.1, [], [], [1, 2, 4, 4])}},
        "NetworkInfo": {"relu": {"inputs": ["conv"]}}}


def test_consolidate_takes_the_union_of_ranges(pkg):
    m = pkg.calibration.consolidate(_profile())
    assert "bad" not in m                         # inconsistent channel record: skipped as the reference does
    assert (m["conv"]["min_value"], m["conv"]["max_value"]) == (-2.0, 3.0)
    assert m["conv"]["channels_min"] == [-2.0, -0.5] and m["conv"]["channels_max"] == [3.0, 1.0]
    assert (m["relu"]["min_value"], m["relu"]["max_value"]) == (0.0, 5.1)


def test_quant_param_rules(pkg):
    qp = pkg.calibration.quant_params
    # reference "asym": scale = (max - min) / 255, zp = round(-min / scale)
    s, z = qp(-1.0, 3.0, "asym")
    assert s == 4.0 / 255 and z == round(1.0 / (4.0 / 255)) == 64
    assert qp(2.0, 2.0, "asym") == (0.0, 0)
    # reference "asym_max_zp_255": degenerate ranges fall back to |max| (or 1), zp clipped to [0, 255]
    assert qp(2.0, 2.0, "asym_max_zp_255") == (2.0, 0)
    assert qp(0.0, 0.0, "asym_max_zp_255") == (1, 0)
    assert qp(-10.0, -5.0, "asym_max_zp_255")[1] == 255
    # this build's rule: the range is widened to contain zero first
    s, z = qp(1.0, 3.0)
    assert np.float32(s) == np.float32(3.0) / np.float32(255.0) and z == 0
    s, z = qp(-1.0, 3.0)
    assert np.float32(s) == np.float32(4.0) / np.float32(255.0) and z == 64
    assert qp(0.0, 0.0) == (1.0, 0)


def test_table_entries_and_c_writer(pkg, odla, tmp_path):
    cal = pkg.calibration
    entries = cal.table_entries(cal.consolidate(_profile()), "asym")
    by = {e[0]: e for e in entries}
    assert by["conv"][5] == [(-2.0, 3.0), (-0.5, 1.0)] and by["relu"][5] is None
    # dimension window for per-channel records [ref: halo_pgq.py:317-320]
    assert cal.table_entries(cal.consolidate(_profile()), "asym", min_dim_chs=5)[0][5] is None
    recs = odla.quant_table(entries)
    assert [(r.value_id, r.ch_idx) for r in recs] == [(b"conv", -2), (b"conv", 0), (b"conv", 1), (b"relu", -1)]
    path = str(tmp_path / "q.c")
    n = cal.write_c_table(entries, path)
    text = open(path).read()
    assert n == 4 and "const int quant_infos_size = 4;" in text
    rows = re.findall(r'\.value_id = \(const odla_value_id\) "(\w+)", \.ch_idx = (-?\d+), \.scale = ([^,]+), \.offset = ([^,]+), '
                      r'\.min = ([^,]+), \.max = ([^}]+)\}', text)
    assert [(r[0], int(r[1])) for r in rows] == [("conv", -2), ("conv", 0), ("conv", 1), ("relu", -1)]
    assert float(rows[0][2]) == 5.0 / 255 and int(rows[0][3]) == 102 and float(rows[1][4]) == -2.0
