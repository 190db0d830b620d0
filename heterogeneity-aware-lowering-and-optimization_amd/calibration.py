"""Post-training-quantisation calibration on top of libodla_hip.so.

The library has a calibration mode (csrc/profiler.cc): between StartProfiling
and StopProfiling every computation is compiled in fp32 with range statistics
behind every named value, and each execution inside StartOneRun / StopOneRun
appends one record per value to a JSON file in the layout of the reference's
profiler (ODLA/platforms/odla_profiler.cc:203-213,247-285 of the reference
tree).  This module drives that mode and turns the file into the
odla_value_quant_info table the int8 plan consumes, following the reference's
driver script (utils/halo_pgq.py:241-332): consolidate the runs, derive scale
and zero point, emit one tensor record (ch_idx = -channels) plus one record per
channel.
"""
import ctypes
import json
import math

from . import odla


class Profiler:
    """Context manager around the library's profiler control functions."""

    def __init__(self, path, channel_axis=None, skip_weights=False, lib=None):
        self.L = lib or odla.load_library()
        self.path = path
        self.channel_axis = channel_axis
        self.skip_weights = skip_weights
        for name, args in (("StartProfiling", [ctypes.c_char_p]), ("StartOneRun", [ctypes.c_char_p]), ("StopOneRun", []),
                           ("StopProfiling", []), ("EnableChannelWiseProf", []), ("SetChannelAxis", [ctypes.c_int]),
                           ("SkipWeightsProfiling", [ctypes.c_bool])):
            f = getattr(self.L, name)
            f.restype = None
            f.argtypes = args

    def __enter__(self):
        self.L.StartProfiling(self.path.encode())
        if self.channel_axis is not None:
            self.L.EnableChannelWiseProf()
            self.L.SetChannelAxis(int(self.channel_axis))
        if self.skip_weights:
            self.L.SkipWeightsProfiling(True)
        return self

    def run(self, tag):
        prof = self

        class _Run:
            def __enter__(self):
                prof.L.StartOneRun(str(tag).encode())

            def __exit__(self, *exc):
                prof.L.StopOneRun()
                return False
        return _Run()

    def __exit__(self, *exc):
        self.L.StopProfiling()
        return False


def load_profile(path):
    with open(path) as f:
        return json.load(f)


def consolidate(profile):
    """Union of the ranges over all runs, per value [ref: utils/halo_pgq.py:241-279]."""
    out = {}
    for run_data in profile["ProfilingResults"].values():
        for name, rec in run_data.items():
            chs = rec["channels"]
            if chs != len(rec["channels_max"]) or chs != len(rec["channels_min"]):
                continue
            if name not in out:
                out[name] = dict(rec, channels_min=list(rec["channels_min"]), channels_max=list(rec["channels_max"]))
                continue
            acc = out[name]
            if acc["channels"] != chs or acc["op_type"] != rec["op_type"]:
                continue
            acc["min_value"] = min(acc["min_value"], rec["min_value"])
            acc["max_value"] = max(acc["max_value"], rec["max_value"])
            acc["channels_min"] = [min(a, b) for a, b in zip(acc["channels_min"], rec["channels_min"])]
            acc["channels_max"] = [max(a, b) for a, b in zip(acc["channels_max"], rec["channels_max"])]
    return out


def quant_params(mn, mx, scheme="asym_zero"):
    """scale and zero point of an 8-bit affine code for the range [mn, mx].

    "asym" and "asym_max_zp_255" are the reference's rules
    [ref: utils/halo_pgq.py:287-302].  "asym_zero" first widens the range to
    contain 0 (so that padding and ReLU floors are exactly representable) and
    clips the zero point to [0, 255]; it is the rule this library's int8 plan
    was validated with.
    """
    if scheme == "asym_zero":
        import numpy as np
        mn = np.float32(min(float(mn), 0.0))
        mx = np.float32(max(float(mx), 0.0))
        scale = np.float32((mx - mn) / np.float32(255.0))
        if not scale > 0:
            scale = np.float32(1.0)
        return float(scale), int(np.clip(np.rint(np.float32(-mn) / scale), 0, 255))
    scale = (mx - mn) / 255
    if scheme == "asym_max_zp_255":
        if scale == 0:
            scale = abs(mx)
        if scale == 0:
            scale = 1
        return scale, round(min(255, max(0, round(0 - mn / scale))))
    if scheme == "asym":
        return scale, round(round(-(mn / scale)) if scale != 0 else 0)
    raise ValueError("unsupported quantization scheme %r" % scheme)


def table_entries(consolidated, scheme="asym_zero", min_dim_chs=0, max_dim_chs=math.inf):
    """(name, scale, zero_point, min, max, [(ch_min, ch_max), ...] or None) per value, the
    input of ``odla.quant_table`` [ref: utils/halo_pgq.py:308-327]."""
    entries = []
    for name, rec in consolidated.items():
        scale, zp = quant_params(rec["min_value"], rec["max_value"], scheme)
        chs = rec["channels"]
        dims = len(rec["shape"])
        if dims < min_dim_chs or dims > max_dim_chs or chs <= 1:
            ch = None
        else:
            ch = list(zip(rec["channels_min"], rec["channels_max"]))
        entries.append((name, scale, zp, rec["min_value"], rec["max_value"], ch))
    return entries


def write_c_table(entries, path):
    """The C source the reference's driver emits for -quantization-info
    [ref: utils/halo_pgq.py:308-332]."""
    fmt = '  {{.value_id = (const odla_value_id) "{}", .ch_idx = {}, .scale = {}, .offset = {}, .min = {}, .max = {}}},\n'
    n = 0
    with open(path, "w") as f:
        f.write("#include <ODLA/ops/odla_ops_quantization.h>\n")
        f.write("const odla_value_quant_info quant_infos[] = {\n")
        for name, scale, zp, mn, mx, ch in entries:
            f.write(fmt.format(name, -(len(ch) if ch else 1), scale, zp, mn, mx))
            n += 1
            for c, (cmn, cmx) in enumerate(ch or []):
                f.write(fmt.format(name, c, 0, 0, cmn, cmx))
                n += 1
        f.write("};\n")
        f.write("const int quant_infos_size = {};\n".format(n))
    return n
