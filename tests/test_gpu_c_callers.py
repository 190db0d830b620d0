"""C programs as callers of the library: sources under tests/c_callers are
compiled with gcc as C11 against include/odla_hip.h, linked with -lodla_hip and
run.  They exercise what ctypes callers cannot: by-value odla_value_type /
odla_values arguments as a C compiler lays them out, compound literals as the
reference's code generator writes them, and the device / memory API.

  model   gen_model.c + main_model.c: the shape of HALO-generated code for
          add1 = (input + w0) + w1; the reference's own test expects 6, 9, 12
          [ref: tests/compile/test_cxx_gen.cc:46-48].
  device  device_info.c: the 13 odla_GetDeviceInfo items of the reference's
          device test [ref: tests/ODLA/device_test.cc:63-89] and a host / device
          memory round trip.
"""
import os
import subprocess

import pytest

import __graft_entry__ as entry
from util import announce

SRC = os.path.join(entry.ROOT, "tests", "c_callers")
INC = os.path.join(entry.ROOT, "include")
LIBDIR = entry.PKG_DIR


def build(tmp_path, name, sources):
    exe = str(tmp_path / name)
    cmd = ["gcc", "-std=c11", "-Wall", "-Werror", "-I", INC] + [os.path.join(SRC, s) for s in sources] + \
          ["-L", LIBDIR, "-lodla_hip", "-Wl,-rpath," + LIBDIR, "-Wl,-rpath,/opt/rocm/lib", "-o", exe]
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    return exe


def test_c_sources_compile_against_the_header(tmp_path):
    """No GPU needed: the C callers compile as C11 with every warning an error."""
    for src in ("gen_model.c", "main_model.c", "device_info.c"):
        subprocess.run(["gcc", "-std=c11", "-Wall", "-Wextra", "-Werror", "-I", INC, "-c", os.path.join(SRC, src),
                        "-o", str(tmp_path / (src + ".o"))], check=True, capture_output=True, text=True)


@pytest.mark.gpu
def test_generated_style_model_prints_6_9_12(tmp_path):
    announce("C caller: generated-style model")
    exe = build(tmp_path, "model", ["gen_model.c", "main_model.c"])
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.split() == ["6.000000", "9.000000", "12.000000", "15.000000"]


@pytest.mark.gpu
def test_device_info_and_memory_api(tmp_path):
    announce("C caller: device info + memory API")
    exe = build(tmp_path, "device", ["device_info.c"])
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "memory round trip ok" in r.stdout
    assert r.stdout.count("ODLA_DEVICE_INFO_") == 13
