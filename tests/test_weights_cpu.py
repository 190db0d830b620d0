"""Weight-container readers (no GPU): the C arrays of ``-emit-data-as-c``, ELF
data symbols, and the Const nodes of a frozen GraphDef - checked on the
reference's own mnist_simple.pb (copied to tests/golden as a data fixture), on
text in the writer's format (lib/target/generic_cpp/generic_cxx_constant_writer.cc:24-36
of the reference tree) and on an object file compiled here.
"""
import os
import shutil
import subprocess

import numpy as np
import pytest

import __graft_entry__ as entry


def test_graphdef_constants_of_mnist_simple(pkg):
    data = open(os.path.join(entry.ROOT, "tests", "golden", "mnist_simple.pb"), "rb").read()
    assert len(data) == 31736
    c = pkg.weights.read_graphdef_constants(data)
    assert sorted(c) == ["Variable", "Variable_1"]
    W, b = c["Variable"], c["Variable_1"]
    assert W.shape == (784, 10) and W.dtype == np.float32 and b.shape == (10,) and b.dtype == np.float32
    assert np.all(np.isfinite(W)) and np.all(np.isfinite(b)) and float(np.abs(W).max()) > 0.1
    # a softmax regression trained by gradient descent from zero keeps the class sums at zero:
    # every gradient (softmax - onehot) sums to zero over the classes
    assert np.max(np.abs(W.sum(axis=1))) <= 1e-5 and abs(float(b.sum())) <= 1e-5
    # the corner pixel of an MNIST image is always blank, so its weights never moved
    assert np.all(W[0] == 0) and np.all(W[783] == 0)


def test_c_arrays_in_the_writers_format(pkg):
    r = np.random.default_rng(3)
    w = r.standard_normal((2, 3, 4)).astype(np.float32)
    idx = r.integers(-5, 5, (7,)).astype(np.int64)
    lines = [
        "//===- Halo Compiler Generated File ---------------------------------------===//",
        "",
        "#include <stdint.h>",
        "#include <ODLA/odla.h>",
        "extern float const conv1_w[2*3*4] = {" + ", ".join("%.10g" % v for v in w.reshape(-1)) + "};",
        "extern int64_t const shape_1[7] = {" + ", ".join(str(int(v)) for v in idx) + "};",
    ]
    c = pkg.weights.read_c_arrays("\n".join(lines) + "\n")
    assert sorted(c) == ["conv1_w", "shape_1"]
    assert c["conv1_w"].shape == (2, 3, 4) and np.array_equal(c["conv1_w"], w)   # 10 digits round-trip fp32
    assert c["shape_1"].dtype == np.int64 and np.array_equal(c["shape_1"], idx)
    with pytest.raises(ValueError):
        pkg.weights.read_c_arrays("extern float const bad[3] = {1, 2};")


@pytest.mark.skipif(shutil.which("gcc") is None, reason="needs gcc to make an object file")
def test_elf_data_symbols(pkg, tmp_path):
    src = tmp_path / "w.c"
    src.write_text("\n".join([
        "const float W[6] = {1.5f, -2.0f, 3.25f, 0.0f, 1e-3f, 7.0f};",
        "const int dims[2] = {2, 3};",
        "float scratch[4];",
        "static int hidden = 5;",
        "int use(void) { return hidden; }",
    ]) + "\n")
    obj = tmp_path / "w.bin"
    subprocess.check_call(["gcc", "-c", "-fno-common", str(src), "-o", str(obj)])
    syms = pkg.weights.read_elf_symbols(obj.read_bytes())
    assert np.array_equal(np.frombuffer(syms["W"], np.float32), np.array([1.5, -2.0, 3.25, 0.0, 1e-3, 7.0], np.float32))
    assert np.frombuffer(syms["dims"], np.int32).tolist() == [2, 3]
    assert syms["scratch"] == bytes(16)
    with pytest.raises(ValueError):
        pkg.weights.read_elf_symbols(b"not an object file")
