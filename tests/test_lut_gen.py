"""LUT generation tool (host code of the library): built-in designs against the
reference's committed tables and against the CPU oracle, and the plug-in route
(a user's C multiplier compiled and evaluated) -- lut/lut_gen.cc:86-127,
developer.md:38-86."""
import ctypes as C
import os
import shutil
import subprocess
import sys

import numpy as np
import pytest

import approxtrain_amd
from approxtrain_amd import lut_gen
from oracle import cpu
from tests.util import LUT_FILES, lut_bytes, lut_path

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("name,m", LUT_FILES)
def test_builtin_tables_equal_reference_files(name, m):
    assert np.array_equal(lut_gen.generate_builtin(name, m), lut_bytes(name, m))


@pytest.mark.parametrize("name,kind", [("MBM", "MBM"), ("MIT", "MIT")])
@pytest.mark.parametrize("m", [2, 4, 6, 9, 11])
def test_builtin_tables_equal_oracle_at_other_widths(name, kind, m):
    """Widths the reference ships no file for: the library's integer rules against the
    oracle's restatement of the functional models (4-byte layout)."""
    got = lut_gen.generate_builtin(name, m, entry_bytes=4)   # carry << 31 | mantissa in place
    want = cpu.lutgen32(kind, m)                               # the oracle keeps the carry at bit 23
    assert np.array_equal(got >> 31, (want >> 23) & 1)
    assert np.array_equal(got & 0x7fffff, want & 0x7fffff)


def test_one_and_four_byte_layouts_agree():
    b1 = lut_gen.generate_builtin("MBM", 5, 1)
    b4 = lut_gen.generate_builtin("MBM", 5, 4)
    assert np.array_equal((b4 >> 31).astype(np.uint8), b1 >> 7)
    assert np.array_equal(((b4 & 0x7fffff) >> (23 - 5)).astype(np.uint8), b1 & 0x7f)


def test_zeros_table():
    assert not lut_gen.generate_builtin("ZEROS", 7).any()


def test_python_callable_multiplier():
    # an exact multiplier truncated to 3 mantissa bits == the ACC rule at width 3
    def f(a, b):
        return float(np.float32(a) * np.float32(b))
    got = lut_gen.generate_from_function(f, 3)
    assert np.array_equal(got, lut_gen.generate_builtin("ACC", 3))


USER_DESIGN = """
/* exact product of operands truncated to 1+8+7 bits, truncated again */
static float trunc_mul(float a, float b) {
    uint32_t ua, ub, up; memcpy(&ua, &a, 4); memcpy(&ub, &b, 4);
    ua &= 0xffff0000u; ub &= 0xffff0000u; memcpy(&a, &ua, 4); memcpy(&b, &ub, 4);
    float p = a * b; memcpy(&up, &p, 4); up &= 0xffff0000u; memcpy(&p, &up, 4); return p;
}
"""


@pytest.mark.skipif(shutil.which("gcc") is None, reason="needs a C compiler")
def test_cli_with_user_source_reproduces_acc7(tmp_path):
    """developer.md's flow: write the multiplier as a C function, generate <NAME>_<m>.bin.
    A truncating exact multiplier is the reference's bfloat16mul, so the file must equal ACC_7.bin."""
    src = tmp_path / "my_design.inl"
    src.write_text(USER_DESIGN)
    out = subprocess.run([sys.executable, "-m", "approxtrain_amd.lut_gen", "--source", str(src), "--function",
                          "trunc_mul", "--name", "MYMUL", "--mant-width", "7", "--out-dir", str(tmp_path)],
                         cwd=ROOT, capture_output=True, text=True)
    assert out.returncode == 0, out.stderr
    made = tmp_path / "MYMUL_7.bin"
    assert out.stdout.strip() == str(made)
    assert made.read_bytes() == lut_bytes("ACC", 7).tobytes()


def test_cli_all_writes_the_reference_set(tmp_path):
    assert lut_gen.main(["--all", "--out-dir", str(tmp_path)]) == 0
    for name, m in LUT_FILES:
        assert (tmp_path / os.path.basename(lut_path(name, m))).read_bytes() == lut_bytes(name, m).tobytes()
    assert (tmp_path / "ZEROS_7.bin").read_bytes() == bytes(16384)


def test_wide_table_file_has_four_byte_entries(tmp_path):
    assert lut_gen.main(["--multiplier", "MIT", "--mant-width", "9", "--out-dir", str(tmp_path)]) == 0
    assert (tmp_path / "MIT_9.bin").stat().st_size == 4 << 18


def test_generator_argument_errors():
    lib = approxtrain_amd.load_library()
    buf = np.zeros(16384, dtype=np.uint8)
    p = buf.ctypes.data_as(C.c_void_p)
    assert lib.amsim_lut_generate_builtin(b"NOPE", 7, 1, p, buf.nbytes) == 1
    assert b"NOPE" in lib.amsim_last_error()
    assert lib.amsim_lut_generate_builtin(b"MBM", 8, 1, p, buf.nbytes) == 3      # 1-byte entries stop at width 7
    assert lib.amsim_lut_generate_builtin(b"MBM", 7, 1, p, 100) == 1            # buffer too small
    assert lib.amsim_lut_generate_builtin(b"MBM", 7, 2, p, buf.nbytes) == 3     # entry size
    assert lib.amsim_lut_generate(None, None, 7, 1, p, buf.nbytes) == 1
