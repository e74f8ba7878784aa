"""Pins the oracle's product layer (functional models, LUT generator, LUT
product) against the reference's golden LUT files and, where oracle/_ref was
built from the reference tree, against the reference's own compiled C models.
CPU only."""
import hashlib
import os
import subprocess

import numpy as np
import pytest

from oracle import cpu
from tests.util import LUT_FILES, lut_bytes, lut_path, product_domain, same_bits_or_both_nan

# sha256 of the nine LUT files the reference tree commits under lut/
SHA256 = {
    "ACC_7": "96a1b918f9dea7db98eceb484d1b606e3cf60982274d7443b9ed65baf4dfcbee",
    "MBM_1": "8d65a89d33fc69d31f85fd8ed396d6dd5672cd59f80bd2ced560d4bbaeb43222",
    "MBM_3": "cd4273f1732ef9e1465ec931a600a90e201fe3b019f57dcbc71cfba3a64db63f",
    "MBM_5": "8f47b6176ee548baffecb54b851764d62d3e02cced8e88c470f88f160bcd8cc1",
    "MBM_7": "dc2c5c50eb820657f593fde6927a18fbb591582e5e050d8cb727895f9a350d7a",
    "MIT_1": "ba57af15c8d49bc2d673bdbcc15b9761dddf25386be00890bb7cf56cc02b0dba",
    "MIT_3": "c1bbddc81e26a9433ce2b47f1b9982c46ab4a00a4df29333f62fe726cc6b358a",
    "MIT_5": "0d5ae887b74f9f16683cc44b19b3ee4a39c919a29aba236e0556310eb98b451a",
    "MIT_7": "ac623c7e6e5bb79b33d6a5b71dcac0fd324788c73c71370e406c0600bbfab667",
}

needs_ref = pytest.mark.skipif(not cpu.ref_available(), reason="oracle/_ref not built (no reference tree)")


@pytest.mark.parametrize("kind,m", LUT_FILES)
def test_golden_lut_fixture_is_the_reference_file(kind, m):
    data = open(lut_path(kind, m), "rb").read()
    assert len(data) == 1 << (2 * m)
    assert hashlib.sha256(data).hexdigest() == SHA256[f"{kind}_{m}"]


@pytest.mark.parametrize("kind,m", LUT_FILES)
def test_lutgen_reproduces_reference_lut(kind, m):
    assert np.array_equal(cpu.lutgen(kind, m), lut_bytes(kind, m))


def test_known_lut_bytes():
    # values quoted from the reference files themselves
    assert lut_bytes("MBM", 1).tolist() == [0x80] * 4
    assert lut_bytes("MIT", 1).tolist() == [0x00, 0x01, 0x01, 0x80]
    mit3 = lut_bytes("MIT", 3).reshape(8, 8)
    assert mit3[0].tolist() == list(range(8))
    assert mit3[1].tolist() == [1, 2, 3, 4, 5, 6, 7, 0x80]


@pytest.mark.parametrize("m", [1, 3, 5, 7])
def test_mitchell_lut_closed_form(m):
    # Mitchell's multiplier is an add of the two fractions: s = ma + mb,
    # carry = s >> m, mantissa = s mod 2^m.
    i, j = np.meshgrid(np.arange(1 << m), np.arange(1 << m), indexing="ij")
    s = i + j
    want = (((s >> m) << 7) | (s & ((1 << m) - 1))).astype(np.uint8).ravel()
    assert np.array_equal(cpu.lutgen("MIT", m), want)


def test_acc_lut_closed_form():
    # truncated exact product of the 8-bit significands
    m = 7
    i, j = np.meshgrid(np.arange(128), np.arange(128), indexing="ij")
    p = (128 + i) * (128 + j)
    nrm = (p >= (1 << 15)).astype(np.int64)
    want = ((nrm << 7) | ((p >> (m + nrm)) & 127)).astype(np.uint8).ravel()
    assert np.array_equal(cpu.lutgen("ACC", 7), want)


@pytest.mark.parametrize("kind,m", LUT_FILES)
def test_lut_symmetry(kind, m):
    t = lut_bytes(kind, m).reshape(1 << m, 1 << m)
    assert np.array_equal(t, t.T)


_GEN = {("MBM", 7): "FMBM16_MULTIPLIER", ("MBM", 5): "FMBM14_MULTIPLIER", ("MBM", 3): "FMBM12_MULTIPLIER",
        ("MBM", 1): "FMBM10_MULTIPLIER", ("MIT", 7): "MITCHEL16_MULTIPLIER", ("MIT", 5): "MITCHEL14_MULTIPLIER",
        ("MIT", 3): "MITCHEL12_MULTIPLIER", ("MIT", 1): "MITCHEL10_MULTIPLIER", ("ACC", 7): "BFLOAT"}


@needs_ref
@pytest.mark.parametrize("kind,m", LUT_FILES)
def test_reference_generator_binary_reproduces_fixture(kind, m, tmp_path):
    exe = os.path.join(os.path.dirname(cpu.__file__), "_ref", "lut_gen_" + _GEN[(kind, m)])
    subprocess.run([exe], cwd=tmp_path, check=True)
    got = np.fromfile(tmp_path / f"{kind}_{m}.bin", dtype=np.uint8)
    assert np.array_equal(got, lut_bytes(kind, m))


@needs_ref
@pytest.mark.parametrize("kind,m", LUT_FILES)
def test_oracle_model_equals_reference_model(kind, m):
    a, b = product_domain(m, seed=100 + m)
    a, b = a.view(np.float32), b.view(np.float32)
    got = cpu.model_array(kind, m, a, b)
    want = cpu.ref_model_array(kind, m, a, b)
    ok = same_bits_or_both_nan(got, want)
    assert ok.all(), f"{(~ok).sum()} mismatches, first at {np.flatnonzero(~ok)[:5]}"


@needs_ref
@pytest.mark.parametrize("kind,m", [km for km in LUT_FILES if km[0] != "ACC"])
def test_lut_product_equals_reference_model(kind, m):
    """The LUT simulation fed the reference's LUT file must be bit-equal to the
    reference's functional model over the whole FP32 domain."""
    lut32 = cpu.expand_u8(lut_bytes(kind, m), m)
    a, b = product_domain(m, seed=200 + m)
    a, b = a.view(np.float32), b.view(np.float32)
    got = cpu.lut_mul_array(lut32, m, a, b)
    want = cpu.ref_model_array(kind, m, a, b)
    ok = same_bits_or_both_nan(got, want)
    assert ok.all(), f"{(~ok).sum()} mismatches, first at {np.flatnonzero(~ok)[:5]}"


@pytest.mark.parametrize("kind,m", [km for km in LUT_FILES if km[0] != "ACC"])
def test_lut_product_equals_oracle_model(kind, m):
    # same statement against the oracle's restated models (runs without _ref)
    lut32 = cpu.expand_u8(lut_bytes(kind, m), m)
    a, b = product_domain(m, seed=300 + m, reps=1)
    a, b = a.view(np.float32), b.view(np.float32)
    ok = same_bits_or_both_nan(cpu.lut_mul_array(lut32, m, a, b), cpu.model_array(kind, m, a, b))
    assert ok.all()


def test_acc_lut_product_equals_bf16_model_on_normal_range():
    # the bf16-truncate model keeps subnormal products, the LUT simulation
    # flushes them; compare where both operands and the product are normal
    lut32 = cpu.expand_u8(lut_bytes("ACC", 7), 7)
    rng = np.random.default_rng(5)
    a = rng.standard_normal(200000).astype(np.float32) * np.float32(2.0) ** rng.integers(-40, 40, 200000)
    b = rng.standard_normal(200000).astype(np.float32) * np.float32(2.0) ** rng.integers(-40, 40, 200000)
    got = cpu.lut_mul_array(lut32, 7, a.astype(np.float32), b.astype(np.float32))
    want = cpu.model_array("ACC", 7, a.astype(np.float32), b.astype(np.float32))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("kind", ["MBM", "MIT"])
def test_lutgen32_matches_u8_expansion_and_extends_to_11(kind):
    for m in (1, 3, 5, 7):
        assert np.array_equal(cpu.lutgen32(kind, m), cpu.expand_u8(lut_bytes(kind, m), m))
    t = cpu.lutgen32(kind, 11).reshape(2048, 2048)
    assert np.array_equal(t, t.T)
    if kind == "MIT":  # closed form holds for every m
        i, j = np.meshgrid(np.arange(2048, dtype=np.uint32), np.arange(2048, dtype=np.uint32), indexing="ij")
        s = i + j
        assert np.array_equal(t, ((s >> 11) << 23) | ((s & 2047) << 12))


def test_oracle_lut_product_against_reference_model_vectors(golden_dir):
    """Golden vectors written by the reference's compiled models; pins the
    oracle where oracle/_ref is not available (e.g. on the GPU box)."""
    data = np.load(os.path.join(golden_dir, "product_vectors.npz"), allow_pickle=False)
    for kind, m in LUT_FILES:
        if kind == "ACC":
            continue
        a, b, want = data[f"{kind}_{m}_a"], data[f"{kind}_{m}_b"], data[f"{kind}_{m}_out"]
        lut32 = cpu.expand_u8(lut_bytes(kind, m), m)
        got = cpu.lut_mul_array(lut32, m, a.view(np.float32), b.view(np.float32))
        assert same_bits_or_both_nan(got, want.view(np.float32)).all()
        got = cpu.model_array(kind, m, a.view(np.float32), b.view(np.float32))
        assert same_bits_or_both_nan(got, want.view(np.float32)).all()
