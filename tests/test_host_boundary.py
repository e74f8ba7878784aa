"""CPU-only checks of the drop-in boundary and the host logic: the C-ABI
library loads and exports every symbol include/amsim.h declares, the geometry
helper matches TensorFlow's VALID/SAME closed form, status plumbing works, and
the Python wrappers validate arguments like the reference's wrappers do.  No
kernel is launched."""
import ctypes as C
import os
import re

import pytest
import torch

import approxtrain_amd
from approxtrain_amd import _lib
from tests.util import tf_same_pads

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(header="amsim.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(amsim_[a-z0-9_]+)\s*\(", text)))


BENCH_ONLY = {"amsim_microbench", "amsim_microbench_wide", "amsim_calibration_copy", "amsim_gemm_plan_info",
              "amsim_lut_force_gather_zeroing"}


def test_library_loads_and_exports_every_declared_symbol():
    lib = approxtrain_amd.load_library()
    names = declared_symbols()
    assert len(names) >= 25
    # measurement and tuning helpers live in their own header: the product header declares only
    # what an op kernel would call
    bench = declared_symbols("amsim_bench.h")
    assert set(bench) == BENCH_ONLY and not BENCH_ONLY & set(names)
    for n in names + bench:
        assert hasattr(lib, n), f"libamsim.so lacks {n}"
    # and the Python binding table covers the same set
    assert sorted(_lib.SIGNATURES) == sorted(names + bench)


def test_header_is_plain_c_and_links_from_c(tmp_path):
    """include/amsim.h must be usable from C (the boundary is a C ABI, not a C++ one): a C99
    program that includes it compiles without warnings, links against libamsim.so and can call
    an entry point that needs no device."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    src = tmp_path / "use_amsim.c"
    src.write_text(
        '#include <stdio.h>\n#include "amsim.h"\n'
        "int main(void) {\n"
        "  int out = 0, pad = 0;\n"
        "  if (amsim_conv_geometry(56, 3, 1, AMSIM_PADDING_SAME, &out, &pad) != AMSIM_OK) return 1;\n"
        "  if (amsim_lut_mant_width((amsim_lut_t)0) != -1) return 2;\n"
        "  if (amsim_conv_geometry(56, 3, 1, 99, &out, &pad) == AMSIM_OK) return 3;\n"
        '  printf("%d %d %s\\n", out, pad, amsim_last_error());\n'
        "  return 0;\n}\n")
    exe = tmp_path / "use_amsim"
    libdir = os.path.dirname(_lib.lib_path())
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"),
                    str(src), "-L", libdir, "-lamsim", "-Wl,-rpath," + libdir, "-o", str(exe)], check=True)
    run = subprocess.run([str(exe)], capture_output=True, text=True)
    assert run.returncode == 0, run.stderr
    assert run.stdout.startswith("56 1 padding must be")


@pytest.mark.parametrize("mask_shape", [(2, 1, 1, 7), (5, 7), (1, 7), (2, 1, 5, 7), (2, 3, 5, 7), (1, 3, 1, 7),
                                        (2, 3, 1, 7), (1, 1, 5, 1), (7,)])
def test_attention_mask_layout_addresses_the_broadcast_mask(mask_shape):
    """The (divisor, batch stride, row stride) triple handed to the library must address exactly
    the element that numpy broadcasting picks, for every (item, query, key)."""
    import numpy as np
    from approxtrain_amd.functors import _mask_layout
    lead, sq, sk = (2, 3), 5, 7
    mask = torch.arange(int(np.prod(mask_shape)), dtype=torch.float32).reshape(mask_shape) + 1.0
    keep, _, div, bstride, rstride = _mask_layout(mask, lead, sq, sk, torch.device("cpu"))
    flat = keep.reshape(-1).numpy()
    want = np.broadcast_to(mask.numpy(), lead + (sq, sk)).reshape(-1, sq, sk)
    for b in range(want.shape[0]):
        for r in range(sq):
            base = (b // div) * bstride + r * rstride
            assert np.array_equal(flat[base:base + sk], want[b, r]), (b, r)


def test_attention_mask_layout_rejects_shapes_that_do_not_broadcast():
    from approxtrain_amd.functors import _mask_layout
    with pytest.raises(ValueError):
        _mask_layout(torch.zeros(2, 4, 7), (2, 3), 5, 7, torch.device("cpu"))
    with pytest.raises(ValueError):
        _mask_layout(torch.zeros(2, 3, 5, 7, 1), (2, 3), 5, 7, torch.device("cpu"))


def test_no_entry_point_crashes_on_null_or_odd_arguments():
    """Every compute entry point called with a null LUT handle, null tensors and extents of
    0 / 1 / -1 / 7 must come back with a status (no launch, no crash), and every workspace query
    with a size (0 for impossible extents)."""
    lib = approxtrain_amd.load_library()
    other = {"amsim_status_string", "amsim_last_error", "amsim_device_info", "amsim_lut_load_file", "amsim_lut_create",
             "amsim_lut_destroy", "amsim_lut_mant_width", "amsim_lut_params", "amsim_lut_generate",
             "amsim_lut_generate_builtin", "amsim_microbench", "amsim_calibration_copy", "amsim_set_split_k", "amsim_set_engine",
             "amsim_conv_geometry", "amsim_gemm_plan_info"}
    for name, (res, args) in _lib.SIGNATURES.items():
        if name in other:
            continue
        for fill in (0, 1, -1, 7):
            vals = []
            for a in args:
                if a is C.c_size_t:
                    vals.append(max(fill, 0))
                elif a in (C.c_int, C.c_int64):
                    vals.append(fill)
                elif a is C.c_float:
                    vals.append(1.0)
                else:
                    vals.append(None)
            out = getattr(lib, name)(*vals)
            if name.endswith("_workspace_bytes") or name.endswith("_workspace_bytes_for"):
                assert out >= 0 and (fill > 0 or out == 0), (name, fill, out)
            else:
                assert out == 1, (name, fill, out)                      # AMSIM_ERR_INVALID: nothing was launched
                assert lib.amsim_last_error(), name


def test_tensorflow_bridge_uses_only_declared_entry_points():
    """The TensorFlow bridge cannot be compiled here (no TensorFlow); at least every C-ABI
    call in it must name an entry point the header declares, and every GPU functor of the
    reference must be defined and instantiated in it."""
    text = open(os.path.join(ROOT, "approxtrain_amd", "tf_bridge", "amsim_tf_bridge.cc")).read()
    code = re.sub(r"//.*", "", text)
    used = set(re.findall(r"\b(amsim_[a-z0-9_]+)\s*\(", code))
    assert used and used <= set(declared_symbols()), used - set(declared_symbols())
    for functor in ("ConvamFunctor", "ConvamInputGradFunctor", "ConvamFilterGradFunctor", "DenseamFunctor",
                    "DenseamWeightGradFunctor", "DenseamInputGradFunctor", "LaunchMatMul"):
        assert re.search(r"void %s<GPUDevice, T>::operator\(\)" % functor, code), functor
        for t in ("float", "int32"):
            assert "template struct %s<GPUDevice, %s>;" % (functor, t) in code, (functor, t)


def test_status_strings():
    lib = approxtrain_amd.load_library()
    assert lib.amsim_status_string(0) == b"ok"
    assert b"workspace" in lib.amsim_status_string(5)


@pytest.mark.parametrize("i,k,s", [(56, 3, 1), (28, 5, 1), (14, 5, 1), (5, 3, 2), (20, 5, 2), (4, 4, 1), (8, 1, 2),
                                   (7, 3, 3), (32, 5, 2)])
def test_conv_geometry_matches_tensorflow_closed_form(i, k, s):
    o, p = _lib.conv_geometry(i, k, s, "SAME")
    oo, pb, _ = tf_same_pads(i, k, s)
    assert (o, p) == (oo, pb)
    o, p = _lib.conv_geometry(i, k, s, "VALID")
    assert (o, p) == (max((i - k + s) // s, 0), 0)


def test_conv_geometry_rejects_bad_padding():
    lib = approxtrain_amd.load_library()
    o, p = C.c_int(), C.c_int()
    assert lib.amsim_conv_geometry(8, 3, 1, 7, C.byref(o), C.byref(p)) == 1
    assert b"padding" in lib.amsim_last_error()


def test_lut_file_name_errors_do_not_exit(tmp_path):
    """The reference exits the process on LUT problems (approx_mul_lut.h:18-40);
    the library returns a status."""
    lib = approxtrain_amd.load_library()
    h = C.c_void_p()
    assert lib.amsim_lut_load_file(b"", C.byref(h)) == 1
    assert lib.amsim_lut_load_file(b"/nonexistent/MBM_7.bin", C.byref(h)) == 2          # I/O
    assert lib.amsim_lut_load_file(b"/nonexistent/nosuffix.bin", C.byref(h)) == 3       # no _<m>
    assert lib.amsim_lut_load_file(b"/nonexistent/MBM_x7.bin", C.byref(h)) == 3        # width not a number
    assert lib.amsim_lut_load_file(b"/nonexistent/MBM_12.bin", C.byref(h)) == 3        # widths stop at 11
    assert lib.amsim_lut_load_file(b"/nonexistent/MBM_9.bin", C.byref(h)) == 2         # 8..11: 4-byte entries; I/O
    short = tmp_path / "MBM_7.bin"
    short.write_bytes(b"\x00" * 100)
    assert lib.amsim_lut_load_file(str(short).encode(), C.byref(h)) == 3               # short file
    assert not h.value


def test_workspace_queries_need_no_device():
    lib = approxtrain_amd.load_library()
    assert lib.amsim_gemm_workspace_bytes(0, 0, 4096, 4096, 4096, 1) > 0
    assert lib.amsim_convam_workspace_bytes(32, 56, 56, 64, 3, 3, 64) > 0
    assert lib.amsim_convam_filter_grad_workspace_bytes(32, 56, 56, 64, 3, 3, 64) > 0
    assert lib.amsim_gemm_workspace_bytes(0, 0, 0, 5, 5, 1) == 0
    assert lib.amsim_matmulam_workspace_bytes(2, 3, 4, 5, 5, 6) == 0  # incompatible batches


def test_planner_invariants_over_random_shapes():
    """The work-shaping plan of the LDS-table engine (host code, no device needed): over random
    problem shapes the reduction slices of the main part and of the tail cover every chunk with no
    empty slice, a tail leaves whole tiles to the main part, and the arrangement that deals a
    chunk's rows out to the four wavefronts is only used with 16-column tiles."""
    import random
    lib = approxtrain_amd.load_library()
    info = (C.c_int64 * 8)()
    rnd = random.Random(3)
    slices = 0
    for _ in range(30000):
        M = rnd.choice([rnd.randint(1, 300), rnd.randint(1, 70000), rnd.randint(1, 300000)])
        N = rnd.choice([rnd.randint(1, 20), rnd.randint(1, 600), rnd.randint(1, 5000)])
        K = rnd.choice([rnd.randint(1, 100), rnd.randint(1, 5000), rnd.randint(1, 200000)])
        batch = rnd.choice([1, 1, 1, 2, 7, 256])
        assert lib.amsim_gemm_plan_info(0, 0, M, N, K, batch, info) == 0
        TN, WR, nsplit, cps, rows_main, tail_nsplit, tail_cps, chunks = list(info)
        shape = (M, N, K, batch, list(info))
        assert TN in (1, 2, 4, 8, 16) and WR in (0, 1, 4), shape
        assert nsplit >= 1 and cps >= 1 and nsplit * cps >= chunks > (nsplit - 1) * cps, shape
        if tail_nsplit:
            assert tail_nsplit * tail_cps >= chunks > (tail_nsplit - 1) * tail_cps, shape
            assert rows_main > 0 and rows_main % (64 * max(WR, 1)) == 0, shape
        if WR == 0:
            slices += 1
            assert TN == 16, shape
    assert slices > 0


def test_functors_refuse_host_tensors():
    from approxtrain_amd import functors
    with pytest.raises(TypeError, match="device memory"):
        functors.gemm("x_7.bin", torch.zeros(2, 2), torch.zeros(2, 2))


def test_amconvolution_argument_validation():
    from approxtrain_amd.amnn_ops import _get_sequence, amconvolution_v2
    x, w = torch.zeros(1, 4, 4, 2), torch.zeros(3, 3, 2, 5)
    assert _get_sequence(2, 2, 3, "strides") == [1, 2, 2, 1]
    assert _get_sequence([2, 3], 2, 3, "strides") == [1, 2, 3, 1]
    assert _get_sequence(None, 2, 3, "strides") == [1, 1, 1, 1]
    with pytest.raises(ValueError):
        _get_sequence([1, 2, 3], 2, 3, "strides")
    with pytest.raises(ValueError, match="Dilation is not supported"):
        amconvolution_v2(x, w, dilations=[1, 2, 2, 1], mant_mul_lut="MBM_7.bin")
    with pytest.raises(ValueError, match="mant_mul_lut"):
        amconvolution_v2(x, w)
    with pytest.raises(ValueError, match="depth"):
        amconvolution_v2(x, torch.zeros(3, 3, 3, 5), mant_mul_lut="MBM_7.bin")
    with pytest.raises(ValueError):
        amconvolution_v2(x, w, data_format="NCHW", mant_mul_lut="MBM_7.bin")


def test_matmulam_argument_validation():
    from approxtrain_amd.math_ops import matmulam
    a, b = torch.zeros(2, 3), torch.zeros(3, 4)
    with pytest.raises(ValueError, match="unsupported args"):
        matmulam(a, b, adjoint_a=True, mant_mul_lut="MBM_7.bin")
    with pytest.raises(ValueError, match="mant_mul_lut"):
        matmulam(a, b)


def test_layers_validate_constructor_arguments():
    from approxtrain_amd.layers import AMConv2D, denseam
    with pytest.raises(ValueError):
        AMConv2D(8, 3, mant_mul_lut="")
    with pytest.raises(ValueError, match="Dilation"):
        AMConv2D(8, 3, dilation_rate=2, mant_mul_lut="MBM_7.bin")
    with pytest.raises(ValueError):
        denseam(8)
    layer = AMConv2D(6, 5, padding="same", mant_mul_lut="MBM_7.bin", in_channels=1)
    assert tuple(layer.kernel.shape) == (5, 5, 1, 6) and layer.get_config()["mant_mul_lut"] == "MBM_7.bin"
    d = denseam(300, mant_mul_lut="MBM_7.bin", input_dim=784)
    assert tuple(d.kernel.shape) == (784, 300)


def test_layers_take_the_keras_constructor_vocabulary():
    """am_convolutional.py:519-558 / amdenselayer.py:93-126: initializers and activations by
    name, regularizers, constraints, name / input_shape / trainable; what the approximate op
    cannot do is refused with a message (channels_first, groups, causal padding)."""
    import math
    from approxtrain_amd.layers import AMConv2D, denseam
    lut = "MBM_7.bin"
    torch.manual_seed(0)
    c = AMConv2D(64, (3, 3), strides=2, padding="same", data_format="channels_last", activation="relu",
                 kernel_initializer="he_normal", bias_initializer="ones", kernel_regularizer=lambda w: (w * w).sum(),
                 kernel_constraint=lambda w: w.clamp(-0.01, 0.01), mant_mul_lut=lut, input_shape=(56, 56, 64), name="conv")
    assert tuple(c.kernel.shape) == (3, 3, 64, 64) and c.layer_name == "conv" and c.activation is torch.relu
    assert abs(float(c.kernel.detach().std()) - math.sqrt(2.0 / 576)) < 0.1 * math.sqrt(2.0 / 576)
    assert float(c.kernel.detach().abs().max()) <= 2.0 * math.sqrt(2.0 / 576) / 0.8796 + 1e-6   # truncated at two sigma
    assert torch.equal(c.bias.detach(), torch.ones(64))
    assert len(c.losses()) == 1 and float(c.losses()[0].detach()) == pytest.approx(float((c.kernel.detach() ** 2).sum()))
    c.apply_constraints()
    assert float(c.kernel.detach().abs().max()) <= 0.01
    d = denseam(10, activation="softmax", kernel_initializer="glorot_uniform", bias_regularizer=lambda b: b.abs().sum(),
                mant_mul_lut=lut, input_dim=300, trainable=False)
    assert float(d.kernel.detach().abs().max()) <= math.sqrt(6.0 / 310) and not d.kernel.requires_grad
    assert callable(d.activation) and torch.allclose(d.activation(torch.zeros(2, 4)), torch.full((2, 4), 0.25))
    custom = denseam(3, kernel_initializer=lambda shape: torch.full(shape, 0.5), mant_mul_lut=lut, input_dim=2)
    assert torch.equal(custom.kernel.detach(), torch.full((2, 3), 0.5))
    for bad in (dict(data_format="channels_first"), dict(groups=2), dict(padding="causal"), dict(activation="nope"),
                dict(kernel_initializer="nope", in_channels=3), dict(kernel_regularizer=0.1), dict(dtype="float16")):
        with pytest.raises(ValueError):
            AMConv2D(8, 3, mant_mul_lut=lut, **bad)
    with pytest.raises(TypeError, match="not understood"):
        AMConv2D(8, 3, mant_mul_lut=lut, kernel_size2=3)
    with pytest.raises(ValueError):
        denseam(8, activation="nope", mant_mul_lut=lut)
