"""LUT generation: the counterpart of the reference's ``lut/lut_gen.sh`` +
``lut/lut_gen.cc`` flow (developer.md:38-86).

A table is written as ``<NAME>_<m>.bin`` (the loader takes the mantissa width
from that suffix, approx_mul_lut.h:22-25): one byte per mantissa pair
(``carry << 7 | mantissa``, lut_gen.cc:114-121) for widths up to 7, 4-byte
entries (``carry << 31 | mantissa in place``) for widths 8 to 11.

Built-in designs::

    python -m approxtrain_amd.lut_gen --multiplier MBM --mant-width 7 --out-dir lut
    python -m approxtrain_amd.lut_gen --all --out-dir lut          # the reference's nine files + ZEROS_7

Your own multiplier, written as a C function ``float f(float, float)`` in a
source or ``.inl`` file the way the reference's designs are::

    python -m approxtrain_amd.lut_gen --source my_design.inl --function my_mul \\
        --name MYMUL --mant-width 7 --out-dir lut

(the file is compiled with ``gcc -O2 -shared`` into a temporary library and
evaluated on every mantissa pair), or from an already built shared object with
``--plugin libmy.so --function my_mul``.
"""
import argparse
import ctypes as C
import os
import subprocess
import sys
import tempfile

import numpy as np

from ._lib import check, load_library

BUILTIN = ("MBM", "MIT", "ACC", "ZEROS")
# what lut/lut_gen.sh produces
REFERENCE_SET = [("MBM", 7), ("MBM", 5), ("MBM", 3), ("MBM", 1), ("MIT", 7), ("MIT", 5), ("MIT", 3), ("MIT", 1),
                 ("ACC", 7), ("ZEROS", 7)]

_FN3 = C.CFUNCTYPE(C.c_float, C.c_float, C.c_float, C.c_void_p)


def _alloc(mant_width, entry_bytes):
    if entry_bytes not in (1, 4):
        raise ValueError("entry_bytes must be 1 or 4")
    return np.zeros(1 << (2 * int(mant_width)), dtype=np.uint8 if entry_bytes == 1 else np.uint32)


def generate_builtin(name, mant_width, entry_bytes=1):
    """Entries of a built-in design (``MBM``, ``MIT``, ``ACC``, ``ZEROS``) as a numpy array."""
    out = _alloc(mant_width, entry_bytes)
    check(load_library().amsim_lut_generate_builtin(str(name).encode(), int(mant_width), int(entry_bytes),
                                                    out.ctypes.data_as(C.c_void_p), out.nbytes))
    return out


def generate_from_function(fn, mant_width, entry_bytes=1, native3=False):
    """Entries of the multiplier ``fn``: a Python callable ``(float, float) -> float`` or a
    ctypes function pointer to a C ``float f(float, float)``.  ``native3=True`` says ``fn`` is a
    C ``float f(float, float, void *)`` and is handed to the library as it is."""
    if native3:
        callee = C.cast(fn, C.c_void_p)
    else:
        if isinstance(fn, C._CFuncPtr):
            fn.restype, fn.argtypes = C.c_float, [C.c_float, C.c_float]
        # the library hands a user pointer as third argument; adapt the two-argument form
        tramp = _FN3(lambda a, b, _user: float(fn(a, b)))
        callee = C.cast(tramp, C.c_void_p)
    out = _alloc(mant_width, entry_bytes)
    check(load_library().amsim_lut_generate(callee, None, int(mant_width), int(entry_bytes),
                                            out.ctypes.data_as(C.c_void_p), out.nbytes))
    return out


def compile_multiplier(source, function, workdir):
    """Compiles a C source / .inl file holding ``float function(float, float)`` into a shared
    object (the role of ``g++ -D<NAME> lut_gen.cc`` in lut/lut_gen.sh) and returns its path."""
    wrapper = os.path.join(workdir, "amsim_user_multiplier.c")
    lib = os.path.join(workdir, "libamsim_user_multiplier.so")
    with open(wrapper, "w") as f:
        f.write('#include <stdint.h>\n#include <math.h>\n#include <string.h>\n#include "%s"\n'
                "float amsim_user_multiplier(float a, float b, void *user) { (void)user; return %s(a, b); }\n" % (os.path.abspath(source), function))
    cc = os.environ.get("CC", "gcc")
    proc = subprocess.run([cc, "-O2", "-shared", "-fPIC", "-ffp-contract=off", "-o", lib, wrapper, "-lm"],
                          capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("compiling %s failed:\n%s" % (source, proc.stderr))
    return lib


def load_plugin(path, function):
    lib = C.CDLL(os.path.abspath(path))
    try:
        return getattr(lib, function)
    except AttributeError:
        raise ValueError("%s exports no function '%s'" % (path, function)) from None


def file_entry_bytes(mant_width):
    """Entry size of a table file: what ``amsim_lut_load_file`` expects for that width."""
    return 1 if mant_width <= 7 else 4


def write_table(entries, name, mant_width, out_dir="."):
    if entries.dtype.itemsize != file_entry_bytes(mant_width):
        raise ValueError("a width-%d table file holds %d-byte entries" % (mant_width, file_entry_bytes(mant_width)))
    os.makedirs(out_dir, exist_ok=True)
    path = os.path.join(out_dir, "%s_%d.bin" % (name, mant_width))
    entries.tofile(path)
    return path


def main(argv=None):
    ap = argparse.ArgumentParser(prog="python -m approxtrain_amd.lut_gen", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--multiplier", choices=BUILTIN, help="built-in design")
    ap.add_argument("--all", action="store_true", help="every table lut/lut_gen.sh makes")
    ap.add_argument("--source", help="C source / .inl file with your multiplier")
    ap.add_argument("--plugin", help="shared object with your multiplier")
    ap.add_argument("--function", help="name of float f(float, float) in --source / --plugin")
    ap.add_argument("--name", help="file name prefix for --source / --plugin tables")
    ap.add_argument("--mant-width", type=int, default=7)
    ap.add_argument("--out-dir", default=".")
    args = ap.parse_args(argv)

    written = []
    if args.all:
        for name, m in REFERENCE_SET:
            written.append(write_table(generate_builtin(name, m), name, m, args.out_dir))
    elif args.multiplier:
        written.append(write_table(generate_builtin(args.multiplier, args.mant_width, file_entry_bytes(args.mant_width)),
                                   args.multiplier, args.mant_width, args.out_dir))
    elif args.source or args.plugin:
        if not args.function or not args.name:
            ap.error("--source / --plugin need --function and --name")
        with tempfile.TemporaryDirectory() as tmp:
            so = compile_multiplier(args.source, args.function, tmp) if args.source else args.plugin
            fn = load_plugin(so, "amsim_user_multiplier" if args.source else args.function)
            entries = generate_from_function(fn, args.mant_width, file_entry_bytes(args.mant_width), native3=bool(args.source))
        written.append(write_table(entries, args.name, args.mant_width, args.out_dir))
    else:
        ap.error("one of --multiplier, --all, --source, --plugin is required")
    for p in written:
        print(p)
    return 0


if __name__ == "__main__":
    sys.exit(main())
