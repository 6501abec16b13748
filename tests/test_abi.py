"""The C-ABI library without a GPU: it loads, exports every symbol include/tdh.h declares,
refuses compute calls before tdh_init, and the Python descriptors match the C structs."""
import ctypes as C
import importlib
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def pkg():
    return importlib.import_module("tiny-cnn_amd")


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "tdh.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tdh_[a-z0-9_]+)\s*\(", text)))


def test_library_is_built_and_loads(pkg):
    assert os.path.exists(pkg.LIB_PATH), "libtdh.so missing: run __graft_entry__.build()"
    assert pkg.lib().tdh_version().decode().startswith("tdh")


def test_every_declared_symbol_is_exported(pkg):
    names = declared_symbols()
    assert len(names) > 40
    lib = pkg.lib()
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared in include/tdh.h but not exported: {missing}"


def test_library_holds_gfx950_code(pkg):
    out = subprocess.run(["strings", "-n", "6", pkg.LIB_PATH], capture_output=True, text=True).stdout
    assert "gfx950" in out


def test_compute_before_init_is_refused(pkg):
    lib = pkg.lib()
    d = pkg.conv_desc(8, 8, 1, 3, 3, 1)
    # a fresh process has not called tdh_init; if another test did, this check is moot
    if getattr(pkg, "_inited", False):
        pytest.skip("device already initialised in this process")
    assert lib.tdh_conv2d_fwd(C.byref(d), 1, None, None, None, None) == -3
    assert b"tdh_init" in lib.tdh_last_error()
    assert lib.tdh_sync() == -3
    p = C.c_void_p()
    assert lib.tdh_malloc(C.byref(p), C.c_size_t(16)) == -3


def test_struct_layouts_match_header(pkg):
    # 12 int32 + pointer; 9 int32; int32 + 8 floats
    assert C.sizeof(pkg.ConvDesc) == 56
    assert C.sizeof(pkg.PoolDesc) == 36
    assert C.sizeof(pkg.OptDesc) == 36
    assert pkg.ConvDesc.tbl.offset == 48
    src = r'''
    #include <stdio.h>
    #include <stddef.h>
    #include "tdh.h"
    int main(void) {
      printf("%zu %zu %zu %zu %zu %zu %zu\n", sizeof(tdh_conv_desc), sizeof(tdh_pool_desc),
             sizeof(tdh_opt), sizeof(tdh_layer), offsetof(tdh_layer, conv),
             offsetof(tdh_layer, pool), offsetof(tdh_layer, fc_in));
      return 0;
    }'''
    import tempfile
    with tempfile.TemporaryDirectory() as tmp:
        open(os.path.join(tmp, "s.c"), "w").write(src)
        subprocess.run(["gcc", "-std=c99", "-I", os.path.join(ROOT, "include"), "-o",
                        os.path.join(tmp, "s"), os.path.join(tmp, "s.c")], check=True)
        got = [int(v) for v in subprocess.run([os.path.join(tmp, "s")], capture_output=True,
                                              text=True).stdout.split()]
    want = [C.sizeof(pkg.ConvDesc), C.sizeof(pkg.PoolDesc), C.sizeof(pkg.OptDesc),
            C.sizeof(pkg.LayerDesc), pkg.LayerDesc.conv.offset, pkg.LayerDesc.pool.offset,
            pkg.LayerDesc.fc_in.offset]
    assert got == want


def test_header_is_plain_c(pkg):
    """No HIP or C++ types cross the boundary: the header compiles as C99 on its own."""
    r = subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Werror", "-fsyntax-only", "-x",
                        "c", os.path.join(ROOT, "include", "tdh.h")], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


def test_optimizer_defaults_match_reference_constructors(pkg):
    o = pkg.opt_desc("adam")
    assert (round(o.alpha, 6), round(o.b1, 6), round(o.b2, 6)) == (0.001, 0.9, 0.999)
    assert (round(o.b1_t, 6), round(o.b2_t, 6)) == (0.9, 0.999) and abs(o.eps - 1e-8) < 1e-12
    o = pkg.opt_desc("momentum")
    assert (round(o.alpha, 6), round(o.mu, 6), o.lam) == (0.01, 0.9, 0.0)
    o = pkg.opt_desc("sgd")
    assert (round(o.alpha, 6), o.lam) == (0.01, 0.0)


def test_shape_helpers_match_reference_formulas(pkg):
    # conv_out_length / pool_out_length, tiny_dnn/util/util.h:329-363
    d = pkg.conv_desc(5, 5, 1, 3, 3, 1, w_stride=2, h_stride=2)
    assert pkg.conv_out_shape(d) == (2, 2)
    d = pkg.conv_desc(32, 32, 3, 5, 5, 32, pad_same=True)
    assert pkg.conv_out_shape(d) == (32, 32)
    d = pkg.conv_desc(7, 7, 1, 3, 3, 1, w_dilation=2, h_dilation=2)
    assert pkg.conv_out_shape(d) == (3, 3)
    assert pkg.pool_out_shape(pkg.pool_desc(4, 4, 1, 2, 1, 2, 1)) == (2, 4)
    assert pkg.pool_out_shape(pkg.pool_desc(7, 7, 1, 2, ceil_mode=True)) == (4, 4)
    assert pkg.pool_out_shape(pkg.pool_desc(7, 7, 1, 2)) == (3, 3)
    assert pkg.pool_out_shape(pkg.pool_desc(4, 4, 1, 2, 2, 1, 1, pad_same=True)) == (4, 4)


def test_host_mirror_header_compiles_and_fails_loudly_without_gpu(tmp_path):
    """The C++ mirror of the reference's operator interface is plain C++14 over include/tdh.h;
    without a GPU its operators throw nn_error instead of computing anything on the host."""
    import subprocess

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = tmp_path / "probe.cpp"
    src.write_text(
        '#include "tiny_dnn_hip.h"\n'
        "#include <cstdio>\n"
        "using namespace tiny_dnn;\n"
        "int main() {\n"
        "  static_assert(static_cast<int>(core::backend_t::hip) == 7, \"hip follows intel_mkl\");\n"
        "  fully_connected_layer l(4, 2);\n"
        "  tensor_t in{{0, 1, 2, 3}}, w{vec_t(8, 1.f)}, b{vec_t(2, .5f)}, out{vec_t(2)};\n"
        "  std::vector<tensor_t *> i{&in, &w, &b}, o{&out};\n"
        "  try { l.forward_propagation(i, o); } catch (const nn_error &e) { std::puts(e.what()); return 42; }\n"
        "  return 0;\n"
        "}\n")
    exe = tmp_path / "probe"
    libdir = os.path.join(root, "tiny-cnn_amd", "lib")
    r = subprocess.run(["g++", "-std=c++14", "-Wall", "-Werror", "-I", os.path.join(root, "include"),
                        "-I", os.path.join(root, "tiny-cnn_amd", "host"), str(src), "-o", str(exe),
                        "-L", libdir, "-ltdh", "-Wl,-rpath," + libdir], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    import torch
    if torch.cuda.is_available():
        return
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert r.returncode == 42 and "tdh:" in r.stdout, (r.returncode, r.stdout, r.stderr)
