"""CPU-side checks of the drop-in boundary: the shared object loads, exports every symbol that
include/int64gemm.h declares, and its host-only table initialisers reproduce the tables the reference's
circuits hold.  Nothing here launches a kernel."""
import ctypes
import os
import re
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "zk-deepseek_amd", "libint64gemm.so")
HEADER = os.path.join(ROOT, "include", "int64gemm.h")

# the 19 symbols whose .argtypes the reference touches at import (inference/kernel.py:209-338):
# a missing one makes `import kernel` raise AttributeError there
REFERENCE_BOUND = [
    "int64_64_bmm_broadcast_launcher", "int64_32_bmm_broadcast_launcher", "complex_int64_mul",
    "rms_norm_32", "rms_norm_64", "einsum_bshd_hdc_bshc", "einsum_bshc_btc_bsht", "einsum_bsht_btc_bshc",
    "einsum_bshc_hdc_bshd", "softmax_q21", "softmax_q19", "softmax_init_q21", "softmax_init_q19",
    "silu_q25", "sigmoid_q25", "silu_init_q25", "silu_q23", "sigmoid_q23", "silu_init_q23",
]


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        import sys
        sys.path.insert(0, os.path.join(ROOT, "zk-deepseek_amd"))
        import build
        build.build(verbose=False)
    return ctypes.CDLL(LIB)


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"^\s*(?:const\s+)?(?:void|int|long|float|double|char)\s*\*?\s*(\w+)\s*\(", text, flags=re.M)


def test_header_declares_reference_abi():
    names = declared_functions()
    assert len(names) == len(set(names))
    for n in REFERENCE_BOUND + ["bf16_to_int32_2d", "wkv_b_bf16_to_int32", "float32_to_int64_2d"]:
        assert n in names, n


def test_library_exports_every_declared_symbol(lib):
    for n in declared_functions():
        assert hasattr(lib, n), n


def test_table_initialisers_match_reference_tables(lib, zk_tables, oracle):
    def table(fn):
        buf = np.zeros(256, np.int64)
        fn(ctypes.c_void_p(buf.ctypes.data))
        return buf
    assert table(lib.softmax_init_q19).tolist() == zk_tables["q19Table"]
    assert table(lib.silu_init_q23).tolist() == zk_tables["q23Table"]
    assert np.array_equal(table(lib.softmax_init_q21), oracle.softmax_init_q21())
    assert np.array_equal(table(lib.silu_init_q25), oracle.silu_init_q25())


def test_error_channel_starts_clean(lib):
    lib.zk_clear_error()
    assert lib.zk_last_error() == 0


def test_kernel_module_mirrors_reference_api():
    """names model.py imports from kernel (inference/model.py:13-15) plus the wrappers of kernel.py:341-688"""
    import kernel
    for n in ["act_quant", "weight_dequant", "fp8_gemm", "int64_bmm_broadcast", "complex_int64_mul_broadcast",
              "einsum_bshd_hdc_bshc", "einsum_bshc_btc_bsht", "einsum_bsht_btc_bshc", "einsum_bshc_hdc_bshd",
              "RMS_Norm_int64", "int64_RMS0", "softmax_init_q19", "softmax_init_q21", "silu_init_q23",
              "silu_init_q25", "softmax_q19", "softmax_q21", "silu_q23", "sigmoid_q23", "silu_q25",
              "sigmoid_q25", "saveTensor"]:
        assert callable(getattr(kernel, n)), n
    assert kernel.rms.shape == (500,) and kernel.rms.device.type == "cpu"
    with pytest.raises(NotImplementedError):
        kernel.fp8_gemm()


def test_dump_writer_host_path(lib, tmp_path):
    """the witness dump writer on host memory (no GPU needed): bytes identical to numpy's tobytes, large tensors go
    through in pieces, an unwritable path is reported by the flush"""
    lib.zk_dump_host.argtypes = [ctypes.c_char_p, ctypes.c_void_p, ctypes.c_size_t]
    lib.zk_dump_flush.restype = ctypes.c_long
    lib.zk_last_error_string.restype = ctypes.c_char_p
    lib.zk_clear_error()
    rng = np.random.default_rng(1)
    arrays = {"empty.bin": np.zeros(0, np.int64), "one.bin": np.array([-5], np.int64),
              "w32.bin": rng.integers(-(1 << 31), 1 << 31, size=(37, 129), dtype=np.int64).astype(np.int32),
              "big.bin": rng.integers(-(1 << 62), 1 << 62, size=(5 << 20) + 3, dtype=np.int64)}       # 40 MB: two pieces
    for name, a in arrays.items():
        assert lib.zk_dump_host(os.fsencode(str(tmp_path / name)), ctypes.c_void_p(a.ctypes.data), a.nbytes) == 0
    big = arrays["big.bin"]
    big[:] = 0                                             # the data was copied before the call returned
    assert lib.zk_dump_flush() == 0
    rng = np.random.default_rng(1)
    want = {"empty.bin": np.zeros(0, np.int64), "one.bin": np.array([-5], np.int64),
            "w32.bin": rng.integers(-(1 << 31), 1 << 31, size=(37, 129), dtype=np.int64).astype(np.int32),
            "big.bin": rng.integers(-(1 << 62), 1 << 62, size=(5 << 20) + 3, dtype=np.int64)}
    for name, a in want.items():
        assert (tmp_path / name).read_bytes() == a.tobytes(order="C"), name
    a = np.arange(4, dtype=np.int64)
    assert lib.zk_dump_host(os.fsencode(str(tmp_path / "no_such_dir" / "x.bin")), ctypes.c_void_p(a.ctypes.data), a.nbytes) == 0
    assert lib.zk_dump_flush() == 1
    assert b"no_such_dir" in lib.zk_last_error_string()
    lib.zk_clear_error()
    assert lib.zk_dump_flush() == 0


def test_header_is_plain_c_and_links(lib, tmp_path):
    """the boundary is a C ABI: the header compiles as C99 with gcc (no C++, no HIP types), and a C program that takes
    the address of every declared function links against the library and runs without a GPU"""
    import subprocess
    names = declared_functions()
    src = tmp_path / "abi.c"
    body = "".join("    keep[%d] = (fn_t)&%s;\n" % (i, n) for i, n in enumerate(names))
    src.write_text('#include "int64gemm.h"\n#include <stdio.h>\ntypedef void (*fn_t)(void);\nint main(void) {\n'
                   '    fn_t keep[%d];\n%s    printf("%%d %%d\\n", keep[0] != 0, zk_last_error());\n    return 0;\n}\n' % (len(names), body))
    exe = tmp_path / "abi"
    libdir = os.path.dirname(LIB)
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.dirname(HEADER),
                           str(src), "-o", str(exe), "-L", libdir, "-lint64gemm", "-Wl,-rpath," + libdir,
                           "-Wl,-rpath-link,/opt/rocm/lib"])
    assert subprocess.check_output([str(exe)]).decode().split() == ["1", "0"]


def test_product_never_touches_the_checker():
    """the CPU restatement under oracle/ is test infrastructure: nothing in the package names it, the library does
    not link it, and the benchmark reaches it only from its CPU-baseline leg"""
    pkg = os.path.join(ROOT, "zk-deepseek_amd")
    for dirpath, dirnames, filenames in os.walk(pkg):
        dirnames[:] = [d for d in dirnames if d not in ("__pycache__", "build")]
        for fn in filenames:
            if fn.endswith((".py", ".hip", ".h", ".cpp", ".c")):
                text = open(os.path.join(dirpath, fn), errors="replace").read().lower()
                assert "oracle" not in text, "%s names the oracle" % os.path.join(dirpath, fn)
    # the shared object carries no reference to the oracle's library or its entry points
    blob = open(LIB, "rb").read()
    assert b"libzkoracle" not in blob
    for sym in (b"ora_int64_64_bmm_broadcast", b"ora_softmax_q19", b"ora_act_q23", b"ora_rms_norm_32", b"ora_gate_route"):
        assert sym not in blob
    # bench.py: every use of the oracle sits inside cpu_leg
    src = open(os.path.join(ROOT, "bench.py")).read()
    start = src.index("def cpu_leg(")
    nxt = re.search(r"^def ", src[start + 1:], re.M)
    end = start + 1 + nxt.start() if nxt else len(src)
    outside = src[:start] + src[end:]
    assert not re.search(r"^\s*(import|from)\s+oracle\b", outside, re.M)
    assert "oracle." not in outside


def test_bench_refuses_more_than_one_gpu_and_defaults_to_one():
    """the benchmark runs on one GPU: `--gpus 2` ends with a message and a non-zero status before anything touches a
    device; with no flags it asks for one GPU and a step count that finishes in minutes"""
    bench = os.path.join(ROOT, "bench.py")
    r = subprocess.run([sys.executable, bench, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2 and "ONE GPU" in r.stderr and r.stdout.strip() == ""
    src = open(bench).read()
    m = re.search(r'add_argument\("--gpus",[^)]*default=(\d+)', src)
    assert m and int(m.group(1)) == 1
    m = re.search(r'add_argument\("--steps",[^)]*default=(\d+)', src)
    assert m and 1 <= int(m.group(1)) <= 1000
