"""CPU-only checks of the C-ABI library: it loads, exports every symbol the header declares, the
host-side pieces (bit-width rule, argument validation, workspace sizing) behave, and the Python
package refuses to run without it.  No kernel is launched here."""
import ctypes as C
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "niti_gfx950.h")


@pytest.fixture(scope="module")
def lib():
    from niti_amd import _lib
    if not os.path.exists(_lib.SO_PATH):
        from niti_amd import build
        build.build()
    return _lib.lib()


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(niti_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound(lib):
    from niti_amd import _lib
    names = declared_symbols()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), "library does not export " + n
        assert n in _lib.SIGNATURES, "ctypes signature table misses " + n
    assert sorted(_lib.SIGNATURES) == names, "signature table lists symbols the header does not declare"


def test_header_cites_the_reference_interfaces():
    text = open(HEADER).read()
    for cite in ("cutlassconv.cpp:57-73", "int8mm.cpp:9-14", "int8pool.cpp:37-57", "int8conv.cpp:35-44",
                 "ti_torch.py:103-147", "ti_torch.py:16-21", "ti_torch.py:403-405", "ti_torch.py:430-432"):
        assert cite in text, cite


def test_version_and_status_strings(lib):
    assert lib.niti_version() >= 100
    assert lib.niti_status_string(0) == b"ok"
    assert b"invalid" in lib.niti_status_string(1)
    assert lib.niti_status_string(99) == b"unknown status"


def test_bitwidth_rule_matches_the_oracle(lib, kat):
    from oracle import niti_oracle as po
    for r, bw in kat["bitwidth_int"].items():
        assert lib.niti_bitwidth(int(r), 0) == bw
    for r, bw in kat["bitwidth_f32"].items():
        assert lib.niti_bitwidth(int(r), 1) == bw
    for k in range(1, 31):
        for d in range(-3, 12):
            r = 2 ** k + d
            if r < 0:
                continue
            assert lib.niti_bitwidth(r, 0) == po.bitwidth_int(r), r
            assert lib.niti_bitwidth(r, 1) == po.bitwidth_f32(r), r     # torch CPU log2, literal reference form


def test_argument_validation_without_a_gpu(lib):
    from niti_amd import _lib
    null = None
    # null pointers / bad extents are rejected before any HIP call
    st = lib.niti_conv2d_i8_fprop(null, null, null, 1, 8, 8, 16, 16, 3, 3, 1, 1, 0, null, null, 0, null)
    assert st == 1 and b"null" in lib.niti_last_error()
    st = lib.niti_conv2d_i8_fprop(null, null, null, 0, 8, 8, 16, 16, 3, 3, 1, 1, 0, null, null, 0, null)
    assert st == 1
    buf = (C.c_char * 4096)()
    p = C.addressof(buf) + (-C.addressof(buf)) % 16
    st = lib.niti_conv2d_i8_fprop(p, p, p, 1, 4, 4, 3, 4, 3, 3, 1, 1, 0, null, null, 0, null)      # C not a multiple of 16
    assert st == 2 and b"multiple of 16" in lib.niti_last_error()
    st = lib.niti_conv2d_i8_fprop(p + 1, p, p, 1, 4, 4, 16, 4, 3, 3, 1, 1, 0, null, null, 0, null)  # misaligned
    assert st == 1 and b"aligned" in lib.niti_last_error()
    st = lib.niti_conv2d_i8_dgrad(p, p, p, 1, 4, 4, 16, 16, 3, 3, 2, 1, 0, null, p, 4096, null)  # stride 2
    assert st == 2
    st = lib.niti_conv2d_i8_wgrad(p, p, p, 4, 8, 8, 16, 16, 3, 3, 1, 1, 0, null, null, 0, null)  # no workspace
    assert st == 3 and b"workspace" in lib.niti_last_error()
    st = lib.niti_requant_i32_i8(p, p, 16, p, 9, 0, 0, 0, null, 0, null, null, null, null, null)  # target_bits 9
    assert st == 1
    st = lib.niti_requant_i32_i8(p, p, 16, p, 7, 1, 0, 0, null, 0, null, null, null, null, null)  # sto without rand
    assert st == 1 and b"rand" in lib.niti_last_error()
    st = lib.niti_maxpool_i8_fwd(p, p, 1, 4, 4, 16, 2, 0, 0, null)                               # stride 0
    assert st == 1
    st = lib.niti_gemm_i8(0, 1, p, p, p, 0, 4, 4, 0, null, null, 0, null)
    assert st == 1
    # classifier head and the generator's words: refused before any HIP call
    st = lib.niti_head_i8_forward(p, p, p, 16, 10, 64, 3, null, null, 0, null, null, null, 7, 0, 0, 0, 0, p, 4096, null, null, null, null, null)
    assert st == 1 and b"dropout" in lib.niti_last_error()                                        # dropout mode 3
    st = lib.niti_head_i8_forward(p, p, p, 16, 10, 64, 2, p, null, 1, null, null, null, 7, 0, 0, 0, 0, p, 4096, null, null, null, null, null)
    assert st == 1 and b"generator" in lib.niti_last_error()                                      # a drawn mask without a state
    st = lib.niti_head_i8_forward(p, p, p, 16, 10, 64, 0, null, null, 0, p, null, null, 7, 0, 0, 0, 0, p, 4096, null, null, null, null, null)
    assert st == 1 and b"loss gradient" in lib.niti_last_error()                                  # targets without an output
    st = lib.niti_head_i8_forward(p, p, p, 16, 17, 64, 0, null, null, 0, null, null, null, 7, 0, 0, 0, 0, p, 4096, null, null, null, null, null)
    assert st == 2                                                                                # 17 output features
    st = lib.niti_head_i8_backward(p, p, null, p, p, 300, 10, 64, 7, 2, 5, 2, 0, 0, p, 4096, null, null, null, null, null, null, 0, null, null, null)
    assert st == 2 and b"M <= 256" in lib.niti_last_error()
    st = lib.niti_head_i8_backward(p, p, null, p, p, 16, 10, 64, 7, 1, 5, 2, 0, 0, p, 4096, null, null, null, null, null, null, 0, null, null, null)
    assert st == 2 and b"random" in lib.niti_last_error()                                         # stochastic rounding
    st = lib.niti_head_i8_backward(p, p, null, p, p, 16, 10, 64, 7, 2, 5, 2, 0, 0, p, 8, null, null, null, null, null, null, 0, null, null, null)
    assert st == 3                                                                                # too few sync words
    assert lib.niti_head_i8_sync_words(1, 16, 10, 64) > 16 and lib.niti_head_i8_sync_words(1, 16, 10, 96) == 0
    assert lib.niti_head_i8_sync_words(0, 16, 10, 64) == lib.niti_fc_i8_sync_words(0, 16, 10, 64) > 0
    assert lib.niti_rng_words_u32(null, 1, p, 4, null) == 1 and lib.niti_rng_words_u32(p, 1, null, 0, null) == 0
    assert lib.niti_loss_grad_i8_rng(p, p, p, null, p, 4, 10, 0, null) == 1 and lib.niti_loss_grad_i8(p, p, p, null, p, 4, 10, 0, null) == 1
    # the first layer's one-launch weight gradient wants its accumulation buffer behind the finishing kernel's slots
    assert lib.niti_conv2d_i8_wgrad_update_sync_words(8, 32, 32, 16, 128, 3, 3, 1, 1) >= 16 + 128 * 32
    assert lib.niti_conv2d_i8_wgrad_update_sync_words(8, 16, 16, 16, 128, 3, 3, 1, 1) < 128 * 32
    # empty inputs are fine
    assert lib.niti_absmax_i32(null, 0, null, null) == 0
    assert lib.niti_fill_u32(null, 0, 0, null) == 0
    assert lib.niti_last_error() == b""


def test_workspace_sizes(lib):
    # filter copies: flipped/transposed filter for a generic data gradient (one byte per element, rounded to
    # 256), tap-major 128 x 64 blocks for the 3x3 kernels, nothing when the kernel reads the filter as stored
    assert lib.niti_conv2d_i8_filter_workspace(2, 9, 9, 3, 10, 5, 5, 1, 2, 1) == 768
    assert lib.niti_conv2d_i8_filter_workspace(2, 9, 9, 16, 16, 5, 5, 1, 2, 0) == 0
    assert lib.niti_conv2d_i8_filter_workspace(128, 32, 32, 128, 256, 3, 3, 1, 1, 0) == 2 * 2 * 9 * 128 * 64
    assert lib.niti_conv2d_i8_filter_workspace(128, 32, 32, 128, 256, 3, 3, 1, 1, 1) == 1 * 4 * 9 * 128 * 64
    # direct GEMM form needs nothing when k is a multiple of 16
    assert lib.niti_gemm_i8_workspace(0, 1, 128, 1024, 8192) == 0
    assert lib.niti_gemm_i8_workspace(0, 1, 128, 10, 100) > 0
    # operands with a slow reduction index are read as stored when n and k are multiples of 32 (the transposed
    # first operand also needs m % 16 == 0, both transposed m % 32 == 0) ...
    # 32 tiles of 32 x 128 and 64 chunks of the reduction: split into 8 parts of int32 partial results
    assert lib.niti_gemm_i8_workspace(0, 0, 128, 1024, 8192) == 8 * 128 * 1024 * 4
    assert lib.niti_gemm_i8_workspace(1, 1, 1024, 128, 8192) == 8 * 128 * 1024 * 4
    assert lib.niti_gemm_i8_workspace(0, 0, 128, 8192, 1024) == 0     # 256 tiles: no split
    assert lib.niti_gemm_i8_workspace(0, 0, 128, 1056, 8192) == 0     # n not a multiple of 128: the 32-byte-piece kernel
    assert lib.niti_gemm_i8_workspace(1, 0, 128, 1024, 8192) == 0
    assert lib.niti_gemm_i8_workspace(1, 1, 1024, 10, 8192) == 32 * 10 * 1024 * 4   # 8 tiles: 32 parts of 2 chunks
    assert lib.niti_gemm_i8_workspace(1, 1, 1056, 10, 8192) == 0
    # ... other shapes re-lay them: b [k,n] -> [n,k16]; a [k,m] -> [m,k16]
    assert lib.niti_gemm_i8_workspace(0, 0, 128, 1000, 8192) == 1000 * 8192
    assert lib.niti_gemm_i8_workspace(1, 1, 1000, 10, 8192) == 1000 * 8192
    assert lib.niti_gemm_i8_workspace(1, 0, 120, 1024, 8192) == 120 * 8192 + 1024 * 8192
    # weight gradient: native 3x3 path = partial-sum slices, generic path = two transposed copies
    n = lib.niti_conv2d_i8_wgrad_workspace(128, 32, 32, 128, 128, 3, 3, 1)
    assert n >= 128 * 9 * 128 * 4 and n % 256 == 0
    g = lib.niti_conv2d_i8_wgrad_workspace(5, 7, 9, 40, 24, 3, 3, 1)
    assert g >= 16 * 7 * 9 * (40 + 24)
    assert lib.niti_conv2d_i8_wgrad_workspace(0, 7, 9, 40, 24, 3, 3, 1) == 0


def test_unknown_flag_bits_are_refused(lib):
    """Flag words are checked before any pointer is touched: bits the entry point does not define are an error."""
    conv = (2, 8, 8, 16, 16, 3, 3, 1, 1)      # N H W C K R S stride pad
    bad = 0x100
    calls = {
        "niti_conv2d_i8_fprop": (None, None, None) + conv + (bad, None, None, 0, None),
        "niti_conv2d_i8_dgrad": (None, None, None) + conv + (bad, None, None, 0, None),
        "niti_conv2d_i8_wgrad": (None, None, None) + conv + (bad, None, None, 0, None),
        "niti_conv2d_i8_fprop_requant": (None, None, None) + conv + (bad, 7, 0, 0, 0, 0, None, 0, None, None, None, None, None, 0, None),
        # the StoShift forms: (pooled output,) random integers behind the output, no method argument
        "niti_conv2d_i8_fprop_requant_sto": (None, None, None, None, None) + conv + (bad, 7, 0, 0, 0, None, 0, None, None, None, None, None, 0, None),
        "niti_conv2d_i8_dgrad_requant_sto": (None, None, None, None) + conv + (bad, 7, 0, 0, 0, None, None, 0, None, None, None, None, None, 0, None),
        "niti_conv2d_i8_wgrad_update": (None, None, None, 16) + conv + (bad, 5, 0, 0, 0, None, 0, None, None, None, None, None, None, None,
                                                                      None, 0, None),
        "niti_gemm_i8": (0, 1, None, None, None, 4, 4, 16, bad, None, None, 0, None),
    }
    for name, args in calls.items():
        assert getattr(lib, name)(*args) == 1, name                       # NITI_ERR_INVALID_ARG
        assert b"flags=0x100" in lib.niti_last_error(), (name, lib.niti_last_error())
    # a forward-copy flag is a data-gradient flag only
    assert lib.niti_conv2d_i8_fprop(None, None, None, *conv, 4, None, None, 0, None) == 1
    assert b"flags=0x4" in lib.niti_last_error()


def test_package_fails_loudly_without_the_library(tmp_path):
    """The product has no CPU fallback: importing the ops with the shared object missing raises."""
    code = (
        "import sys, os\n"
        "sys.path.insert(0, %r)\n"
        "from niti_amd import _lib\n"
        "_lib.SO_PATH = os.path.join(%r, 'missing.so')\n"
        "try:\n"
        "    _lib.lib()\n"
        "except ImportError as e:\n"
        "    print('ImportError', 'no fallback' in str(e))\n"
    ) % (ROOT, str(tmp_path))
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert "ImportError True" in out.stdout, out.stdout + out.stderr


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "niti_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, os.path.join(dirpath, f)


def test_bench_refuses_more_than_one_gpu():
    """One GPU per box: bench.py says so instead of starting ranks."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert out.returncode != 0 and "one GPU" in out.stderr and out.stdout.strip() == ""
