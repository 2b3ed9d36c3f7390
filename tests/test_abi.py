"""The C-ABI library: it loads without a GPU, exports every function include/kitty_hip.h declares,
its structs have the layout the ctypes binding assumes, and arguments are rejected on the host
before anything is launched."""
import ctypes
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "kitty_hip.h")


@pytest.fixture(scope="module")
def lib():
    from kitty_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from kitty_amd import build
        build.build(verbose=False)
    return _lib.lib()


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    return sorted(set(re.findall(r"\b(kitty_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree(lib):
    from kitty_amd import _lib
    names = declared_functions()
    assert len(names) >= 10
    assert sorted(_lib.EXPORTS) == names
    for n in names:
        assert hasattr(lib, n), f"{n} declared in kitty_hip.h but not exported"
    assert lib.kitty_abi_version() == _lib.ABI_VERSION == 2


def test_struct_layout_matches_c(tmp_path):
    from kitty_amd import _lib
    fields = [f[0] for f in _lib.KittyKVLayer._fields_]
    src = tmp_path / "layout.c"
    src.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "kitty_hip.h"\nint main(void){\n'
                   'printf("%zu\\n", sizeof(kitty_kv_layer));\n'
                   + "".join(f'printf("%zu\\n", offsetof(kitty_kv_layer, {f}));\n' for f in fields)
                   + "return 0;}\n")
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), "-o", str(exe), str(src)])
    out = [int(x) for x in subprocess.check_output([str(exe)]).split()]
    assert out[0] == ctypes.sizeof(_lib.KittyKVLayer)
    assert out[1:] == [getattr(_lib.KittyKVLayer, f).offset for f in fields]


def test_host_side_rejection_without_gpu(lib):
    """Negative return codes come from host checks that run before any HIP call."""
    from kitty_amd import _lib
    E_NULL, E_SHAPE, E_RANGE, E_ALIGN, E_WORKSPACE = -1, -2, -3, -4, -5
    assert lib.kitty_quant_pack_v(None, 0, 0, 0, 1, 1, 128, 128, 0, 1, 128, None, 0, 0, None, 0, None, 0, 0, None, None) == E_NULL
    assert b"NULL" in lib.kitty_last_error()
    fake = ctypes.c_void_p(4096)
    rc = lib.kitty_quant_pack_k(fake, 256, 256, 256, 1, 1, 128, 96, 0, 1, 128, 32, None, fake, 1, 0, fake, 5248, fake, 512, 1, None, None)
    assert rc == E_SHAPE and b"head_dim 64, 128 or 256" in lib.kitty_last_error()
    # head_dim 64 is served (by the plain kernels for other head dimensions): the checks go on to the strides
    rc = lib.kitty_quant_pack_k(fake, 256, 256, 256, 1, 1, 128, 64, 0, 1, 128, 16, None, fake, 1, 0, fake, 2000, fake, 256, 1, None, None)
    assert rc == E_RANGE and b"page stride too small" in lib.kitty_last_error()
    rc = lib.kitty_quant_pack_k(fake, 512, 512, 512, 1, 1, 128, 256, 0, 1, 128, 256, None, fake, 1, 0, fake, 16640, fake, 1024, 1, None, None)
    assert rc == E_SHAPE and b"uint8 slot map" in lib.kitty_last_error()
    rc = lib.kitty_quant_pack_k(fake, 32768, 32768, 256, 1, 1, 128, 128, 64, 1, 128, 32, None, fake, 1, 0, fake, 5248, fake, 512, 1, None, None)
    assert rc == E_RANGE and b"exceed" in lib.kitty_last_error()
    rc = lib.kitty_quant_pack_k(ctypes.c_void_p(4098), 32768, 32768, 256, 1, 1, 128, 128, 0, 1, 128, 32, None, fake, 1, 0, fake, 5248, fake, 512, 1, None, None)
    assert rc == E_ALIGN
    rc = lib.kitty_select_boost_k(fake, 32768, 32768, 256, 1, 1, 128, 128, 0, 1, 128, 129, fake, None)
    assert rc == E_SHAPE
    assert lib.kitty_decode_attn(None, None, 1, 4, 0.1, None, None, 0, 1, 0, None) == E_NULL
    L = _lib.KittyKVLayer()
    L.H_KV, L.D, L.D_BOOSTED, L.PAGE_SIZE, L.S, L.MAX_PAGE = 1, 128, 32, 128, 32, 4
    for f in ("key_cache", "key_meta", "value_cache", "value_meta", "page_table_k", "page_table_v", "sink_k", "sink_v",
              "qbuf_k", "qbuf_v", "local_v"):
        setattr(L, f, 4096)
    L.key_cache_stride_page, L.value_cache_stride_page = 5248, 4096
    L.key_meta_stride_page = L.value_meta_stride_page = 512
    L.sink_stride_b = L.sink_stride_h = 8192
    L.win_stride_b = L.win_stride_h = 32768
    args = lambda hq, ws, wsb, splits, variant=0: (ctypes.byref(L), fake, 1, hq, 0.1, fake, ws, wsb, splits, variant, None)
    assert lib.kitty_decode_attn(*args(17, fake, 1 << 20, 1)) == E_SHAPE            # KV_GROUP > 16
    assert b"MAX_KV_GROUP" in lib.kitty_last_error()
    assert lib.kitty_decode_attn(*args(4, fake, 16, 4)) == E_WORKSPACE
    assert lib.kitty_decode_attn(*args(4, fake, 1 << 20, 4, variant=7)) == E_SHAPE
    L.counts[2] = 5                                                                # K and V lengths disagree
    assert lib.kitty_decode_attn(*args(4, fake, 1 << 20, 4)) == E_RANGE
    assert b"seqlen_K" in lib.kitty_last_error()
    L.counts[2] = 0
    L.D = 96
    assert lib.kitty_decode_attn(*args(4, fake, 1 << 20, 4)) == E_SHAPE
    L.D = 128
    L.cache_pages_k = -1                                                           # a negative page count
    assert lib.kitty_decode_attn(*args(4, fake, 1 << 20, 4)) == E_RANGE
    L.cache_pages_k, L.counts[1], L.counts[2] = 0, 1, 0                            # a packed page but no page array
    L.counts[5] = 128
    assert lib.kitty_decode_attn(*args(4, fake, 1 << 20, 4)) == E_RANGE and b"cache_pages" in lib.kitty_last_error()
    L.counts[1] = L.counts[5] = 0
    L.cache_pages_k = L.cache_pages_v = 4
    tok = lambda k, v, sb, sh, B, cos=None, sin=None, rs=0: lib.kitty_append_token(ctypes.byref(L), k, v, sb, sh, cos, sin, rs, B, None)
    assert tok(fake, fake, 256, 256, 1) == E_NULL    # no seq_counts
    assert b"seq_counts" in lib.kitty_last_error()
    assert lib.kitty_flush_full(ctypes.byref(L), 1, None) == E_NULL
    assert lib.kitty_append_chunk(ctypes.byref(L), fake, fake, 32768, 32768, 256, 1, 8, None) == E_NULL
    L.seq_counts = 4096
    assert tok(None, fake, 256, 256, 1) == E_NULL
    assert tok(fake, fake, 250, 256, 1) == E_ALIGN
    assert tok(fake, fake, 256, 256, 0) == E_RANGE
    assert tok(fake, fake, 256, 256, 1, cos=fake) == E_NULL and b"rope" in lib.kitty_last_error()   # cos without sin
    assert tok(fake, fake, 256, 256, 1, cos=fake, sin=fake, rs=100) == E_ALIGN
    assert lib.kitty_append_chunk(ctypes.byref(L), fake, fake, 32768, 32768, 256, 1, 0, None) == E_RANGE
    assert lib.kitty_append_chunk(ctypes.byref(L), fake, fake, 32768, 32768, 250, 1, 8, None) == E_ALIGN
    L.cache_pages_v = -3
    assert lib.kitty_flush_full(ctypes.byref(L), 1, None) == E_RANGE
    L.cache_pages_v = 4
    L.PAGE_SIZE = 256
    assert lib.kitty_flush_full(ctypes.byref(L), 1, None) == E_SHAPE
    # the partials (max / sum pairs, then accumulator rows) and, 256-aligned, a work list of 4 + B * splits words
    assert lib.kitty_decode_attn_workspace_bytes(16, 32, 128, 16) == (
        16 * 32 * 16 * 2 * 4 + 16 * 32 * 16 * 128 * 4 + (4 + 16 * 16) * 4 + 240)
    assert lib.kitty_decode_attn_workspace_bytes(16, 32, 96, 16) == 0
    assert lib.kitty_decode_attn_workspace_bytes(16, 32, 64, 16) == (
        16 * 32 * 16 * 2 * 4 + 16 * 32 * 16 * 64 * 4 + (4 + 16 * 16) * 4 + 240)
    ds = lib.kitty_decode_attn_default_splits
    assert 1 <= ds(16, 8, 257, 0) <= 257
    assert ds(1, 8, 1025, 0) > ds(16, 8, 1025, 0)
    # long splits: two waves per SIMD of the device (256 compute units when there is none to ask); short
    # splits (under 8 tiles): 15/16 of that; body splits of 2.5 tiles at least, and then at most 3/4
    # of a workgroup per SIMD if body splits of 4 tiles or fewer allow it, else at most six
    # workgroups per compute unit; at least 12 for long sequences with their own lengths
    assert ds(16, 8, 257, 0) == 16
    assert ds(1, 8, 1025, 0) == 240
    assert ds(1, 8, 33, 0) == 2 * 33 // 5 + 3 == 16
    assert ds(1, 8, 129, 0) == 54
    assert ds(4, 8, 65, 0) == 768 // 32 == 24 and ds(2, 8, 129, 0) == 48
    assert ds(8, 8, 65, 0) == 1536 // 64 == 24 and ds(2, 8, 257, 0) == 1536 // 16 == 96 and ds(1, 8, 513, 0) == 192
    assert ds(0, 8, 33, 0) == 1
    assert ds(64, 8, 131, 0) == 4 and ds(64, 8, 131, 1) == 12 and ds(64, 8, 40, 1) == 4


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from kitty_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        _lib.lib()


def test_bench_refuses_more_than_one_gpu():
    """The measured path is the one-GPU kernel path: `bench.py --gpus N` with N > 1 says so and exits."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "one-GPU" in (r.stdout + r.stderr)
