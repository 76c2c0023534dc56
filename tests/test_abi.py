"""The C-ABI library loads without a GPU, exports every symbol include/ovfcc.h declares, and its
host-only entry points validate arguments the way the plugin's support gate must."""
import ctypes
import os
import re

import numpy as np
import pytest

from openvino_amd import _lib, fc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(bench: bool):
    """Every function that include/*.h declares: the benchmark header's, or all the others'."""
    names = set()
    for header in sorted(os.listdir(os.path.join(ROOT, "include"))):
        if not header.endswith(".h") or (header == "ovfcc_bench.h") != bench:
            continue
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names.update(re.findall(r"\b(ovfcc_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_every_declared_symbol_is_exported():
    _lib.load()
    product = ctypes.CDLL(_lib.LIB_PATH)
    names = declared_symbols(bench=False)
    assert len(names) >= 25
    for name in names:
        assert hasattr(product, name), f"{name} is declared under include/ but libovfcc.so does not export it"
    assert sorted(_lib.SYMBOLS) == names


def test_benchmark_helpers_live_in_their_own_library():
    _lib.load()
    product, bench = ctypes.CDLL(_lib.LIB_PATH), ctypes.CDLL(_lib.BENCH_LIB_PATH)
    names = declared_symbols(bench=True)
    assert sorted(_lib.BENCH_SYMBOLS) == names
    for name in names:
        assert hasattr(bench, name), f"{name} is declared in include/ovfcc_bench.h but libovfcc_bench.so does not export it"
        assert not hasattr(product, name), f"{name} belongs to the benchmark library, not to libovfcc.so"


def test_version_and_error_string():
    L = _lib.load()
    assert L.ovfcc_version().startswith(b"ovfcc")
    d = fc.make_desc(16, 128, 100, "u4")
    assert fc.validate(d) == _lib.EINVAL
    assert b"group_size" in L.ovfcc_last_error()


@pytest.mark.parametrize("mutate,code", [
    (dict(N=0), _lib.EINVAL), (dict(K=-4), _lib.EINVAL), (dict(group_size=0), _lib.EINVAL),
    (dict(group_size=96), _lib.EINVAL), (dict(w_type=_lib.F16), _lib.EUNSUPPORTED),
    (dict(scale_type=_lib.F32), _lib.EUNSUPPORTED), (dict(zp_type=_lib.I4), _lib.EUNSUPPORTED),
    (dict(act_type=_lib.F32), _lib.EUNSUPPORTED), (dict(out_type=_lib.U8), _lib.EUNSUPPORTED),
    (dict(bias_type=_lib.F32), _lib.EUNSUPPORTED), (dict(flags=32), _lib.EINVAL), (dict(flags=64), _lib.EINVAL),
    (dict(flags=4), _lib.EINVAL), (dict(flags=1, N=63), _lib.EINVAL),
    (dict(flags=8 | 32 | 64), _lib.EINVAL), (dict(flags=128), _lib.EINVAL),   # asymmetric: per token only; unknown bit
])
def test_descriptor_gate(mutate, code):
    d = fc.make_desc(64, 256, 128, "u4", "u4")
    assert fc.validate(d) == _lib.OK
    for k, v in mutate.items():
        setattr(d, k, v)
    assert fc.validate(d) == code
    assert _lib.load().ovfcc_last_error() != b""
    if "flags" in mutate and mutate["flags"] == 64:   # ... and only together with the permission itself
        d.flags = _lib.DYNQUANT_I8 | _lib.DYNQUANT_ASYM
        assert fc.validate(d) == _lib.OK


def test_glu_descriptor_and_layout():
    """A gated-linear-unit node keeps the tiled layout when its halves are whole tiles (N % 32 == 0), and the
    repacker alternates gate and up tiles: unrepacking restores the OpenVINO order."""
    assert fc.validate(fc.make_desc(64, 256, 128, "u4", "u4", glu="swish")) == _lib.OK
    assert fc.validate(fc.make_desc(64, 256, 128, "u4", "u4", glu="gelu_tanh", glu_gate_second=True)) == _lib.OK
    assert fc.tiled_sizes(fc.make_desc(64, 256, 128, "u4", "u4", glu="swish"))[0] == 64 * 256 // 2
    assert fc.tiled_sizes(fc.make_desc(48, 256, 128, "u4", "u4"))[0] == 48 * 256 // 2
    assert fc.tiled_sizes(fc.make_desc(48, 256, 128, "u4", "u4", glu="swish"))[0] == 0      # halves of 24 channels
    rng = np.random.default_rng(5)
    N, K = 64, 256
    W = rng.integers(0, 256, N * K // 2, dtype=np.uint8)
    S = rng.uniform(0.01, 0.02, (N, 2)).astype(np.float16)
    Z = rng.integers(0, 256, N * 2 // 2, dtype=np.uint8)
    plain = fc.make_desc(N, K, 128, "u4", "u4")
    wt0, st0, zt0 = fc.repack_host(plain, W, S, Z)
    for second in (False, True):
        d = fc.make_desc(N, K, 128, "u4", "u4", glu="swish", glu_gate_second=second)
        wt, st, zt = fc.repack_host(d, W, S, Z)
        tile_w = wt0.size // 4                          # bytes of one 16-channel tile row
        order = [2, 0, 3, 1] if second else [0, 2, 1, 3]  # tiles: gate j, up j, ...
        assert np.array_equal(wt.reshape(4, tile_w), wt0.reshape(4, tile_w)[order])
        assert np.array_equal(st.reshape(4, -1), st0.reshape(4, -1)[order])
        assert np.array_equal(zt.reshape(4, -1), zt0.reshape(4, -1)[order])
        w2, s2, z2 = fc.unrepack_host(d, wt, st, zt)
        assert np.array_equal(w2, W) and np.array_equal(s2, S) and np.array_equal(z2, Z)


def test_null_descriptor_and_null_outputs():
    L = _lib.load()
    assert L.ovfcc_desc_validate(None) == _lib.EINVAL
    d = fc.make_desc(64, 256, 128, "u4")
    assert L.ovfcc_tiled_sizes(ctypes.byref(d), None, None, None) == _lib.EINVAL
    assert L.ovfcc_repack_host(ctypes.byref(d), None, None, None, None, None, None) == _lib.EINVAL
    assert L.ovfcc_init(0, None) == _lib.EINVAL
    assert L.ovfcc_request_create(None, None) == _lib.EINVAL
    assert L.ovfcc_fc_run(None, None, None, None, 1) == _lib.EINVAL
    assert L.ovfcc_request_sync(None) == _lib.EINVAL


def test_layout_choice_and_sizes():
    # tiled: N % 16 == 0, K % 128 == 0, G % 128 == 0 -- or G of 32 or 64 under 4-bit weights
    assert fc.tiled_sizes(fc.make_desc(4096, 4096, 128, "u4", "u4")) == (4096 * 4096 // 2, 4096 * 32 * 2, 4096 * 32)
    assert fc.tiled_sizes(fc.make_desc(4096, 4096, 128, "i4")) == (4096 * 4096 // 2, 4096 * 32 * 2, 0)
    assert fc.tiled_sizes(fc.make_desc(1024, 8192, 8192, "u8", "u8")) == (1024 * 8192, 1024 * 2, 1024)
    assert fc.tiled_sizes(fc.make_desc(64, 256, 256, "u8", "u8", zp_scalar=True)) == (64 * 256, 64 * 2, 0)
    # fallbacks keep the OpenVINO layout
    assert fc.tiled_sizes(fc.make_desc(16, 256, 64, "u4", "u4")) == (16 * 256 // 2, 16 * 4 * 2, 16 * 4)
    assert fc.tiled_sizes(fc.make_desc(32, 128, 32, "i4")) == (32 * 128 // 2, 32 * 4 * 2, 0)
    # fallbacks keep the OpenVINO layout
    for d in (fc.make_desc(8, 4, 4, "u8"), fc.make_desc(24, 128, 128, "u4"), fc.make_desc(16, 192, 64, "u4"),
              fc.make_desc(16, 256, 64, "u8"), fc.make_desc(16, 256, 16, "u4")):
        assert fc.tiled_sizes(d) == (0, 0, 0)


def test_unpack_entry_points_match_golden():
    L = _lib.load()
    raw = np.array([0x12, 0x3a, 0xcf, 0xe4, 0x79, 0xbd, 0x08, 0x56], np.uint8)
    u = np.empty(16, np.uint8)
    i = np.empty(16, np.int8)
    assert L.ovfcc_unpack_u4(raw.ctypes.data, 16, u.ctypes.data) == 0
    assert L.ovfcc_unpack_i4(raw.ctypes.data, 16, i.ctypes.data) == 0
    assert u.tolist() == [2, 1, 10, 3, 15, 12, 4, 14, 9, 7, 13, 11, 8, 0, 6, 5]
    assert i.tolist() == [2, 1, -6, 3, -1, -4, 4, -2, -7, 7, -3, -5, -8, 0, 6, 5]


def test_no_device_fails_loudly():
    """Without a GPU the product refuses to run: there is no CPU path behind the ABI."""
    L = _lib.load()
    if L.ovfcc_device_count() > 0:
        pytest.skip("a GPU is visible")
    h = ctypes.c_void_p()
    assert L.ovfcc_init(0, ctypes.byref(h)) == _lib.EDEVICE
    assert b"no HIP device" in L.ovfcc_last_error()
    with pytest.raises(_lib.OvfccError):
        fc.Device(0)
