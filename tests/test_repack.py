"""The compile-time repacker: bit-exact round trip, and a lane-by-lane numpy emulation of the
register unpack the kernels perform on the tiled layout, checked against the oracle's view of the
same OpenVINO-layout bytes."""
import numpy as np
import pytest

from openvino_amd import datagen, fc

SHAPES = [
    # (w_type, zp_type, N, K, G)
    ("u4", "u4", 32, 256, 128), ("u4", "none", 16, 128, 128), ("i4", "none", 48, 384, 128),
    ("i4", "u4", 16, 512, 256), ("u4", "u8", 64, 256, 128), ("u8", "u8", 32, 256, 256),
    ("u8", "none", 16, 128, 128), ("u8", "u8", 16, 512, 128),
    ("u4", "u4", 16, 14336, 128),           # 112 groups per channel
    ("i4", "none", 1024, 4096, 128),        # a real k/v projection
    # groups of 64 and 32 inputs (4-bit weights): two and four groups per k-block
    ("u4", "u4", 32, 256, 64), ("u4", "u8", 16, 384, 32), ("i4", "none", 48, 128, 64), ("i4", "u4", 32, 512, 32),
]


def emulate_unpack(desc, wt, N, K):
    """What the kernels reconstruct from the tiled weights: integer (q + unsigned offset) per (n, k)."""
    NT, KB = N // 16, K // 128
    if desc.w_type in (1, 2):
        d = wt.view(np.uint32).reshape(NT, KB, 64, 4)
        # element pairs come out of the masks 0x000F000F, 0x00F000F0 on w and on w >> 8
        pos = [0, 4, 1, 5, 2, 6, 3, 7]
        elems = np.stack([(d >> (4 * p)) & 0xF for p in pos], axis=-1)      # [NT,KB,lane,j,e]
        out = np.zeros((N, K), np.int32)
        lane = np.arange(64)
        n_local, kq = lane & 15, lane >> 4
        for j in range(4):
            for e in range(8):
                k_local = 32 * j + 8 * kq + e                                   # [64]
                for l in range(64):
                    out[n_local[l]::16, k_local[l]::128] = elems[:, :, l, j, e]
        return out
    d = wt.reshape(NT, KB * 2, 64, 4, 4).astype(np.int32)                       # [NT,KT,lane,dword,byte]
    out = np.zeros((N, K), np.int32)
    for l in range(64):
        n_local, kq = l & 15, l >> 4
        for dw in range(4):
            for b in range(4):
                k_local = 32 * (dw >> 1) + 8 * kq + 4 * (dw & 1) + b
                out[n_local::16, k_local::64] = d[:, :, l, dw, b]
    return out


@pytest.mark.parametrize("wt_,zt_,N,K,G", SHAPES)
def test_round_trip_and_unpack_emulation(oracle, wt_, zt_, N, K, G):
    c = datagen.make_case(123, 0, K, N, wt_, G, zt_)
    desc = fc.make_desc(N, K, G, wt_, zt_)
    wt, st, zt = fc.repack_host(desc, c.w, c.scale, c.zp)
    assert wt.size == (N * K // 2 if wt_ in ("u4", "i4") else N * K)

    # inverse restores OpenVINO's bytes exactly
    w2, s2, z2 = fc.unrepack_host(desc, wt, st, zt)
    assert np.array_equal(w2, c.w)
    assert np.array_equal(s2.view(np.uint16), c.scale.view(np.uint16))
    if c.zp is not None:
        assert np.array_equal(z2, c.zp)

    # the kernels' register unpack sees the right element at every (n, k)
    offset = {"i4": 8, "i8": 128}.get(wt_, 0)
    if wt_ == "u4":
        q = oracle.unpack_u4(c.w, N * K).astype(np.int32)
    elif wt_ == "i4":
        q = oracle.unpack_i4(c.w, N * K).astype(np.int32)
    else:
        q = c.w.astype(np.int32)
    assert np.array_equal(emulate_unpack(desc, wt, N, K), q.reshape(N, K) + offset)

    # scale / zero-point tables: [N/16][groups][16]; with G < 128, [N/16][K/128][16][groups per k-block]
    ng = K // G

    def channel_major(t):
        if G >= 128:
            return t.reshape(N // 16, ng, 16).transpose(0, 2, 1).reshape(N, ng)
        return t.reshape(N // 16, K // 128, 16, 128 // G).transpose(0, 2, 1, 3).reshape(N, ng)

    assert np.array_equal(channel_major(st).view(np.uint16), c.scale.view(np.uint16))
    if zt is not None:
        zq = (oracle.unpack_u4(c.zp, N * ng) if zt_ == "u4" else c.zp).astype(np.int32).reshape(N, ng)
        assert np.array_equal(channel_major(zt), zq + offset)


def test_repack_rejects_untiled_shapes():
    desc = fc.make_desc(24, 128, 128, "u4")
    with pytest.raises(fc.OvfccError):
        fc.repack_host(desc, np.zeros(24 * 64, np.uint8), np.zeros((24, 1), np.float16))
    # groups of 16 inputs, and groups below 128 inputs with 8-bit weights, keep OpenVINO's layout
    for wt_, G in (("u4", 16), ("u8", 64), ("u8", 32)):
        desc = fc.make_desc(16, 128, G, wt_)
        assert fc.tiled_sizes(desc) == (0, 0, 0)


def test_half_magic_numbers_are_exact():
    """0x6400|q == 1024+q and 0x5400|(q<<4) == 64+q as halves; subtracting 1024+zp / 64+zp is exact."""
    q = np.arange(16, dtype=np.uint16)
    lo = (q | 0x6400).view(np.float16).astype(np.float32)
    hi = ((q << 4) | 0x5400).view(np.float16).astype(np.float32)
    assert np.array_equal(lo, 1024.0 + q) and np.array_equal(hi, 64.0 + q)
    for zp in range(0, 24):
        assert np.array_equal((lo.astype(np.float16) - np.float16(1024 + zp)).astype(np.float32), q - np.float32(zp))
        assert np.array_equal((hi.astype(np.float16) - np.float16(64 + zp)).astype(np.float32), q - np.float32(zp))
    b = np.arange(256, dtype=np.uint16)
    by = (b | 0x6400).view(np.float16)
    for zp in (0, 100, 156, 255, 383):
        assert np.array_equal((by - np.float16(1024 + zp)).astype(np.float32), b.astype(np.float32) - zp)


@pytest.mark.parametrize("wt_,zt_,N,K,G", [s for s in SHAPES if s[2] * s[3] <= 1 << 20] + [("u4", "u4", 48, 128, 128)])
def test_input_major_constants_give_the_same_tiles(wt_, zt_, N, K, G):
    """OVFCC_W_INPUT_MAJOR: W [K, N] and scales / zero-points [K / G, N] (a MatMul with transpose_b = false) are
    transposed once on the host; the tiles are those of the [N, K] constants.  The transposed inputs come from
    numpy, not from the library."""
    c = datagen.make_case(321, 0, K, N, wt_, G, zt_)
    plain = fc.repack_host(fc.make_desc(N, K, G, wt_, zt_), c.w, c.scale, c.zp)
    w_kn, s_kn, z_kn = datagen.to_input_major(c)
    if N != K:
        assert not np.array_equal(w_kn, c.w)
    turned = fc.repack_host(fc.make_desc(N, K, G, wt_, zt_, input_major=True), w_kn, s_kn, z_kn)
    for a, b in zip(plain, turned):
        assert (a is None) == (b is None)
        if a is not None:
            assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
    # tiles unpack to the [N, K] order only
    with pytest.raises(fc.OvfccError):
        fc.unrepack_host(fc.make_desc(N, K, G, wt_, zt_, input_major=True), *plain)


def test_input_major_nibble_transpose_known_answer():
    """A 2 x 3 u4 matrix by hand: [[1, 2, 3], [4, 5, 6]] packs low nibble first to 21 43 65; its transpose
    [[1, 4], [2, 5], [3, 6]] packs to 41 52 63."""
    from openvino_amd import datagen as d
    rows = np.array([[1, 2, 3], [4, 5, 6]], np.uint8)
    assert d.pack_nibbles(rows).tolist() == [0x21, 0x43, 0x65]
    assert d.pack_nibbles(rows.T).tolist() == [0x41, 0x52, 0x63]
    assert d.unpack_nibbles(d.pack_nibbles(rows.T), 6).reshape(3, 2).T.tolist() == rows.tolist()


def test_signed_weights_with_byte_zero_points_stay_untiled():
    """The tiled zero-point table stores zp + 8 (i4) or zp + 128 (i8) in one byte.  With 8-bit zero-points per group
    that sum can pass 255, so such nodes keep OpenVINO's layout (the plain kernel subtracts the zero-point itself);
    i4 with 4-bit zero-points (at most 15 + 8) is tiled and its table holds zp + 8 exactly."""
    for wt_ in ("i8", "i4"):
        desc = fc.make_desc(16, 128, 128, wt_, zp_type="u8")
        assert fc.tiled_sizes(desc) == (0, 0, 0), wt_
        with pytest.raises(fc.OvfccError):
            fc.repack_host(desc, np.zeros(16 * 128, np.uint8), np.ones((16, 1), np.float16), np.full((16, 1), 200, np.uint8))
    # a scalar zero-point travels as an integer, not in the byte table: tiled
    assert fc.tiled_sizes(fc.make_desc(16, 128, 128, "i8", zp_type="u8", zp_scalar=True))[0] > 0
    desc = fc.make_desc(16, 256, 128, "i4", zp_type="u4")
    assert fc.tiled_sizes(desc)[2] == 16 * 2
    zp = np.full(16, 0xFF, np.uint8)                      # every zero-point 15, two per byte
    _, _, zt = fc.repack_host(desc, np.zeros(16 * 128, np.uint8), np.ones((16, 2), np.float16), zp)
    assert np.all(zt == 23)
