"""The device-side tile schedule, exercised through its host mirror (no GPU)."""
import ctypes

import numpy as np
import pytest


def _schedule(native, rows, n, force_bm=0):
    lib = native.lib
    e = len(rows)
    ps = np.array([[m, n, 512] for m in rows], dtype=np.int32)
    ws = np.zeros(lib.esmoe_gemm_workspace_bytes(e) // 4, dtype=np.int32)
    rc = lib.esmoe_host_schedule(ps.ctypes.data_as(ctypes.c_void_p), e, n, force_bm, ws.ctypes.data_as(ctypes.c_void_p))
    assert rc == 0, native.last_error()
    total = int(ws[1])
    tiles = []
    out = np.zeros(5, dtype=np.int32)
    for item in range(total):
        rc = lib.esmoe_host_decode_item(ps.ctypes.data_as(ctypes.c_void_p), ws.ctypes.data_as(ctypes.c_void_p), e, n,
                                        force_bm, item, out.ctypes.data_as(ctypes.c_void_p))
        assert rc == 0
        tiles.append(tuple(int(v) for v in out))
    return tiles


@pytest.mark.parametrize("force_bm", [0, 16, 32, 64, 128, 192, 256])
@pytest.mark.parametrize("n", [128, 384, 4096])
def test_tiles_cover_every_output_element_exactly_once(esmoe, force_bm, n):
    from expert_specialization_moe_amd import _native

    rows = [0, 1, 16, 17, 127, 128, 129, 300, 0, 1000, 64, 33]
    tiles = _schedule(_native, rows, n, force_bm)
    cover = [np.zeros((m, n), dtype=np.int32) for m in rows]
    for e, bm, bn, m0, n0 in tiles:
        assert bn == 256 and bm in (16, 32, 64, 128, 192, 256)
        assert m0 < rows[e] and n0 < n and m0 % 16 == 0 and n0 % 256 == 0
        if force_bm:
            assert bm == force_bm
        cover[e][m0:m0 + bm, n0:n0 + bn] += 1
    for c in cover:
        assert (c == 1).all()


def test_auto_shapes_waste_less_than_any_single_shape(esmoe):
    from expert_specialization_moe_amd import _native

    rows = [3841, 965, 323, 215, 162, 132, 81, 77, 40, 17, 11, 0]

    def padded_rows(tiles):
        return sum(bm for _, bm, _, _, n0 in tiles if n0 == 0)

    auto = padded_rows(_schedule(_native, rows, 256, 0))
    for bm in (64, 128, 256):
        assert auto <= padded_rows(_schedule(_native, rows, 256, bm))
    # slack: less than half of the remainder tile per expert (menu 16/32/64/128 rows)
    assert auto - sum(rows) <= 64 * len(rows)


def test_order_is_most_rows_first(esmoe):
    from expert_specialization_moe_amd import _native

    rows = [5, 900, 0, 64, 900, 7]
    tiles = _schedule(_native, rows, 256, 0)
    seq = []
    for e, *_ in tiles:
        if not seq or seq[-1] != e:
            seq.append(e)
    assert seq == [1, 4, 3, 5, 0]  # ties by expert index, empty experts absent
