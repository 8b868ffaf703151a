"""The device-side tile schedule, exercised through its host mirror (no GPU)."""
import ctypes

import numpy as np
import pytest


def _schedule(native, rows, n, force_bm=0, with_origin=False, mx=0):
    """Every tile the kernel would compute: all tickets of the 8 per-XCD queues, then the light items."""
    lib = native.lib
    e = len(rows)
    ps = np.array([[m, n, 512] for m in rows], dtype=np.int32)
    ws = np.zeros(lib.esmoe_gemm_workspace_bytes(e) // 4, dtype=np.int32)
    psp, wsp = ps.ctypes.data_as(ctypes.c_void_p), ws.ctypes.data_as(ctypes.c_void_p)
    rc = lib.esmoe_host_schedule(psp, e, n, force_bm, mx, wsp)
    assert rc == 0, native.last_error()
    light_total, heavy_blocks = int(ws[1]), int(ws[2])
    tiles, origin = [], []
    out = np.zeros(5, dtype=np.int32)
    seen_blocks = 0
    for xcd in range(8):
        ticket = 0
        while True:
            rc = lib.esmoe_host_decode_heavy(psp, wsp, e, n, force_bm, mx, xcd, ticket, out.ctypes.data_as(ctypes.c_void_p))
            assert rc in (0, 1, 2), native.last_error()
            if rc == 2:
                break
            if rc == 0:
                tiles.append(tuple(int(v) for v in out))
                origin.append(("heavy", xcd, ticket // 32))
            ticket += 1
        assert ticket % 32 == 0  # queues end on a block boundary
        seen_blocks += ticket // 32
    assert seen_blocks == heavy_blocks
    for item in range(light_total):
        rc = lib.esmoe_host_decode_light(psp, wsp, e, n, force_bm, mx, item, out.ctypes.data_as(ctypes.c_void_p))
        assert rc in (0, 1), native.last_error()
        if rc == 1:      # second half of a 128-column last tile
            continue
        tiles.append(tuple(int(v) for v in out))
        origin.append(("light", item))
    return (tiles, origin) if with_origin else tiles


@pytest.mark.parametrize("mx", [0, 1, 2, 3])   # bit 0: mxfp8, bit 1: fused SwiGLU epilogue
@pytest.mark.parametrize("force_bm", [0, 16, 32, 64, 128, 192])
@pytest.mark.parametrize("n", [128, 384, 4096])
def test_tiles_cover_every_output_element_exactly_once(esmoe, force_bm, n, mx):
    from expert_specialization_moe_amd import _native

    rows = [0, 1, 16, 17, 127, 128, 129, 300, 0, 1000, 64, 33, 449, 577]
    tiles = _schedule(_native, rows, n, force_bm, mx=mx)
    cover = [np.zeros((m, n), dtype=np.int32) for m in rows]
    for e, bm, bn, m0, n0 in tiles:
        assert bn in (128, 256) and bm in (16, 32, 64, 128, 192)
        assert m0 < rows[e] and n0 < n and m0 % 16 == 0 and n0 % bn == 0
        if bn == 128:   # half items: light experts of a plain launch with no forced height
            assert rows[e] <= 64 and not force_bm and not (mx & 2)
        if force_bm:
            assert bm == force_bm
        cover[e][m0:m0 + bm, n0:n0 + bn] += 1
        if not force_bm:
            # full tiles of 192 rows for both kernels, then one remainder tile
            assert bm <= 192 and m0 % 192 == 0
    for c in cover:
        assert (c == 1).all()


def test_both_kernels_use_192_row_full_tiles(esmoe):
    from expert_specialization_moe_amd import _native

    heights = lambda mx: sorted({t[1] for t in _schedule(_native, [700], 256, 0, mx=mx)})
    assert heights(0) == [128, 192]      # 3 x 192 + 124 -> 128
    assert heights(1) == [128, 192]


@pytest.mark.parametrize("light_experts", [1, 7, 9, 40])
def test_the_last_128_light_items_go_out_as_halves(esmoe, light_experts):
    """A plain launch hands its last 128 light items out as two 128-column halves each, in item order; a fused launch
    and a forced tile height keep whole items."""
    from expert_specialization_moe_amd import _native

    n = 4096                                   # 16 items per light expert
    rows = [900] + [1 + 3 * i % 60 for i in range(light_experts)]
    items = 16 * light_experts
    tiles, origin = _schedule(_native, rows, n, 0, with_origin=True)
    light = [t for t, o in zip(tiles, origin) if o[0] == "light"]
    narrow = min(items, 128)
    assert len(light) == items + narrow
    whole, halves = light[:items - narrow], light[items - narrow:]
    assert all(t[2] == 256 for t in whole) and all(t[2] == 128 for t in halves)
    for a, b in zip(halves[0::2], halves[1::2]):
        assert a[0] == b[0] and a[1] == b[1] and a[4] % 256 == 0 and b[4] == a[4] + 128
    for kind, force in ((2, 0), (0, 64)):
        tiles = _schedule(_native, rows, n, force, mx=kind)
        assert all(t[2] == 256 for t in tiles)


def test_auto_shapes_waste_less_than_any_single_shape(esmoe):
    from expert_specialization_moe_amd import _native

    rows = [3841, 965, 323, 215, 162, 132, 81, 77, 40, 17, 11, 0]

    def padded_rows(tiles):
        return sum(bm for _, bm, _, _, n0 in tiles if n0 == 0)

    auto = padded_rows(_schedule(_native, rows, 256, 0))
    for bm in (64, 128, 192):
        assert auto <= padded_rows(_schedule(_native, rows, 256, bm))
    # slack: less than half of the remainder tile per expert (menu 16/32/64/128 rows)
    assert auto - sum(rows) <= 64 * len(rows)


def test_order_is_fewest_rows_first_for_heavy_and_most_rows_first_for_light(esmoe):
    from expert_specialization_moe_amd import _native

    rows = [5, 900, 0, 64, 900, 7, 65]
    tiles, origin = _schedule(_native, rows, 256, 0, with_origin=True)
    # heavy experts (more than 64 rows) in block order, fewest rows first; light ones in item order, most rows first;
    # ties by expert index, empty absent
    heavy = sorted((o[2] * 8 + o[1], t[0]) for t, o in zip(tiles, origin) if o[0] == "heavy")
    light = [t[0] for t, o in zip(tiles, origin) if o[0] == "light"]

    def runs(seq):
        r = []
        for e in seq:
            if not r or r[-1] != e:
                r.append(e)
        return r

    assert runs([e for _, e in heavy]) == [6, 1, 4]
    assert runs(light) == [3, 5, 0]


def test_heavy_blocks_are_rectangles_of_one_expert_on_one_xcd(esmoe):
    from expert_specialization_moe_amd import _native

    rows = [3841, 965, 323, 215, 70, 12]
    n = 4096
    tiles, origin = _schedule(_native, rows, n, 0, with_origin=True)
    blocks = {}
    for t, o in zip(tiles, origin):
        if o[0] == "heavy":
            blocks.setdefault((o[1], o[2]), []).append(t)
    assert blocks
    for (xcd, rnd), ts in blocks.items():
        assert len({t[0] for t in ts}) == 1 and len(ts) <= 32
        bm, bn = len({t[3] for t in ts}), len({t[4] for t in ts})
        assert bm <= 8 and bm * bn <= 32 and len(ts) == bm * bn
    # a block's weight panel is contiguous
    for ts in blocks.values():
        n0s = sorted({t[4] for t in ts})
        assert n0s[-1] - n0s[0] == 256 * (len(n0s) - 1)
