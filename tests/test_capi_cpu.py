"""CPU-side checks of the C ABI: the library loads, exports every symbol the header
declares, and the kernel-selection rule table (a pure function) gives known answers."""
import ctypes as C
import os
import re

import pytest

from vecops_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "vecops_hip.h")).read()
    return sorted(set(re.findall(r"VECOPS_HIP_EXPORT[^;(]*?\b(vecops_hip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = capi.lib()
    names = declared_symbols()
    assert sorted(names) == sorted(capi.EXPORTS)
    for name in names:
        assert getattr(lib, name) is not None
    assert lib.vecops_hip_abi_version() == 1


def _operand(dtype, shape, strides=None, data=0x1000):
    o = capi.Operand()
    o.data, o.dtype, o.rank = data, dtype, len(shape)
    if strides is None:
        strides, acc = [], 1
        for s in reversed(shape):
            strides.insert(0, acc)
            acc *= s
    for i, (s, st) in enumerate(zip(shape, strides)):
        o.sizes[i], o.strides[i] = s, st
    return o


def _plan(a, b, c, compute=0):
    plan = capi.Plan()
    rc = capi.lib().vecops_hip_plan_matmul(C.byref(a), C.byref(b), None, C.byref(c), compute, C.byref(plan))
    return rc, plan


def test_rule_table_known_answers():
    # BASELINE config 2: 256 tiles of 256x256, one per compute unit
    rc, p = _plan(_operand(capi.BF16, (4096, 4096)), _operand(capi.BF16, (4096, 4096)),
                  _operand(capi.BF16, (4096, 4096)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_256" and p.split_k == 1 and p.workspace_bytes == 0
    assert p.vector_a == 1 and p.vector_b == 1
    # config 4
    rc, p = _plan(_operand(capi.I8, (2048, 4096)), _operand(capi.I8, (11008, 4096)),
                  _operand(capi.I32, (2048, 11008)))
    # 344 tiles of 256x256 would take two rounds, the second a third full; 1376 of 128x128 two and two thirds at two
    # workgroups per unit; 256 tiles of 256x352 are exactly one round
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_256x352" and p.split_k == 1 and p.workspace_bytes == 0
    # bf16 and f16 operands take that tile too (the same loop on their 16x16x32 instructions), to their own type or fp32
    for dtype, out in ((capi.BF16, capi.BF16), (capi.BF16, capi.F32), (capi.F16, capi.F16)):
        rc, p = _plan(_operand(dtype, (2048, 4096)), _operand(dtype, (11008, 4096)), _operand(out, (2048, 11008)))
        assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_256x352" and p.split_k == 1 and p.workspace_bytes == 0
    # 4096 x 11008: 512 of them are two rounds where 688 square ones are three; 6144^3: 432 against 576; 4096^3 and
    # 8192^3 keep the square tile (192 wide ones leave a quarter of the units idle; 768 are three rounds against four
    # of less work)
    for (m, n, k), family in (((4096, 11008, 4096), "tile_256x352"), ((6144, 6144, 6144), "tile_256x352"),
                              ((4096, 4096, 4096), "tile_256"), ((8192, 8192, 8192), "tile_256"), ((4096, 4096, 11008), "tile_256")):
        rc, p = _plan(_operand(capi.BF16, (m, k)), _operand(capi.BF16, (n, k)), _operand(capi.BF16, (m, n)))
        assert rc == 0 and capi.FAMILY_NAMES[p.family] == family, (m, n, k, p.family)
    # the same extents where that tile cannot serve: B as [K,N], rows of A that are not 16-byte aligned, a K that is no
    # multiple of 128 - the 128x128 tile as before; an M that is no multiple of 256 is served (rows past M are fetched
    # as zeros and not stored)
    rc, p = _plan(_operand(capi.BF16, (2048, 4096)), _operand(capi.BF16, (11008, 4096), strides=(1, 11008)), _operand(capi.BF16, (2048, 11008)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_128"
    rc, p = _plan(_operand(capi.I8, (2040, 4096)), _operand(capi.I8, (11008, 4096)), _operand(capi.I32, (2040, 11008)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_256x352"
    rc, p = _plan(_operand(capi.I8, (2048, 4096), strides=(4104, 1)), _operand(capi.I8, (11008, 4096)),
                  _operand(capi.I32, (2048, 11008)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_128"
    rc, p = _plan(_operand(capi.I8, (2048, 4160)), _operand(capi.I8, (11008, 4160)), _operand(capi.I32, (2048, 11008)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_128"
    # int8 4096^3 keeps the square tile (192 of the wide ones would leave a quarter of the units idle)
    rc, p = _plan(_operand(capi.I8, (4096, 4096)), _operand(capi.I8, (4096, 4096)), _operand(capi.I32, (4096, 4096)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_256"
    # 8 x 777 x 1000: seven rows of 128x256 tiles pad M to 896, four rows of 256-row tiles would pad it to 1024
    rc, p = _plan(_operand(capi.BF16, (8, 777, 3001)), _operand(capi.BF16, (8, 1000, 3001)),
                  _operand(capi.F32, (8, 777, 1000)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_128x256"
    # problems of one and a half to two rounds of big tiles keep them
    rc, p = _plan(_operand(capi.BF16, (5120, 5120)), _operand(capi.BF16, (5120, 5120)), _operand(capi.BF16, (5120, 5120)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_256"
    rc, p = _plan(_operand(capi.BF16, (2048, 4096)), _operand(capi.BF16, (14336, 4096)), _operand(capi.BF16, (2048, 14336)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_256"
    # half a round of big tiles or a round of rectangles against one round of 128x128 pairs (two live on a compute
    # unit at a time): the small tile, for both classes; int8 also up to eight K tiles
    for dt, out in ((capi.BF16, capi.BF16), (capi.I8, capi.I32)):
        for m in (1536, 2048):
            rc, p = _plan(_operand(dt, (m, 4096)), _operand(dt, (4096, 4096)), _operand(out, (m, 4096)))
            assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_128" and p.split_k == 1
        rc, p = _plan(_operand(dt, (3072, 4096)), _operand(dt, (4096, 4096)), _operand(out, (3072, 4096)))
        assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_256"
    rc, p = _plan(_operand(capi.I8, (4096, 1024)), _operand(capi.I8, (4096, 1024)), _operand(capi.I32, (4096, 4096)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_128"
    rc, p = _plan(_operand(capi.BF16, (4096, 1024)), _operand(capi.BF16, (4096, 1024)), _operand(capi.BF16, (4096, 4096)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_256"
    # 3000^3: 256 tiles of 192 x 192 are one full round, where 144 big tiles leave 112 units idle (B as [N,K] or [K,N];
    # with rows that are not 16-byte aligned, which the 192 x 192 tile does not take: the big tiles, ahead of 576 small
    # ones in three rounds); so are 232 for 768 x 11008 and 224 for 1344 x 6144
    rc, p = _plan(_operand(capi.BF16, (3000, 3000)), _operand(capi.BF16, (3000, 3000)), _operand(capi.F32, (3000, 3000)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_192" and p.split_k == 1 and p.workspace_bytes == 0
    b_kn = _operand(capi.BF16, (3000, 3000))
    b_kn.strides[0], b_kn.strides[1] = 1, 3000
    rc, p = _plan(_operand(capi.BF16, (3000, 3000)), b_kn, _operand(capi.F32, (3000, 3000)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_192"
    rc, p = _plan(_operand(capi.BF16, (3000, 3000), strides=(3004, 1)), _operand(capi.BF16, (3000, 3000)), _operand(capi.F32, (3000, 3000)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_256"
    # one round of bigger tiles by a K split, where the 128 x 128 pairs fill their round badly or are split already and
    # K is long: 81 tiles of 256 x 256 in three parts, 64 / 128 of 192 x 192 in four / two; a shorter K, or parts that
    # would leave a tenth of the units idle, keep the pairs
    for (m, n, k), family, split in (((2304, 2304, 8192), "tile_256", 3), ((768, 3072, 12288), "tile_192", 4),
                                     ((1500, 3000, 8192), "tile_192", 2), ((2304, 2304, 4096), "tile_128", 1),
                                     ((2000, 2600, 6144), "tile_128", 1), ((2048, 4096, 11008), "tile_128", 1)):
        rc, p = _plan(_operand(capi.BF16, (m, k)), _operand(capi.BF16, (n, k)), _operand(capi.BF16, (m, n)))
        assert rc == 0 and capi.FAMILY_NAMES[p.family] == family and p.split_k == split, (m, n, k, p.family, p.split_k)
        assert p.workspace_bytes == (split * m * n * 4 if split > 1 else 0)
    # fp32 operands multiplied as bf16 go through staging registers: the small tile only up to half the units' worth of
    # 128 x 128 tiles, and from 96 tiles and 32 K tiles on two K parts of the 128 x 128 tile
    for (m, n, k), family, split in (((1024, 1024, 1024), "tile_64", 1), ((1408, 1408, 1408), "tile_64", 1), ((1536, 1536, 1536), "tile_128", 1),
                                     ((1024, 2048, 4096), "tile_128", 2), ((1280, 1280, 4096), "tile_128", 2), ((1024, 2048, 1024), "tile_64", 1)):
        rc, p = _plan(_operand(capi.F32, (m, k)), _operand(capi.F32, (n, k)), _operand(capi.F32, (m, n)))
        assert rc == 0 and capi.FAMILY_NAMES[p.family] == family and p.split_k == split, (m, n, k, p.family, p.split_k)
    for m, n in ((768, 11008), (1344, 6144), (3072, 3072)):
        rc, p = _plan(_operand(capi.BF16, (m, 4096)), _operand(capi.BF16, (n, 4096)), _operand(capi.BF16, (m, n)))
        assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_192", (m, n)
    # 4096 x 4224: 272 big tiles would leave the second round 6 % full; 192 tiles of 256x352 are one round, three
    # quarters full (1056 of 128x128, five per compute unit, where that tile cannot serve: B as [K,N])
    rc, p = _plan(_operand(capi.BF16, (4096, 4096)), _operand(capi.BF16, (4224, 4096)), _operand(capi.F32, (4096, 4224)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_256x352"
    rc, p = _plan(_operand(capi.BF16, (4096, 4096)), _operand(capi.BF16, (4224, 4096), strides=(1, 4224)), _operand(capi.F32, (4096, 4224)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_128"
    # config 3's 3000 x 3000 x 17: one K tile, the output is the work - several small workgroups per compute unit
    rc, p = _plan(_operand(capi.BF16, (3000, 17)), _operand(capi.BF16, (3000, 17)), _operand(capi.F32, (3000, 3000)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_128" and p.split_k == 1
    rc, p = _plan(_operand(capi.BF16, (8192, 512)), _operand(capi.BF16, (8192, 512)), _operand(capi.F32, (8192, 8192)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_256"      # from eight K tiles on the big tile is ahead again
    # 128 tiles of 128x128 leave every other compute unit idle, but a lone workgroup of the four-stage kernel does not
    # wait out its loads (25 us against 28 for 512 tiles of 64x64); operands that kernel does not serve - here a K
    # that is no whole number of K tiles - still take the small tiles
    rc, p = _plan(_operand(capi.BF16, (512, 4096)), _operand(capi.BF16, (4096, 4096)), _operand(capi.BF16, (512, 4096)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_128" and p.split_k == 1
    rc, p = _plan(_operand(capi.BF16, (512, 4104)), _operand(capi.BF16, (4096, 4104)), _operand(capi.BF16, (512, 4096)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_64" and p.split_k == 1
    rc, p = _plan(_operand(capi.BF16, (1024, 4096)), _operand(capi.BF16, (4096, 4096)), _operand(capi.BF16, (1024, 4096)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_128"
    # one row against a long weight matrix: the skinny family, no workspace
    rc, p = _plan(_operand(capi.BF16, (1, 4096)), _operand(capi.BF16, (14336, 4096)), _operand(capi.BF16, (1, 14336)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "skinny" and p.workspace_bytes == 0
    # fp32 memory takes it too, whichever way it is multiplied (a lane's chunk is 8 elements, 4 in fp32 compute)
    rc, p = _plan(_operand(capi.F32, (4, 4096)), _operand(capi.F32, (14336, 4096)), _operand(capi.F32, (4, 14336)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "skinny"
    rc, p = _plan(_operand(capi.F32, (4, 516)), _operand(capi.F32, (14336, 516)), _operand(capi.F32, (4, 14336)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] != "skinny"
    rc, p = _plan(_operand(capi.F32, (4, 516)), _operand(capi.F32, (14336, 516)), _operand(capi.F32, (4, 14336)), compute=1)
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "skinny"
    # ... but not with a K that 16-byte loads cannot cover
    rc, p = _plan(_operand(capi.BF16, (1, 129)), _operand(capi.BF16, (4097, 129)), _operand(capi.F32, (1, 4097)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] != "skinny"
    # int8 decode shapes are skinny too (signed bytes, K a multiple of 16); an unsigned side is not
    rc, p = _plan(_operand(capi.I8, (4, 4096)), _operand(capi.I8, (11008, 4096)), _operand(capi.I32, (4, 11008)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "skinny" and p.workspace_bytes == 0
    rc, p = _plan(_operand(capi.U8, (4, 4096)), _operand(capi.I8, (11008, 4096)), _operand(capi.I32, (4, 11008)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] != "skinny"
    rc, p = _plan(_operand(capi.I8, (4, 4104)), _operand(capi.I8, (11008, 4104)), _operand(capi.I32, (4, 11008)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] != "skinny"
    # tiny output, long K (config 3's 255x63x8191): small tile and split-K with workspace
    rc, p = _plan(_operand(capi.BF16, (255, 8191)), _operand(capi.BF16, (63, 8191)), _operand(capi.F32, (255, 63)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_64" and p.split_k > 1
    assert p.workspace_bytes == p.split_k * 255 * 63 * 4
    assert p.vector_a == 1                                   # rows need not be 16-byte aligned for 16-byte loads
    # 32 to 256 tiles of 128 x 128, operands the four-stage kernel serves (both K-contiguous and aligned, whole K
    # tiles): at most one workgroup per compute unit - whole from 96 tiles on (in two parts where the units allow and
    # the split rule's costs favour it), K split to fill the units once below that; more than half but at most 160
    # tiles and sixty K tiles per part keep the two-stage kernel's split (two co-resident workgroups on every unit)
    for (m, n, k), family, split in (((640, 4096, 4096), "tile_128", 1), ((768, 4096, 4096), "tile_128", 1),
                                     ((1024, 2048, 8192), "tile_128", 2), ((768, 3072, 12288), "tile_192", 4),
                                     ((512, 4096, 4096), "tile_128", 1), ((640, 4096, 2048), "tile_128", 1),
                                     ((896, 4096, 4096), "tile_128", 1), ((2048, 2048, 2048), "tile_128", 1),
                                     ((512, 2048, 16384), "tile_128", 4), ((384, 3072, 8192), "tile_128", 3),
                                     ((512, 3072, 8192), "tile_128", 2), ((512, 3072, 4096), "tile_128", 2),
                                     ((256, 4096, 4096), "tile_128", 4), ((512, 1024, 8192), "tile_128", 8),
                                     ((128, 8192, 8192), "tile_128", 4), ((384, 2048, 4096), "tile_128", 5),
                                     ((1024, 4096, 11008), "tile_128", 1), ((1024, 4096, 6144), "tile_128", 1),
                                     ((1024, 4096, 4096), "tile_128", 1), ((896, 4096, 11008), "tile_128", 1),
                                     # (96 .. 128 tiles: whole up to 64 K tiles, in two parts from 80 on)
                                     ((512, 4096, 5120), "tile_128", 2), ((512, 4096, 6144), "tile_128", 2),
                                     ((512, 4096, 3072), "tile_128", 1)):
        rc, p = _plan(_operand(capi.BF16, (m, k)), _operand(capi.BF16, (n, k)), _operand(capi.BF16, (m, n)))
        assert rc == 0 and capi.FAMILY_NAMES[p.family] == family and p.split_k == split, (m, n, k, p.family, p.split_k)
        assert p.workspace_bytes == (split * m * n * 4 if split > 1 else 0)
    # 16-bit operands with B as [K,N] (strides (1, N)) are served too (the tile lies [k][n] in LDS) and plan alike
    for (m, n, k), family, split in (((768, 4096, 4096), "tile_128", 1), ((512, 4096, 4096), "tile_128", 1),
                                     ((1024, 4096, 11008), "tile_128", 1), ((1024, 4096, 6144), "tile_128", 1),
                                     ((512, 2048, 16384), "tile_128", 4), ((768, 3072, 12288), "tile_192", 4)):
        rc, p = _plan(_operand(capi.BF16, (m, k)), _operand(capi.BF16, (n, k), strides=(1, n)), _operand(capi.BF16, (m, n)))
        assert rc == 0 and capi.FAMILY_NAMES[p.family] == family and p.split_k == split, (m, n, k, p.family, p.split_k)
    # operands it does not serve keep the two-stage kernel's rules: a K that is not whole K tiles - K split so that two
    # workgroups sit on (nearly) every unit, from twenty K tiles per part; the big tile in four parts for 64 of them and
    # a long K
    for (m, n, k), family, split in (((768, 4096, 4104), "tile_128", 2), ((512, 4096, 4104), "tile_64", 1),
                                     ((1024, 4096, 11016), "tile_256", 4), ((1024, 4096, 6152), "tile_128", 2),
                                     ((512, 2048, 16392), "tile_128", 8)):
        rc, p = _plan(_operand(capi.BF16, (m, k)), _operand(capi.BF16, (n, k)), _operand(capi.BF16, (m, n)))
        assert rc == 0 and capi.FAMILY_NAMES[p.family] == family and p.split_k == split, (m, n, k, p.family, p.split_k)
    for (m, n, k), family, split in (((1024, 4096, 11008), "tile_128", 1), ((1024, 4096, 8192), "tile_128", 1),
                                     ((768, 4096, 4096), "tile_128", 1), ((768, 3072, 12288), "tile_128", 1),
                                     ((512, 2048, 16384), "tile_128", 4), ((512, 1024, 8192), "tile_64", 2)):
        rc, p = _plan(_operand(capi.I8, (m, k)), _operand(capi.I8, (n, k)), _operand(capi.I32, (m, n)))
        assert rc == 0 and capi.FAMILY_NAMES[p.family] == family and p.split_k == split, (m, n, k, p.family, p.split_k)
    # fp32 compute: a part-filled round of 128 x 128 tiles (up to 192) loses to four times as many 64 x 64 ones - the
    # fullest unit's tiles times their area decide; a full round keeps the bigger tile
    for n, family in ((1536, "tile_64"), (1664, "tile_64"), (1792, "tile_128"), (2048, "tile_128"), (1024, "tile_64")):
        rc, p = _plan(_operand(capi.F32, (n, n)), _operand(capi.F32, (n, n)), _operand(capi.F32, (n, n)), compute=1)
        assert rc == 0 and capi.FAMILY_NAMES[p.family] == family and p.split_k == 1, (n, p.family, p.split_k)
    # two rounds of 128 x 128 tiles and eight more: the last column of tiles is a product of its own (64 x 64 tiles, K in
    # five parts), the rest fills two rounds; a required family runs the product whole
    # (B as [K,N]: with B [N,K] these extents take the 256 x 352 tile, 192 of them in one round)
    big_n = (_operand(capi.BF16, (1536, 4096)), _operand(capi.BF16, (11008, 4096), strides=(1, 11008)), _operand(capi.BF16, (1536, 11008)))
    rc, p = _plan(*big_n)
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_128" and p.split_k == 1 and p.peeled_columns == 128
    assert p.workspace_bytes == 5 * 1536 * 128 * 4
    rc, p = _plan_family(*big_n, "tile_128", capi.SELECT_REQUIRE)
    assert rc == 0 and p.peeled_columns == 0 and p.workspace_bytes == 0
    rc, p = _plan(_operand(capi.BF16, (2048, 4096)), _operand(capi.BF16, (11008, 4096), strides=(1, 11008)), _operand(capi.BF16, (2048, 11008)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_128" and p.peeled_columns == 0   # 1376 tiles: the third round is two thirds full
    # a split must pay for its second kernel: sixteen or thirty-two K tiles are walked in one go, sixty-four are not
    for (m, n, k), split in (((384, 384, 1024), 1), ((640, 640, 2048), 1), ((512, 512, 4096), 4), ((64, 64, 65536), 64)):
        rc, p = _plan(_operand(capi.BF16, (m, k)), _operand(capi.BF16, (n, k)), _operand(capi.F32, (m, n)))
        assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_64" and p.split_k == split, (m, n, k, p.split_k)
    # empty problems
    rc, p = _plan(_operand(capi.BF16, (0, 64)), _operand(capi.BF16, (8, 64)), _operand(capi.F32, (0, 8)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "none"
    rc, p = _plan(_operand(capi.BF16, (4, 0)), _operand(capi.BF16, (8, 0)), _operand(capi.F32, (4, 8)))
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "zero_k"
    # B handed over as [K,N] row-major
    rc, p = _plan(_operand(capi.BF16, (512, 512)), _operand(capi.BF16, (512, 512), (1, 512)),
                  _operand(capi.F32, (512, 512)))
    assert rc == 0 and p.b_layout == 1


def test_plan_validation():
    rc, _ = _plan(_operand(capi.BF16, (4, 8)), _operand(capi.BF16, (5, 9)), _operand(capi.F32, (4, 5)))
    assert rc == 1 and b"K of a" in capi.lib().vecops_hip_last_error()
    rc, _ = _plan(_operand(capi.BF16, (4, 8)), _operand(capi.BF16, (5, 8)), _operand(capi.F32, (4, 6)))
    assert rc == 1
    rc, _ = _plan(_operand(capi.BF16, (2, 4, 8)), _operand(capi.BF16, (3, 5, 8)), _operand(capi.F32, (2, 4, 5)))
    assert rc == 1                                           # batch extents differ
    rc, _ = _plan(_operand(capi.BF16, (4, 8)), _operand(capi.I8, (5, 8)), _operand(capi.F32, (4, 5)))
    assert rc == 2                                           # NotApplicable: another recipe may take it
    rc, _ = _plan(_operand(capi.I8, (4, 8)), _operand(capi.I8, (5, 8)), _operand(capi.F32, (4, 5)))
    assert rc == 2


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIB_PATH", "/nonexistent/libvecops_hip.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        capi.lib()


def _plan_family(a, b, c, family, selection, split_k=0):
    plan = capi.Plan()
    request = capi.family_request(family, selection, split_k)
    rc = capi.lib().vecops_hip_plan_matmul_family(C.byref(a), C.byref(b), None, C.byref(c), 0, C.byref(request), C.byref(plan))
    return rc, plan


def test_family_request_known_answers():
    """The explicit family request (vecops' family_selection::Prefer / Require) is part of the pure planning function."""
    big = (_operand(capi.BF16, (4096, 4096)), _operand(capi.BF16, (4096, 4096)), _operand(capi.BF16, (4096, 4096)))
    for family in ("tile_256", "tile_128", "tile_64", "tile_256x128", "tile_128x256"):
        rc, p = _plan_family(*big, family, capi.SELECT_REQUIRE)
        assert rc == 0 and capi.FAMILY_NAMES[p.family] == family and p.split_k == 1 and p.workspace_bytes == 0
    # a required family that cannot serve: not applicable; preferred: the rule table's own answer
    rc, _ = _plan_family(*big, "skinny", capi.SELECT_REQUIRE)
    assert rc == 2 and b"skinny" in capi.lib().vecops_hip_last_error()
    rc, p = _plan_family(*big, "skinny", capi.SELECT_PREFER)
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_256"
    rc, _ = _plan_family(*big, "zero_k", capi.SELECT_REQUIRE)
    assert rc == 2
    # the caller's K split: clamped to the K tiles there are (4096 / 64 = 64), partial sums in the workspace
    rc, p = _plan_family(*big, "tile_128", capi.SELECT_REQUIRE, split_k=4)
    assert rc == 0 and p.split_k == 4 and p.workspace_bytes == 4 * 4096 * 4096 * 4
    rc, p = _plan_family(*big, "tile_128", capi.SELECT_REQUIRE, split_k=1000)
    assert rc == 0 and p.split_k == 64
    # the skinny family on a decode shape; a tile family required there instead
    skinny = (_operand(capi.BF16, (4, 4096)), _operand(capi.BF16, (14336, 4096)), _operand(capi.F32, (4, 14336)))
    rc, p = _plan_family(*skinny, "skinny", capi.SELECT_REQUIRE)
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "skinny"
    rc, p = _plan_family(*skinny, "tile_64", capi.SELECT_REQUIRE)
    assert rc == 0 and capi.FAMILY_NAMES[p.family] == "tile_64"
    # malformed requests
    request = capi.family_request(10, capi.SELECT_REQUIRE)
    plan = capi.Plan()
    assert capi.lib().vecops_hip_plan_matmul_family(C.byref(big[0]), C.byref(big[1]), None, C.byref(big[2]), 0,
                                                    C.byref(request), C.byref(plan)) == 1
    request = capi.family_request("tile_64", 5)
    assert capi.lib().vecops_hip_plan_matmul_family(C.byref(big[0]), C.byref(big[1]), None, C.byref(big[2]), 0,
                                                    C.byref(request), C.byref(plan)) == 1
    # no request = automatic
    assert capi.lib().vecops_hip_plan_matmul_family(C.byref(big[0]), C.byref(big[1]), None, C.byref(big[2]), 0, None,
                                                    C.byref(plan)) == 0 and capi.FAMILY_NAMES[plan.family] == "tile_256"
