"""Host model of the index arithmetic of the two kernels of a one-token decode step (k_w13_token and
k_w2_combine_token, promoe_amd/csrc/moe_kernels.hip) and of their launcher (moe_decode_token_int4), swept over
layer shapes.

For every workgroup of the w13 launch the model restates which (class, unit, block) it takes
(gemv_resolve_route_n: routed workgroups first, then the publisher, then the shared expert's), the byte
ranges of its buffer descriptors inside the expert image, every offset a lane sends through them, every
offset into the wave-private LDS areas against the dynamic LDS size the launcher passes, the output elements
against the extents of h_r / h_s, and what the publishing workgroup stores against the sizes
moe_forward_prepare allocates.  For the w2 + combine launch it walks the load cursor of all 16 waves and
checks that every (unit, pair of groups) is read exactly once, that every in-range offset of the four
descriptors of a load lies inside the image / the h vector, and that items past a unit's last group fall
outside the descriptor (they read zeros).  Any index outside its buffer fails the sweep.
"""
import itertools
import os
import re

import pytest

from promoe_amd import layout as LY

# The model's constants come out of the kernel source, and the rules it restates (launcher choices, block order,
# workgroup -> rows mapping) are checked to stand in the source word for word: a change there fails this file
# until the model follows.
_SRC = open(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "promoe_amd", "csrc",
                         "moe_kernels.hip")).read()


def _define(name):
    m = re.search(r"^#define %s(\([a-z]+\))? +(.+?)(?: *//.*)?$" % name, _SRC, re.M)
    assert m, "no #define %s in moe_kernels.hip" % name
    return m.group(2).strip()


def _source_has(*lines):
    flat = " ".join(_SRC.split())
    for ln in lines:
        assert " ".join(ln.split()) in flat, "moe_kernels.hip no longer contains: " + ln


_W13T_WAVE_DW = _define("W13T_WAVE_DW")          # an expression in (ch)
W2C_WAVES = int(_define("W2C_WAVES"))
GATE_PARTS = int(_define("GATE_PARTS"))
GATE_COPY_WORDS = int(_define("GATE_COPY_WORDS"))


def test_restated_rules_stand_in_the_source():
    _source_has(
        # launcher: tiles in flight per wave of k_w13_token, its LDS size, its grid
        "int ch = gpw >= 4 ? ((gpw % 4 == 0) ? 4 : (gpw % 3 == 0 ? 3 : 4)) : gpw;",
        "static size_t w13_token_lds(int ch) { return (size_t)4 * W13T_WAVE_DW(ch) * 4 + 4 * 2 * 16 * 4; }",
        "int grid = a.n_sh_blocks + k * (I / 16) + 1;",
        "a.g_nblk = GATE_PARTS * ((n_gate_rows + 3) / 4);",
        # block order of k_w13_token: gate workgroups, routed, publisher, shared
        "if ((int)blockIdx.x < a.g_nblk) {",
        "const int n_rt = k * a.cls[1].nblk + 1;",
        "const bool publisher = !sh && rr == k * wk.c.nblk;",
        "const int e = ((int)blockIdx.x >> 3) * 4 + w;",
        # launcher of k_w2_combine_token and its workgroup -> rows mapping
        "const int loads_per_wave = (k * ((c.G + 1) / 2) + (c.G_sh + 1) / 2 + W2C_WAVES - 1) / W2C_WAVES;",
        "if (loads_per_wave <= 3) hipLaunchKernelGGL((k_w2_combine_token<2, 3>), dim3(H / 8)",
        "else if (H / 16 >= 256)",
        "if (NI == 2 && (gridDim.x & 15) == 0) {",
        "b16 = (q >> 1) * 8 + ((int)blockIdx.x & 7);",
        "extern \"C\" int64_t moe_gate_ws_bytes(void) { return (int64_t)GATE_COPIES * GATE_COPY_WORDS * 8; }",
        "#define GATE_COPIES (GATE_PARTS + 1)")


def w13_wave_dw(ch):
    return int(eval(_W13T_WAVE_DW, {"ch": ch}))


def w13_token_lds(ch):
    return 4 * w13_wave_dw(ch) * 4 + 4 * 2 * 16 * 4


def launcher_ch(H):
    gpw = (H // 128 + 3) // 4
    ch = (4 if gpw % 4 == 0 else (3 if gpw % 3 == 0 else 4)) if gpw >= 4 else gpw
    return max(ch, 1)


def model_route_launch(E, k, H, I, I_sh):
    """k_w13_token<CH>.  Returns the number of working workgroups checked; asserts on any out-of-range index."""
    lay_r = LY.int4_layout(H, I)
    lay_s = LY.int4_layout(H, I_sh) if I_sh else None
    K, G = H, H // 128
    n_sh = I_sh // 16 if I_sh else 0
    nblk_r = I // 16
    n_rt = k * nblk_r + 1
    grid = n_sh + k * nblk_r + 1
    CH = launcher_ch(H)
    lds = w13_token_lds(CH)
    assert lds <= 64 * 1024
    WDW = w13_wave_dw(CH)
    # a wave's LDS area in dwords: xs [CH][64], xsum [CH][4], wsc [2CH][8], wzz [2CH][2]; red behind the four areas
    o_xsum, o_wsc, o_wzz = CH * 64, CH * 68, CH * 68 + CH * 16
    assert o_wzz + CH * 4 == WDW and (4 * WDW + 4 * 2 * 16) * 4 == lds
    for lane in range(64):
        r, qd = lane & 15, lane >> 4
        xj, scj, zzj = lane >> 4, lane >> 3, lane >> 1
        if xj < CH:                                   # ((uint4 *)xs)[lane], xsum[lane >> 2]
            assert (lane + 1) * 4 <= o_xsum and o_xsum + (lane >> 2) < o_wsc
        if scj < 2 * CH:
            assert o_wsc + lane < o_wzz               # wsc[lane]
        if zzj < 2 * CH:
            assert o_wzz + lane < WDW                 # wzz[lane]
        for j in range(CH):                           # reads in front of the products
            assert (max(j, CH + j) * 16 + r) * 2 + 2 <= (o_wzz - o_wsc) * 4     # wsc_h[(CH + j) * 16 + r]
            assert (CH + j) * 8 + (r >> 1) < (WDW - o_wzz) * 4                  # wzz_b[(CH + j) * 8 + (r >> 1)]
            assert (j * 128 + qd * 32 + 32) * 2 <= o_xsum * 4                   # 4 x uint4 at xs + j*128 + qd*32
            assert j * 4 + qd < o_wsc - o_xsum                                  # xsum[j * 4 + qd]
    assert (3 * 2 + 1) * 16 + 15 < 4 * 2 * 16                                   # red[(w * 2 + ab) * 16 + lane]
    # offsets a wave sends through its descriptors (lengths: K * 2, 2 G KiB, 2 G * 32, 2 G * 8)
    for w in range(4):
        GPW = (G - w + 3) >> 2
        assert GPW <= (G + 3) // 4
        for jc in range(0, GPW, CH):
            for j in range(CH):
                g = w + 4 * (jc + j) if jc + j < GPW else 0
                assert 0 <= g < G
                assert g * 256 + 15 * 16 + 16 <= K * 2
                for half in (0, G):
                    assert ((half + g) * 8 + 7) * 4 + 4 <= 2 * G * 32
                    assert ((half + g) * 2 + 1) * 4 + 4 <= 2 * G * 8
                    assert 63 * 16 + (half + g) * 1024 + 16 <= 2 * G * 1024
    # gate workgroups in front of the grid (launches that sum the gate rows themselves): eight per block of four
    # rows; a wave writes word e of one of GATE_PARTS + 1 copies of GATE_COPY_WORDS words
    for rows in (E, E + 1):
        g_nblk = GATE_PARTS * ((rows + 3) // 4)
        covered = set()
        for bxg in range(g_nblk):
            for w in range(4):
                e = (bxg >> 3) * 4 + w
                if e < rows:
                    covered.add((bxg & 7, e))
                    assert e < GATE_COPY_WORDS
                    for copy in range(GATE_PARTS + 1):
                        assert (copy * GATE_COPY_WORDS + e) * 8 + 8 <= (GATE_PARTS + 1) * GATE_COPY_WORDS * 8
        # with workgroup i on part i mod 8 of the chip, every part sums every row
        assert covered == {(p_, e) for p_ in range(GATE_PARTS) for e in range(rows)}
    n_checked = 0
    n_pub = 0
    for bx in range(grid):
        sh = bx >= n_rt
        rr = bx - n_rt if sh else bx
        nblk = (I_sh // 16) if sh else nblk_r
        publisher = (not sh) and rr == k * nblk
        u = 0 if (sh or publisher) else rr // nblk
        b = rr - u * nblk
        if publisher:
            n_pub += 1
            continue            # m = 0: returns before any weight or LDS access
        lay = lay_s if sh else lay_r
        rows_out, out_stride = (1, I_sh) if sh else (k, I)
        assert 0 <= u < (1 if sh else k) and 0 <= b < nblk, (bx, u, b)
        rbA = 2 * b
        # the three descriptors over the image: section offset + rbA * G * bytes-per-tile, two blocks long
        for off, nxt, per_tile in (("off13_q", "off13_s", 1024), ("off13_s", "off13_z", 32), ("off13_z", "off2_q", 8)):
            lo = lay[off] + rbA * G * per_tile
            assert lay[off] <= lo and lo + 2 * G * per_tile <= lay[nxt], (bx, off)
        # output: h[row0 * out_stride + b * 16 + tid], tid < 16; row0 = u (routed) or 0 (shared)
        row0 = 0 if sh else u
        assert row0 * out_stride + b * 16 + 15 < rows_out * out_stride, (bx, row0, b)
        n_checked += 1
    assert n_checked == grid - 1 and n_pub == 1
    # what the publisher stores, against moe_forward_prepare's allocations for max_tokens >= 1
    P = k                                   # T = 1
    max_units = min(E, P)
    for pos in range(k):                    # one lane per selected expert, pos = its rank among them
        assert pos < max_units              # units[pos], active_ids[pos], pinned unit list [max_units]
        assert pos < P                      # sorted_pair[pos], sorted_tok[pos]; idx / w / pos_of_pair [lane < k]
        assert 16 * (pos + 1) <= 16 * k and 16 * k + 4 * (pos + 1) <= 32 * max(k, 1)   # unit_ws: KUnit[k] then float[k]
    # counts[e], offsets[e] for e < E, offsets[E]: arrays of E and E + 1 ints
    return n_checked


def w2c_rows_of(bx, grid, NI):
    """(b16, part) of workgroup bx (k_w2_combine_token): pairs that share a tile get indices equal mod 8."""
    b16, part = bx // NI, bx % NI
    if NI == 2 and grid % 16 == 0:
        q = bx >> 3
        part, b16 = q & 1, (q >> 1) * 8 + (bx & 7)
    return b16, part


def launcher_w2c(k, H, I, I_sh):
    G, G_sh = I // 128, (I_sh // 128 if I_sh else 0)
    loads_per_wave = (k * ((G + 1) // 2) + (G_sh + 1) // 2 + W2C_WAVES - 1) // W2C_WAVES
    if loads_per_wave <= 3:
        return 2, 3
    if H // 16 >= 256:
        return 1, 7
    return 2, 6


def model_w2_combine_launch(k, H, I, I_sh, NI=2, CHUNK=3):
    """k_w2_combine_token<NI, CHUNK>: grid H / (16 / NI); LDS = per wave the activations and 32-wide sums of a
    chunk's items, then the waves' partial sums."""
    RW = 16 // NI
    G, G_sh = I // 128, (I_sh // 128 if I_sh else 0)
    lay_r = LY.int4_layout(H, I)
    lay_s = LY.int4_layout(H, I_sh) if I_sh else None
    WAVE_DW = CHUNK * NI * 64 + CHUNK * NI * 4
    lds = W2C_WAVES * (CHUNK * NI * 68) * 4 + W2C_WAVES * 16 * 4
    assert lds <= 150 * 1024 and k < 64 and H % 16 == 0
    assert (W2C_WAVES * WAVE_DW + W2C_WAVES * RW) * 4 <= lds        # red[w * RW + lane], lane < RW
    GP, GP_sh = (G + NI - 1) // NI, (G_sh + NI - 1) // NI
    # ---- the load cursor of every wave: which (unit, load) it requests, chunk by chunk ----
    seen = {}
    max_gp = 0
    for w in range(W2C_WAVES):
        u, gp = 0, w
        while u < k and gp >= GP:
            gp -= GP; u += 1
        trips = 0
        while u < k or gp < GP_sh:
            trips += 1
            assert trips <= 4096
            for c in range(CHUNK):
                valid = u < k or gp < GP_sh
                assert 0 <= u <= k            # readlane(ub, u): lane k holds the shared expert, k < 64
                if valid:
                    shd = u >= k
                    assert gp < (GP_sh if shd else GP)
                    key = (u, gp)
                    assert key not in seen, key
                    seen[key] = w
                    max_gp = max(max_gp, gp)
                    gp += W2C_WAVES
                    while u < k and gp >= GP:
                        gp -= GP; u += 1
                else:
                    assert u == k and gp < GP_sh + W2C_WAVES   # an absent load: descriptors of length 0
    want = {(u, gp) for u in range(k) for gp in range(GP)} | {(k, gp) for gp in range(GP_sh)}
    assert set(seen) == want
    # ---- per-lane offsets of one load against its four descriptors ----
    grid = H // RW
    for shd, Gu, lay, GPu in ((False, G, lay_r, GP), (True, G_sh, lay_s, GP_sh)):
        if Gu == 0:
            continue
        # the image holds H / 16 row blocks of Gu tiles each; a descriptor covers block b16's Gu tiles
        assert lay["off2_q"] + (H // 16) * Gu * 1024 <= lay["off2_s"]
        assert lay["off2_s"] + (H // 16) * Gu * 32 <= lay["off2_z"]
        assert lay["off2_z"] + (H // 16) * Gu * 8 <= lay["total_bytes"]
        for gp in range(GPu):
            g0 = NI * gp
            for part in range(NI):
                for lane in range(64):
                    r, qd = lane & 15, lane >> 4
                    mine, rr = r // RW, RW * part + (r % RW)
                    assert mine < NI and rr < 16
                    item_exists = g0 + mine < Gu
                    vq = mine * 1024 + (qd * 16 + rr) * 16 + g0 * 1024
                    vs = mine * 32 + 2 * rr + g0 * 32
                    vz = mine * 8 + (rr >> 1) + g0 * 8
                    # inside the descriptor exactly when the item exists (otherwise the load returns 0)
                    assert (vq + 16 <= Gu * 1024) == item_exists, (gp, lane)
                    assert (vs + 2 <= Gu * 32) == item_exists
                    assert (vz + 1 <= Gu * 8) == item_exists
                    lj, lpart = lane >> 4, lane & 15
                    if lj < NI:
                        vh = lj * 256 + lpart * 16 + g0 * 256
                        assert (vh + 16 <= Gu * 256) == (g0 + lj < Gu)
                        # wave-private LDS: ((uint4 *)hs)[(c * NI + lj) * 16 + lpart], xsum[(c * NI + lj) * 4 + (lpart >> 2)]
                        c = CHUNK - 1
                        assert ((c * NI + lj) * 16 + lpart + 1) * 4 <= CHUNK * NI * 64
                        assert CHUNK * NI * 64 + (c * NI + lj) * 4 + (lpart >> 2) < WAVE_DW
                    c = CHUNK - 1
                    assert ((c * NI + mine) * 128 + qd * 32 + 32) * 2 <= CHUNK * NI * 64 * 4
                    assert (c * NI + mine) * 4 + qd < CHUNK * NI * 4
    # the h vectors behind the rh descriptors: unit u's I values inside h_r [k, I], the shared expert's inside h_s
    for u in range(k):
        assert u * I + G * 128 <= k * I
    assert G_sh * 128 <= max(I_sh, 0)
    # output rows: every (tile, part) exactly once
    seen_rows = set()
    for bx in range(grid):
        b16, part = w2c_rows_of(bx, grid, NI)
        assert 0 <= part < NI and 0 <= b16 < H // 16 and b16 * 16 + RW * part + RW - 1 < H
        seen_rows.add((b16, part))
    assert len(seen_rows) == grid == (H // 16) * NI
    return grid


SHAPES = [
    # E, k, H, I, I_sh
    (64, 6, 2048, 1408, 2816),    # DeepSeek-MoE-16B
    (60, 4, 2048, 1408, 5632),    # Qwen1.5-MoE
    (8, 2, 4096, 14336, 0),       # Mixtral (H = 4096 is the largest hidden size the one-token path takes)
    (4, 4, 128, 128, 0),          # smallest legal shape, k = E
    (4, 1, 128, 128, 128),
    (200, 8, 512, 128, 0),        # E > 128: four logit columns
    (256, 32, 256, 256, 256),     # the limits of E and k
    (16, 6, 2048, 1408, 2816),
    (3, 3, 384, 640, 128),        # odd group counts per wave
    (65, 6, 2304, 2176, 2560),    # E just above one logit column, K not a multiple of 512
]


@pytest.mark.parametrize("E,k,H,I,I_sh", SHAPES)
def test_one_token_launch_stays_inside_its_buffers(E, k, H, I, I_sh):
    n = model_route_launch(E, k, H, I, I_sh)
    assert n == (I_sh // 16 if I_sh else 0) + k * (I // 16)
    if k < 64 and H % 16 == 0:                       # the rule of moe_forward for the fused w2 + combine pass
        ni, chunk = launcher_w2c(k, H, I, I_sh)
        model_w2_combine_launch(k, H, I, I_sh, ni, chunk)
        for ni, chunk in ((2, 3), (1, 7), (2, 6)):   # every instantiation, whatever the launcher would pick
            model_w2_combine_launch(k, H, I, I_sh, ni, chunk)


def test_sweep_of_small_shapes():
    n = 0
    for H, I, I_sh, (E, k) in itertools.product((128, 256, 640), (128, 384), (0, 128, 512), ((1, 1), (5, 2), (64, 6), (130, 7))):
        model_route_launch(E, k, H, I, I_sh)
        model_w2_combine_launch(k, H, I, I_sh, *launcher_w2c(k, H, I, I_sh))
        n += 1
    assert n == 72
