"""Host model of the index arithmetic of the one-token decode GEMV (k_gemv_int4 with in-kernel routing,
promoe_amd/csrc/moe_kernels.hip) and of its launcher (moe_decode_token_int4), swept over layer shapes.

For every workgroup of the launch the model restates which (class, unit, block) it takes, the byte ranges
of its three buffer resources inside the expert image, every LDS offset it stages to or reads from against
the dynamic LDS size the launcher passes, the output elements it stores against the extents of h_r / h_s,
and what the publishing workgroup stores against the sizes moe_forward_prepare allocates.  Any index
outside its buffer fails the sweep.  The w2 + combine kernel of the same step is modelled the same way.
"""
import itertools

import pytest

from promoe_amd import layout as LY


def gemv_lds(tmax, K):
    G = K // 128
    return tmax * K * 2 + tmax * (K // 32) * 4 + 2 * G * 32 + 2 * G * 8 + 4 * tmax * 2 * 16 * 4


def model_route_launch(E, k, H, I, I_sh):
    """Returns the number of workgroups checked; asserts on any out-of-range index."""
    lay_r = LY.int4_layout(H, I)
    lay_s = LY.int4_layout(H, I_sh) if I_sh else None
    K, G = H, H // 128
    n_sh = I_sh // 16 if I_sh else 0
    nblk_r = I // 16
    grid = n_sh + k * nblk_r + 1
    lds = gemv_lds(1, H)
    assert lds <= 64 * 1024
    # LDS carve-up of the kernel (TMAX = 1)
    o_xs, o_xsum = 0, K * 2
    o_sc = o_xsum + (K // 32) * 4
    o_zz = o_sc + 2 * G * 32
    o_red = o_zz + 2 * G * 8
    assert o_red + 4 * 1 * 2 * 16 * 4 <= lds
    vec_per_row, n_sc, n_zz = K // 8, 2 * G * 32 // 4, 2 * G * 8 // 4
    # staging stores, all 256 threads
    for tid in range(256):
        if tid < vec_per_row:
            assert o_xs + (tid + 1) * 16 <= o_xsum
            assert o_xsum + ((tid >> 2) + 1) * 4 <= o_sc
        for v in range(tid + 256, vec_per_row, 256):
            assert o_xs + (v + 1) * 16 <= o_xsum and o_xsum + ((v >> 2) + 1) * 4 <= o_sc
        for i in [tid, tid + 256] + list(range(tid + 512, n_sc, 256)):
            if i < n_sc:
                assert o_sc + (i + 1) * 4 <= o_zz
        for i in [tid] + list(range(tid + 256, n_zz, 256)):
            if i < n_zz:
                assert o_zz + (i + 1) * 4 <= o_red
    # reads of the product loop: every wave w, group g = w + 4j < G, lane (r, qd)
    for w in range(4):
        for g in range(w, G, 4):
            for qd in range(4):
                assert (g * 128 + qd * 32 + 32) * 2 <= o_xsum - o_xs
                assert (g * 4 + qd + 1) * 4 <= o_sc - o_xsum
            for r in range(16):
                assert ((G + g) * 16 + r + 1) * 2 <= o_zz - o_sc
                assert (G + g) * 8 + (r >> 1) + 1 <= o_red - o_zz
    # reduction buffer: red[((w*TMAX + t)*2 + ab)*16 + lane], lane < 16
    assert ((3 * 1 + 0) * 2 + 1) * 16 + 15 < 4 * 1 * 2 * 16

    n_checked = 0
    for bx in range(grid):
        sh = bx < n_sh
        rr = bx if sh else bx - n_sh
        nblk = (I_sh // 16) if sh else nblk_r
        publisher = (not sh) and rr == k * nblk
        u = 0 if (sh or publisher) else rr // nblk
        b = rr - u * nblk
        if publisher:
            continue            # m = 0: returns before any weight or LDS access
        lay = lay_s if sh else lay_r
        rows_out, out_stride = (1, I_sh) if sh else (k, I)
        assert 0 <= u < (1 if sh else k) and 0 <= b < nblk
        rbA = 2 * b
        # the three buffer resources: base + section offset + rbA * G * bytes-per-tile, two blocks long
        for off, nxt, per_tile in (("off13_q", "off13_s", 1024), ("off13_s", "off13_z", 32), ("off13_z", "off2_q", 8)):
            lo = lay[off] + rbA * G * per_tile
            assert lay[off] <= lo and lo + 2 * G * per_tile <= lay[nxt], (bx, off)
        # weight tiles: lane * 16 + g * 1024 and (G + g) * 1024 inside the 2 G KiB range
        assert 63 * 16 + 16 + (G + G - 1) * 1024 <= 2 * G * 1024
        # output: h[(row0 + t) * out_stride + b * 16 + r], row0 = u (routed) or 0 (shared), t = 0
        row0 = 0 if sh else u
        assert row0 * out_stride + b * 16 + 15 < rows_out * out_stride, (bx, row0, b)
        n_checked += 1
    assert n_checked == grid - 1
    # what the publisher stores, against moe_forward_prepare's allocations for max_tokens >= 1
    P = k                                   # T = 1
    max_units = min(E, P)
    for pos in range(k):                    # one lane per selected expert, pos = its rank among them
        assert pos < max_units              # units[pos], active_ids[pos], pinned unit list [max_units]
        assert pos < P                      # sorted_pair[pos], sorted_tok[pos]; idx / w / pos_of_pair [lane < k]
        assert 16 * (pos + 1) <= 16 * k and 16 * k + 4 * (pos + 1) <= 32 * max(k, 1)   # unit_ws: KUnit[k] then float[k]
    # counts[e], offsets[e] for e < E, offsets[E]: arrays of E and E + 1 ints
    return n_checked


def model_w2_combine_launch(k, H, I, I_sh, NI=2):
    """k_w2_combine_token<NI>: grid H / (16 / NI), LDS = staged h vectors + 32-wide sums + reduction."""
    RW = 16 // NI
    G, G_sh = I // 128, (I_sh // 128 if I_sh else 0)
    lay_r = LY.int4_layout(H, I)
    lay_s = LY.int4_layout(H, I_sh) if I_sh else None
    n_h = k * I + I_sh
    lds = n_h * 2 + (n_h // 32) * 4 + 16 * 16 * 4
    assert lds <= 150 * 1024
    o_xsum = n_h * 2
    o_red = o_xsum + (n_h // 32) * 4
    assert o_red + 16 * RW * 4 <= lds
    nvec = n_h // 8
    for v in range(nvec):                     # staging: vector v of the concatenated h vectors
        el = v * 8
        assert (el + 8 <= k * I) or (el >= k * I and el - k * I + 8 <= I_sh), v   # never straddles h_r | h_s
        assert (v + 1) * 16 <= o_xsum and ((v >> 2) + 1) * 4 <= o_red - o_xsum
    grid = H // RW
    for bx in range(grid):
        b16, part = bx // NI, bx % NI
        for r in range(16):
            rr = RW * part + (r % RW)
            assert rr < 16
            # items: (unit u < k, group g < G) and (shared, g < G_sh)
            for shd, Gu, lay in ((False, G, lay_r), (True, G_sh, lay_s)):
                if Gu == 0:
                    continue
                for lg in (0, Gu - 1):
                    t_idx = b16 * Gu + lg
                    for qd in range(4):
                        assert lay["off2_q"] + t_idx * 1024 + (qd * 16 + rr) * 16 + 16 <= lay["off2_s"]
                    assert lay["off2_s"] + t_idx * 32 + 2 * rr + 2 <= lay["off2_z"]
                    assert lay["off2_z"] + t_idx * 8 + (rr >> 1) + 1 <= lay["total_bytes"]
                    for u in ((k,) if shd else (0, k - 1)):
                        ho = (k * I if shd else u * I) + lg * 128
                        assert (ho + 3 * 32 + 32) <= n_h and ((ho + 96) >> 5) < n_h // 32
        # output rows of this workgroup
        assert b16 * 16 + RW * part + RW - 1 < H
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
    n_h = k * I + I_sh
    if n_h * 2 + (n_h // 32) * 4 + 1024 <= 150 * 1024:   # the rule of moe_forward for the fused w2 + combine pass
        for NI in (1, 2, 4):
            model_w2_combine_launch(k, H, I, I_sh, NI)


def test_sweep_of_small_shapes():
    n = 0
    for H, I, I_sh, (E, k) in itertools.product((128, 256, 640), (128, 384), (0, 128, 512), ((1, 1), (5, 2), (64, 6), (130, 7))):
        model_route_launch(E, k, H, I, I_sh)
        model_w2_combine_launch(k, H, I, I_sh, 2)
        n += 1
    assert n == 72
