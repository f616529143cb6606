"""The multi-threaded synthesis used for layers at the configured sizes must be the numpy path bit for
bit: quantiser against oracle.quantize_int4, slot image against layout.pack_expert_int4 (through the
exchange format), dequantiser against oracle.dequant_int4."""
import numpy as np
import torch

from oracle import moe_oracle as O
from promoe_amd import layout as LY
from tests import synth as S


def test_fast_int4_path_equals_numpy_path():
    H, I = 256, 384
    g = torch.Generator().manual_seed(3)
    ws = [torch.randn(n, k, generator=g) * 0.02 for n, k in ((I, H), (I, H), (H, I))]
    ws[0][5, 128:256] = 0.0          # an all-zero group (scale falls back to 1)
    ws[2][7, :128] = 0.013           # a constant group
    fast, ex = [], []
    for w in ws:
        q, s, z = S.fast_quantize_int4(w)
        qn, sn, zn = O.quantize_int4(w.numpy())
        assert np.array_equal(q.numpy(), qn) and np.array_equal(z.numpy(), zn)
        assert np.array_equal(s.numpy().view(np.uint16), sn.view(np.uint16))
        fast.append((q, s, z))
        qw, qz = O.pack_int4(qn, zn)
        ex.append((qw, sn, qz))
        n, k = w.shape
        assert np.array_equal(S.fast_dequant_int4(q, s, z).numpy(), O.dequant_int4(qw, sn, qz, n, k))
    assert np.array_equal(S.fast_pack_expert_int4(*fast, H, I), LY.pack_expert_int4(*ex, H, I))


def test_lazy_layer_alias_and_on_demand_dequantisation():
    a = S.LazyInt4Layer(256, 128, 4, I_sh=128, seed=1, zipf=1.1)
    b = S.LazyInt4Layer(256, 128, 4, I_sh=128, seed=2, alias_of=a, perm=[2, 0, 3, 1])
    assert np.array_equal(b.slots[0], a.slots[2]) and not np.array_equal(a.wg, b.wg)
    ex = a.experts_for(np.array([[1, 3]]))
    assert ex[0] is None and ex[2] is None and ex[1][0].shape == (128, 256) and ex[3][2].shape == (256, 128)
    assert np.array_equal(b.expert_fp32(1)[0], a.expert_fp32(0)[0])
    assert a.shared_fp32[0].shape == (128, 256)
