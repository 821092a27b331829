"""GPU parity for the attention kernels without a reference counterpart (decode over a KV cache, KV append)."""
import numpy as np
import pytest

from tests.conftest import max_rel_err

pytestmark = pytest.mark.gpu


def rnd(po, n, tid, std=1.0):
    return po.fill_normal(n, 0, tid, 0.0, std, 1)


@pytest.mark.parametrize("B,h,d,L,Lmax", [(2, 4, 128, 1024, 1024), (3, 2, 64, 100, 128), (1, 1, 128, 1, 8), (2, 3, 128, 37, 64),
                                           (1, 2, 128, 4096, 4096), (32, 48, 128, 129, 160)])
def test_attn_decode(dev, po, B, h, d, L, Lmax):
    q = rnd(po, B * h * d, 50).reshape(B, h, d)
    kc = rnd(po, B * h * Lmax * d, 51).reshape(B, h, Lmax, d)
    vc = rnd(po, B * h * Lmax * d, 52).reshape(B, h, Lmax, d)
    scalar = 1.0 / np.sqrt(d)
    ref = po.attn_decode(q, kc, vc, L, scalar, 1)
    ref32 = po.attn_decode(q, kc, vc, L, scalar, 0)
    ws_bytes = dev.lib.lg_attn_decode_workspace_bytes(B, h, d, Lmax)
    ws = dev.empty((max(1, ws_bytes // 4),), 0)
    out = dev.empty((B, h, d), 1)
    dev.call("lg_attn_decode_f16", dev.up(q, 1), dev.up(kc, 1), dev.up(vc, 1), out, ws, B, h, d, L, Lmax, float(scalar))
    got = dev.down(out)
    assert max_rel_err(got, ref) < 1e-2          # the stated tolerance against the fp16-semantics oracle
    assert max_rel_err(got, ref32) < 3e-3        # and close to the exact fp32 result


@pytest.mark.parametrize("B,h,d,pos,Lmax", [(4, 6, 128, 17, 64), (2, 2, 64, 0, 4)])
def test_kv_append(dev, po, B, h, d, pos, Lmax):
    n = h * d
    Q, K, V = (rnd(po, B * n, 53 + i).reshape(B, n) for i in range(3))
    bq, bk, bv = (rnd(po, n, 56 + i, 0.3) for i in range(3))
    kc0 = rnd(po, B * h * Lmax * d, 59).reshape(B, h, Lmax, d)
    vc0 = rnd(po, B * h * Lmax * d, 60).reshape(B, h, Lmax, d)
    dkc, dvc = dev.up(kc0, 1), dev.up(vc0, 1)
    dq = dev.empty((B, h, d), 1)
    dev.call("lg_kv_append_f16", dq, dkc, dvc, dev.up(Q, 1), dev.up(bq, 1), dev.up(K, 1), dev.up(bk, 1), dev.up(V, 1),
             dev.up(bv, 1), B, h, d, pos, Lmax)
    kc, vc = kc0.copy(), vc0.copy()
    kc[:, :, pos, :] = po.round_f16(K + bk).reshape(B, h, d)
    vc[:, :, pos, :] = po.round_f16(V + bv).reshape(B, h, d)
    assert np.array_equal(dev.down(dkc), kc)
    assert np.array_equal(dev.down(dvc), vc)
    assert np.array_equal(dev.down(dq), po.round_f16(Q + bq).reshape(B, h, d))
