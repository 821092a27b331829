"""The decode attention entry point that allocates nothing: its split-KV partials live in device memory that belongs to the
library.  It must give the results of lg_attn_decode_f16 (same kernels, caller-owned workspace) bit for bit, also on a
second call with a smaller input, which finds the first call's partials still in the shared array."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def rnd(po, n, tid, std=1.0):
    return po.fill_normal(n, 0, tid, 0.0, std, 1)


def run_pair(dev, po, B, h, d, L, Lmax, tid):
    q = dev.up(rnd(po, B * h * d, tid).reshape(B, h, d), 1)
    kc = dev.up(rnd(po, B * h * Lmax * d, tid + 1).reshape(B, h, Lmax, d), 1)
    vc = dev.up(rnd(po, B * h * Lmax * d, tid + 2).reshape(B, h, Lmax, d), 1)
    scalar = float(1.0 / np.sqrt(d))
    ws = dev.empty((dev.lib.lg_attn_decode_workspace_bytes(B, h, d, Lmax) // 4,), 0)
    want = dev.empty((B, h, d), 1)
    got = dev.empty((B, h, d), 1)
    got.fill_(-7.0)
    dev.call("lg_attn_decode_f16", q, kc, vc, want, ws, B, h, d, L, Lmax, scalar)
    dev.call("lg_attn_decode_static_f16", q, kc, vc, got, B, h, d, L, Lmax, scalar)
    return dev.down(got), dev.down(want)


def test_static_scratch_entry_matches_the_workspace_entry_twice(dev, po):
    # first call: 8 x 8 heads x 2048 keys -> 16 key splits, 1024 partial slots; second, smaller: 2 x 3 heads x 700 keys
    # -> 4 splits of other boundaries, which overwrite only part of what the first call left in the array
    for (B, h, d, L, Lmax, tid) in ((8, 8, 128, 2048, 2048, 300), (2, 3, 128, 700, 1024, 310), (3, 5, 96, 400, 512, 320),
                                    (40, 48, 64, 90, 128, 330)):
        got, want = run_pair(dev, po, B, h, d, L, Lmax, tid)
        assert np.array_equal(got, want), "B=%d h=%d d=%d L=%d" % (B, h, d, L)
    # and the oracle agrees with the last small case (the parity bar of the workspace entry itself)
    q = rnd(po, 2 * 3 * 128, 310).reshape(2, 3, 128)
    kc = rnd(po, 2 * 3 * 1024 * 128, 311).reshape(2, 3, 1024, 128)
    vc = rnd(po, 2 * 3 * 1024 * 128, 312).reshape(2, 3, 1024, 128)
    out = dev.empty((2, 3, 128), 1)
    dev.call("lg_attn_decode_static_f16", dev.up(q, 1), dev.up(kc, 1), dev.up(vc, 1), out, 2, 3, 128, 700, 1024, float(1 / np.sqrt(128)))
    ref = po.attn_decode(q, kc, vc, 700, 1 / np.sqrt(128), 1)
    assert float(np.abs(dev.down(out) - ref).max() / np.abs(ref).max()) < 1e-2


def test_static_scratch_entry_leaves_free_device_memory_unchanged(dev, po):
    """The property the entry exists for: after one warm-up call (the first call on a device looks the array's address up),
    calls of any size inside the limit change nothing in the device's free memory, and neither does the first call of a shape
    that was not seen before."""
    import torch
    B, h, d, Lmax = 8, 8, 128, 2048
    q = dev.up(rnd(po, B * h * d, 400).reshape(B, h, d), 1)
    kc = dev.up(rnd(po, B * h * Lmax * d, 401).reshape(B, h, Lmax, d), 1)
    vc = dev.up(rnd(po, B * h * Lmax * d, 402).reshape(B, h, Lmax, d), 1)
    out = dev.empty((B, h, d), 1)
    scalar = float(1.0 / np.sqrt(d))
    dev.call("lg_attn_decode_static_f16", q, kc, vc, out, B, h, d, 64, Lmax, scalar)     # warm-up
    dev.sync()
    free0 = torch.cuda.mem_get_info()[0]
    for (b, L) in ((8, 2048), (3, 700), (8, 1), (1, 2048), (5, 1333)):
        dev.call("lg_attn_decode_static_f16", q, kc, vc, out, b, h, d, L, Lmax, scalar)
        dev.sync()
        assert torch.cuda.mem_get_info()[0] == free0, "batch %d, %d keys changed the free device memory" % (b, L)


def test_static_scratch_entry_rejects_what_exceeds_its_maximum(dev):
    t = dev.empty((16,), 1)
    rc = dev.call_rc("lg_attn_decode_static_f16", t, t, t, t, 1, 1, 256, 8, 8, 1.0)
    assert rc == dev.capi.ERR_INVALID and "exceeds the maximum" in dev.capi.last_error()
