"""GPU parity for the attention kernels without a reference counterpart (decode over a KV cache, KV append)."""
import numpy as np
import pytest

from tests.conftest import max_rel_err

pytestmark = pytest.mark.gpu


def rnd(po, n, tid, std=1.0):
    return po.fill_normal(n, 0, tid, 0.0, std, 1)


@pytest.mark.parametrize("B,h,d,L,Lmax", [(2, 4, 128, 1024, 1024), (3, 2, 64, 100, 128), (1, 1, 128, 1, 8), (2, 3, 128, 37, 64),
                                           (1, 2, 128, 4096, 4096), (32, 48, 128, 129, 160), (2, 3, 96, 1000, 1024), (5, 4, 96, 33, 40),
                                           (1, 64, 96, 300, 300)])
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


def test_attn_decode_workspace_serves_every_smaller_batch(dev, po):
    """A workspace sized once for the largest batch must do for every smaller one, although a smaller batch may split its
    keys further (48 heads x 20 sequences use more partial slots than 48 x 32)."""
    h, d, L = 48, 128, 512
    size = dev.lib.lg_attn_decode_workspace_bytes(32, h, d, L)
    for B in (1, 7, 20, 32):
        assert dev.lib.lg_attn_decode_workspace_bytes(B, h, d, L) <= size
    guard = 4096
    ws = dev.empty((size // 4 + guard,), 0)
    ws.fill_(12345.0)
    kc = rnd(po, 20 * h * L * d, 51).reshape(20, h, L, d)
    vc = rnd(po, 20 * h * L * d, 52).reshape(20, h, L, d)
    q = rnd(po, 20 * h * d, 50).reshape(20, h, d)
    out = dev.empty((20, h, d), 1)
    dev.call("lg_attn_decode_f16", dev.up(q, 1), dev.up(kc, 1), dev.up(vc, 1), out, ws, 20, h, d, L, L, float(1 / np.sqrt(d)))
    assert max_rel_err(dev.down(out), po.attn_decode(q, kc, vc, L, 1 / np.sqrt(d), 1)) < 1e-2
    assert np.all(dev.down(ws)[size // 4:] == 12345.0), "the kernel wrote beyond the advertised workspace size"


@pytest.mark.parametrize("h,d,Lmax,slots,seqs", [
    (4, 128, 256, 6, [(5, 200), (0, 1), (3, 256), (2, 77)]),
    (48, 128, 1088, 4, [(3, 1000), (1, 130)]),
    (3, 96, 64, 3, [(2, 64), (0, 17), (1, 5)]),
    (2, 64, 512, 9, [(8, 512)] + [(i, 40 + 50 * i) for i in range(8)])])
def test_attn_decode_varlen(dev, po, h, d, Lmax, slots, seqs):
    """Sequences of different lengths in arbitrary cache slots, one launch: every sequence must equal the oracle's decode
    attention over its own slot and length (the oracle is called once per sequence)."""
    kc = rnd(po, slots * h * Lmax * d, 51).reshape(slots, h, Lmax, d)
    vc = rnd(po, slots * h * Lmax * d, 52).reshape(slots, h, Lmax, d)
    B = len(seqs)
    q = rnd(po, B * h * d, 50).reshape(B, h, d)
    scalar = 1.0 / np.sqrt(d)
    import ctypes as C
    slot = (C.c_int * B)(*[s for s, _ in seqs])
    length = (C.c_int * B)(*[n for _, n in seqs])
    ws = dev.empty((dev.lib.lg_attn_decode_workspace_bytes(B, h, d, Lmax) // 4,), 0)
    out = dev.empty((B, h, d), 1)
    dev.call("lg_attn_decode_varlen_f16", dev.up(q, 1), dev.up(kc, 1), dev.up(vc, 1), out, ws, B, h, d, slot, length, Lmax, float(scalar))
    got = dev.down(out)
    for b, (s, n) in enumerate(seqs):
        ref = po.attn_decode(q[b:b + 1], kc[s:s + 1], vc[s:s + 1], n, scalar, 1)
        assert max_rel_err(got[b:b + 1], ref) < 1e-2, "sequence %d (slot %d, len %d)" % (b, s, n)
    # bad arguments are refused on the host
    length[0] = Lmax + 1
    assert dev.call_rc("lg_attn_decode_varlen_f16", dev.up(q, 1), dev.up(kc, 1), dev.up(vc, 1), out, ws, B, h, d, slot, length, Lmax, float(scalar)) == 1


def test_kv_append_varlen(dev, po):
    import ctypes as C
    B, h, d, Lmax, slots = 3, 4, 96, 16, 5
    n = h * d
    Q, K, V = (rnd(po, B * n, 53 + i).reshape(B, n) for i in range(3))
    bq, bk, bv = (rnd(po, n, 56 + i, 0.3) for i in range(3))
    kc0 = rnd(po, slots * h * Lmax * d, 59).reshape(slots, h, Lmax, d)
    vc0 = rnd(po, slots * h * Lmax * d, 60).reshape(slots, h, Lmax, d)
    dkc, dvc = dev.up(kc0, 1), dev.up(vc0, 1)
    dq = dev.empty((B, h, d), 1)
    slot, pos = [4, 0, 2], [15, 0, 7]
    dev.call("lg_kv_append_varlen_f16", dq, dkc, dvc, dev.up(Q, 1), dev.up(bq, 1), dev.up(K, 1), dev.up(bk, 1), dev.up(V, 1),
             dev.up(bv, 1), B, h, d, (C.c_int * B)(*slot), (C.c_int * B)(*pos), Lmax)
    kc, vc = kc0.copy(), vc0.copy()
    for b in range(B):
        kc[slot[b], :, pos[b], :] = po.round_f16(K[b] + bk).reshape(h, d)
        vc[slot[b], :, pos[b], :] = po.round_f16(V[b] + bv).reshape(h, d)
    assert np.array_equal(dev.down(dkc), kc)
    assert np.array_equal(dev.down(dvc), vc)
    assert np.array_equal(dev.down(dq), po.round_f16(Q + bq).reshape(B, h, d))


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


@pytest.mark.parametrize("B,h,S,d,mode,kv_rows,layout", [
    (2, 3, 128, 128, "causal", 128, 0), (1, 2, 200, 64, "causal", 256, 1), (2, 2, 77, 128, "mask", 77, 1),
    (1, 1, 512, 128, "none", 512, 0), (1, 2, 1000, 128, "causal", 1024, 1), (1, 1, 5, 64, "causal", 8, 0),
    (2, 4, 115, 96, "causal", 128, 1), (1, 2, 300, 96, "mask", 300, 0), (1, 3, 64, 96, "none", 64, 1),
    # batch * heads a multiple of 8 with several query blocks: the block -> (head, query block) placement is remapped
    (2, 4, 300, 128, "causal", 320, 1), (1, 8, 520, 64, "causal", 520, 0), (2, 4, 300, 128, "none", 300, 0),
    (1, 16, 260, 96, "causal", 260, 1)])
def test_attn_prefill_fused(dev, po, B, h, S, d, mode, kv_rows, layout):
    """Fused attention == qk_gemm -> softmax -> qkv_gemm (-> transpose) of the oracle, fp16 semantics."""
    q = rnd(po, B * h * S * d, 70).reshape(B, h, S, d)
    k = rnd(po, B * h * S * d, 71).reshape(B, h, S, d)
    v = rnd(po, B * h * S * d, 72).reshape(B, h, S, d)
    scalar = 1.0 / np.sqrt(d)
    if mode == "mask":
        mask = (po.fill_normal(B * S * S, 0, 73).reshape(B, S, S) > -0.8).astype(np.float32)
        mask[:, 3, :] = 0.0  # a fully masked row must still follow the additive -10000 semantics
        nb = B * h
        scores = np.zeros((nb, S, S), dtype=np.float32)
        po.gemm_strided_batched(1, 0, S, S, d, k.reshape(nb, S, d), d, S * d, q.reshape(nb, S, d), d, S * d, scores, S, S * S, nb, 1)
        po.attn_softmax(scores.reshape(B, h, S, S), mask, scalar, 1)
        ref = np.zeros((nb, S, d), dtype=np.float32)
        po.gemm_strided_batched(0, 0, d, S, S, v.reshape(nb, S, d), d, S * d, scores, S, S * S, ref, d, S * d, nb, 1)
        ref = ref.reshape(B, h, S, d)
        dmask = dev.up(mask, 1)
    else:
        ref = po.attn_prefill(q, k, v, scalar, mode == "causal", 1)
        dmask = None
    kpad = np.zeros((B, h, kv_rows, d), dtype=np.float32); vpad = np.full((B, h, kv_rows, d), 7.0, dtype=np.float32)
    kpad[:, :, :S] = k; vpad[:, :, :S] = v
    out = dev.empty((B, S, h, d) if layout else (B, h, S, d), 1)
    dev.call("lg_attn_prefill_f16", dev.up(q, 1), dev.up(kpad, 1), dev.up(vpad, 1), dmask if dmask is not None else 0, out,
             B, S, h, d, kv_rows, float(scalar), int(mode == "causal"), layout)
    got = dev.down(out)
    if layout:
        got = got.transpose(0, 2, 1, 3)
    if mode == "mask":
        # On the fully masked row the reference's half kernel adds -10000 in fp16 (spacing 8 at that magnitude), which
        # quantises the scores; the fused kernel adds it in fp32.  There the fp32-semantics oracle is the yardstick:
        # a constant shift cancels and the row is the plain softmax.
        scores32 = np.zeros((B * h, S, S), dtype=np.float32)
        nb = B * h
        po.gemm_strided_batched(1, 0, S, S, d, k.reshape(nb, S, d), d, S * d, q.reshape(nb, S, d), d, S * d, scores32, S, S * S, nb, 0)
        po.attn_softmax(scores32.reshape(B, h, S, S), mask, scalar, 0)
        ref32 = np.zeros((nb, S, d), dtype=np.float32)
        po.gemm_strided_batched(0, 0, d, S, S, v.reshape(nb, S, d), d, S * d, scores32, S, S * S, ref32, d, S * d, nb, 0)
        ref32 = ref32.reshape(B, h, S, d)
        assert max_rel_err(got[:, :, 3], ref32[:, :, 3]) < 1e-2
        got = np.delete(got, 3, axis=2)
        ref = np.delete(ref, 3, axis=2)
    assert max_rel_err(got, ref) < 1e-2


@pytest.mark.parametrize("B,h,d,S,past,kv_rows,causal", [
    (2, 4, 128, 128, 128, 256, 1), (1, 8, 128, 200, 312, 512, 1), (1, 3, 64, 64, 1, 80, 1), (2, 2, 96, 100, 57, 160, 1),
    (1, 8, 128, 128, 896, 1024, 1), (1, 4, 128, 70, 130, 200, 0), (1, 48, 128, 256, 768, 1088, 1)])
def test_attn_prefill_that_continues_a_sequence(dev, po, B, h, d, S, past, kv_rows, causal):
    """A chunk of S queries at positions past .. past + S - 1 over past + S keys and values (chunked prefill over a KV cache)
    must equal rows past .. of the oracle's attention over the whole sequence: with a causal mask row i sees keys 0 .. past + i;
    without one every query sees all past + S keys, which is the last S rows of the full non-causal attention."""
    L = past + S
    q = rnd(po, B * h * L * d, 80).reshape(B, h, L, d)
    k = rnd(po, B * h * L * d, 81).reshape(B, h, L, d)
    v = rnd(po, B * h * L * d, 82).reshape(B, h, L, d)
    scalar = 1.0 / np.sqrt(d)
    ref = po.attn_prefill(q, k, v, scalar, bool(causal), 1)[:, :, past:]
    kpad = np.zeros((B, h, kv_rows, d), dtype=np.float32); vpad = np.full((B, h, kv_rows, d), 7.0, dtype=np.float32)
    kpad[:, :, :L] = k; vpad[:, :, :L] = v
    out = dev.empty((B, S, h, d), 1)
    dev.call("lg_attn_prefill_past_f16", dev.up(np.ascontiguousarray(q[:, :, past:]), 1), dev.up(kpad, 1), dev.up(vpad, 1), out,
             B, S, past, h, d, kv_rows, float(scalar), causal, 1)
    got = dev.down(out).transpose(0, 2, 1, 3)
    assert max_rel_err(got, ref) < 4e-3
    # past = 0 is the plain entry, bit for bit
    a, b = dev.empty((B, L, h, d), 1), dev.empty((B, L, h, d), 1)
    dq = dev.up(q, 1)
    dev.call("lg_attn_prefill_past_f16", dq, dev.up(kpad, 1), dev.up(vpad, 1), a, B, L, 0, h, d, kv_rows, float(scalar), causal, 1)
    dev.call("lg_attn_prefill_f16", dq, dev.up(kpad, 1), dev.up(vpad, 1), 0, b, B, L, h, d, kv_rows, float(scalar), causal, 1)
    assert np.array_equal(dev.down(a), dev.down(b))
    # more positions than the buffers hold are refused on the host
    assert dev.call_rc("lg_attn_prefill_past_f16", dq, dq, dq, a, B, S, kv_rows - S + 1, h, d, kv_rows, float(scalar), causal, 1) == dev.capi.ERR_INVALID
