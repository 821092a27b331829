"""GPU parity of whole layers assembled by the C++ launch-vector runtime against the CPU oracle.

The model initialises its own parameters on the device (seeded generator); the test downloads them, so the oracle
sees bit-identical weights.  Tolerance for fp16: max |gpu - oracle| / max |oracle| <= 1e-2 (the stated bar).
"""
import importlib

import numpy as np
import pytest

from tests.conftest import elementwise_err, max_rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def host(liger):
    return importlib.import_module("24ppopp-liger_amd.host")


def oracle_weights(params, layer=0):
    """Weights of one layer under the oracle's names; a packed QKV projection is split into its three column blocks."""
    pre = "layer%d." % layer
    w = {k[len(pre):]: v for k, v in params.items() if k.startswith(pre)}
    if "wqkv" in w:
        hl = w["wqkv"].shape[1] // 3
        for i, n in enumerate("qkv"):
            w["w" + n] = np.ascontiguousarray(w["wqkv"][:, i * hl:(i + 1) * hl])
            w["b" + n] = np.ascontiguousarray(w["bqkv"][i * hl:(i + 1) * hl])
    return w


def run_layer_case(dev, po, host, dtype, B, S, heads, d, F, norm_mode, causal, fused, ws=1, layers=1, seed=0, weight_layout=0,
                   ffn_act=0, packed_qkv=False):
    H = heads * d
    m = host.Model(dtype, B, S, heads, d, layer_num=layers, world_size=ws, ffn_inner=F, norm_mode=norm_mode, causal=causal,
                   fused=fused, weight_layout=weight_layout, seed=seed, ffn_act=ffn_act, packed_qkv=packed_qkv)
    params = m.download_params()
    x = po.fill_normal(B * S * H, seed, 99, 0.0, 1.0, dtype).reshape(B * S, H)
    dx = dev.up(x, dtype)
    dy = dev.empty((B * S, H), dtype)
    m.run(dx.data_ptr(), dy.data_ptr(), B, S, None, dev.stream)
    got = dev.down(dy)
    shape = dict(batch=B, seq=S, hidden=H, head_num=heads // ws, size_per_head=d, ffn_inner=(F or 4 * H) // ws,
                 causal=int(causal), norm_mode=norm_mode, dtype=dtype, ffn_act=ffn_act)
    ref = x
    for l in range(layers):
        ref = po.encoder_forward(shape, oracle_weights(params, l), ref)
    return got, ref, m


def test_cfg1_plumbing_fp32_prelayernorm(dev, po, host):
    """BASELINE config 1: hidden 256, 4 heads x 64, FFN 1024 (GELU), pre-LayerNorm, batch 2, seq 32, fp32, seed 0."""
    got, ref, m = run_layer_case(dev, po, host, 0, 2, 32, 4, 64, 1024, host.PRE_LN_RESID, False, False)
    assert m.kernels_per_layer() == 15
    assert max_rel_err(got, ref) < 2e-5


def test_cfg1_reference_assembly_fp32(dev, po, host):
    """The order src/layer/bert.h assembles (MHA -> LN -> MLP -> LN), 14 entries per layer on one GPU."""
    got, ref, m = run_layer_case(dev, po, host, 0, 2, 32, 4, 64, 1024, host.POST_NORESID, False, False)
    assert m.kernels_per_layer() == 14
    labels = [e["label"] for e in m.describe(2, 32)]
    assert labels == ["q_gemm", "k_gemm", "v_gemm", "qkv_bias_transpose", "qk_gemm", "softmax", "pv_gemm", "transpose_back",
                      "out_proj", "layer_norm", "ffn1", "bias+gelu", "ffn2", "layer_norm"]
    assert max_rel_err(got, ref) < 2e-5


@pytest.mark.parametrize("weight_layout", [0, 1])
@pytest.mark.parametrize("mode,key", [(0, "post_noresid"), (1, "pre_ln_resid")])
def test_cfg1_layer_against_the_committed_torch_fixture(dev, host, mode, key, weight_layout):
    """BASELINE config 1 on the GPU against tests/golden/cfg1_layer_torch.npz directly (no oracle in between): the
    fixture's weights are uploaded into the model, the input is the fixture's input, the output must match what torch
    computed in float64 from the same numbers."""
    import os
    from tests.golden.make_golden import cfg1_weights
    w, x = cfg1_weights()
    m = host.Model(0, 2, 32, 4, 64, layer_num=1, ffn_inner=1024, norm_mode=mode, causal=False, fused=False,
                   weight_layout=weight_layout, seed=3)
    m.upload_params({"layer0." + k: v for k, v in w.items()})
    back = m.download_params()
    assert all(np.array_equal(back["layer0." + k], v) for k, v in w.items())
    dx, dy = dev.up(x, 0), dev.empty((64, 256), 0)
    m.run(dx.data_ptr(), dy.data_ptr(), 2, 32, None, dev.stream)
    want = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "cfg1_layer_torch.npz"))[key]
    assert max_rel_err(dev.down(dy), want) < 2e-5


@pytest.mark.parametrize("norm_mode", [0, 1])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("fused", [False, True])
def test_fp16_layer_small(dev, po, host, norm_mode, causal, fused):
    got, ref, _ = run_layer_case(dev, po, host, 1, 2, 96, 4, 64, 512, norm_mode, causal, fused)
    assert max_rel_err(got, ref) < 1e-2 and elementwise_err(got, ref) < 1e-2


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("weight_layout", [0, 1, 2])
def test_fp16_tp2_shard_two_layers(dev, po, host, fused, weight_layout):
    """One TP=2 shard (half the heads, half the FFN) of a 2-layer stack, GLM-like head size 128, ragged seq; weights
    stored [in, out] (the reference's layout) or [out, in]."""
    got, ref, _ = run_layer_case(dev, po, host, 1, 2, 200, 8, 128, 2048, 0, True, fused, ws=2, layers=2, weight_layout=weight_layout)
    assert max_rel_err(got, ref) < 1e-2 and elementwise_err(got, ref) < 1e-2


@pytest.mark.parametrize("weight_layout", [0, 1, 2])
def test_fp16_layer_on_the_pipelined_gemm(dev, po, host, weight_layout):
    """Shapes that are multiples of the 256 x 256 x 64 tile, so every weight GEMM takes the pipelined kernel
    (hidden 1024, 8 heads x 128, FFN 2048, 512 tokens)."""
    got, ref, _ = run_layer_case(dev, po, host, 1, 2, 256, 8, 128, 2048, 0, True, True, weight_layout=weight_layout)
    assert max_rel_err(got, ref) < 1e-2 and elementwise_err(got, ref) < 1e-2


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("weight_layout", [0, 1, 2])
def test_fp16_layer_with_the_published_head_size(dev, po, host, fused, weight_layout):
    """The reference's published configuration uses 96-wide heads, batch 2 and sequences of 16 to 115 tokens (main.cu:14-21):
    one TP=2 shard of a two-layer stack with that head size at the longest of those sequences."""
    got, ref, _ = run_layer_case(dev, po, host, 1, 2, 115, 8, 96, 3072, 0, True, fused, ws=2, layers=2, weight_layout=weight_layout)
    assert max_rel_err(got, ref) < 1e-2 and elementwise_err(got, ref) < 1e-2


@pytest.mark.parametrize("heads,d", [(4, 64), (4, 96)])
def test_decode_step_matches_oracle(dev, po, host, heads, d):
    """Fused prefill fills the KV cache, then two decode steps; each is checked against the oracle's decoder step."""
    B, S, F, Lmax = 2, 40, 512, 64
    H = heads * d
    m = host.Model(1, B, S, heads, d, layer_num=1, ffn_inner=F, causal=True, fused=True, max_cache_len=Lmax, seed=3)
    w = oracle_weights(m.download_params())
    x = po.fill_normal(B * S * H, 3, 99, 0.0, 1.0, 1).reshape(B * S, H)
    dx, dy = dev.up(x, 1), dev.empty((B * S, H), 1)
    m.run(dx.data_ptr(), dy.data_ptr(), B, S, None, dev.stream, cache_slot=0)
    shape = dict(batch=B, seq=S, hidden=H, head_num=heads, size_per_head=d, ffn_inner=F, causal=1, norm_mode=0, dtype=1)
    ref_prefill = po.encoder_forward(shape, w, x)
    assert max_rel_err(dev.down(dy), ref_prefill) < 1e-2
    # oracle-side cache from the same prefill
    q = po.gemm(x, w["wq"], 1); k = po.gemm(x, w["wk"], 1); v = po.gemm(x, w["wv"], 1)
    _, kb, vb = po.add_qkv_bias_transpose(q, w["bq"], k, w["bk"], v, w["bv"], B, S, heads, d, 1)
    kc = np.zeros((B, heads, Lmax, d), dtype=np.float32); vc = np.zeros_like(kc)
    kc[:, :, :S] = kb; vc[:, :, :S] = vb
    tok = po.fill_normal(B * H, 3, 100, 0.0, 1.0, 1).reshape(B, H)
    for step in range(2):
        dt_in, dt_out = dev.up(tok, 1), dev.empty((B, H), 1)
        m.run_decode(dt_in.data_ptr(), dt_out.data_ptr(), B, S + step, 0, None, dev.stream)
        ref = po.decoder_step(shape, w, tok, kc, vc, S + step)
        got = dev.down(dt_out)
        assert max_rel_err(got, ref) < 1e-2 and elementwise_err(got, ref) < 1e-2
        tok = po.round_f16(ref)


@pytest.mark.parametrize("heads,d,lens", [(4, 64, [40, 17, 33]), (8, 128, [64, 5, 23, 48, 9, 31])])
def test_decode_step_over_sequences_of_different_lengths(dev, po, host, heads, d, lens):
    """Decode steps of different requests as one launch vector: sequences of different lengths, prefilled one by one into
    scattered cache slots, take one batched step (per-sequence K/V destinations in the Q/K/V epilogue, per-sequence lengths
    in the attention).  Every sequence must equal the oracle's decoder step over its own cache, and its cache rows the
    oracle's; a second step checks that the first one appended K and V where the next one reads them."""
    F, Lmax, slots_total = 512, 72, 8
    H = heads * d
    n = len(lens)
    slots = [(3 * i + 1) % slots_total for i in range(n)]         # scattered, not in sequence order
    m = host.Model(1, slots_total, max(lens), heads, d, layer_num=1, ffn_inner=F, causal=True, fused=True, max_cache_len=Lmax, seed=5)
    w = oracle_weights(m.download_params())
    kcs, vcs = [], []
    for i, S in enumerate(lens):
        x = po.fill_normal(S * H, 5, 200 + i, 0.0, 1.0, 1).reshape(S, H)
        dx, dy = dev.up(x, 1), dev.empty((S, H), 1)
        m.run(dx.data_ptr(), dy.data_ptr(), 1, S, None, dev.stream, cache_slot=slots[i])
        q = po.gemm(x, w["wq"], 1); k = po.gemm(x, w["wk"], 1); v = po.gemm(x, w["wv"], 1)
        _, kb, vb = po.add_qkv_bias_transpose(q, w["bq"], k, w["bk"], v, w["bv"], 1, S, heads, d, 1)
        kc = np.zeros((1, heads, Lmax, d), dtype=np.float32); vc = np.zeros_like(kc)
        kc[:, :, :S] = kb; vc[:, :, :S] = vb
        kcs.append(kc); vcs.append(vc)
    dev.sync()
    tok = po.fill_normal(n * H, 5, 300, 0.0, 1.0, 1).reshape(n, H)
    pasts = list(lens)
    for step in range(2):
        dt_in, dt_out = dev.up(tok, 1), dev.empty((n, H), 1)
        m.run_decode_seqs(dt_in.data_ptr(), dt_out.data_ptr(), slots, pasts, None, dev.stream)
        got = dev.down(dt_out)
        nxt = np.empty_like(tok)
        for i in range(n):
            shape = dict(batch=1, seq=lens[i], hidden=H, head_num=heads, size_per_head=d, ffn_inner=F, causal=1, norm_mode=0, dtype=1)
            ref = po.decoder_step(shape, w, tok[i:i + 1], kcs[i], vcs[i], pasts[i])   # appends to the oracle-side cache
            assert max_rel_err(got[i:i + 1], ref) < 1e-2, "step %d, sequence %d (slot %d, %d cached)" % (step, i, slots[i], pasts[i])
            nxt[i] = po.round_f16(ref)[0]
        tok = nxt
        pasts = [p + 1 for p in pasts]
    # a request outside the cache is refused before anything is launched
    with pytest.raises(dev.capi.LigerError):
        m.run_decode_seqs(dt_in.data_ptr(), dt_out.data_ptr(), slots, [Lmax] * n, None, dev.stream)


@pytest.mark.parametrize("dtype,fused", [(0, False), (1, False), (1, True)])
@pytest.mark.parametrize("norm_mode", [0, 1])
def test_geglu_layer(dev, po, host, dtype, fused, norm_mode):
    """GeGLU FFN (FFN-1 [H, 2F] = [gate | up] -> gelu(gate) * up -> FFN-2) behind the same launch vector."""
    got, ref, m = run_layer_case(dev, po, host, dtype, 2, 96, 4, 64, 512, norm_mode, True, fused, ffn_act=1)
    labels = [e["label"] for e in m.describe(2, 96)]
    # the fused assembly forms the product in FFN-1's epilogue (weights stored with gate and up interleaved); the oracle sees
    # the downloaded, de-interleaved [gate | up] weights either way
    assert ("ffn1+bias+geglu" in labels and "bias+geglu" not in labels) if fused else ("bias+geglu" in labels)
    assert max_rel_err(got, ref) < (2e-5 if dtype == 0 else 1e-2)


@pytest.mark.parametrize("weight_layout", [0, 1, 2])
def test_geglu_fused_upload_round_trip_and_decode(dev, po, host, weight_layout):
    """Fused GeGLU with weights uploaded in the logical [gate | up] order (the model stores them interleaved): prefill and
    one decode step against the oracle, and download(upload(w)) == w."""
    B, S, heads, d, F = 2, 64, 4, 64, 512
    H = heads * d
    m = host.Model(1, B, S, heads, d, layer_num=1, ffn_inner=F, causal=True, fused=True, ffn_act=1, max_cache_len=S + 8,
                   weight_layout=weight_layout, seed=5)
    w1 = po.fill_normal(H * 2 * F, 5, 70, 0.0, 0.05, 1).reshape(H, 2 * F)
    b1 = po.fill_normal(2 * F, 5, 71, 0.0, 0.3, 1)
    m.upload_params({"layer0.w1": w1, "layer0.b1": b1})
    params = m.download_params()
    assert np.array_equal(params["layer0.w1"], w1) and np.array_equal(params["layer0.b1"], b1)
    w = {k[len("layer0."):]: v for k, v in params.items() if k.startswith("layer0.")}
    shape = dict(batch=B, seq=S, hidden=H, head_num=heads, size_per_head=d, ffn_inner=F, causal=1, norm_mode=0, dtype=1, ffn_act=1)
    x = po.fill_normal(B * S * H, 5, 99, 0.0, 1.0, 1).reshape(B * S, H)
    dx, dy = dev.up(x, 1), dev.empty((B * S, H), 1)
    m.run(dx.data_ptr(), dy.data_ptr(), B, S, None, dev.stream, cache_slot=0)
    assert max_rel_err(dev.down(dy), po.encoder_forward(shape, w, x)) < 1e-2
    # decode step: the few-token FFN-1 takes the weight-streaming kernel, whose reduce step forms the product
    k = po.gemm(x, w["wk"], 1)
    v = po.gemm(x, w["wv"], 1)
    _, kb, vb = po.add_qkv_bias_transpose(k, w["bk"], k, w["bk"], v, w["bv"], B, S, heads, d, 1)
    kc = np.zeros((B, heads, S + 8, d), dtype=np.float32)
    vc = np.zeros_like(kc)
    kc[:, :, :S], vc[:, :, :S] = kb, vb
    tok = po.fill_normal(B * H, 5, 100, 0.0, 1.0, 1).reshape(B, H)
    dt_in, dt_out = dev.up(tok, 1), dev.empty((B, H), 1)
    m.run_decode(dt_in.data_ptr(), dt_out.data_ptr(), B, S, 0, None, dev.stream)
    assert max_rel_err(dev.down(dt_out), po.decoder_step(shape, w, tok, kc, vc, S)) < 1e-2


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("weight_layout", [0, 1])
def test_packed_qkv_layer(dev, po, host, dtype, weight_layout):
    """One [H, 3 Hl] projection + the reference's fused bias/transpose kernel instead of three GEMMs: 12 entries, same
    result as the oracle run with the three column blocks of the packed weight."""
    got, ref, m = run_layer_case(dev, po, host, dtype, 2, 80, 4, 64, 512, 0, True, False, ws=2, weight_layout=weight_layout,
                                 packed_qkv=True)
    labels = [e["label"] for e in m.describe(2, 80)]
    assert labels[:2] == ["qkv_gemm", "fused_qkv_bias_transpose"] and m.kernels_per_layer() == 12
    assert max_rel_err(got, ref) < (2e-5 if dtype == 0 else 1e-2)


@pytest.mark.parametrize("weight_layout", [0, 1, 2])
@pytest.mark.parametrize("B,S", [(2, 80), (3, 256)])
def test_packed_qkv_fused_layer_and_decode(dev, po, host, weight_layout, B, S):
    """Packed [H, 3 Hl] projection in the fused assembly: one grouped launch whose epilogue routes q to its buffer and k, v
    straight into the KV cache (B x S = 768 token rows take the pipelined kernel as ONE launch, 160 rows the per-member
    path), then a decode step that reads the same packed parameters.  The oracle gets the three column blocks."""
    heads, d, F = 4, 64, 512
    H = heads * d
    m = host.Model(1, B, S, heads, d, layer_num=1, ffn_inner=F, causal=True, fused=True, packed_qkv=True, max_cache_len=S + 8,
                   weight_layout=weight_layout, seed=9)
    assert [e["label"] for e in m.describe(B, S)][:2] == ["qkv_gemm+bias+heads", "attn_prefill_fused"]
    p = {k[len("layer0."):]: v for k, v in m.download_params().items() if k.startswith("layer0.")}
    w = dict(p)
    for i, t in enumerate("qkv"):
        w["w" + t] = np.ascontiguousarray(p["wqkv"][:, i * H:(i + 1) * H])
        w["b" + t] = np.ascontiguousarray(p["bqkv"][i * H:(i + 1) * H])
    del w["wqkv"], w["bqkv"]
    shape = dict(batch=B, seq=S, hidden=H, head_num=heads, size_per_head=d, ffn_inner=F, causal=1, norm_mode=0, dtype=1)
    x = po.fill_normal(B * S * H, 9, 99, 0.0, 1.0, 1).reshape(B * S, H)
    dx, dy = dev.up(x, 1), dev.empty((B * S, H), 1)
    m.run(dx.data_ptr(), dy.data_ptr(), B, S, None, dev.stream, cache_slot=0)
    assert max_rel_err(dev.down(dy), po.encoder_forward(shape, w, x)) < 1e-2
    k = po.gemm(x, w["wk"], 1)
    v = po.gemm(x, w["wv"], 1)
    _, kb, vb = po.add_qkv_bias_transpose(k, w["bk"], k, w["bk"], v, w["bv"], B, S, heads, d, 1)
    kc = np.zeros((B, heads, S + 8, d), dtype=np.float32)
    vc = np.zeros_like(kc)
    kc[:, :, :S], vc[:, :, :S] = kb, vb
    tok = po.fill_normal(B * H, 9, 100, 0.0, 1.0, 1).reshape(B, H)
    dt_in, dt_out = dev.up(tok, 1), dev.empty((B, H), 1)
    m.run_decode(dt_in.data_ptr(), dt_out.data_ptr(), B, S, 0, None, dev.stream)
    assert max_rel_err(dev.down(dt_out), po.decoder_step(shape, w, tok, kc, vc, S)) < 1e-2


@pytest.mark.parametrize("weight_layout", [1, 2])
@pytest.mark.parametrize("S,chunk", [(256, 64), (200, 96), (130, 128)])
def test_chunked_prefill_equals_the_whole_prefill_and_the_oracle(dev, po, host, S, chunk, weight_layout):
    """One sequence prefilled in chunks over its KV-cache slot (every chunk through both layers before the next): the hidden
    states must equal the oracle's two stacked layers on the whole prompt, and the whole-prompt launch vector up to rounding;
    the caches must end up the same, so that a decode step after either gives the same token."""
    heads, d, F, layers, Lmax = 8, 128, 2048, 2, 320
    H = heads * d
    m = host.Model(1, 3, 256, heads, d, layer_num=layers, ffn_inner=F, causal=True, fused=True, max_cache_len=Lmax,
                   weight_layout=weight_layout, seed=4)
    P = m.download_params()
    x = po.fill_normal(S * H, 4, 99, 0.0, 1.0, 1).reshape(S, H)
    dx = dev.up(x, 1)
    whole, parts = dev.empty((S, H), 1), dev.empty((S, H), 1)
    m.run(dx.data_ptr(), whole.data_ptr(), 1, S, None, dev.stream, cache_slot=0)
    m.run_chunked(dx.data_ptr(), parts.data_ptr(), S, chunk, 2, None, dev.stream)
    shape = dict(batch=1, seq=S, hidden=H, head_num=heads, size_per_head=d, ffn_inner=F, causal=1, norm_mode=0, dtype=1)
    ref = x
    for l in range(layers):
        w = {k[len("layer%d." % l):]: v for k, v in P.items() if k.startswith("layer%d." % l)}
        ref = po.round_f16(po.encoder_forward(shape, w, ref))
    got = dev.down(parts)
    assert max_rel_err(got, ref) < 1e-2 and elementwise_err(got, ref) < 1e-2
    assert max_rel_err(got, dev.down(whole)) < 4e-3
    # the caches of both slots hold the same keys and values (up to rounding), in every layer
    for l in range(layers):
        pk, pv = m.kv_cache(l)
        for ptr in (pk, pv):
            c = dev.empty((3, heads, Lmax, d), 1)
            dev.capi.call("lg_memcpy_d2d_async", c.data_ptr(), ptr, c.numel() * 2, None)
            c = dev.down(c)
            assert max_rel_err(c[2, :, :S], c[0, :, :S]) < 4e-3
    # a decode step on top of the chunked prefill against the oracle's decoder step on the whole-prompt caches
    tok = po.fill_normal(H, 4, 100, 0.0, 1.0, 1).reshape(1, H)
    o = dev.empty((1, H), 1)
    m.run_decode(dev.up(tok, 1).data_ptr(), o.data_ptr(), 1, S, 2, None, dev.stream)
    o0 = dev.empty((1, H), 1)
    m.run_decode(dev.up(tok, 1).data_ptr(), o0.data_ptr(), 1, S, 0, None, dev.stream)
    assert max_rel_err(dev.down(o), dev.down(o0)) < 4e-3
    # refusals: a chunked run needs a cache slot that holds the sequence
    with pytest.raises(host.capi.LigerError):
        m.run_chunked(dx.data_ptr(), parts.data_ptr(), S, chunk, -1, None, dev.stream)


@pytest.mark.parametrize("dtype,fused,packed", [(1, True, False), (1, True, True), (1, False, False), (0, False, False)])
@pytest.mark.parametrize("weight_layout", [0, 1, 2])
@pytest.mark.parametrize("src_layout", [0, 1])
def test_parameters_loaded_from_device_memory_are_relaid_exactly(dev, po, host, dtype, fused, packed, weight_layout, src_layout):
    """lgh_model_load_param: every parameter of a donor model, handed over as a plain [in, out] (what the reference's (N,N)
    GEMM call implies) or [out, in] device array, lands in the receiving layer's storage layout bit for bit -- the
    downloaded parameters are equal and the layer's output equals the donor's bit for bit."""
    if weight_layout == 2 and dtype == 0:
        pytest.skip("fragment blocks are fp16 only")
    B, S, heads, d, F = 2, 48, 4, 64, 512
    H = heads * d
    mk = lambda seed: host.Model(dtype, B, S, heads, d, ffn_inner=F, causal=True, fused=fused, packed_qkv=packed,
                                 weight_layout=weight_layout, seed=seed)
    donor, m = mk(3), mk(4)
    want = donor.download_params()
    before = m.download_params()
    assert any(not np.array_equal(before[k], want[k]) for k in want)
    keep = []
    for name, a in want.items():
        plain = a if (a.ndim == 1 or src_layout == 0) else np.ascontiguousarray(a.T)
        t = dev.up(plain, dtype)
        keep.append(t)
        m.load_param(name, t.data_ptr(), src_layout, dev.stream)
    dev.sync()
    got = m.download_params()
    for k in want:
        assert np.array_equal(got[k], want[k]), k
    x = po.fill_normal(B * S * H, 0, 99, 0.0, 1.0, dtype).reshape(B * S, H)
    dx = dev.up(x, dtype)
    y0, y1 = dev.empty((B * S, H), dtype), dev.empty((B * S, H), dtype)
    donor.run(dx.data_ptr(), y0.data_ptr(), B, S, None, dev.stream)
    m.run(dx.data_ptr(), y1.data_ptr(), B, S, None, dev.stream)
    assert np.array_equal(dev.down(y0), dev.down(y1))
    donor.close()
    m.close()
