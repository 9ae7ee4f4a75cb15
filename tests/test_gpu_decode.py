"""The on-device decode step (jitnn_hip_llama_*) against the CPU oracle's composition of the reference operators."""
import numpy as np
import pytest
import torch

import quantizers
from decode_oracle import SLOTS, decode_ref
from helpers import GGML_ID, norm_err

pytestmark = pytest.mark.gpu

MIX = {"attn_q": "Q4_K", "attn_k": "Q4_K", "attn_v": "Q6_K", "attn_o": "Q4_K", "ffn_gate": "Q4_K", "ffn_up": "Q4_K", "ffn_down": "Q6_K"}


def build(jn, cfg, seed, mix=MIX, out_fmt="Q6_K"):
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    d, qd, kd, ffn = cfg["d_model"], cfg["heads"] * cfg["head_dim"], cfg["kv_heads"] * cfg["head_dim"], cfg["ffn"]
    shapes = {"attn_q": (qd, d), "attn_k": (kd, d), "attn_v": (kd, d), "attn_o": (d, qd), "ffn_gate": (ffn, d), "ffn_up": (ffn, d),
              "ffn_down": (d, ffn)}
    dec = jn.LlamaDecoder(**cfg)
    layers = []
    for li in range(cfg["layers"]):
        L = {}
        for si, slot in enumerate(SLOTS):
            n, k = shapes[slot]
            fmt = mix[slot]
            raw = quantizers.quantize(fmt, torch.randn(n, k, generator=g) * 0.02).numpy()
            L[slot] = (GGML_ID[fmt], raw, n, k)
            dec.set_weight(li, si, jn.Tensor.quantized(jn.DType[fmt], raw, n, k))
        for ni, name in enumerate(("attn_norm", "ffn_norm")):
            L[name] = (1.0 + 0.1 * rng.standard_normal(d)).astype(np.float32)
            dec.set_norm(li, ni, L[name])
        layers.append(L)
    out_norm = (1.0 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    dec.set_norm(0, 2, out_norm)
    raw = quantizers.quantize(out_fmt, torch.randn(cfg["vocab"], d, generator=g) * 0.02).numpy()
    out_w = (GGML_ID[out_fmt], raw, cfg["vocab"], d)
    dec.set_weight(0, 7, jn.Tensor.quantized(jn.DType[out_fmt], raw, cfg["vocab"], d))
    return dec, layers, out_norm, out_w


@pytest.fixture(scope="module")
def jn():
    import jitnn_amd
    jitnn_amd.init()
    return jitnn_amd


@pytest.mark.parametrize("mix_name", ["q4_k_m", "q8_0"])
def test_decode_wide_model(jn, mix_name):
    """A residual stream of 5120 values - rows longer than 4096 for q, k, v, gate and up, which the norm-fused launches do not
    take: a norm kernel of its own, then every linear with one wave per 1024 values (five here) - two tokens on a pre-filled
    cache."""
    cfg = dict(layers=1, d_model=5120, heads=8, kv_heads=2, head_dim=64, ffn=768, vocab=512, max_ctx=40, rms_eps=1e-5, rope_theta=1e4)
    mix = {"q4_k_m": MIX, "q8_0": {s: "Q8_0" for s in SLOTS}}[mix_name]
    dec, layers, out_norm, out_w = build(jn, cfg, 9, mix, "Q6_K")
    rng = np.random.default_rng(2)
    ctx0 = 33
    kc = np.zeros((cfg["layers"], cfg["max_ctx"], cfg["kv_heads"], cfg["head_dim"]), dtype=np.float32)
    vc = np.zeros_like(kc)
    kc[:, :ctx0] = rng.standard_normal(kc[:, :ctx0].shape)
    vc[:, :ctx0] = rng.standard_normal(vc[:, :ctx0].shape)
    dec.kv_write(0, 0, kc[0, :ctx0], vc[0, :ctx0])
    for step in range(2):
        pos = ctx0 + step
        x = rng.standard_normal(cfg["d_model"]).astype(np.float32)
        ref = decode_ref(cfg, layers, out_norm, out_w, kc, vc, x, pos)
        y = dec.decode(x, pos)
        assert norm_err(y, ref) <= 1e-4, (mix_name, step, norm_err(y, ref))
    dec.close()


@pytest.mark.parametrize("mix_name", ["q4_k_m", "q8_0", "q4_0_q5_k", "q4_k_q5_k", "q5_k_m", "q6_k", "q4_1"])
def test_decode_small_model(jn, mix_name):
    """Two layers, grouped heads 8/2 of size 64, three tokens decoded in a row on a pre-filled cache.  The mixes cover the
    two-format q, k | v launches the library has (Q4_K | Q6_K, Q4_K | Q5_K, Q5_K | Q6_K), a single format for all three and a
    pair it launches separately (Q4_0 | Q5_K); every format of the path as the gate / up pair of the fused SwiGLU launch."""
    cfg = dict(layers=2, d_model=512, heads=8, kv_heads=2, head_dim=64, ffn=1024, vocab=1000, max_ctx=48, rms_eps=1e-5, rope_theta=5e5)
    mix = {"q4_k_m": MIX, "q8_0": {s: "Q8_0" for s in SLOTS},
           "q4_0_q5_k": {**{s: "Q4_0" for s in SLOTS}, "attn_v": "Q5_K", "ffn_down": "Q5_K", "attn_o": "Q4_1"},
           "q4_k_q5_k": {**{s: "Q4_K" for s in SLOTS}, "attn_v": "Q5_K", "ffn_down": "Q5_K"},
           "q5_k_m": {**{s: "Q5_K" for s in SLOTS}, "attn_v": "Q6_K", "ffn_down": "Q6_K"},
           "q6_k": {s: "Q6_K" for s in SLOTS}, "q4_1": {s: "Q4_1" for s in SLOTS}}[mix_name]
    dec, layers, out_norm, out_w = build(jn, cfg, 5, mix, "Q8_0" if mix_name == "q8_0" else "Q6_K")
    rng = np.random.default_rng(1)
    ctx0 = 37
    kc = np.zeros((cfg["layers"], cfg["max_ctx"], cfg["kv_heads"], cfg["head_dim"]), dtype=np.float32)
    vc = np.zeros_like(kc)
    kc[:, :ctx0] = rng.standard_normal(kc[:, :ctx0].shape)
    vc[:, :ctx0] = rng.standard_normal(vc[:, :ctx0].shape)
    for li in range(cfg["layers"]):
        dec.kv_write(li, 0, kc[li, :ctx0], vc[li, :ctx0])
    for step in range(3):
        pos = ctx0 + step
        x = rng.standard_normal(cfg["d_model"]).astype(np.float32)
        ref = decode_ref(cfg, layers, out_norm, out_w, kc, vc, x, pos)
        y = dec.decode(x, pos)
        assert norm_err(y, ref) <= 1e-4, (mix_name, step, norm_err(y, ref))
        for li in range(cfg["layers"]):  # the appended (rotated) keys and the values
            k, v = dec.kv_read(li, pos, 1)
            assert np.allclose(k[0], kc[li, pos], rtol=1e-5, atol=1e-6)
            assert np.allclose(v[0], vc[li, pos], rtol=1e-5, atol=1e-6)
    dec.close()


def test_decode_8b_shaped_layer(jn):
    """One layer at the 8B shape of BASELINE config 5 (d_model 4096, 32/8 heads of 128, FFN 14336, context 512) with a
    cut-down vocabulary, Q4_K_M mix."""
    cfg = dict(layers=1, d_model=4096, heads=32, kv_heads=8, head_dim=128, ffn=14336, vocab=2048, max_ctx=513, rms_eps=1e-5, rope_theta=5e5)
    dec, layers, out_norm, out_w = build(jn, cfg, 9)
    rng = np.random.default_rng(2)
    kc = np.zeros((1, 513, 8, 128), dtype=np.float32)
    vc = np.zeros_like(kc)
    kc[:, :512] = rng.standard_normal((1, 512, 8, 128))
    vc[:, :512] = rng.standard_normal((1, 512, 8, 128))
    dec.kv_write(0, 0, kc[0, :512], vc[0, :512])
    x = rng.standard_normal(4096).astype(np.float32)
    ref = decode_ref(cfg, layers, out_norm, out_w, kc, vc, x, 512)
    y = dec.decode(x, 512)
    assert norm_err(y, ref) <= 1e-4, norm_err(y, ref)
    dec.close()


@pytest.mark.parametrize("heads,kv_heads,head_dim,ctx", [(4, 2, 64, 1500), (4, 1, 128, 2077), (2, 2, 192, 700), (2, 1, 256, 1111)])
def test_decode_long_context(jn, heads, kv_heads, head_dim, ctx):
    """One token over a long cache: more than 32 key chunks per head, so the merge of the chunks runs with eight (five,
    four) threads per value instead of two; the last chunk is partly filled."""
    cfg = dict(layers=1, d_model=256, heads=heads, kv_heads=kv_heads, head_dim=head_dim, ffn=256, vocab=100, max_ctx=ctx + 2, rms_eps=1e-5,
               rope_theta=5e5)
    dec, layers, out_norm, out_w = build(jn, cfg, 31, {s: "Q8_0" for s in SLOTS}, "Q8_0")
    rng = np.random.default_rng(7)
    kc = np.zeros((1, cfg["max_ctx"], kv_heads, head_dim), dtype=np.float32)
    vc = np.zeros_like(kc)
    kc[:, :ctx] = rng.standard_normal(kc[:, :ctx].shape)
    vc[:, :ctx] = rng.standard_normal(vc[:, :ctx].shape)
    dec.kv_write(0, 0, kc[0, :ctx], vc[0, :ctx])
    for step in range(2):
        x = rng.standard_normal(cfg["d_model"]).astype(np.float32)
        ref = decode_ref(cfg, layers, out_norm, out_w, kc, vc, x, ctx + step)
        y = dec.decode(x, ctx + step)
        assert norm_err(y, ref) <= 1e-4, (head_dim, step, norm_err(y, ref))
    dec.close()


def test_decode_argument_checks(jn):
    cfg = dict(layers=1, d_model=256, heads=4, kv_heads=2, head_dim=64, ffn=512, vocab=64, max_ctx=8, rms_eps=1e-5, rope_theta=1e4)
    dec = jn.LlamaDecoder(**cfg)
    with pytest.raises(ValueError, match="has no weight"):
        dec.decode(np.zeros(256, dtype=np.float32), 0)
    w = jn.Tensor.quantized(jn.DType.Q4_K, np.zeros(144 * 3, dtype=np.uint8), 3, 256)
    with pytest.raises(ValueError, match="needs shape"):
        dec.set_weight(0, 0, w)
    with pytest.raises(ValueError):
        jn.LlamaDecoder(**{**cfg, "heads": 3})
    with pytest.raises(ValueError):
        jn.LlamaDecoder(**{**cfg, "head_dim": 80})
    dec.close()


@pytest.mark.parametrize("pos0,tokens,bar", [(5, 3, 1e-4), (0, 20, 1e-4), (9, 70, 1e-2)])
def test_prefill_matches_token_by_token_reference(jn, pos0, tokens, bar):
    """Many tokens at once against the oracle's decode step run token by token on the same cache: the last token's
    logits and every appended key and value.  Up to 64 tokens the linears are the FP32-grade GEMV kernels (bar 1e-4);
    beyond, the FP16-operand matrix-core path (2e-3 per linear, two layers deep: 1e-2 on the logits)."""
    cfg = dict(layers=2, d_model=512, heads=8, kv_heads=2, head_dim=64, ffn=1024, vocab=1000, max_ctx=96, rms_eps=1e-5, rope_theta=5e5)
    dec, layers, out_norm, out_w = build(jn, cfg, 11)
    rng = np.random.default_rng(3)
    kc = np.zeros((cfg["layers"], cfg["max_ctx"], cfg["kv_heads"], cfg["head_dim"]), dtype=np.float32)
    vc = np.zeros_like(kc)
    kc[:, :pos0] = rng.standard_normal(kc[:, :pos0].shape)
    vc[:, :pos0] = rng.standard_normal(vc[:, :pos0].shape)
    for li in range(cfg["layers"]):
        if pos0:
            dec.kv_write(li, 0, kc[li, :pos0], vc[li, :pos0])
    x = rng.standard_normal((tokens, cfg["d_model"])).astype(np.float32)
    ref = None
    for t in range(tokens):
        ref = decode_ref(cfg, layers, out_norm, out_w, kc, vc, x[t], pos0 + t)
    y = dec.prefill(x, pos0)
    assert norm_err(y, ref) <= bar, norm_err(y, ref)
    for li in range(cfg["layers"]):
        k, v = dec.kv_read(li, pos0, tokens)
        # layer 0's keys and values are one linear of the normalised input each: the bar of that linear's path (2e-3 on
        # FP16 operands); deeper layers sit behind attention and further linears
        kv_bar = bar if tokens <= 64 or li > 0 else 2e-3
        assert norm_err(k, kc[li, pos0:pos0 + tokens]) <= kv_bar and norm_err(v, vc[li, pos0:pos0 + tokens]) <= kv_bar, li
    # decoding goes on from the prefilled cache
    xn = rng.standard_normal(cfg["d_model"]).astype(np.float32)
    ref = decode_ref(cfg, layers, out_norm, out_w, kc, vc, xn, pos0 + tokens)
    assert norm_err(dec.decode(xn, pos0 + tokens), ref) <= bar
    dec.close()


@pytest.mark.parametrize("tokens,bar", [(40, 1e-4), (70, 5e-3)])
@pytest.mark.parametrize("heads,kv_heads,head_dim", [(4, 2, 128), (6, 2, 64), (2, 2, 192), (2, 1, 256)])
def test_prefill_head_shapes(jn, heads, kv_heads, head_dim, tokens, bar):
    """Every head size the attention kernels are built for, groups of 1, 2 and 3 query heads per key/value head; 40 tokens
    (FP32 attention, GEMV linears) and 70 tokens (FP16-operand attention and linears) after 7 cached positions: several
    key chunks, the last one partly filled."""
    cfg = dict(layers=1, d_model=512, heads=heads, kv_heads=kv_heads, head_dim=head_dim, ffn=512, vocab=300, max_ctx=96, rms_eps=1e-5,
               rope_theta=5e5)
    dec, layers, out_norm, out_w = build(jn, cfg, 17, {s: "Q8_0" for s in SLOTS}, "Q8_0")
    rng = np.random.default_rng(4)
    pos0 = 7
    kc = np.zeros((1, cfg["max_ctx"], kv_heads, head_dim), dtype=np.float32)
    vc = np.zeros_like(kc)
    kc[:, :pos0] = rng.standard_normal(kc[:, :pos0].shape)
    vc[:, :pos0] = rng.standard_normal(vc[:, :pos0].shape)
    dec.kv_write(0, 0, kc[0, :pos0], vc[0, :pos0])
    x = rng.standard_normal((tokens, cfg["d_model"])).astype(np.float32)
    for t in range(tokens):
        ref = decode_ref(cfg, layers, out_norm, out_w, kc, vc, x[t], pos0 + t)
    y = dec.prefill(x, pos0)
    assert norm_err(y, ref) <= bar, norm_err(y, ref)
    k, v = dec.kv_read(0, pos0, tokens)
    kv_bar = bar if tokens <= 64 else 2e-3  # one linear of the normalised input: the bar of the linear's own path
    assert norm_err(k, kc[0, pos0:pos0 + tokens]) <= kv_bar and norm_err(v, vc[0, pos0:pos0 + tokens]) <= kv_bar
    # one more token on the prefilled cache: the single-token attention kernel of this head size
    xn = rng.standard_normal(cfg["d_model"]).astype(np.float32)
    ref = decode_ref(cfg, layers, out_norm, out_w, kc, vc, xn, pos0 + tokens)
    assert norm_err(dec.decode(xn, pos0 + tokens), ref) <= bar
    kn, vn = dec.kv_read(0, pos0 + tokens, 1)
    assert norm_err(kn[0], kc[0, pos0 + tokens]) <= kv_bar and norm_err(vn[0], vc[0, pos0 + tokens]) <= kv_bar
    dec.close()


@pytest.mark.parametrize("fmt,ffn", [("Q4_K", 768), ("Q5_K", 768), ("Q6_K", 768), ("Q4_0", 1056), ("Q4_1", 1056), ("Q8_0", 1056)])
def test_prefill_ffn_formats(jn, fmt, ffn):
    """A prompt beyond the GEMV range in every format: the gate and up projections are one matrix-core product with the
    SwiGLU in its epilogue (64 gate rows and 64 up rows per workgroup; 1056 rows leave the last tile half empty), 130
    tokens are a whole token tile and a ragged one."""
    cfg = dict(layers=1, d_model=512, heads=4, kv_heads=2, head_dim=128, ffn=ffn, vocab=300, max_ctx=160, rms_eps=1e-5, rope_theta=5e5)
    dec, layers, out_norm, out_w = build(jn, cfg, 23, {s: fmt for s in SLOTS}, "Q8_0")
    rng = np.random.default_rng(6)
    tokens, pos0 = 130, 3
    kc = np.zeros((1, cfg["max_ctx"], 2, 128), dtype=np.float32)
    vc = np.zeros_like(kc)
    kc[:, :pos0] = rng.standard_normal(kc[:, :pos0].shape)
    vc[:, :pos0] = rng.standard_normal(vc[:, :pos0].shape)
    dec.kv_write(0, 0, kc[0, :pos0], vc[0, :pos0])
    x = rng.standard_normal((tokens, cfg["d_model"])).astype(np.float32)
    for t in range(tokens):
        ref = decode_ref(cfg, layers, out_norm, out_w, kc, vc, x[t], pos0 + t)
    y = dec.prefill(x, pos0)
    assert norm_err(y, ref) <= 5e-3, (fmt, norm_err(y, ref))
    dec.close()


@pytest.mark.parametrize("heads,kv_heads,head_dim", [(4, 4, 128), (8, 2, 128), (8, 1, 64), (5, 1, 64), (6, 3, 128)])
def test_prefill_long_prompt_attention(jn, heads, kv_heads, head_dim):
    """The matrix-core attention of long prompts on several key chunks: groups of 1, 2, 4, 5 and 8 query heads per key/value
    head (with 5 the 128-row block of a workgroup is ragged), 19 cached positions in front of 150 tokens - three chunks of
    64 keys, the last partly filled, token blocks that end inside the prompt - against the oracle run token by token."""
    tokens, pos0 = 150, 19
    cfg = dict(layers=1, d_model=256, heads=heads, kv_heads=kv_heads, head_dim=head_dim, ffn=256, vocab=200, max_ctx=192, rms_eps=1e-5,
               rope_theta=5e5)
    dec, layers, out_norm, out_w = build(jn, cfg, 23, {s: "Q8_0" for s in SLOTS}, "Q8_0")
    rng = np.random.default_rng(6)
    kc = np.zeros((1, cfg["max_ctx"], kv_heads, head_dim), dtype=np.float32)
    vc = np.zeros_like(kc)
    kc[:, :pos0] = rng.standard_normal(kc[:, :pos0].shape)
    vc[:, :pos0] = rng.standard_normal(vc[:, :pos0].shape)
    dec.kv_write(0, 0, kc[0, :pos0], vc[0, :pos0])
    x = rng.standard_normal((tokens, cfg["d_model"])).astype(np.float32)
    refs = [decode_ref(cfg, layers, out_norm, out_w, kc, vc, x[t], pos0 + t) for t in range(tokens)]
    y = dec.prefill(x, pos0)
    assert norm_err(y, refs[-1]) <= 5e-3, norm_err(y, refs[-1])
    k, v = dec.kv_read(0, pos0, tokens)
    assert norm_err(k, kc[0, pos0:pos0 + tokens]) <= 2e-3 and norm_err(v, vc[0, pos0:pos0 + tokens]) <= 2e-3
    # a shorter prompt on a fresh cache ends in the middle of a token block: its last token must match too
    dec.kv_write(0, 0, kc[0, :pos0], vc[0, :pos0])
    short = 97
    y = dec.prefill(x[:short], pos0)
    assert norm_err(y, refs[short - 1]) <= 5e-3, norm_err(y, refs[short - 1])
    dec.close()


def test_prefill_argument_checks(jn):
    cfg = dict(layers=1, d_model=256, heads=4, kv_heads=2, head_dim=64, ffn=512, vocab=64, max_ctx=8, rms_eps=1e-5, rope_theta=1e4)
    dec, *_ = build(jn, cfg, 13, {s: "Q8_0" for s in SLOTS}, "Q8_0")
    x = np.zeros((4, 256), dtype=np.float32)
    with pytest.raises(ValueError):
        dec.prefill(x, 5)  # positions 5..8 of a cache of 8
    with pytest.raises(ValueError):
        dec.prefill(np.zeros((4, 128), dtype=np.float32), 0)
    assert dec.prefill(x, 4, logits=False) is None
    dec.close()
