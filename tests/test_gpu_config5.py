"""BASELINE config 5 at its full size: the 32-layer, d_model 4096, 32 / 8 heads of 128, FFN 14336, vocabulary 128256
Q4_K_M decode step at context 512 against the composed CPU oracle, and a 512-token prompt through layers of that shape
against the oracle applied token by token.  Weights are N(0, 0.02) through quantizers.py (drawn and quantised on
the GPU with torch to keep the set-up short; the bytes then go to the oracle and, through the C ABI, to the library)."""
import os

import numpy as np
import pytest
import torch

import quantizers
from decode_oracle import SLOTS, decode_ref, prefill_ref
from helpers import GGML_ID, norm_err

pytestmark = pytest.mark.gpu

MIX = {"attn_q": "Q4_K", "attn_k": "Q4_K", "attn_v": "Q6_K", "attn_o": "Q4_K", "ffn_gate": "Q4_K", "ffn_up": "Q4_K", "ffn_down": "Q6_K"}
THREADS = max(1, min(16, (os.cpu_count() or 1)))


@pytest.fixture(scope="module")
def jn():
    import jitnn_amd
    jitnn_amd.init()
    return jitnn_amd


def build_8b(jn, layers, vocab, max_ctx, seed):
    cfg = dict(layers=layers, d_model=4096, heads=32, kv_heads=8, head_dim=128, ffn=14336, vocab=vocab, max_ctx=max_ctx, rms_eps=1e-5,
               rope_theta=5e5)
    g = torch.Generator(device="cuda").manual_seed(seed)
    rng = np.random.default_rng(seed)
    shapes = {"attn_q": (4096, 4096), "attn_k": (1024, 4096), "attn_v": (1024, 4096), "attn_o": (4096, 4096), "ffn_gate": (14336, 4096),
              "ffn_up": (14336, 4096), "ffn_down": (4096, 14336)}
    dec = jn.LlamaDecoder(**cfg)
    stack = []
    for li in range(layers):
        L = {}
        for si, slot in enumerate(SLOTS):
            n, k = shapes[slot]
            fmt = MIX[slot]
            raw = quantizers.quantize(fmt, torch.randn(n, k, generator=g, device="cuda") * 0.02).cpu().numpy()
            L[slot] = (GGML_ID[fmt], raw, n, k)
            dec.set_weight(li, si, jn.Tensor.quantized(jn.DType[fmt], raw, n, k))
        for ni, name in enumerate(("attn_norm", "ffn_norm")):
            L[name] = (1.0 + 0.1 * rng.standard_normal(4096)).astype(np.float32)
            dec.set_norm(li, ni, L[name])
        stack.append(L)
        if li % 8 == 7:
            print(f"  built layer {li + 1} of {layers}", flush=True)
    out_norm = (1.0 + 0.1 * rng.standard_normal(4096)).astype(np.float32)
    dec.set_norm(0, 2, out_norm)
    parts = [quantizers.quantize("Q6_K", torch.randn(min(8192, vocab - r0), 4096, generator=g, device="cuda") * 0.02) for r0 in range(0, vocab, 8192)]
    raw = torch.cat(parts).cpu().numpy()
    out_w = (GGML_ID["Q6_K"], raw, vocab, 4096)
    dec.set_weight(0, 7, jn.Tensor.quantized(jn.DType.Q6_K, raw, vocab, 4096))
    torch.cuda.empty_cache()
    return cfg, dec, stack, out_norm, out_w


def test_decode_step_full_depth_8b(jn):
    """All 32 layers and the 128256-row output head at context 512, one token: logits and the appended cache rows of the
    first and last layer against the oracle (bar 1e-4 of the largest logit)."""
    cfg, dec, stack, out_norm, out_w = build_8b(jn, 32, 128256, 513, 2024)
    rng = np.random.default_rng(6)
    kc = np.zeros((32, 513, 8, 128), dtype=np.float32)
    vc = np.zeros_like(kc)
    kc[:, :512] = rng.standard_normal((32, 512, 8, 128), dtype=np.float32)
    vc[:, :512] = rng.standard_normal((32, 512, 8, 128), dtype=np.float32)
    for li in range(32):
        dec.kv_write(li, 0, kc[li, :512], vc[li, :512])
    x = rng.standard_normal(4096).astype(np.float32)
    ref = decode_ref(cfg, stack, out_norm, out_w, kc, vc, x, 512, threads=THREADS)
    y = dec.decode(x, 512)
    err = norm_err(y, ref)
    print(f"32-layer decode step: normalised max error of the logits {err:.3e}", flush=True)
    assert err <= 1e-4, err
    assert int(np.argmax(y)) == int(np.argmax(ref))
    for li in (0, 31):
        k, v = dec.kv_read(li, 512, 1)
        assert norm_err(k[0], kc[li, 512]) <= 1e-4 and norm_err(v[0], vc[li, 512]) <= 1e-4, li
    dec.close()


def test_prefill_512_tokens_8b_layers(jn):
    """A 512-token prompt from an empty cache through two layers of the 8B shape and a 32064-row head (FP16-operand
    matrix-core linears and attention): layer 0's appended keys and values are one such linear of the normalised input
    each (bar 2e-3, the bar of that path); what lies behind further linears and the attention - layer 1's rows, the last
    token's logits - is held to 5e-3."""
    cfg, dec, stack, out_norm, out_w = build_8b(jn, 2, 32064, 513, 2025)
    rng = np.random.default_rng(7)
    kc = np.zeros((2, 513, 8, 128), dtype=np.float32)
    vc = np.zeros_like(kc)
    x = rng.standard_normal((512, 4096)).astype(np.float32)
    ref = prefill_ref(cfg, stack, out_norm, out_w, kc, vc, x, 0)
    y = dec.prefill(x, 0)
    k0, v0 = dec.kv_read(0, 0, 512)
    k1, v1 = dec.kv_read(1, 0, 512)
    e = dict(k0=norm_err(k0, kc[0, :512]), v0=norm_err(v0, vc[0, :512]), k1=norm_err(k1, kc[1, :512]), v1=norm_err(v1, vc[1, :512]),
             logits=norm_err(y, ref))
    print("512-token prefill, 2 layers of the 8B shape:", {n: f"{v:.2e}" for n, v in e.items()}, flush=True)
    assert e["k0"] <= 2e-3 and e["v0"] <= 2e-3, e
    assert e["k1"] <= 5e-3 and e["v1"] <= 5e-3 and e["logits"] <= 5e-3, e
    # decoding goes on from the prefilled cache: one more token, against the oracle's step on the oracle's cache
    xn = rng.standard_normal(4096).astype(np.float32)
    ref = decode_ref(cfg, stack, out_norm, out_w, kc, vc, xn, 512, threads=THREADS)
    e = norm_err(dec.decode(xn, 512), ref)
    assert e <= 5e-3, e
    dec.close()
