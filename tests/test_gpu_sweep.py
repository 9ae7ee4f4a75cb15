"""Seeded random sweeps: Gguf.linear over formats, shapes and row counts, and the prefill / decode steps over model shapes
and per-slot format mixes (the four extra formats included), each against the CPU oracle."""
import numpy as np
import pytest
import torch

import quantizers
from decode_oracle import SLOTS, decode_ref
from helpers import BLOCK, GGML_ID, norm_err, random_valid_blocks

pytestmark = pytest.mark.gpu

F32 = ["Q8_0", "Q4_0", "Q4_1", "Q5_0", "Q5_1"]
F256 = ["Q4_K", "Q5_K", "Q6_K", "Q3_K", "Q2_K"]
# scale ranges that keep random blocks of the extra formats at the magnitude of N(0, 0.02) weights
EXTRA_SCALE = {"Q5_0": (5e-4, 3e-3), "Q5_1": (3e-4, 1.5e-3), "Q3_K": (1e-4, 4e-4), "Q2_K": (2e-4, 1e-3)}


@pytest.fixture(scope="module")
def jn():
    import jitnn_amd
    jitnn_amd.init()
    return jitnn_amd


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_linear_sweep(jn, seed):
    """150 random (format, n, k, rows, bias) per seed, n from 1 to 2500, rows of one block to 14336 values, 1 to 600 rows.  Bar
    per activation row against its largest output: 1e-4 up to 64 rows, 2e-3 beyond (FP16 operands on the matrix cores); an output row that cancels to nearly nothing (one or two weight rows) is measured against sum |w| |x|."""
    from oracle import oracle
    rng = np.random.default_rng(seed)
    allf = F32 + F256
    for case in range(150):
        fmt = allf[rng.integers(len(allf))]
        qk = BLOCK[fmt][0]
        n = [int(rng.integers(1, 40)), int(rng.choice([16, 32, 64, 128, 256, 512, 1024]) + rng.integers(-2, 3)), int(rng.integers(1, 2500))][rng.integers(3)]
        k = [qk * int(rng.integers(1, 8)), 256 * int(rng.integers(1, 17)), 4096 + 256 * int(rng.integers(1, 40)),
             qk * int(rng.integers(1, 4096 // qk + 1))][rng.integers(4)]
        rows = [int(rng.integers(1, 9)), int(rng.integers(9, 65)), int(rng.integers(65, 130)), int(rng.integers(130, 600)),
                int(rng.choice([1, 2, 8, 9, 64, 65, 128, 129, 256, 257]))][rng.integers(5)]
        while n * k * rows > 1e8:  # what the scalar oracle does in a fraction of a second
            if rows > 70:
                rows //= 2
            elif n > 64:
                n //= 2
            else:
                k = max(qk, (k // 2) // qk * qk)
        raw = random_valid_blocks(rng, fmt, n, k)
        bias = rng.standard_normal(n).astype(np.float32) if rng.integers(2) else None
        x = rng.standard_normal((rows, k)).astype(np.float32)
        if rows > 2 and rng.integers(3) == 0:
            x[0] *= np.float32(1e5)
            x[1] *= np.float32(1e-5)
        w = jn.Tensor.quantized(jn.DType[fmt], raw, n, k)
        y = jn.Gguf.linear(jn.Tensor.of(x), w, jn.Tensor.of(bias) if bias is not None else None).numpy().astype(np.float64)
        ref = oracle.gguf_linear(GGML_ID[fmt], x, raw, bias, n, k).astype(np.float64)
        fp16 = rows > 64
        err = np.abs(y - ref)
        worst = float((err.max(axis=1) / np.maximum(np.abs(ref).max(axis=1), 1e-37)).max())
        if worst > (2e-3 if fp16 else 1e-4):
            mag = np.abs(x.astype(np.float64)) @ np.abs(oracle.dequantize(GGML_ID[fmt], raw, n * k).reshape(n, k).astype(np.float64)).T
            nat = float((err / np.maximum(mag, 1e-300)).max())
            assert nat <= (2.0 ** -9 if fp16 else 2e-6), (seed, case, fmt, n, k, rows, worst, nat)


def _raw(fmt, n, k, g, rng):
    if fmt in EXTRA_SCALE:
        return random_valid_blocks(rng, fmt, n, k, *EXTRA_SCALE[fmt])
    return quantizers.quantize(fmt, torch.randn(n, k, generator=g) * 0.02).numpy()


@pytest.mark.parametrize("seed", [1, 2])
def test_step_sweep(jn, seed):
    """15 random models per seed - head sizes 64 to 256, 1 to 4 key/value heads with 1 to 8 query heads each, every slot in a
    format of its own (any of the ten whose block divides the slot's row length) - on 1 to 200 tokens after 0 to 100 cached
    positions: last logits, every appended key and value, and one more single-token step, against the oracle's decode
    step run token by token.  Bars as in test_gpu_decode.py: 1e-4 up to 64 tokens, 1e-2 beyond."""
    rng = np.random.default_rng(seed)
    allf = F32 + F256
    done = 0
    while done < 15:
        head_dim, kv_heads = int(rng.choice([64, 128, 192, 256])), int(rng.choice([1, 2, 3, 4]))
        heads = kv_heads * int(rng.choice([1, 2, 3, 4, 5, 8]))
        if heads * head_dim > 2048:
            continue
        d, ffn, layers = int(rng.choice([256, 512, 768, 1024])), int(rng.choice([256, 512, 768, 1280])), int(rng.choice([1, 2]))
        tokens, pos0 = int(rng.choice([1, 2, 8, 9, 40, 64, 65, 97, 128, 129, 200])), int(rng.choice([0, 1, 31, 32, 33, 100]))
        cfg = dict(layers=layers, d_model=d, heads=heads, kv_heads=kv_heads, head_dim=head_dim, ffn=ffn, vocab=int(rng.integers(50, 400)),
                   max_ctx=pos0 + tokens + 2 + int(rng.integers(0, 40)), rms_eps=1e-5, rope_theta=float(rng.choice([1e4, 5e5])))
        qd, kd = heads * head_dim, kv_heads * head_dim
        shapes = {"attn_q": (qd, d), "attn_k": (kd, d), "attn_v": (kd, d), "attn_o": (d, qd), "ffn_gate": (ffn, d), "ffn_up": (ffn, d),
                  "ffn_down": (d, ffn)}
        pick = lambda k: (allf if k % 256 == 0 else F32)[rng.integers(len(allf) if k % 256 == 0 else len(F32))]
        mix = {s: pick(shapes[s][1]) for s in SLOTS}
        if rng.integers(2):  # the usual case: q and k, gate and up of one format
            mix["attn_k"], mix["ffn_up"] = mix["attn_q"], mix["ffn_gate"]
        out_fmt = pick(d)
        g = torch.Generator().manual_seed(int(rng.integers(1 << 30)))
        dec = jn.LlamaDecoder(**cfg)
        L = []
        for li in range(layers):
            layer = {}
            for si, slot in enumerate(SLOTS):
                n, k = shapes[slot]
                raw = _raw(mix[slot], n, k, g, rng)
                layer[slot] = (GGML_ID[mix[slot]], raw, n, k)
                dec.set_weight(li, si, jn.Tensor.quantized(jn.DType[mix[slot]], raw, n, k))
            for ni, name in enumerate(("attn_norm", "ffn_norm")):
                layer[name] = (1.0 + 0.1 * rng.standard_normal(d)).astype(np.float32)
                dec.set_norm(li, ni, layer[name])
            L.append(layer)
        out_norm = (1.0 + 0.1 * rng.standard_normal(d)).astype(np.float32)
        dec.set_norm(0, 2, out_norm)
        raw = _raw(out_fmt, cfg["vocab"], d, g, rng)
        out_w = (GGML_ID[out_fmt], raw, cfg["vocab"], d)
        dec.set_weight(0, 7, jn.Tensor.quantized(jn.DType[out_fmt], raw, cfg["vocab"], d))
        kc = np.zeros((layers, cfg["max_ctx"], kv_heads, head_dim), dtype=np.float32)
        vc = np.zeros_like(kc)
        kc[:, :pos0] = rng.standard_normal(kc[:, :pos0].shape)
        vc[:, :pos0] = rng.standard_normal(vc[:, :pos0].shape)
        for li in range(layers):
            if pos0:
                dec.kv_write(li, 0, kc[li, :pos0], vc[li, :pos0])
        x = rng.standard_normal((tokens, d)).astype(np.float32)
        for t in range(tokens):
            ref = decode_ref(cfg, L, out_norm, out_w, kc, vc, x[t], pos0 + t)
        y = dec.prefill(x, pos0) if tokens > 1 or rng.integers(2) else dec.decode(x[0], pos0)
        bar = 1e-4 if tokens <= 64 else 1e-2
        what = (seed, done, cfg, tokens, pos0, mix, out_fmt)
        assert norm_err(y, ref) <= bar, what
        for li in range(layers):
            k, v = dec.kv_read(li, pos0, tokens)
            assert norm_err(k, kc[li, pos0:pos0 + tokens]) <= bar and norm_err(v, vc[li, pos0:pos0 + tokens]) <= bar, what
        xn = rng.standard_normal(d).astype(np.float32)
        ref = decode_ref(cfg, L, out_norm, out_w, kc, vc, xn, pos0 + tokens)
        assert norm_err(dec.decode(xn, pos0 + tokens), ref) <= bar, what
        dec.close()
        done += 1
