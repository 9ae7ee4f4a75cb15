"""The generation loop (jitnn_amd.Llm over jitnn_hip_llama_generate) - the reference's jitnn-llm Llm.generate, whose
arithmetic lives in the third-party jitllm engine, so parity here is behavioural, as in the reference's own test
(jitnn-llm/src/test/java/ai/beestream/jitnn/llm/LlmAccelTest.java:44-60: the answer is not blank, greedy generation is
deterministic, the streamed pieces add up to the text) - plus what the CPU oracle can pin on a model file the test writes
itself: every embedding row bit for bit, and at every step the chosen token is the arg-max of the oracle's logits."""
import numpy as np
import pytest
import torch

import quantizers
from decode_oracle import SLOTS, decode_ref
from gguf_writer import write_gguf
from helpers import GGML_ID

WORDS = ["the", "cat", "sat", "on", "mat", "dog", "ran", "to", "park", "and", "a", "bird", "sang", "in", "tree", "hello", "world"]


def spm_vocab():
    """<unk>, <s>, </s>, the 256 byte tokens, single characters, then word pieces whose scores grow with their length."""
    toks = ["<unk>", "<s>", "</s>"] + [f"<0x{b:02X}>" for b in range(256)]
    types = [2, 3, 3] + [6] * 256
    scores = [0.0] * len(toks)
    pieces = ["▁"] + [chr(c) for c in range(ord("a"), ord("z") + 1)]
    for w in WORDS:
        for n in range(2, len(w) + 1):
            pieces.append(w[:n])
        pieces.append("▁" + w)
        for n in range(1, len(w)):
            pieces.append("▁" + w[:n])
    seen = set(toks)
    for p in pieces:
        if p not in seen:
            seen.add(p)
            toks.append(p)
            types.append(1)
            scores.append(float(len(p)) - 10.0)
    return toks, scores, types


def bpe_vocab():
    from jitnn_amd.tokenizer import _byte_to_unicode
    b2u = _byte_to_unicode()
    toks = [b2u[b] for b in range(256)]
    merges = []
    sp = b2u[ord(" ")]
    for w in WORDS:
        for lead in (sp, ""):  # the merges that start at the space come first, so that " word" wins over "word"
            cur = (lead + w[0]) if lead else w[0]
            if lead and cur not in toks:
                merges.append(f"{lead} {w[0]}")
                toks.append(cur)
            for ch in w[1:]:
                if cur + ch not in toks:
                    merges.append(f"{cur} {ch}")
                    toks.append(cur + ch)
                cur += ch
    toks += ["<|begin|>", "<|end|>"]
    types = [1] * (len(toks) - 2) + [3, 3]
    return toks, merges, types


def test_spm_tokenizer_round_trip_and_byte_fallback():
    from jitnn_amd.tokenizer import StreamDecoder, Tokenizer
    toks, scores, types = spm_vocab()
    tk = Tokenizer("llama", toks, scores, types, None, bos=1, eos=2, add_bos=True)
    ids = tk.encode("the cat sat on the mat")
    assert ids[0] == 1 and [toks[i] for i in ids[1:]] == ["▁the", "▁cat", "▁sat", "▁on", "▁the", "▁mat"]
    assert tk.decode(ids, strip_leading_space=True) == "the cat sat on the mat"
    text = "a bird sang: ¡olé! 東京 42"
    ids = tk.encode(text, add_bos=False)
    assert any(types[i] == 6 for i in ids)          # characters outside the vocabulary went to byte tokens
    assert tk.decode(ids, strip_leading_space=True) == text
    sd = StreamDecoder(tk)
    pieces = [sd.push(i) for i in ids] + [sd.flush()]
    assert "".join(pieces) == tk.decode(ids)         # a character split over byte tokens is held back until whole
    assert tk.encode("", add_bos=False) == []


def test_bpe_tokenizer_round_trip():
    from jitnn_amd.tokenizer import Tokenizer
    toks, merges, types = bpe_vocab()
    tk = Tokenizer("gpt2", toks, None, types, merges, bos=len(toks) - 2, eos=len(toks) - 1, add_bos=False)
    ids = tk.encode("hello world and a bird")
    assert [tk.decode([i]) for i in ids] == ["hello", " world", " and", " a", " bird"]
    text = "the dog ran to the park, 3 times! ¿sí?"
    assert tk.decode(tk.encode(text)) == text
    assert tk.decode([len(toks) - 1]) == ""          # control tokens print nothing


def test_sample_token_limits_and_distribution():
    """The sampler of generate(request): its limits are the greedy choice, its draws follow the renormalised softmax of the
    candidates that top_k and top_p leave, and a seed fixes them."""
    from jitnn_amd.llm import sample_token
    rng = np.random.default_rng(0)
    logits = rng.standard_normal(50).astype(np.float32) * 2
    logits[[7, 31]] = logits.max() + 1.0  # two equal maxima: the lower index
    logits[3] = np.nan
    for kw in (dict(temperature=0.0, top_k=0, top_p=1.0), dict(temperature=1.0, top_k=1, top_p=1.0), dict(temperature=1e-4, top_k=0, top_p=1.0)):
        picks = {sample_token(logits, rng=np.random.default_rng(s), **kw) for s in range(20)}
        assert picks <= {7, 31}
    assert sample_token(logits, 0.0, 0, 1.0, rng) == 7 and sample_token(logits, 1.0, 1, 1.0, rng) == 7
    assert sample_token(logits, 1.0, 0, 1e-9, np.random.default_rng(1)) == 7  # a nucleus of one token
    # frequencies over many draws against the closed form, with and without the limits
    clean = np.where(np.isnan(logits), -np.inf, logits).astype(np.float64)
    for temperature, top_k, top_p in ((1.0, 0, 1.0), (0.7, 5, 1.0), (1.5, 0, 0.6), (1.0, 8, 0.9)):
        order = np.argsort(-clean, kind="stable")
        if top_k:
            order = order[:top_k]
        p = np.exp((clean[order] - clean[order[0]]) / temperature)
        p /= p.sum()
        if top_p < 1.0:
            keep = int(np.argmax(np.cumsum(p) >= top_p)) + 1
            order, p = order[:keep], p[:keep] / p[:keep].sum()
        want = np.zeros(50)
        want[order] = p
        g = np.random.default_rng(11)
        n = 40000
        got = np.bincount([sample_token(logits, temperature, top_k, top_p, g) for _ in range(n)], minlength=50) / n
        assert got[want == 0].sum() == 0 and np.abs(got - want).max() < 4 * np.sqrt(0.25 / n), (temperature, top_k, top_p)
    a = [sample_token(logits, 1.0, 0, 1.0, np.random.default_rng(5)) for _ in range(3)]
    assert len(set(a)) == 1  # same seed, same draw


def test_stop_filter_holds_back_what_may_become_a_stop_sequence():
    from jitnn_amd.llm import GenerationRequest, StopFilter
    f = StopFilter(["END", "\n\n"])
    out = [f.push(p) for p in ["abc E", "N", "x \n", "y EN", "D tail", "more"]]
    assert out == [("abc ", False), ("", False), ("ENx ", False), ("\ny ", False), ("", True), ("", True)]
    assert f.flush() == "" and f.stopped
    f = StopFilter(["END"])
    assert f.push("so it E") == ("so it ", False) and f.flush() == "E"  # what was held back comes out at the end
    f = StopFilter([])
    assert f.push("anything") == ("anything", False)
    assert GenerationRequest("p", stop="x").stop == ("x",) and GenerationRequest("p", stop=["a", ""]).stop == ("a",)
    for bad in (dict(max_new_tokens=-1), dict(temperature=-0.1), dict(top_p=0.0), dict(top_p=1.5), dict(top_k=-2)):
        with pytest.raises(ValueError):
            GenerationRequest("p", **bad)


# ------------------------------------------------------------------------------------------------ on the GPU

CFG = dict(layers=2, d_model=256, heads=4, kv_heads=2, head_dim=64, ffn=512, max_ctx=64, rms_eps=1e-5, rope_theta=10000.0)
MIX = {"attn_q": "Q4_K", "attn_k": "Q4_K", "attn_v": "Q6_K", "attn_o": "Q4_K", "ffn_gate": "Q4_K", "ffn_up": "Q4_K", "ffn_down": "Q6_K"}
GGUF_NAME = {"attn_q": "attn_q", "attn_k": "attn_k", "attn_v": "attn_v", "attn_o": "attn_output", "ffn_gate": "ffn_gate", "ffn_up": "ffn_up",
             "ffn_down": "ffn_down"}


def write_model(path, arch, seed, embd_fmt="Q8_0", tied=False):
    """A random Llama-style model with an SPM vocabulary; returns what the oracle needs."""
    toks, scores, types = spm_vocab()
    vocab = len(toks)
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    d, qd, kd, ffn = CFG["d_model"], CFG["heads"] * CFG["head_dim"], CFG["kv_heads"] * CFG["head_dim"], CFG["ffn"]
    shapes = {"attn_q": (qd, d), "attn_k": (kd, d), "attn_v": (kd, d), "attn_o": (d, qd), "ffn_gate": (ffn, d), "ffn_up": (ffn, d), "ffn_down": (d, ffn)}
    tensors, layers = [], []
    emb_w = torch.randn(vocab, d, generator=g)
    if embd_fmt == "F32":
        emb_raw = emb_w.numpy().astype(np.float32)
    elif embd_fmt == "F16":
        emb_raw = emb_w.numpy().astype(np.float16)
    else:
        emb_raw = quantizers.quantize(embd_fmt, emb_w).numpy()
    emb_id = {"F32": 0, "F16": 1}.get(embd_fmt, GGML_ID.get(embd_fmt))
    tensors.append(("token_embd.weight", (vocab, d), emb_id, emb_raw))
    for l in range(CFG["layers"]):
        L = {}
        for slot in SLOTS:
            n, k = shapes[slot]
            raw = quantizers.quantize(MIX[slot], torch.randn(n, k, generator=g) * 0.08).numpy()
            L[slot] = (GGML_ID[MIX[slot]], raw, n, k)
            tensors.append((f"blk.{l}.{GGUF_NAME[slot]}.weight", (n, k), GGML_ID[MIX[slot]], raw))
        for nm in ("attn_norm", "ffn_norm"):
            L[nm] = (1.0 + 0.1 * rng.standard_normal(d)).astype(np.float32)
            tensors.append((f"blk.{l}.{nm}.weight", (d,), 0, L[nm]))
        layers.append(L)
    out_norm = (1.0 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    tensors.append(("output_norm.weight", (d,), 0, out_norm))
    if tied:
        out_w = (emb_id, emb_raw, vocab, d)
    else:
        raw = quantizers.quantize("Q6_K", torch.randn(vocab, d, generator=g) * 0.08).numpy()
        out_w = (GGML_ID["Q6_K"], raw, vocab, d)
        tensors.append(("output.weight", (vocab, d), GGML_ID["Q6_K"], raw))
    meta = {"general.architecture": arch, "general.name": "tiny test model", f"{arch}.block_count": CFG["layers"], f"{arch}.embedding_length": d,
            f"{arch}.attention.head_count": CFG["heads"], f"{arch}.attention.head_count_kv": CFG["kv_heads"], f"{arch}.feed_forward_length": ffn,
            f"{arch}.attention.layer_norm_rms_epsilon": float(CFG["rms_eps"]), f"{arch}.rope.freq_base": float(CFG["rope_theta"]),
            f"{arch}.context_length": CFG["max_ctx"], "tokenizer.ggml.model": "llama", "tokenizer.ggml.tokens": toks,
            "tokenizer.ggml.scores": [float(s) for s in scores], "tokenizer.ggml.token_type": [int(t) for t in types],
            "tokenizer.ggml.bos_token_id": 1, "tokenizer.ggml.eos_token_id": 2, "tokenizer.ggml.add_bos_token": True}
    write_gguf(path, meta, tensors)
    return dict(layers=layers, out_norm=out_norm, out_w=out_w, emb=(emb_id, emb_raw), vocab=vocab)


def embedding_rows(emb, vocab, d):
    from oracle import oracle
    tid, raw = emb
    if tid == 0:
        return np.asarray(raw, dtype=np.float32).reshape(vocab, d)
    if tid == 1:
        return np.asarray(raw).view(np.float16).reshape(vocab, d).astype(np.float32)
    return oracle.dequantize(tid, raw, vocab * d).reshape(vocab, d)


@pytest.mark.gpu
@pytest.mark.parametrize("arch,embd_fmt,tied", [("llama", "Q8_0", False), ("testarch", "Q4_K", False), ("llama", "F16", False), ("llama", "Q6_K", True)])
def test_generate_from_a_gguf_file(tmp_path, arch, embd_fmt, tied):
    import jitnn_amd
    path = tmp_path / "tiny.gguf"
    ref = write_model(path, arch, 7, embd_fmt, tied)
    cfg = dict(CFG, vocab=ref["vocab"])
    with jitnn_amd.Llm.load(path) as llm:
        info = llm.info()
        assert (info.architecture, info.layers, info.d_model, info.heads, info.kv_heads, info.vocab) == (arch, 2, 256, 4, 2, ref["vocab"])
        # LlmAccelTest.weightsAreJitnnTensorsToo: the file's weights are tensors of this library too
        wq = llm.gguf().tensor("blk.0.attn_q.weight")
        assert wq.dim(1) == llm.gguf().integer(f"{arch}.embedding_length") and np.isfinite(wq.to_float_array()[0])
        # embedding lookup: every row, bit for bit
        table = embedding_rows(ref["emb"], ref["vocab"], 256)
        got = llm.model().embed(np.arange(ref["vocab"]))
        assert np.array_equal(got.view(np.uint32), table.view(np.uint32))
        # LlmAccelTest.generatesGreedily: not blank, deterministic, streamed pieces add up
        streamed = []
        prompt = "the cat sat on the"
        a = llm.generate(prompt, 12, streamed.append)
        b = llm.generate(prompt, 12)
        assert a.strip() != "" and a == b and a == "".join(streamed)
        # token level against the oracle: the prompt token by token, then every chosen token is the arg-max of the oracle's logits
        ids = llm.tokenizer().encode(prompt)
        out = llm.generate_tokens(ids, 12)
        assert llm.tokenizer().decode(out) == a or llm.tokenizer().decode(out).startswith(a)
        kc = np.zeros((2, CFG["max_ctx"], 2, 64), dtype=np.float32)
        vc = np.zeros_like(kc)
        inter = arch == "llama"
        logits = None
        for pos, t in enumerate(ids):
            logits = decode_ref(cfg, ref["layers"], ref["out_norm"], ref["out_w"], kc, vc, table[t], pos, rope_interleaved=inter)
        pos = len(ids)
        for step, t in enumerate(out):
            best = int(np.argmax(logits))
            margin = float(logits[best] - logits[t]) / max(float(np.abs(logits).max()), 1e-6)
            assert t == best or margin <= 1e-4, (step, t, best, margin)  # (a different token only on a tie within the GEMV bar)
            if step + 1 < len(out):
                logits = decode_ref(cfg, ref["layers"], ref["out_norm"], ref["out_w"], kc, vc, table[t], pos, rope_interleaved=inter)
                pos += 1
        # stops at the end-of-sequence token: make it the most likely continuation by asking for it as the eos id
        first = out[0]
        assert llm.model().generate(ids, 5, eos_token=first) == []


@pytest.mark.gpu
def test_generate_request_sampling_and_stop(tmp_path):
    """generate(request) (Llm.java:84-93): temperature 0 is the greedy loop of the library token for token; a seed fixes a
    sampled continuation; a stop sequence ends the text in front of itself; the length limit and the end-of-sequence token
    are told apart; the streamed pieces add up to the text."""
    import jitnn_amd
    from jitnn_amd import GenerationRequest
    path = tmp_path / "tiny.gguf"
    write_model(path, "llama", 7)
    with jitnn_amd.Llm.load(path) as llm:
        prompt = "the cat sat on the"
        ids = llm.tokenizer().encode(prompt)
        greedy_ids, greedy = llm.generate_tokens(ids, 12), llm.generate(prompt, 12)
        streamed = []
        r = llm.generate(GenerationRequest(prompt, 12, on_token=streamed.append))
        assert r.tokens == greedy_ids and r.text == greedy == "".join(streamed) and r.prompt_tokens == len(ids)
        assert r.finish_reason == ("length" if len(greedy_ids) == 12 else "eos")
        a = llm.generate(GenerationRequest(prompt, 16, temperature=0.9, top_k=40, top_p=0.95, seed=3))
        b = llm.generate(GenerationRequest(prompt, 16, temperature=0.9, top_k=40, top_p=0.95, seed=3))
        others = [llm.generate(GenerationRequest(prompt, 16, temperature=0.9, seed=s)).tokens for s in range(4, 10)]
        assert a.tokens == b.tokens and a.text == b.text and any(t != a.tokens for t in others)
        assert llm.generate(GenerationRequest(prompt, 16, temperature=5.0, top_k=1, seed=1)).tokens == llm.generate_tokens(ids, 16)
        # a stop sequence taken from the middle of the greedy text: the text ends in front of it
        if len(greedy) >= 6:
            stop = greedy[len(greedy) // 2:len(greedy) // 2 + 3]
            streamed = []
            s = llm.generate(GenerationRequest(prompt, 12, stop=[stop], on_token=streamed.append))
            assert s.finish_reason == "stop" and s.text == greedy[:greedy.find(stop)] == "".join(streamed)
        assert llm.generate(GenerationRequest(prompt, 0)).tokens == []
        with pytest.raises(ValueError):
            llm.generate(GenerationRequest(prompt, 10 ** 6))


@pytest.mark.gpu
def test_argmax_kernel_ties_and_nan():
    import jitnn_amd
    dec = jitnn_amd.LlamaDecoder(1, 256, 4, 2, 64, 512, 5000, 8)
    rng = np.random.default_rng(3)
    x = rng.standard_normal(5000).astype(np.float32)
    assert dec.argmax(x) == int(np.argmax(x))
    x[[77, 4091, 1300]] = 9.0          # equal maxima: the lowest index wins, as a sequential scan would choose
    assert dec.argmax(x) == 77
    x[5] = np.nan                       # NaN never wins
    assert dec.argmax(x) == 77
    x[:] = -np.inf
    x[4999] = -1e30
    assert dec.argmax(x) == 4999
    dec.close()


@pytest.mark.gpu
def test_embedding_ids_outside_the_vocabulary():
    """jitnn_hip_llama_embed_dev takes its ids from the caller's device memory: an id below 0 or at / past the vocabulary reads
    nothing and gives a row of NaN (both table kinds), the rows of the valid ids beside it are right; the host mirror
    refuses such ids before anything is launched."""
    import ctypes as C
    import jitnn_amd
    from jitnn_amd import _lib
    vocab, d = 300, 256
    rng = np.random.default_rng(8)
    table = rng.standard_normal((vocab, d)).astype(np.float32)
    for fmt in ("F32", "Q8_0"):
        dec = jitnn_amd.LlamaDecoder(1, d, 4, 2, 64, 512, vocab, 8)
        if fmt == "F32":
            dec.set_embedding(0, table)
            want = table
        else:
            from oracle import oracle
            raw = oracle.quantize_q8_0(table.reshape(-1))
            dec.set_embedding(GGML_ID["Q8_0"], raw)
            want = oracle.dequantize(GGML_ID["Q8_0"], raw, vocab * d).reshape(vocab, d)
        with pytest.raises(ValueError):
            dec.embed([0, -1])
        with pytest.raises(ValueError):
            dec.embed([vocab])
        ids = torch.tensor([5, -1, vocab - 1, vocab, 2 ** 31 - 1, 0], dtype=torch.int32, device="cuda")
        x = torch.zeros(ids.numel(), d, device="cuda")
        _lib.check(_lib.lib.jitnn_hip_llama_embed_dev(dec.handle, C.c_void_p(ids.data_ptr()), ids.numel(), C.c_void_p(x.data_ptr()), None), "embed")
        torch.cuda.synchronize()
        got = x.cpu().numpy()
        for row, i in enumerate(ids.tolist()):
            if 0 <= i < vocab:
                assert np.array_equal(got[row], want[i]), (fmt, i)
            else:
                assert np.isnan(got[row]).all(), (fmt, i)
        dec.close()


def test_generate_argument_checks():
    pytest.importorskip("torch")
    import jitnn_amd
    from jitnn_amd import _lib
    assert _lib.lib.jitnn_hip_llama_generate(None, None, 1, 0, 1, -1, None, None, None) == _lib.EINVAL
    assert _lib.lib.jitnn_hip_llama_set_embedding(None, 0, None, 0) == _lib.EINVAL
    with pytest.raises(ValueError):
        jitnn_amd.Tokenizer("wordpiece", ["a"])
