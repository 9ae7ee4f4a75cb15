"""How the library behaves as a runtime component: replay of a captured decode step, several host threads and streams
at once, and the documented behaviour on non-finite activations.  All through the C ABI's device-pointer entry points,
with torch as the owner of device memory and streams."""
import ctypes as C
import threading

import numpy as np
import pytest
import torch

import quantizers
from helpers import GGML_ID, HOT_FORMATS, norm_err, random_valid_blocks

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def jn():
    import jitnn_amd
    jitnn_amd.init()
    return jitnn_amd


def vp(t):
    return C.c_void_p(t.data_ptr())


def linear_dev(jn, w, x, y, stream, bias=None):
    from jitnn_amd import _lib
    _lib.check(_lib.lib.jitnn_hip_linear_dev(w.handle, vp(x), x.shape[0], vp(bias) if bias is not None else None, vp(y),
                                             C.c_void_p(stream.cuda_stream)), "jitnn_hip_linear_dev")


def small_model(jn, seed=5):
    from decode_oracle import SLOTS
    cfg = dict(layers=2, d_model=512, heads=8, kv_heads=2, head_dim=64, ffn=1024, vocab=1000, max_ctx=48, rms_eps=1e-5, rope_theta=5e5)
    mix = {"attn_q": "Q4_K", "attn_k": "Q4_K", "attn_v": "Q6_K", "attn_o": "Q4_K", "ffn_gate": "Q4_K", "ffn_up": "Q4_K", "ffn_down": "Q6_K"}
    g = torch.Generator().manual_seed(seed)
    shapes = {"attn_q": (512, 512), "attn_k": (128, 512), "attn_v": (128, 512), "attn_o": (512, 512), "ffn_gate": (1024, 512),
              "ffn_up": (1024, 512), "ffn_down": (512, 1024)}
    dec = jn.LlamaDecoder(**cfg)
    for li in range(2):
        for si, slot in enumerate(SLOTS):
            n, k = shapes[slot]
            dec.set_weight(li, si, jn.Tensor.quantized(jn.DType[mix[slot]], quantizers.quantize(mix[slot], torch.randn(n, k, generator=g) * 0.02).numpy(), n, k))
        dec.set_norm(li, 0, np.ones(512, dtype=np.float32))
        dec.set_norm(li, 1, np.ones(512, dtype=np.float32))
    dec.set_norm(0, 2, np.ones(512, dtype=np.float32))
    dec.set_weight(0, 7, jn.Tensor.quantized(jn.DType.Q6_K, quantizers.quantize("Q6_K", torch.randn(1000, 512, generator=g) * 0.02).numpy(), 1000, 512))
    rng = np.random.default_rng(seed)
    for li in range(2):
        dec.kv_write(li, 0, rng.standard_normal((37, 2, 64)).astype(np.float32), rng.standard_normal((37, 2, 64)).astype(np.float32))
    return cfg, dec


def test_decode_step_replays_as_a_graph(jn):
    """The single-token step allocates nothing and records no memset, so it can be captured; every replay - with eager
    work of the same library and synchronisations in between - gives the bits of the eager step on the same input."""
    cfg, dec = small_model(jn)
    x = torch.randn(512, device="cuda", generator=torch.Generator(device="cuda").manual_seed(1))
    eager = torch.empty(1000, device="cuda")
    out = torch.empty(1000, device="cuda")
    st = torch.cuda.current_stream()
    dec.decode_dev(x.data_ptr(), 37, eager.data_ptr(), st.cuda_stream)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        dec.decode_dev(x.data_ptr(), 37, out.data_ptr(), torch.cuda.current_stream().cuda_stream)
    w = jn.Tensor.quantized(jn.DType.Q4_K, random_valid_blocks(np.random.default_rng(2), "Q4_K", 64, 512), 64, 512)
    xe, ye = torch.randn(3, 512, device="cuda"), torch.empty(3, 64, device="cuda")
    for i in range(4):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), i
        # eager work between the replays: another linear, and the same step at another position into another buffer
        linear_dev(jn, w, xe, ye, torch.cuda.current_stream())
        other = torch.empty(1000, device="cuda")
        dec.decode_dev(x.data_ptr(), 38 + i, other.data_ptr(), torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
    # a new input in the captured buffer is picked up by the next replay
    x.mul_(0.5)
    dec.decode_dev(x.data_ptr(), 37, eager.data_ptr(), torch.cuda.current_stream().cuda_stream)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, eager)
    dec.close()


@pytest.mark.parametrize("rows", [5, 96])
def test_two_host_threads_two_streams(jn, rows):
    """Two host threads, each on a stream of its own, call the library at the same time (5 rows: GEMV kernels; 96 rows: the
    many-row path with its per-thread scratch); every result equals the one the same call gives alone."""
    from oracle import oracle
    rng = np.random.default_rng(rows)
    n, k = 320, 2048
    raws = [random_valid_blocks(rng, f, n, k) for f in ("Q4_K", "Q6_K")]
    ws = [jn.Tensor.quantized(jn.DType[f], r, n, k) for f, r in zip(("Q4_K", "Q6_K"), raws)]
    iters = 24
    xs = [torch.randn(iters, rows, k, device="cuda", generator=torch.Generator(device="cuda").manual_seed(10 + t)) for t in range(2)]
    alone = [torch.empty(iters, rows, n, device="cuda") for _ in range(2)]
    for t in range(2):
        for i in range(iters):
            linear_dev(jn, ws[t], xs[t][i], alone[t][i], torch.cuda.current_stream())
    torch.cuda.synchronize()
    ref = oracle.gguf_linear(GGML_ID["Q4_K"], xs[0][0].cpu().numpy(), raws[0], None, n, k)
    assert norm_err(alone[0][0].cpu().numpy(), ref) <= (1e-4 if rows <= 64 else 2e-3)
    got = [torch.zeros(iters, rows, n, device="cuda") for _ in range(2)]
    errors = []
    start = threading.Barrier(2)

    def work(t):
        try:
            s = torch.cuda.Stream()
            start.wait()
            for i in range(iters):
                linear_dev(jn, ws[t], xs[t][i], got[t][i], s)
            s.synchronize()
        except Exception as e:  # surfaced below
            errors.append(e)

    threads = [threading.Thread(target=work, args=(t,)) for t in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
    torch.cuda.synchronize()
    for t in range(2):
        assert torch.equal(got[t], alone[t]), t


def test_worker_thread_gives_its_scratch_back(jn):
    """A thread that only ever calls a device-pointer entry point (here one 2048-row linear, which takes the thread's
    many-row scratch: 64 MiB of FP16 operands and more) returns that scratch when it ends: six such threads one after the
    other leave the free device memory where the first left it - a thread that kept its scratch would cost 64 MiB each,
    320 MiB over the five that are compared.  (The bar of 96 MiB leaves room for what the HIP runtime takes for itself
    along the way - pool blocks of several MiB per new host thread have been seen.)"""
    rng = np.random.default_rng(21)
    n, k, rows = 64, 16384, 2048
    w = jn.Tensor.quantized(jn.DType.Q4_K, random_valid_blocks(rng, "Q4_K", n, k), n, k)
    x = torch.randn(rows, k, device="cuda", generator=torch.Generator(device="cuda").manual_seed(4))
    y = torch.empty(rows, n, device="cuda")
    s = torch.cuda.Stream()
    errors = []

    def work():
        try:
            linear_dev(jn, w, x, y, s)
            s.synchronize()
        except Exception as e:  # surfaced below
            errors.append(e)

    def once():
        th = threading.Thread(target=work)
        th.start()
        th.join()
        torch.cuda.synchronize()
        return torch.cuda.mem_get_info()[0]

    free = [once() for _ in range(7)]   # (one-off allocations of the runtime happen in the first)
    assert not errors, errors
    assert free[1] - free[6] < (96 << 20), free


def test_one_thread_alternating_streams_many_rows(jn):
    """One host thread feeding the many-row path from two streams in turn: the second stream's call waits for the first
    one's use of the thread's scratch instead of overwriting it."""
    rng = np.random.default_rng(9)
    n, k, rows = 256, 4096, 130
    w = jn.Tensor.quantized(jn.DType.Q4_K, random_valid_blocks(rng, "Q4_K", n, k), n, k)
    xs = torch.randn(8, rows, k, device="cuda", generator=torch.Generator(device="cuda").manual_seed(3))
    alone = torch.empty(8, rows, n, device="cuda")
    for i in range(8):
        linear_dev(jn, w, xs[i], alone[i], torch.cuda.current_stream())
    torch.cuda.synchronize()
    s = [torch.cuda.Stream(), torch.cuda.Stream()]
    got = torch.zeros(8, rows, n, device="cuda")
    for i in range(8):
        linear_dev(jn, w, xs[i], got[i], s[i & 1])
    torch.cuda.synchronize()
    assert torch.equal(got, alone)


@pytest.mark.parametrize("fmt", HOT_FORMATS)
@pytest.mark.parametrize("rows", [1, 2, 4, 8, 80])
def test_non_finite_activations(jn, fmt, rows):
    """The reference's FP64 loop gives +-Inf or NaN in every output of a row that holds an Inf, and NaN for a NaN; this
    library gives a non-finite value in the same places - the same one of +Inf, -Inf and NaN up to four rows, NaN where the
    reference has +-Inf on the kernels of more rows, which split or rescale activations - and leaves the other rows of the batch
    untouched."""
    from oracle import oracle
    rng = np.random.default_rng(rows + GGML_ID[fmt])
    n, k = 48, 1024
    raw = random_valid_blocks(rng, fmt, n, k)
    w = jn.Tensor.quantized(jn.DType[fmt], raw, n, k)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    ref_clean = oracle.gguf_linear(GGML_ID[fmt], x, raw, None, n, k)
    bad = x.copy()
    bad[0, 517] = np.inf
    if rows > 1:
        bad[rows - 1, 3] = np.nan
    with np.errstate(invalid="ignore", over="ignore"):
        ref = oracle.gguf_linear(GGML_ID[fmt], bad, raw, None, n, k)
    y = jn.Gguf.linear(jn.Tensor.of(bad), w, None).numpy()
    assert not np.isfinite(ref[0]).any() and not np.isfinite(y[0]).any()
    if rows <= 4:
        # the kernel of one to four rows multiplies a slice that holds a non-finite activation weight by weight in FP32:
        # +Inf, -Inf and NaN fall where the reference's FP64 sum has them, in every row
        for r in range(rows):
            assert np.array_equal(np.isnan(y[r]), np.isnan(ref[r])), (fmt, rows, r)
            assert np.array_equal(np.isposinf(y[r]), np.isposinf(ref[r])) and np.array_equal(np.isneginf(y[r]), np.isneginf(ref[r])), (fmt, rows, r)
    if rows > 1:
        assert np.isnan(ref[rows - 1]).all() and np.isnan(y[rows - 1]).all()
    bar = 1e-4 if rows <= 64 else 2e-3
    for r in range(1, rows - 1):
        assert norm_err(y[r], ref_clean[r]) <= bar, (fmt, rows, r)
