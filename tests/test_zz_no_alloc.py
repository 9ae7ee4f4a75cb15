"""jitnn_hip_linear_noalloc_dev - the entry point that takes the scratch of a many-row launch from the library's fixed
device array instead of a buffer it may have to allocate - against jitnn_hip_linear_dev on the same inputs: the same
kernels on the same operands, so the same bits.  Calls in a row, each smaller than the first (the array keeps the earlier
calls' contents): the many-row kernel with K slices, the one-pass kernel for 9..64 rows, the GEMV range (no scratch at
all); then the size limit."""
import ctypes as C

import numpy as np
import pytest
import torch

from helpers import GGML_ID, norm_err, random_valid_blocks

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def jn():
    import jitnn_amd
    jitnn_amd.init()
    return jitnn_amd


def vp(t):
    return C.c_void_p(t.data_ptr())


def run(lib, name, w, x, bias, n):
    y = torch.full((x.shape[0], n), float("nan"), device="cuda")
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = getattr(lib.lib, name)(w.handle, vp(x), x.shape[0], vp(bias) if bias is not None else None, vp(y), st)
    lib.check(rc, name)
    torch.cuda.synchronize()
    return y


def test_noalloc_linear_matches_linear_dev(jn):
    from jitnn_amd import _lib as lib
    assert lib.lib.jitnn_hip_noalloc_scratch_bytes() == 64 << 20
    rng = np.random.default_rng(12)
    g = torch.Generator(device="cuda").manual_seed(12)
    # 4096 x 4096 at 512 rows splits K into slices (partial sums in the scratch); the second call is smaller in every way
    # (then: a ragged Q6_K launch, the one-pass kernel for 9..64 rows of Q4_K / Q5_K / Q4_1 - its prepared operands live in
    # the scratch too -, a 32-value format with rows of odd block counts, and a GEMV call that needs no scratch at all)
    calls = [("Q4_K", 4096, 4096, 512, True), ("Q6_K", 300, 1024, 97, False), ("Q4_K", 640, 2048, 40, True), ("Q5_K", 100, 1024, 17, False),
             ("Q4_1", 250, 1536, 33, True), ("Q8_0", 131, 32 * 9, 70, True), ("Q4_K", 192, 2048, 5, False)]
    for fmt, n, k, rows, with_bias in calls:
        w = jn.Tensor.quantized(jn.DType[fmt], random_valid_blocks(rng, fmt, n, k), n, k)
        x = torch.randn(rows, k, device="cuda", generator=g)
        bias = torch.randn(n, device="cuda", generator=g) if with_bias else None
        ref = run(lib, "jitnn_hip_linear_dev", w, x, bias, n)
        got = run(lib, "jitnn_hip_linear_noalloc_dev", w, x, bias, n)
        assert torch.isfinite(ref).all()
        assert torch.equal(got, ref), (fmt, n, k, rows)
        again = run(lib, "jitnn_hip_linear_noalloc_dev", w, x, bias, n)
        assert torch.equal(again, ref), (fmt, n, k, rows, "second call")


def test_noalloc_linear_against_the_oracle_without_allocating_and_under_graph_replay(jn):
    """The entry point against the CPU oracle (not only against its sibling), the property it exists for - a first-ever
    call of a size no earlier call of this process has had leaves the free device memory where it was -, and a many-row
    call captured into a HIP graph: every replay, with eager work between the replays, equals the eager result."""
    from jitnn_amd import _lib as lib
    from oracle import oracle
    rng = np.random.default_rng(14)
    g = torch.Generator(device="cuda").manual_seed(14)
    n, k, rows = 1536, 5120, 600   # (a size no other test of the suite uses)
    raw = random_valid_blocks(rng, "Q4_K", n, k)
    w = jn.Tensor.quantized(jn.DType.Q4_K, raw, n, k)
    x = torch.randn(rows, k, device="cuda", generator=g)
    y = torch.full((rows, n), float("nan"), device="cuda")
    st = torch.cuda.current_stream()
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    lib.check(lib.lib.jitnn_hip_linear_noalloc_dev(w.handle, vp(x), rows, None, vp(y), C.c_void_p(st.cuda_stream)), "noalloc")
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    sel = np.unique(np.linspace(0, rows - 1, 24).astype(np.int64))
    ref = oracle.gguf_linear(GGML_ID["Q4_K"], x[torch.as_tensor(sel, device="cuda")].cpu().numpy(), raw, None, n, k)
    assert norm_err(y.cpu().numpy()[sel], ref) <= 2e-3   # (more than 64 rows: the FP16 matrix-core path's bar)
    eager = y.clone()
    side = torch.cuda.Stream()
    side.wait_stream(st)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        y.fill_(0)
        with torch.cuda.graph(graph, stream=side):
            lib.check(lib.lib.jitnn_hip_linear_noalloc_dev(w.handle, vp(x), rows, None, vp(y), C.c_void_p(side.cuda_stream)), "noalloc (capture)")
    torch.cuda.synchronize()
    for i in range(3):
        y.fill_(float(i))                      # eager work between the replays
        small = run(lib, "jitnn_hip_linear_noalloc_dev", w, x[:40].contiguous(), None, n)   # the scratch is used by another call in between
        assert torch.isfinite(small).all()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager), i


def test_noalloc_linear_rejects_what_does_not_fit(jn):
    from jitnn_amd import _lib as lib
    rng = np.random.default_rng(13)
    n, k, rows = 64, 16384, 4096  # 4096 x 16384 FP16 activations alone are 128 MiB
    w = jn.Tensor.quantized(jn.DType.Q4_0, random_valid_blocks(rng, "Q4_0", n, k), n, k)
    x = torch.zeros(rows, k, device="cuda")
    y = torch.zeros(rows, n, device="cuda")
    rc = lib.lib.jitnn_hip_linear_noalloc_dev(w.handle, vp(x), rows, None, vp(y), None)
    assert rc == lib.EINVAL and "scratch" in lib.last_error()
    torch.cuda.synchronize()
