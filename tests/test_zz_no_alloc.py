"""The entry point that allocates nothing, called through ctypes as a caller outside Python would:
``gemm_bf16_decode_split_static`` (partial sums in the library's own array on the GPU) against
``gemm_bf16_decode`` + ``sum_partials`` with a workspace of the caller's, on two calls in a row,
the second with a smaller input, so that what the first call left in the array must not matter."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

_i, _f, _vp, _sz = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t
STATIC_FLOATS = 1 << 20


def _lib():
    from mlx_lm_amd.ops import build

    lib = build.load("gemm_bf16_decode")
    assert hasattr(lib, "gemm_bf16_decode_split_static") and hasattr(lib, "gemm_bf16_decode_static_init")
    return lib


def _p(t):
    return _vp(t.data_ptr() if t is not None else 0)


def _stream():
    return _vp(torch.cuda.current_stream().cuda_stream)


def _existing(lib, out, a, w, bias, flags, n_splits):
    M, K = a.shape
    N = w.shape[0]
    ws = torch.full((n_splits * M * N,), float("nan"), dtype=torch.float32, device="cuda")
    nul = _vp(0)
    rc = lib.gemm_bf16_decode(_p(out), _p(a), _i(K), nul, _i(0), nul, nul, _f(0.0), _p(w), _p(bias), _i(M), _i(N),
                              _i(K), _i(K), _i(N), _i(flags), nul, nul, _sz(0), nul, _i(0), nul, nul, _i(0),
                              _i(0), _i(0), _i(0), _i(n_splits), _p(ws), _sz(ws.numel()), _stream())
    assert rc == 0, lib.mlxlm_last_error().decode()
    rc = lib.sum_partials(_p(out), _p(ws), _i(n_splits), _p(bias), _i(M), _i(N), _i(N), _i(flags), nul, nul,
                          _sz(0), nul, _i(0), nul, nul, _i(0), _i(0), _i(0), _i(0), _stream())
    assert rc == 0, lib.mlxlm_last_error().decode()


def _static(lib, out, a, w, bias, flags, n_splits):
    M, K = a.shape
    N = w.shape[0]
    return lib.gemm_bf16_decode_split_static(_p(out), _p(a), _i(K), _p(w), _p(bias), _i(M), _i(N), _i(K), _i(K),
                                             _i(N), _i(flags), _i(n_splits), _stream())


def test_split_product_without_a_workspace_twice_in_a_row():
    lib = _lib()
    assert lib.gemm_bf16_decode_static_init() == 0, lib.mlxlm_last_error().decode()
    g = torch.Generator().manual_seed(0)
    # (rows, features, K, parts, flags): bfloat16 out with GELU; then smaller, adding into float32
    for M, N, K, n_splits, flags in ((16, 1600, 6400, 5, 1), (5, 200, 1600, 3, 2)):
        a = torch.randn(M, K, generator=g).to(torch.bfloat16).cuda()
        w = (0.05 * torch.randn(N, K, generator=g)).to(torch.bfloat16).cuda()
        bias = torch.randn(N, generator=g).cuda()
        dtype = torch.float32 if flags & 6 else torch.bfloat16
        start = torch.randn(M, N, generator=g).to(dtype).cuda()
        want, got = start.clone(), start.clone()
        _existing(lib, want, a, w, bias, flags, n_splits)
        torch.cuda.synchronize()
        # free bytes of the device as the driver counts them: a hipMalloc inside the call would
        # show here (torch's own counters see only torch's allocator)
        before = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
        rc = _static(lib, got, a, w, bias, flags, n_splits)
        assert rc == 0, lib.mlxlm_last_error().decode()
        torch.cuda.synchronize()
        assert (torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()) == before
        assert torch.equal(got, want), (M, N, K)
        ref = a.float() @ w.float().t() + bias
        if flags & 1:
            ref = torch.nn.functional.gelu(ref, approximate="tanh")
        if flags & 2:
            ref = ref + start.float()
        assert (got.float() - ref).abs().max().item() <= 2e-2 * ref.abs().max().item()


def test_sizes_beyond_the_array_and_other_flags_are_refused():
    lib = _lib()
    a = torch.zeros(16, 6400, dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(8192, 6400, dtype=torch.bfloat16, device="cuda")
    out = torch.zeros(16, 8192, dtype=torch.bfloat16, device="cuda")
    assert 9 * 16 * 8192 > STATIC_FLOATS
    assert _static(lib, out, a, w, None, 0, 9) == 1
    assert "array holds" in lib.mlxlm_last_error().decode()
    assert _static(lib, out, a, w, None, 8, 2) == 1  # the cache scatter is not offered here
    assert "flags" in lib.mlxlm_last_error().decode()
    assert _static(lib, out, a, w, None, 0, 8) == 0  # exactly what fits
    torch.cuda.synchronize()


def test_the_call_can_be_captured_into_a_graph():
    """Under stream capture (global mode) an allocating call is an error that ends the capture; this
    one is recorded, and every replay gives what the eager entry points give."""
    lib = _lib()
    assert lib.gemm_bf16_decode_static_init() == 0, lib.mlxlm_last_error().decode()
    g = torch.Generator().manual_seed(1)
    M, N, K, n_splits, flags = 8, 1600, 1600, 4, 4
    a = torch.randn(M, K, generator=g).to(torch.bfloat16).cuda()
    w = (0.05 * torch.randn(N, K, generator=g)).to(torch.bfloat16).cuda()
    bias = torch.randn(N, generator=g).cuda()
    want = torch.zeros(M, N, dtype=torch.float32, device="cuda")
    got = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    assert _static(lib, got, a, w, bias, flags, n_splits) == 0  # warm-up: modules loaded, address looked up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, capture_error_mode="global"):
        rc = _static(lib, got, a, w, bias, flags, n_splits)
    assert rc == 0, lib.mlxlm_last_error().decode()
    for trial in range(3):
        a.copy_(torch.randn(M, K, generator=g).to(torch.bfloat16))  # eager work between the replays
        _existing(lib, want, a, w, bias, flags, n_splits)
        got.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, want), trial
