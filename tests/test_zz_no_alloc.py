"""dfhip_gemm_bf16_nt_splitk_static - the split-K GEMM whose arrival counters and fp32 partial blocks
live in a device array inside the library - against dfhip_gemm_bf16_nt_splitk with a caller's
workspace, through the C ABI.  Integer bar: the same bits.  Calls come in pairs, the second with a
smaller input, because every call on a GPU shares the one array and finds what the last call left.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu


def randn(shape, seed, std=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return torch.randn(shape, generator=g) * std


def both(lib, M, N, K, split_k, seed):
    """(with a caller's workspace, with the library's array, oracle rows) for one seeded problem."""
    a = randn((M, K), seed).bfloat16().cuda()
    w = randn((N, K), seed + 1, 0.03).bfloat16().cuda()
    stream = torch.cuda.current_stream().cuda_stream
    nbytes = lib.dfhip_gemm_bf16_splitk_workspace_bytes(M, N, split_k)
    ws = torch.zeros(max(nbytes, 16), dtype=torch.uint8, device="cuda")
    want = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    got = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    torch.cuda.synchronize()
    print(f"split-K static: M={M} N={N} K={K} split_k={split_k} seed={seed}", flush=True)
    assert lib.dfhip_gemm_bf16_nt_splitk(a.data_ptr(), K, w.data_ptr(), K, want.data_ptr(), N, M, N, K, split_k,
                                         ws.data_ptr(), nbytes, stream) == 0
    assert lib.dfhip_gemm_bf16_nt_splitk_static(a.data_ptr(), K, w.data_ptr(), K, got.data_ptr(), N, M, N, K,
                                                split_k, stream) == 0
    torch.cuda.synchronize()
    rows = torch.tensor([0, M // 2, M - 1])
    exact = a[rows].double().cpu() @ w.double().cpu().t()
    return want, got, rows, exact


# (first call, second and smaller call); the pairs cover the 256x256 ring kernel, the weight-streaming
# kernel (M <= 128) and a change of kernel between the two calls
PAIRS = [
    ((2048, 4096, 14336, 2), (700, 520, 1024, 4)),     # the full down projection: exactly the array's limit
    ((128, 4096, 4096, 6), (48, 1024, 2048, 3)),       # weight-streaming kernel, then a smaller one
    ((1300, 1024, 2048, 8), (16, 1024, 1024, 2)),      # ring kernel, then the weight-streaming kernel
]


@pytest.mark.parametrize("first,second", PAIRS)
def test_static_scratch_split_k_has_the_bits_of_the_workspace_entry_point(first, second):
    from dynaflow_amd import _cabi

    lib = _cabi.load()
    for seed, (M, N, K, split_k) in ((71, first), (73, second)):
        want, got, rows, exact = both(lib, M, N, K, split_k, seed)
        assert torch.equal(want, got), (M, N, K, split_k)
        err = (got[rows].double().cpu() - exact).abs().max() / exact.abs().max()
        assert err < 2 ** -7, err


def test_static_scratch_split_k_refuses_what_does_not_fit():
    from dynaflow_amd import _cabi

    lib = _cabi.load()
    M, N, K = 4096, 4096, 4096      # 256 tiles x 2 parts x 256 KiB = 128 MiB of partial blocks
    a = torch.zeros((M, K), dtype=torch.bfloat16, device="cuda")
    w = torch.zeros((N, K), dtype=torch.bfloat16, device="cuda")
    c = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.dfhip_gemm_bf16_nt_splitk_static(a.data_ptr(), K, w.data_ptr(), K, c.data_ptr(), N, M, N, K, 2, stream)
    assert rc == -8
    assert b"scratch" in lib.dfhip_status_string(rc)
    # split_k = 1 needs no scratch at all and runs
    assert lib.dfhip_gemm_bf16_nt_splitk_static(a.data_ptr(), K, w.data_ptr(), K, c.data_ptr(), N, M, N, K, 1,
                                                stream) == 0
    torch.cuda.synchronize()
    assert float(c.float().abs().max()) == 0.0


def test_static_scratch_split_k_under_graph_capture_replays_with_the_same_bits():
    """Once the library knows the array's address on this GPU (any earlier call outside capture: here the eager
    one) the call is legal in a captured graph: the counters are cleared by a fill kernel, no memset node and no
    allocation are recorded.  Replayed three times with eager work and synchronisations in between; every replay
    must give the bits of the eager call, also after the input changed."""
    from dynaflow_amd import _cabi

    lib = _cabi.load()
    M, N, K, split_k = 768, 1024, 2048, 4
    a = randn((M, K), 81).bfloat16().cuda()
    w = randn((N, K), 82, 0.03).bfloat16().cuda()
    eager = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    replayed = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")

    def call(out):
        rc = lib.dfhip_gemm_bf16_nt_splitk_static(a.data_ptr(), K, w.data_ptr(), K, out.data_ptr(), N, M, N, K,
                                                  split_k, torch.cuda.current_stream().cuda_stream)
        assert rc == 0, rc

    print(f"split-K static under capture: M={M} N={N} K={K} split_k={split_k}", flush=True)
    call(eager)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(replayed)
    for round_ in range(3):
        if round_:
            a.copy_(randn((M, K), 83 + round_).bfloat16())     # eager work between the replays
            call(eager)
        replayed.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(eager, replayed), round_
