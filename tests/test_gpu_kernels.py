"""Parity of every C-ABI kernel against the CPU oracle, on an MI355X.

Integer / byte results (e4m3 codes, bf16 bit patterns of elementwise ops) are
compared bit for bit, except where a transcendental is involved: SiLU uses expf,
whose last-ulp rounding may differ between libm and the device library, so bf16
outputs may differ by one ulp on a small fraction of elements.  GEMM results are
compared as max|got - want| / max|want| with the tolerance of the precision:
fp32 1e-5, bf16 2e-2, fp8 5e-2 (against the dequantised fp32 product).
"""
import numpy as np
import pytest
import torch

from oracle import cref, mlp

pytestmark = pytest.mark.gpu

TOL = {"fp32": 1e-5, "bf16": 2e-2, "fp8": 5e-2}


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the GPU"
    from dynaflow_amd import _cabi, ops as _ops

    _cabi.load()
    return _ops


def rel_err(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    return ((got - want).abs().max() / want.abs().max().clamp_min(1e-30)).item()


def u16(t):
    return t.contiguous().cpu().view(torch.int16).numpy().view(np.uint16)


def from_u16(a):
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def ulp_diff(a, b):
    return (a.cpu().view(torch.int16).int() - b.cpu().view(torch.int16).int()).abs()


def randn(shape, seed, std=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return torch.randn(shape, generator=g) * std


def test_device_info(ops):
    from dynaflow_amd import _cabi

    info = _cabi.device_info(0)
    assert info["arch_name"].startswith("gfx950")
    assert info["compute_units"] == 256 and info["wavefront_size"] == 64
    assert info["lds_bytes_per_block"] >= 160 * 1024


@pytest.mark.parametrize("M,N,K", [(1, 8, 64), (7, 24, 64), (128, 128, 128), (300, 264, 192), (257, 512, 256),
                                   (512, 1032, 320)])
@pytest.mark.parametrize("variant", [-1, 0, 1, 2, 3, 4, 5, 7])
def test_gemm_bf16_against_c_oracle(ops, M, N, K, variant):
    a = randn((M, K), 1).bfloat16()
    w = randn((N, K), 2, 0.05).bfloat16()
    want = from_u16(cref.gemm_nt_bf16(u16(a), u16(w)))
    if variant < 0:
        got = ops.linear(a.cuda(), w.cuda())
    else:
        got = ops.linear_variant(a.cuda(), w.cuda(), variant)
    torch.cuda.synchronize()
    assert got.shape == (M, N) and got.dtype == torch.bfloat16
    assert rel_err(got.float(), want.float()) < TOL["bf16"]
    # much tighter in practice: fp32 accumulation and one rounding, so each entry is within
    # one bf16 ulp of the exact value, plus fp32 accumulation noise on entries that cancel
    g, w_ = got.float().cpu(), want.float()
    assert bool(((g - w_).abs() <= 2 ** -7 * w_.abs() + 2e-4 * w_.abs().max()).all())


def test_gemm_bf16_row_strided_views_and_batched_input(ops):
    a_full = randn((64, 512), 3).bfloat16().cuda()
    w = randn((96, 256), 4, 0.05).bfloat16().cuda()
    a = a_full[:, 128:384]  # row stride 512, 16-byte aligned start
    got = ops.linear(a, w)
    want = torch.nn.functional.linear(a.float().cpu(), w.float().cpu())
    assert rel_err(got.float(), want) < TOL["bf16"]
    a3 = randn((4, 16, 256), 5).bfloat16().cuda()
    got3 = ops.linear(a3, w)
    assert got3.shape == (4, 16, 96)
    assert rel_err(got3.float(), torch.nn.functional.linear(a3.float().cpu(), w.float().cpu())) < TOL["bf16"]


def test_gemm_bf16_is_linear_in_its_input(ops):
    """Size-independent property at a large shape: (a1 + a2) W == a1 W + a2 W when the sums are exact."""
    M, N, K = 2048, 4096, 4096
    a1 = (torch.randint(-4, 5, (M, K), generator=torch.Generator().manual_seed(1)).float() / 4).bfloat16().cuda()
    a2 = (torch.randint(-4, 5, (M, K), generator=torch.Generator().manual_seed(2)).float() / 4).bfloat16().cuda()
    w = (torch.randint(-8, 9, (N, K), generator=torch.Generator().manual_seed(3)).float() / 64).bfloat16().cuda()
    # small integers over powers of two: every product and partial sum is exact in fp32
    y1, y2, y12 = ops.linear(a1, w).float(), ops.linear(a2, w).float(), ops.linear(a1 + a2, w).float()
    torch.cuda.synchronize()
    assert rel_err(y12, y1 + y2) < 2 ** -7
    # and the exact value on a sample of entries
    rows = torch.tensor([0, 1, 777, 2047])
    want = (a1[rows].double().cpu() @ w.double().cpu().t())
    assert rel_err(ops.linear(a1[rows].contiguous(), w).float(), want.bfloat16().float()) < 2 ** -7


@pytest.mark.parametrize("M,N,K", [(1, 4, 4), (5, 7, 12), (130, 129, 64), (256, 2816, 1024)])
def test_gemm_f32(ops, M, N, K):
    a = randn((M, K), 6)
    w = randn((N, K), 7, 0.02)
    want = torch.from_numpy(cref.gemm_nt_f32(a.numpy(), w.numpy())) if M * N * K < 5e7 else a.double() @ w.double().t()
    got = ops.linear(a.cuda(), w.cuda())
    assert got.dtype == torch.float32
    assert rel_err(got, want) < TOL["fp32"]


@pytest.mark.parametrize("M,D", [(1, 8), (3, 40), (128, 2816), (257, 14336)])
@pytest.mark.parametrize("round_silu", [False, True])
def test_silu_mul_bf16_bits(ops, M, D, round_silu):
    g = randn((M, D), 8, 3.0).bfloat16()
    u = randn((M, D), 9).bfloat16()
    want = from_u16(cref.silu_mul_bf16(u16(g), u16(u), round_silu))
    got = ops.silu_mul(g.cuda(), u.cuda(), round_silu)
    d = ulp_diff(got, want)
    # the kernel takes silu from the hardware exponential and reciprocal (a few fp32 ulp from the C oracle's
    # expf and division): a handful of results round to the neighbouring bf16 value, and with the intermediate
    # rounding such a neighbour can move the product by one more
    assert d.max() <= (2 if round_silu else 1) and (d > 0).float().mean() < 5e-3


def test_silu_mul_special_values_and_packed_layout(ops):
    vals = torch.tensor([0.0, -0.0, 1.0, -1.0, 20.0, -20.0, 88.0, -88.0, 100.0, -100.0, 3.0e38, -3.0e38,
                         float("inf"), -float("inf"), 1e-30, -1e-30]).bfloat16()
    g = vals.repeat(4, 1)
    u = torch.full_like(g, 2.0)
    want = from_u16(cref.silu_mul_bf16(u16(g), u16(u), False))
    got = ops.silu_mul(g.cuda(), u.cuda(), False).cpu()
    same = (got.view(torch.int16) == want.view(torch.int16)) | (torch.isnan(got.float()) & torch.isnan(want.float()))
    # silu(-88) = -5e-37: the hardware reciprocal of e^88 is a denormal and is flushed, the kernel gives -0
    same |= ((got.float() - want.float()).abs() < 1e-30) & (torch.signbit(got) == torch.signbit(want))
    assert bool(same.all()), (got, want)
    # packed gate_up[M, 2D]: halves passed as row-strided views
    packed = randn((33, 2 * 64), 10, 2.0).bfloat16().cuda()
    got = ops.silu_mul(packed[:, :64], packed[:, 64:], False)
    want = ops.silu_mul(packed[:, :64].contiguous(), packed[:, 64:].contiguous(), False)
    assert torch.equal(got, want)


def test_silu_mul_f32(ops):
    g, u = randn((37, 100), 11, 3.0), randn((37, 100), 12)
    got = ops.silu_mul(g.cuda(), u.cuda())
    want = (g.double() / (1 + torch.exp(-g.double()))) * u.double()
    assert rel_err(got, want) < TOL["fp32"]


@pytest.mark.parametrize("M,H", [(1, 8), (5, 512), (64, 4096), (3, 16384)])
def test_rms_norm(ops, M, H):
    x = randn((M, H), 13).bfloat16()
    w = (1 + 0.1 * randn((H,), 14)).bfloat16()
    want = from_u16(cref.rmsnorm_bf16(u16(x), u16(w), 1e-5))
    got = ops.rms_norm(x.cuda(), w.cuda(), 1e-5)
    # the row sum of squares is reduced in a different order than the sequential C loop, so the
    # scale can differ in its last bit; after the two roundings that is at most 2 bf16 ulps
    d = ulp_diff(got, want)
    assert d.max() <= 2 and (d > 0).float().mean() < 1e-2
    res = randn((M, H), 15).bfloat16()
    out, new_res = ops.add_rms_norm(x.cuda(), res.cuda(), w.cuda(), 1e-5)
    want_out, want_res = mlp.rms_norm(x, w, 1e-5, residual=res)
    assert torch.equal(new_res.cpu(), want_res)
    assert ulp_diff(out, want_out).max() <= 2


def test_transpose_weight(ops):
    w = randn((200, 136), 16).bfloat16().cuda()
    assert torch.equal(ops.transpose_weight(w), w.t().contiguous())


@pytest.mark.parametrize("M,D", [(1, 8), (9, 72), (256, 1024)])
def test_quant_fp8_codes_are_bit_exact(ops, M, D):
    x = randn((M, D), 17, 2.5).bfloat16()
    want_q, want_s = mlp.quant_e4m3(x)
    q, s = ops.quant_fp8(x.cuda())
    torch.cuda.synchronize()
    assert torch.equal(s.cpu(), want_s)
    got = q.cpu().view(torch.uint8)
    same = (got == want_q) | ((got & 0x7F == 0) & (want_q & 0x7F == 0))
    assert bool(same.all())
    # all-zero input: scale floor, codes zero
    q0, s0 = ops.quant_fp8(torch.zeros(2, 16, dtype=torch.bfloat16, device="cuda"))
    assert s0.item() == pytest.approx(1e-12 / 448) and int(q0.view(torch.uint8).max()) & 0x7F == 0


def test_silu_mul_quant_fp8(ops):
    g = randn((130, 256), 18, 3.0).bfloat16()
    u = randn((130, 256), 19).bfloat16()
    act = ops.silu_mul(g.cuda(), u.cuda(), False)
    want_q, want_s = mlp.quant_e4m3(act.cpu())
    q, s = ops.silu_mul_quant_fp8(g.cuda(), u.cuda())
    assert torch.equal(s.cpu(), want_s)
    got = q.cpu().view(torch.uint8)
    assert bool(((got == want_q) | ((got & 0x7F == 0) & (want_q & 0x7F == 0))).all())


@pytest.mark.parametrize("M,N,K", [(1, 8, 128), (65, 72, 256), (300, 264, 384), (512, 1024, 1024),
                                   (2048, 1024, 1024), (1100, 2056, 384), (1536, 1536, 128)])
def test_gemm_fp8_against_dequantised_fp32(ops, M, N, K):
    x = randn((M, K), 20).bfloat16()
    w = randn((N, K), 21, 0.02).bfloat16()
    xq, xs = mlp.quant_e4m3(x)
    wq, ws = mlp.quant_e4m3_per_channel(w)
    want = mlp.dequant(xq, xs) @ mlp.dequant(wq, ws).t()
    got = ops.linear_fp8(xq.cuda().view(torch.float8_e4m3fn), wq.cuda().view(torch.float8_e4m3fn), xs.cuda(), ws.cuda())
    assert got.dtype == torch.bfloat16 and got.shape == (M, N)
    assert rel_err(got.float(), want) < 2 ** -7  # products of e4m3 values are exact in fp32; one bf16 rounding
    # and the whole quantise->multiply chain against the unquantised product, at the fp8 tolerance
    assert rel_err(got.float(), x.float() @ w.float().t()) < TOL["fp8"] * (1 if K >= 256 else 4)


def test_kernel_errors_become_exceptions(ops):
    from dynaflow_amd import _cabi

    a = torch.zeros(4, 72, dtype=torch.bfloat16, device="cuda")  # K % 64 != 0
    w = torch.zeros(8, 72, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(_cabi.KernelError):
        ops.linear(a, w)
    with pytest.raises(RuntimeError):
        ops.linear(a, torch.zeros(8, 64, dtype=torch.bfloat16, device="cuda"))


@pytest.mark.parametrize("M,N,K,split_k", [(300, 264, 512, 2), (300, 264, 512, 3), (256, 512, 512, 8), (513, 256, 1024, 4)])
def test_gemm_bf16_split_k_against_c_oracle(ops, M, N, K, split_k):
    """Split-K through the C ABI: parts leave fp32 blocks in a workspace, the last part of a tile adds them to its own."""
    from dynaflow_amd import _cabi

    lib = _cabi.load()
    a = randn((M, K), 31).bfloat16()
    w = randn((N, K), 32, 0.05).bfloat16()
    want = from_u16(cref.gemm_nt_bf16(u16(a), u16(w))).float()
    ag, wg = a.cuda(), w.cuda()
    nbytes = lib.dfhip_gemm_bf16_splitk_workspace_bytes(M, N, split_k)
    assert nbytes > 0
    ws = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    outs = []
    for _ in range(3):  # the arrival counters must come back to zero after every launch
        out = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
        rc = lib.dfhip_gemm_bf16_nt_splitk(ag.data_ptr(), K, wg.data_ptr(), K, out.data_ptr(), N, M, N, K, split_k,
                                           ws.data_ptr(), nbytes, stream)
        assert rc == 0
        torch.cuda.synchronize()
        outs.append(out)
    g = outs[0].float().cpu()
    assert bool(((g - want).abs() <= 2 ** -7 * want.abs() + 2e-4 * want.abs().max()).all())
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[1], outs[2])
    tiles = ((M + 255) // 256) * ((N + 255) // 256)
    assert int(ws[: tiles * 4].view(torch.int32).abs().sum()) == 0
    # too small a workspace and too many parts are refused
    assert lib.dfhip_gemm_bf16_nt_splitk(ag.data_ptr(), K, wg.data_ptr(), K, out.data_ptr(), N, M, N, K, split_k,
                                         ws.data_ptr(), 16, stream) == -7
    assert lib.dfhip_gemm_bf16_nt_splitk(ag.data_ptr(), K, wg.data_ptr(), K, out.data_ptr(), N, M, N, K, 9,
                                         ws.data_ptr(), nbytes, stream) == -7


def test_split_k_last_part_gives_up_after_a_bounded_wait(ops):
    """The last part of a tile waits for the other parts' arrival count.  Forced from the host: the counters
    start at -5, so the count it waits for is never reached.  Every workgroup still ends (the wait is bounded,
    about half a second here), the tiles come back as NaN instead of a sum with missing parts, the counters are
    left at zero, and the next launch with the same workspace is correct."""
    from dynaflow_amd import _cabi

    lib = _cabi.load()
    M, N, K, split_k = 300, 264, 512, 2
    a = randn((M, K), 35).bfloat16().cuda()
    w = randn((N, K), 36, 0.05).bfloat16().cuda()
    nbytes = lib.dfhip_gemm_bf16_splitk_workspace_bytes(M, N, split_k)
    ws = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    tiles = ((M + 255) // 256) * ((N + 255) // 256)
    ws[: tiles * 4].view(torch.int32).fill_(-5)
    stream = torch.cuda.current_stream().cuda_stream
    out = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    assert lib.dfhip_gemm_bf16_nt_splitk(a.data_ptr(), K, w.data_ptr(), K, out.data_ptr(), N, M, N, K, split_k,
                                         ws.data_ptr(), nbytes, stream) == 0
    torch.cuda.synchronize()
    assert bool(torch.isnan(out.float()).all())
    assert int(ws[: tiles * 4].view(torch.int32).abs().sum()) == 0
    assert lib.dfhip_gemm_bf16_nt_splitk(a.data_ptr(), K, w.data_ptr(), K, out.data_ptr(), N, M, N, K, split_k,
                                         ws.data_ptr(), nbytes, stream) == 0
    torch.cuda.synchronize()
    want = a.float() @ w.float().t()
    assert rel_err(out.float(), want) < 2 ** -7


def test_down_projection_shape_uses_split_k_and_matches_unsplit(ops):
    """[2048,14336] x [4096,14336]^T has 128 tiles for 256 CUs: the plan splits K in two."""
    import ctypes
    from dynaflow_amd import _cabi

    lib = _cabi.load()
    v, s = ctypes.c_int(), ctypes.c_int()
    assert lib.dfhip_gemm_bf16_plan(2048, 4096, 14336, ctypes.byref(v), ctypes.byref(s)) == 0
    assert (v.value, s.value) == (0, 2)
    assert lib.dfhip_gemm_bf16_plan(2048, 14336, 4096, ctypes.byref(v), ctypes.byref(s)) == 0
    assert (v.value, s.value) == (5, 1)
    a = randn((2048, 14336), 33).bfloat16().cuda()
    w = randn((4096, 14336), 34, 0.02).bfloat16().cuda()
    split = ops.linear(a, w)
    again = ops.linear(a, w)
    whole = ops.linear_variant(a, w, -2)   # same kernel, K not split
    torch.cuda.synchronize()
    assert torch.equal(split, again)
    assert rel_err(split.float(), whole.float()) < 2 ** -7
    rows = torch.tensor([0, 255, 256, 1023, 2047])
    want = a[rows].double().cpu() @ w.double().cpu().t()
    assert rel_err(split[rows].float(), want) < 2 ** -7


@pytest.mark.parametrize("M,I,K", [(1, 8, 64), (300, 264, 192), (257, 136, 128), (512, 1408, 512),
                                   (2048, 14336, 128), (2000, 14328, 192), (128, 2048, 1024), (100, 1032, 1088),
                                   (256, 2048, 1024), (200, 1032, 1088),
                                   (1024, 8064, 640), (768, 10080, 704), (2048, 14336, 640)])
def test_gate_up_silu_fused_epilogue(ops, M, I, K):
    """One launch for linear, linear, silu, mul.  The epilogue applies the roundings of the separate kernels,
    so the result has the same bits as linear, linear, silu_mul.  The two large shapes take the 256 x (112
    gate + 112 up) tile (I = 7 * 2^k fills the rounds of 256 workgroups), the others the 256 x (128 + 128)
    tile; (2000, 14328) has ragged tiles in both directions.  The last four (M <= 256) take the weight-streaming
    kernel with both weights in one 128 x (32 gate + 32 up) x 2 tile, the last two of them in two row tiles.
    The last three have more full 256 x 112 tiles than the GPU has compute units and at least ten slabs of K:
    one workgroup per compute unit walks 2 tiles (288 tiles), 1 or 2 (270 tiles in panels of 3 tile rows,
    unevenly dealt to the XCDs) and 4 tiles, storing a tile while it multiplies the next."""
    x = randn((M, K), 41).bfloat16()
    wg = randn((I, K), 42, 0.05).bfloat16()
    wu = randn((I, K), 43, 0.05).bfloat16()
    got = ops.gate_up_silu(x.cuda(), wg.cuda(), wu.cuda())
    assert got.shape == (M, I) and got.dtype == torch.bfloat16
    # (-2: the planned kernel with K not split - a split changes the order of the fp32 additions)
    two = ops.silu_mul(ops.linear_variant(x.cuda(), wg.cuda(), -2), ops.linear_variant(x.cuda(), wu.cuda(), -2), True)
    assert torch.equal(got, two)
    # and against a float64 evaluation (three bf16 roundings; the one of the gate is amplified by
    # up to |1 + g(1 - sigmoid(g))| in silu)
    rows = torch.arange(0, M, max(1, M // 64))
    g = x[rows].double() @ wg.double().t()
    want = (g / (1 + torch.exp(-g))) * (x[rows].double() @ wu.double().t())
    g32, w32 = got[rows.cuda()].float().cpu(), want.float()
    assert bool(((g32 - w32).abs() <= 2 ** -5 * w32.abs() + 2e-3 * w32.abs().max()).all())


@pytest.mark.parametrize("M,I,K,share", [(128, 14336, 4096, 2), (100, 14336, 4096, 2), (1, 14336, 4096, 2),
                                         (128, 1088, 1024, 16), (77, 3000, 2048, 16), (256, 14336, 4096, 1),
                                         (200, 14336, 4096, 1), (129, 28672, 8192, 1)])
def test_weight_streaming_gate_up_silu_wide_tile_has_the_bits_of_the_narrow_one(ops, M, I, K, share):
    """Decode-sized gate/up/SiLU launches take 128 outputs per workgroup instead of 64 when the launches that run
    side by side (`share`), or the two row tiles of 129 .. 256 rows, still make at least 192 workgroups: the same
    instruction over K in the same order, so the same bits as the narrow tile - checked against launches of at
    most 128 rows planned alone (which take the narrow tile unless they have 192 column tiles of their own, as
    with 28672 outputs) and against the separate operators.
    Ragged rows and outputs (I = 1088, 3000 are no multiples of 128) included."""
    x = randn((M, K), 44).bfloat16().cuda()
    wg = randn((I, K), 45, 0.02).bfloat16().cuda()
    wu = randn((I, K), 46, 0.02).bfloat16().cuda()
    with ops.launch_options(side_by_side=share):
        got = ops.gate_up_silu(x, wg, wu)
    narrow = torch.cat([ops.gate_up_silu(x[lo:lo + 128].contiguous(), wg, wu) for lo in range(0, M, 128)])
    assert torch.equal(got, narrow)
    separate = ops.silu_mul(ops.linear_variant(x, wg, -2), ops.linear_variant(x, wu, -2), True)
    assert torch.equal(got, separate)


def test_plan_prefers_224_wide_tiles_for_llama_intermediate_size(ops):
    import ctypes

    from dynaflow_amd import _cabi

    lib = _cabi.load()
    v, s = ctypes.c_int(), ctypes.c_int()
    for shape, want in (((2048, 14336, 4096), (5, 1)), ((8192, 14336, 4096), (0, 1)), ((8192, 4096, 4096), (0, 1)),
                        ((2048, 4096, 14336), (0, 2)), ((2048, 28672, 8192), (5, 1)),
                        # more than 128 rows: the weight-streaming kernel only while its tiles fit one round
                        ((512, 14336, 4096), (7, 1)), ((640, 4096, 4096), (6, 1)), ((256, 14336, 4096), (6, 1)),
                        ((1024, 4096, 4096), (6, 1)), ((1024, 4096, 14336), (0, 4)), ((1024, 6144, 4096), (7, 1)),
                        # few 256 x 256 tiles and a short K: 256 x 128 tiles instead of a split along K
                        ((2048, 4096, 4096), (7, 1))):
        assert lib.dfhip_gemm_bf16_plan(*shape, ctypes.byref(v), ctypes.byref(s)) == 0
        assert (v.value, s.value) == want, shape


@pytest.mark.parametrize("B,S,heads,d", [(1, 5, 1, 16), (3, 17, 4, 64), (2, 128, 8, 128)])
def test_rope_against_complex_rotation(ops, B, S, heads, d):
    from dynaflow_amd.decoder import rope_tables
    from oracle import decoder as ref_decoder

    t = randn((B, S, heads, d), 51).bfloat16()
    cos, sin = rope_tables(S, d, 500000.0)
    got = ops.rope(t.cuda(), cos.cuda(), sin.cuda())
    want = ref_decoder.rope(t, 500000.0)          # float64 complex multiplication
    assert got.shape == t.shape
    assert bool(((got.float().cpu() - want.float()).abs() <= 2 ** -7 * want.float().abs() + 1e-6).all())
    assert torch.equal(got[:, 0].cpu(), t[:, 0])  # position 0 is the identity


def test_rope_pair_and_stacked_projections_have_the_bits_of_the_separate_operators(ops):
    """q / k / v as one product against stacked weights, then q and k rotated by one launch straight from the
    column ranges of that product: every result equals the separate operators' bit for bit (k's heads sit
    right behind q's, so the one-launch path is taken; with separate tensors the operator falls back)."""
    from dynaflow_amd.decoder import rope_tables

    B, S, hq, hk, d, H = 2, 64, 8, 2, 128, 1024
    x = randn((B, S, H), 61).bfloat16().cuda()
    wq, wk, wv = (randn((n, H), 62 + i, 0.03).bfloat16().cuda() for i, n in enumerate((hq * d, hk * d, hk * d)))
    cos, sin = (t.cuda() for t in rope_tables(S, d, 500000.0))
    q, k, v = ops.linear_multi(x, [wq, wk, wv])
    assert q.data_ptr() + hq * d * 2 == k.data_ptr()                 # column ranges of one buffer
    # the stacked product picks its own kernel plan: equal to the separate products up to the order of the
    # fp32 additions (a split along K or not), i.e. within a bf16 rounding of the separate results
    for got, w in ((q, wq), (k, wk), (v, wv)):
        want = ops.linear(x, w)
        assert got.shape == want.shape
        assert rel_err(got.float(), want.float()) < 2 ** -7
    q4, k4 = q.view(B, S, hq, d), k.view(B, S, hk, d)
    rq, rk = ops.rope_pair(q4, k4, cos, sin)
    assert rq.data_ptr() + hq * d * 2 == rk.data_ptr()               # one launch, one buffer
    assert torch.equal(rq, ops.rope(q4.contiguous(), cos, sin)) and torch.equal(rk, ops.rope(k4.contiguous(), cos, sin))
    sq, sk = ops.rope_pair(q4.contiguous(), k4.contiguous(), cos, sin)   # separate tensors: two launches
    assert torch.equal(sq, rq) and torch.equal(sk, rk)
    # attention reads the token-strided views in place
    att = ops.causal_attention(rq, rk, v.view(B, S, hk, d))
    assert torch.equal(att, ops.causal_attention(rq.contiguous(), rk.contiguous(), v.view(B, S, hk, d).contiguous()))


@pytest.mark.parametrize("M,N,K", [(7, 24, 64), (128, 128, 128), (50, 264, 192), (128, 1032, 320), (1, 8, 64),
                                   (200, 264, 192), (512, 136, 128), (300, 1032, 320)])
def test_weight_streaming_gemm_small_shapes(ops, M, N, K):
    """The last three have two to four row tiles of 128 (the last one ragged)."""
    a = randn((M, K), 1).bfloat16()
    w = randn((N, K), 2, 0.05).bfloat16()
    want = from_u16(cref.gemm_nt_bf16(u16(a), u16(w)))
    got = ops.linear_variant(a.cuda(), w.cuda(), 6)
    torch.cuda.synchronize()
    g, w_ = got.float().cpu(), want.float()
    assert got.shape == (M, N)
    assert bool(((g - w_).abs() <= 2 ** -7 * w_.abs() + 2e-4 * w_.abs().max()).all())


@pytest.mark.parametrize("M,N,K,split", [(128, 4096, 4096, 5), (100, 6144, 4096, 5), (128, 14336, 4096, 2),
                                         (128, 4096, 14336, 8), (16, 1024, 1024, 1), (256, 4096, 4096, 4),
                                         (192, 14336, 4096, 1), (300, 4096, 14336, 2), (512, 6144, 4096, 1),
                                         (384, 4096, 4096, 2), (1000, 4096, 4096, 1), (256, 4096, 14336, 4)])
def test_weight_streaming_gemm_decode_shapes(ops, M, N, K, split):
    """M <= 128, and up to 512 rows (1024 with K <= 8192) while the 128 x 128 tiles fit one round of 256
    workgroups: the plan picks
    the weight-streaming kernel and splits K over as many workgroups as fit one round of 256 (at least 12 slabs of K
    per part); the parts are added in a
    fixed order, so the result is the same on every run."""
    import ctypes

    from dynaflow_amd import _cabi

    lib = _cabi.load()
    v, s = ctypes.c_int(), ctypes.c_int()
    assert lib.dfhip_gemm_bf16_plan(M, N, K, ctypes.byref(v), ctypes.byref(s)) == 0
    assert (v.value, s.value) == (6, split)
    a = randn((M, K), 61).bfloat16().cuda()
    w = randn((N, K), 62, 0.02).bfloat16().cuda()
    got = ops.linear(a, w)
    again = ops.linear(a, w)
    whole = ops.linear_variant(a, w, -2)     # the same kernel, K not split
    torch.cuda.synchronize()
    assert torch.equal(got, again)
    want = a.double().cpu() @ w.double().cpu().t()
    assert rel_err(got.float(), want) < 2 ** -7 and rel_err(whole.float(), want) < 2 ** -7
    g, w_ = got.float().cpu(), want.float()
    assert bool(((g - w_).abs() <= 2 ** -7 * w_.abs() + 2e-4 * w_.abs().max()).all())


@pytest.mark.parametrize("M,N,K", [(300, 264, 192), (7, 24, 64), (2048, 14336, 256), (2048, 4096, 256),
                                   (2048, 4096, 2048), (128, 4096, 4096), (100, 1032, 1088), (2000, 14328, 192),
                                   (256, 4096, 4096), (300, 1032, 1088)])
def test_linear_with_residual_epilogue(ops, M, N, K):
    """linear + add in one launch on every kernel the plan can pick (small tile, ring with and without split-K,
    256 x 224 tile, weight-streaming): the epilogue rounds like the two separate kernels, so the bits match."""
    x = randn((M, K), 71).bfloat16().cuda()
    w = randn((N, K), 72, 0.05).bfloat16().cuda()
    r = randn((M, N), 73).bfloat16().cuda()
    got = ops.linear_add(x, w, r)
    want = r + ops.linear(x, w)
    torch.cuda.synchronize()
    assert got.shape == (M, N) and torch.equal(got, want)
    assert torch.equal(ops.linear_add(x, w, r), got)      # run-to-run


@pytest.mark.parametrize("M,N,K", [(1, 8, 128), (300, 264, 384), (512, 1032, 1024), (2048, 3584, 256), (1100, 2056, 384)])
@pytest.mark.parametrize("variant", [0, 1, 2])
def test_gemm_fp8_variants_agree(ops, M, N, K, variant):
    """Every fp8 kernel (256x256 ring, register-staged 128x128, 256x224 ring) on the same operands: products of
    e4m3 values are exact in fp32 and all kernels add them in the same order, so the results are bit-identical."""
    x = randn((M, K), 20).bfloat16()
    w = randn((N, K), 21, 0.02).bfloat16()
    xq, xs = mlp.quant_e4m3(x)
    wq, ws = mlp.quant_e4m3_per_channel(w)
    args = (xq.cuda().view(torch.float8_e4m3fn), wq.cuda().view(torch.float8_e4m3fn), xs.cuda(), ws.cuda())
    got = ops.linear_fp8_variant(*args, variant)
    want = mlp.dequant(xq, xs) @ mlp.dequant(wq, ws).t()
    assert got.shape == (M, N) and rel_err(got.float(), want) < 2 ** -7
    assert torch.equal(got, ops.linear_fp8_variant(*args, 1))


@pytest.mark.parametrize("M,I,K", [(1, 8, 128), (300, 264, 384), (512, 1024, 1024), (2048, 3584, 256), (1100, 2056, 384)])
def test_fp8_gate_up_silu_epilogue_has_the_bits_of_the_separate_operators(ops, M, I, K):
    """One launch for the gate and up projection with SiLU*mul + absmax as the epilogue, then the re-quantiser:
    codes and scale must equal ``silu_mul_quant_fp8(linear_fp8(x, w_gate), linear_fp8(x, w_up))`` bit for bit
    (ragged last row / column tiles included), run to run as well."""
    x = randn((M, K), 30).bfloat16()
    wg = randn((I, K), 31, 0.05).bfloat16()
    wu = randn((I, K), 32, 0.05).bfloat16()
    xq, xs = mlp.quant_e4m3(x)
    wgq, wgs = mlp.quant_e4m3_per_channel(wg)
    wuq, wus = mlp.quant_e4m3_per_channel(wu)
    f8 = torch.float8_e4m3fn
    xq, wgq, wuq = xq.cuda().view(f8), wgq.cuda().view(f8), wuq.cuda().view(f8)
    xs, wgs, wus = xs.cuda(), wgs.cuda(), wus.cuda()
    want_q, want_s = ops.silu_mul_quant_fp8(ops.linear_fp8(xq, wgq, xs, wgs), ops.linear_fp8(xq, wuq, xs, wus))
    got_q, got_s = ops.gate_up_silu_quant_fp8(xq, wgq, wuq, xs, wgs, wus)
    torch.cuda.synchronize()
    assert got_q.shape == (M, I) and got_q.dtype == f8
    assert torch.equal(got_s, want_s)
    assert torch.equal(got_q.view(torch.uint8), want_q.view(torch.uint8))
    again_q, again_s = ops.gate_up_silu_quant_fp8(xq, wgq, wuq, xs, wgs, wus)
    assert torch.equal(again_q.view(torch.uint8), got_q.view(torch.uint8)) and torch.equal(again_s, got_s)


def _seeded_shapes(seed, count):
    import random
    rng = random.Random(seed)
    shapes = []
    for it in range(count):
        M = rng.choice([1, 17, 128, 129, 255, 256, 257, 511, 513, 700, 1024, 1500, 2048, 3000])
        N = 8 * rng.randint(1, 600) if it % 3 else rng.choice([224, 448, 896, 1792, 3584, 4096, 6144])
        K = 64 * rng.randint(1, 40) if it % 2 else rng.choice([64, 128, 192, 4096, 2048])
        shapes.append((M, N, K))
    return shapes


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", _seeded_shapes(20261, 24))
def test_planned_gemm_on_seeded_random_shapes(ops, M, N, K):
    """Whatever kernel and split the plan picks for a shape (ragged rows and columns, short and long K):
    `linear` against the fp32 product of the same bf16 operands (tolerance 2^-7 of the largest output: bf16
    output rounding plus fp32 accumulation order), `linear_add` with the bits of `linear` followed by `add`,
    and the fused gate/up/SiLU launch with the bits of the three separate launches."""
    a = randn((M, K), 51).bfloat16().cuda()
    w = randn((N, K), 52, 0.05).bfloat16().cuda()
    r = randn((M, N), 53).bfloat16().cuda()
    want = a.float() @ w.float().t()
    y = ops.linear(a, w)
    err = ((y.float() - want).abs().max() / want.abs().max().clamp_min(1e-30)).item()
    assert err <= 2.0 ** -7, (M, N, K, err)
    assert torch.equal(ops.linear_add(a, w, r), r + y)
    inter = (N // 16) * 8
    if inter >= 8:
        wg, wu = w[:inter].contiguous(), w[inter:2 * inter].contiguous()
        fused = ops.gate_up_silu(a, wg, wu)
        separate = ops.silu_mul(ops.linear_variant(a, wg, -2), ops.linear_variant(a, wu, -2), True)
        assert torch.equal(fused, separate)
    # the same operators planned for launches that share the GPU with one or three others of their shape: another
    # kernel or split for some shapes, the same product
    for share in (2, 4):
        with ops.launch_options(side_by_side=share):
            y_shared = ops.linear(a, w)
            err = ((y_shared.float() - want).abs().max() / want.abs().max().clamp_min(1e-30)).item()
            assert err <= 2.0 ** -7, (M, N, K, share, err)
            assert torch.equal(ops.linear_add(a, w, r), r + y_shared)
            if inter >= 8:
                assert torch.equal(ops.gate_up_silu(a, wg, wu), separate)


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(1, 8, 128), (100, 3584, 1536), (257, 1808, 384), (1100, 2456, 3072),
                                   (2048, 224, 2304), (4096, 3000, 640), (256, 8192, 1024), (700, 28672, 256)])
def test_planned_fp8_gemm_on_assorted_shapes(ops, M, N, K):
    """e4m3 `linear` with per-tensor activation scale and per-row weight scales against the fp32 product of the
    dequantised operands (tolerance 2^-6 of the largest output: the bf16 rounding of the output dominates)."""
    x = randn((M, K), 61).bfloat16().cuda()
    w = randn((N, K), 62, 0.05).bfloat16().cuda()
    xq, xs = ops.quant_fp8(x)
    ws = (w.float().abs().amax(dim=1) / 448.0).clamp_min(1e-12)
    wq = (w.float() / ws[:, None]).to(torch.float8_e4m3fn)
    got = ops.linear_fp8(xq, wq, xs, ws)
    want = (xq.float() * xs) @ (wq.float() * ws[:, None]).t()
    err = ((got.float() - want).abs().max() / want.abs().max().clamp_min(1e-30)).item()
    assert err <= 2.0 ** -6, (M, N, K, err)


def test_zero_row_inputs_give_empty_outputs(ops):
    """A nano-batch without tokens (a split index repeated) reaches the operators as a [0, H] tensor: every
    operator returns the empty tensor of the right shape and launches nothing; the C ABI itself refuses M = 0."""
    from dynaflow_amd import _cabi

    H, I = 128, 256
    x = torch.zeros(0, H, dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(I, H, dtype=torch.bfloat16, device="cuda")
    wd = torch.zeros(H, I, dtype=torch.bfloat16, device="cuda")
    act = ops.gate_up_silu(x, w, w)
    assert act.shape == (0, I) and act.dtype == torch.bfloat16
    assert ops.linear(x, w).shape == (0, I)
    assert ops.silu_mul(ops.linear(x, w), ops.linear(x, w), True).shape == (0, I)
    assert ops.linear(act, wd).shape == (0, H)
    assert ops.linear_add(act, wd, x).shape == (0, H)
    assert ops.rms_norm(x, torch.ones(H, dtype=torch.bfloat16, device="cuda"), 1e-5).shape == (0, H)
    both = ops.linear_multi(x, [w, w])
    assert [tuple(t.shape) for t in both] == [(0, I), (0, I)]
    x32 = torch.zeros(0, H, device="cuda")
    assert ops.linear(x32, w.float()).shape == (0, I)
    lib = _cabi.load()
    rc = lib.dfhip_gemm_bf16_nt(w.data_ptr(), H, w.data_ptr(), H, w.data_ptr(), I, 0, I, H, 0)
    assert rc == -2          # DFHIP_ERR_BAD_SHAPE
