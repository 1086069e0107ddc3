"""The C-ABI library loads on a host without a GPU and exports every symbol that
include/dynaflow_hip.h declares (no kernel is launched here)."""
import ctypes
import os
import re

import pytest
import torch

from dynaflow_amd import _cabi

HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "dynaflow_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dfhip_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert declared_symbols() == sorted(_cabi.SIGNATURES)


def test_library_exports_every_declared_symbol():
    assert _cabi.is_built(), "build the library first: make -C dynaflow_amd/csrc"
    lib = ctypes.CDLL(_cabi.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(lib, name), name


def test_version_arch_and_status_text():
    lib = _cabi.load()
    assert lib.dfhip_version() >= 1000
    assert lib.dfhip_arch() == b"gfx950"
    assert lib.dfhip_status_string(0) == b"ok"
    assert b"null" in lib.dfhip_status_string(-1)
    with pytest.raises(_cabi.KernelError) as err:
        _cabi.check("dfhip_gemm_bf16_nt", -2)
    assert "unsupported shape" in str(err.value)


def test_argument_checks_run_before_any_launch():
    lib = _cabi.load()
    # null pointers and bad shapes are rejected on the host; nothing reaches a device
    assert lib.dfhip_gemm_bf16_nt(None, 64, None, 64, None, 64, 1, 8, 64, None) == -1
    assert lib.dfhip_gemm_bf16_nt(16, 64, 16, 64, 16, 64, 1, 8, 63, None) == -2      # K % 64
    assert lib.dfhip_gemm_bf16_nt(16, 32, 16, 64, 16, 64, 1, 8, 64, None) == -3      # lda < K
    assert lib.dfhip_gemm_bf16_nt(8, 64, 16, 64, 16, 64, 1, 8, 64, None) == -4       # alignment
    # a tile's 256 rows must stay within 32-bit byte offsets: leading dimensions from 2^22 elements on are refused
    assert lib.dfhip_gemm_bf16_nt(16, 1 << 22, 16, 64, 16, 64, 1, 8, 64, None) == -3
    assert lib.dfhip_gemm_bf16_nt(16, 64, 16, 1 << 22, 16, 64, 1, 8, 64, None) == -3
    assert lib.dfhip_gemm_bf16_nt_variant(16, 64, 16, 64, 16, 64, 1, 8, 64, 99, None) == -7
    assert lib.dfhip_silu_mul_bf16(16, 8, 16, 8, 16, 8, 1, 7, 0, None) == -2
    assert lib.dfhip_rmsnorm_bf16(16, None, 16, 16, None, 1, 20000, 1e-5, None) == -2
    assert lib.dfhip_gemm_fp8_nt(16, 128, 16, 128, 16, 8, None, None, 1, 8, 128, None) == -1
    # the split-K entry point with the library's own scratch array refuses what does not fit it
    assert lib.dfhip_gemm_bf16_nt_splitk_static(16, 4096, 16, 4096, 16, 4096, 4096, 4096, 4096, 2, None) == -8
    assert lib.dfhip_gemm_bf16_nt_splitk_static(None, 4096, 16, 4096, 16, 4096, 4096, 4096, 4096, 2, None) == -1
    assert lib.dfhip_gemm_bf16_nt_splitk_static(16, 4096, 16, 4096, 16, 4096, 256, 256, 4096, 17, None) == -7
    # decode attention with the append in the same launch: pointers, head grouping, capacity, row stride, alignment
    one = lib.dfhip_decode_attention_append_bf16
    assert one(None, 768, 16, 16, 16, 16, 16, 16, 16, 512, 1, 4, 1, 128, 1, 32, 32, 0.1, None) == -1
    assert one(16, 768, 16, 16, 16, 16, 16, 16, 16, 512, 1, 4, 3, 128, 1, 32, 32, 0.1, None) == -2      # 4 % 3
    assert one(16, 768, 16, 16, 16, 16, 16, 16, 16, 512, 1, 4, 1, 128, 1, 48, 32, 0.1, None) == -2      # capacity % 32
    assert one(16, 512, 16, 16, 16, 16, 16, 16, 16, 512, 1, 4, 1, 128, 1, 32, 32, 0.1, None) == -3      # row too short
    assert one(8, 768, 16, 16, 16, 16, 16, 16, 16, 512, 1, 4, 1, 128, 1, 32, 32, 0.1, None) == -4       # alignment
    assert b"scratch" in lib.dfhip_status_string(-8)


def _splitk_launch_order(lib, tiles, split_k):
    """{tile: [(launch index, part), ...]} of a split-K launch, replayed on the host."""
    tile, part = ctypes.c_int(-1), ctypes.c_int(-1)
    order = {}
    for pid in range(tiles * split_k):
        assert lib.dfhip_gemm_bf16_splitk_work(pid, tiles, split_k, ctypes.byref(tile), ctypes.byref(part)) == 0
        order.setdefault(tile.value, []).append((pid, part.value))
    return order


@pytest.mark.parametrize("tiles,split_k", [
    (128, 2),            # down projection of a 2048-token nano-batch: [2048,14336] x [4096,14336]^T
    (100, 2), (36, 7), (50, 5), (6, 3),     # tile counts that are no multiple of the 8 XCDs
    (1, 8), (7, 8), (8, 8), (9, 2), (33, 4), (64, 4), (127, 2),
])
def test_split_k_waiter_is_the_last_of_its_tile_to_be_dispatched(tiles, split_k):
    """The part of a tile that waits for the others (part split_k - 1) must have the highest launch index of that
    tile: workgroups are dispatched in launch order, so everything it waits for is then running or done, whatever
    the tile count and however few compute units the launch gets.  Also: every (tile, part) is computed exactly
    once, and the parts of one K range are dealt to the XCDs (launch index % 8) in contiguous tile ranges."""
    lib = _cabi.load()
    order = _splitk_launch_order(lib, tiles, split_k)
    assert sorted(order) == list(range(tiles))
    for tile, work in order.items():
        assert sorted(part for _, part in work) == list(range(split_k)), (tile, work)
        waiter = max(work)                       # highest launch index of the tile
        assert waiter[1] == split_k - 1, (tile, work)
    for p in range(split_k):
        by_xcd = {}
        for tile, work in order.items():
            pid = next(pid for pid, part in work if part == p)
            by_xcd.setdefault(pid % 8, []).append(tile)
        for tiles_of_xcd in by_xcd.values():
            tiles_of_xcd.sort()
            assert tiles_of_xcd == list(range(tiles_of_xcd[0], tiles_of_xcd[0] + len(tiles_of_xcd)))


def test_split_k_planned_shapes_keep_the_waiter_last():
    """The same for the split the plan picks on the shapes the layers use (and their side-by-side plans)."""
    lib = _cabi.load()
    variant, split_k = ctypes.c_int(0), ctypes.c_int(1)
    seen = 0
    for M in (256, 300, 512, 768, 1024, 1536, 2048, 4096, 8192):
        for N, K in ((4096, 14336), (4096, 4096), (6144, 4096), (14336, 4096), (8192, 28672), (264, 512)):
            for share in (1, 2, 4):
                assert lib.dfhip_gemm_bf16_plan_shared(M, N, K, share, ctypes.byref(variant), ctypes.byref(split_k)) == 0
                if variant.value != 0 or split_k.value < 2:
                    continue
                seen += 1
                tiles = ((M + 255) // 256) * ((N + 255) // 256)
                for tile, work in _splitk_launch_order(lib, tiles, split_k.value).items():
                    assert max(work)[1] == split_k.value - 1, (M, N, K, share, tile, work)
    assert seen > 0
    bad = ctypes.c_int(0)
    assert lib.dfhip_gemm_bf16_splitk_work(16, 8, 2, ctypes.byref(bad), ctypes.byref(bad)) == -7
    assert lib.dfhip_gemm_bf16_splitk_work(0, 8, 2, None, ctypes.byref(bad)) == -1


def test_operators_refuse_host_tensors():
    from dynaflow_amd import ops

    x = torch.randn(4, 64).bfloat16()
    w = torch.randn(8, 64).bfloat16()
    with pytest.raises((RuntimeError, NotImplementedError)):
        ops.linear(x, w)
    with pytest.raises((RuntimeError, NotImplementedError)):
        ops.silu_mul(x, x)


def test_missing_library_is_loud(monkeypatch):
    monkeypatch.setattr(_cabi, "_lib", None)
    monkeypatch.setattr(_cabi, "LIB_PATH", "/nonexistent/libdynaflow_hip.so")
    with pytest.raises(_cabi.KernelLibraryMissing):
        _cabi.load()


def test_header_is_plain_c_and_cpp():
    """The boundary is a C ABI: the header must go through a C99 compiler (no C++ in the signatures) and through a
    C++ compiler alike."""
    import shutil
    import subprocess

    gcc, gpp = shutil.which("gcc"), shutil.which("g++")
    if not gcc or not gpp:
        pytest.skip("no host compiler")
    subprocess.run([gcc, "-fsyntax-only", "-x", "c", "-std=c99", "-Wall", "-Werror", "-pedantic", HEADER], check=True)
    subprocess.run([gpp, "-fsyntax-only", "-x", "c++", "-std=c++11", "-Wall", "-Werror", HEADER], check=True)


def test_the_product_never_imports_the_oracle():
    """The oracle is test infrastructure: nothing in the package may import it, and the bench only inside its
    CPU leg (`cpu_baseline`), the smoke test only inside `smoke`."""
    import ast
    import pathlib

    root = pathlib.Path(__file__).resolve().parents[1]

    def oracle_imports(tree):
        found = []
        for node in ast.walk(tree):
            if isinstance(node, ast.Import):
                found += [node for a in node.names if a.name.split(".")[0] == "oracle"]
            elif isinstance(node, ast.ImportFrom) and (node.module or "").split(".")[0] == "oracle":
                found.append(node)
        return found

    for path in (root / "dynaflow_amd").rglob("*.py"):
        assert not oracle_imports(ast.parse(path.read_text())), f"{path} imports the oracle"
    for name, allowed in (("bench.py", "cpu_baseline"), ("__graft_entry__.py", "smoke")):
        tree = ast.parse((root / name).read_text())
        inside = set()
        for node in ast.walk(tree):
            if isinstance(node, ast.FunctionDef) and node.name == allowed:
                inside = {id(n) for n in oracle_imports(node)}
        assert inside, f"{name}: {allowed} was expected to use the oracle"
        assert {id(n) for n in oracle_imports(tree)} == inside, f"{name} imports the oracle outside {allowed}"


def test_bench_refuses_more_than_one_gpu_and_a_box_without_one():
    """`bench.py --gpus N` with N above 1 exits with a message that says so (before anything touches a GPU), and
    on a machine without a GPU the default run says that it needs one instead of printing a figure."""
    import pathlib
    import subprocess
    import sys

    root = pathlib.Path(__file__).resolve().parents[1]
    many = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                          timeout=120)
    assert many.returncode != 0 and many.stdout.strip() == ""
    assert "one GPU" in many.stderr and "--gpus 2" in many.stderr
    import torch

    if torch.cuda.is_available():
        return
    none = subprocess.run([sys.executable, str(root / "bench.py")], capture_output=True, text=True, timeout=300)
    assert none.returncode != 0 and none.stdout.strip() == ""
    assert "no GPU" in none.stderr
