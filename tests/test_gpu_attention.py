"""Prefill attention kernel on an MI355X, through the C ABI, against the float64 oracle."""
import pytest
import torch

from oracle import decoder as ref

pytestmark = pytest.mark.gpu
D = 128
TOL_BF16 = 2e-2


def rel_err(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    return ((got - want).abs().max() / want.abs().max().clamp_min(1e-30)).item()


@pytest.fixture(scope="module")
def ops():
    from dynaflow_amd import ops as _ops

    return _ops


def inputs(B, S, Hq, Hkv, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, S, Hq, D, generator=g).bfloat16()
    k = torch.randn(B, S, Hkv, D, generator=g).bfloat16()
    v = torch.randn(B, S, Hkv, D, generator=g).bfloat16()
    return q, k, v


@pytest.mark.parametrize("B,S,Hq,Hkv", [(1, 64, 1, 1), (2, 128, 4, 2), (3, 320, 8, 2), (1, 512, 4, 1), (2, 256, 3, 3),
                                        (8, 64, 4, 1), (1, 192, 2, 1), (1, 320, 3, 1), (1, 128, 8, 1),
                                        (2, 448, 16, 4), (1, 1024, 4, 1)])
def test_causal_attention_against_oracle(ops, B, S, Hq, Hkv):
    q, k, v = inputs(B, S, Hq, Hkv, S + Hq)
    print(f"causal attention B={B} S={S} Hq={Hq} Hkv={Hkv}", flush=True)
    got = ops.causal_attention(q.cuda(), k.cuda(), v.cuda())
    torch.cuda.synchronize()
    want = ref.attention(q.double(), k.double(), v.double())
    assert got.shape == (B, S, Hq, D) and got.dtype == torch.bfloat16
    assert rel_err(got.float(), want) < TOL_BF16
    # row by row: the first rows attend to few positions and are the most sensitive to a wrong mask
    err = (got.double().cpu() - want).abs().amax(dim=(0, 2, 3))
    assert bool((err < 0.05).all()), err.argmax()


def test_causal_attention_first_token_and_constant_values(ops):
    q, k, v = inputs(2, 192, 4, 2, 5)
    got = ops.causal_attention(q.cuda(), k.cuda(), v.cuda()).cpu()
    assert torch.equal(got[:, 0], v[:, 0].repeat_interleave(2, dim=1))     # one position: its value
    const = ops.causal_attention(q.cuda(), k.cuda(), torch.full_like(v, 0.75).cuda()).cpu()
    assert torch.equal(const, torch.full_like(const, 0.75))                 # softmax weights sum to 1


def test_causal_attention_strided_inputs(ops):
    """q, k, v as column blocks of one [T, (Hq + 2 Hkv) * 128] projection output: token stride != heads * 128."""
    B, S, Hq, Hkv = 2, 128, 4, 2
    g = torch.Generator().manual_seed(3)
    qkv = torch.randn(B * S, (Hq + 2 * Hkv) * D, generator=g).bfloat16().cuda()
    q = qkv[:, : Hq * D].view(B, S, Hq, D)
    k = qkv[:, Hq * D:(Hq + Hkv) * D].view(B, S, Hkv, D)
    v = qkv[:, (Hq + Hkv) * D:].view(B, S, Hkv, D)
    got = ops.causal_attention(q, k, v)
    want = ops.causal_attention(q.contiguous(), k.contiguous(), v.contiguous())
    assert torch.equal(got, want)
    assert rel_err(got.float(), ref.attention(q.double().cpu(), k.double().cpu(), v.double().cpu())) < TOL_BF16


def test_causal_attention_full_size_properties(ops):
    """4 sequences x 2048 tokens, 32 query / 8 kv heads (one nano-batch of the decoder configuration):
    sampled (sequence, head) pairs against the oracle, run-to-run bit identity, agreement with
    PyTorch's fused attention within the bf16 tolerance."""
    B, S, Hq, Hkv = 4, 2048, 32, 8
    gen = torch.Generator(device="cuda").manual_seed(9)
    q = torch.randn(B, S, Hq, D, generator=gen, device="cuda").bfloat16()
    k = torch.randn(B, S, Hkv, D, generator=gen, device="cuda").bfloat16()
    v = torch.randn(B, S, Hkv, D, generator=gen, device="cuda").bfloat16()
    print("causal attention full size", flush=True)
    got = ops.causal_attention(q, k, v)
    again = ops.causal_attention(q, k, v)
    torch.cuda.synchronize()
    assert torch.equal(got, again)
    for b, h in ((0, 0), (3, 31), (1, 13)):
        kv = h // (Hq // Hkv)
        want = ref.attention(q[b:b + 1, :, h:h + 1].double().cpu(), k[b:b + 1, :, kv:kv + 1].double().cpu(),
                             v[b:b + 1, :, kv:kv + 1].double().cpu())
        assert rel_err(got[b:b + 1, :, h:h + 1].float(), want) < TOL_BF16, (b, h)
    fused = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), is_causal=True, enable_gqa=True).transpose(1, 2)
    assert rel_err(got.float(), fused.float()) < TOL_BF16


def test_causal_attention_under_graph_capture(ops):
    q, k, v = (t.cuda() for t in inputs(2, 256, 4, 2, 21))
    eager = ops.causal_attention(q, k, v).clone()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = ops.causal_attention(q, k, v)
    for i in range(3):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {i}"
        torch.randn(256, 256, device="cuda").sum().item()


@pytest.mark.parametrize("Hq,Hkv", [(4, 2), (8, 2), (4, 1)])
def test_causal_attention_scores_that_outgrow_the_first_tile(ops, Hq, Hkv):
    """Rows whose later scores exceed the maximum of their first tile by far more than 2^64: the fast pass
    of those workgroups overflows its sums, notices, and the safe pass recomputes them with a running maximum.
    Half of the (sequence, head) pairs are affected, the others stay on the fast pass; both must match the
    oracle, and a second call gives the same bits.  Two and four query heads per kv head: both kernels (64 query
    rows per wave; 32 rows per wave with two workgroups per compute unit)."""
    B, S = 2, 512
    q, k, v = inputs(B, S, Hq, Hkv, 77)
    direction = torch.nn.functional.normalize(torch.randn(D, generator=torch.Generator().manual_seed(1)), dim=0)
    q[0] = (q[0].float() + 30.0 * direction).bfloat16()              # sequence 0: queries aligned with ...
    k[0, 300:] = (k[0, 300:].float() + 30.0 * direction).bfloat16()  # ... the late keys: logits of about +80 nats
    got = ops.causal_attention(q.cuda(), k.cuda(), v.cuda())
    again = ops.causal_attention(q.cuda(), k.cuda(), v.cuda())
    torch.cuda.synchronize()
    want = ref.attention(q.double(), k.double(), v.double())
    assert torch.isfinite(got.float()).all()
    assert rel_err(got.float(), want) < TOL_BF16
    err = (got.double().cpu() - want).abs().amax(dim=(2, 3))
    assert bool((err < 0.05).all()), err.argmax()
    assert torch.equal(got, again)
