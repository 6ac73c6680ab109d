"""The benchmark configurations at their full sizes, where the CPU oracle would take hours:
checked through what the mathematics fixes whatever the size (Freivalds' product check,
exactness of fp16 products and of max, softmax rows summing to one, a permute undone by its
inverse) and against double-precision restatements of sampled rows / heads on the host."""
import numpy as np
import pytest

import bench
import einsummable_amd as ea
from helpers import stream_handle

pytestmark = pytest.mark.gpu

E = ea.Einsummable


def run(km, e, out, inns):
    assert km.build(e) == 0
    km(e, stream_handle(), out.data_ptr(), [t.data_ptr() for t in inns])


def test_c1_f32_matmul_2048_cubed(km):
    import torch

    n = 2048
    g = torch.Generator(device="cuda").manual_seed(11)
    a = torch.rand(n, n, device="cuda", generator=g) * 2 - 1
    b = torch.rand(n, n, device="cuda", generator=g) * 2 - 1
    c = torch.empty(n, n, device="cuda")
    e = E.from_str("ij,jk->ik", dict(i=n, j=n, k=n), "*[hole|f32@0,hole|f32@1]", "+")
    run(km, e, c, [a, b])
    torch.cuda.synchronize()
    assert km.describe(e).startswith("contraction_mfma_f32")
    A, B, C = (t.cpu().numpy().astype(np.float64) for t in (a, b, c))
    # Freivalds: C v = A (B v) for random v; a wrong tile, a dropped k-slice or a transposed
    # operand changes the left side by far more than the rounding bound
    r = np.random.RandomState(12)
    for _ in range(4):
        v = r.uniform(-1, 1, n)
        lhs, rhs = C @ v, A @ (B @ v)
        assert np.max(np.abs(lhs - rhs)) <= 1e-4 * np.sqrt(np.mean(rhs * rhs))
    # sampled entries against double precision: 1e-4 of the result's magnitude
    rows = r.randint(0, n, 64)
    want = A[rows] @ B
    scale = np.sqrt(np.mean(want * want))
    assert np.max(np.abs(C[rows] - want)) <= 1e-4 * max(scale, 1.0) * 4


def test_f32_product_whose_result_is_streamed_past_the_caches(km):
    # 4096 x 4096 f32 = 64 MiB: the size from which the result is stored with streaming
    # stores (written as instructions); a short reduction keeps the check cheap
    import torch

    m, k = 4096, 256
    g = torch.Generator(device="cuda").manual_seed(13)
    a = torch.rand(m, k, device="cuda", generator=g) * 2 - 1
    b = torch.rand(m, k, device="cuda", generator=g) * 2 - 1
    c = torch.full((m, m), float("nan"), device="cuda")
    e = E.from_str("ij,kj->ik", dict(i=m, j=k, k=m), "*[hole|f32@0,hole|f32@1]", "+")
    run(km, e, c, [a, b])
    torch.cuda.synchronize()
    assert "load=direct_to_lds" in km.describe(e)
    A, B, C = (t.cpu().numpy().astype(np.float64) for t in (a, b, c))
    assert not np.isnan(C).any()              # every element was written
    r = np.random.RandomState(14)
    for _ in range(4):
        v = r.uniform(-1, 1, m)
        lhs, rhs = C @ v, A @ (B.T @ v)
        assert np.max(np.abs(lhs - rhs)) <= 1e-4 * np.sqrt(np.mean(rhs * rhs))
    rows = r.randint(0, m, 64)
    want = A[rows] @ B.T
    assert np.max(np.abs(C[rows] - want)) <= 1e-4 * np.sqrt(np.mean(want * want)) * 4


def test_c2_elementwise_and_reductions_8192_squared(km):
    import torch

    n = 8192
    g = torch.Generator(device="cuda").manual_seed(13)
    x = torch.randn(n, n, device="cuda", dtype=torch.float16, generator=g)
    y = torch.randn(n, n, device="cuda", dtype=torch.float16, generator=g)
    z, ex = torch.empty_like(x), torch.empty_like(x)
    m = torch.empty(n, device="cuda", dtype=torch.float16)
    s = torch.empty(n, device="cuda", dtype=torch.float16)
    nodes = bench.c2_nodes(n)
    run(km, nodes[0][1], z, [x, y])
    run(km, nodes[1][1], m, [x])
    run(km, nodes[2][1], ex, [x, m])
    run(km, nodes[3][1], s, [ex])
    torch.cuda.synchronize()
    X, Y = x.cpu().numpy(), y.cpu().numpy()
    # the product of two fp16 values is exact in fp32, so max(x,0)*y rounds once: exact
    want = (np.maximum(X.astype(np.float32), 0) * Y.astype(np.float32)).astype(np.float16)
    assert np.array_equal(z.cpu().numpy() + np.float16(0), want + np.float16(0))
    # max is exact in any order
    M = m.cpu().numpy()
    assert np.array_equal(M, X.max(axis=1))
    # exp(x - m): in (0, 1], equal to 1 where the maximum sits; 1e-2 against double
    EX = ex.cpu().numpy()
    assert EX.max() == 1.0 and EX.min() >= 0.0
    assert np.all(EX[np.arange(n), X.argmax(axis=1)] == 1.0)
    rows = np.random.RandomState(14).randint(0, n, 128)
    d = (X[rows].astype(np.float32) - M[rows, None].astype(np.float32)).astype(np.float16)
    ref = np.exp(d.astype(np.float64))
    assert np.max(np.abs(EX[rows] - ref) / np.maximum(ref, 1e-3)) <= 1e-2
    # row sums of the stored exponentials: 1e-2 against double
    ref_s = EX.astype(np.float64).sum(axis=1)
    assert np.max(np.abs(s.cpu().numpy() - ref_s) / ref_s) <= 1e-2


def test_c3a_permute_512_mib_and_its_inverse(km):
    import torch

    a, b, c, d = 32, 2048, 32, 128
    g = torch.Generator(device="cuda").manual_seed(15)
    x = torch.randn(a, b, c, d, device="cuda", dtype=torch.float16, generator=g)
    y = torch.empty(a, c, b, d, device="cuda", dtype=torch.float16)
    back = torch.empty_like(x)
    fwd = E([a, c, b, d], [[0, 2, 1, 3]], 4, "hole|f16@0")      # abcd -> acbd
    inv = E([a, b, c, d], [[0, 2, 1, 3]], 4, "hole|f16@0")      # acbd -> abcd
    run(km, fwd, y, [x])
    run(km, inv, back, [y])
    torch.cuda.synchronize()
    assert torch.equal(back.view(torch.int16), x.view(torch.int16))
    assert torch.equal(y.view(torch.int16), x.permute(0, 2, 1, 3).contiguous().view(torch.int16))


@pytest.mark.parametrize("chain", ["c4_nodes", "c4_fused_nodes"])
def test_c4_attention_chain_b4_h32_s2048_d128(km, chain):
    import torch

    b, h, s, d = 4, 32, 2048, 128
    g = torch.Generator(device="cuda").manual_seed(16)
    mem = {k: torch.randn(b, h, s, d, device="cuda", dtype=torch.float16, generator=g)
           for k in ("Q", "K", "V")}
    mem["S"] = torch.empty(b, h, s, s, device="cuda", dtype=torch.float16)
    mem["O"] = torch.empty(b, h, s, d, device="cuda", dtype=torch.float16)
    mem["m"] = torch.empty(b * h * s, device="cuda", dtype=torch.float16)
    mem["l"] = torch.empty(b * h * s, device="cuda", dtype=torch.float16)
    nodes = getattr(bench, chain)(b, h, s, d)
    heads = [(0, 0), (1, 17), (3, 31)]
    scores = {}
    for name, e, out, inns, _w, _u in nodes:
        run(km, e, mem[out], [mem[i] for i in inns])
        if name.startswith("scores"):
            torch.cuda.synchronize()
            scores = {bh: mem["S"][bh].cpu().numpy() for bh in heads}
    torch.cuda.synchronize()
    # softmax rows sum to one (fp16 entries: 2048 roundings of at most 2^-11 relative each)
    P = mem["S"]
    sums = P.float().sum(dim=-1)
    assert float((sums - 1).abs().max()) <= 1e-2
    for bh in heads:
        Q, K, V = (mem[k][bh].cpu().numpy().astype(np.float64) for k in ("Q", "K", "V"))
        logits = Q @ K.T
        if chain == "c4_fused_nodes":       # its first node already holds the scaled logits
            logits = logits * float(np.float16(0.0883789))
        got = scores[bh].astype(np.float64)
        scale = np.sqrt(np.mean(logits * logits))
        assert np.max(np.abs(got - logits) / np.maximum(np.abs(logits), scale)) <= 1e-2
        # the head end to end against double precision: every intermediate of the chain is
        # an fp16 tensor (unit round-off 4.9e-4), so individual outputs carry a few of those
        z = logits * 0.0883789 if chain == "c4_nodes" else logits
        p = np.exp(z - z.max(axis=1, keepdims=True))
        want = (p / p.sum(axis=1, keepdims=True)) @ V
        out = mem["O"][bh].cpu().numpy().astype(np.float64)
        err = np.abs(out - want)
        rms = np.sqrt(np.mean(want * want))
        assert np.sqrt(np.mean(err * err)) <= 2e-3 * rms
        assert np.mean(err > 1e-2 * np.maximum(np.abs(want), rms)) <= 1e-3
