"""es_km_execute_static_workspace: the execute entry point that allocates nothing (the
workspace is device memory of the library's own).  Through the C ABI its results must be
bit-identical to es_km_execute with a workspace of the caller's, on calls in a row that share
the workspace, the later ones with smaller inputs."""
import numpy as np
import pytest

import einsummable_amd as ea
from helpers import (NP, assert_bits_equal, assert_close, empty_device, normal, oracle_einsummable,
                     rng, stream_handle, to_device, to_host, uniform)

import oracle

pytestmark = pytest.mark.gpu

E = ea.Einsummable
MUL = {"f16": "*[hole|f16@0,hole|f16@1]", "f32": "*[hole|f32@0,hole|f32@1]"}


def both_ways(km, e, inputs):
    """(result with the caller's workspace, result with the library's), flat numpy arrays."""
    import torch

    ws = km.build(e)
    assert ws is not None
    od, _ = oracle.scalarop_info(e.join)
    d_in = [to_device(x) for x in inputs]
    ptrs = [t.data_ptr() for t in d_in]
    d_a = empty_device(e.out_nelem(), NP[od])
    d_b = empty_device(e.out_nelem(), NP[od])
    d_ws = torch.empty(max(ws, 1), dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    # nothing below this line may allocate on the device: torch's counters see torch's own
    # allocations, the driver's free-memory figure sees the library's as well (a hipMalloc,
    # a stream or an event of its own would lower it)
    km(e, stream_handle(), d_a.data_ptr(), ptrs, (d_ws.data_ptr(), ws) if ws else None)
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    free_before = torch.cuda.mem_get_info()[0]
    km.execute_static_workspace(e, stream_handle(), d_b.data_ptr(), ptrs)
    km.execute_static_workspace(e, stream_handle(), d_b.data_ptr(), ptrs)
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
    assert torch.cuda.mem_get_info()[0] == free_before
    return to_host(d_a, NP[od]), to_host(d_b, NP[od]), ws


def test_split_k_contraction_twice_the_second_one_smaller(km):
    r = rng(7)
    # a skinny activation against a weight: cut along k, fp32 partial tiles in the workspace
    for i, j, k in ((8, 4096, 520), (8, 2048, 264), (1, 1024, 256)):
        e = E.from_str("ij,kj->ik", dict(i=i, j=j, k=k), MUL["f16"], "+")
        xs = [uniform(r, i * j, np.float16), uniform(r, k * j, np.float16)]
        a, b, ws = both_ways(km, e, xs)
        assert ws > 0 and "split_k=" in km.describe(e), km.describe(e)
        assert_bits_equal(b, a, "static workspace, split-K %dx%dx%d" % (i, j, k))
        assert_close(b, oracle_einsummable(e, xs), ea.F16, what="split-K vs oracle")


def test_two_pass_reductions_twice_the_second_one_smaller(km):
    r = rng(8)
    cases = [
        E([256, 4000], [[1, 0]], 1, "hole|f32@0", "+"),      # ba->a, slices of b side by side
        E([64, 1000], [[1, 0]], 1, "hole|f32@0", "+"),
        E([3, 131072], [[0, 1]], 1, "hole|f16@0", "+"),      # a few very long rows
        E([1, 262144], [[0, 1]], 1, "hole|f32@0", "^"),
    ]
    for e in cases:
        xs = [normal(r, int(np.prod(e.inn_shape(0))), NP[oracle.scalarop_info(e.join)[0]], 0.5)]
        a, b, ws = both_ways(km, e, xs)
        assert ws > 0 and "splits=" in km.describe(e), km.describe(e)
        assert_bits_equal(b, a, "static workspace, %s" % km.describe(e))
        assert_close(b, oracle_einsummable(e, xs), oracle.scalarop_info(e.join)[0],
                     what="two-pass reduction vs oracle")


def test_staged_transposed_input_and_plain_nodes(km):
    r = rng(9)
    e = E.from_str("ab,ba->ab", dict(a=2048, b=1536), "+[hole|f16@0,hole|f16@1]")
    xs = [normal(r, 2048 * 1536, np.float16), normal(r, 2048 * 1536, np.float16)]
    a, b, ws = both_ways(km, e, xs)
    assert ws > 0 and km.describe(e).startswith("staged ["), km.describe(e)
    assert_bits_equal(b, a, "static workspace, staged elementwise")
    want = (xs[0].reshape(2048, 1536).astype(np.float32) +
            xs[1].reshape(1536, 2048).T.astype(np.float32)).astype(np.float16)
    assert_bits_equal(b, want.reshape(-1), "staged elementwise vs numpy")
    # an einsummable without a workspace runs as with es_km_execute
    e = E([64, 512], [[0, 1]], 2, "exp[hole|f32@0]")
    xs = [normal(r, 64 * 512, np.float32)]
    a, b, ws = both_ways(km, e, xs)
    assert ws == 0
    assert_bits_equal(b, a, "static workspace, no workspace needed")


def test_a_workspace_beyond_the_limit_is_refused(km):
    import torch

    # an 8192 x 8192 f16 input laid out the other way round is transposed into the workspace:
    # 128 MiB
    e = E.from_str("ab,ba->ab", dict(a=8192, b=8192), "+[hole|f16@0,hole|f16@1]")
    ws = km.build(e)
    assert ws == 8192 * 8192 * 2, (ws, km.describe(e))
    d = torch.zeros(8, dtype=torch.float16, device="cuda")
    with pytest.raises(ea.KmError) as ei:
        km.execute_static_workspace(e, stream_handle(), d.data_ptr(), [d.data_ptr(), d.data_ptr()])
    assert ei.value.code == -3 and "67108864" in str(ei.value), str(ei.value)
    # and an einsummable that was never built
    e = E([4, 4], [[0, 1]], 2, "log[hole|f32@0]")
    with pytest.raises(ea.KmError) as ei:
        km.execute_static_workspace(e, stream_handle(), d.data_ptr(), [d.data_ptr()])
    assert ei.value.code == -2
