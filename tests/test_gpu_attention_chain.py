"""Batched attention as a chain of apply nodes (scores, scale, the four softmax pieces, P.V),
the node list bench.py times at full size, here at a size the CPU oracle replays in seconds.
Every node is replayed on the oracle, from the bytes the kernel read, in higher precision
and rounded to fp16, like the kernels: fp16 bound (1e-2 relative, floor = RMS of the result);
the end of the chain is checked against what softmax fixes (rows sum to one)."""
import numpy as np
import pytest

import bench
import einsummable_amd as ea
import oracle
from helpers import assert_close, normal, rng, stream_handle, to_device

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("chain", ["c4_nodes", "c4_fused_nodes"])
@pytest.mark.parametrize("b,h,s,d", [(1, 2, 136, 128), (2, 3, 72, 64)])
def test_attention_chain_matches_oracle(km, b, h, s, d, chain):
    import torch

    r = rng(40)
    host = {k: normal(r, b * h * s * d, np.float16) for k in ("Q", "K", "V")}
    host["S"] = np.zeros(b * h * s * s, np.float16)
    host["O"] = np.zeros(b * h * s * d, np.float16)
    host["m"] = np.zeros(b * h * s, np.float16)
    host["l"] = np.zeros(b * h * s, np.float16)
    dev = {k: to_device(v.copy()) for k, v in host.items()}
    nodes = getattr(bench, chain)(b, h, s, d)
    # bench.c4_nodes carries 1/sqrt(128) as the reference prints it; the chain is linear in
    # it up to the softmax, so the same constant is right for the parity check at any d
    for name, e, out, inns, _w, _u in nodes:
        assert km.build(e) == 0, name
        # the oracle sees the bytes the kernel sees (nodes overwrite their first input)
        seen = [dev[i].cpu().numpy().reshape(-1) for i in inns]
        km(e, stream_handle(), dev[out].data_ptr(), [dev[i].data_ptr() for i in inns])
        host[out] = oracle.einsummable(e.join_shape, e.inns, e.out_rank, e.join, e.castable,
                                       seen, oracle.WIDE)
        torch.cuda.synchronize()
        got = dev[out].cpu().numpy().reshape(-1)
        assert_close(got, host[out], ea.F16, what="attention chain after " + name)
    p = dev["S"].cpu().numpy().astype(np.float64).reshape(-1, s)
    np.testing.assert_allclose(p.sum(axis=1), 1.0, rtol=2e-2)
