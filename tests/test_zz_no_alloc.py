"""fta_bwd_noalloc (the backward entry point that allocates nothing: its scratch is a buffer inside
the library's device image) against fta_bwd with a caller workspace: the same kernels run, so the
results must be bit-identical.  Two calls in a row, the second with a smaller input (the buffer
keeps the first call's contents), through the C ABI with ctypes."""
import math

import pytest
import torch

from oracle import tt_attn_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _both(lib, fta_lib, B, H, L1, L2, D, sm, seed):
    print(f"case noalloc B={B} H={H} L1={L1} L2={L2} D={D} seed={seed}", flush=True)
    q, k, v, b, do = orc.make_inputs(B, H, L1, L2, D, seed=seed, device=DEV)
    t5 = lambda t: fta_lib.t5(t.data_ptr(), t.stride())
    t4 = lambda t: fta_lib.t4(t.data_ptr(), t.stride())
    o = torch.empty_like(q)
    lse = torch.empty(B, H, L1, L2, device=DEV, dtype=torch.float32)
    fta_lib.check(lib.fta_fwd(t5(q), t5(k), t5(v), t4(b), t5(o), lse.data_ptr(), B, H, L1, L2, D, sm, 0))
    nan16 = torch.tensor(float("nan"), dtype=torch.float16, device=DEV)
    outs = []
    for noalloc in (False, True):
        dq, dk, dv, db = (torch.empty_like(t).fill_(nan16) for t in (q, k, v, b))
        if noalloc:
            call = lambda: lib.fta_bwd_noalloc(t5(q), t5(k), t5(v), t4(b), t5(o), lse.data_ptr(), t5(do), t5(dq), t5(dk), t5(dv),
                                               t4(db), B, H, L1, L2, D, sm, 0)
            # a first call may load the code object and look up the buffer's address; after it, a call must
            # leave the device's free memory as it found it -- hipMemGetInfo sees an allocation made anywhere
            # in the process, torch's own counter only those of its caching allocator
            fta_lib.check(call())
            torch.cuda.synchronize()
            before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
            rc = call()
            torch.cuda.synchronize()
            assert torch.cuda.memory_allocated() == before
            assert torch.cuda.mem_get_info()[0] == free_before, "fta_bwd_noalloc changed the device's free memory"
        else:
            n = lib.fta_bwd_workspace_bytes(B, H, L1, L2, D)
            ws = torch.empty(n, dtype=torch.uint8, device=DEV)
            rc = lib.fta_bwd(t5(q), t5(k), t5(v), t4(b), t5(o), lse.data_ptr(), t5(do), t5(dq), t5(dk), t5(dv), t4(db),
                             ws.data_ptr(), n, B, H, L1, L2, D, sm, 0)
        fta_lib.check(rc)
        torch.cuda.synchronize()
        outs.append((dq, dk, dv, db))
    for name, a, c in zip(("dq", "dk", "dv", "db"), *outs):
        assert bool(torch.isfinite(c.float()).all()), name
        assert torch.equal(a, c), f"{name}: fta_bwd_noalloc differs from fta_bwd"
    # and against the oracle, to the usual bar (gradients relative-L2 <= 1e-2)
    ref = orc.oracle_backward(q, k, v, b, sm, do, dtype=torch.float32)
    for name, c in zip(("dq", "dk", "dv", "db"), outs[1]):
        assert orc.rel_l2(c, ref[name]) <= 1e-2, name


def test_noalloc_backward_matches_the_workspace_backward_twice_in_a_row():
    import fta_lib
    lib = fta_lib.load()
    _both(lib, fta_lib, 2, 2, 24, 512, 32, 1.0 / math.sqrt(32), seed=31)   # pipelined kernels, 2 chunks of partials
    _both(lib, fta_lib, 1, 1, 5, 128, 64, 0.3, seed=32)                    # smaller, general kernels, delta pre-pass


def test_noalloc_backward_refuses_sizes_beyond_its_buffer():
    import fta_lib
    lib = fta_lib.load()
    B, H, L1, L2, D = 4, 8, 1024, 1024, 32
    assert lib.fta_bwd_workspace_bytes(B, H, L1, L2, D) > fta_lib.STATIC_WORKSPACE_BYTES
    fake = fta_lib.t5(0x10000, (H * L1 * L2 * D, L1 * L2 * D, L2 * D, D))
    fake4 = fta_lib.t4(0x10000, (H * L2 * L2, L2 * L2, L2))
    rc = lib.fta_bwd_noalloc(fake, fake, fake, fake4, fake, 0x10000, fake, fake, fake, fake, fake4, B, H, L1, L2, D, 0.5, 0)
    assert rc == -10 and "fta_bwd_noalloc" in fta_lib.strerror(rc)
