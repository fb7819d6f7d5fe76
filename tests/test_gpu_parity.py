"""GPU parity tests: the HIP path (through the C ABI, via the drop-in attention()) against the
fp32 oracle on the same seeded inputs, on the configurations the baseline names, plus
size-independent properties (determinism, dBias rows summing to zero, bias-shift invariance,
row independence).  Tolerances are the north-star ones: O max-abs <= 1e-2, gradients
relative-L2 <= 1e-2."""
import math

import pytest
import torch

from oracle import tt_attn_oracle as orc

pytestmark = pytest.mark.gpu

O_MAX_ABS = 1e-2
GRAD_REL_L2 = 1e-2
DEV = "cuda:0"


def _oracle(q, k, v, b, sm, do):
    B, H, L1, L2, D = q.shape
    chunk = max(1, min(L1, (1 << 27) // (L2 * L2 * B * H)))  # <= 512 MiB of fp32 scores at a time
    return orc.oracle_backward(q, k, v, b, sm, do, dtype=torch.float32, l1_chunk=chunk)


def _run(q, k, v, b, sm, do):
    import flash_tt_attn as fta
    qq, kk, vv, bb = (t.detach().requires_grad_(True) for t in (q, k, v, b))
    o = fta.attention(qq, kk, vv, bb, sm)
    dq, dk, dv, db = torch.autograd.grad(o, (qq, kk, vv, bb), do)
    torch.cuda.synchronize()
    return {"o": o, "dq": dq, "dk": dk, "dv": dv, "db": db}


def _compare(got, ref, tag=""):
    err = (got["o"].float() - ref["o"]).abs().max().item()
    assert err <= O_MAX_ABS, f"{tag} O max-abs {err}"
    for n in ("dq", "dk", "dv", "db"):
        r = orc.rel_l2(got[n], ref[n])
        assert r <= GRAD_REL_L2, f"{tag} {n} rel-L2 {r}"


def _case(B, H, L1, L2, D, sm, seed=20, std=1.0, bias_std=1.0):
    print(f"case B={B} H={H} L1={L1} L2={L2} D={D} sm={sm:.4f} seed={seed}", flush=True)
    q, k, v, b, do = orc.make_inputs(B, H, L1, L2, D, seed=seed, std=std, bias_std=bias_std, device=DEV)
    got = _run(q, k, v, b, sm, do)
    _compare(got, _oracle(q, k, v, b, sm, do), f"B{B}H{H}L{L1}x{L2}D{D}")
    return got


def test_upstream_test_op_shape_and_inputs():
    # flash_tt_attn.py:666-712 as it runs from __main__ (:868): B=2,H=4,L=256,D=32, N(0,0.5), sm=0.5
    got = _case(2, 4, 256, 256, 32, 0.5, seed=20, std=0.5, bias_std=0.5)
    # upstream's own bar: atol 1e-2 on O and grads (2e-2 on dBias)
    q, k, v, b, do = orc.make_inputs(2, 4, 256, 256, 32, seed=20, std=0.5, bias_std=0.5, device=DEV)
    ref = _oracle(q, k, v, b, 0.5, do)
    for n, tol in (("o", 1e-2), ("dq", 1e-2), ("dk", 1e-2), ("dv", 1e-2), ("db", 2e-2)):
        assert (got[n].float() - ref[n]).abs().max().item() <= tol, n


@pytest.mark.parametrize("L", [128, 256, 512, 1024])
def test_benchmark_shapes_b4_h8_d32(L):
    # BASELINE configs[1]; sm_scale 1.3 as the upstream benchmark (:783)
    _case(4, 8, L, L, 32, 1.3)


def test_benchmark_shape_softmax_scale_rsqrt_d():
    _case(4, 8, 512, 512, 32, 1.0 / math.sqrt(32))


def test_alphafold_crop_projected_inputs():
    # BASELINE configs[2]: B=1,H=4,D=32,L=384; q/k/v/bias are linear projections of a pair tensor
    # (non-contiguous permuted views are handed to attention() as they are)
    H, D, L, C = 4, 32, 384, 128
    g = torch.Generator(device="cpu").manual_seed(7)
    z = torch.randn(1, L, L, C, generator=g)
    xavier = lambda i, o: (torch.rand(i, o, generator=g) * 2 - 1) * math.sqrt(6.0 / (i + o))
    proj = lambda w: (z @ w).view(1, L, L, H, D).permute(0, 3, 1, 2, 4).to(torch.float16).to(DEV)
    q, k, v = proj(xavier(C, H * D)), proj(xavier(C, H * D)), proj(xavier(C, H * D))
    b = (z @ xavier(C, H)).permute(0, 3, 1, 2).to(torch.float16).to(DEV)
    do = torch.randn(1, H, L, L, D, generator=g).to(torch.float16).to(DEV)
    assert not q.is_contiguous()
    sm = 1.0 / math.sqrt(D)
    got = _run(q, k, v, b, sm, do)
    _compare(got, _oracle(q, k, v, b, sm, do), "af2-crop")


@pytest.mark.parametrize("L1,L2", [(40, 384), (17, 300), (9, 1408)])
def test_head_dim_64_rows_of_an_odd_number_of_128_key_blocks(L1, L2):
    """D=64 rows of an odd number of 128-key blocks.  Tiled as 384 keys: the hand-scheduled dQ/dBias kernel
    takes them as two key ranges of 192 keys (one slab of six tiles per wave), summed into dQ across the two
    launches, the hand-scheduled dK/dV kernel as one range of 384 queries (twelve tiles of the bias in a
    wave's accumulation registers), the hand-scheduled forward as two slabs of 192 keys.  1408 keys: the
    backward tiles them as they are (key ranges 4 x 256 + 2 x 192, query ranges 4 x 256 + 384), the forward,
    which has no shape for eleven blocks, as 1536."""
    _case(2, 2, L1, L2, 64, 0.125, seed=13)
    import fta_lib
    d = fta_lib.describe_plan(2, 2, L1, L2, 64)
    short = L2 <= 384
    assert d["dq"]["kernel"].startswith("fta_bwd_dq1_kernel") and d["dq"]["launches"] == (2 if short else 6)
    assert d["dkdv"]["kernel"].startswith("fta_bwd_dkdv1_kernel") and d["dkdv"]["launches"] == (1 if short else 5)
    assert d["workspace"]["tiled_length"] == (384 if short else 1408)
    assert d["fwd"]["kernel"].startswith("fta_fwd2_kernel<64,6," if short else "fta_fwd_kernel")
    assert d["fwd"]["tiled_length"] == (384 if short else 1536)


@pytest.mark.parametrize("L", [1024, 1536])
def test_long_crop_peaked_softmax(L):
    # BASELINE configs[3]: bias scaled by 3
    _case(1, 4, L, L, 32, 1.0 / math.sqrt(32), bias_std=3.0)


def test_ending_node_by_manual_permute_d64():
    # BASELINE configs[4]: B=2,H=8,D=64,L=512, inputs transposed L1<->L2 (non-contiguous views)
    B, H, L, D = 2, 8, 512, 64
    sm = 1.0 / math.sqrt(D)
    q, k, v, b, do = orc.make_inputs(B, H, L, L, D, seed=5, device=DEV)
    qt, kt, vt, dot = (t.transpose(2, 3) for t in (q, k, v, do))
    assert not qt.is_contiguous()
    got = _run(qt, kt, vt, b, sm, dot)
    ref = _oracle(qt, kt, vt, b, sm, dot)
    _compare(got, ref, "ending-node")
    # transposed back, the result is the incoming-edge attention of the untransposed tensors
    assert got["o"].transpose(2, 3).shape == q.shape


def _masked_bias(b, L2, where, value):
    """Key mask written into the bias: `where` = 'trailing' masks the last 37 keys of every query,
    'leading' the first 70 (more than the 64 keys the forward looks at first), 'ragged' a different
    number of trailing keys per (b, h) plus single keys in the middle.  No query loses all its keys."""
    b = b.clone()
    mv = {"-inf": float("-inf"), "-1e9": -1e9, "-60000": -60000.0}[value]
    mv = torch.tensor(mv, dtype=torch.float32).to(torch.float16).item()  # -1e9 becomes -inf in fp16
    if where == "trailing":
        b[..., L2 - 37:] = mv
    elif where == "leading":
        b[..., :70] = mv
    else:
        for i in range(b.shape[0] * b.shape[1]):
            b.view(-1, L2, L2)[i, :, L2 - 1 - 19 * i:] = mv
        b[..., ::2, 5] = mv
        b[..., 1::3, L2 // 2 + 3] = mv
    return b


@pytest.mark.parametrize("value", ["-inf", "-1e9", "-60000"])
@pytest.mark.parametrize("where", ["trailing", "leading", "ragged"])
@pytest.mark.parametrize("D,L2", [(32, 256), (32, 384), (32, 512), (64, 256), (64, 384), (64, 512)])
def test_key_mask_written_into_the_bias(D, L2, where, value):
    """A key-padding mask in the bias (-inf, -1e9 cast to fp16, -60000) on part of every row: the
    masked keys get weight 0 and zero gradients, as upstream (flash_tt_attn.py:78, :344-346,
    :418-420); everything stays finite and within the usual tolerances.  L2 = 256/512 run the
    pipelined backward kernels, 384 the general ones."""
    B, H, L1, sm = 1, 2, 9, 1.0 / math.sqrt(D)
    print(f"case mask D={D} L2={L2} {where} {value}", flush=True)
    q, k, v, b, do = orc.make_inputs(B, H, L1, L2, D, seed=13, device=DEV)
    b = _masked_bias(b, L2, where, value)
    got = _run(q, k, v, b, sm, do)
    assert all(torch.isfinite(got[n].float()).all() for n in got)
    _compare(got, _oracle(q, k, v, b, sm, do), f"mask D{D} L{L2} {where} {value}")
    masked = b.float() < -40000
    assert bool((got["db"].float()[masked] == 0).all()), "a masked key received a bias gradient"


@pytest.mark.parametrize("D,L2", [(32, 512), (64, 256)])
def test_key_mask_general_backward_kernels(general_kernels, D, L2):
    B, H, L1, sm = 1, 2, 9, 1.0 / math.sqrt(D)
    print(f"case mask-general D={D} L2={L2}", flush=True)
    q, k, v, b, do = orc.make_inputs(B, H, L1, L2, D, seed=14, device=DEV)
    for where in ("trailing", "leading"):
        bm = _masked_bias(b, L2, where, "-inf")
        got = _run(q, k, v, bm, sm, do)
        assert all(torch.isfinite(got[n].float()).all() for n in got)
        _compare(got, _oracle(q, k, v, bm, sm, do), f"mask-general D{D} L{L2} {where}")


def test_cpu_plumbing_config_on_the_gpu_in_fp16():
    # BASELINE configs[0] (B1 H4 L64 D32, seed 20, sm 1/sqrt(D)) is an fp32 CPU configuration by
    # definition; its fp16 cast also runs on the HIP path (L2 = 64 is below the kernels' 128-key tile)
    _case(1, 4, 64, 64, 32, 1.0 / math.sqrt(32), seed=20)


def test_rectangular_l1_and_edge_sizes():
    _case(1, 1, 1, 128, 32, 0.7)      # a single row: plain biased attention
    _case(1, 3, 5, 256, 64, 0.3)      # L1 not a multiple of anything
    _case(2, 1, 33, 384, 32, 0.9)
    _case(1, 1, 9, 768, 32, 0.2)


@pytest.fixture
def general_kernels():
    """Selects the general backward kernels where the pipelined ones would run (library test hook)."""
    import fta_lib
    lib = fta_lib.load()
    old = lib.fta_debug_select_kernels(3)
    yield lib
    lib.fta_debug_select_kernels(old)


def test_general_backward_kernels(general_kernels):
    # The pipelined one-wave-per-SIMD backward kernels cover every tiled length from 256 on at D=32; the
    # general kernels otherwise only run for shorter rows, D=64 dK/dV and the feature paths.
    import fta_lib
    assert "dq1" not in fta_lib.describe_plan(1, 2, 24, 512, 32)["dq"]["kernel"]
    assert "dkdv1" not in fta_lib.describe_plan(1, 2, 24, 512, 32)["dkdv"]["kernel"]
    _case(1, 2, 24, 512, 32, 0.4, seed=5)
    _case(1, 1, 16, 256, 64, 0.25, seed=6)
    _case(1, 2, 10, 300, 32, 0.3, seed=9)   # their tail-masking instances (the pipelined kernels have their own)


def test_zero_softmax_scale():
    # sm_scale = 0: the scores are the bias alone; nothing in the kernels divides by the scale
    _case(1, 2, 16, 512, 32, 0.0, seed=7)
    _case(1, 1, 8, 384, 32, 0.0, seed=8)


def test_only_some_inputs_require_grad_and_example_flow():
    import flash_tt_attn as fta
    q, k, v, b, do = orc.make_inputs(1, 2, 4, 128, 32, seed=3, device=DEV)
    q.requires_grad_(True); b.requires_grad_(True)
    out = fta.attention(q, k, v, b, 1.0 / math.sqrt(32))
    torch.nn.functional.mse_loss(out, torch.randn_like(out)).backward()
    assert q.grad is not None and b.grad is not None and k.grad is None and v.grad is None
    assert q.grad.dtype == torch.float16 and b.grad.shape == b.shape


def test_results_are_deterministic_bitwise():
    q, k, v, b, do = orc.make_inputs(2, 2, 128, 512, 32, seed=11, device=DEV)
    a = _run(q, k, v, b, 1.3, do)
    c = _run(q, k, v, b, 1.3, do)
    for n in a:
        assert torch.equal(a[n], c[n]), n


def test_properties_at_full_benchmark_size():
    # B=4,H=8,L=512,D=32: properties that need no oracle
    B, H, L, D, sm = 4, 8, 512, 32, 1.0 / math.sqrt(32)
    q, k, v, b, do = orc.make_inputs(B, H, L, L, D, seed=20, device=DEV)
    # bias on a 1/64 grid within [-4, 4] so that adding small integers stays exact in fp16
    b = (torch.round(b.float().clamp(-4, 4) * 64) / 64).to(torch.float16)
    a = _run(q, k, v, b, sm, do)
    # sum_k dS = 0  =>  every dBias row sums to (nearly) zero; compare with the row's own scale
    db = a["db"].float()
    assert (db.sum(-1).abs() / db.abs().sum(-1).clamp_min(1e-6)).max().item() < 5e-3
    # adding a constant to a query row of the bias changes nothing
    shift = torch.randint(-2, 3, (B, H, L, 1), device=DEV).float()
    b2 = (b.float() + shift).to(torch.float16)
    assert torch.equal(b2.float() - shift, b.float())
    c = _run(q, k, v, b2, sm, do)
    assert (a["o"].float() - c["o"].float()).abs().max().item() <= 2e-3
    for n in ("dq", "dk", "dv", "db"):
        assert orc.rel_l2(c[n], a[n].float()) <= 2e-3, n
    # L1 rows are independent in O/dQ/dK/dV: perturbing row 7 leaves row 3 bit-identical
    q2 = q.clone(); q2[:, :, 7] += 1
    d = _run(q2, k, v, b, sm, do)
    for n in ("o", "dq", "dk", "dv"):
        assert torch.equal(a[n][:, :, 3], d[n][:, :, 3]), n
    assert not torch.equal(a["db"], d["db"])
    # lse is consistent with the scores: exp2(S*log2e - lse) sums to one (checked on one slice)
    import fta_lib, flash_tt_attn as fta
    lse = torch.empty(B, H, L, L, device=DEV, dtype=torch.float32)
    o = torch.empty_like(q)
    fta_lib.check(fta_lib.load().fta_fwd(fta._t5(q), fta._t5(k), fta._t5(v), fta._t4(b), fta._t5(o), lse.data_ptr(),
                                         B, H, L, L, D, sm, torch.cuda.current_stream().cuda_stream))
    s = (q[1, 2, 5].float() @ k[1, 2, 5].float().T) * sm + b[1, 2].float()
    assert (torch.exp2(s * orc.LOG2E - lse[1, 2, 5][:, None]).sum(-1) - 1).abs().max().item() < 1e-3
    assert torch.equal(o, a["o"])


def test_sequence_length_sweep_harness():
    """The sweep harness (upstream bench_attention, flash_tt_attn.py:762): both providers, both modes,
    both metrics give finite numbers at a small point; the library is not slower than the naive
    formulation there; an unknown provider raises like upstream (:828)."""
    import bench_attention as ba
    for mode in ("fwd", "bwd"):
        t_hip = ba.bench_attention(1, 2, 128, 32, mode, "hip", metric="time")
        t_ref = ba.bench_attention(1, 2, 128, 32, mode, "vanilla-torch", metric="time")
        m_hip = ba.bench_attention(1, 2, 128, 32, mode, "triton-fp16", metric="memory")
        m_ref = ba.bench_attention(1, 2, 128, 32, mode, "vanilla-torch", metric="memory")
        print(f"{mode}: hip {t_hip:.3f} ms {m_hip:.4f} GB, naive {t_ref:.3f} ms {m_ref:.4f} GB", flush=True)
        assert all(math.isfinite(x) and x > 0 for x in (t_hip, t_ref, m_hip, m_ref))
        assert m_hip < m_ref  # O(L^2 D) against O(L^3)
    with pytest.raises(ValueError):
        ba.bench_attention(1, 2, 128, 32, "fwd", "sdpa", metric="time")


def test_sweep_writes_the_files_of_upstreams_test_results(tmp_path):
    """sweep(out=...) leaves what upstream's perf_report leaves in test_results/: per (mode, metric) a CSV
    "L,<line names>" and a PNG of the same name, and a results.html that shows the four images."""
    import bench_attention as ba
    tables = ba.sweep(1, 2, 32, Ls=(128, 256), vanilla_max_L=128, out=str(tmp_path))
    assert set(tables) == {("fwd", "memory"), ("fwd", "time"), ("bwd", "memory"), ("bwd", "time")}
    stems = [f"fused-attention-batch1-head2-d32-{m}-{k}" for m in ("fwd", "bwd") for k in ("latency", "memory")]
    for stem in stems:
        lines = (tmp_path / (stem + ".csv")).read_text().splitlines()
        assert lines[0] == "L,HIP [FP16],Vanilla PyTorch" and len(lines) == 3
        assert lines[1].startswith("128.000000,") and lines[2].endswith(",nan")   # naive provider not run past 128
        png = (tmp_path / (stem + ".png")).read_bytes()
        assert png[:8] == b"\x89PNG\r\n\x1a\n" and len(png) > 2000
    html = (tmp_path / "results.html").read_text()
    assert html.count("<image src=") == 4 and all(stem + ".png" in html for stem in stems)


@pytest.mark.parametrize("B,H,L1,L2,D", [(1, 2, 100, 100, 32), (1, 1, 7, 200, 64), (2, 2, 320, 320, 32), (1, 2, 48, 48, 32),
                                         (1, 1, 3, 1408, 32), (1, 1, 3, 1300, 32), (1, 1, 2, 3200, 32), (1, 1, 2, 900, 64),
                                         (1, 2, 5, 4, 32), (1, 2, 9, 333, 32), (1, 1, 4, 131, 64),
                                         (1, 1, 5, 2, 64), (2, 2, 11, 511, 32), (1, 2, 6, 257, 32), (1, 1, 3, 1026, 32),
                                         (1, 2, 5, 510, 64), (1, 1, 2, 4095, 32), (1, 1, 2, 2047, 64)])
def test_lengths_that_are_not_multiples_of_128(B, H, L1, L2, D):
    """Upstream needs power-of-two lengths (flash_tt_attn.py:618) and has no masking; here the kernels
    tile a row in 128-key blocks and mask the tail of the last block themselves (1408 and 3200 are
    tiled as 1536 and 3584: no workgroup shape fits 11 or 25 blocks).  Any length goes: where it is not
    a multiple of 4 (333, 131, 511, 1 ...) the rows of the bias and of dBias start on 2-byte boundaries and
    are read and written entry by entry where a vector access would straddle.  Same oracle, same
    tolerances; the masked keys must not leak into any output."""
    got = _case(B, H, L1, L2, D, 1.0 / math.sqrt(D), seed=7)
    assert got["o"].shape == (B, H, L1, L2, D) and got["db"].shape == (B, H, L2, L2)
    assert all(torch.isfinite(got[n].float()).all() for n in got)


def test_rows_of_a_single_key():
    """L2 = 1: the softmax of one score is 1, so O = V and dV = dO whatever Q, K and the bias are, and
    dQ, dK, dBias vanish (compared absolutely: a relative error against zero says nothing)."""
    q, k, v, b, do = orc.make_inputs(1, 2, 6, 1, 32, seed=7, device=DEV)
    got = _run(q, k, v, b, 0.3, do)
    assert (got["o"].float() - v.float()).abs().max().item() <= 2e-3
    assert (got["dv"].float() - do.float()).abs().max().item() <= 2e-3
    for n in ("dq", "dk", "db"):
        assert got[n].float().abs().max().item() <= 2e-3, n


@pytest.mark.parametrize("L2", [200, 203])
def test_no_padded_copies_for_lengths_that_are_not_multiples_of_128(L2):
    """L2 = 200 (or 203) is tiled as 256 inside the kernels: peak memory of forward + backward stays within 5 %
    of what the same call needs at a length that is a multiple of 128, scaled by the tensor sizes
    (no padded copies of q, k, v, dO or of the outputs)."""
    import flash_tt_attn as fta
    B, H, L1, D, sm = 2, 4, 200, 32, 0.2

    def peak(L2):
        q, k, v, b, do = orc.make_inputs(B, H, L1, L2, D, seed=3, device=DEV)
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        base = torch.cuda.memory_allocated()
        _run(q, k, v, b, sm, do)
        return torch.cuda.max_memory_allocated() - base, q.numel() * 2

    p200, n200 = peak(L2)
    # what attention() must hold at this L2: o + lse, four gradients, the workspace (laid out for 256 keys)
    import fta_lib
    ws = fta_lib.load().fta_bwd_workspace_bytes(B, H, L1, L2, D)
    need = 4 * n200 + B * H * L1 * L2 * 4 + B * H * L2 * L2 * 2 + ws
    print(f"peak {p200} need {need}", flush=True)
    assert p200 <= 1.05 * need


@pytest.mark.parametrize("D,L1,L2", [(32, 9, 512), (32, 5, 256), (32, 4, 384), (32, 3, 128), (32, 3, 1024), (64, 6, 512), (64, 5, 256),
                                     (64, 3, 768)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_bias_rows_off_the_8_byte_boundary_at_whole_tile_lengths(D, L1, L2, dtype):
    """The bias as a window of a larger tensor whose rows start on odd 2-byte boundaries (row stride L2 + 3,
    first column 1), at lengths that need no tail masking: every kernel family then takes the instances that
    read the bias entry by entry (the others load it in aligned 8-byte pieces), and dBias is written through
    the same window."""
    import flash_tt_attn as fta
    B, H, sm = 1, 2, 1.0 / math.sqrt(D)
    q, k, v, b, do = orc.make_inputs(B, H, L1, L2, D, seed=23, dtype=dtype, device=DEV)
    big = torch.zeros(B, H, L2 + 2, L2 + 3, dtype=dtype, device=DEV)
    big[:, :, 1:L2 + 1, 1:L2 + 1] = b
    bw = big[:, :, 1:L2 + 1, 1:L2 + 1]
    assert bw.stride(2) % 4 != 0   # (consecutive rows start on different offsets within 8 bytes)
    plain, window = _run(q, k, v, b, sm, do), _run(q, k, v, bw, sm, do)
    for n in ("o", "dq", "dk", "dv", "db"):
        assert torch.equal(plain[n], window[n]), n   # same arithmetic on the same values, whatever the loads
    ref = _oracle(q, k, v, b, sm, do)
    if dtype == torch.float16:
        _compare(window, ref, f"odd bias rows D{D} L{L2}")


@pytest.mark.parametrize("D,L2", [(32, L) for L in range(128, 4097, 128)] + [(64, L) for L in range(128, 2049, 128)])
def test_every_length_the_library_reports_as_supported(D, L2):
    """Each multiple of 128 up to the longest row built (4096 at D=32, the end of upstream's sweep,
    flash_tt_attn.py:724; 2048 at D=64) either has a workgroup shape of its own or is tiled as the
    next length that has; both ways the result must match the oracle -- a plan that is valid must
    also be launchable."""
    _case(1, 1, 2, L2, D, 1.0 / math.sqrt(D), seed=11)


def test_random_shapes_scales_and_layouts():
    """A seeded draw of shapes (L1 from 1 to 64 or square, L2 over the supported lengths, both head
    dims), softmax scales, bias spreads and layouts (contiguous or L1<->L2 transposed views), each run
    twice: oracle tolerances and bitwise run-to-run equality."""
    import random
    rng = random.Random(5)
    for c in range(14):
        D = rng.choice([32, 32, 64])
        L2 = rng.choice([128, 256, 384, 512, 640, 1024] if D == 32 else [128, 256, 512, 768])
        L1 = rng.choice([1, 3, 8, 17, 33, 64])
        B, H = rng.choice([(1, 1), (1, 2), (2, 1), (1, 3)])
        sm = rng.choice([1.0 / math.sqrt(D), 0.5, 1.3, 0.05])
        bias_std = rng.choice([0.5, 1.0, 2.0])
        transposed = rng.random() < 0.3 and L2 <= 256
        if transposed:
            L1 = L2
        seed = rng.randrange(1 << 30)
        print(f"case {c}: transposed={transposed} B={B} H={H} L1={L1} L2={L2} D={D} sm={sm:.3f} bias_std={bias_std} seed={seed}", flush=True)
        q, k, v, b, do = orc.make_inputs(B, H, L1, L2, D, seed=seed, std=1.0, bias_std=bias_std, device=DEV)
        if transposed:
            q, k, v, do = (t.transpose(2, 3).contiguous().transpose(2, 3) for t in (q, k, v, do))
        ref = _oracle(q, k, v, b, sm, do)
        first = _run(q, k, v, b, sm, do)
        _compare(first, ref, f"case {c}")
        again = _run(q, k, v, b, sm, do)
        for n in first:
            assert torch.equal(first[n], again[n]), f"case {c}: {n} differs between two runs"


@pytest.mark.parametrize("D,L2,L1", [(32, 128, 3), (32, 256, 9), (32, 384, 5), (32, 512, 17), (32, 640, 2), (32, 1024, 3),
                                     (32, 1536, 2), (32, 2048, 1), (64, 128, 5), (64, 256, 3), (64, 512, 9), (64, 768, 2),
                                     (32, 200, 5), (32, 1300, 2), (32, 4, 3), (32, 2560, 1), (32, 4096, 1), (64, 100, 3),
                                     (64, 1024, 2), (64, 900, 2), (32, 896, 2), (32, 800, 3), (32, 1152, 2), (32, 1280, 1),
                                     (32, 1664, 1), (32, 1792, 1), (32, 1920, 1), (64, 384, 4), (64, 300, 3), (64, 1280, 1), (64, 1900, 1), (64, 2048, 1),
                                     (32, 203, 4), (32, 1301, 2), (64, 131, 3), (32, 3, 2), (32, 511, 3), (64, 513, 2)])
def test_kernels_write_nothing_outside_their_outputs(D, L2, L1):
    """Every output and the workspace sit inside one buffer, each between guard bands of a known
    pattern; after a forward and a backward through the C ABI the guards must be untouched and every
    output element overwritten (the library promises full overwrites without pre-zeroing)."""
    import fta_lib
    lib = fta_lib.load()
    B, H, sm = 1, 2, 1.0 / math.sqrt(D)
    print(f"case guards D={D} L2={L2} L1={L1}", flush=True)
    q, k, v, b, do = orc.make_inputs(B, H, L1, L2, D, seed=3, device=DEV)
    GUARD = 1 << 16  # bytes between neighbours
    n5, n4 = B * H * L1 * L2 * D * 2, B * H * L2 * L2 * 2
    nws = lib.fta_bwd_workspace_bytes(B, H, L1, L2, D)
    sizes = {"o": n5, "lse": B * H * L1 * L2 * 4, "dq": n5, "dk": n5, "dv": n5, "db": n4, "ws": nws}
    total = GUARD + sum((s + GUARD + 255) // 256 * 256 for s in sizes.values())
    buf = torch.full((total,), 0xA5, dtype=torch.uint8, device=DEV)
    off, view = GUARD, {}
    for name, s in sizes.items():
        view[name] = buf[off:off + s]
        off += (s + GUARD + 255) // 256 * 256
    sentinel = torch.tensor(float("nan"), dtype=torch.float16, device=DEV)
    as5 = lambda name: view[name].view(torch.float16).view(B, H, L1, L2, D)
    o, dq, dk, dv = as5("o"), as5("dq"), as5("dk"), as5("dv")
    db = view["db"].view(torch.float16).view(B, H, L2, L2)
    lse = view["lse"].view(torch.float32)
    for t in (o, dq, dk, dv, db):
        t.fill_(sentinel)
    lse.fill_(float("nan"))
    t5 = lambda t: fta_lib.t5(t.data_ptr(), t.stride())
    t4 = lambda t: fta_lib.t4(t.data_ptr(), t.stride())
    fta_lib.check(lib.fta_fwd(t5(q), t5(k), t5(v), t4(b), t5(o), lse.data_ptr(), B, H, L1, L2, D, sm, 0))
    fta_lib.check(lib.fta_bwd(t5(q), t5(k), t5(v), t4(b), t5(o), lse.data_ptr(), t5(do), t5(dq), t5(dk), t5(dv), t4(db),
                              view["ws"].data_ptr(), nws, B, H, L1, L2, D, sm, 0))
    torch.cuda.synchronize()
    inside = torch.zeros(total, dtype=torch.bool, device=DEV)
    for name in sizes:
        start = view[name].data_ptr() - buf.data_ptr()
        inside[start:start + sizes[name]] = True
    assert bool((buf[~inside] == 0xA5).all()), "a kernel wrote outside its outputs"
    for name, t in (("o", o), ("dq", dq), ("dk", dk), ("dv", dv), ("db", db), ("lse", lse)):
        assert bool(torch.isfinite(t.float()).all()), f"{name} was not fully overwritten"
    ref = _oracle(q, k, v, b, sm, do)
    _compare({"o": o, "dq": dq, "dk": dk, "dv": dv, "db": db}, ref, f"guards D{D} L{L2}")


@pytest.mark.parametrize("args", [(), ("5", "256", "64"), ("2", "512", "32")])
def test_c_abi_from_plain_cpp_without_torch(args):
    """fta_c_demo (built with the library) drives fta_fwd / fta_bwd with hipMalloc'ed buffers only and
    checks every output against its own double-precision loops."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "flash-triangle-attention_amd", "fta_c_demo")
    assert os.path.exists(exe), "build the library first (flash-triangle-attention_amd/build.py)"
    r = subprocess.run([exe, *args], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0 and "PASS" in r.stdout


def test_tensors_beyond_4_gib_are_addressed_with_64_bit_offsets():
    """B4 H8 L1=4200 L2=512 D32: every pair tensor holds 2.2e9 elements = 4.4 GB, so element and byte offsets
    pass 2^31 and 2^32.  Rows (b, h, i) are independent for O, dQ, dK and dV: the first, the last and a few
    in between are compared with the oracle run on that row alone; dBias is checked on one query's row
    against the sum over all 4200 L1 rows formed directly."""
    import flash_tt_attn as fta
    B, H, L1, L2, D = 4, 8, 4200, 512, 32
    sm = 1.0 / math.sqrt(D)
    g = torch.Generator(device=DEV).manual_seed(7)

    def mk(*shape):
        return torch.empty(*shape, dtype=torch.float16, device=DEV).normal_(generator=g)

    q, k, v, do = (mk(B, H, L1, L2, D) for _ in range(4))
    b = mk(B, H, L2, L2)
    assert q.numel() * 2 > 2 ** 32
    qq, kk, vv, bb = (t.requires_grad_(True) for t in (q, k, v, b))
    o = fta.attention(qq, kk, vv, bb, sm)
    dq, dk, dv, db = torch.autograd.grad(o, (qq, kk, vv, bb), do)
    torch.cuda.synchronize()
    q, k, v, b = (t.detach() for t in (q, k, v, b))
    for bi, hi, i in [(0, 0, 0), (B - 1, H - 1, L1 - 1), (B - 1, 0, L1 // 2), (2, H - 1, 4099), (1, 3, 2049), (3, 7, 4100)]:
        row = lambda t: t[bi:bi + 1, hi:hi + 1, i:i + 1]
        ref = orc.oracle_backward(row(q), row(k), row(v), b[bi:bi + 1, hi:hi + 1], sm, row(do), dtype=torch.float32, l1_chunk=1)
        got = {"o": row(o), "dq": row(dq), "dk": row(dk), "dv": row(dv)}
        err = (got["o"].float() - ref["o"]).abs().max().item()
        assert err <= 1e-2, f"row {(bi, hi, i)}: O max-abs {err}"
        for n in ("dq", "dk", "dv"):
            e = orc.rel_l2(got[n], ref[n])
            assert e <= 1e-2, f"row {(bi, hi, i)}: {n} rel-L2 {e}"
    bi, hi, j = B - 1, H - 1, L2 - 5
    s = sm * torch.einsum("id,ikd->ik", q[bi, hi, :, j].float(), k[bi, hi].float()) + b[bi, hi, j].float()[None]
    p = torch.softmax(s, -1)
    dp = torch.einsum("id,ikd->ik", do[bi, hi, :, j].float(), v[bi, hi].float())
    ref_db = (p * (dp - (p * dp).sum(-1, keepdim=True))).sum(0)
    e = orc.rel_l2(db[bi, hi, j], ref_db)
    assert e <= 1e-2, f"dBias[{bi},{hi},{j}] rel-L2 {e}"
    assert torch.isfinite(db.float()).all()


def test_gradient_error_does_not_grow_with_the_number_of_key_ranges():
    """Rows longer than one workgroup's stage are worked off in several launches per gradient, each
    adding its key (or query) range's share to the 16-bit gradient the launch before it stored.  The
    re-rounding must not pile up: on the same input distribution the relative-L2 error of every
    gradient at L2 = 2048 and 4096 (L1 = 64, D = 32) stays within 1.5x of the one-launch length 512."""
    sm, errs = 1.0 / math.sqrt(32), {}
    for L2 in (512, 2048, 4096):
        print(f"case key ranges L1=64 L2={L2}", flush=True)
        q, k, v, b, do = orc.make_inputs(1, 1, 64, L2, 32, seed=77, device=DEV)
        got, ref = _run(q, k, v, b, sm, do), _oracle(q, k, v, b, sm, do)
        _compare(got, ref, f"key ranges L2={L2}")
        errs[L2] = {n: orc.rel_l2(got[n], ref[n]) for n in ("dq", "dk", "dv", "db")}
        print(L2, {n: f"{e:.2e}" for n, e in errs[L2].items()}, flush=True)
        del got, ref
        torch.cuda.empty_cache()
    for L2 in (2048, 4096):
        for n, e in errs[L2].items():
            assert e <= 1.5 * errs[512][n], f"{n}: rel-L2 {e:.2e} at L2={L2} against {errs[512][n]:.2e} at L2=512"


@pytest.mark.parametrize("L2,masked", [(512, (256, 512)), (512, (0, 256)), (512, (0, 40)), (500, (250, 300)), (256, (0, 33)),
                                       (200, (150, 200)), (512, None), (256, None)])
def test_head_dim_64_forward_of_one_and_two_slabs_with_masked_key_ranges(L2, masked):
    """D=64 rows of up to 512 keys run the hand-scheduled forward: one slab of 256 keys per wave, or two
    whose partial results are merged once per row.  Key masks that blank a whole slab, a row's first tile
    (which fixes the softmax reference) or a range across the slab boundary must leave the merge exact:
    a masked slab contributes weight 0, not NaN."""
    import fta_lib
    assert fta_lib.describe_plan(2, 3, 21, L2, 64)["fwd"]["kernel"].startswith("fta_fwd2_kernel")
    print(f"case D=64 L2={L2} masked={masked}", flush=True)
    q, k, v, b, do = orc.make_inputs(2, 3, 21, L2, 64, seed=41, device=DEV)
    if masked is not None:
        b = b.clone()
        b[..., masked[0]:masked[1]] = float("-inf")
    for sm in (0.125, 1.3):
        got = _run(q, k, v, b, sm, do)
        assert all(bool(torch.isfinite(got[n].float()).all()) for n in got)
        _compare(got, _oracle(q, k, v, b, sm, do), f"D64 L{L2} mask {masked} sm {sm}")
