"""Host-side checks that need no GPU: the library loads, exports every symbol the header declares,
rejects bad arguments before any GPU call, and the Python module mirrors the upstream surface."""
import ctypes
import os
import re

import pytest
import torch

import fta_lib
from fta_lib import Tensor4, Tensor5

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "fta.h")


def _declared_functions():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    return sorted(set(re.findall(r"\b(fta_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = fta_lib.load()
    names = _declared_functions()
    assert {"fta_fwd", "fta_bwd", "fta_bwd_workspace_bytes", "fta_strerror", "fta_version",
            "fta_check_fwd", "fta_check_bwd", "fta_bwd_profile"} <= set(names)
    for n in names:
        assert hasattr(lib, n), n
    assert set(names) == set(fta_lib.SIGNATURES), "ctypes binding and header disagree"
    assert lib.fta_version() == int(re.search(r"#define FTA_VERSION (\d+)", open(HEADER).read()).group(1))


FAKE = 0x10000  # non-null, 16-byte aligned, never dereferenced by the check functions


def _t5(B, H, L1, L2, D, ptr=FAKE, strides=None):
    s = strides or (H * L1 * L2 * D, L1 * L2 * D, L2 * D, D)
    return fta_lib.t5(ptr, s)


def _t4(B, H, L2, ptr=FAKE, strides=None):
    s = strides or (H * L2 * L2, L2 * L2, L2)
    return fta_lib.t4(ptr, s)


def _check_fwd(B=1, H=2, L1=4, L2=128, D=32, sm=0.5, **kw):
    lib = fta_lib.load()
    a = dict(q=_t5(B, H, L1, L2, D), k=_t5(B, H, L1, L2, D), v=_t5(B, H, L1, L2, D), bias=_t4(B, H, L2),
             o=_t5(B, H, L1, L2, D), lse=FAKE)
    a.update(kw)
    return lib.fta_check_fwd(a["q"], a["k"], a["v"], a["bias"], a["o"], a["lse"], B, H, L1, L2, D, sm)


def test_check_fwd_accepts_valid_and_names_each_error():
    assert _check_fwd() == 0
    assert _check_fwd(L1=7) == 0                      # L1 need not equal L2
    assert _check_fwd(D=16) == -3 and _check_fwd(D=128) == -3
    assert _check_fwd(L2=100) == 0 and _check_fwd(L2=64) == 0 and _check_fwd(L2=4096) == 0
    assert _check_fwd(L2=102) == 0 and _check_fwd(L2=2) == 0 and _check_fwd(L2=1) == 0 and _check_fwd(L2=4095) == 0   # any length
    assert _check_fwd(L2=0) == -4 and _check_fwd(L2=4097) == -4
    assert _check_fwd(L2=2048, D=64) == 0 and _check_fwd(L2=2047, D=64) == 0 and _check_fwd(L2=2049, D=64) == -4
    assert _check_fwd(L1=0) == -4
    assert _check_fwd(B=0) == -5
    assert _check_fwd(sm=float("inf")) == -8 and _check_fwd(sm=float("nan")) == -8
    assert _check_fwd(q=_t5(1, 2, 4, 128, 32, ptr=0)) == -1
    assert _check_fwd(lse=0) == -1
    assert _check_fwd(k=_t5(1, 2, 4, 128, 32, ptr=FAKE + 2)) == -2
    assert _check_fwd(v=_t5(1, 2, 4, 128, 32, strides=(32772, 16384, 4096, 33))) == -6
    # bias rows may start anywhere (a length that is not a multiple of 4 puts them on 2-byte boundaries)
    assert _check_fwd(bias=_t4(1, 2, 128, strides=(32768, 16384, 130))) == 0
    assert _check_fwd(bias=_t4(1, 2, 128, ptr=FAKE + 2, strides=(33282, 16641, 129))) == 0
    assert _check_fwd(bias=_t4(1, 2, 128, ptr=FAKE + 1)) == -2 and _check_fwd(bias=_t4(1, 2, 128, strides=(32768, 16384, -128))) == -6
    # an output whose rows overlap is refused; a transposed (L1<->L2) output is fine
    assert _check_fwd(o=_t5(1, 2, 4, 128, 32, strides=(32768, 16384, 4096, 16))) == -6
    assert _check_fwd(o=_t5(1, 2, 4, 128, 32, strides=(32768, 16384, 32, 128))) == 0
    # rows of a slice more than 4 GiB apart do not fit the kernels' 32-bit row offsets
    far = 2**31 // 128
    assert _check_fwd(k=_t5(1, 2, 4, 128, 32, strides=(far * 1024, far * 512, far * 128, far))) == -6
    assert _check_fwd(k=_t5(1, 2, 4, 128, 32, strides=(far * 1024, far * 512, far * 128, far - 8))) == 0
    for code in range(-9, 1):
        assert fta_lib.strerror(code)


def test_workspace_and_check_bwd():
    lib = fta_lib.load()
    B, H, L1, L2, D = 2, 2, 16, 256, 32
    n = lib.fta_bwd_workspace_bytes(B, H, L1, L2, D)
    assert n >= B * H * L1 * L2 * 4 + B * H * L2 * L2 * 4
    assert lib.fta_bwd_workspace_bytes(B, H, L1, 200, D) >= n      # 200 keys are tiled as 256 (general kernels: plus delta)
    assert lib.fta_bwd_workspace_bytes(B, H, L1, 202, D) == lib.fta_bwd_workspace_bytes(B, H, L1, 200, D)   # any length
    assert lib.fta_bwd_workspace_bytes(B, H, L1, 0, D) == 0 and lib.fta_bwd_workspace_bytes(B, H, L1, fta_lib.MAX_L2 + 1, D) == 0
    assert lib.fta_bwd_workspace_bytes(B, H, L1, L2, 48) == 0
    t5 = lambda: _t5(B, H, L1, L2, D)
    t4 = lambda: _t4(B, H, L2)
    args = lambda ws=FAKE, nb=n, dq=None, db=None: (t5(), t5(), t5(), t4(), t5(), FAKE, t5(), dq or t5(), t5(), t5(),
                                                    db or t4(), ws, nb, B, H, L1, L2, D, 0.5)
    assert lib.fta_check_bwd(*args()) == 0
    assert lib.fta_check_bwd(*args(nb=n - 1)) == -7
    assert lib.fta_check_bwd(*args(ws=0)) == -1
    assert lib.fta_check_bwd(*args(ws=FAKE + 4)) == -2
    assert lib.fta_check_bwd(*args(dq=_t5(B, H, L1, L2, D, strides=(0, 0, 0, 32)))) == -6
    assert lib.fta_check_bwd(*args(db=_t4(B, H, L2, strides=(0, 0, 256)))) == -6
    far = 2**31 // L2
    assert lib.fta_check_bwd(*args(dq=_t5(B, H, L1, L2, D, strides=(far * L2 * L1 * H, far * L2 * L1, far * L2, far)))) == -6


@pytest.mark.parametrize("D,L2", [(32, 128), (32, 384), (32, 512), (32, 1024), (32, 1536), (64, 512)])
def test_required_shapes_are_plannable(D, L2):
    assert _check_fwd(L2=L2, D=D, L1=L2) == 0
    assert fta_lib.load().fta_bwd_workspace_bytes(1, 4, L2, L2, D) > 0


def test_python_surface_mirrors_upstream():
    import flash_tt_attn as fta
    assert fta.attention == fta._attention.apply
    assert issubclass(fta._attention, torch.autograd.Function)
    q = torch.randn(1, 1, 2, 4, 8)
    # the naive formulation is exported for callers and runs on the CPU
    out = fta.reference_tt_attn(q, q, q, torch.zeros(1, 1, 4, 4), 0.3)
    assert out.shape == q.shape


def test_attention_has_no_cpu_fallback():
    import flash_tt_attn as fta
    q = torch.randn(1, 1, 2, 128, 32, dtype=torch.float16)
    b = torch.zeros(1, 1, 128, 128, dtype=torch.float16)
    with pytest.raises(ValueError):
        fta.attention(q, q, q, b, 0.5)          # CPU tensors: refused, not computed some other way
    with pytest.raises(AssertionError):
        fta.attention(q, q, q, b.float(), 0.5)   # dtype mismatch (upstream :561)
    with pytest.raises(AssertionError):
        fta.attention(q[..., :24], q[..., :24], q[..., :24], b, 0.5)  # head dim (upstream :560)
    q16 = torch.randn(1, 1, 2, 128, 16, dtype=torch.float16)
    with pytest.raises(ValueError):
        fta.attention(q16, q16, q16, b, 0.5)     # admitted upstream, not built here


def test_root_alias_module_exports_the_same_objects():
    import importlib.util
    spec = importlib.util.spec_from_file_location("flash_tt_attn_root_alias", os.path.join(ROOT, "flash_tt_attn.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    assert callable(mod.attention) and callable(mod.reference_tt_attn)


def test_sweep_harness_imports_without_gpu():
    """bench_attention.py mirrors upstream's harness signature (flash_tt_attn.py:762) and, like the
    module itself, imports on a machine without a GPU."""
    import inspect
    import bench_attention as ba
    assert list(inspect.signature(ba.bench_attention).parameters) == ["B", "H", "L", "D", "mode", "provider", "device", "metric"]
    assert "triton-fp16" in ba.HIP_PROVIDERS and "hip" in ba.HIP_PROVIDERS


def test_sequence_length_support_query():
    """fta_seq_len_supported: every length up to the longest row built for the head dim."""
    lib = fta_lib.load()
    assert fta_lib.MAX_L2 == int(re.search(r"#define FTA_MAX_L2 (\d+)", open(HEADER).read()).group(1))
    for L2, D, want in [(128, 32, 1), (512, 32, 1), (384, 32, 1), (1536, 32, 1), (2048, 32, 1), (512, 64, 1), (768, 64, 1),
                        (100, 32, 1), (4, 32, 1), (2176, 32, 1), (1408, 32, 1), (4096, 32, 1), (1024, 64, 1), (100, 64, 1),
                        (0, 32, 0), (102, 32, 1), (1, 32, 1), (4095, 32, 1), (4097, 32, 0), (1028, 64, 1), (2048, 64, 1), (2049, 64, 0), (512, 16, 0)]:
        assert lib.fta_seq_len_supported(L2, D) == want, (L2, D)


def test_length_support_with_options_agrees_with_the_entry_points():
    """fta_seq_len_supported_ex is the question fta_fwd_ex / fta_bwd_ex answer with FTA_ERR_SEQ_LEN: for every
    option set and every length (here: every third one), "supported" coincides with a non-zero workspace size, and the plain
    query is the query with default options.  (Every option set is built for every length of the plain
    call; the query exists because that need not stay so.)"""
    lib = fta_lib.load()
    sets = {"default": None, "bf16": fta_lib.Options(fta_lib.DTYPE_BF16, 0, 0.0, 0, 0),
            "dropout": fta_lib.Options(fta_lib.DTYPE_F16, 0, 0.25, 7, 0), "bf16 dropout": fta_lib.Options(fta_lib.DTYPE_BF16, 0, 0.1, 7, 0),
            "precise": fta_lib.Options(fta_lib.DTYPE_F16, 0, 0.0, 0, 1)}
    for name, opt in sets.items():
        ref = ctypes.byref(opt) if opt is not None else None
        for D in (32, 64):
            for L2 in range(0, fta_lib.MAX_L2 + 9, 3):
                ok = lib.fta_seq_len_supported_ex(L2, D, ref)
                assert ok == (1 if lib.fta_bwd_workspace_bytes_ex(1, 1, 1, L2, D, ref) > 0 else 0), (name, D, L2)
                assert ok == lib.fta_seq_len_supported(L2, D), (name, D, L2)
    assert lib.fta_seq_len_supported(2048, 64) == 1 and lib.fta_seq_len_supported_ex(2048, 64, ctypes.byref(sets["dropout"])) == 1
    assert lib.fta_seq_len_supported_ex(2049, 64, ctypes.byref(sets["dropout"])) == 0
    bad = fta_lib.Options(7, 0, 0.0, 0, 0)
    assert lib.fta_seq_len_supported_ex(512, 32, ctypes.byref(bad)) == 0


def test_plan_description_with_options_names_the_kernels_that_run():
    bf16 = fta_lib.Options(fta_lib.DTYPE_BF16, 0, 0.0, 0, 0)
    small = fta_lib.describe_plan(4, 8, 512, 512, 32, 0.17, bf16)
    large = fta_lib.describe_plan(4, 8, 512, 512, 32, 1.3, bf16)
    assert small["options"] == {"type": "BF16", "dropout": 0, "precise_or_vector_alu_backward": 0, "scaled_operand_pair": 0, "natural_exponent": 0}
    assert "dq1" in small["dq"]["kernel"] and "dkdv1" in small["dkdv"]["kernel"]
    # a large scale keeps the hand-scheduled kernels at D = 32 (instances that carry the scaled operand as a
    # pair of bf16 values); D = 64 has no such instances and takes the vector-ALU backward
    assert large["options"] == {"type": "BF16", "dropout": 0, "precise_or_vector_alu_backward": 0, "scaled_operand_pair": 1, "natural_exponent": 0}
    assert "dq1" in large["dq"]["kernel"] and "dkdv1" in large["dkdv"]["kernel"]
    wide = fta_lib.describe_plan(2, 8, 512, 512, 64, 1.3, bf16)
    assert wide["options"]["precise_or_vector_alu_backward"] == 1 and wide["options"]["scaled_operand_pair"] == 0
    assert "dq1" not in wide["dq"]["kernel"] and "dkdv1" not in wide["dkdv"]["kernel"]
    assert fta_lib.describe_plan(2, 8, 512, 512, 64, 0.125, bf16)["options"]["precise_or_vector_alu_backward"] == 0
    # the precise mode of fp16: at D = 32 the hand-scheduled kernels' instances with the operand pair and the
    # exponent in natural units, at D = 64 and for short rows the vector-ALU backward
    precise = fta_lib.Options(fta_lib.DTYPE_F16, 0, 0.0, 0, 1)
    p32 = fta_lib.describe_plan(4, 8, 512, 512, 32, 1.3, precise)
    assert p32["options"] == {"type": "F16", "dropout": 0, "precise_or_vector_alu_backward": 0, "scaled_operand_pair": 1, "natural_exponent": 1}
    assert "dq1" in p32["dq"]["kernel"] and "dkdv1" in p32["dkdv"]["kernel"]
    for args in ((2, 8, 512, 512, 64, 0.125), (4, 8, 128, 128, 32, 0.17)):
        d = fta_lib.describe_plan(*args, precise)
        assert d["options"]["precise_or_vector_alu_backward"] == 1 and d["options"]["natural_exponent"] == 0
        assert "dq1" not in d["dq"]["kernel"] and "dkdv1" not in d["dkdv"]["kernel"]
    drop = fta_lib.describe_plan(4, 8, 512, 512, 32, 1.0, fta_lib.Options(fta_lib.DTYPE_F16, 0, 0.1, 1, 0))
    assert drop["options"]["dropout"] == 1 and drop["fwd"]["kernel"].startswith("fta_fwd_kernel")
    assert fta_lib.describe_plan(4, 8, 512, 512, 32)["fwd"]["kernel"].startswith("fta_fwd1_kernel")


def test_plan_description_is_consistent_for_every_supported_length():
    lib = fta_lib.load()
    for D, lengths in ((32, list(range(128, 4097, 128)) + [4, 100, 1300, 2820, 1, 103, 1301, 4095]), (64, list(range(128, 1025, 128)) + [52, 900, 51, 1023])):
        for L2 in lengths:
            if not lib.fta_seq_len_supported(L2, D):
                continue
            for B, H, L1 in ((1, 1, 1), (4, 8, L2), (1, 4, 37)):
                d = fta_lib.describe_plan(B, H, L1, L2, D)
                assert set(d) == {"fwd", "dq", "dkdv", "workspace", "options"}
                assert d.pop("options") == {"type": "F16", "dropout": 0, "precise_or_vector_alu_backward": 0, "scaled_operand_pair": 0, "natural_exponent": 0}
                for stage in ("fwd", "dq", "dkdv"):
                    s = d[stage]
                    assert s["kernel"].startswith("fta_") and s["launches"] >= 1 and s["grid"] >= 1
                    assert s["block"] in (64, 128, 192, 256, 320, 384, 448, 512)
                    assert 0 < s["lds"] <= 160 * 1024, (D, L2, stage, s)
                tiled = d["workspace"].pop("tiled_length")
                assert tiled % 128 == 0 and L2 <= tiled < L2 + 512
                if tiled >= 256 and D == 32:  # the hand-scheduled kernels also mask a tail (instances of their own)
                    assert "dq1" in d["dq"]["kernel"] and "dkdv1" in d["dkdv"]["kernel"]
                assert sum(d["workspace"].values()) == lib.fta_bwd_workspace_bytes(B, H, L1, L2, D)
    # the benchmark shape runs the hand-scheduled backward kernels, once each
    d = fta_lib.describe_plan(4, 8, 512, 512, 32)
    assert d["dq"]["kernel"] == "fta_bwd_dq1_kernel<32,2>" and d["dq"]["launches"] == 1
    assert d["dkdv"]["kernel"] == "fta_bwd_dkdv1_kernel<32,16>" and d["dkdv"]["launches"] == 1
    # argument errors as everywhere else; a short buffer is reported, not overrun
    buf = ctypes.create_string_buffer(16)
    assert lib.fta_describe_plan(4, 8, 512, 512, 32, buf, 16) == -7 and len(buf.value) < 16
    assert lib.fta_describe_plan(4, 8, 512, 4100, 32, buf, 16) == -4
    assert fta_lib.describe_plan(4, 8, 512, 501, 32)["workspace"]["tiled_length"] == 512
    assert lib.fta_describe_plan(4, 8, 512, 512, 48, buf, 16) == -3
    assert lib.fta_describe_plan(4, 8, 512, 512, 32, None, 0) == -1


def test_chunk_counts_fill_the_last_round_of_workgroups():
    """With few (b,h) slices the L1-chunk count decides how full the last round of workgroups on the
    256 CUs is; the planner picks counts that fill it where the sizes allow."""
    for shape in ((1, 4, 1536, 1536, 32), (1, 8, 768, 768, 32), (4, 8, 512, 512, 32), (4, 8, 1024, 1024, 32), (1, 4, 384, 384, 32)):
        d = fta_lib.describe_plan(*shape)
        for stage in ("fwd", "dq", "dkdv"):
            grid = d[stage]["grid"]
            # (two small workgroups fit a CU, except those of the hand-scheduled kernels: their waves take a
            # SIMD's whole register file)
            two = d[stage]["block"] <= 256 and d[stage]["lds"] <= 80 * 1024 and "1_kernel" not in d[stage]["kernel"]
            slots = 512 if two else 256
            fill = grid / (-(-grid // slots) * slots)
            assert fill >= 0.9, (shape, stage, d[stage], fill)
    # never fewer than 8 rows per chunk, never more chunks than rows allow
    d = fta_lib.describe_plan(1, 1, 16, 512, 32)
    assert d["dq"]["grid"] <= 8 * 2 and d["fwd"]["grid"] <= 4 * 2
