"""CPU-side tests: the public operator's validation (reference: flash_colsum/ops.py:58-97,
tests/test_core.py:113-134), the C-ABI library's exports and its host-side argument checks.
No kernel is launched here."""
import ctypes
import os
import re
import types

import pytest
import torch

import flash_colsum
from flash_colsum import _hip, flash_colsum as op

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


class FakeCuda:
    """Stands in for a GPU tensor in validation tests: only what the checks read."""

    def __init__(self, *shape):
        self.shape = torch.Size(shape)
        self.ndim = len(shape)
        self.device = types.SimpleNamespace(type="cuda")


def test_exports_match_reference_package():
    assert callable(flash_colsum.flash_colsum) and callable(flash_colsum.naive_colsum)
    assert flash_colsum.__version__ == "1.0.0"


def test_validation_messages_and_order():
    with pytest.raises(ValueError, match="4D"):
        op(torch.zeros(2, 3, 4), torch.zeros(2, 3, 4))
    # device check comes before every shape check (ops.py:62)
    with pytest.raises(ValueError, match="CUDA"):
        op(torch.zeros(1, 8, 128, 64), torch.zeros(1, 8, 128, 64))
    with pytest.raises(ValueError, match="CUDA"):
        op(torch.zeros(2, 8, 128, 64), torch.zeros(2, 8, 256, 64), is_causal=True, cls_len=0)
    # cls_len checks come before the causal batch check (ops.py:65-68)
    with pytest.raises(ValueError, match="only supported for non-causal"):
        op(FakeCuda(2, 8, 128, 64), FakeCuda(2, 8, 1024, 64), is_causal=True, cls_len=1)
    with pytest.raises(ValueError, match="must be positive"):
        op(FakeCuda(2, 8, 128, 64), FakeCuda(2, 8, 256, 64), cls_len=0)
    with pytest.raises(ValueError, match="batch size 1"):
        op(FakeCuda(2, 8, 128, 64), FakeCuda(2, 8, 1024, 64), is_causal=True)
    with pytest.raises(ValueError, match="same heads and head_dim"):
        op(FakeCuda(1, 8, 128, 64), FakeCuda(1, 4, 1024, 64), is_causal=True)
    with pytest.raises(ValueError, match="same heads and head_dim"):
        op(FakeCuda(1, 8, 128, 64), FakeCuda(1, 8, 1024, 128), is_causal=True)
    with pytest.raises(ValueError, match="same shape"):
        op(FakeCuda(2, 8, 128, 64), FakeCuda(2, 8, 256, 64))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "flash_colsum.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fcs_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _hip.lib()
    names = _declared_symbols()
    assert set(names) >= {"fcs_abi_version", "fcs_colsum_causal_bf16", "fcs_colsum_causal_f16", "fcs_colsum_noncausal_bf16",
                          "fcs_colsum_noncausal_f16", "fcs_colsum_noncausal_f16_static", "fcs_colsum_general",
                          "fcs_topk_f32", "fcs_threshold_f32", "fcs_strerror", "fcs_workspace_bytes", "fcs_colsum_call",
                          "fcs_plan_describe", "fcs_static_scratch_init"}
    for n in names:
        assert getattr(lib, n) is not None
    assert lib.fcs_abi_version() == 5


def test_strerror_is_total():
    for code in range(-9, 3):
        assert isinstance(_hip.strerror(code), str) and _hip.strerror(code)
    assert "head dim" in _hip.strerror(-3)


def test_workspace_bytes():
    wb = _hip.workspace_bytes
    assert wb(False, 0, 1, 1, 1, 64) == 0 and wb(False, 1, 1, 1, 0, 64) == 0
    for args in [(False, 8, 16, 2048, 2048, 64, -1), (False, 32, 16, 577, 577, 64, 1),
                 (True, 1, 32, 128, 4096, 128, -1), (True, 1, 32, 512, 65536, 128, -1), (False, 1, 1, 1, 1, 64, -1)]:
        n = wb(*args)
        assert n > 0 and n % 256 == 0
    # never more than a few floats per (row, head) plus a few partial outputs: O(S), not O(S^2)
    assert wb(False, 8, 16, 2048, 2048, 64) < 64 << 20
    assert wb(True, 1, 32, 512, 65536, 128) < 64 << 20
    # fused path: one slab per workgroup along the query axis.  B8 H16 S2048 runs as one generation of
    # 256 workgroups (two row blocks x sixteen heads each): 32 slabs of (8, 2048) floats
    assert wb(False, 8, 16, 2048, 2048, 64) == 32 * 8 * 2048 * 4
    # B256 H16 S1024 (64-row blocks): eight row blocks per workgroup, two slabs of two query groups
    assert wb(False, 256, 16, 1024, 1024, 64) == 2 * 2 * 256 * 1024 * 4


def test_workspace_plan_over_random_shapes():
    """The launch plan behind fcs_workspace_bytes() must hold for any shape: aligned, nonzero,
    linear in the sequence lengths (never quadratic), and independent of cls_n beyond its clamp."""
    import random

    rng = random.Random(7)
    wb = _hip.workspace_bytes
    for _ in range(400):
        causal = rng.random() < 0.4
        b = 1 if causal else rng.choice([1, 2, 7, 32, 300])
        h = rng.choice([1, 2, 8, 16, 32, 40])
        if b * h > 65535:
            continue
        d = rng.choice([64, 128, 40, 192, 256])
        sk = rng.choice([1, 5, 64, 577, 2048, 2049, 8191, 65536, 262144])
        sq = rng.choice([1, 16, 128, 512, 1000]) if causal else sk
        cls_n = -1 if causal else rng.choice([-1, 1, 2, 4, 5, 100, sq, sq + 7])
        n = wb(causal, b, h, sq, sk, d, cls_n)
        assert n > 0 and n % 256 == 0, (causal, b, h, sq, sk, d, cls_n, n)
        # a few floats per (batch, head, row) plus at most a few thousand partial rows of Sk floats
        bound = 64 * b * h * (sq + 1024) + 4 * 4096 * (b * sk + 1024) + (1 << 20)
        assert n <= bound, (causal, b, h, sq, sk, d, cls_n, n, bound)
        if cls_n >= sq:
            assert n == wb(causal, b, h, sq, sk, d, -1)


def test_argument_errors_are_reported_without_a_gpu():
    lib = _hip.lib()
    st = (ctypes.c_int64 * 4)(8 * 16 * 64, 16 * 64, 64, 1)
    bad_last = (ctypes.c_int64 * 4)(8 * 16 * 64, 16 * 64, 64, 2)
    unaligned = (ctypes.c_int64 * 4)(8 * 16 * 66, 16 * 66, 66, 1)
    p = ctypes.c_void_p(4096)  # never dereferenced: every call below fails its host checks
    nc, ca = lib.fcs_colsum_noncausal_f16, lib.fcs_colsum_causal_f16
    assert nc(None, p, p, None, p, 1 << 30, 2, 8, 16, 64, st, st, 0.125, -1, None) == -1
    assert nc(p, p, None, None, p, 1 << 30, 2, 8, 16, 64, st, st, 0.125, -1, None) == -1
    assert nc(p, p, p, None, p, 1 << 30, 0, 8, 16, 64, st, st, 0.125, -1, None) == -2
    assert nc(p, p, p, None, p, 1 << 30, 2, 8, 16, 64, st, st, 0.125, 0, None) == -2
    assert nc(p, p, p, None, p, 1 << 30, 2, 8, 16, 84, st, st, 0.125, -1, None) == -3
    assert nc(p, p, p, None, p, 1 << 30, 2, 8, 16, 264, st, st, 0.125, -1, None) == -3
    assert nc(p, p, p, None, p, 1 << 30, 2, 8, 16, 64, bad_last, st, 0.125, -1, None) == -4
    assert nc(p, p, p, None, p, 1 << 30, 2, 8, 16, 64, st, unaligned, 0.125, -1, None) == -4
    assert nc(ctypes.c_void_p(4098), p, p, None, p, 1 << 30, 2, 8, 16, 64, st, st, 0.125, -1, None) == -4
    assert nc(p, p, p, None, p, 16, 2, 8, 16, 64, st, st, 0.125, -1, None) == -5
    assert nc(p, p, p, None, None, 0, 2, 8, 16, 64, st, st, 0.125, -1, None) == -1
    assert nc(p, p, p, None, p, 1 << 30, 2, 8, 16, 64, st, st, float("nan"), -1, None) == -6
    assert ca(p, p, p, None, p, 1 << 30, 8, 16, 64, 64, -1, st, st, 0.125, None) == -2
    assert ca(p, p, p, None, p, 1 << 30, 8, 16, 64, 4, 48, st, st, 0.125, None) == -3
    assert ca(p, p, p, None, p, 16, 8, 16, 64, 64, 48, st, st, 0.125, None) == -5
    # the bf16 entry points share the checks
    nb, cb = lib.fcs_colsum_noncausal_bf16, lib.fcs_colsum_causal_bf16
    assert nb(None, p, p, None, p, 1 << 30, 2, 8, 16, 64, st, st, 0.125, -1, None) == -1
    assert nb(p, p, p, None, p, 1 << 30, 2, 8, 16, 81, st, st, 0.125, -1, None) == -3
    assert nb(p, p, p, None, p, 16, 2, 8, 16, 64, st, st, 0.125, -1, None) == -5
    assert cb(p, p, p, None, p, 1 << 30, 8, 16, 64, 64, -1, st, st, 0.125, None) == -2
    assert cb(p, p, p, None, p, 16, 8, 16, 64, 64, 48, st, st, 0.125, None) == -5


def _call_struct(**kw):
    c = _hip._Call()
    c.struct_bytes = ctypes.sizeof(_hip._Call)
    c.dtype, c.causal, c.B, c.Hq, c.Hk, c.Sq, c.Sk, c.D, c.cls_n, c.k_past, c.scale = 0, 0, 2, 8, 8, 1024, 1024, 64, -1, 0, 0.125
    c.q_strides = (ctypes.c_int64 * 4)(8 * 1024 * 64, 1024 * 64, 64, 1)
    c.k_strides = (ctypes.c_int64 * 4)(8 * 1024 * 64, 1024 * 64, 64, 1)
    c.q = c.k = c.out = c.ws = 4096  # never dereferenced
    c.ws_bytes = 1 << 30
    for name, v in kw.items():
        setattr(c, name, v)
    return c


def test_struct_call_reports_argument_errors_without_a_gpu():
    lib = _hip.lib()
    call = lib.fcs_colsum_call
    assert call(None) == -1
    assert call(ctypes.byref(_call_struct(struct_bytes=8))) == -9 and "fcs_call_t" in _hip.strerror(-9)
    assert call(ctypes.byref(_call_struct(dtype=7))) == -8
    assert call(ctypes.byref(_call_struct(q=None))) == -1
    assert call(ctypes.byref(_call_struct(B=0))) == -2
    assert call(ctypes.byref(_call_struct(Hk=3))) == -2
    assert call(ctypes.byref(_call_struct(causal=1, k_past=-1))) == -2
    assert call(ctypes.byref(_call_struct(D=12))) == -3
    assert call(ctypes.byref(_call_struct(q=4098))) == -4
    assert call(ctypes.byref(_call_struct(ws_bytes=1024))) == -5
    assert call(ctypes.byref(_call_struct(ws=4100))) == -5
    assert call(ctypes.byref(_call_struct(scale=float("inf")))) == -6
    # the struct mirrors the C declaration field for field
    text = open(os.path.join(ROOT, "include", "flash_colsum.h")).read()
    body = re.search(r"typedef struct fcs_call \{(.*?)\} fcs_call_t;", text, flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    declared = []
    for stmt in body.split(";"):
        stmt = stmt.strip()
        if stmt:
            declared += [n.strip(" *").split("[")[0] for n in stmt.split(",")]
            declared[-len(stmt.split(",")):] = [n.split()[-1].strip("*") for n in declared[-len(stmt.split(",")):]]
    assert declared == [f[0] for f in _hip._Call._fields_], declared


def test_plan_description_and_k_past_clamp():
    """The launch plan as text: which kernels a call gets.  Any k_past >= K_len means "no mask" and must plan
    (and run) like k_past = K_len, INT_MAX included: the kernels add it to row numbers in 32 bits."""
    d = _hip.plan_description
    t = d((8, 16, 2048, 64), (8, 16, 2048, 64))
    assert "fcs_fused_kernel<64,8,false,8,false,true>" in t and "fcs_finalize_kernel<8>" in t
    assert "fcs_fewrows_kernel<64,1,false>" in d((32, 16, 577, 64), (32, 16, 577, 64), cls_n=1)
    # short sequences: one wave per 32 rows; three heads per workgroup fill the 256 compute units at B 64, H 12
    t = d((64, 12, 197, 64), (64, 12, 197, 64))
    assert "fcs_small_kernel<7,false,true> grid 256, 3 heads x 7 row tiles" in t, t
    assert "fcs_small_kernel<9,true,false>" in d((32, 16, 257, 64), (32, 16, 257, 64), bf16=True)
    assert "fcs_small_kernel<1,false,false>" in d((2, 3, 5, 40), (2, 3, 5, 40))
    assert "fcs_fused_kernel" in d((6, 24, 197, 64), (6, 24, 197, 64), cls_n=33)  # two row tiles per head: too many heads per step
    assert "fcs_fused_kernel" in d((2, 4, 289, 64), (2, 4, 289, 64))
    # head dims other than 64 on the single-pass kernels: 128-wide ones above 64 channels, zeros past the head dim
    assert "fcs_fused_kernel<128,8,true,0,false,true> " in d((8, 16, 1024, 128), (8, 16, 1024, 128))
    assert "fcs_fused_kernel<128,4,true,0,false,true,true>" in d((8, 16, 1024, 96), (8, 16, 1024, 96))
    assert "fcs_fused_kernel<64,8,true,0,true,true,true>" in d((8, 16, 2048, 32), (8, 16, 2048, 32), bf16=True)
    assert "fcs_rowstream_kernel<128" in d((8, 16, 2048, 96), (8, 16, 2048, 96))     # 72 .. 120 channels stop at 1536 keys
    assert "fcs_rowstream_kernel<256" in d((8, 16, 1024, 160), (8, 16, 1024, 160))
    t = d((1, 32, 512, 128), (1, 32, 65536, 128), causal=True)
    assert "fcs_rowstream_kernel<128,2,8,false,false>" in t and "fcs_colstream_kernel<128,2,8,false,false>" in t
    # 64-wide heads, 32 x 512 = 16384 averaged rows: both passes on the pre-scaled operand for the keys every row sees
    t = d((1, 32, 512, 64), (1, 32, 65536, 64), causal=True)
    assert "fcs_rowstream_kernel<64,2,8,false,true>" in t and "fcs_colstream_kernel<64,2,8,false,true>" in t
    t = d((1, 32, 128, 64), (1, 32, 4096, 64), causal=True)
    assert "fcs_rowstream_kernel<64,1,4,false,false>" in t and "fcs_colstream_kernel<64,1,4,false,false>" in t
    assert "bf16" not in t and "fcs_fused_kernel<64,8,true,8,true,false>" in d((8, 16, 2048, 64), (8, 16, 2048, 64), bf16=True)
    base = d((1, 4, 100, 128), (1, 4, 1000, 128), causal=True, k_past=1000)
    for kp in (1001, 5000, 2 ** 31 - 1, 2 ** 40):
        assert d((1, 4, 100, 128), (1, 4, 1000, 128), causal=True, k_past=kp) == base
    c = _call_struct(causal=1, Sq=100, k_past=2 ** 31 - 1)
    buf = ctypes.create_string_buffer(1024)
    n = _hip.lib().fcs_plan_describe(ctypes.byref(c), buf, len(buf))
    c.k_past = 1024
    buf2 = ctypes.create_string_buffer(1024)
    assert n > 0 and _hip.lib().fcs_plan_describe(ctypes.byref(c), buf2, len(buf2)) == n and buf.value == buf2.value
    # snprintf semantics: truncated output, full length returned
    small = ctypes.create_string_buffer(8)
    assert _hip.lib().fcs_plan_describe(ctypes.byref(c), small, len(small)) == n and len(small.value) == 7
    assert _hip.lib().fcs_plan_describe(ctypes.byref(_call_struct(B=0)), buf, len(buf)) == 0


def test_more_than_65535_batch_entries_times_heads_plan():
    """Both passes of the two-pass path launch one-dimensional grids: no 16-bit grid axis limits B * H."""
    assert _hip.workspace_bytes(False, 4096, 32, 64, 4096, 64) > 0
    assert _hip.workspace_bytes(True, 70000, 1, 8, 300, 128) > 0
    assert "grid" in _hip.plan_description((4096, 32, 64, 128), (4096, 32, 64, 128))


def test_kernel_inputs_with_odd_strides_on_unit_dimensions():
    """torch calls a tensor contiguous whatever the strides of its size-1 dimensions; the library wants every
    stride a multiple of 8 elements, so such tensors must still be checked (and copied when needed)."""
    import torch

    base = torch.zeros(4 * 77 * 64 + 64, dtype=torch.float16)
    t = base.as_strided((4, 1, 77, 64), (77 * 64, 3, 64, 1))  # one head, head stride 3
    assert t.is_contiguous()
    u = _hip._as_kernel_input(t)
    assert u.stride(1) % 8 == 0 and u.stride(2) % 8 == 0
    t = base.as_strided((4, 2, 1, 64), (2 * 64, 64, 5, 1))  # one row, row stride 5
    assert t.is_contiguous()
    u = _hip._as_kernel_input(t)
    assert u.stride(1) % 8 == 0 and u.stride(2) % 8 == 0
    v = torch.zeros((2, 3, 16, 64), dtype=torch.float16)
    assert _hip._as_kernel_input(v) is v


def test_topk_argument_errors_without_a_gpu():
    lib = _hip.lib()
    p = ctypes.c_void_p(4096)
    assert lib.fcs_topk_f32(None, 1, 8, 2, p, None, 0, None) == -1
    assert lib.fcs_topk_f32(p, 1, 8, 0, p, None, 0, None) == -2
    assert lib.fcs_topk_f32(p, 1, 8, 9, p, None, 0, None) == -2
    assert lib.fcs_topk_f32(p, 1, 100000, _hip.TOPK_SORT_MAX + 1, p, None, 1, None) == -2
    assert lib.fcs_threshold_f32(p, 1, 8, 0.5, p, None, None) == -1
    assert lib.fcs_threshold_f32(p, 0, 8, 0.5, p, p, None) == -2
    assert lib.fcs_threshold_f32(p, 1, 8, float("nan"), p, p, None) == -6
    text = open(os.path.join(ROOT, "include", "flash_colsum.h")).read()
    assert f"#define FCS_TOPK_SORT_MAX {_hip.TOPK_SORT_MAX}" in text


def test_missing_library_is_loud(monkeypatch, tmp_path):
    monkeypatch.setattr(_hip, "_lib", None)
    monkeypatch.setattr(_hip, "_LIB_PATH", str(tmp_path / "libflashcolsum.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        _hip.lib()


def integration_stub():
    """The binding stub that the integration notes at the repository root show to a maintainer of the
    reference, executed as written (only the library's file name is replaced by its path in this tree)."""
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    blocks = re.findall(r"```python\n(.*?)```", text, flags=re.S)
    code = next(b for b in blocks if "_flash_colsum_batched" in b)
    assert '"libflashcolsum.so"' in code
    ns = {}
    exec(compile(code.replace('"libflashcolsum.so"', repr(_hip._LIB_PATH)), "INTEGRATION.md", "exec"), ns)
    return ns


def test_integration_stub_binds_and_reports_errors():
    ns = integration_stub()
    lib = ns["_lib"]
    for name in ("_flash_colsum_batched", "_flash_colsum_non_batched", "_flash_colsum_causal"):
        assert callable(ns[name])
    # the error path of the stub: a negative code becomes the library's text
    p = ctypes.c_void_p(4096)
    st = (ctypes.c_int64 * 4)(8 * 16 * 64, 16 * 64, 64, 2)
    rc = lib.fcs_colsum_noncausal_f16(p, p, p, None, p, 1 << 30, 2, 8, 16, 64, st, st, 0.125, -1, None)
    assert rc == -4 and "stride" in lib.fcs_strerror(rc).decode()
    rc = lib.fcs_colsum_causal_bf16(p, p, p, None, p, 16, 8, 16, 64, 64, 48, st, st, 0.125, None)
    assert rc < 0 and lib.fcs_strerror(rc).decode()
