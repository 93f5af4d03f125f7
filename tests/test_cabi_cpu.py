"""CPU-side checks of the C-ABI library and the host logic: no kernel is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def native():
    from stickbreaking_attention import _native

    if not os.path.exists(_native.library_path()):
        import __graft_entry__

        __graft_entry__.build()
    return _native


def declared_functions():
    text = open(os.path.join(ROOT, "include", "sba.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"^\s*(?:const\s+)?(?:int|char\s*\*|const char\s*\*)\s*\**\s*(sba_\w+)\s*\(", text, flags=re.M)


def test_library_exports_every_declared_symbol(native):
    names = declared_functions()
    assert set(names) == set(native.EXPORTS) == {"sba_version", "sba_strerror", "sba_workspace_bytes", "sba_plan_host", "sba_fwd",
                                                 "sba_fwd_static", "sba_bwd", "sba_bwd_kernels"}
    lib = native.lib()
    for n in names:
        assert hasattr(lib, n), n
    assert lib.sba_version() == native.ABI_VERSION == 5
    assert lib.sba_strerror(0) == b"ok"
    for code in range(-9, 0):
        assert lib.sba_strerror(code) not in (b"ok", b"unknown status")
    assert lib.sba_strerror(-99) == b"unknown status"


def test_struct_layout_matches_header(native, tmp_path):
    src = tmp_path / "sz.c"
    src.write_text('#include "sba.h"\n#include <stdio.h>\n#include <stddef.h>\nint main(){printf("%zu %zu %zu %zu %zu %zu %zu %zu %zu %zu\\n", '
                   "sizeof(SbaArgs), offsetof(SbaArgs,q), offsetof(SbaArgs,carry), offsetof(SbaArgs,d_o), "
                   "offsetof(SbaArgs,workspace), offsetof(SbaArgs,trace_events), offsetof(SbaArgs,carry_slots), "
                   "offsetof(SbaArgs,backward_kernels), sizeof(SbaPlan), offsetof(SbaPlan,pairs));}\n")
    exe = tmp_path / "sz"
    import subprocess

    subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    got = [int(x) for x in subprocess.check_output([str(exe)]).split()]
    A = native.SbaArgs
    P = native.SbaPlan
    assert got == [ctypes.sizeof(A), A.q.offset, A.carry.offset, A.d_o.offset, A.workspace.offset, A.trace_events.offset,
                   A.carry_slots.offset, A.backward_kernels.offset, ctypes.sizeof(P), P.pairs.offset]


def _args(native, H, D, T, B, varlen=True, max_seqlen=0, dtype=0):
    a = native.SbaArgs()
    a.dtype, a.head_dim, a.num_heads, a.num_seqs, a.total_tokens, a.max_seqlen = dtype, D, H, B, T, max_seqlen
    a.cu_seqlens = 0x1000 if varlen else None        # only tested for NULL-ness by the size query
    return a


def test_workspace_sizes_cover_any_batch(native):
    """The carry buffer is sized from (T, max_seqlen, num_seqs) alone; it must cover the exact need
    sum_s 256 M_s (M_s + 1), M_s = ceil(L_s / 128), of every batch with those totals (one fp32 per row and
    32-key sub-tile the row sweeps)."""
    lib = native.lib()
    rng = np.random.default_rng(0)
    for _ in range(200):
        B = int(rng.integers(1, 40))
        lengths = rng.integers(1, int(rng.choice([4, 70, 300, 5000])), size=B)
        T, mx, H = int(lengths.sum()), int(lengths.max()), int(rng.integers(1, 9))
        need = sum(256 * m * (m + 1) for m in (-(-int(n) // 128) for n in lengths)) * H * 4
        fwd, bwd, carry = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
        for hint in (mx, 0):
            a = _args(native, H, 64, T, B, max_seqlen=hint)
            assert lib.sba_workspace_bytes(ctypes.byref(a), ctypes.byref(fwd), ctypes.byref(bwd), ctypes.byref(carry)) == 0
            assert carry.value >= need and bwd.value >= fwd.value + carry.value
            assert fwd.value >= 256 + 16 * (-(-T // 128) + B) + 8 * B
    # fixed-length mode is exact
    a = _args(native, 3, 128, 500, 4, varlen=False)
    assert lib.sba_workspace_bytes(ctypes.byref(a), None, None, ctypes.byref(carry)) == 0
    assert carry.value == -(-(4 * 256 * 4 * 5 * 3 * 4) // 256) * 256


def test_python_carry_size_matches_library(native):
    """The operators size the carry buffer from shapes alone (traceable by torch.compile); that formula must
    agree with what the library reports."""
    lib = native.lib()
    rng = np.random.default_rng(1)
    carry = ctypes.c_size_t()
    for _ in range(200):
        H, B, T = int(rng.integers(1, 40)), int(rng.integers(1, 50)), int(rng.integers(1, 100000))
        for hint in (0, int(rng.integers(1, T + 1)), T + 5):
            a = _args(native, H, 64, T, B, max_seqlen=hint)
            assert lib.sba_workspace_bytes(ctypes.byref(a), None, None, ctypes.byref(carry)) == 0
            assert native.carry_elems(H, T, B, hint, False) * 4 == carry.value
        a = _args(native, H, 64, T, B, varlen=False)
        assert lib.sba_workspace_bytes(ctypes.byref(a), None, None, ctypes.byref(carry)) == 0
        assert native.carry_elems(H, T, B, None, True) * 4 == carry.value


def test_exact_carry_slots_shrink_the_buffers(native):
    """With the exact per-head slot count from the host plan the carry buffer (and the backward's prefix plane) are the
    need itself, not the total_tokens * max_seqlen / 64 bound: the adversarial batch (2048 short sequences and one of
    16384) drops from about 4.5x the need to 1.0x."""
    import bench

    lib = native.lib()
    lengths = bench.lengths_for("c5")
    T, H = sum(lengths), 32
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lengths)]), dtype=torch.int32)
    plan = native.plan_host(cu, True, T)
    exact = sum(256 * m * (m + 1) for m in (-(-n // 128) for n in lengths))
    assert plan.status == 0 and plan.carry_slots == exact and plan.longest == 16384 and plan.covered_tokens == T
    assert plan.query_tiles == sum(-(-n // 128) for n in lengths) and plan.key_tiles == sum(-(-n // 64) for n in lengths)
    assert plan.pairs == sum(n * (n - 1) // 2 for n in lengths)
    carry_bound, carry_exact, bwd_exact = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
    a = _args(native, H, 128, T, len(lengths), max_seqlen=16384)
    assert lib.sba_workspace_bytes(ctypes.byref(a), None, None, ctypes.byref(carry_bound)) == 0
    a.carry_slots = plan.carry_slots
    assert lib.sba_workspace_bytes(ctypes.byref(a), None, ctypes.byref(bwd_exact), ctypes.byref(carry_exact)) == 0
    need = exact * H * 4
    assert need <= carry_exact.value <= need + 256 and carry_bound.value > 4 * need
    assert bwd_exact.value <= 1.2 * need + (1 << 22)          # prefix plane + tile lists + per-row scalars
    assert native.carry_elems(H, T, len(lengths), 16384, False, exact) * 4 == carry_exact.value
    a.carry_slots = -1
    assert lib.sba_workspace_bytes(ctypes.byref(a), None, None, None) == -6
    a.carry_slots, a.recompute_carry = 0, 2
    assert lib.sba_workspace_bytes(ctypes.byref(a), None, None, None) == -6
    # rebuilding the products inside the backward moves the carry plane into the backward's workspace
    a.carry_slots, a.recompute_carry = plan.carry_slots, 1
    bwd_recompute = ctypes.c_size_t()
    assert lib.sba_workspace_bytes(ctypes.byref(a), None, ctypes.byref(bwd_recompute), None) == 0
    assert bwd_recompute.value == bwd_exact.value + carry_exact.value
    a.dtype = 1
    assert lib.sba_workspace_bytes(ctypes.byref(a), None, None, None) == -2           # not for fp32
    # a backward workspace smaller than the whole call is taken as a limit (the heads go through in groups), but it
    # must hold at least one head: refused on the host, before anything is launched
    a.dtype = 0
    a.num_heads = 1
    one_head = ctypes.c_size_t()
    assert lib.sba_workspace_bytes(ctypes.byref(a), None, ctypes.byref(one_head), None) == 0
    assert one_head.value < bwd_recompute.value / 16
    a.num_heads = H
    a.workspace, a.workspace_bytes = 256, one_head.value - 256          # never dereferenced: the size check comes first
    assert lib.sba_bwd(ctypes.byref(a)) == -7


def test_host_plan_rejects_what_the_scheduler_rejects(native):
    """sba_plan_host runs the scheduler's own reading of cu_seqlens (one shared function) on a host copy: decreasing
    ends, ends beyond total_tokens, negative entries and a leading entry other than 0 void the schedule; empty
    sequences and trailing uncovered tokens are fine."""
    T = 100
    good = [
        ([10, 10, 40, 100], False, 100), ([0, 10, 40], True, 40), ([100], False, 100), ([0, 0, 0], False, 0),
        ([5], False, 5), ([0, 100], True, 100),
    ]
    for cu, lead, covered in good:
        for dt in (torch.int32, torch.int64):
            plan = native.plan_host(torch.tensor(cu, dtype=dt), lead, T)
            assert plan.status == 0 and plan.covered_tokens == covered, (cu, lead)
    bad = [([10, 5, 40], False), ([10, 101], False), ([-1, 10], False), ([3, 10], True), ([0, 50, 20], True),
           ([2 ** 40, 2 ** 40 + 1], False), ([10, -2 ** 31], False)]
    for cu, lead in bad:
        plan = native.plan_host(torch.tensor(cu, dtype=torch.int64), lead, T)
        assert plan.status == 1 and plan.query_tiles == 0 and plan.key_tiles == 0 and plan.carry_slots == 0, (cu, lead)
    # for every valid batch the tile counts stay inside what sba_workspace_bytes reserves from shapes alone
    rng = np.random.default_rng(5)
    for _ in range(300):
        B = int(rng.integers(1, 60))
        lengths = rng.integers(0, int(rng.choice([3, 70, 300, 3000])), size=B)
        pad = int(rng.integers(0, 200))
        total = int(lengths.sum()) + pad
        if total == 0:
            continue
        plan = native.plan_host(torch.tensor(np.cumsum(lengths)), False, total)
        assert plan.status == 0 and plan.covered_tokens == int(lengths.sum())
        assert plan.query_tiles <= -(-total // 128) + B and plan.key_tiles <= -(-total // 64) + B
        idle = -(-total // 128) + B - plan.query_tiles          # workgroups left to zero-fill the uncovered rows
        assert idle * 128 >= pad
        mx = max(int(lengths.max()), 1)
        assert plan.carry_slots <= -(-(total * mx) // 64) + 6 * total + 512 * B
    # fixed-length mode
    a = native.plan_host(None, False, 500, num_seqs=4)
    assert a.status == 0 and a.query_tiles == 16 and a.carry_slots == 4 * 256 * 4 * 5 and a.pairs == 4 * 500 * 499 // 2


def test_custom_ops_are_registered(native):
    """The four launchers are torch.library operators named like the reference's (utils.py:20-40 with
    sb_varlen_fwd.py:453, sb_varlen_bwd.py:541, sb_attn/sb_fwd.py:175, sb_attn/sb_bwd.py:207), out-parameter style."""
    from stickbreaking_attention import utils

    assert utils.PACKAGE_NAME == "stickbreaking_attention" and abs(utils.inv_log2 - 1.4426950408889634) < 1e-15
    ns = torch.ops.stickbreaking_attention
    for name, mutated in (("varlen_fwd", ("o", "rem", "neg_log_acc", "carry")), ("varlen_bwd", ("dq", "dk", "dv")),
                          ("attn_fwd", ("o", "rem", "neg_log_acc", "carry")), ("attn_bwd", ("dq", "dk", "dv"))):
        schema = getattr(ns, name).default._schema
        assert len(schema.returns) == 0
        assert tuple(a.name for a in schema.arguments if a.alias_info is not None and a.alias_info.is_write) == mutated


def test_size_query_validates(native):
    lib = native.lib()
    assert lib.sba_workspace_bytes(None, None, None, None) == -1
    assert lib.sba_workspace_bytes(ctypes.byref(_args(native, 0, 64, 10, 1)), None, None, None) == -6
    assert lib.sba_workspace_bytes(ctypes.byref(_args(native, 1, 0, 10, 1)), None, None, None) == -3
    assert lib.sba_workspace_bytes(ctypes.byref(_args(native, 1, 129, 10, 1)), None, None, None) == -3
    assert lib.sba_workspace_bytes(ctypes.byref(_args(native, 1, 64, 10, 1, dtype=9)), None, None, None) == -2


def test_operators_refuse_cpu_tensors(native):
    from stickbreaking_attention import sb_attn, sb_attn_varlen

    q = torch.zeros(2, 8, 16)
    with pytest.raises(RuntimeError, match="GPU only"):
        sb_attn_varlen(q, q, q, torch.tensor([8]), 8, zero_start=False)
    with pytest.raises(RuntimeError, match="GPU only"):
        sb_attn(q[None], q[None], q[None])
    with pytest.raises(AssertionError):
        sb_attn_varlen(q, q, q, torch.tensor([3, 8]), 8, zero_start=True)


def test_missing_library_fails_loudly(native, monkeypatch):
    monkeypatch.setattr(native, "_lib", None)
    monkeypatch.setattr(native, "_LIB_NAME", "libsba_absent.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        native.lib()


def test_workload_generators():
    import bench

    for name, total, count in (("c1", 448, 3), ("c2", 16384, None), ("c3", 32768, None), ("c4", 32768, 8), ("c5", None, 2049)):
        lengths = bench.lengths_for(name)
        assert all(n >= 1 for n in lengths)
        if total:
            assert sum(lengths) == total
        if count:
            assert len(lengths) == count
    assert max(bench.lengths_for("c3")) <= 8192 and bench.lengths_for("c5")[-1] == 16384
    assert bench.visible_pairs([4096] * 8, 32) == 8 * 32 * 4096 * 4095 // 2 == 2146959360
