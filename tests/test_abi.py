"""C-ABI checks that need no GPU: the library loads, exports every symbol the
header declares, its structs match the ctypes mirror, and invalid calls are
rejected with the documented status before anything is launched."""
import ctypes as C
import os
import re
import subprocess

import pytest
import torch

from ma import _hip_lib as L

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ma_hip.h")


def declared_functions():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"^\s*(?:const\s+char\s*\*|int|uint64_t)\s+(ma_\w+)\s*\(", src, flags=re.M)))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    assert set(L.EXPORTS) <= set(names), names
    assert "ma_fwd" in names and "ma_r_step" in names


def test_library_exports_every_declared_symbol():
    lib = L.load()
    for name in declared_functions():
        assert hasattr(lib, name), f"libma_hip.so does not export {name}"
    assert lib.ma_abi_version() == L.ABI_VERSION


def test_struct_layout_matches_header(tmp_path):
    prog = tmp_path / "sz.c"
    prog.write_text(
        '#include <stdio.h>\n#include <stddef.h>\n#include "ma_hip.h"\n'
        "int main(void){printf(\"%zu %zu %zu %zu %zu %zu %zu %zu\\n\", sizeof(ma_fwd_params), offsetof(ma_fwd_params,E),"
        " offsetof(ma_fwd_params,q_stride), offsetof(ma_fwd_params,mask_stride), offsetof(ma_fwd_params,eps),"
        " offsetof(ma_fwd_params,error_word), sizeof(ma_bwd_params), sizeof(ma_ws_layout)); return 0;}\n")
    exe = tmp_path / "sz"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(prog), "-o", str(exe)],
                   check=True)
    got = [int(x) for x in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()]
    F = L.FwdParams
    assert got == [C.sizeof(F), F.E.offset, F.q_stride.offset, F.mask_stride.offset, F.eps.offset,
                   F.error_word.offset, C.sizeof(L.BwdParams), C.sizeof(L.WsLayout)]


def good_params(**kw):
    p = L.FwdParams()
    p.E, p.H, p.N, p.D, p.Dv, p.B, p.T = 2, 3, 50, 16, 16, 8, 2
    p.dtype_qk = p.dtype_v = L.MA_F16
    for name, inner in (("q_stride", 16), ("k_stride", 16), ("v_stride", 16), ("out_stride", 16)):
        setattr(p, name, (C.c_int64 * 3)(3 * 50 * inner, 50 * inner, inner))
    p.eps = 1e-12
    for k, v in kw.items():
        setattr(p, k, v)
    return p


def test_workspace_layout_is_ordered_and_aligned():
    lib = L.load()
    p = good_params()
    lay = L.WsLayout()
    assert lib.ma_fwd_workspace_layout(p, lay) == L.MA_OK
    offs = [lay.sync, lay.aR, lay.cR, lay.aL, lay.cL, lay.Y, lay.stats, lay.total]
    assert lay.sync == 0 and offs == sorted(offs) and all(o % 256 == 0 for o in offs)
    rows = 2 * 3 * 7 * 8                       # E*H*Np with Np = ceil(50/8)*8
    assert lay.cR - lay.aR >= rows * 16 * 2 and lay.aL - lay.cR >= rows * 4
    assert lib.ma_fwd_workspace_bytes(p) == lay.total


@pytest.mark.parametrize("field,value,status", [
    ("E", 0, L.MA_ERR_SHAPE), ("N", -3, L.MA_ERR_SHAPE), ("B", 0, L.MA_ERR_SHAPE), ("T", 0, L.MA_ERR_SHAPE),
    ("Dv", 0, L.MA_ERR_SHAPE), ("dtype_qk", 7, L.MA_ERR_DTYPE), ("dtype_v", -1, L.MA_ERR_DTYPE),
    ("variant", 9, L.MA_ERR_VARIANT), ("variant", -1, L.MA_ERR_VARIANT),
])
def test_invalid_problem_is_rejected(field, value, status):
    lib = L.load()
    p = good_params(**{field: value})
    assert lib.ma_fwd_workspace_layout(p, L.WsLayout()) == status
    assert lib.ma_fwd_workspace_bytes(p) == 0
    assert lib.ma_fwd(p, None) == status
    assert L.strerror(status)


def test_overlapping_rows_and_negative_strides_are_rejected():
    lib = L.load()
    p = good_params()
    p.q_stride = (C.c_int64 * 3)(2400, 800, 8)       # row stride < D
    assert lib.ma_fwd_workspace_bytes(p) == 0
    assert lib.ma_fwd(p, None) == L.MA_ERR_STRIDE
    p = good_params()
    p.v_stride = (C.c_int64 * 3)(-1, 800, 16)
    assert lib.ma_fwd(p, None) == L.MA_ERR_STRIDE
    p = good_params()
    if p.H > 1:                                       # output slices of different heads may not coincide
        p.out_stride = (C.c_int64 * 3)(p.out_stride[0], 0, p.out_stride[2])
        assert lib.ma_fwd(p, None) == L.MA_ERR_STRIDE
    p = good_params()
    p.k_stride = (C.c_int64 * 3)(0, 0, p.k_stride[2])  # inputs may be broadcast over batch and heads
    assert lib.ma_fwd_workspace_bytes(p) > 0


def test_pointer_and_workspace_checks_precede_any_launch():
    lib = L.load()
    p = good_params()
    assert lib.ma_fwd(p, None) == L.MA_ERR_NULL                      # q/k/v/out NULL
    p.q = p.k = p.v = p.out = 0x10000
    assert lib.ma_fwd(p, None) == L.MA_ERR_WORKSPACE                 # no workspace
    need = lib.ma_fwd_workspace_bytes(p)
    p.workspace, p.workspace_bytes = 0x100000, need - 1
    assert lib.ma_fwd(p, None) == L.MA_ERR_WORKSPACE                 # too small
    p.workspace, p.workspace_bytes = 0x100010, need
    assert lib.ma_fwd(p, None) == L.MA_ERR_WORKSPACE                 # misaligned
    p.workspace = 0x100000
    p.q = 0x10001                                                    # fp16 pointer must be 2-byte aligned
    assert lib.ma_fwd(p, None) == L.MA_ERR_STRIDE
    for fn in (lib.ma_l_step, lib.ma_z_step):
        assert fn(good_params(), None) == L.MA_ERR_NULL
    assert lib.ma_r_step(good_params(), 1, 0, None) == L.MA_ERR_NULL
    assert lib.ma_fwd(None, None) == L.MA_ERR_NULL
    # ma_matrix: NULL output, NULL q / k, missing workspace, one-launch variants
    assert lib.ma_matrix(good_params(), None, None) == L.MA_ERR_NULL
    assert lib.ma_matrix(good_params(), 0x20000, None) == L.MA_ERR_NULL
    pm = good_params()
    pm.q = pm.k = 0x10000
    assert lib.ma_matrix(pm, 0x20002, None) == L.MA_ERR_STRIDE         # fp32 output must be 4-byte aligned
    assert lib.ma_matrix(pm, 0x20000, None) == L.MA_ERR_WORKSPACE      # v / out are not needed
    for name in ("fused", "resident", "chained"):
        pm.variant = L.VARIANTS[name]
        assert lib.ma_matrix(pm, 0x20000, None) == L.MA_ERR_UNSUPPORTED
    pm.variant = 99
    assert lib.ma_matrix(pm, 0x20000, None) == L.MA_ERR_VARIANT


def test_select_variant_reports_a_known_variant():
    lib = L.load()
    v = lib.ma_fwd_select_variant(good_params())
    assert v in (L.VARIANTS["generic"], L.VARIANTS["staged"], L.VARIANTS["chained"], L.VARIANTS["resident"], L.VARIANTS["fused"])
    p32 = good_params(dtype_qk=L.MA_F32, dtype_v=L.MA_F32)
    assert lib.ma_fwd_select_variant(p32) in (L.VARIANTS["generic"], L.VARIANTS["staged"], L.VARIANTS["resident"])


def test_auto_resolves_to_a_variant_that_takes_the_problem():
    """Over a random sample of problems: what AUTO resolves to is a variant that accepts the problem when it is asked for
    by name, the answer does not depend on the device-ownership flag unless it is the team kernel, and a kernel name exists."""
    import random
    lib = L.load()
    rnd = random.Random(11)
    seen = set()
    for _ in range(4000):
        E, H = rnd.choice([1, 1, 2, 3, 4, 8, 16, 32, 64]), rnd.choice([1, 2, 3, 4, 6, 8, 12, 16])
        B = rnd.choice([8, 14, 16, 24, 32, 45, 48, 64, 80, 96, 128, 160, 256])
        M = rnd.choice([1, 2, 3, 4, 8, 13, 16, 24, 32, 46, 64, 90, 128, 200])
        N = max(1, M * B - rnd.randint(0, B - 1))
        D = rnd.choice([32, 40, 48, 60, 64, 72, 80, 96, 128])
        if E * H * N * D > 3e8:
            continue
        p = good_params()
        p.E, p.H, p.N, p.D, p.Dv, p.B, p.T = E, H, N, D, D, B, rnd.randint(1, 3)
        p.dtype_qk = p.dtype_v = rnd.choice([L.MA_F16, L.MA_BF16, L.MA_F32])
        for field in ("q_stride", "k_stride", "v_stride", "out_stride"):
            setattr(p, field, (C.c_int64 * 3)(H * N * D, N * D, D))
        p.variant, p.flags = L.VARIANTS["auto"], 0
        shared = lib.ma_fwd_select_variant(p)
        p.flags = L.MA_FLAG_DEVICE_EXCLUSIVE
        owned = lib.ma_fwd_select_variant(p)
        assert shared >= 0 and owned >= 0, (E, H, N, D, B)
        assert shared != L.VARIANTS["fused"]
        assert owned == shared or owned == L.VARIANTS["fused"], (E, H, N, D, B)
        assert lib.ma_fwd_kernel_name(p) is not None
        for v in (shared, owned):
            p.variant = v
            assert lib.ma_fwd_select_variant(p) == v, (E, H, N, D, B, v)
            seen.add(v)
    assert seen == {L.VARIANTS[n] for n in ("generic", "staged", "fused", "resident", "chained")}


def test_kernel_name_follows_the_resolved_variant():
    lib = L.load()

    def name(E, H, N, D, B, dt=L.MA_F16, T=2, variant="auto", flags=0):
        p = good_params()
        p.E, p.H, p.N, p.D, p.Dv, p.B, p.T, p.flags = E, H, N, D, D, B, T, flags
        p.dtype_qk = p.dtype_v = dt
        p.variant = L.VARIANTS[variant]
        for field in ("q_stride", "k_stride", "v_stride", "out_stride"):
            setattr(p, field, (C.c_int64 * 3)(H * N * D, N * D, D))
        got = lib.ma_fwd_kernel_name(p)
        return got.decode() if got is not None else None

    assert name(1, 16, 4096, 64, 64) == "chain_fwd_mfma"
    assert name(1, 16, 4096, 64, 64, flags=L.MA_FLAG_DEVICE_EXCLUSIVE) == "fused_fwd_mfma"
    assert name(64, 12, 256, 64, 16) == "resident_head_mfma"      # the head fits in LDS with its inputs
    assert name(64, 4, 197, 64, 16) == "resident_head_mfma"       # ... a head per compute unit: the widest workgroup
    assert name(64, 12, 197, 64, 16) == "resident_head2_mfma"     # three short heads per compute unit: narrow workgroups, two tiles each
    assert name(128, 12, 64, 64, 16, T=1) == "resident_head_mfma"    # ... and four tiles where four fit a share of the LDS
    assert name(128, 12, 64, 128, 16) == "resident_head2_mfma"        # (not in the 128-column class)
    assert name(16, 12, 512, 64, 32) == "resident_head2_mfma"     # twice that length: the state and one input tile at a time
    assert name(16, 12, 512, 64, 32, T=1) == "resident_head2_mfma"
    assert name(8, 12, 512, 64, 32) == "chain_fwd_mfma"           # ... 96 heads do not fill the device
    assert name(16, 12, 1000, 32, 32, variant="resident") == "resident_fwd_mfma"   # state only
    assert name(1, 16, 4096, 64, 256) == "r_step_mfma"
    assert name(1, 1, 256, 64, 16, dt=L.MA_F32, T=1) == "head_t1_f32"
    assert name(1, 1, 256, 64, 16, dt=L.MA_F32, T=2) == "r_step_f32"
    assert name(8, 8, 197, 64, 16, dt=L.MA_F32) == "head_fwd_f32"
    assert name(1, 16, 4096, 60, 64) == "r_step_kernel"           # D % 8 != 0: the FMA kernels
    assert name(1, 16, 0, 64, 64) is None                         # invalid problem


def test_check_maps_status_to_python_exceptions():
    with pytest.raises(ValueError):
        L.check(L.MA_ERR_SHAPE, "x")
    with pytest.raises(NotImplementedError):
        L.check(L.MA_ERR_UNSUPPORTED, "x")
    with pytest.raises(RuntimeError):
        L.check(L.MA_ERR_WORKSPACE, "x")
    L.check(L.MA_OK, "x")


def test_auto_variant_policy():
    """AUTO: generic when the MFMA kernels do not apply; resident for many heads of small problems
    whose state fits in LDS; the fused kernel for 8 or 16 heads of ~4096 tokens in 64-row problems, but
    only for callers that state that they own the device (MA_FLAG_DEVICE_EXCLUSIVE);
    per-stage launches where the one-launch kernels are at a disadvantage (uneven head counts of 128-row problems, wide heads with many blocks,
    very few long heads); the chained kernel otherwise."""
    lib = L.load()

    def auto(E, H, N, D, B, dt=L.MA_F16, Dv=None, T=2, exclusive=False):
        p = L.FwdParams()
        p.flags = L.MA_FLAG_DEVICE_EXCLUSIVE if exclusive else 0
        p.E, p.H, p.N, p.D, p.Dv, p.B, p.T = E, H, N, D, Dv or D, B, T
        p.dtype_qk = p.dtype_v = dt
        for name, w in (("q_stride", D), ("k_stride", D), ("v_stride", p.Dv), ("out_stride", p.Dv)):
            setattr(p, name, (C.c_int64 * 3)(H * N * w, N * w, w))
        p.eps = 1e-12
        return L.VARIANT_NAMES[lib.ma_fwd_select_variant(p)]

    ex = dict(exclusive=True)
    assert auto(1, 16, 4096, 64, 64, **ex) == "fused"         # 16 heads x 64 workgroups: every head has a full team at once
    assert auto(1, 16, 4096, 64, 64, T=1, **ex) == "fused"
    assert auto(2, 16, 4096, 64, 64, **ex) == "chained"
    assert auto(1, 8, 8192, 64, 64, **ex) == "fused"          # with more than one step also 128 tasks per phase: 8 heads of 8192 tokens,
    assert auto(1, 16, 4096, 64, 128, **ex) == "fused"        # 16 heads of 4096 in 128-row blocks (two positions per workgroup)
    assert auto(1, 8, 8192, 72, 128, **ex) == "fused"         # 8 heads also with head dims up to 80
    # the fused kernel's workgroups wait for each other: without the caller's word that the device is its
    # own, AUTO stays with kernels that make progress beside any other work
    for T_ in (1, 2, 3):
        for shape in ((1, 16, 4096, 64, 64), (1, 8, 8192, 64, 64), (1, 16, 4096, 64, 128), (1, 8, 8192, 72, 128)):
            assert auto(*shape, T=T_) in ("chained", "staged"), (shape, T_)
    assert auto(1, 16, 4096, 64, 64) == "chained"
    assert auto(1, 16, 4096, 64, 64, T=1) == "chained"
    assert auto(1, 16, 4096, 72, 64) == "chained"       # ... 16 heads not
    assert auto(1, 8, 6144, 64, 64) == "chained"        # 96 blocks: the team kernel would run them as 128
    assert auto(1, 8, 8192, 64, 64, T=1) == "staged"    # a single step: two launches
    assert auto(1, 8, 4096, 64, 64, T=1) == "chained"   # ... and teams only when they fill every workgroup slot (16 heads)
    assert auto(1, 8, 2048, 64, 128, T=1) == "staged"   # few 128-row problems: the stage launches run them as halves
    assert auto(1, 16, 2048, 64, 128, T=1) == "chained" # ... 256 of them on 16 heads: one launch again
    assert auto(1, 4, 4096, 64, 128) == "staged"        # more steps: only very few problems, or at most 4 heads
    assert auto(1, 8, 2048, 64, 128) == "chained"
    assert auto(1, 8, 1024, 64, 32) == "chained"        # teams of 16 workgroups: the chained kernel is ahead
    assert auto(1, 12, 4096, 64, 64) == "chained"       # 12 heads do not sit evenly on 8 XCDs: no teams
    assert auto(1, 12, 4096, 64, 64, T=1) == "staged"   # ... and with a single step two launches beat an unbalanced one
    assert auto(1, 16, 16384, 64, 128) == "chained"     # 128-row problems both ways, heads even over the XCDs
    assert auto(1, 12, 16384, 64, 128) == "staged"      # 12 heads on 8 XCDs: uneven
    assert auto(16, 12, 512, 64, 128) == "chained"      # 192 heads of four 128-row blocks: several positions per L / Z tile
    assert auto(16, 12, 384, 64, 96) == "chained"       # ... also for 96-row blocks
    assert auto(1, 16, 8192, 64, 90) == "chained"       # 92 blocks of 90 rows: the chained kernel has the 96-row class too
    assert auto(64, 12, 197, 64, 16) == "resident"
    assert auto(16, 12, 512, 64, 32) == "resident"     # 512-token heads: the state and one input tile at a time in LDS
    assert auto(8, 12, 512, 64, 32) == "chained"       # ... when there are enough heads for the compute units (a head has one to itself)
    assert auto(32, 12, 512, 64, 32) == "resident"     # (384 heads, 1.5 passes over 256 CUs: still 0.85 of the chained kernel's time)
    assert auto(16, 12, 512, 64, 32, T=1) == "resident"
    assert auto(8, 16, 512, 64, 32) == "resident"      # 128 heads: for long heads that are a single strip one way
    assert auto(8, 16, 500, 64, 24) == "chained"
    assert auto(8, 16, 512, 64, 32, T=1) == "chained"
    assert auto(8, 24, 256, 128, 16) == "resident"     # head dim 128: 256 tokens are a two-tile head
    assert auto(8, 24, 272, 128, 16) == "chained"      # ... longer ones only in whole passes over the compute units
    assert auto(8, 32, 272, 128, 16) == "resident"
    assert auto(16, 12, 512, 64, 64) == "chained"      # 64-row blocks (eight waves per workgroup)
    assert auto(16, 12, 768, 64, 32) == "chained"      # beyond two tiles: the one-tile form is no match for the chained kernel here
    assert auto(16, 12, 512, 64, 64) == "chained"      # ... and for problems of one or two strips
    assert auto(32, 12, 256, 64, 64) == "chained"      # 64-row blocks never run resident
    assert auto(16, 12, 256, 64, 32) == "resident"     # 256-token heads fit in LDS with their inputs: from 128 heads on
    assert auto(2, 16, 256, 64, 32) == "chained"       # ... fewer heads of 32-row blocks stay with the chained kernel
    assert auto(1, 2, 256, 64, 16) == "resident"       # ... those of 16-row blocks do not when there is more than one step
    assert auto(1, 2, 256, 64, 16, T=1) == "chained"
    assert auto(16, 12, 197, 64, 16, T=1) == "resident"
    assert auto(8, 16, 1024, 72, 32) == "chained"
    assert auto(4, 16, 16384, 64, 128) == "chained"
    assert auto(512, 16, 1024, 64, 32) == "staged"      # more heads than the chained kernel has flag words for
    assert auto(2, 16, 8192, 64, 64) == "chained"       # 128 blocks of 64 rows (long documents), head dim 64
    assert auto(2, 16, 8192, 128, 64) == "staged"       # ... but not for wide heads
    assert auto(2, 16, 5000, 64, 64) == "chained"       # 79 blocks: the 96-row class
    assert auto(1, 2, 8192, 64, 64) == "staged"         # two long heads would run on two of the eight XCDs
    assert auto(2, 2, 197, 64, 16) == "resident"        # few short heads in 16-row blocks, two steps: whole in LDS
    assert auto(2, 2, 197, 64, 16, T=1) == "chained"    # ... a single step: one launch of the chained kernel
    assert auto(1, 1, 16, 64, 4) == "resident"
    assert auto(1, 1, 16, 64, 4, T=1) == "chained"
    assert auto(1, 16, 4096, 64, 64, dt=L.MA_F32) == "staged"       # fp32 MFMA stage kernels
    assert auto(1, 2, 7600, 48, 128, dt=L.MA_F32) == "staged"
    assert auto(1, 1, 256, 64, 16, dt=L.MA_F32, T=1) == "resident"  # few small fp32 heads, one step: a workgroup per (head, position)
    assert auto(1, 1, 256, 64, 16, dt=L.MA_F32, T=2) == "staged"    # ... more steps: spread over compute units by the stage launches
    assert auto(1, 17, 256, 64, 16, dt=L.MA_F32, T=1) == "staged"   # ... more than 256 workgroups likewise
    assert auto(8, 8, 197, 64, 16, dt=L.MA_F32) == "resident"       # from 64 heads on: one workgroup per head, one launch
    assert auto(64, 12, 197, 64, 16, dt=L.MA_F32) == "resident"
    assert auto(1, 2, 128, 32, 16, dt=L.MA_F32) == "resident"       # ... and for very small heads always
    assert auto(8, 8, 272, 64, 16, dt=L.MA_F32) == "staged"         # 17 blocks
    assert auto(8, 8, 256, 80, 16, dt=L.MA_F32) == "staged"         # head dim above 64
    assert auto(1, 16, 16384, 128, 128, dt=L.MA_F32) == "generic"   # 128 x 128 fp32 tiles do not fit the LDS
    assert auto(1, 16, 4096, 62, 64, dt=L.MA_F32) == "generic"      # D % 4 != 0
    assert auto(1, 16, 4096, 64, 64, Dv=128) == "generic"
    assert auto(1, 16, 4096, 60, 64) == "generic"       # D % 8 != 0
    assert auto(1, 16, 4096, 64, 256) == "staged"       # blocks of 129 .. 256 rows: per-stage launches only
    assert auto(1, 16, 32768, 64, 128) == "staged"      # 129 .. 256 blocks likewise (heads of up to 65536 tokens)
    assert auto(1, 16, 65536, 64, 256) == "staged"
    assert auto(1, 16, 4096, 64, 257) == "generic"      # B > 256
    for name in ("fused", "chained", "resident"):       # the one-launch kernels stop at 128 rows
        p = L.FwdParams()
        p.E, p.H, p.N, p.D, p.Dv, p.B, p.T = 1, 16, 4096, 64, 64, 256, 2
        p.dtype_qk = p.dtype_v = L.MA_F16
        for field in ("q_stride", "k_stride", "v_stride", "out_stride"):
            setattr(p, field, (C.c_int64 * 3)(4096 * 64, 4096 * 64, 64))
        p.eps = 1e-12
        p.variant = L.VARIANTS[name]
        assert lib.ma_fwd_select_variant(p) == L.MA_ERR_UNSUPPORTED
    assert auto(1, 16, 65537, 64, 256) == "generic"     # more than 256 blocks


def good_bwd_params(**kw):
    b = L.BwdParams()
    b.fwd = good_params(**kw)
    for name, inner in (("dout_stride", 16), ("dq_stride", 16), ("dk_stride", 16), ("dv_stride", 16)):
        setattr(b, name, (C.c_int64 * 3)(3 * 50 * inner, 50 * inner, inner))
    return b


def test_backward_workspace_and_argument_checks_precede_any_launch():
    """ma_bwd validates before it launches: everything here runs without a GPU."""
    lib = L.load()
    b = good_bwd_params()
    need = lib.ma_bwd_workspace_bytes(b)
    rows, T, D = 2 * 3 * 7 * 8, 2, 16
    # every step's state (T aL + T-1 aR slots of 16-bit rows), fp32 state gradients and fp32 dq, dk, dv
    assert need >= (2 * T - 1) * rows * D * 2 + 3 * rows * D * 4 + 3 * rows * D * 4
    assert need % 256 == 0
    assert lib.ma_bwd_workspace_bytes(good_bwd_params(T=3)) > need
    assert lib.ma_bwd(None, None) == L.MA_ERR_NULL
    assert lib.ma_bwd(b, None) == L.MA_ERR_NULL                        # q / k / v / dout / dq / dk / dv NULL
    b.fwd.q = b.fwd.k = b.fwd.v = b.dout = b.dq = b.dk = b.dv = 0x10000
    assert lib.ma_bwd(b, None) == L.MA_ERR_WORKSPACE                   # fwd.out is not needed; no workspace
    b.fwd.workspace, b.fwd.workspace_bytes = 0x100000, need - 1
    assert lib.ma_bwd(b, None) == L.MA_ERR_WORKSPACE                   # too small
    b.fwd.workspace, b.fwd.workspace_bytes = 0x100010, need
    assert lib.ma_bwd(b, None) == L.MA_ERR_WORKSPACE                   # misaligned
    b.fwd.workspace = 0x100000
    b.dq = 0x10001                                                     # fp16 pointer must be 2-byte aligned
    assert lib.ma_bwd(b, None) == L.MA_ERR_STRIDE
    b.dq = 0x10000
    for name in ("fused", "resident", "chained"):                      # the T steps run as separate launches
        b.fwd.variant = L.VARIANTS[name]
        assert lib.ma_bwd(b, None) == L.MA_ERR_UNSUPPORTED
        assert lib.ma_bwd_workspace_bytes(b) == 0
    b.fwd.variant = L.VARIANTS["auto"]
    b.dk_stride = (C.c_int64 * 3)(0, 50 * 16, 16)                      # gradient slices of batch entries coincide
    assert lib.ma_bwd(b, None) == L.MA_ERR_STRIDE
    b.dk_stride = (C.c_int64 * 3)(3 * 50 * 16, 50 * 16, 8)             # rows of dk overlap
    assert lib.ma_bwd(b, None) == L.MA_ERR_STRIDE
    bad = good_bwd_params(B=5000)                                      # beyond the backward kernels' block size
    bad.fwd.N = 20000
    bad.fwd.q = bad.fwd.k = bad.fwd.v = bad.dout = bad.dq = bad.dk = bad.dv = 0x10000
    for name in ("q_stride", "k_stride", "v_stride", "out_stride"):
        setattr(bad.fwd, name, (C.c_int64 * 3)(3 * 20000 * 16, 20000 * 16, 16))
    for name in ("dout_stride", "dq_stride", "dk_stride", "dv_stride"):
        setattr(bad, name, (C.c_int64 * 3)(3 * 20000 * 16, 20000 * 16, 16))
    need = lib.ma_bwd_workspace_bytes(bad)
    bad.fwd.workspace, bad.fwd.workspace_bytes = 0x100000, need
    assert need > 0 and lib.ma_bwd(bad, None) == L.MA_ERR_UNSUPPORTED
