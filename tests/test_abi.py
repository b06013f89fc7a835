"""The C ABI library loads without a GPU, exports every symbol the header declares, and
rejects bad arguments before touching the device."""
import ctypes
import os
import re

import pytest

from expertscattergather_amd import _abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "egs_hip.h")
HEADERS = sorted(os.path.join(ROOT, "include", f) for f in os.listdir(os.path.join(ROOT, "include")) if f.endswith(".h"))


def declared_functions():
    names = set()
    for header in HEADERS:
        text = re.sub(r"/\*.*?\*/", "", open(header).read(), flags=re.S)
        names.update(re.findall(r"\b(egs_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


@pytest.fixture(scope="module")
def lib():
    if not _abi.is_built():
        from expertscattergather_amd import build
        build.build()
    return _abi.lib()


def test_header_and_binding_agree(lib):
    names = declared_functions()
    assert len(names) >= 12
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in egs_hip.h but not exported"
    assert sorted(_abi.SIGNATURES) == names, "the ctypes table must list exactly the header's functions"


def test_version_and_status_strings(lib):
    assert lib.egs_abi_version() == _abi.ABI_VERSION == 1
    assert lib.egs_status_string(0) == b"ok"
    assert lib.egs_status_string(_abi.EGS_ERR_BAD_DTYPE) == b"Unknown dtype"
    for code in range(-11, 0):
        assert lib.egs_status_string(code) not in (b"", b"unknown status")
    assert lib.egs_status_string(-99) == b"unknown status"
    assert lib.egs_last_hip_error() == b""


def test_enums_match_header():
    text = open(HEADER).read()
    for name, value in (("EGS_F32", _abi.F32), ("EGS_F16", _abi.F16), ("EGS_BF16", _abi.BF16),
                        ("EGS_FP8_E4M3", _abi.FP8_E4M3), ("EGS_IND_I16", _abi.IND_I16), ("EGS_IND_I32", _abi.IND_I32),
                        ("EGS_IND_I64", _abi.IND_I64), ("EGS_IND_U8", _abi.IND_U8), ("EGS_W_EIJ", _abi.W_EIJ),
                        ("EGS_W_EJI", _abi.W_EJI), ("EGS_SCATTER_DETERMINISTIC", _abi.SCATTER_DETERMINISTIC),
                        ("EGS_SCATTER_ATOMIC", _abi.SCATTER_ATOMIC), ("EGS_SCATTER_COMPACT", _abi.SCATTER_COMPACT), ("EGS_OP_GATHER_BACKWARD", _abi.OP_GATHER_BACKWARD),
                        ("EGS_OP_SCATTER_BACKWARD", _abi.OP_SCATTER_BACKWARD), ("EGS_ERR_HIP", _abi.EGS_ERR_HIP)):
        m = re.search(rf"\b{name}\s*=\s*(-?\d+)", text)
        assert m and int(m.group(1)) == value, name


def test_argument_validation_needs_no_gpu(lib):
    d = _abi.Dims(2, 8, 3, 4, 16, 8)
    p = 0x1000  # never dereferenced: every call below must fail validation first
    g = lib.egs_gather_gemm
    assert g(None, p, p, p, None, d, 128, 16, 2, 2, 2, 0, None) == -1          # null X
    assert g(p, p, p, p, None, None, 128, 16, 2, 2, 2, 0, None) == -1          # null dims
    assert g(p, p, p, p, None, d, 128, 16, 7, 7, 2, 0, None) == -3             # unknown dtype
    assert g(p, p, p, p, None, d, 128, 16, 2, 2, 9, 0, None) == -3             # unknown index dtype
    assert g(p, p, p, p, None, d, 128, 16, 2, 2, 2, 5, None) == -4             # unknown layout
    assert g(p, p, p, p, None, d, 128, 16, 2, 0, 2, 0, None) == -9             # mixed dtypes
    assert g(p, p, p, p, None, d, 128, 16, 2, 3, 2, 0, None) == -1             # fp8 weights without scales
    assert g(p, p, p, p, None, d, 128, 8, 2, 2, 2, 0, None) == -10             # token stride < row
    assert g(p + 1, p, p, p, None, d, 128, 16, 2, 2, 2, 0, None) == -7         # misaligned
    bad = _abi.Dims(2, 8, -3, 4, 16, 8)
    assert g(p, p, p, p, None, bad, 128, 16, 2, 2, 2, 0, None) == -2
    sc = lib.egs_gemm_scatter
    assert sc(p, p, p, p, p, 1 << 30, d, 2, 2, 1, 7, None) == -5               # unknown mode
    assert sc(p, p, p, p, None, 0, d, 2, 2, 1, 0, None) == -6                  # workspace missing
    need = lib.egs_workspace_bytes(_abi.OP_GEMM_SCATTER, 0, d, 2)
    assert need > 0
    assert sc(p, p, p, p, 0x2000, need - 1, d, 2, 2, 1, 0, None) == -6          # workspace too small
    assert sc(p, p, p, p, 0x2001, need, d, 2, 2, 1, 0, None) == -7              # workspace not 256-byte aligned
    dw = lib.egs_dw
    assert dw(p, p, p, None, None, 0, d, 128, 16, 2, 2, 2, 0, None) == -1
    assert lib.egs_validate_indices(p, 2, -1, 8, p, None) == -2
    assert lib.egs_validate_indices(None, 2, 4, 8, p, None) == -1
    # empty problems succeed without any pointer
    empty = _abi.Dims(0, 8, 3, 4, 16, 8)
    assert g(None, None, None, None, None, empty, 0, 0, 2, 2, 2, 0, None) == 0
    assert sc(None, None, None, None, None, 0, empty, 2, 2, 1, 0, None) == 0


def test_builtin_scratch_entry_point_checks_sizes_first(lib):
    # sizes whose partial sums do not fit the built-in buffer are refused before any pointer is looked at
    big = _abi.Dims(16, 512, 4, 256, 1024, 1024)
    assert lib.egs_workspace_bytes(_abi.OP_DW, 0, big, _abi.BF16) > _abi.BUILTIN_SCRATCH_BYTES
    f = lib.egs_dw_builtin_scratch
    p = 0x1000
    assert f(p, p, p, p, big, 512 * 1024, 1024, 2, 2, 2, 0, None) == _abi.EGS_ERR_SCRATCH_LIMIT == -11
    d = _abi.Dims(2, 8, 3, 4, 16, 8)
    assert f(p, p, p, None, d, 128, 16, 2, 2, 2, 0, None) == -1               # null output
    assert f(p, p, p, p, d, 128, 16, 7, 2, 2, 0, None) == -3                  # unknown dtype
    assert f(p, p, p, p, d, 128, 16, 2, 2, 2, 5, None) == -4                  # unknown layout
    text = open(HEADER).read()
    m = re.search(r"#define\s+EGS_BUILTIN_SCRATCH_BYTES\s+\((\d+)u\s*<<\s*(\d+)\)", text)
    assert m and int(m.group(1)) << int(m.group(2)) == _abi.BUILTIN_SCRATCH_BYTES


def test_workspace_sizes_are_consistent(lib):
    wb = lib.egs_workspace_bytes
    # the default shape in bf16 runs on kernels that need no scratch at all: the one-kernel scatter keeps its product rows
    # in LDS and the one-pass weight gradient has no partial sums
    d = _abi.Dims(64, 256, 32, 32, 128, 64)
    for op in (_abi.OP_GATHER_GEMM, _abi.OP_GEMM_SCATTER, _abi.OP_DW, _abi.OP_GATHER_BACKWARD, _abi.OP_SCATTER_BACKWARD):
        assert wb(op, 0, d, _abi.BF16) == 0 and wb(op, 1, d, _abi.BF16) == 0
    # more picks per batch element than the one-kernel scatter holds: routing table + fp32 product rows (deterministic) or
    # rows in the element type (atomic mode with a 16-bit type); fewer experts than the one-pass weight gradient wants: splits
    assert wb(_abi.OP_GEMM_SCATTER, 0, _abi.Dims(16, 256, 8, 256, 128, 64), _abi.BF16) == 0   # 2048 picks: two passes, still no scratch
    d = _abi.Dims(16, 256, 8, 640, 128, 64)
    rows = 16 * 8 * 640 * 128
    det, fast, dw = wb(_abi.OP_GEMM_SCATTER, 0, d, _abi.BF16), wb(_abi.OP_GEMM_SCATTER, 1, d, _abi.BF16), wb(_abi.OP_DW, 0, d, _abi.BF16)
    assert rows * 4 <= det <= rows * 4 * 1.1 and rows * 2 <= fast <= rows * 2 * 1.1 and dw > 0
    assert wb(_abi.OP_GATHER_BACKWARD, 0, d, _abi.BF16) == det + dw
    assert wb(_abi.OP_SCATTER_BACKWARD, 0, d, _abi.BF16) == dw
    assert wb(_abi.OP_GEMM_SCATTER, 1, d, _abi.F32) == 0                      # fp32 atomic mode adds into the output
    assert det % 256 == 0 and dw % 256 == 0
    # compact mode (16-bit types, reduction 32 / 64 / 128, T <= 1024): no workspace at all for the scatter
    assert wb(_abi.OP_GEMM_SCATTER, _abi.SCATTER_COMPACT, d, _abi.BF16) == 0
    assert wb(_abi.OP_GATHER_BACKWARD, _abi.SCATTER_COMPACT, d, _abi.BF16) == dw
    assert wb(_abi.OP_GEMM_SCATTER, _abi.SCATTER_COMPACT, d, _abi.F32) == wb(_abi.OP_GEMM_SCATTER, 0, d, _abi.F32)   # fp32: as deterministic
    assert wb(_abi.OP_GEMM_SCATTER, _abi.SCATTER_COMPACT, _abi.Dims(8, 4096, 128, 256, 1024, 256), _abi.BF16) == \
        wb(_abi.OP_GEMM_SCATTER, 0, _abi.Dims(8, 4096, 128, 256, 1024, 256), _abi.BF16)                              # T > 1024
    assert wb(99, 0, d, 2) == 0 and wb(_abi.OP_DW, 0, d, 9) == 0
    # an entry point checks the workspace against the kernels its actual operands select: an output that is not
    # 16-byte aligned cannot take the one-kernel scatter and is refused without the general path's workspace
    d = _abi.Dims(64, 256, 32, 32, 128, 64)
    p = 0x1000
    assert lib.egs_gemm_scatter(p, p, p, p + 2, None, 0, d, _abi.BF16, _abi.IND_I64, _abi.W_EJI, 0, None) == -6


def test_check_raises_like_the_reference():
    with pytest.raises(ValueError, match="Unknown dtype"):
        _abi.check(_abi.EGS_ERR_BAD_DTYPE, "x")
    with pytest.raises(RuntimeError, match="workspace"):
        _abi.check(-6, "x")
    _abi.check(0, "x")


def test_inference_block_entry_point_validates_without_a_gpu(lib):
    ok = _abi.Dims(64, 256, 32, 32, 128, 64)
    assert lib.egs_expert_mlp_supported(ok, _abi.BF16) == 1 and lib.egs_expert_mlp_supported(ok, _abi.F16) == 1
    assert lib.egs_expert_mlp_supported(ok, _abi.F32) == 0                                         # 16-bit types only
    assert lib.egs_expert_mlp_supported(_abi.Dims(64, 256, 32, 32, 128, 128), _abi.BF16) == 0      # J = 128
    assert lib.egs_expert_mlp_supported(_abi.Dims(64, 256, 32, 64, 128, 64), _abi.BF16) == 0       # 2048 picks per batch element
    assert lib.egs_expert_mlp_supported(_abi.Dims(64, 256, 32, 32, 96, 64), _abi.BF16) == 0        # I not 32 / 64 / 128
    p = 0x1000
    args = (p, p, p, p, p)
    assert lib.egs_expert_mlp_forward(*args, ok, 256 * 128, 128, _abi.BF16, _abi.IND_I64, 9, None) == -5    # unknown activation
    assert lib.egs_expert_mlp_forward(*args, ok, 256 * 128, 128, 7, _abi.IND_I64, _abi.ACT_RELU, None) == _abi.EGS_ERR_BAD_DTYPE
    assert lib.egs_expert_mlp_forward(*args, ok, 256 * 128, 64, _abi.BF16, _abi.IND_I64, _abi.ACT_RELU, None) == -10   # token stride < I
    assert lib.egs_expert_mlp_forward(None, p, p, p, p, ok, 256 * 128, 128, _abi.BF16, _abi.IND_I64, _abi.ACT_RELU, None) == -1
    assert lib.egs_expert_mlp_forward(*args, _abi.Dims(64, 256, 32, 32, 128, 128), 256 * 128, 128, _abi.BF16, _abi.IND_I64,
                                      _abi.ACT_RELU, None) == _abi.EGS_ERR_UNSUPPORTED
    assert lib.egs_expert_mlp_forward(p, p, p, p, p + 2, ok, 256 * 128, 128, _abi.BF16, _abi.IND_I64, _abi.ACT_RELU,
                                      None) == _abi.EGS_ERR_UNSUPPORTED                                # output off the 16-byte grid


def test_routing_table_entry_points_validate_without_a_gpu(lib):
    tb = lib.egs_routing_table_bytes
    d = _abi.Dims(64, 256, 32, 32, 128, 64)
    seg, perm = -(-64 * 257 * 4 // 256) * 256, 64 * 32 * 32 * 4
    assert tb(d, _abi.BF16) == tb(d, _abi.F16) == tb(d, _abi.F32) == seg + perm     # [B][T + 1] offsets, then [B][E * K] picks
    wide = _abi.Dims(64, 256, 32, 32, 128, 128)
    assert tb(wide, _abi.F32) == 0 and tb(wide, _abi.BF16) == seg + perm     # fp32 one-kernel scatter: reduction 32 / 64 only
    assert tb(_abi.Dims(64, 256, 48, 32, 128, 64), _abi.BF16) > 0            # scatter in passes, up to 2048 picks
    assert tb(_abi.Dims(64, 256, 96, 32, 128, 64), _abi.BF16) == 0           # ... beyond that it sorts for itself
    assert tb(_abi.Dims(16, 256, 8, 640, 128, 64), _abi.BF16) == 0           # general path builds its own in the workspace
    assert tb(None, _abi.BF16) == 0 and tb(d, 9) == 0
    p, t, nb = 0x1000, 0x4000, seg + perm
    gf, sf, gb = lib.egs_expert_gather_forward_table, lib.egs_expert_scatter_forward_table, lib.egs_expert_gather_backward_table
    ld = (256 * 128, 128)
    assert gf(p, p, p, p, t, nb - 1, d, *ld, _abi.BF16, _abi.IND_I64, None) == -6            # table too small
    assert gf(p, p, p, p, t + 16, nb, d, *ld, _abi.BF16, _abi.IND_I64, None) == -7           # not 256-byte aligned
    assert gf(p, p, p, p, t, nb, wide, *ld, _abi.F32, _abi.IND_I64, None) == _abi.EGS_ERR_UNSUPPORTED
    assert gf(None, p, p, p, t, nb, d, *ld, _abi.BF16, _abi.IND_I64, None) == -1
    assert sf(p, p, p, t, nb - 1, p, None, 0, d, _abi.BF16, _abi.IND_I64, 0, None) == -6
    assert sf(p, p, p, t, nb, p, None, 0, _abi.Dims(64, 256, 32, 32, 256, 64), _abi.F32, _abi.IND_I64, 0, None) == _abi.EGS_ERR_UNSUPPORTED
    assert sf(p, p, p, t, nb, p, None, 0, d, _abi.BF16, _abi.IND_I64, 7, None) == -5          # unknown mode
    assert gb(p, p, p, t, nb - 1, p, p, p, None, 0, d, *ld, _abi.BF16, _abi.IND_I64, 0, None) == -6
    assert gb(p, p, p, t + 16, nb, p, p, p, None, 0, d, *ld, _abi.BF16, _abi.IND_I64, 0, None) == -7
    big = _abi.Dims(64, 256, 96, 32, 128, 64)
    assert gb(p, p, p, t, nb, p, p, p, None, 0, big, *ld, _abi.BF16, _abi.IND_I64, 0, None) == _abi.EGS_ERR_UNSUPPORTED


def test_integer_call_module_reaches_the_same_entry_points(lib):
    fast = _abi.pycall()
    assert fast is not None, "expertscattergather_amd/_egs_pycall*.so is part of the build"
    assert fast.abi_version() == _abi.ABI_VERSION
    p, dims, ld = 0x1000, (64, 256, 32, 32, 128, 64), (256 * 128, 128)
    d = _abi.Dims(*dims)
    # the same refusals as through ctypes, before any HIP call
    assert fast.gather_forward(0, p, p, p, 0, 0, *dims, *ld, _abi.BF16, _abi.IND_I64, 0) == -1 == \
        lib.egs_expert_gather_forward(None, p, p, p, d, *ld, _abi.BF16, _abi.IND_I64, None)
    assert fast.gather_forward(p, p, p, p, 0, 0, *dims, *ld, 7, _abi.IND_I64, 0) == _abi.EGS_ERR_BAD_DTYPE
    assert fast.gather_forward(p, p, p, p, 0x4000, 16, *dims, *ld, _abi.BF16, _abi.IND_I64, 0) == -6       # table too small
    assert fast.gather_forward(p, p, p, p, 0, 0, 64, 256, -3, 32, 128, 64, *ld, _abi.BF16, _abi.IND_I64, 0) == -2   # negative size
    assert fast.scatter_forward(p, p, p, 0, 0, p, 0, 0, *dims, _abi.BF16, _abi.IND_I64, 7, 0) == -5          # unknown mode
    assert fast.scatter_forward(p, p, p, 0, 0, p + 2, 0, 0, *dims, _abi.BF16, _abi.IND_I64, 0, 0) == -6      # general path, no workspace
    assert fast.gather_backward(p, p, p, 0x4000, 16, p, p, p, 0, 0, *dims, *ld, _abi.BF16, _abi.IND_I64, 0, 0) == -6
    assert fast.gather_backward(p, p, p, 0, 0, p, p, 0, 0, 0, *dims, *ld, _abi.BF16, _abi.IND_I64, 0, 0) == -1    # null grad_W
    assert fast.scatter_backward(p, p, p, p, p, 0, 0, 0, *dims, *ld, _abi.BF16, _abi.IND_I64, 0) == -1
    assert fast.scatter_backward(p, p, p, p, p, p, 0, 0, *dims, 256 * 128, 64, _abi.BF16, _abi.IND_I64, 0) == -10  # token stride < row
    empty = (0, 256, 32, 32, 128, 64)
    assert fast.gather_forward(0, 0, 0, 0, 0, 0, *empty, 0, 0, _abi.BF16, _abi.IND_I64, 0) == 0
    with pytest.raises(TypeError):
        fast.gather_forward(p, p, p)
    with pytest.raises(TypeError):
        fast.scatter_forward(p, p, p, None, 0, p, 0, 0, *dims, _abi.BF16, _abi.IND_I64, 0, 0)


def test_header_compiles_as_c99_and_the_library_links_from_c(lib, tmp_path):
    import shutil
    import subprocess
    cc = shutil.which("gcc") or shutil.which("cc")
    if cc is None:
        pytest.skip("no C compiler")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    libdir = os.path.dirname(_abi.LIB_PATH)
    exe = str(tmp_path / "abi_from_c")
    build = subprocess.run([cc, "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(root, "include"),
                            os.path.join(root, "tests", "c", "abi_from_c.c"), "-L", libdir, "-legs_hip", f"-Wl,-rpath,{libdir}", "-o", exe],
                           capture_output=True, text=True)
    assert build.returncode == 0, build.stderr
    run = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert run.returncode == 0 and run.stdout.startswith("ok"), run.stdout + run.stderr


def test_planning_functions_survive_arbitrary_sizes(lib):
    # the size queries run the same selection code as the entry points: whatever the sizes, they answer (no
    # division by zero, no overflow into nonsense), in multiples of 256 bytes, and agree with themselves
    import random
    rnd = random.Random(3)
    pick = lambda: rnd.choice([0, 1, 2, 3, 7, 8, 16, 31, 32, 33, 64, 100, 128, 256, 300, 512, 1024, 4096, 65536, 2 ** 31 - 1])
    for _ in range(3000):
        d = _abi.Dims(pick(), pick(), pick(), pick(), pick(), pick())
        for dt in (_abi.F32, _abi.F16, _abi.BF16):
            sizes = [lib.egs_workspace_bytes(op, mode, d, dt) for op in range(5) for mode in (0, 1)]
            assert all(s % 256 == 0 for s in sizes), (tuple(getattr(d, f) for f in "BTEKIJ"), sizes)
            assert sizes == [lib.egs_workspace_bytes(op, mode, d, dt) for op in range(5) for mode in (0, 1)]
            assert lib.egs_expert_mlp_supported(d, dt) in (0, 1)
            assert lib.egs_routing_table_bytes(d, dt) % 256 == 0
        assert lib.egs_gather_gemm_fp8act_workspace_bytes(d) % 256 == 0
    assert lib.egs_workspace_bytes(1, 0, None, _abi.BF16) == 0 and lib.egs_expert_mlp_supported(None, _abi.BF16) == 0
