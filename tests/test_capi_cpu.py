"""Host-side checks of the C ABI that need no GPU: the library loads, exports
every declared symbol, and its size arithmetic and argument validation (which
run before any HIP call) behave as documented."""
import ctypes as C
import os
import re

import pytest

from luminal_amd import capi, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "luminal_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lhip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = capi.load_library()
    names = declared_symbols()
    assert len(names) >= 15
    for n in names:
        assert hasattr(lib, n), f"{n} declared in luminal_hip.h but not exported"
    # and the binding covers every declaration
    assert sorted(capi.SIGNATURES) == names


def test_status_strings():
    lib = capi.load_library()
    assert lib.lhip_status_string(0) == b"LHIP_OK"
    assert lib.lhip_status_string(2) == b"LHIP_ERR_INVALID_SHAPE"
    assert lib.lhip_status_string(99) == b"LHIP_ERR_UNKNOWN"
    assert re.fullmatch(rb"\d+\.\d+\.\d+", lib.lhip_version())


def test_size_laws():
    lib = capi.load_library()
    for name, (n, k) in synth.LLAMA3_8B_PROJ.items():
        raw = lib.lhip_q8_0_raw_nbytes(n, k)
        assert raw == n * k + n * k // 16, name  # examples/llama/src/loader.rs:128
        assert lib.lhip_q8_0_planar_nbytes(n, k) == raw  # same bytes, re-arranged
        assert lib.lhip_q8_0_planar_scale_offset(n, k) == n * k
    # quant plane padded to 256 B
    assert lib.lhip_q8_0_planar_scale_offset(3, 32) == 256
    assert lib.lhip_q8_0_planar_nbytes(3, 32) == 256 + 6
    # invalid shapes give 0
    for n, k in [(0, 32), (4, 0), (4, 31), (4, 48), (-1, 32), (1 << 31, 32)]:
        assert lib.lhip_q8_0_raw_nbytes(n, k) == 0
        assert lib.lhip_q8_0_planar_nbytes(n, k) == 0


def test_gemm_plans_show_in_the_workspace_size():
    """lhip_q8_0_matmul_bf16_workspace_nbytes is the f32 planes of the plan the plain entry point takes (host code
    only): K slices of the whole product, of the column tiles a last partly filled round of 256 workgroups would hold,
    of the weight-streaming kernel, or none."""
    lib = capi.load_library()
    ws = lib.lhip_q8_0_matmul_bf16_workspace_nbytes
    # 8 x 112 tiles of 256 x 128 = 3.5 rounds: 96 column tiles in whole rounds, 16 (2048 columns) in two K slices
    assert ws(2048, 14336, 4096, 0) == 2 * 2048 * 2048 * 4
    assert ws(2048, 14336, 4096, 2) == 2 * 2048 * 2048 * 4
    # 8 x 1002 tiles: 992 column tiles in 31 whole rounds, the other 10 (1280 columns) in two K slices
    assert ws(2048, 128256, 4096, 0) == 2 * 2048 * (128256 - 992 * 128) * 4
    # 4 x 81 tiles with a ragged last one: 64 column tiles in one round, 17 (2084 columns) in two K slices
    assert ws(1024, 80 * 128 + 36, 2048, 1) == 2 * 1024 * 2084 * 4
    # exactly one round, or 224 tiles that K slices cannot bring to 256: one launch, no planes
    assert ws(2048, 4096, 4096, 0) == 0
    assert ws(512, 14336, 4096, 0) == 0
    # fewer tiles than CUs and a long K: slices of the whole product (64 tiles x 4 slices)
    assert ws(512, 4096, 14336, 0) == 4 * 512 * 4096 * 4
    # at most 128 rows: the weight-streaming kernel, two K slices over strips that fill the chip
    assert ws(128, 14336, 4096, 0) == 2 * 128 * 14336 * 4
    assert ws(128, 128256, 4096, 0) == 0
    # no such product
    assert ws(128, 14336, 4100, 0) == 0 and ws(0, 14336, 4096, 0) == 0 and ws(128, 14336, 4096, 3) == 0


def test_argument_validation_before_any_device_work():
    lib = capi.load_library()
    ok_ptr = 0x1000  # never dereferenced: validation fails first
    assert lib.lhip_q8_0_matmul_f32(None, ok_ptr, ok_ptr, 1, 32, 32, None) == capi.LHIP_ERR_NULL_PTR
    assert lib.lhip_q8_0_matmul_f32(ok_ptr, None, ok_ptr, 1, 32, 32, None) == capi.LHIP_ERR_NULL_PTR
    assert lib.lhip_q8_0_matmul_f32(ok_ptr, ok_ptr, None, 1, 32, 32, None) == capi.LHIP_ERR_NULL_PTR
    assert lib.lhip_q8_0_matmul_f32(ok_ptr, ok_ptr, ok_ptr, 1, 32, 33, None) == capi.LHIP_ERR_INVALID_SHAPE
    assert lib.lhip_q8_0_matmul_f32(ok_ptr, ok_ptr, ok_ptr, 0, 32, 32, None) == capi.LHIP_ERR_INVALID_SHAPE
    assert lib.lhip_q8_0_matmul_f32(ok_ptr, ok_ptr, ok_ptr, 1, 0, 32, None) == capi.LHIP_ERR_INVALID_SHAPE
    assert lib.lhip_q8_0_matmul_f32(ok_ptr + 16, ok_ptr, ok_ptr, 1, 32, 32, None) == capi.LHIP_ERR_MISALIGNED
    assert lib.lhip_q8_0_matmul_f32(ok_ptr, ok_ptr + 4, ok_ptr, 1, 32, 32, None) == capi.LHIP_ERR_MISALIGNED
    assert lib.lhip_q8_0_repack(None, ok_ptr, 1, 32, None) == capi.LHIP_ERR_NULL_PTR
    assert lib.lhip_q8_0_repack(ok_ptr + 1, ok_ptr, 1, 32, None) == capi.LHIP_ERR_MISALIGNED
    assert lib.lhip_q8_0_repack(ok_ptr, ok_ptr + 128, 1, 32, None) == capi.LHIP_ERR_MISALIGNED
    assert lib.lhip_q8_0_unpack(ok_ptr, ok_ptr, 1, 40, None) == capi.LHIP_ERR_INVALID_SHAPE
    assert lib.lhip_q8_0_dequant_f32(ok_ptr, None, 1, 32, None) == capi.LHIP_ERR_NULL_PTR
    assert lib.lhip_q8_0_gather_f32(ok_ptr, ok_ptr, ok_ptr, 0, 4, 32, None) == capi.LHIP_ERR_INVALID_SHAPE
    assert lib.lhip_q8_0_gather_f32(ok_ptr, None, ok_ptr, 1, 4, 32, None) == capi.LHIP_ERR_NULL_PTR
    out = C.c_void_p()
    assert lib.lhip_malloc(None, 16) == capi.LHIP_ERR_NULL_PTR
    assert lib.lhip_malloc(C.byref(out), 0) == capi.LHIP_ERR_INVALID_SHAPE
    assert lib.lhip_free(None) == capi.LHIP_OK
    assert lib.lhip_memcpy_h2d(None, ok_ptr, 4, None) == capi.LHIP_ERR_NULL_PTR


def test_check_raises_with_status_name():
    with pytest.raises(capi.LhipError) as e:
        capi.check(capi.LHIP_ERR_INVALID_SHAPE, "somewhere")
    assert "LHIP_ERR_INVALID_SHAPE" in str(e.value) and e.value.status == 2


def test_missing_library_fails_loudly(tmp_path):
    with pytest.raises(capi.LhipError):
        capi.load_library(str(tmp_path / "nope.so"))


def test_gemv_byte_model():
    # figures the roofline fraction is computed from
    assert synth.q8_0_gemv_bytes(4096, 4096) == 17858560
    assert synth.q8_0_gemv_bytes(1024, 4096) == 4476928
    assert synth.q8_0_gemv_bytes(14336, 4096) == 62464000
    assert synth.q8_0_gemv_bytes(4096, 14336) == 62464000
    assert synth.q8_0_gemv_bytes(128256, 4096) == 558699520


def test_rust_bindings_name_exported_symbols_with_the_header_arity():
    """crates/luminal_hip/src/ffi.rs is not compiled here (no Rust toolchain): at least every function it declares
    must exist in the library with as many parameters as the header gives it."""
    text = open(os.path.join(ROOT, "crates", "luminal_hip", "src", "ffi.rs")).read()
    block = text[text.index('extern "C" {'):]
    block = block[: block.index("\n}")]
    rust = {m.group(1): m.group(2) for m in re.finditer(r"pub fn (lhip_[a-z0-9_]+)\(([^)]*)\)", block)}
    assert len(rust) >= 12
    header = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    lib = capi.load_library()
    for name, params in rust.items():
        assert hasattr(lib, name), name
        decl = re.search(r"\b%s\s*\(([^)]*)\)" % name, header)
        assert decl, name
        c_params = [p for p in decl.group(1).split(",") if p.strip() not in ("", "void")]
        rust_params = [p for p in params.split(",") if p.strip()]
        assert len(c_params) == len(rust_params), name


def kernel_names_in_header():
    text = open(os.path.join(ROOT, "include", "luminal_hip_kernels.h")).read()
    macro = text[text.index("#define LHIP_KERNEL_Q8_0_GEMV_NAMES"):]
    macro = macro[: macro.index("\n\n")]
    return re.findall(r'"(lhip_kernel_[a-z0-9_]+)"', macro)


def test_code_object_holds_every_kernel_the_header_names():
    names = kernel_names_in_header()
    assert len(names) == 16 and len(set(names)) == 16
    blob = open(os.path.join(ROOT, "luminal_amd", "luminal_hip_kernels.hsaco"), "rb").read()
    assert blob[:4] == b"\x7fELF"
    for n in names:
        assert n.encode() + b".kd\0" in blob, n  # kernel descriptor symbol


def test_kernel_plan_names_a_kernel_of_the_code_object_and_its_launch_shape():
    import ctypes as C
    lib = capi.load_library()
    names = set(kernel_names_in_header())

    def plan(n, k, f16):
        name = C.create_string_buffer(64)
        grid, block, lds = (C.c_uint32 * 3)(), (C.c_uint32 * 3)(), C.c_uint32()
        st = lib.lhip_q8_0_gemv_kernel_plan(n, k, f16, name, 64, grid, block, C.byref(lds))
        return st, name.value.decode(), list(grid), list(block), lds.value

    assert plan(4096, 4096, 0) == (0, "lhip_kernel_q8_0_gemv_f32_pipe_r1s2w4", [768, 1, 1], [256, 1, 1], 16384)
    assert plan(128256, 4096, 1) == (0, "lhip_kernel_q8_0_gemv_f16_pipe_r2s4w4", [256, 1, 1], [256, 1, 1], 16384)
    assert plan(4096, 14336, 0) == (0, "lhip_kernel_q8_0_gemv_f32_pipe_r1s2w16", [256, 1, 1], [1024, 1, 1], 57344)
    assert plan(37, 96, 0) == (0, "lhip_kernel_q8_0_gemv_f32_oneshot_r1", [10, 1, 1], [256, 1, 1], 0)
    for n, k in [(1, 32), (100, 1024), (5000, 3072), (8192, 1056), (300, 15360), (40000, 8192), (7, 20480)]:
        for f16 in (0, 1):
            st, name, grid, block, lds = plan(n, k, f16)
            assert st == 0 and name in names
            assert block[0] % 64 == 0 and block[0] <= 1024 and grid[0] >= 1 and lds <= 65536
            assert ("pipe" in name) == (lds == 4 * k)
    assert plan(4096, 48, 0)[0] == capi.LHIP_ERR_INVALID_SHAPE
    name = C.create_string_buffer(8)
    grid, block, lds = (C.c_uint32 * 3)(), (C.c_uint32 * 3)(), C.c_uint32()
    assert lib.lhip_q8_0_gemv_kernel_plan(64, 64, 0, name, 8, grid, block, C.byref(lds)) == capi.LHIP_ERR_INVALID_SHAPE
    assert lib.lhip_q8_0_gemv_kernel_plan(64, 64, 0, None, 64, grid, block, C.byref(lds)) == capi.LHIP_ERR_NULL_PTR
