"""The kernel-level route: luminal_hip_kernels.hsaco loaded and launched with the HIP module API alone
(hipModuleLoad / hipModuleGetFunction / hipModuleLaunchKernel through ctypes), the way the reference's host code
drives its kernels (crates/luminal_cuda/src/lib.rs:237-258, crates/luminal_cuda/src/quantized.rs:131-148), against
the library's own entry points: same bits.
"""
import ctypes as C
import os

import numpy as np
import pytest

torch = pytest.importorskip("torch")

from luminal_amd import capi, synth  # noqa: E402
from luminal_amd.quantized import Q8Weight  # noqa: E402

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
MODULE_PATH = os.path.join(os.path.dirname(capi.LIB_PATH), "luminal_hip_kernels.hsaco")


def hip_runtime():
    """The HIP runtime this process already uses (the one torch and libluminal_hip.so are bound to)."""
    capi.load_library()
    torch.zeros(1, device=DEV)
    with open("/proc/self/maps") as f:
        paths = {line.split()[-1] for line in f if "libamdhip64" in line}
    assert len(paths) == 1, paths
    hip = C.CDLL(paths.pop())
    hip.hipModuleLoad.argtypes = [C.POINTER(C.c_void_p), C.c_char_p]
    hip.hipModuleGetFunction.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_char_p]
    hip.hipModuleLaunchKernel.argtypes = [C.c_void_p] + [C.c_uint] * 7 + [C.c_void_p, C.POINTER(C.c_void_p), C.c_void_p]
    hip.hipModuleUnload.argtypes = [C.c_void_p]
    hip.hipDeviceSynchronize.argtypes = []
    return hip


@pytest.fixture(scope="module")
def module():
    assert os.path.exists(MODULE_PATH), "build it with `python -m luminal_amd.build`"
    hip = hip_runtime()
    mod = C.c_void_p()
    assert hip.hipModuleLoad(C.byref(mod), MODULE_PATH.encode()) == 0
    yield hip, mod
    assert hip.hipDeviceSynchronize() == 0
    assert hip.hipModuleUnload(mod) == 0


def plan(n, k, f16):
    name = C.create_string_buffer(64)
    grid, block, lds = (C.c_uint32 * 3)(), (C.c_uint32 * 3)(), C.c_uint32()
    capi.check(capi.load_library().lhip_q8_0_gemv_kernel_plan(n, k, int(f16), name, 64, grid, block, C.byref(lds)),
               "lhip_q8_0_gemv_kernel_plan")
    return name.value, list(grid), list(block), lds.value


def launch(hip, mod, name, grid, block, lds, w, x, y, n, k):
    fn = C.c_void_p()
    assert hip.hipModuleGetFunction(C.byref(fn), mod, name) == 0, name
    off = capi.load_library().lhip_q8_0_planar_scale_offset(n, k)
    vals = [C.c_void_p(w.planar.data_ptr()), C.c_void_p(w.planar.data_ptr() + off), C.c_void_p(x.data_ptr()),
            C.c_void_p(y.data_ptr()), C.c_int32(n), C.c_int32(k)]
    args = (C.c_void_p * len(vals))(*[C.cast(C.pointer(v), C.c_void_p) for v in vals])
    stream = torch.cuda.current_stream().cuda_stream
    assert hip.hipModuleLaunchKernel(fn, *grid, *block, lds, C.c_void_p(stream), args, None) == 0, name
    torch.cuda.synchronize()


# (n, k, rows): the Llama-3-8B projections (lm_head runs the two-row kernel), short and long K, ragged shapes
CASES = [
    (4096, 4096, 1), (1024, 4096, 2), (14336, 4096, 1), (4096, 14336, 1), (128256, 4096, 1),
    (37, 96, 3), (257, 1024, 2), (130, 3072, 1), (64, 15360, 1), (9000, 1056, 1), (5000, 32, 2), (33, 20480, 1),
]


@pytest.mark.parametrize("f16", [False, True], ids=["f32", "f16"])
@pytest.mark.parametrize("n,k,m", CASES)
def test_module_launch_equals_the_library_call(module, n, k, m, f16):
    hip, mod = module
    lib = capi.load_library()
    qs, d = synth.q8_0_random(n, k, seed=n + 3 * k)
    w = Q8Weight.from_raw(synth.q8_0_raw_blocks(qs, d), n, k, DEV)
    rng = np.random.default_rng(n * 7 + k)
    dt = torch.float16 if f16 else torch.float32
    x = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).to(DEV).to(dt)
    name, grid, block, lds = plan(n, k, f16)
    grid[1] = m
    y_mod = torch.full((m, n), float("nan"), device=DEV, dtype=dt)
    launch(hip, mod, name, grid, block, lds, w, x, y_mod, n, k)
    y_lib = torch.empty((m, n), device=DEV, dtype=dt)
    fn = lib.lhip_q8_0_matmul_f16 if f16 else lib.lhip_q8_0_matmul_f32
    capi.check(fn(w.planar.data_ptr(), x.data_ptr(), y_lib.data_ptr(), m, n, k, None), "lhip_q8_0_matmul")
    torch.cuda.synchronize()
    as_int = torch.int16 if f16 else torch.int32
    assert torch.equal(y_mod.view(as_int), y_lib.view(as_int)), name


def test_result_of_the_persistent_kernel_does_not_depend_on_the_grid(module):
    hip, mod = module
    n, k = 1000, 2048
    qs, d = synth.q8_0_random(n, k, seed=5)
    w = Q8Weight.from_raw(synth.q8_0_raw_blocks(qs, d), n, k, DEV)
    x = torch.randn(1, k, device=DEV)
    name, grid, block, lds = plan(n, k, False)
    assert name == b"lhip_kernel_q8_0_gemv_f32_pipe_r1s2w4" and grid[0] == 250
    outs = []
    for gx in (grid[0], 1, 7, 100):
        y = torch.full((1, n), float("nan"), device=DEV)
        launch(hip, mod, name, [gx, 1, 1], block, lds, w, x, y, n, k)
        outs.append(y)
    for y in outs[1:]:
        assert torch.equal(y.view(torch.int32), outs[0].view(torch.int32))
