"""The code-object path: a host that owns module loading itself, as the reference's CUDA backend
does with its embedded image (ops/cuda/kernels.zig:69-218, :1980-2007) and a Zig `hip` backend
would with `@embedFile`.  Nothing of the library is used here: the gfx950 code object is loaded
with hipModuleLoadData, its extern "C" kernels are found by name and launched with
hipModuleLaunchKernel from a parameter block (ops/cuda/kernels.zig:1245-1252), on memory from
hipMalloc -- the driver-level calls of ops/cuda/driver.zig:44-76, HIP flavour."""
import ctypes as C
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from antfly_amd import _lib, synth  # noqa: E402
from oracle import oracle as O  # noqa: E402
from tests import gpu_util as G  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
IMAGE = os.path.join(ROOT, "antfly_amd", "lib", "antfly_hip_kernels.hsaco")
Q4, Q8 = _lib.TYPE_Q4_0, _lib.TYPE_Q8_0


class Hip:
    """The dlopen table a `hip` driver module binds (no torch, no libantfly)."""

    def __init__(self):
        self.lib = C.CDLL("libamdhip64.so")
        self.check(self.lib.hipInit(0))
        self.check(self.lib.hipSetDevice(0))
        self.stream = C.c_void_p()
        self.check(self.lib.hipStreamCreate(C.byref(self.stream)))

    def check(self, rc):
        if rc != 0:
            self.lib.hipGetErrorName.restype = C.c_char_p
            raise RuntimeError(f"hip error {rc}: {self.lib.hipGetErrorName(rc)}")

    def alloc(self, nbytes):
        p = C.c_void_p()
        self.check(self.lib.hipMalloc(C.byref(p), C.c_size_t(max(nbytes, 16))))
        return p

    def upload(self, a):
        a = np.ascontiguousarray(a)
        p = self.alloc(a.nbytes)
        self.check(self.lib.hipMemcpyHtoDAsync(p, a.ctypes.data_as(C.c_void_p), C.c_size_t(a.nbytes), self.stream))
        self.check(self.lib.hipStreamSynchronize(self.stream))
        return p

    def download(self, p, shape, dtype):
        out = np.empty(shape, dtype)
        self.check(self.lib.hipMemcpyDtoHAsync(out.ctypes.data_as(C.c_void_p), p, C.c_size_t(out.nbytes), self.stream))
        self.check(self.lib.hipStreamSynchronize(self.stream))
        return out

    def launch(self, fn, grid, block, lds, *args):
        params = (C.c_void_p * len(args))(*[C.cast(C.byref(a), C.c_void_p) for a in args])
        self.check(self.lib.hipModuleLaunchKernel(fn, grid[0], grid[1], 1, block[0], block[1], 1, C.c_uint(lds), self.stream,
                                                  params, None))


@pytest.fixture(scope="module")
def module():
    if not os.path.exists(IMAGE):
        pytest.fail(f"code object not built: {IMAGE}")
    hip = Hip()
    image = open(IMAGE, "rb").read()
    mod = C.c_void_p()
    hip.check(hip.lib.hipModuleLoadData(C.byref(mod), image))
    fns = {}
    for name in ("termite_hip_zero_fill", "termite_hip_prepare_weight_q4_0", "termite_hip_prepare_weight_q8_0",
                 "termite_hip_linear_q4_0_f32", "termite_hip_linear_q8_0_f32"):
        f = C.c_void_p()
        hip.check(hip.lib.hipModuleGetFunction(C.byref(f), mod, name.encode()))
        fns[name] = f
    yield hip, fns
    hip.check(hip.lib.hipModuleUnload(mod))


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("in_dim,out_dim", [(4096, 1024), (14336, 512), (1120, 515), (4096, 14336)])
def test_module_kernels_from_a_parameter_block(module, fmt, in_dim, out_dim):
    hip, fns = module
    print(f"case: code object fmt={fmt} in={in_dim} out={out_dim}", flush=True)
    name = "q4_0" if fmt == Q4 else "q8_0"
    kb = in_dim // 32
    w = synth.weights(fmt, 900 + out_dim, out_dim, in_dim)
    x = synth.activations(901, 1, in_dim)
    # ---- load-time repack with the module's own kernels
    want_prepared = G.numpy_prepare(fmt, w, out_dim, in_dim)
    raw_d = hip.upload(w)
    prep_d = hip.alloc(want_prepared.size)
    blocks = out_dim * kb
    fill_from = (blocks * (18 if fmt == Q4 else 34)) & ~15
    n16 = (want_prepared.size - fill_from) // 16
    hip.launch(fns["termite_hip_zero_fill"], ((n16 + 255) // 256, 1), (256, 1), 0,
               C.c_void_p(prep_d.value + fill_from), C.c_ulonglong(n16))
    hip.launch(fns[f"termite_hip_prepare_weight_{name}"], ((blocks + 255) // 256, 1), (256, 1), 0,
               prep_d, raw_d, C.c_uint(out_dim), C.c_uint(kb))
    assert np.array_equal(hip.download(prep_d, (want_prepared.size,), np.uint8), want_prepared)
    # ---- the matmul entry: (dst, input, weight, rows, in_dim, out_dim) + launch geometry
    cols = 4 if fmt == Q4 else 2
    slices = (kb + 127) // 128
    groups = (out_dim + cols - 1) // cols
    groups_per_wg = max(1, min(16 // slices, (groups + 255) // 256))
    grid = (groups + groups_per_wg - 1) // groups_per_wg
    x_d = hip.upload(x)
    y_d = hip.upload(np.full((1, out_dim), np.nan, np.float32))
    hip.launch(fns[f"termite_hip_linear_{name}_f32"], (grid, 1), (64 * slices, groups_per_wg), in_dim + kb * 8 + 1024,
               y_d, x_d, prep_d, C.c_uint(1), C.c_uint(in_dim), C.c_uint(out_dim), C.c_uint(groups_per_wg),
               C.c_uint(1 if grid <= 256 else 0))
    y = hip.download(y_d, (1, out_dim), np.float32)
    ref = O.linear_no_bias(fmt, x, w, 1, in_dim, out_dim, workers=8)
    assert G.max_rel_err(y, ref.astype(np.float64)) <= 2e-5
    # the library's launcher gives the same bits (same kernel body)
    assert np.array_equal(y, G.linear(fmt, _lib.LAYOUT_PREPARED, x, G.prepare(fmt, w, out_dim, in_dim), 1, in_dim, out_dim))
    for p in (raw_d, prep_d, x_d, y_d):
        hip.check(hip.lib.hipFree(p))
