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


ENTRIES = ("termite_hip_zero_fill", "termite_hip_prepare_weight_q4_0", "termite_hip_prepare_weight_q8_0",
           "termite_hip_linear_q4_0_f32", "termite_hip_linear_q8_0_f32", "termite_hip_linear_q4_0_f32_route",
           "termite_hip_linear_q8_0_f32_route", "termite_hip_quantize_activations", "termite_hip_linear_q4_0_rows_f32",
           "termite_hip_linear_q8_0_rows_f32", "termite_hip_gemm_q4_0_f32", "termite_hip_gemm_q8_0_f32",
           "termite_hip_gemm_q4_0_f32_small", "termite_hip_gemm_q8_0_f32_small")


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
    for name in ENTRIES:
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


def prepared_on_device(hip, fns, fmt, w, out_dim, in_dim):
    """The module's own repack (checked byte for byte in the test above)."""
    name = "q4_0" if fmt == Q4 else "q8_0"
    kb = in_dim // 32
    size = G.numpy_prepare(fmt, w, out_dim, in_dim).size
    raw_d, prep_d = hip.upload(w), hip.alloc(size)
    blocks = out_dim * kb
    fill_from = (blocks * (18 if fmt == Q4 else 34)) & ~15
    n16 = (size - fill_from) // 16
    hip.launch(fns["termite_hip_zero_fill"], ((n16 + 255) // 256, 1), (256, 1), 0, C.c_void_p(prep_d.value + fill_from),
               C.c_ulonglong(n16))
    hip.launch(fns[f"termite_hip_prepare_weight_{name}"], ((blocks + 255) // 256, 1), (256, 1), 0, prep_d, raw_d,
               C.c_uint(out_dim), C.c_uint(kb))
    hip.check(hip.lib.hipFree(raw_d))
    return prep_d


def quantized_on_device(hip, fns, x_d, rows, in_dim):
    kb = in_dim // 32
    q_d, s_d, m_d = hip.alloc(rows * in_dim), hip.alloc(rows * kb * 4), hip.alloc(rows * kb * 4)
    units = rows * in_dim // 4
    hip.launch(fns["termite_hip_quantize_activations"], (min((units + 255) // 256, 4096), 1), (256, 1), 0, q_d, s_d, m_d, x_d,
               C.c_uint(rows), C.c_uint(in_dim))
    return q_d, s_d, m_d


def fused_lds(rows, in_dim):
    return rows * (in_dim + in_dim // 32 * 8) + 256 * max(rows, 4)


@pytest.mark.parametrize("fmt,rows,in_dim,out_dim", [(Q4, 2, 4096, 1024), (Q4, 3, 4096, 520), (Q4, 4, 4096, 14336), (Q8, 2, 4096, 1030),
                                                     (Q4, 4, 2048, 512), (Q4, 5, 4096, 512), (Q8, 3, 4096, 512), (Q4, 2, 8192, 512)])
def test_module_small_batch_entry_quantizes_in_the_kernel(module, fmt, rows, in_dim, out_dim):
    """Rows 2 .. 4 (Q4_0) / 2 (Q8_0) through the same entry as one row; a row count or K it does not serve leaves NaN."""
    hip, fns = module
    print(f"case: code object fused rows fmt={fmt} rows={rows} in={in_dim} out={out_dim}", flush=True)
    name = "q4_0" if fmt == Q4 else "q8_0"
    kb = in_dim // 32
    w = synth.weights(fmt, 910 + out_dim, out_dim, in_dim)
    x = synth.activations(911 + rows, rows, in_dim)
    prep_d = prepared_on_device(hip, fns, fmt, w, out_dim, in_dim)
    cols = 4 if fmt == Q4 else 2
    slices = (kb + 127) // 128
    groups = (out_dim + cols - 1) // cols
    groups_per_wg = max(1, min(16 // slices, (groups + 255) // 256))
    grid = (groups + groups_per_wg - 1) // groups_per_wg
    x_d = hip.upload(x)
    y_d = hip.upload(np.zeros((rows, out_dim), np.float32))
    hip.launch(fns[f"termite_hip_linear_{name}_f32"], (grid, 1), (64 * slices, groups_per_wg), fused_lds(rows, in_dim),
               y_d, x_d, prep_d, C.c_uint(rows), C.c_uint(in_dim), C.c_uint(out_dim), C.c_uint(groups_per_wg),
               C.c_uint(1 if grid <= 256 else 0))
    y = hip.download(y_d, (rows, out_dim), np.float32)
    served = rows <= (4 if fmt == Q4 else 2) and in_dim <= 4096 and (rows <= 2 or rows * kb <= 512)
    if served:
        ref = O.linear_no_bias(fmt, x, w, rows, in_dim, out_dim, workers=8)
        assert G.max_rel_err(y, ref.astype(np.float64)) <= 2e-5
    else:
        assert np.isnan(y).all()
    for p in (prep_d, x_d, y_d):
        hip.check(hip.lib.hipFree(p))


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("rows,in_dim,out_dim", [(2, 32, 3), (3, 64, 100), (1, 4096, 100)])
def test_module_f32_route_entry(module, fmt, rows, in_dim, out_dim):
    """The small shapes the CPU engine multiplies in f32 (route B), the reference's own smoke shape among them."""
    hip, fns = module
    print(f"case: code object route B fmt={fmt} rows={rows} in={in_dim} out={out_dim}", flush=True)
    assert not O.uses_activation_quant(rows, in_dim, out_dim)
    name = "q4_0" if fmt == Q4 else "q8_0"
    w = synth.weights(fmt, 920 + out_dim, out_dim, in_dim)
    x = synth.activations(921, rows, in_dim)
    prep_d = prepared_on_device(hip, fns, fmt, w, out_dim, in_dim)
    x_d = hip.upload(x)
    y_d = hip.upload(np.full((rows, out_dim), np.nan, np.float32))
    hip.launch(fns[f"termite_hip_linear_{name}_f32_route"], (out_dim, rows), (64, 1), 0, y_d, x_d, prep_d, C.c_uint(rows),
               C.c_uint(in_dim), C.c_uint(out_dim))
    y = hip.download(y_d, (rows, out_dim), np.float32)
    ref = O.linear_no_bias(fmt, x, w, rows, in_dim, out_dim, workers=1)
    assert G.max_rel_err(y, ref.astype(np.float64)) <= 2e-5
    for p in (prep_d, x_d, y_d):
        hip.check(hip.lib.hipFree(p))


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("rows,in_dim,out_dim", [(5, 4096, 1024), (8, 14336, 512), (7, 1120, 515)])
def test_module_quantizer_and_rows_entries(module, fmt, rows, in_dim, out_dim):
    """small_batch beyond the fused rows: the module's quantizer, then its rows kernel."""
    hip, fns = module
    print(f"case: code object rows kernel fmt={fmt} rows={rows} in={in_dim} out={out_dim}", flush=True)
    name = "q4_0" if fmt == Q4 else "q8_0"
    kb = in_dim // 32
    w = synth.weights(fmt, 930 + out_dim, out_dim, in_dim)
    x = synth.activations(931, rows, in_dim)
    prep_d = prepared_on_device(hip, fns, fmt, w, out_dim, in_dim)
    x_d = hip.upload(x)
    q_d, s_d, m_d = quantized_on_device(hip, fns, x_d, rows, in_dim)
    qx, sx, sums = O.quantize_activation_rows(x, rows, in_dim)
    assert np.array_equal(hip.download(q_d, (rows, in_dim), np.int8), np.asarray(qx).reshape(rows, in_dim))
    assert np.array_equal(hip.download(s_d, (rows, kb), np.float32).view(np.uint32), np.asarray(sx, np.float32).reshape(rows, kb).view(np.uint32))
    assert np.array_equal(hip.download(m_d, (rows, kb), np.int32), np.asarray(sums).reshape(rows, kb))
    cols = 4 if fmt == Q4 else 2
    slices = (kb + 127) // 128
    waves = max(8 // slices * slices, slices)
    groups = (out_dim + cols - 1) // cols
    grid = (groups + waves // slices - 1) // (waves // slices)
    y_d = hip.upload(np.full((rows, out_dim), np.nan, np.float32))
    hip.launch(fns[f"termite_hip_linear_{name}_rows_f32"], (grid, 1), (64 * waves, 1), fused_lds(rows, in_dim), y_d, x_d, prep_d,
               C.c_uint(rows), C.c_uint(in_dim), C.c_uint(out_dim), q_d, s_d, m_d)
    y = hip.download(y_d, (rows, out_dim), np.float32)
    ref = O.linear_no_bias(fmt, x, w, rows, in_dim, out_dim, workers=8)
    assert G.max_rel_err(y, ref.astype(np.float64)) <= 2e-5
    for p in (prep_d, x_d, y_d, q_d, s_d, m_d):
        hip.check(hip.lib.hipFree(p))


GEMM_LDS = {("q8_0", False): 110592, ("q4_0", False): 143360, ("q8_0", True): 110592, ("q4_0", True): 143360}


@pytest.mark.parametrize("fmt", [Q4, Q8])
@pytest.mark.parametrize("rows,in_dim,out_dim,small", [(130, 512, 520, True), (128, 1024, 2048, False), (70, 96, 513, True),
                                                       (512, 4096, 4096, False)])
def test_module_prefill_entries(module, fmt, rows, in_dim, out_dim, small):
    """The mm bucket: the module's quantizer, then its int8-MFMA GEMM on 64 x 128 or 32 x 64 tiles."""
    hip, fns = module
    print(f"case: code object gemm fmt={fmt} rows={rows} in={in_dim} out={out_dim} small={small}", flush=True)
    name = "q4_0" if fmt == Q4 else "q8_0"
    w = synth.weights(fmt, 940 + out_dim, out_dim, in_dim)
    x = synth.activations(941, rows, in_dim)
    prep_d = prepared_on_device(hip, fns, fmt, w, out_dim, in_dim)
    x_d = hip.upload(x)
    q_d, s_d, m_d = quantized_on_device(hip, fns, x_d, rows, in_dim)
    tm, tn, threads = (32, 64, 512) if small else (64, 128, 1024)
    m_tiles, n_tiles = (rows + tm - 1) // tm, (out_dim + tn - 1) // tn
    grid = (n_tiles + 7) // 8 * m_tiles * 8
    y_d = hip.upload(np.full((rows, out_dim), np.nan, np.float32))
    hip.launch(fns[f"termite_hip_gemm_{name}_f32" + ("_small" if small else "")], (grid, 1), (threads, 1), GEMM_LDS[(name, small)],
               y_d, x_d, prep_d, C.c_uint(rows), C.c_uint(in_dim), C.c_uint(out_dim), q_d, s_d, C.c_uint(m_tiles), C.c_uint(n_tiles))
    y = hip.download(y_d, (rows, out_dim), np.float32)
    if rows * in_dim * out_dim <= 512 * 4096 * 512:
        ref = O.linear_no_bias(fmt, x, w, rows, in_dim, out_dim, workers=8)
        assert G.max_rel_err(y, ref.astype(np.float64)) <= 2e-5
    else:  # the full prefill configuration: against the library's launcher, which is held to the oracle at this size elsewhere
        want = G.linear(fmt, _lib.LAYOUT_PREPARED, x, G.prepare(fmt, w, out_dim, in_dim), rows, in_dim, out_dim, dispatch=3)
        assert G.max_rel_err(y, want.astype(np.float64)) <= 2e-5
        if fmt == Q8:
            assert np.array_equal(y, want)
    for p in (prep_d, x_d, y_d, q_d, s_d, m_d):
        hip.check(hip.lib.hipFree(p))
