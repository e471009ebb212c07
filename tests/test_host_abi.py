"""CPU-only checks of the C ABI: the library loads, exports every declared
symbol, and the host logic (dispatch vocabulary, launcher argument checks, plan
validation) behaves like the reference's.  No kernel is launched."""
import ctypes as C
import os
import re

import pytest

from antfly_amd import _lib, kernels, quant_matmul as qm
from antfly_amd._lib import Buffer

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "antfly_hip_qmatmul.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)  # drop comments
    declared = set(re.findall(r"\b(afhip_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 40
    L = C.CDLL(_lib.LIB_PATH)
    missing = [name for name in sorted(declared) if not hasattr(L, name)]
    assert not missing, missing
    # the Python binding declares exactly the header's functions
    assert declared == set(_lib.SIGNATURES)


def test_status_strings():
    L = _lib.lib()
    assert L.afhip_status_string(0) == b"ok"
    assert L.afhip_status_string(_lib.ERR_INVALID_PARTITION_PLAN) == b"InvalidPartitionPlan"
    assert L.afhip_status_string(_lib.ERR_UNSUPPORTED_TENSOR_TYPE) == b"UnsupportedTensorType"


def test_dispatch_buckets_match_reference(kats):
    k = kats["dispatch"]
    for case in k["select"]:
        shape = qm.Shape(case["rows"], case["in_dim"], case["out_dim"], qm.Format[case["format"]])
        assert qm.select(shape).name == case["dispatch"], case
    for case in k["plan"]:
        p = qm.plan(qm.Shape(case["rows"], case["in_dim"], case["out_dim"], qm.Format[case["format"]]))
        assert p.primitive.name == case["primitive"] and p.operator.name == case["operator"], case
    for rows, name in k["row_buckets"]:
        assert qm.rowBucket(rows).name == name
    # K must be a multiple of the 32-value block for both formats
    for fmt in (qm.Format.q4_0, qm.Format.q8_0):
        assert qm.select(qm.Shape(1, 48, 64, fmt)) == qm.DispatchKind.scalar
        assert qm.select(qm.Shape(1, 64, 64, fmt)) == qm.DispatchKind.mmv
        assert qm.select(qm.Shape(1, 0, 64, fmt)) == qm.DispatchKind.scalar
        assert qm.select(qm.Shape(1, 64, 0, fmt)) == qm.DispatchKind.scalar
    p = qm.plan(qm.Shape(5, 14336, 4096, qm.Format.q4_0))
    assert (p.dispatch, p.row_bucket, p.rows, p.in_dim, p.out_dim) == (qm.DispatchKind.small_batch, qm.RowBucket.rows_2_8, 5, 14336, 4096)
    assert qm.formatFromTensorType(2) == qm.Format.q4_0 and qm.formatFromTensorType(8) == qm.Format.q8_0
    assert qm.formatFromTensorType(12) == qm.Format.q4_k and qm.formatFromTensorType(14) == qm.Format.unknown
    # Q4_K: K must be whole 256-value super-blocks
    assert qm.select(qm.Shape(1, 128, 64, qm.Format.q4_k)) == qm.DispatchKind.scalar
    assert qm.select(qm.Shape(3, 512, 64, qm.Format.q4_k)) == qm.DispatchKind.small_batch


def test_route_gate_matches_cpu_engine():
    L = _lib.lib()
    assert L.afhip_uses_activation_quant(1, 4096, 14336) == 1
    assert L.afhip_uses_activation_quant(1, 4096, 511) == 0
    assert L.afhip_uses_activation_quant(1, 64, 4096) == 0   # two blocks per row
    assert L.afhip_uses_activation_quant(1, 96, 512) == 1


def test_launcher_argument_checks_before_any_launch():
    big = Buffer(0x1000, 1 << 40)
    # in_dim not a multiple of 32, or zero -> InvalidHipState (kernels.zig:1231,1266)
    for fn in (kernels.launchLinearQ8_0F32, kernels.launchLinearQ4_0F32):
        with pytest.raises(_lib.InvalidHipState):
            fn(None, big, big, big, 1, 33, 8)
        with pytest.raises(_lib.InvalidHipState):
            fn(None, big, big, big, 1, 0, 8)
        # short output / input / weight buffers
        with pytest.raises(_lib.InvalidHipState):
            fn(None, Buffer(0x1000, 4 * 8 - 1), big, big, 1, 32, 8)
        with pytest.raises(_lib.InvalidHipState):
            fn(None, big, Buffer(0x1000, 4 * 32 - 1), big, 1, 32, 8)
        with pytest.raises(_lib.InvalidHipState):
            fn(None, big, big, Buffer(0x1000, 8 * 18 - 1), 1, 32, 8)
        # rows * out_dim == 0 is a successful no-op
        fn(None, big, big, big, 0, 32, 8)
        fn(None, big, big, big, 4, 32, 0)
        # dimension overflow
        with pytest.raises(_lib.InvalidHipState):
            fn(None, big, big, big, 1 << 62, 32, 1 << 10)
    with pytest.raises(_lib.UnsupportedTensorType):
        kernels.launchLinearF32(None, 14, 0, big, big, big, 1, 256, 8)  # Q6_K is another operator
    with pytest.raises(_lib.InvalidHipState):
        kernels.launchLinearF32(None, 12, 0, big, big, big, 1, 128, 8)  # Q4_K: K must be whole super-blocks
    with pytest.raises(_lib.InvalidHipState):
        kernels.launchLinearF32(None, 12, 0, big, big, Buffer(0x1000, 8 * 144 - 1), 1, 256, 8)
    # raw-layout activation-quantized route needs the caller's scratch
    assert kernels.workspaceBytes(2, 5, 14336, 4096) >= 5 * 14336 + 5 * 448 * 8
    assert kernels.workspaceBytes(2, 0, 14336, 4096) == 0
    with pytest.raises(_lib.InvalidHipState):
        kernels.launchLinearQ4_0F32(None, big, big, big, 1, 4096, 4096)
    with pytest.raises(_lib.InvalidHipState):
        kernels.launchPrepareWeight(None, 2, Buffer(0x1000, 17), Buffer(0x2000, 18), 1, 32)
    with pytest.raises(_lib.InvalidHipState):
        kernels.launchQuantizeActivations(None, big, 1, 48, big, big)


def test_q4_k_prefill_workspace_sizes():
    """Scratch of Q4_K: none for one or two rows; three to eight rows: X as digit planes in MFMA operand
    order (8 KB per super-block, plus a scale per row and super-block and a sum per row and sub-block, laid
    out for eight rows); rows of the prefill GEMM (more than one GEMV launch holds: seven at K = 4096, three at
    K = 14336): the split of X (three bf16 parts = 6 bytes per value, plus 64 bytes of sum parts per row and
    super-block) and, while the row x column grid is small, room for the partial sums of the K shares (a power
    of two, at most eight, at least two super-blocks each) -- the larger of the two where both apply."""
    Q4K = _lib.TYPE_Q4_K
    planes = lambda k: k // 256 * (8192 + 32 + 256)
    for rows in (1, 2):
        assert kernels.workspaceBytes(Q4K, rows, 4096, 4096) == 0
        assert kernels.workspaceBytes(Q4K, rows, 14336, 4096) == 0
    for rows in (3, 6):
        assert kernels.workspaceBytes(Q4K, rows, 4096, 4096) == planes(4096)
    assert kernels.workspaceBytes(Q4K, 7, 4096, 4096) >= max(planes(4096), 7 * 4096 * 6)
    assert kernels.workspaceBytes(Q4K, 3, 14336, 4096) >= max(planes(14336), 3 * 14336 * 6)
    assert kernels.workspaceBytes(Q4K, 9, 4096, 4096) > 9 * 4096 * 6
    for rows, k, n in [(13, 4096, 14336), (64, 4096, 4096), (512, 4096, 14336), (40, 512, 40), (33, 14336, 4096)]:
        split = (rows * k * 6 + rows * (k // 256) * 64 + 255) // 256 * 256
        got = kernels.workspaceBytes(Q4K, rows, k, n)
        extra = got - split
        assert extra >= 0 and extra % (rows * n * 4) == 0, (rows, k, n, got)
        shares = extra // (rows * n * 4)
        assert shares in (0, 2, 4, 8) and (shares == 0 or (k // 256) // shares >= 2), (rows, k, n, shares)
    # a grid that fills the chip anyway shares nothing out
    assert kernels.workspaceBytes(Q4K, 2048, 4096, 14336) == 2048 * 4096 * 6 + 2048 * 16 * 64
    # the smallest prefill on a small matrix spreads K over workgroups
    assert kernels.workspaceBytes(Q4K, 13, 4096, 4096) > 13 * 4096 * 6 + 13 * 16 * 64


def test_linear_workspace_covers_every_kernel_family():
    """The scratch size is the largest of what the kernels a shape may run on need.  Nine rows and
    more on a grid too small for the chip: behind the quantized activations, the partial sums of
    2, 4 or 8 K shares (at least 16 blocks each) of the tiled GEMM.  Up to eight rows (and
    eight-row slices of a forced plan) on a K longer than 4096: the sums of the K slices of the
    small-batch kernel, for a pair of matrices.  Up to 128 rows: X in MFMA operand order (rows
    padded to 32), its scales, and the partial sums of the K shares (128 blocks of Q4_0, 64 of
    Q8_0 each) of the single-shot MFMA kernel, for a pair of matrices."""
    def up256(v):
        return (v + 255) // 256 * 256

    def quantized(rows, k):  # int8 values padded to 256 bytes, f32 scales, i32 sums
        return up256(rows * k) + rows * (k // 32) * 8

    def batch(rows, k, n):
        slices = (k // 32 + 127) // 128
        return slices * min(rows, 8) * n * 4 * 2 if slices > 1 else 0

    def mfma(fmt, rows, k, n):
        if rows > 128:
            return 0
        padded = (rows + 31) // 32 * 32
        share = 128 if fmt == _lib.TYPE_Q4_0 else 64
        shares = (k // 32 + share - 1) // share
        return up256(padded * k + (k // 32) * padded * 4) + (2 * shares * rows * n * 4 if shares > 1 else 0)

    for fmt in (_lib.TYPE_Q4_0, _lib.TYPE_Q8_0):
        for rows, k, n in [(16, 4096, 4096), (64, 14336, 4096), (9, 1024, 64), (128, 4096, 1024)]:
            got = kernels.workspaceBytes(fmt, rows, k, n)
            assert got >= max(quantized(rows, k), batch(rows, k, n), mfma(fmt, rows, k, n))
            if got > max(batch(rows, k, n), mfma(fmt, rows, k, n)):  # the tiled GEMM's K shares decide
                extra = got - up256(quantized(rows, k))
                assert extra > 0 and extra % (rows * n * 4) == 0
                shares = extra // (rows * n * 4)
                assert shares in (2, 4, 8) and (k // 32) // shares >= 16
        assert kernels.workspaceBytes(fmt, 128, 4096, 1024) > quantized(128, 4096)   # 128 workgroups: K is shared out
        assert kernels.workspaceBytes(fmt, 8, 4096, 4096) == max(quantized(8, 4096), mfma(fmt, 8, 4096, 4096))
        assert kernels.workspaceBytes(fmt, 512, 4096, 4096) == quantized(512, 4096)
        assert kernels.workspaceBytes(fmt, 16, 512, 4096) == max(quantized(16, 512), mfma(fmt, 16, 512, 4096))
        assert kernels.workspaceBytes(fmt, 5, 14336, 4096) == max(quantized(5, 14336), batch(5, 14336, 4096), mfma(fmt, 5, 14336, 4096))
        assert batch(5, 14336, 4096) == 4 * 5 * 4096 * 4 * 2
    assert mfma(_lib.TYPE_Q4_0, 33, 4096, 512) == 64 * 4096 + 128 * 64 * 4
    assert kernels.workspaceBytes(_lib.TYPE_Q4_0, 100, 4096, 8192) >= mfma(_lib.TYPE_Q4_0, 100, 4096, 8192) == 128 * 4096 + 128 * 128 * 4
    assert mfma(_lib.TYPE_Q8_0, 4, 4096, 512) == 32 * 4096 + 128 * 32 * 4 + 2 * 2 * 4 * 512 * 4


def test_zig_backend_sources_bind_what_exists():
    """The Zig `hip` backend sources (zig/pkg/inference/src/ops/hip) cannot be compiled in this
    image; this keeps them honest against what can be checked here: every C-ABI function they
    declare is in the header with the same argument count, and every kernel they look up by
    name is an extern "C" entry of the code object's source."""
    zig_dir = os.path.join(ROOT, "zig", "pkg", "inference", "src", "ops", "hip")
    names = sorted(os.listdir(zig_dir))
    assert names == ["buffer.zig", "context.zig", "driver.zig", "hip_compute.zig", "kernels.zig", "scratch.zig"]
    kernels_zig = open(os.path.join(zig_dir, "kernels.zig")).read()
    header = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "antfly_hip_qmatmul.h")).read(), flags=re.S)
    externs = re.findall(r'extern "c" fn (afhip_[a-z0-9_]+)\((.*?)\)\s*[a-z_]+;', kernels_zig, flags=re.S)
    assert len(externs) >= 3
    for name, params in externs:
        m = re.search(r"\b" + name + r"\s*\((.*?)\);", header, flags=re.S)
        assert m, name
        zig_args = [p for p in params.split(",") if p.strip()]
        c_args = [p for p in m.group(1).split(",") if p.strip() and p.strip() != "void"]
        assert len(zig_args) == len(c_args), (name, zig_args, c_args)
    entries = set(re.findall(r'"(termite_hip_[a-z0-9_]+)"', kernels_zig))
    source = open(os.path.join(ROOT, "antfly_amd", "csrc", "code_object_kernels.hip")).read()
    exported = set(re.findall(r'extern "C" __global__[^\n]*void (termite_hip_[a-z0-9_]+)\(', source))
    assert entries and entries <= exported, entries - exported
    # the driver table binds only symbols libamdhip64 exports under these names
    driver_zig = open(os.path.join(zig_dir, "driver.zig")).read()
    table = re.findall(r"^\s+(hip[A-Za-z]+): \*const fn", driver_zig, flags=re.M)
    assert len(table) >= 20 and len(set(table)) == len(table)
    try:
        hip = C.CDLL("libamdhip64.so")
    except OSError:
        pytest.skip("libamdhip64.so not loadable here")
    missing = [n for n in table if not hasattr(hip, n)]
    assert not missing, missing


def test_session_wiring_patches_are_well_formed_and_apply():
    """zig/patches/*.patch (the `--backend hip` wiring, unified diffs against the antfly tree): headers and hunk line
    counts are consistent, the added lines name the hip backend, and -- where the reference tree is present (it
    is not on a GPU box) -- every context and removed line is found at the place the hunk header names."""
    pdir = os.path.join(ROOT, "zig", "patches")
    names = sorted(n for n in os.listdir(pdir) if n.endswith(".patch"))
    assert len(names) >= 9
    ref_root = "/root/reference"
    for name in names:
        lines = open(os.path.join(pdir, name)).read().split("\n")
        assert lines[0].startswith("--- a/zig/pkg/inference/") and lines[1].startswith("+++ b/zig/pkg/inference/"), name
        rel = lines[0][len("--- a/"):]
        assert lines[1][len("+++ b/"):] == rel
        ref_lines = None
        if os.path.exists(os.path.join(ref_root, rel)):
            ref_lines = open(os.path.join(ref_root, rel)).read().split("\n")
        i, hunks, added = 2, 0, []
        while i < len(lines) and lines[i]:
            m = re.match(r"@@ -(\d+),(\d+) \+(\d+),(\d+) @@", lines[i])
            assert m, (name, lines[i])
            old_at, old_n, new_n = int(m.group(1)), int(m.group(2)), int(m.group(4))
            i += 1
            seen_old = seen_new = 0
            while i < len(lines) and lines[i] and not lines[i].startswith("@@"):
                tag, text = lines[i][0], lines[i][1:]
                assert tag in " +-", (name, lines[i])
                if tag in " -":
                    if ref_lines is not None:
                        assert ref_lines[old_at - 1 + seen_old] == text, (name, old_at + seen_old, text)
                    seen_old += 1
                if tag in " +":
                    seen_new += 1
                if tag == "+":
                    added.append(text)
                i += 1
            assert (seen_old, seen_new) == (old_n, new_n), (name, m.group(0))
            hunks += 1
        assert hunks >= 1, name
        assert added and any(re.search(r"hip|Hip", t) for t in added), name
