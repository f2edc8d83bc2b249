"""Host-side checks that need no GPU: the C-ABI library loads and exports what
include/wol_c_api.h declares, argument errors come back as statuses before any
device work, the layout index helper is a bijection that agrees with the
numpy statement of the layout, and the Python mirror reproduces the
reference's shape contract and error behaviour."""
import ctypes
import os
import re

import numpy as np
import pytest

import helpers as H

ROOT = H.ROOT


@pytest.fixture(scope="module")
def lib():
    from paddle_amd import _lib

    return _lib


def test_library_exports_every_declared_symbol(lib):
    hdr = open(os.path.join(ROOT, "include", "wol_c_api.h")).read()
    hdr += open(os.path.join(ROOT, "include", "wol_diag.h")).read()
    declared = set(re.findall(r"\b(wol_[a-z0-9_]+)\s*\(", hdr))
    declared -= {"wol_status"}
    assert declared == set(lib.SYMBOLS), declared ^ set(lib.SYMBOLS)
    raw = ctypes.CDLL(lib.LIB_PATH)
    for name in declared:
        assert hasattr(raw, name), name


def test_no_kernel_spills_registers():
    # build.sh keeps the compiler's per-kernel resource remarks and refuses a
    # build in which a kernel spills; this reads the same files (absent when the
    # library was built elsewhere and only the .so travelled)
    import glob

    files = glob.glob(os.path.join(ROOT, "paddle_amd", "csrc", "build", "*.resources.txt"))
    if not files:
        pytest.skip("no resource remarks beside the build")
    kernels = 0
    for f in files:
        text = open(f).read()
        kernels += text.count("Function Name:")
        assert not re.search(r"(VGPRs Spill|ScratchSize \[bytes/lane\]): [1-9]", text), f
    assert kernels > 500  # the streaming kernel alone has several hundred instantiations


def test_status_strings_and_version(lib):
    L = lib.lib
    assert L.wol_layout_version() == 1
    assert L.wol_status_str(0) == b"ok"
    seen = {L.wol_status_str(i) for i in range(0, 12)}
    assert len(seen) == 12
    assert L.wol_status_str(99) == b"unknown status"


def test_workspace_queries(lib):
    L = lib.lib
    assert L.wol_quantize_workspace(4096, 11008, 4, -1) == 4 * 11008
    assert L.wol_quantize_workspace(4096, 11008, 4, 128) == 0
    assert L.wol_quantize_workspace(4095, 11008, 4, 128) == 0  # invalid shape
    assert L.wol_linear_workspace(1, 4096, 11008, 4, 128) == 0       # streaming kernel
    assert L.wol_linear_workspace(2048, 4096, 12288, 8, -1) == 0     # one workgroup per tile covers all of K
    assert L.wol_linear_workspace(1024, 4096, 4096, 8, 64) == 2 * 1024 * 4096 * 4  # 128 tiles: two K runs
    # group-wise int8 takes 256 x 256 tiles like per-channel int8: 192 of them, one round, no K runs
    assert L.wol_linear_workspace(1024, 4096, 12288, 8, 64) == 0
    # group-wise int4, 256 x 128 tiles, 384 of them: the 256 of the whole round run as they are, the other 128
    # (4096 columns) in two K runs
    assert L.wol_linear_workspace(1024, 4096, 12288, 4, 128) == 2 * 1024 * 4096 * 4
    # 256 x 256 tiles on the columns of whole rounds, one 256 x 128 column tile left over: four K runs of it
    assert L.wol_linear_workspace(700, 2048, 22016, 8, 64) == 4 * 700 * 256 * 4
    # small M on the GEMM: whole fp32 [M, N] partial buffers, at most 16 of them
    for M, K, N, bits, g in [(64, 8192, 28672, 4, 128), (48, 4096, 11008, 4, -1), (24, 8192, 28672, 4, 128)]:
        need = L.wol_linear_workspace(M, K, N, bits, g)
        assert need == L.wol_linear_workspace_for(M, K, N, bits, g, lib.KERNEL_GEMM)
        assert need % (M * N * 4) == 0 and 2 <= need // (M * N * 4) <= 16, (M, K, N, need)
    # the batched kernel with K runs: one fp32 [M, N] buffer per run (K / 2048, or K / 4096 from 13824 on)
    assert L.wol_linear_workspace(32, 4096, 11008, 4, -1) == 2 * 32 * 11008 * 4
    assert L.wol_linear_workspace(12, 13824, 5120, 4, 128) == 4 * 12 * 5120 * 4
    assert L.wol_linear_workspace_for(4, 4096, 4096, 8, 64, lib.KERNEL_BATCH_SPLIT) == 2 * 4 * 4096 * 4
    assert L.wol_linear_workspace_for(33, 4096, 4096, 8, 64, lib.KERNEL_BATCH_SPLIT) == 0  # not built for 33 rows
    assert L.wol_linear_workspace(16, 8192, 28672, 4, 128) == 0  # the one-launch batched kernel
    assert L.wol_linear_workspace_for(16, 8192, 28672, 4, 128, lib.KERNEL_GEMM) > 0
    assert L.wol_linear_workspace_for(16, 4096, 11008, 4, 128, lib.KERNEL_STREAM) == 0
    assert L.wol_linear_workspace_for(16, 4160, 11008, 4, 128, lib.KERNEL_GEMM) == 0  # K not a multiple of the k tile


def test_argument_errors_return_before_device_work(lib):
    L = lib.lib
    p = ctypes.c_void_p(0x1000)  # never dereferenced: every call fails validation first
    q = lambda **kw: L.wol_quantize(kw.get("w", p), kw.get("dt", 0), kw.get("K", 64), kw.get("N", 16), kw.get("bits", 8),
                                    kw.get("g", 64), kw.get("rm", 0), kw.get("layout", 2), p, p, None, 0, None)
    assert q(dt=2) == 2
    assert q(bits=5) == 3
    assert q(g=32) == 4
    assert q(K=32) == 5 and q(N=8) == 5 and q(K=0) == 5
    assert q(layout=7) == 6
    assert q(rm=3) == 7
    assert q(w=None) == 1
    assert q(w=ctypes.c_void_p(0x1008)) == 9
    assert q(g=-1) == 8  # per-channel needs the abs-max workspace
    lin = lambda **kw: L.wol_linear(kw.get("x", p), p, kw.get("bias", None), p, kw.get("dt", 1), kw.get("M", 1),
                                    kw.get("K", 64), kw.get("N", 16), kw.get("bits", 4), kw.get("g", -1),
                                    kw.get("out", p), None, 0, None)
    assert lin(dt=5) == 2 and lin(bits=2) == 3 and lin(g=100) == 4 and lin(K=100) == 5 and lin(M=-1) == 5
    assert lin(K=(1 << 24) + 64) == 5 and lin(N=(1 << 24) + 16) == 5 and lin(M=(1 << 24) + 1) == 5
    assert lin(x=None) == 1
    assert lin(x=ctypes.c_void_p(0x1004)) == 9
    # the output rows and the bias are accessed 16 bytes at a time as well
    assert lin(out=ctypes.c_void_p(0x1008)) == 9 and lin(bias=ctypes.c_void_p(0x1002)) == 9
    assert lin(out=None) == 1
    fused = lambda **kw: L.wol_linear_fused(p, None, p, kw.get("bias", None), p, 1, 1, 64, 32, 4, -1, 0,
                                            kw.get("out", p), None, 0, None)
    assert fused(out=ctypes.c_void_p(0x1008)) == 9 and fused(bias=ctypes.c_void_p(0x1004)) == 9
    assert lin(M=0) == 0  # empty batch is a no-op
    on = lambda **kw: L.wol_linear_on(p, p, None, kw.get("scale", p), 1, kw.get("M", 1), 64, 16, 4, -1, p, 0,
                                      kw.get("kernel", 0), None, 0, None)
    assert on(kernel=3) == 5 and on(kernel=-1) == 5
    assert on(kernel=lib.KERNEL_STREAM, M=65) == 5  # the streaming kernel stops at 64 rows
    assert on(scale=ctypes.c_void_p(0x1002)) == 9
    assert L.wol_dequantize(p, 9, p, 0, 64, 16, 8, -1, p, None) == 6
    assert L.wol_repack(p, 0, p, 2, 64, 16, 8, None) == 6  # in-place is refused
    assert L.wol_repack(p, 0, ctypes.c_void_p(0x2000), 2, 64, 24, 8, None) == 5
    with pytest.raises(ValueError, match="InvalidArgument"):
        lib.check(5)
    with pytest.raises(lib.WolError):
        lib.check(10)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("K", [64, 128, 192, 320])
def test_code_offset_is_a_bijection_matching_the_layout(lib, bits, K):
    L = lib.lib
    N = 48
    rng = np.random.default_rng(K + bits)
    bound = 127 if bits == 8 else 7
    q = rng.integers(-bound, bound + 1, (K, N)).astype(np.int32)
    want = {0: H.canonical_from_q(q, bits).view(np.uint8).reshape(-1),
            1: H.paddle_hip_from_q(q, bits).view(np.uint8).reshape(-1),
            2: H.gfx950_from_q(q, bits)}
    for layout in (0, 1, 2):
        buf = np.zeros(K * N * bits // 8, np.uint8)
        hits = np.zeros(K * N * bits // 8 * (2 if bits == 4 else 1), np.int32)
        sh = ctypes.c_int(0)
        for k in range(K):
            for n in range(N):
                off = L.wol_code_offset(layout, K, N, bits, k, n, ctypes.byref(sh))
                assert 0 <= off < buf.size
                if bits == 8:
                    v = (q[k, n] + 128) & 0xFF if layout == 2 else q[k, n] & 0xFF
                    buf[off] = v
                    hits[off] += 1
                else:
                    v = (q[k, n] & 0xF) if layout == 0 else (q[k, n] + 8) & 0xF
                    buf[off] |= v << sh.value
                    hits[2 * off + sh.value // 4] += 1
        assert (hits == 1).all()  # every slot written exactly once: a permutation
        assert np.array_equal(buf, want[layout]), layout
    assert L.wol_code_offset(2, K, N, bits, K, 0, None) == -1
    assert L.wol_code_offset(2, K, N, bits, 0, -1, None) == -1


def test_strip_slices_are_self_contained(lib):
    # a slice of the gfx950 tensor along N at a multiple of 16 is the gfx950
    # tensor of the sliced weight (what column-parallel sharding relies on)
    rng = np.random.default_rng(1)
    for bits in (8, 4):
        bound = 127 if bits == 8 else 7
        q = rng.integers(-bound, bound + 1, (192, 64)).astype(np.int32)
        full = H.gfx950_from_q(q, bits)
        per_strip = 16 * 192 * bits // 8
        assert np.array_equal(full[per_strip:3 * per_strip], H.gfx950_from_q(q[:, 16:48], bits))


# ------------------------------------------------------------ Python mirror
def test_infer_meta_contracts():
    from paddle_amd.nn.quant import quantized_linear as QL

    assert QL.weight_quantize_infer_meta((4096, 11008), "weight_only_int8", -1) == ([11008, 4096], [11008])
    assert QL.weight_quantize_infer_meta((4096, 11008), "weight_only_int4", 128) == ([5504, 4096], [32, 11008])
    assert QL.weight_quantize_infer_meta((192, 32), "weight_only_int8", 128) == ([32, 192], [2, 32])
    assert QL.weight_quantize_infer_meta((64, 16), "llm.int8", -1) == ([16, 64], [16])
    for bad in (((64,), "weight_only_int8", -1), ((63, 16), "weight_only_int8", -1), ((64, 8), "weight_only_int8", -1),
                ((64, 16), "weight_only_int8", 32), ((64, 16), "int8", -1)):
        with pytest.raises(ValueError, match="InvalidArgument"):
            QL.weight_quantize_infer_meta(*bad)
    assert QL.weight_dequantize_infer_meta((256, 64), (256,), "weight_only_int8", -1) == [64, 256]
    assert QL.weight_dequantize_infer_meta((128, 64), (1, 256), "weight_only_int4", 64) == [64, 256]
    for bad in (((256, 64), (255,), "weight_only_int8", -1), ((256, 64), (256,), "llm.int8", -1),
                ((256, 64), (1, 256), "weight_only_int8", -1), ((256, 64), (2, 256), "weight_only_int8", 64),
                ((256, 64), (1, 128), "weight_only_int8", 64)):
        with pytest.raises(ValueError, match="InvalidArgument"):
            QL.weight_dequantize_infer_meta(*bad)
    assert QL.weight_only_linear_infer_meta((2, 3, 64), (256, 64), (256,), (256,), "int8", -1) == ([2, 3, 256], 256)
    assert QL.weight_only_linear_infer_meta((1, 128), (144, 128), None, (1, 288), "int4", 128) == ([1, 288], 288)
    for bad in (((1, 64), (256, 64), None, (256,), "int2", -1), ((1, 64), (256, 64), None, (256,), "int8", 32),
                ((1, 64), (24, 64), None, (48,), "int4", -1), ((1, 65), (256, 64), None, (256,), "int8", -1),
                ((1, 64), (256, 64), (1, 256), (256,), "int8", -1), ((1, 64), (256, 64), None, (1, 256), "int8", -1),
                ((1, 64), (256, 64), None, (256,), "int8", 64), ((1, 128), (256, 128), None, (1, 256), "int8", 64)):
        with pytest.raises(ValueError, match="InvalidArgument"):
            QL.weight_only_linear_infer_meta(*bad)


def test_python_api_argument_checks():
    import torch

    from paddle_amd.nn import quant as Q

    x = torch.zeros(64, 16, dtype=torch.float16)
    with pytest.raises(AssertionError, match="group_size"):
        Q.weight_quantize(x, group_size=32)
    with pytest.raises(AssertionError, match="group_size"):
        Q.weight_dequantize(torch.zeros(16, 64, dtype=torch.int8), torch.zeros(16), group_size=7)
    with pytest.raises(AssertionError, match="group size"):
        Q.weight_only_linear(x, torch.zeros(16, 16, dtype=torch.int8), weight_scale=torch.zeros(16), group_size=1)
    with pytest.raises(ValueError, match="divisible by 64"):
        Q.weight_quantize(torch.zeros(32, 16, dtype=torch.float16))
    with pytest.raises(ValueError, match="float16 or bfloat16"):
        Q.weight_quantize(torch.zeros(64, 16, dtype=torch.float32))
    with pytest.raises(TypeError):
        Q.weight_dequantize(torch.zeros(16, 64, dtype=torch.int8), torch.zeros(16), out_dtype="float32")
    with pytest.raises(RuntimeError, match="GPU"):
        Q.weight_quantize(x)  # CPU tensors: there is no CPU kernel to fall back to
    assert Q.weight_quantize.__defaults__ == ("weight_only_int8", None, -1)
    assert Q.weight_dequantize.__defaults__ == ("weight_only_int8", "float16", -1)
    assert Q.weight_only_linear.__defaults__ == (None, None, "int8", None, -1)


def test_read_floor_argument_errors(lib):
    f = lib.lib.wol_read_floor
    assert f(None, 4096, 11008, 4, None, None) == 1  # null pointers
    assert f(None, 4096, 11008, 5, None, None) == 3  # bits
    assert f(None, 4096, 11000, 4, None, None) == 5  # N % 16
    assert f(None, 64, 16, 4, None, None) == 5  # a strip smaller than one piece per wavefront


def test_mfma_probe_argument_errors(lib):
    L = lib.lib
    p = ctypes.c_void_p(0x1000)
    need = 64 * 8 * 49152 + 65536
    assert L.wol_mfma_probe(9, p, need, 1, 1, p, None) == 5 and L.wol_mfma_probe(-1, p, need, 1, 1, p, None) == 5
    assert L.wol_mfma_probe(0, p, need, 0, 1, p, None) == 5 and L.wol_mfma_probe(0, p, need, 1, 0, p, None) == 5
    assert L.wol_mfma_probe(0, None, need, 1, 1, p, None) == 1
    assert L.wol_mfma_probe(0, ctypes.c_void_p(0x1008), need, 1, 1, p, None) == 9
    assert L.wol_mfma_probe(5, p, need - 1, 1, 1, p, None) == 8  # too few operand bytes for the variants that load


def test_decode_phases_argument_errors(lib):
    L = lib.lib
    p = ctypes.c_void_p(0x1000)
    big = 1 << 30
    assert L.wol_decode_phases(p, p, p, 4096, 11008, 128, p, p, big, None) not in (1, 5, 8, 9)  # valid: fails only for want of a device
    assert L.wol_decode_phases(p, p, p, 8192, 11008, 128, p, p, big, None) == 5   # built for K = 4096
    assert L.wol_decode_phases(p, p, p, 4096, 11000, 128, p, p, big, None) == 5
    assert L.wol_decode_phases(p, p, p, 4096, 11008, -1, p, p, big, None) == 5    # group-wise scales only
    assert L.wol_decode_phases(p, p, None, 4096, 11008, 128, p, p, big, None) == 1
    assert L.wol_decode_phases(p, p, p, 4096, 11008, 128, ctypes.c_void_p(0x1002), p, big, None) == 9
    assert L.wol_decode_phases(p, p, p, 4096, 11008, 128, p, p, 688 * 64 * 8 - 1, None) == 8


def test_prefill_phases_argument_errors(lib):
    L = lib.lib
    p = ctypes.c_void_p(0x1000)
    big = 1 << 30
    assert L.wol_prefill_phases(p, p, p, 256, 4096, 256, p, p, big, None) not in (1, 5, 8, 9)  # valid: fails only for want of a device
    assert L.wol_prefill_phases(p, p, p, 255, 4096, 256, p, p, big, None) == 5
    assert L.wol_prefill_phases(p, p, p, 256, 4096, 128, p, p, big, None) == 5
    assert L.wol_prefill_phases(p, p, p, 256, 128, 256, p, p, big, None) == 5   # fewer k tiles than stages
    assert L.wol_prefill_phases(p, p, p, 256, 4100, 256, p, p, big, None) == 5
    assert L.wol_prefill_phases(p, None, p, 256, 4096, 256, p, p, big, None) == 1
    assert L.wol_prefill_phases(p, p, p, 256, 4096, 256, p, None, big, None) == 1
    assert L.wol_prefill_phases(ctypes.c_void_p(0x1004), p, p, 256, 4096, 256, p, p, big, None) == 9
    assert L.wol_prefill_phases(p, p, p, 512, 4096, 512, p, p, 4 * 64 * 8 - 1, None) == 8


def test_linear_plan_names_the_kernel_per_shape(lib):
    # wol_linear's choice between its three kernels, as the library reports it
    # (no device work): one row streams a workgroup per strip; 5..16 rows go to
    # the batched decode kernel from 2.5 strips per CU on, 2 to 4 rows only where
    # the streaming kernel has to walk its units or, on int4 at K >= 4096, from
    # five strips per CU on, and only for the K it is built for; above 64 rows the GEMM
    def plan(M, K, N, bits, g):
        buf = ctypes.create_string_buffer(256)
        ws = lib.lib.wol_linear_workspace(M, K, N, bits, g)
        assert lib.lib.wol_linear_plan(M, K, N, bits, g, ws, buf, 256) == 0
        return buf.value.decode()

    assert "stream_kernel" in plan(1, 4096, 11008, 4, 128)
    assert "batch_kernel" in plan(16, 4096, 11008, 4, -1)
    assert "stream_kernel" in plan(2, 4096, 11008, 4, -1)
    assert "issued at once" in plan(2, 4096, 28672, 8, -1)   # whatever the number of strips
    assert "batch_kernel" in plan(2, 4096, 28672, 4, -1)
    assert "batch_kernel" in plan(2, 8192, 11008, 4, -1)     # 32 units of two rows per strip: the streaming kernel would walk
    assert "stream_kernel" in plan(4, 4096, 11008, 4, -1)
    assert "stream_kernel" in plan(4, 4096, 16384, 8, -1)
    assert "issued at once" in plan(1, 8192, 28672, 4, 128)
    assert "batch_kernel" in plan(4, 8192, 28672, 4, 128)
    assert "stream_kernel" in plan(8, 4096, 12288, 8, 64)   # 64 units per strip, sixteen wavefronts with four each
    assert "batch_kernel" in plan(8, 4096, 22016, 8, 64)    # from five strips per CU on
    assert "batch_kernel" in plan(8, 4096, 12288, 4, 128)
    assert "stream_kernel" in plan(8, 4096, 4096, 8, 64)    # one strip per CU
    assert "stream_kernel" in plan(8, 11008, 4096, 8, 64)   # a K the batched kernel is not built for
    assert "stream_kernel" in plan(8, 8192, 28672, 8, -1)   # int8 at K = 8192 does not fit its registers
    assert "gemm_dma_kernel" in plan(2048, 4096, 12288, 8, -1)
    assert "256x256" in plan(2048, 4096, 12288, 8, -1)
    assert lib.lib.wol_linear_plan(4, 4096, 100, 8, -1, 0, ctypes.create_string_buffer(8), 8) == 5


def test_linear_plan_is_the_same_with_the_advised_scratch_as_with_any_larger(lib):
    # wol_linear_workspace() bytes are enough for the kernel wol_linear would
    # take with unlimited scratch -- also where that is 0 bytes (a GEMM that
    # needs no K runs, a decode kernel): the choice must not flip between the
    # two.  Sweep of the region between the decode kernels and the prefill GEMM.
    size_max = ctypes.c_size_t(-1).value

    def plan(M, K, N, bits, g, ws):
        buf = ctypes.create_string_buffer(256)
        assert lib.lib.wol_linear_plan(M, K, N, bits, g, ws, buf, 256) == 0
        return buf.value.decode()

    flips = []
    for bits in (4, 8):
        for g in (-1, 128):
            for K in (1024, 2048, 4096, 8192, 11008):
                for N in (2048, 4096, 11008, 12288, 14336, 28672):
                    for M in (1, 2, 8, 12, 16, 17, 20, 24, 27, 32, 40, 49, 56, 57, 64, 65, 128):
                        need = lib.lib.wol_linear_workspace(M, K, N, bits, g)
                        a, b = plan(M, K, N, bits, g, need), plan(M, K, N, bits, g, size_max)
                        if a != b:
                            flips.append((M, K, N, bits, g, a, b))
    assert not flips, flips[:5]


@pytest.mark.parametrize("bits", [8, 4])
def test_repack_host_matches_the_layout_definitions(lib, bits):
    # the CPU-side re-layout (what a CPU weight_quantize calls to hand out GFX950
    # weights) against the numpy statements of the three layouts, every pair
    from oracle import wo_oracle as O

    K, N = 192, 96
    wb = H.make_weight(K, N, H.BF16, seed=8)
    oc, _ = O.weight_quantize(wb, H.BF16, bits, 64)
    q = H.q_from_canonical(oc, bits)
    forms = {0: np.ascontiguousarray(oc).view(np.uint8).reshape(-1),
             1: H.paddle_hip_from_q(q, bits).view(np.uint8).reshape(-1),
             2: H.gfx950_from_q(q, bits).reshape(-1)}
    for li, src in forms.items():
        for lo, want in forms.items():
            out = np.full(src.size, 0xEE, np.uint8)
            rc = lib.lib.wol_repack_host(src.ctypes.data, li, out.ctypes.data, lo, K, N, bits)
            assert rc == 0 and np.array_equal(out, want), (li, lo)
    assert lib.lib.wol_repack_host(forms[0].ctypes.data, 0, forms[0].ctypes.data, 2, K, N, bits) == 6
    assert lib.lib.wol_repack_host(forms[0].ctypes.data, 5, forms[1].ctypes.data, 2, K, N, bits) == 6
