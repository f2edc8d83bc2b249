"""Guard on the rules that choose a kernel for wol_linear: a timing test, kept in
a file of its own that is collected late so that a slow machine cannot hide the
parity tests behind it."""
import pytest

pytestmark = pytest.mark.gpu


def _time_linear(lib, args, out_f32, kernel, tail, n=30):
    import torch

    def go():
        rc = lib.wol_linear_on(*args, out_f32, kernel, *tail)
        assert rc == 0, rc

    for _ in range(5):
        go()
    torch.cuda.synchronize()
    ts = []
    for _ in range(5):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            go()
        e1.record()
        torch.cuda.synchronize()
        ts.append(e0.elapsed_time(e1) / n)
    return sorted(ts)[len(ts) // 2]


def test_dispatcher_is_never_far_from_the_best_pinned_kernel(device):
    # The rules that choose a kernel are fitted to measurements; this guards
    # them against gross mistakes (a rule that sends a decode call to the GEMM,
    # or the other way round): on shapes from every region of the rules the
    # kernel wol_linear takes is at most twice as slow as the fastest kernel
    # that accepts the shape.  Eager launches, median of five timings.
    import torch
    from paddle_amd import _lib
    from paddle_amd.nn import quant as Q

    L = _lib.lib
    cases = [(1, 4096, 11008, 4, 128), (4, 4096, 11008, 4, -1), (8, 4096, 12288, 8, 64), (16, 4096, 11008, 4, -1),
             (16, 11008, 4096, 4, -1), (12, 13824, 5120, 4, 128), (16, 6144, 6144, 8, -1), (24, 4096, 11008, 8, 64),
             (32, 8192, 8192, 4, 128), (32, 8192, 28672, 4, 128), (64, 4096, 11008, 4, -1), (48, 4096, 4096, 8, 64),
             (128, 4096, 4096, 8, -1)]
    worst = []
    for M, K, N, bits, g in cases:
        w = (torch.randn(K, N, device=device) * 0.02).to(torch.bfloat16)
        codes, scale = Q.weight_quantize(w, algo="weight_only_int8" if bits == 8 else "weight_only_int4", group_size=g)
        del w
        x = torch.randn(M, K, device=device).to(torch.bfloat16)
        out = torch.empty(M, N, device=device, dtype=torch.bfloat16)
        times = {}
        for kernel in (_lib.KERNEL_AUTO, _lib.KERNEL_STREAM, _lib.KERNEL_GEMM, _lib.KERNEL_BATCH,
                       _lib.KERNEL_BATCH_SPLIT):
            wsb = L.wol_linear_workspace_for(M, K, N, bits, g, kernel)
            ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device=device)
            args = (x.data_ptr(), codes.data_ptr(), None, scale.data_ptr(), 1, M, K, N, bits, g, out.data_ptr())
            tail = (ws.data_ptr(), wsb, None)
            if L.wol_linear_on(*args, 0, kernel, *tail) != 0:
                continue  # the kernel does not take this shape
            times[kernel] = _time_linear(L, args, 0, kernel, tail)
        best = min(v for k, v in times.items() if k != _lib.KERNEL_AUTO)
        print("case", M, K, N, bits, g, {k: round(v * 1e3, 1) for k, v in times.items()}, flush=True)
        worst.append((times[_lib.KERNEL_AUTO] / best, M, K, N, bits, g))
    assert max(worst)[0] <= 2.0, sorted(worst, reverse=True)[:3]
