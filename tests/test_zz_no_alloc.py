"""The allocation-free entry point fp6mi_linear_native_static (split-K partial sums in a static device array of the
library) against fp6mi_linear_native with a caller workspace: same kernels, so the outputs must be identical bit for bit,
on two calls in a row, the second on a smaller problem (the array keeps the first call's contents)."""
import numpy as np
import pytest
import torch

import oracle
import fp6_llm_amd as fp6
from fp6_llm_amd import _lib, synth

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _both(E, M, OC, IC, N, splitK, seed):
    L = _lib.lib()
    raw, sc, x = synth.uniform_problem(seed, OC, IC, N, E, M)
    native = fp6.weight_prepacking_native_cpu(E, M, torch.from_numpy(raw)).to(DEV)
    scd, xd = torch.from_numpy(sc).to(DEV), torch.from_numpy(x).to(DEV)
    stream = torch.cuda.current_stream().cuda_stream
    ws = torch.empty(max(1, splitK * N * OC), dtype=torch.float32, device=DEV)
    want = torch.full((N, OC), float("nan"), dtype=torch.float16, device=DEV)
    got = torch.full((N, OC), float("nan"), dtype=torch.float16, device=DEV)
    rc = L.fp6mi_linear_native(E, M, stream, native.data_ptr(), scd.data_ptr(), xd.data_ptr(), want.data_ptr(), OC, N, IC, ws.data_ptr(), splitK)
    assert rc == 0, L.fp6mi_error_string(rc)
    rc = L.fp6mi_linear_native_static(E, M, stream, native.data_ptr(), scd.data_ptr(), xd.data_ptr(), got.data_ptr(), OC, N, IC, splitK)
    assert rc == 0, L.fp6mi_error_string(rc)
    torch.cuda.synchronize()
    assert torch.equal(got, want), (E, M, OC, IC, N, splitK)
    ref = oracle.gemm_f64(oracle.dequant(raw, sc, E, M), x)
    err = np.abs(got.cpu().numpy().astype(np.float64) - ref) / np.maximum(np.abs(ref), np.sqrt((ref ** 2).mean()))
    assert err.max() <= 1e-2, err.max()     # the bar of every GEMM test here: max |y - r| / max(|r|, rms r) <= 1e-2


def test_static_workspace_entry_point_matches_the_workspace_one():
    L = _lib.lib()
    assert L.fp6mi_static_workspace_bytes() == 32 << 20
    assert L.fp6mi_init() == 0
    _both(3, 2, 1024, 4096, 40, 4, 4100)    # tile kernel, 4 splits: 655 360 bytes of partial sums
    _both(3, 2, 512, 2048, 8, 3, 4101)      # right after it, smaller, the stream kernel, 3 splits
    _both(2, 2, 256, 1024, 1, 1, 4102)      # splitK = 1 does not touch the array
    _both(2, 1, 768, 1088, 17, 2, 4103)


def test_static_workspace_entry_point_allocates_nothing_and_can_be_captured():
    """After fp6mi_init the entry point must not touch the allocator: the device's free memory is the same before and after
    eager calls, and a call with split-K recorded as the only work of a stream capture (where an allocation or a lazy
    symbol lookup would break the capture) replays to the eager result."""
    L = _lib.lib()
    assert L.fp6mi_init() == 0
    E, M, OC, IC, N, splitK = 3, 2, 1024, 4096, 40, 4
    raw, sc, x = synth.uniform_problem(4110, OC, IC, N, E, M)
    native = fp6.weight_prepacking_native_cpu(E, M, torch.from_numpy(raw)).to(DEV)
    scd, xd = torch.from_numpy(sc).to(DEV), torch.from_numpy(x).to(DEV)
    eager = torch.empty((N, OC), dtype=torch.float16, device=DEV)
    got = torch.full((N, OC), float("nan"), dtype=torch.float16, device=DEV)

    def call(stream, out, n=N, k=splitK):
        return L.fp6mi_linear_native_static(E, M, stream, native.data_ptr(), scd.data_ptr(), xd.data_ptr(), out.data_ptr(), OC, n, IC, k)

    assert call(torch.cuda.current_stream().cuda_stream, eager) == 0       # also loads the kernels' code objects
    assert call(torch.cuda.current_stream().cuda_stream, eager, 8, 3) == 0
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]                              # hipMemGetInfo: the driver's view, not torch's pool
    for _ in range(3):
        assert call(torch.cuda.current_stream().cuda_stream, eager, 8, 3) == 0
        assert call(torch.cuda.current_stream().cuda_stream, eager) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            assert call(s.cuda_stream, got) == 0
    for rep in range(2):
        got.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, eager), rep


def test_static_workspace_entry_point_rejects_what_does_not_fit():
    L = _lib.lib()
    p = torch.zeros(64, dtype=torch.float16, device=DEV).data_ptr()
    # 8 splits x 8192 x 256 floats = 64 MiB > 32 MiB: refused on the host, nothing is launched
    assert L.fp6mi_linear_native_static(3, 2, None, p, p, p, p, 8192, 256, 8192, 8) == -7
    assert L.fp6mi_linear_native_static(3, 2, None, p, p, p, p, 100, 1, 64, 2) == -2
    assert L.fp6mi_linear_native_static(3, 2, None, p, p, p, p, 256, 1, 64, 0) == -5
    assert len(L.fp6mi_error_string(-7)) > 8
