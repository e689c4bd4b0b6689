"""unit_gemm_f16_static: the k-split fp16 GEMM whose partial-tile planes live in a device array inside the library
(the entry point allocates nothing), checked through the C ABI against unit_gemm_f16_ws, the same kernels on a
caller workspace: bit-identical, on two calls in a row, the second with a smaller input."""
import ctypes

import numpy as np
import pytest
import torch

from unit_amd import _lib, rng

pytestmark = pytest.mark.gpu


def _run(L, dev, M, N, K, out_f16, seed):
    a = torch.from_numpy(rng.normal_f16((M, K), seed, 1.0 / np.sqrt(K))).to(dev)
    b = torch.from_numpy(rng.normal_f16((K, N), seed + 1)).to(dev)
    dt = torch.float16 if out_f16 else torch.float32
    need = ctypes.c_size_t()
    _lib.check(L.unit_gemm_f16_ws_bytes(M, N, K, ctypes.byref(need)))
    ws = torch.full((max(need.value, 16),), 0x77, dtype=torch.uint8, device=dev)
    want = torch.full((M, N), -1, dtype=dt, device=dev)
    got = torch.full((M, N), -2, dtype=dt, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    _lib.check(L.unit_gemm_f16_ws(a.data_ptr(), b.data_ptr(), want.data_ptr(), M, N, K, int(out_f16), ws.data_ptr(),
                                  ws.numel(), stream))
    _lib.check(L.unit_gemm_f16_static(a.data_ptr(), b.data_ptr(), got.data_ptr(), M, N, K, int(out_f16), stream))
    name = _lib.last_variant()
    torch.cuda.synchronize()
    ref = a.double().cpu().numpy() @ b.double().cpu().numpy()
    err = np.abs(got.double().cpu().numpy() - ref) / np.maximum(np.abs(ref), 1e-3 * np.abs(ref).max())
    return want, got, name, need.value, float(err.max())


@pytest.mark.parametrize("out_f16", [False, True])
def test_static_scratch_gemm_matches_the_workspace_entry_point(dev, out_f16):
    L = _lib.load()
    # first call: 21 k-splits of 128 x 768 (8.3 MB of planes); second call, right after, a smaller problem
    # (16 splits of 96 x 64) whose planes land on the first one's leftovers
    for (M, N, K), seed in (((128, 768, 3072), 31), ((96, 64, 4096), 33)):
        want, got, name, need, err = _run(L, dev, M, N, K, out_f16, seed)
        assert need > 0 and "planes" in name, (name, need)
        assert torch.equal(want, got), (M, N, K, name)
        assert err <= 1e-2 + (2e-3 if out_f16 else 0), (err, name)  # max relative error against float64


def test_static_scratch_gemm_without_k_splits_and_beyond_its_limit(dev):
    L = _lib.load()
    want, got, name, need, err = _run(L, dev, 2048, 2048, 256, False, 35)  # 256 tiles: no k-splits, no scratch
    assert need == 0 and torch.equal(want, got) and err <= 1e-2, (name, need, err)
    # 224 tiles of 128 x 128 with a long reduction take three k-splits: 44 MB of planes, more than the 16 MiB array
    M, N, K = 1792, 2048, 4096
    nbytes = ctypes.c_size_t()
    _lib.check(L.unit_gemm_f16_ws_bytes(M, N, K, ctypes.byref(nbytes)))
    assert nbytes.value == 3 * M * N * 4
    a = torch.zeros((M, K), dtype=torch.float16, device=dev)
    b = torch.zeros((K, N), dtype=torch.float16, device=dev)
    c = torch.zeros((M, N), dtype=torch.float32, device=dev)
    rc = L.unit_gemm_f16_static(a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == -1 and b"static buffer holds" in L.unit_last_error()


def test_static_scratch_gemm_allocates_nothing_and_replays_in_a_graph(dev):
    """The property the entry point is for: after one call outside capture (it resolves the scratch array's address
    on this device), a k-split call and a call without k-splits are captured into one HIP graph; every replay --
    with eager launches and synchronisations between them -- reproduces the eager results bit for bit, and the free
    device memory is the same before and after the calls."""
    L = _lib.load()
    shapes = ((128, 768, 3072), (512, 512, 256))  # 21 k-splits through the scratch array; 16 tiles, no split
    ops = []
    for i, (M, N, K) in enumerate(shapes):
        a = torch.from_numpy(rng.normal_f16((M, K), 41 + i, 1.0 / np.sqrt(K))).to(dev)
        b = torch.from_numpy(rng.normal_f16((K, N), 51 + i)).to(dev)
        ops.append((a, b, torch.empty((M, N), dtype=torch.float32, device=dev), M, N, K))

    def run(stream):
        for a, b, c, M, N, K in ops:
            _lib.check(L.unit_gemm_f16_static(a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K, 0, stream))

    run(torch.cuda.current_stream().cuda_stream)  # outside capture: symbol address, kernel attributes
    torch.cuda.synchronize()
    eager = [c.clone() for _, _, c, _, _, _ in ops]
    free_before = torch.cuda.mem_get_info()[0]
    run(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run(torch.cuda.current_stream().cuda_stream)
    for replay in range(3):
        for _, _, c, _, _, _ in ops:
            c.fill_(float(replay) - 7.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for want, (_, _, c, _, _, _) in zip(eager, ops):
            assert torch.equal(want, c), replay
        # eager work of the same entry point between replays: the shared scratch array is rewritten
        a, b, c, M, N, K = ops[0]
        other = torch.empty_like(c)
        _lib.check(L.unit_gemm_f16_static(a.data_ptr(), b.data_ptr(), other.data_ptr(), M, N, K, 0,
                                          torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        assert torch.equal(other, eager[0])
