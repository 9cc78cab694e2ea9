"""ti_bmm_i8_static_scratch: the split-K GEMM entry point that allocates nothing (its ticket counters
and partial sums live in a fixed array of the library's device image).  Called through the C ABI
with raw ctypes and compared, bit for bit, with ti_bmm_i8_config (which allocates its workspace) on
two calls in a row, the second with a smaller input; then captured into a HIP graph on a stream that
has no workspace.  Collected last on purpose (file name)."""
import ctypes

import numpy as np
import pytest
import torch

import oracle as O
from tests.util import DEV, cpu, gpu, rand_i8, rng

pytestmark = pytest.mark.gpu


def _call(fn, a, w, bias, alpha, beta, out, epi, config, stream=None):
    from triton_int_amd import _lib as L
    M, K = a.shape
    N = w.shape[0]
    st = L.current_stream(a.device) if stream is None else stream
    return fn(a.data_ptr(), 0, a.stride(0), 1, w.data_ptr(), 0, w.stride(0), 1, out.data_ptr(), 0, out.stride(0), 1,
              1, M, N, K, bias.data_ptr(), L.TORCH_TO_BIAS[bias.dtype], alpha.data_ptr(), beta.data_ptr(),
              epi, L.TORCH_TO_DT[out.dtype], L.ROUND_RNE_CLAMP, config, st)


def test_static_scratch_entry_point_matches_the_allocating_one():
    from triton_int_amd import _lib as L
    lib = L.lib()
    names = [lib.ti_gemm_config_name(i).decode() for i in range(lib.ti_gemm_num_configs())]
    alpha = torch.tensor(0.0004, device=DEV)
    beta = torch.tensor(0.05, device=DEV)
    # two calls in a row, the second smaller (fewer tiles, fewer splits, shorter K): what the first
    # left in the scratch must not leak into the second
    for (M, N, K, cfg_name, splits) in [(200, 1040, 8192, "ws_128x128", 7), (96, 272, 2064, "ws_128x128", 3),
                                        (300, 528, 4112, "ws_256x128", 4), (130, 400, 1040, "ws_256x160", 2),
                                        (128, 6848, 10240, None, 0), (64, 1024, 8192, None, 0)]:
        g = rng(M + N + K)
        a, w = rand_i8(g, M, K, lo=-128), rand_i8(g, N, K, lo=-128)
        b8, bf = rand_i8(g, N), g.standard_normal(N).astype(np.float32)
        ga, gw, gb8, gbf = gpu(a), gpu(w), gpu(b8), gpu(bf)
        config = -1 if cfg_name is None else ([i for i, n in enumerate(names) if n.startswith(cfg_name)][0] | (splits << 8))
        for bias, dt, epi in ((gb8, torch.int8, L.EPI_SCALE_I8), (gbf, torch.float32, L.EPI_SCALE_F)):
            want = torch.empty((M, N), dtype=dt, device=DEV)
            rc = _call(lib.ti_bmm_i8_config, ga, gw, bias, alpha, beta, want, epi, config)
            assert rc == 0, lib.ti_last_error().decode()
            used = (lib.ti_gemm_last_config(), lib.ti_gemm_last_splits())
            assert used[1] > 1, "the case is meant to split K"
            got = torch.full((M, N), 77, dtype=dt, device=DEV)
            torch.cuda.synchronize()
            free0 = torch.cuda.mem_get_info()[0]
            rc = _call(lib.ti_bmm_i8_static_scratch, ga, gw, bias, alpha, beta, got, epi, config)
            assert rc == 0, lib.ti_last_error().decode()
            assert (lib.ti_gemm_last_config(), lib.ti_gemm_last_splits()) == used
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info()[0] == free0, "the call changed the device's free memory"
            assert torch.equal(got, want), (M, N, K, cfg_name, splits, dt)
        if M * N * K < 5e8:   # and the oracle, where it is quick
            assert np.array_equal(cpu(got), O.linear_a8_w8_bfp32_ofp32(a, w, bf, np.float32(0.0004), np.float32(0.05)))


def test_static_scratch_rejects_what_does_not_fit_and_is_capturable():
    from triton_int_amd import _lib as L
    lib = L.lib()
    names = [lib.ti_gemm_config_name(i).decode() for i in range(lib.ti_gemm_num_configs())]
    ws256 = [i for i, n in enumerate(names) if n.startswith("ws_256x128")][0]
    alpha, beta = torch.tensor(0.0004, device=DEV), torch.tensor(0.05, device=DEV)
    g = rng(9)
    # 8 splits of 4 x 16 tiles of 256 x 128 int32 = 64 MiB of partial sums: more than the 32 MiB array
    M, N, K = 1024, 2048, 8192
    ga, gw, gbf = gpu(rand_i8(g, M, K)), gpu(rand_i8(g, N, K)), gpu(g.standard_normal(N).astype(np.float32))
    out = torch.empty((M, N), dtype=torch.float32, device=DEV)
    rc = _call(lib.ti_bmm_i8_static_scratch, ga, gw, gbf, alpha, beta, out, L.EPI_SCALE_F, ws256 | (8 << 8))
    assert rc == -2 and "static scratch" in lib.ti_last_error().decode()        # TI_E_SHAPE, nothing launched
    assert _call(lib.ti_bmm_i8_static_scratch, ga, gw, gbf, alpha, beta, out, L.EPI_SCALE_F, ws256 | (2 << 8)) == 0
    want = torch.empty_like(out)
    assert _call(lib.ti_bmm_i8_config, ga, gw, gbf, alpha, beta, want, L.EPI_SCALE_F, ws256) == 0
    assert torch.equal(out, want)
    # a split the library chooses itself and that does not fit gives way to the unsplit launch: same result
    M2, N2, K2 = 129, 11264, 32768
    ga2, gw2, gbf2 = gpu(rand_i8(g, M2, K2)), gpu(rand_i8(g, N2, K2)), gpu(g.standard_normal(N2).astype(np.float32))
    out2, want2 = torch.empty((M2, N2), dtype=torch.float32, device=DEV), torch.empty((M2, N2), dtype=torch.float32, device=DEV)
    assert _call(lib.ti_bmm_i8_config, ga2, gw2, gbf2, alpha, beta, want2, L.EPI_SCALE_F, -1) == 0 and lib.ti_gemm_last_splits() > 1
    assert _call(lib.ti_bmm_i8_static_scratch, ga2, gw2, gbf2, alpha, beta, out2, L.EPI_SCALE_F, -1) == 0 and lib.ti_gemm_last_splits() == 1
    assert torch.equal(out2, want2)
    del ga2, gw2, gbf2, out2, want2
    # unsplit launches use no scratch at all and are never refused for size
    assert _call(lib.ti_bmm_i8_static_scratch, ga, gw, gbf, alpha, beta, out, L.EPI_SCALE_F, -1) == 0
    assert torch.equal(out, want)
    # captured on a stream that never had a workspace: replays give the eager result every time
    M, N, K = 128, 1024, 8192
    ga, gw, gbf = gpu(rand_i8(g, M, K)), gpu(rand_i8(g, N, K)), gpu(g.standard_normal(N).astype(np.float32))
    out = torch.empty((M, N), dtype=torch.float32, device=DEV)
    want = torch.empty_like(out)
    assert _call(lib.ti_bmm_i8_config, ga, gw, gbf, alpha, beta, want, L.EPI_SCALE_F, -1) == 0 and lib.ti_gemm_last_splits() > 1
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = _call(lib.ti_bmm_i8_static_scratch, ga, gw, gbf, alpha, beta, out, L.EPI_SCALE_F, -1, stream=side.cuda_stream)
    assert rc == 0 and lib.ti_gemm_last_splits() > 1
    for _ in range(3):
        out.fill_(-1.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)
